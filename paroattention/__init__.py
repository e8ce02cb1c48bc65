"""`import paroattention` for callers written against the reference package: this name resolves to
paroatten_amd (the MI355X implementation of the same public surface: paroattention/__init__.py:1-5 of the
reference), and so do its submodules `core`, `quant`, `cogvideox`, `wan`, `prefetch_utils`, `prefetch_wan`, `utils`,
`_qattn_sm80`, `_fused`, `_rope`.  Nothing is defined here."""
import paroatten_amd

paroatten_amd.install_alias(__name__)
