"""Wan 2.1 attention processor: the reference's `paroattention.wan` processor class
(paroattention/wan.py:25-327) on the fused kernels.

`PARO_WanAttnProcessor2_0` keeps the constructor, injected attributes, call signature and return
value.  The reference's body cannot run to completion (debugging comparisons and an interactive
breakpoint sit between the attention call and the return, wan.py:277-296); this implements the
sequence it intends: projections -> per-head RMS norms -> rotary embedding -> per-head permutation
-> per-warp INT8 -> block-sparse attention -> inverse permutation -> output projection, with the
same fusions as the CogVideoX processor.  Differences in arithmetic:
  * the rotation is evaluated in fp32 from fp32 cos/sin tables made once from the complex
    `rotary_emb` (the reference multiplies in complex128, wan.py:161-167); both round to the same
    16-bit value except for rare last-bit differences;
  * the latent grid (21x45x80 hard-coded at wan.py:33-35) is the `grid` argument/attribute; the
    720p and 480p grids are recognised from the token count.
The transformer/block classes of wan.py:353-783 are diffusers model definitions, not part of the
attention path; `set_paro_processors` installs this processor on an existing transformer instead.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F

from . import permute as PM
from . import rope
from .cogvideox import SHARED_TABLES, _ParoProcessorBase
from .permute import PERMUTATIONS, PERMUTATIONS_INV  # noqa: F401

WAN_GRIDS = {21 * 45 * 80: (21, 45, 80), 21 * 30 * 52: (21, 30, 52)}
WAN_I2V_IMAGE_TOKENS = 257   # CLIP image-context tokens in front of the text context (wan.py:129-131)


def permute_qk(query, key, value, permute_plan, i_block, grid=(21, 45, 80), n_text=0):
    """Drop-in for wan.py:25-63 (in place, all tokens are image tokens)."""
    return PM.permute_qk(query, key, value, permute_plan, i_block, grid=grid, n_text=n_text)


def permute_attn_out(attn_out, permute_plan, i_block, grid=(21, 45, 80), n_text=0):
    """Drop-in for wan.py:65-111 (in place)."""
    return PM.permute_attn_out(attn_out, permute_plan, i_block, grid=grid, n_text=n_text)


class PARO_WanAttnProcessor2_0(_ParoProcessorBase):
    def _tables(self, rotary_emb, device, head_dim):
        # (shared by all the processors of the model: the rotary tensor of a step is converted once)
        if isinstance(rotary_emb, (tuple, list)):
            # later diffusers versions hand over (cos, sin) as real tensors [1, N, 1, D] with the frequency of
            # every channel pair repeated over the pair: already the kernel's form
            cos_t, sin_t = rotary_emb
            return SHARED_TABLES.get((cos_t, sin_t), device,
                                     lambda: (cos_t.reshape(-1, head_dim).float().contiguous(),
                                              sin_t.reshape(-1, head_dim).float().contiguous()))
        return SHARED_TABLES.get((rotary_emb,), device,
                                 lambda: rope.complex_to_real_tables(rotary_emb.reshape(-1, head_dim // 2)))

    def __call__(self, attn, hidden_states: torch.Tensor, encoder_hidden_states: Optional[torch.Tensor] = None,
                 attention_mask: Optional[torch.Tensor] = None, rotary_emb: Optional[torch.Tensor] = None):
        encoder_hidden_states_img = None
        if getattr(attn, "add_k_proj", None) is not None and encoder_hidden_states is not None:
            encoder_hidden_states_img = encoder_hidden_states[:, :WAN_I2V_IMAGE_TOKENS]
            encoder_hidden_states = encoder_hidden_states[:, WAN_I2V_IMAGE_TOKENS:]
        self_attention = encoder_hidden_states is None
        if self_attention:
            encoder_hidden_states = hidden_states

        query = attn.to_q(hidden_states)
        key = attn.to_k(encoder_hidden_states)
        value = attn.to_v(encoder_hidden_states)
        if attn.norm_q is not None:
            query = attn.norm_q(query)
        if attn.norm_k is not None:
            key = attn.norm_k(key)
        batch_size, sequence_length, inner_dim = query.shape
        head_dim = inner_dim // attn.heads
        query = query.unflatten(2, (attn.heads, -1)).transpose(1, 2)
        key = key.unflatten(2, (attn.heads, -1)).transpose(1, 2)
        value = value.unflatten(2, (attn.heads, -1)).transpose(1, 2)

        sparse = self_attention and self.i_timestep >= 0
        if not self_attention:
            # cross-attention (text context): keys have another length, the block plan does not apply
            if rotary_emb is not None:
                raise ValueError("rotary_emb with cross-attention inputs is not supported")
            out = F.scaled_dot_product_attention(query, key, value, attn_mask=attention_mask, dropout_p=0.0,
                                                 is_causal=False)
            hidden_states = out.transpose(1, 2).flatten(2, 3).type_as(query)
            if encoder_hidden_states_img is not None:
                hidden_states = hidden_states + self._image_context(attn, query, encoder_hidden_states_img)
            hidden_states = attn.to_out[0](hidden_states)
            return attn.to_out[1](hidden_states)

        grid = self._grid_for(sequence_length, WAN_GRIDS)
        cos = sin = None
        if rotary_emb is not None:
            cos, sin = self._tables(rotary_emb, query.device, head_dim)
        if sparse:
            orders = self._orders(query.device)
        else:
            orders = torch.zeros(attn.heads, dtype=torch.int32, device=query.device)   # order 0 = identity
        done = self._timer.start()
        token_major = torch.empty((batch_size, sequence_length, attn.heads, head_dim), dtype=query.dtype,
                                  device=query.device)
        if sparse:
            ops = self._prepare(query, key, value, orders, grid, 0, cos, sin)
            self._sparse_attention(ops, token_major.transpose(1, 2), 1.0 / (head_dim ** 0.5), orders, grid, 0)
            done.record()
        else:
            qp, kp, vp = self._rope_permute(query, key, value, orders, grid, 0, cos, sin)
            out = F.scaled_dot_product_attention(qp, kp, vp, attn_mask=attention_mask, dropout_p=0.0, is_causal=False)
            token_major.copy_(out.transpose(1, 2))
            done.record()
        self.call_count += 1
        if len(self._timer._pending) >= 64:
            self._timer.fold(block=False)

        hidden_states = token_major.view(batch_size, sequence_length, inner_dim)
        hidden_states = attn.to_out[0](hidden_states)
        hidden_states = attn.to_out[1](hidden_states)
        return hidden_states

    @staticmethod
    def _image_context(attn, query, encoder_hidden_states_img):
        """I2V: dense attention of the queries over the 257 image-context tokens (wan.py:169-183)."""
        key_img = attn.norm_added_k(attn.add_k_proj(encoder_hidden_states_img))
        value_img = attn.add_v_proj(encoder_hidden_states_img)
        key_img = key_img.unflatten(2, (attn.heads, -1)).transpose(1, 2)
        value_img = value_img.unflatten(2, (attn.heads, -1)).transpose(1, 2)
        out = F.scaled_dot_product_attention(query, key_img, value_img, attn_mask=None, dropout_p=0.0, is_causal=False)
        return out.transpose(1, 2).flatten(2, 3).type_as(query)


PARO_WanAttnProcessor = PARO_WanAttnProcessor2_0


def set_paro_processors(transformer, permute_plan, sparse_mask=None, prefetch_stream=None, grid=None,
                        processor_cls=None):
    """Install one processor per block on `attn1` of `transformer.blocks` (Wan) or
    `transformer.transformer_blocks` (CogVideoX) and inject the plan state the way the example
    pipelines do (example/pipeline_cogvideox.py:120-136): `i_block`, `i_timestep = 0`, `permute_plan`
    and either the device-resident `sparse_mask` [T,L,H,nb,nb] or a `prefetch_stream`."""
    if (sparse_mask is None) == (prefetch_stream is None):
        raise ValueError("give exactly one of sparse_mask and prefetch_stream")
    blocks = getattr(transformer, "transformer_blocks", None)
    if blocks is None:
        blocks = transformer.blocks
        cls = processor_cls or PARO_WanAttnProcessor2_0
    else:
        from .cogvideox import PARO_CogVideoXAttnProcessor2_0
        cls = processor_cls or PARO_CogVideoXAttnProcessor2_0
    procs = []
    for i_block, block in enumerate(blocks):
        p = cls(grid=grid)
        p.permute_plan = permute_plan
        p.i_block = i_block
        p.i_timestep = 0
        if prefetch_stream is not None:
            p.prefetch_stream = prefetch_stream
        else:
            p.sparse_mask = sparse_mask
        if hasattr(block.attn1, "set_processor"):
            block.attn1.set_processor(p)
        else:
            block.attn1.processor = p
        procs.append(p)
    return procs


_DIFFUSERS_WAN = {}


def diffusers_wan_classes():
    """`PARO_WanTransformerBlock` and `PARO_WanTransformer3DModel` (paroattention/wan.py:525-783): in the reference
    these are copies of diffusers' Wan transformer whose only change is the processor of `attn1` (wan.py:550).
    Here they are SUBCLASSES of the installed diffusers classes, built on first use: the block installs a
    `PARO_WanAttnProcessor2_0` on its `attn1`, the model builds its blocks from that class, everything else
    (weights, config, `from_pretrained`, forward) is diffusers' own.  Raises ImportError without diffusers."""
    if _DIFFUSERS_WAN:
        return _DIFFUSERS_WAN
    try:
        from diffusers.models.transformers import transformer_wan as tw
    except Exception as e:
        raise ImportError("PARO_WanTransformer3DModel / PARO_WanTransformerBlock subclass diffusers' Wan transformer, "
                          f"and diffusers is not importable here ({e}); on an existing model use "
                          "paroatten_amd.set_paro_processors(model, permute_plan, ...)") from e

    class PARO_WanTransformerBlock(tw.WanTransformerBlock):
        def __init__(self, *args, **kwargs):
            super().__init__(*args, **kwargs)
            self.attn1.set_processor(PARO_WanAttnProcessor2_0())

    class PARO_WanTransformer3DModel(tw.WanTransformer3DModel):
        def __init__(self, *args, **kwargs):
            super().__init__(*args, **kwargs)
            # (the blocks exist by now; their projections and norms are what the processor drives)
            for block in self.blocks:
                block.attn1.set_processor(PARO_WanAttnProcessor2_0())

    _DIFFUSERS_WAN.update(PARO_WanTransformerBlock=PARO_WanTransformerBlock,
                          PARO_WanTransformer3DModel=PARO_WanTransformer3DModel)
    return _DIFFUSERS_WAN


def __getattr__(name):
    if name in ("PARO_WanTransformerBlock", "PARO_WanTransformer3DModel"):
        return diffusers_wan_classes()[name]
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
