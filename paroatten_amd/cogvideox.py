"""CogVideoX attention processor: the reference's `paroattention.cogvideox`
(paroattention/cogvideox.py:22-250) on the fused kernels.

`PARO_CogVideoXAttnProcessor2_0` keeps the reference's constructor, injected attributes
(`permute_plan`, `i_block`, `i_timestep`, and `sparse_mask` or `prefetch_stream`), call signature,
return value and `get_time_stats()`.  What changes underneath:
  * RoPE, the per-head permutation of Q, K, V, the INT8 quantisation of Q/K and the FP8 packing of V
    are one pass that reads the projections in their native token-major memory ([B,N,H*D] viewed as
    [B,H,N,D] through strides) and writes only what the attention kernel reads: no transpose copy,
    no in-place rotate pass, no Python loop over heads, no host sync, no `.to(float16)` of V;
  * the inverse permutation is folded into the attention kernel's stores, which go straight to
    token-major memory, so the reshape for the output projection is a view;
  * (F,H,W), literals in the reference (cogvideox.py:31-33), are the `grid` argument/attribute;
  * timing is kept by events that are only read in get_time_stats(): no synchronize per call.
"""
from __future__ import annotations

import weakref

from typing import Optional, Sequence, Tuple

import torch
import torch.nn.functional as F

from . import _qattn_sm80 as qattn
from . import permute as PM
from .permute import permute_attn_out, permute_qk  # noqa: F401  (same module-level names as the reference)
from .quant import per_warp_int8 as per_warp_int8_cuda  # noqa: F401  (the reference's module-level name)

COG_GRID = (13, 30, 45)   # frames x height x width of CogVideoX-5b latents after patching (cogvideox.py:31-33)


class _PathTimer:
    """start/stop event pairs folded into a running total without ever blocking the caller."""

    def __init__(self):
        self.total_ms = 0.0
        self._pending = []

    def start(self):
        s = torch.cuda.Event(enable_timing=True)
        e = torch.cuda.Event(enable_timing=True)
        s.record()
        self._pending.append((s, e))
        return e

    def fold(self, block: bool):
        keep = []
        for s, e in self._pending:
            if block:
                e.synchronize()
            if e.query():
                self.total_ms += s.elapsed_time(e)
            else:
                keep.append((s, e))
        self._pending = keep


class _SharedTables:
    """fp32 (cos, sin) tables in the form the kernels read, derived once per source and shared by every processor
    of the process: the 40-odd layers of a step all receive the same rotary tensors (Wan rebuilds its `rotary_emb`
    on every forward, so a cache per processor would convert it 40 times a step and keep 40 copies, ~77 MB each
    at 720p).  A source is recognised by the identity of its tensor objects (held weakly: an address alone can
    come back with other contents) and their version counters; the two most recent sources are kept."""

    KEEP = 2

    def __init__(self):
        self._entries = []   # [(device string, [(weakref, version), ...], cos, sin)], most recent last

    def get(self, src, device, make):
        dev = str(device)
        for i, (d, refs, cos, sin) in enumerate(self._entries):
            if d == dev and len(refs) == len(src) and all(r() is t and t._version == v for t, (r, v) in zip(src, refs)):
                if i != len(self._entries) - 1:
                    self._entries.append(self._entries.pop(i))
                return cos, sin
        cos, sin = make()
        cos = cos.to(device=device, dtype=torch.float32).contiguous()
        sin = sin.to(device=device, dtype=torch.float32).contiguous()
        self._entries.append((dev, [(weakref.ref(t), t._version) for t in src], cos, sin))
        del self._entries[:-self.KEEP]
        return cos, sin

    def clear(self):
        self._entries = []


SHARED_TABLES = _SharedTables()


class _ParoProcessorBase:
    """State and helpers shared by the CogVideoX and Wan processors."""

    def __init__(self, grid: Optional[Sequence[int]] = None, smooth_k: bool = False, exact_exp: bool = False,
                 pv_f16: bool = False):
        if not hasattr(F, "scaled_dot_product_attention"):
            raise ImportError("this attention processor requires PyTorch 2.0 or newer")
        self.grid = None if grid is None else tuple(int(x) for x in grid)
        self.smooth_k = smooth_k
        self.exact_exp = exact_exp
        # accuracy mode of the attention kernel: the float16 P.V product of the reference instead of FP8
        # (about half the speed; V is then permuted and tiled in float16 by two more passes)
        self.pv_f16 = pv_f16
        self._timer = _PathTimer()
        self.time_accum = {"total": 0.0}
        self.call_count = 0
        self._orders_cache = {}
        self.i_timestep = 0
        self.i_block = 0

    # ---- plan / mask plumbing ---------------------------------------------------------------
    def _orders(self, device) -> torch.Tensor:
        key = (id(self.permute_plan), int(self.i_block), str(device))
        o = self._orders_cache.get(key)
        if o is None:
            o = PM.head_orders(self.permute_plan, int(self.i_block), device)
            self._orders_cache = {key: o}
        return o

    def _mask(self) -> torch.Tensor:
        """bool [H,nb,nb] on the device, shared by the batch (the reference stacks it per CFG
        branch, cogvideox.py:188-193; the kernel takes a batch stride of 0 instead)."""
        ps = getattr(self, "prefetch_stream", None)
        if ps is not None:
            return ps.mask_for(self.i_timestep, self.i_block)
        # the callback's value after the last denoising step is T (prefetch_utils.py:22-25): clamp as the
        # prefetch stream does
        t = min(max(int(self.i_timestep), 0), self.sparse_mask.shape[0] - 1)
        m = self.sparse_mask[t, self.i_block]
        if m.dtype != torch.bool:
            m = m.bool()
        return m

    def _grid_for(self, n_img: int, known) -> Tuple[int, int, int]:
        """(F, H, W) of the latent grid.  A token count does not determine it (21*30*52 = 21*52*30: a
        portrait video has the same count as a landscape one), so the `grid` given to the processor
        wins; without it the model's default landscape grid is assumed for a known token count, as
        the reference hard-codes it (cogvideox.py:31-33, wan.py:33-35), with a warning the first time."""
        g = self.grid
        if g is None:
            g = known.get(n_img)
            if g is not None and not getattr(self, "_grid_warned", False):
                import warnings
                warnings.warn(f"PARO processor: no grid given, assuming (F, H, W) = {g} for {n_img} image tokens; "
                              "pass grid=(F, H, W) if the latent has another orientation", stacklevel=3)
                self._grid_warned = True
        if g is None or g[0] * g[1] * g[2] != n_img:
            raise ValueError(f"{n_img} image tokens do not match grid {g}: set the processor's `grid` to (F, H, W)")
        return g

    @staticmethod
    def _rope_permute(query, key, value, orders, grid, n_text, cos, sin, rotate_key=True):
        """One launch when q, k, v share strides (plain projections); otherwise (a norm layer returned
        q/k in another memory order than v, or keys that must not be rotated) one launch per group."""
        same = query.stride() == key.stride() == value.stride()
        if same and (rotate_key or cos is None):
            return PM.rope_permute(query, key, value, orders, grid, n_text, cos, sin)
        if rotate_key and query.stride() == key.stride():
            qp, kp, _ = PM.rope_permute(query, key, None, orders, grid, n_text, cos, sin)
        else:
            qp, _, _ = PM.rope_permute(query, None, None, orders, grid, n_text, cos, sin)
            _, kp, _ = PM.rope_permute(None, key, None, orders, grid, n_text,
                                       cos if rotate_key else None, sin if rotate_key else None)
        _, _, vp = PM.rope_permute(None, None, value, orders, grid, n_text)
        return qp, kp, vp

    def _prepare(self, query, key, value, orders, grid, n_text, cos, sin, rotate_key=True):
        """RoPE + permutation + INT8 Q/K + FP8 V in one pass, straight from the projections."""
        if not rotate_key and cos is not None:
            # keys that must not be rotated: rotate the queries separately, then prepare without tables
            query, _, _ = PM.rope_permute(query, None, None, torch.zeros_like(orders), grid, n_text, cos, sin)
            cos = sin = None
        # (smoothing: the mean of the rotated K is taken inside the same call)
        ops = PM.rope_permute_quant(query, key, value, orders, grid, n_text, cos, sin,
                                    km="mean" if self.smooth_k else None)
        if self.pv_f16:
            _, _, vp = PM.rope_permute(None, None, value, orders, grid, n_text)
            ops = ops._replace(v8=qattn.v_f16_tiles(vp), v_scale=None, v_mean=None)
        return ops

    def _sparse_attention(self, ops, out, sm_scale, orders, grid, n_text):
        """Block-sparse attention on the prepared operands; the inverse permutation (permute_attn_out)
        is part of the kernel's stores, `out` is the [B,H,N,D] view of the token-major result."""
        qattn.attn_sparse_prepacked(ops.q8, ops.k8, ops.v8, ops.v_scale, ops.v_mean, out, ops.q_scale, ops.k_scale,
                                    sm_scale, self._mask(), exact_exp=self.exact_exp,
                                    unpermute=(orders, grid, n_text), pv_f16=self.pv_f16)

    def get_time_stats(self):
        self._timer.fold(block=True)
        self.time_accum["total"] = self._timer.total_ms
        return {"total_ms": self.time_accum["total"]}


class PARO_CogVideoXAttnProcessor2_0(_ParoProcessorBase):
    r"""Joint text+video self-attention of CogVideoX with PAROAttention in place of dense SDPA
    (paroattention/cogvideox.py:112-250).  `i_timestep < 0` selects dense SDPA, as there (:215-221)."""

    def _tables(self, image_rotary_emb, device):
        cos, sin = image_rotary_emb
        return SHARED_TABLES.get((cos, sin), device, lambda: (cos, sin))

    def __call__(self, attn, hidden_states: torch.Tensor, encoder_hidden_states: torch.Tensor,
                 attention_mask: Optional[torch.Tensor] = None,
                 image_rotary_emb: Optional[torch.Tensor] = None):
        text_seq_length = encoder_hidden_states.size(1)
        hidden_states = torch.cat([encoder_hidden_states, hidden_states], dim=1)
        batch_size, sequence_length, _ = hidden_states.shape

        query = attn.to_q(hidden_states)
        key = attn.to_k(hidden_states)
        value = attn.to_v(hidden_states)
        head_dim = key.shape[-1] // attn.heads
        # [B,H,N,D] views of the token-major projections: the permutation kernel follows the strides
        query = query.view(batch_size, -1, attn.heads, head_dim).transpose(1, 2)
        key = key.view(batch_size, -1, attn.heads, head_dim).transpose(1, 2)
        value = value.view(batch_size, -1, attn.heads, head_dim).transpose(1, 2)
        if attn.norm_q is not None:
            query = attn.norm_q(query)
        if attn.norm_k is not None:
            key = attn.norm_k(key)

        grid = self._grid_for(sequence_length - text_seq_length, {COG_GRID[0] * COG_GRID[1] * COG_GRID[2]: COG_GRID})
        cos = sin = None
        if image_rotary_emb is not None:
            cos, sin = self._tables(image_rotary_emb, query.device)
        dense = self.i_timestep < 0
        if dense:
            orders = torch.zeros(attn.heads, dtype=torch.int32, device=query.device)   # order 0 = identity
        else:
            orders = self._orders(query.device)
        rotate_key = not getattr(attn, "is_cross_attention", False)   # cogvideox.py:170-172
        done = self._timer.start()
        token_major = torch.empty((batch_size, sequence_length, attn.heads, head_dim), dtype=query.dtype,
                                  device=query.device)
        if dense:
            qp, kp, vp = self._rope_permute(query, key, value, orders, grid, text_seq_length, cos, sin, rotate_key)
            if attention_mask is not None:
                attention_mask = attn.prepare_attention_mask(attention_mask, sequence_length, batch_size)
                attention_mask = attention_mask.view(batch_size, attn.heads, -1, attention_mask.shape[-1])
            out = F.scaled_dot_product_attention(qp, kp, vp, attn_mask=attention_mask, dropout_p=0.0, is_causal=False)
            token_major.copy_(out.transpose(1, 2))
            done.record()
        else:
            ops = self._prepare(query, key, value, orders, grid, text_seq_length, cos, sin, rotate_key)
            self._sparse_attention(ops, token_major.transpose(1, 2), 1.0 / (head_dim ** 0.5), orders, grid,
                                   text_seq_length)
            done.record()
        self.call_count += 1
        if len(self._timer._pending) >= 64:
            self._timer.fold(block=False)

        hidden_states = token_major.view(batch_size, sequence_length, attn.heads * head_dim)
        hidden_states = attn.to_out[0](hidden_states)   # linear projection
        hidden_states = attn.to_out[1](hidden_states)   # dropout
        encoder_hidden_states, hidden_states = hidden_states.split(
            [text_seq_length, hidden_states.size(1) - text_seq_length], dim=1)
        return hidden_states, encoder_hidden_states


# the same class under its name without the diffusers version suffix
PARO_CogVideoXAttnProcessor = PARO_CogVideoXAttnProcessor2_0
