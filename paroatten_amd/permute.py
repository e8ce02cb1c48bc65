"""Fused RoPE + per-head token permutation and its inverse.

Replaces the reference's Python head loops `permute_qk` / `permute_attn_out`
(paroattention/cogvideox.py:22-110, paroattention/wan.py:25-111) and the separate RoPE pass in
front of them (cogvideox.py:167-172, wan.py:161-167) by one launch that reads Q, K, V once and
writes them once, and one launch for the output.  All functions take HND tensors [B,H,N,D].
"""
from __future__ import annotations

from typing import NamedTuple, Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import load, ptr, stream_of

# index -> order of the (F,H,W) axes, and the inverse orders (cogvideox.py:38-45, :85-92)
PERMUTATIONS = ((0, 1, 2), (0, 2, 1), (1, 2, 0), (1, 0, 2), (2, 1, 0), (2, 0, 1))
PERMUTATIONS_INV = ((0, 1, 2), (0, 2, 1), (2, 0, 1), (1, 0, 2), (2, 1, 0), (1, 2, 0))


def head_orders(permute_plan, i_block: int, device) -> torch.Tensor:
    """int32 [H] on `device` from a plan dict {'permute': int[L,H], ...}; values checked 0..5."""
    o = torch.as_tensor(permute_plan["permute"][i_block])
    if o.numel() and (int(o.min()) < 0 or int(o.max()) > 5):
        raise ValueError("permute plan entries must be in 0..5")
    return o.to(device=device, dtype=torch.int32).contiguous()


def _check_hnd(t: torch.Tensor, name: str):
    _lib.require_gpu(t, name)
    if t.dim() != 4:
        raise RuntimeError(f"Tensor {name} must have dimension number (4)")
    if t.dtype not in _lib.DTYPE_CODE:
        raise RuntimeError(f"Tensor {name} must be float16 or bfloat16")
    if t.stride(-1) != 1:
        raise RuntimeError(f"Tensor {name} must be contiguous at the last dimension")


def _check_orders(orders: torch.Tensor, H: int):
    _lib.require_gpu(orders, "orders")
    if orders.dtype != torch.int32 or orders.dim() != 1 or orders.numel() != H or not orders.is_contiguous():
        raise RuntimeError(f"orders must be a contiguous int32 tensor of {H} entries (one per head)")


def rope_permute(q: Optional[torch.Tensor], k: Optional[torch.Tensor], v: Optional[torch.Tensor],
                 orders: torch.Tensor, grid: Sequence[int], n_text: int,
                 cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None
                 ) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor], Optional[torch.Tensor]]:
    """out[b,h,perm_h(t)] = rope(in[b,h,t]) for q and k, permutation only for v; text tokens
    [0,n_text) are copied through.  cos/sin: fp32 [F*H*W, D] (full-width tables, every frequency
    may be repeated over its channel pair as diffusers does); None = no rotation."""
    ref = next(t for t in (q, k, v) if t is not None)
    _check_hnd(ref, "input")
    B, H, N, D = ref.shape
    for t in (q, k, v):
        if t is not None:
            _check_hnd(t, "input")
            if t.shape != ref.shape or t.stride() != ref.stride() or t.dtype != ref.dtype:
                raise RuntimeError("q, k, v must share shape, strides and dtype")
    _check_orders(orders, H)
    F, Hh, W = (int(x) for x in grid)
    if cos is not None:
        for t, n in ((cos, "cos"), (sin, "sin")):
            _lib.require_gpu(t, n)
            if t.dtype != torch.float32 or tuple(t.shape) != (F * Hh * W, D) or not t.is_contiguous():
                raise RuntimeError(f"Tensor {n} must be contiguous float32 of shape ({F * Hh * W}, {D})")
    outs = [None if t is None else torch.empty((B, H, N, D), dtype=t.dtype, device=t.device) for t in (q, k, v)]
    o_ref = next(o for o in outs if o is not None)
    _lib.on(ref).paro_rope_permute_fwd(
        ptr(q), ptr(k), ptr(v), ptr(outs[0]), ptr(outs[1]), ptr(outs[2]), _lib.DTYPE_CODE[ref.dtype],
        ptr(cos), ptr(sin), ptr(orders), B, H, N, D, int(n_text), F, Hh, W,
        ref.stride(0), ref.stride(1), ref.stride(2), o_ref.stride(0), o_ref.stride(1), o_ref.stride(2),
        stream_of(ref))
    return tuple(outs)


class PreparedOperands(NamedTuple):
    """What the attention kernel reads: see rope_permute_quant."""
    q8: torch.Tensor
    q_scale: torch.Tensor
    k8: torch.Tensor
    k_scale: torch.Tensor
    v8: torch.Tensor
    v_scale: torch.Tensor
    v_mean: Optional[torch.Tensor]
    k_mean: Optional[torch.Tensor] = None   # the rotated K mean, when the call computed it itself (km="mean")


def _tables_ok(cos, sin, n_img, D):
    if cos is None:
        return
    for t, n in ((cos, "cos"), (sin, "sin")):
        _lib.require_gpu(t, n)
        if t.dtype != torch.float32 or tuple(t.shape) != (n_img, D) or not t.is_contiguous():
            raise RuntimeError(f"Tensor {n} must be contiguous float32 of shape ({n_img}, {D})")


def rope_k_mean(k: torch.Tensor, grid: Sequence[int], n_text: int, cos: Optional[torch.Tensor] = None,
                sin: Optional[torch.Tensor] = None) -> torch.Tensor:
    """[B,H,1,D] in k's dtype: the token mean of K after the rotation, i.e. the `km` the reference's
    quantiser expects (paroattention/quant.py:105-180) when it runs behind the processor's RoPE."""
    _check_hnd(k, "key")
    B, H, N, D = k.shape
    F, Hh, W = (int(x) for x in grid)
    _tables_ok(cos, sin, F * Hh * W, D)
    lib = load()
    km = torch.empty((B, H, 1, D), dtype=k.dtype, device=k.device)
    ws = torch.empty(int(lib.paro_prep_workspace_bytes(B, H, N, D)), dtype=torch.uint8, device=k.device)
    _lib.on(k).paro_rope_k_mean(ptr(k), _lib.DTYPE_CODE[k.dtype], ptr(cos), ptr(sin), ptr(km), ptr(ws), ws.numel(),
                               B, H, N, D, int(n_text), F, Hh, W, k.stride(0), k.stride(1), k.stride(2),
                               km.stride(0), km.stride(1), stream_of(k))
    return km


def rope_permute_quant(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, orders: torch.Tensor,
                       grid: Sequence[int], n_text: int, cos: Optional[torch.Tensor] = None,
                       sin: Optional[torch.Tensor] = None, km=None,
                       smooth_v: bool = True) -> PreparedOperands:
    """rope_permute + per_warp_int8(BLKQ=64, WARPQ=32, BLKK=64, km) + per_channel_fp8 in one pass, with
    bit-identical INT8 results and without the permuted 16-bit tensors ever being written.  q, k, v:
    [B,H,N,D] views, each with its own strides (e.g. the transposed token-major projections); km: None,
    [B,H,1,D] in the input dtype (see rope_k_mean), or the string "mean": the mean of the rotated K is taken
    inside the same call (its pass over K shares a launch with the V statistics) and returned as the `k_mean`
    field of the result."""
    _check_hnd(q, "query")
    B, H, N, D = q.shape
    for t, n in ((k, "key"), (v, "value")):
        _check_hnd(t, n)
        if t.shape != q.shape or t.dtype != q.dtype:
            raise RuntimeError("q, k, v must share shape and dtype")
    _check_orders(orders, H)
    F, Hh, W = (int(x) for x in grid)
    _tables_ok(cos, sin, F * Hh * W, D)
    ms_b = ms_h = 0
    compute_km = isinstance(km, str)
    if compute_km:
        if km != "mean":
            raise ValueError("km must be None, a tensor, or the string 'mean'")
        km = torch.empty((B, H, 1, D), dtype=q.dtype, device=q.device)
    if km is not None:
        _lib.require_gpu(km, "km")
        if km.dtype != q.dtype or tuple(km.shape) != (B, H, 1, D) or km.stride(-1) != 1:
            raise RuntimeError(f"Tensor km must have shape ({B}, {H}, 1, {D}) and the dtype of key")
        ms_b, ms_h = km.stride(0), km.stride(1)
    lib = load()
    dev = q.device
    nb = (N + 63) // 64
    q8 = torch.empty((B, H, N, D), dtype=torch.int8, device=dev)
    k8 = torch.empty((B, H, N, D), dtype=torch.int8, device=dev)
    q_scale = torch.empty((B, H, nb * 2), dtype=torch.float32, device=dev)
    k_scale = torch.empty((B, H, nb), dtype=torch.float32, device=dev)
    v8 = torch.empty(int(lib.paro_v_fp8_bytes(B, H, N, D)), dtype=torch.uint8, device=dev)
    v_scale = torch.empty((B, H, D), dtype=torch.float32, device=dev)
    v_mean = torch.empty((B, H, D), dtype=torch.float32, device=dev)
    ws_bytes = lib.paro_prep_smooth_workspace_bytes(B, H, N, D) if compute_km else lib.paro_prep_workspace_bytes(B, H, N, D)
    ws = torch.empty(int(ws_bytes), dtype=torch.uint8, device=dev)
    entry = _lib.on(q).paro_rope_k_mean_permute_quant_fwd if compute_km else _lib.on(q).paro_rope_permute_quant_fwd
    entry(
        ptr(q), ptr(k), ptr(v), _lib.DTYPE_CODE[q.dtype], ptr(cos), ptr(sin), ptr(orders), ptr(km),
        ptr(q8), ptr(q_scale), ptr(k8), ptr(k_scale), ptr(v8), ptr(v_scale), ptr(v_mean), ptr(ws), ws.numel(),
        B, H, N, D, int(n_text), F, Hh, W, q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1),
        k.stride(2), v.stride(0), v.stride(1), v.stride(2), ms_b, ms_h, 1 if smooth_v else 0, stream_of(q))
    return PreparedOperands(q8, q_scale, k8, k_scale, v8, v_scale, v_mean if smooth_v else None, km if compute_km else None)


def permute_inverse(o: torch.Tensor, orders: torch.Tensor, grid: Sequence[int], n_text: int,
                    out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[b,h,t] = o[b,h,perm_h(t)]: undoes rope_permute's token order on the attention output.
    `out`, if given, is any [B,H,N,D] view with a contiguous last dimension that does not overlap `o`
    (e.g. the transpose of an [B,N,H,D] buffer, which makes the result token-major for the output
    projection without another pass)."""
    _check_hnd(o, "attn_out")
    B, H, N, D = o.shape
    _check_orders(orders, H)
    F, Hh, W = (int(x) for x in grid)
    if out is None:
        out = torch.empty((B, H, N, D), dtype=o.dtype, device=o.device)
    else:
        _check_hnd(out, "out")
        if out.shape != o.shape or out.dtype != o.dtype or out.device != o.device:
            raise RuntimeError("out must have attn_out's shape, dtype and device")
    _lib.on(o).paro_permute_inv(ptr(o), ptr(out), _lib.DTYPE_CODE[o.dtype], ptr(orders), B, H, N, D, int(n_text),
                                  F, Hh, W, o.stride(0), o.stride(1), o.stride(2),
                                  out.stride(0), out.stride(1), out.stride(2), stream_of(o))
    return out


def permute_index_map(orders: torch.Tensor, grid: Sequence[int]) -> torch.Tensor:
    """int32 [H, F*H*W]: new position of every image token, per head (the integer index law)."""
    _check_orders(orders, orders.numel())
    F, Hh, W = (int(x) for x in grid)
    idx = torch.empty((orders.numel(), F * Hh * W), dtype=torch.int32, device=orders.device)
    _lib.on(idx).paro_permute_index_map(ptr(idx), ptr(orders), orders.numel(), F, Hh, W, stream_of(idx))
    return idx


def permute_qk(query, key, value, permute_plan, i_block, grid=(13, 30, 45), n_text=226):
    """Drop-in for the reference's permute_qk (cogvideox.py:22-62): permutes the image tokens of
    query, key and value IN PLACE per head and returns them.  (F,H,W) and the text length, literals
    in the reference, are arguments with the CogVideoX values as defaults."""
    orders = head_orders(permute_plan, i_block, query.device)
    qo, ko, vo = rope_permute(query, key, value, orders, grid, n_text)
    query.copy_(qo)
    key.copy_(ko)
    value.copy_(vo)
    return query, key, value


def permute_attn_out(attn_out, permute_plan, i_block, grid=(13, 30, 45), n_text=226):
    """Drop-in for the reference's permute_attn_out (cogvideox.py:64-110), in place."""
    orders = head_orders(permute_plan, i_block, attn_out.device)
    attn_out.copy_(permute_inverse(attn_out, orders, grid, n_text))
    return attn_out
