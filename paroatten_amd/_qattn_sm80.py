"""Mirror of the reference's `paroattention._qattn_sm80` extension module
(csrc/qattn/pybind_sm80.cpp:21-27, csrc/qattn/attn_cuda_sm80.h:19-69).

`qk_int8_sv_f16_accum_f16_attn` keeps the reference's positional signature, integer flags,
validation order and messages (csrc/qattn/qk_int_sv_f16_cuda_sm80.cu:905-1080) and runs the
gfx950 kernels of libparoatten_hip.so: V -> FP8 tiles, then INT8 QK^T / online softmax / FP8 P.V
with fp32 accumulation.  The module keeps the reference's name although nothing here is sm80:
callers import it under that name (paroattention/core.py:3, paroattention/cogvideox.py:13).

Differences, all relaxations or added checks:
  * `value` may be float16 (as in the reference) or bfloat16 (saves the caller's `.to(float16)`);
  * keyword `exact_exp=True` evaluates the softmax exponentials in fp32 before the FP8 rounding instead
    of building the e4m3 byte directly (slower, slightly more accurate; always on with return_lse);
  * keyword `pv_f16=True` is the accuracy mode (PARO_ATTN_PV_F16): the P.V product in float16 with fp32
    accumulation, as the reference's kernel of this name computes it, instead of FP8 e4m3 P and V: true
    exponentials, V as given (smooth_v has nothing to act on); about half the speed;
  * `qk_quant_gran=3` (per thread: eight q scales per 32 rows, four k scales per 64 keys, indexed as
    csrc/qattn/qk_int_sv_f16_cuda_sm80.cu:112-116, 129-133) runs the two-wave kernel;
    quant.per_thread_int8 makes such scales (the reference has no quantiser for them);
  * keyword `pacing=True/False` picks the launch form of the attention kernel (see PARO_ATTN_PACED in
    include/paroatten.h; bit-identical results), None leaves it to the library;
  * `sparse` IS validated (the reference reads it through a raw pointer unchecked): bool or uint8,
    on the GPU, contiguous, shape [B,H,nbq,nbk] or [H,nbq,nbk] (shared by the batch);
  * the INT4 and INT8-P.V variants registered by the reference are experimental prototypes with
    no working caller; they raise NotImplementedError here.
"""
from __future__ import annotations

import torch

from . import _lib
from ._lib import load, ptr, stream_of


def _chk(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _flags(exact_exp, pacing, two_waves=False, pv_f16=False):
    """pacing: None (the library chooses), True (PARO_ATTN_PACED) or False (PARO_ATTN_UNPACED); two_waves:
    PARO_ATTN_TWO_WAVES.  Launch and kernel form only: results are bit-identical.  pv_f16: PARO_ATTN_PV_F16, the
    float16 P.V product."""
    f = _lib.PARO_ATTN_EXACT_EXP if exact_exp else 0
    if pv_f16:
        f |= _lib.PARO_ATTN_PV_F16
    if pacing is not None:
        f |= _lib.PARO_ATTN_PACED if pacing else _lib.PARO_ATTN_UNPACED
    if two_waves:
        f |= _lib.PARO_ATTN_TWO_WAVES
    return f


def workspace_bytes(B, Hkv, Nk, D, pv_f16=False):
    if pv_f16:
        return int(load().paro_attn_workspace_bytes_for(B, Hkv, Nk, D, _lib.PARO_ATTN_PV_F16))
    return int(load().paro_attn_workspace_bytes(B, Hkv, Nk, D))


def v_f16_tiles(value, tensor_layout="HND"):
    """V [B,Hkv,N,D] ("HND") or [B,N,Hkv,D] ("NHD"), float16 or bfloat16 -> the float16 tiles that the attention
    kernel's accuracy mode reads (paro_v_f16_pack): uint8 tensor of paro_v_f16_bytes() bytes."""
    _chk(value.is_cuda and value.dim() == 4 and value.stride(-1) == 1 and value.dtype in _lib.DTYPE_CODE,
         "Tensor value must be a float16/bfloat16 GPU tensor [B,H,N,D] with a contiguous last dimension")
    if tensor_layout == "NHD":
        value = value.transpose(1, 2)
    B, Hkv, N, D = value.shape
    out = torch.empty(int(load().paro_v_f16_bytes(B, Hkv, N, D)), dtype=torch.uint8, device=value.device)
    _lib.on(value).paro_v_f16_pack(ptr(value), _lib.DTYPE_CODE[value.dtype], ptr(out), B, Hkv, N, D,
                                   value.stride(0), value.stride(1), value.stride(2), stream_of(value))
    return out


def qk_int8_sv_f16_accum_f16_attn(query, key, value, output, query_scale, key_scale, tensor_layout, is_causal,
                                  qk_quant_gran, sm_scale, return_lse, sparse, *, smooth_v=True, exact_exp=False,
                                  workspace=None, pacing=None, two_waves=False, pv_f16=False):
    for t, n in ((query, "query"), (key, "key"), (value, "value"), (output, "output"),
                 (query_scale, "query_scale"), (key_scale, "key_scale")):
        _chk(t.is_cuda, f"Tensor {n} must be on CUDA")
    _chk(query.is_contiguous(), "Tensor query must be contiguous")
    _chk(key.is_contiguous(), "Tensor key must be contiguous")
    _chk(value.stride(-1) == 1, "Tensor value must be contiguous at the last dimension")
    _chk(output.stride(-1) == 1, "Tensor output must be contiguous at the last dimension")
    _chk(query_scale.is_contiguous(), "Tensor query_scale must be contiguous")
    _chk(key_scale.is_contiguous(), "Tensor key_scale must be contiguous")
    _chk(query.dtype == torch.int8, "Tensor query must have dtype (torch::kInt8)")
    _chk(key.dtype == torch.int8, "Tensor key must have dtype (torch::kInt8)")
    _chk(value.dtype in (torch.float16, torch.bfloat16), "Tensor value must have dtype (torch::kHalf)")
    _chk(query_scale.dtype == torch.float32, "Tensor query_scale must have dtype (torch::kFloat32)")
    _chk(key_scale.dtype == torch.float32, "Tensor key_scale must have dtype (torch::kFloat32)")
    for t, n, d in ((query, "query", 4), (key, "key", 4), (value, "value", 4), (output, "output", 4),
                    (query_scale, "query_scale", 3), (key_scale, "key_scale", 3)):
        _chk(t.dim() == d, f"Tensor {n} must have dimension number ({d})")
    D, B = query.size(3), query.size(0)
    if tensor_layout == 0:
        Nq, Nk, H, Hkv = query.size(1), key.size(1), query.size(2), key.size(2)
        _chk(tuple(key.shape) == (B, Nk, Hkv, D), "Tensor key must have shape (batch_size, kv_len, num_kv_heads, head_dim)")
        _chk(tuple(value.shape) == (B, Nk, Hkv, D), "Tensor value must have shape (batch_size, kv_len, num_kv_heads, head_dim)")
        sn, sh = 1, 2
    elif tensor_layout == 1:
        Nq, Nk, H, Hkv = query.size(2), key.size(2), query.size(1), key.size(1)
        _chk(tuple(key.shape) == (B, Hkv, Nk, D), "Tensor key must have shape (batch_size, num_kv_heads, kv_len, head_dim)")
        _chk(tuple(value.shape) == (B, Hkv, Nk, D), "Tensor value must have shape (batch_size, num_kv_heads, kv_len, head_dim)")
        sn, sh = 2, 1
    else:
        raise ValueError("tensor_layout must be 0 or 1")
    if H % Hkv != 0:
        raise ValueError(f"num_qo_heads ({H}) must be divisible by num_kv_heads ({Hkv})")
    if D not in (64, 128):
        raise ValueError(f"Unsupported head dim: {D}")
    if is_causal not in (0, 1):
        raise ValueError(f"Unsupported causal mode: {int(is_causal)}")
    if qk_quant_gran not in (2, 3):
        raise ValueError(f"Unsupported qk_quant_gran: {int(qk_quant_gran)}")
    if return_lse not in (0, 1):
        raise ValueError(f"Unsupported causal mode: {int(return_lse)}")  # sic: the reference's text
    if output.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError(f"qk_int8_sv_f16_accum_f16_attn failed to dispatch data type {output.dtype}")
    _chk(tuple(output.shape) == tuple(query.shape), "Tensor output must have the shape of query")
    nbq, nbk = (Nq + 63) // 64, (Nk + 63) // 64
    if qk_quant_gran == 2:
        _chk(tuple(query_scale.shape) == (B, H, nbq * 2),
             "Tensor query_scale must have shape (batch_size, num_qo_heads, div_ceil(qo_len, CTA_Q) * (CTA_Q / WARP_Q))")
        _chk(tuple(key_scale.shape) == (B, Hkv, nbk),
             "Tensor key_scale must have shape (batch_size, num_kv_heads, div_ceil(kv_len, CTA_K) * (CTA_K / WARP_K))")
    else:   # per thread (csrc/qattn/qk_int_sv_f16_cuda_sm80.cu:1034-1038)
        _chk(tuple(query_scale.shape) == (B, H, nbq * 2 * 8),
             "Tensor query_scale must have shape (batch_size, num_qo_heads, div_ceil(qo_len, CTA_Q) * (CTA_Q / WARP_Q) * 8)")
        _chk(tuple(key_scale.shape) == (B, Hkv, nbk * 4),
             "Tensor key_scale must have shape (batch_size, num_kv_heads, div_ceil(kv_len, CTA_K) * (CTA_K / WARP_K) * 4)")
        if pv_f16:
            raise NotImplementedError("qk_quant_gran 3 (per thread) is not available with pv_f16")
    # the mask: checked here, unlike the reference
    _chk(sparse.is_cuda, "Tensor sparse must be on CUDA")
    _chk(sparse.dtype in (torch.bool, torch.uint8), "Tensor sparse must have dtype (torch::kBool)")
    _chk(sparse.is_contiguous(), "Tensor sparse must be contiguous")
    if sparse.dim() == 4:
        _chk(tuple(sparse.shape) == (B, H, nbq, nbk),
             f"Tensor sparse must have shape (batch_size, num_qo_heads, {nbq}, {nbk}), got {tuple(sparse.shape)}")
        sparse_bs = sparse.stride(0)
    else:
        _chk(sparse.dim() == 3 and tuple(sparse.shape) == (H, nbq, nbk),
             f"Tensor sparse must have shape ([batch_size,] num_qo_heads, {nbq}, {nbk}), got {tuple(sparse.shape)}")
        sparse_bs = 0
    lse = torch.empty(0)
    if return_lse:
        lse = torch.empty((B, H, Nq), dtype=torch.float32, device=query.device)
    need = workspace_bytes(B, Hkv, Nk, D, pv_f16)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=query.device)
    else:
        _chk(workspace.is_cuda and workspace.is_contiguous() and workspace.numel() * workspace.element_size() >= need,
             f"workspace must be a contiguous GPU buffer of at least {need} bytes")
    _lib.on(query).paro_qk_int8_sv_f16_attn(
        ptr(query), ptr(key), ptr(value), _lib.DTYPE_CODE[value.dtype], ptr(output), _lib.DTYPE_CODE[output.dtype],
        ptr(query_scale), ptr(key_scale), ptr(sparse), sparse_bs, ptr(lse) if return_lse else None,
        ptr(workspace), workspace.numel() * workspace.element_size(),
        B, H, Hkv, Nq, Nk, D,
        query.stride(0), query.stride(sh), query.stride(sn),
        key.stride(0), key.stride(sh), key.stride(sn),
        value.stride(0), value.stride(sh), value.stride(sn),
        output.stride(0), output.stride(sh), output.stride(sn),
        tensor_layout, is_causal, qk_quant_gran, float(sm_scale), 1 if smooth_v else 0,
        _flags(exact_exp, pacing, two_waves, pv_f16), stream_of(query))
    return lse


def attn_sparse_prepacked(q8, k8, v8, v_scale, v_mean, output, query_scale, key_scale, sm_scale, sparse,
                          is_causal=0, return_lse=0, exact_exp=False, unpermute=None, pacing=None,
                          two_waves=False, pv_f16=False):
    """The attention kernel alone, on operands that are already in its formats (HND, contiguous):
    q8/k8 int8 [B,H,N,D] / [B,Hkv,Nk,D], v8 = FP8 tiles from paro_v_fp8_pack or the fused
    preparation, v_scale / v_mean f32 [B,Hkv,D] (v_mean None: V was not mean-smoothed).  With pv_f16=True
    v8 holds the float16 tiles of v_f16_tiles() and v_scale / v_mean may be None.  No
    counterpart in the reference, whose extension converts V on every call."""
    for t, n in ((q8, "query"), (k8, "key"), (v8, "value"), (output, "output"), (query_scale, "query_scale"),
                 (key_scale, "key_scale"), (v_scale, "v_scale"), (sparse, "sparse")):
        if t is None and pv_f16 and n == "v_scale":
            continue
        _chk(t.is_cuda, f"Tensor {n} must be on CUDA")
        _chk(t.is_contiguous() or n == "output", f"Tensor {n} must be contiguous")
    _chk(q8.dtype == torch.int8 and k8.dtype == torch.int8, "Tensor query/key must have dtype (torch::kInt8)")
    _chk(q8.dim() == 4 and k8.dim() == 4, "Tensor query/key must have dimension number (4)")
    B, H, Nq, D = q8.shape
    Hkv, Nk = k8.size(1), k8.size(2)
    if D not in (64, 128):
        raise ValueError(f"Unsupported head dim: {D}")
    if H % Hkv != 0:
        raise ValueError(f"num_qo_heads ({H}) must be divisible by num_kv_heads ({Hkv})")
    nbq, nbk = (Nq + 63) // 64, (Nk + 63) // 64
    if pv_f16:
        _chk(v8.numel() * v8.element_size() == load().paro_v_f16_bytes(B, Hkv, Nk, D),
             "Tensor value has the wrong size for float16 tiles")
    else:
        _chk(v8.numel() * v8.element_size() == load().paro_v_fp8_bytes(B, Hkv, Nk, D),
             "Tensor value has the wrong size for FP8 tiles")
    _chk(tuple(query_scale.shape) == (B, H, nbq * 2) and tuple(key_scale.shape) == (B, Hkv, nbk),
         "Tensor query_scale / key_scale must have shapes (B, H, 2*nbq) / (B, Hkv, nbk)")
    _chk((v_scale is None and pv_f16 or tuple(v_scale.shape) == (B, Hkv, D))
         and (v_mean is None or tuple(v_mean.shape) == (B, Hkv, D)),
         "Tensor v_scale / v_mean must have shape (B, Hkv, head_dim)")
    _chk(tuple(output.shape) == (B, H, Nq, D) and output.stride(-1) == 1 and output.dtype in _lib.DTYPE_CODE,
         "Tensor output must be float16/bfloat16 [B,H,N,D] with a contiguous last dimension")
    _chk(sparse.dtype in (torch.bool, torch.uint8), "Tensor sparse must have dtype (torch::kBool)")
    if sparse.dim() == 4:
        _chk(tuple(sparse.shape) == (B, H, nbq, nbk), f"Tensor sparse must have shape ({B}, {H}, {nbq}, {nbk})")
        sparse_bs = sparse.stride(0)
    else:
        _chk(tuple(sparse.shape) == (H, nbq, nbk), f"Tensor sparse must have shape ([{B},] {H}, {nbq}, {nbk})")
        sparse_bs = 0
    lse = torch.empty((B, H, Nq), dtype=torch.float32, device=q8.device) if return_lse else torch.empty(0)
    flags = _flags(exact_exp, pacing, two_waves, pv_f16)
    strides = (q8.stride(0), q8.stride(1), q8.stride(2), k8.stride(0), k8.stride(1), k8.stride(2),
               output.stride(0), output.stride(1), output.stride(2))
    if unpermute is None:
        _lib.on(q8).paro_attn_sparse_fwd(
            ptr(q8), ptr(k8), ptr(v8), ptr(query_scale), ptr(key_scale), ptr(v_scale), ptr(v_mean), ptr(sparse),
            sparse_bs, ptr(output), _lib.DTYPE_CODE[output.dtype], ptr(lse) if return_lse else None, None,
            B, H, Hkv, Nq, Nk, D, *strides, float(sm_scale), int(is_causal), flags, stream_of(q8))
    else:
        orders, grid, n_text = unpermute
        _chk(orders.is_cuda and orders.dtype == torch.int32 and orders.dim() == 1 and orders.numel() == H
             and orders.is_contiguous(), f"orders must be a contiguous int32 GPU tensor of {H} entries")
        F_, Hh, W = (int(x) for x in grid)
        _lib.on(q8).paro_attn_sparse_unpermute_fwd(
            ptr(q8), ptr(k8), ptr(v8), ptr(query_scale), ptr(key_scale), ptr(v_scale), ptr(v_mean), ptr(sparse),
            sparse_bs, ptr(output), _lib.DTYPE_CODE[output.dtype], ptr(lse) if return_lse else None,
            B, H, Hkv, Nq, Nk, D, *strides, float(sm_scale), int(is_causal), flags,
            ptr(orders), int(n_text), F_, Hh, W, stream_of(q8))
    return lse


def _prototype(name):
    def fn(*args, **kwargs):
        raise NotImplementedError(
            f"{name}: experimental variant of the reference (INT4 Q/K or INT8 P.V) without a working "
            "caller; gfx950 has no int4 MFMA and the INT8 P.V prototype is numerically unsound. "
            "Use qk_int8_sv_f16_accum_f16_attn.")
    fn.__name__ = name
    return fn


qk_int4_sv_f16_accum_f16_attn = _prototype("qk_int4_sv_f16_accum_f16_attn")
qk_int4_sv_int8_accum_f16_attn = _prototype("qk_int4_sv_int8_accum_f16_attn")
qk_int8_sv_int8_accum_f16_attn = _prototype("qk_int8_sv_int8_accum_f16_attn")
