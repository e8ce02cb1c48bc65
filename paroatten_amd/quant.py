"""Q/K INT8 and V FP8 quantisation wrappers: the reference's `paroattention.quant`
(paroattention/quant.py:22-293) with the same names, arguments, defaults and return shapes.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _fused, _lib
from ._lib import load, ptr, stream_of


def _dims(t: torch.Tensor, tensor_layout: str):
    if tensor_layout == "HND":
        b, h, n, d = t.shape
    elif tensor_layout == "NHD":
        b, n, h, d = t.shape
    else:
        raise ValueError(f"Unknown tensor layout: {tensor_layout}")
    return b, h, n, d


def _quant_k(k, km, k_int8, k_scale, BLKK, layout_flag):
    if km is not None:
        km = km.squeeze(1) if layout_flag == 0 else km.squeeze(2)
        _fused.quant_per_block_int8_fuse_sub_mean_cuda(k, km, k_int8, k_scale, BLKK, layout_flag)
    else:
        _fused.quant_per_block_int8_cuda(k, k_int8, k_scale, BLKK, layout_flag)


def per_block_int8(q, k, km: Optional[torch.Tensor] = None, BLKQ: int = 128, BLKK: int = 64,
                   sm_scale: Optional[float] = None, tensor_layout: str = "HND"):
    """One scale per BLKQ query tokens / BLKK key tokens; `sm_scale * 1.44269504` is folded into
    Q before quantisation (paroattention/quant.py:22-103).  Returns
    (q_int8, q_scale [B,Hq,ceil(Nq/BLKQ)], k_int8, k_scale [B,Hkv,ceil(Nk/BLKK)])."""
    b, h_qo, qo_len, head_dim = _dims(q, tensor_layout)
    _, h_kv, kv_len, _ = _dims(k, tensor_layout)
    layout_flag = 0 if tensor_layout == "NHD" else 1
    q_int8 = torch.empty(q.shape, dtype=torch.int8, device=q.device)
    k_int8 = torch.empty(k.shape, dtype=torch.int8, device=k.device)
    q_scale = torch.empty((b, h_qo, (qo_len + BLKQ - 1) // BLKQ), device=q.device, dtype=torch.float32)
    k_scale = torch.empty((b, h_kv, (kv_len + BLKK - 1) // BLKK), device=q.device, dtype=torch.float32)
    if sm_scale is None:
        sm_scale = head_dim ** -0.5
    sm_scale *= 1.44269504
    _fused.quant_per_block_int8_cuda(q, q_int8, q_scale, sm_scale, BLKQ, layout_flag)
    _quant_k(k, km, k_int8, k_scale, BLKK, layout_flag)
    return q_int8, q_scale, k_int8, k_scale


def per_warp_int8(q, k, km: Optional[torch.Tensor] = None, BLKQ: int = 128, WARPQ: int = 32, BLKK: int = 64,
                  tensor_layout: str = "HND"):
    """One scale per WARPQ query tokens (ceil(Nq/BLKQ)*(BLKQ/WARPQ) of them) and per BLKK key
    tokens; no softmax scale folded in (paroattention/quant.py:105-180).  `km` [B,Hkv,1,D] (HND) is
    subtracted from K before quantisation (K mean-smoothing)."""
    b, h_qo, qo_len, head_dim = _dims(q, tensor_layout)
    _, h_kv, kv_len, _ = _dims(k, tensor_layout)
    layout_flag = 0 if tensor_layout == "NHD" else 1
    q_int8 = torch.empty(q.shape, dtype=torch.int8, device=q.device)
    k_int8 = torch.empty(k.shape, dtype=torch.int8, device=k.device)
    q_scale = torch.empty((b, h_qo, ((qo_len + BLKQ - 1) // BLKQ) * (BLKQ // WARPQ)), device=q.device,
                          dtype=torch.float32)
    k_scale = torch.empty((b, h_kv, (kv_len + BLKK - 1) // BLKK), device=q.device, dtype=torch.float32)
    _fused.quant_per_warp_int8_cuda(q, q_int8, q_scale, BLKQ, WARPQ, layout_flag)
    _quant_k(k, km, k_int8, k_scale, BLKK, layout_flag)
    return q_int8, q_scale, k_int8, k_scale


def per_thread_int8(q, k, km: Optional[torch.Tensor] = None, tensor_layout: str = "HND"):
    """Scales of the attention kernel's per-thread granularity (qk_quant_gran 3: csrc/qattn/
    qk_int_sv_f16_cuda_sm80.cu:112-116, 129-133, shapes :1034-1038): eight per 32 query tokens (scale g for the
    tokens r with r % 8 == g), four per 64 key tokens (scale j for the tokens c with (c % 8) / 2 == j), the same
    arithmetic as per_warp_int8 otherwise.  The reference has no quantiser of this granularity (its
    paroattention/core.py:204-205 calls the per-block one); the grouping is the one its kernel's indexing implies.
    Returns (q_int8, q_scale [B,Hq,ceil(Nq/64)*16], k_int8, k_scale [B,Hkv,ceil(Nk/64)*4])."""
    layout_flag = 0 if tensor_layout == "NHD" else 1
    outs = []
    for x, mean, is_key in ((q, None, 0), (k, km, 1)):
        b, h, n, d = _dims(x, tensor_layout)
        _lib.require_gpu(x, "k" if is_key else "q")
        if x.dtype not in (torch.float16, torch.bfloat16):
            raise RuntimeError(f"per_thread_int8 failed to dispatch data type {x.dtype}")
        if d not in (64, 128):
            raise ValueError(f"Unsupported head dim: {d}")
        if x.stride(-1) != 1:
            raise RuntimeError("Tensor input must be contiguous at the last dimension")
        x8 = torch.empty(x.shape, dtype=torch.int8, device=x.device)
        scale = torch.empty((b, h, (n + 63) // 64 * (4 if is_key else 16)), dtype=torch.float32, device=x.device)
        xs_n, xs_h = (x.stride(1), x.stride(2)) if layout_flag == 0 else (x.stride(2), x.stride(1))
        os_n, os_h = (x8.stride(1), x8.stride(2)) if layout_flag == 0 else (x8.stride(2), x8.stride(1))
        ms_b = ms_h = 0
        if mean is not None:
            mean = mean.squeeze(1) if layout_flag == 0 else mean.squeeze(2)
            if tuple(mean.shape) != (b, h, d) or mean.dtype != x.dtype or mean.stride(-1) != 1:
                raise RuntimeError("Tensor mean must have shape (batch_size, num_heads, head_dim), the input's dtype "
                                   "and a contiguous last dimension")
            ms_b, ms_h = mean.stride(0), mean.stride(1)
        _lib.on(x).paro_quant_int8_per_thread(ptr(x), _lib.DTYPE_CODE[x.dtype], ptr(mean), ptr(x8), ptr(scale), b, h, n, d,
                                              x.stride(0), xs_h, xs_n, ms_b, ms_h, x8.stride(0), os_h, os_n, is_key,
                                              stream_of(x))
        outs += [x8, scale]
    return tuple(outs)


def sub_mean(v: torch.Tensor, tensor_layout: str = "HND"):
    """(v - mean over tokens) as float16, and the mean in v's dtype (paroattention/quant.py:182-222)."""
    layout_flag = 0 if tensor_layout == "NHD" else 1
    vm = v.mean(dim=1 if layout_flag == 0 else 2)
    v_smoothed = torch.empty(v.shape, dtype=torch.float16, device=v.device)
    _fused.sub_mean_cuda(v, vm, v_smoothed, layout_flag)
    return v_smoothed, vm


def per_channel_fp8(v: torch.Tensor, tensor_layout: str = "HND", scale_max: float = 448.0, smooth_v: bool = True,
                    tile_order: bool = True):
    """V -> float8_e4m3fn with one scale (and, if smooth_v, one mean) per (batch, head, channel)
    (paroattention/quant.py:224-293).  Returns (v_fp8, v_scale [B,H,D] f32, vm [B,H,D] f32 or None).

    v_fp8 has the reference's shape ([B,H,D,ceil64(N)] for HND, [B,D,H,ceil64(N)] for NHD) and
    byte count, but its bytes are in the 64-token MFMA tile order this library's attention kernel
    reads (include/paroatten.h, paro_v_fp8_pack), grouped [B,H,tile,...] for either layout, where
    the reference's are in the fragment order of NVIDIA's fp8 mma.  The mean divides by the true
    token count, and `vm` is the offset the attention epilogue adds back: that mean plus the mean rounding
    residual of the channel's codes.

    tile_order=False runs the reference's own sequence instead (transpose_pad_permute_cuda, then
    mean_scale_fuse_quant_cuda or scale_fuse_quant_cuda): bytes in the reference's order, statistics over
    ceil16(N) tokens, any scale_max.  Nothing in this library consumes that form."""
    if not tile_order:
        b, h, n, d = _dims(v, tensor_layout)
        layout_flag = 0 if tensor_layout == "NHD" else 1
        padded = (n + 63) // 64 * 64
        shape = (b, h, d, padded) if tensor_layout == "HND" else (b, d, h, padded)
        vt = torch.empty(shape, dtype=v.dtype, device=v.device)
        _fused.transpose_pad_permute_cuda(v, vt, layout_flag)
        v_fp8 = torch.empty(shape, dtype=torch.float8_e4m3fn, device=v.device)
        v_scale = torch.empty((b, h, d), dtype=torch.float32, device=v.device)
        if smooth_v:
            vm = torch.empty((b, h, d), dtype=torch.float32, device=v.device)
            _fused.mean_scale_fuse_quant_cuda(vt, v_fp8, vm, v_scale, n, scale_max, layout_flag)
            return v_fp8, v_scale, vm
        _fused.scale_fuse_quant_cuda(vt, v_fp8, v_scale, n, scale_max, layout_flag)
        return v_fp8, v_scale, None
    if scale_max != 448.0:
        raise ValueError("per_channel_fp8: only scale_max=448.0 (the e4m3 maximum) is supported")
    b, h, n, d = _dims(v, tensor_layout)
    _lib.require_gpu(v, "v")
    if v.dtype not in _lib.DTYPE_CODE:
        raise RuntimeError(f"per_channel_fp8 failed to dispatch data type {v.dtype}")
    if v.stride(-1) != 1:
        raise RuntimeError("Tensor v must be contiguous at the last dimension")
    lib = load()
    padded = (n + 63) // 64 * 64
    shape = (b, h, d, padded) if tensor_layout == "HND" else (b, d, h, padded)
    v_fp8 = torch.empty(shape, dtype=torch.float8_e4m3fn, device=v.device)
    v_scale = torch.empty((b, h, d), dtype=torch.float32, device=v.device)
    vm = torch.empty((b, h, d), dtype=torch.float32, device=v.device)
    partial = torch.empty(int(lib.paro_v_fp8_partial_floats(b, h, n, d)), dtype=torch.float32, device=v.device)
    sn, sh = (2, 1) if tensor_layout == "HND" else (1, 2)
    _lib.on(v).paro_v_fp8_pack(ptr(v), _lib.DTYPE_CODE[v.dtype], ptr(v_fp8), ptr(v_scale), ptr(vm), ptr(partial),
                              b, h, n, d, v.stride(0), v.stride(sh), v.stride(sn), 1 if smooth_v else 0,
                              stream_of(v))
    return v_fp8, v_scale, (vm if smooth_v else None)
