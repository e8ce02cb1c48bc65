"""Operator entry points: the reference's `paroattention.core` (paroattention/core.py:13-216).

`paroattn_qk_int8_pv_fp16_cuda` keeps its name, arguments, defaults and return convention although
P.V now runs in FP8 on the MFMA units with fp32 accumulation (the name is the API, not the
arithmetic).  `paroattn`, which cannot run in the reference (an interactive breakpoint and a
keyword call into a positional binding, core.py:80-83), keeps its signature and forwards here.
"""
from __future__ import annotations

from typing import Any, Optional

import torch

from . import _qattn_sm80 as qattn
from .quant import per_thread_int8
from .quant import per_warp_int8 as per_warp_int8_cuda


def paroattn(q, k, v, tensor_layout: str = "HND", is_causal: bool = False, sm_scale: Optional[float] = None,
             return_lse: bool = False, sparse: Optional[torch.Tensor] = None, **kwargs: Any):
    """Block-sparse quantised attention, layout/shape conventions as below.  `sparse=None` means
    every block is kept (dense)."""
    if sparse is None:
        seq_dim = 1 if tensor_layout == "NHD" else 2
        head_dim_ = 2 if tensor_layout == "NHD" else 1
        nbq = (q.size(seq_dim) + 63) // 64
        nbk = (k.size(seq_dim) + 63) // 64
        sparse = torch.ones((q.size(head_dim_), nbq, nbk), dtype=torch.bool, device=q.device)
    return paroattn_qk_int8_pv_fp16_cuda(q, k, v, sparse, tensor_layout=tensor_layout, is_causal=is_causal,
                                         sm_scale=sm_scale, return_lse=return_lse, **kwargs)


@torch.compiler.disable
def paroattn_qk_int8_pv_fp16_cuda(q, k, v, sparse, tensor_layout: str = "HND", is_causal: bool = False,
                                  qk_quant_gran: str = "per_warp", sm_scale: Optional[float] = None,
                                  return_lse: bool = False, smooth_k: bool = False, smooth_v: bool = True,
                                  exact_exp: bool = False, two_waves: bool = False, pv_f16: bool = False, **kwargs: Any):
    """INT8 Q.K^T, FP8 P.V block-sparse attention.

    q [B,Hq,Nq,D] / k, v [B,Hkv,Nk,D] ("HND") or [B,N,H,D] ("NHD"), float16 or bfloat16, same
    device and dtype, last dim contiguous; D <= 128 (padded to 64 or 128).  sparse: bool
    [B,Hq,ceil(Nq/64),ceil(Nk/64)] or [Hq,..] shared by the batch, True = compute that 64x64 block.
    Returns o (q's dtype and shape) or (o, lse) with lse the natural-log sum-exp per row.
    smooth_k subtracts the per-(batch,head) token mean of K before quantisation (softmax is
    invariant to it; the returned lse is corrected by sm_scale * q . mean, so it is that of the given q and k); smooth_v does the same for V inside the FP8 conversion and adds the mean back;
    exact_exp trades speed for fp32-evaluated softmax exponentials (see _qattn_sm80); two_waves picks the
    two-waves-per-q-block kernel where the library would take the one-wave one (bit-identical results);
    pv_f16 is the accuracy mode: the P.V product in float16 with fp32 accumulation, as the reference computes
    it (qk_int8_sv_f16_accum_f16_attn), instead of FP8 e4m3: about half the speed, float16 instead of e4m3 error
    on rows that a few keys dominate.
    """
    dtype = q.dtype
    assert q.is_cuda, "Input tensors must be on cuda."
    assert dtype in [torch.float16, torch.bfloat16], "Input tensors must be in dtype of torch.float16 or torch.bfloat16"
    assert qk_quant_gran in ["per_warp", "per_thread"], "qk_quant_gran must be either 'per_warp' or 'per_thread'."
    assert q.device == k.device == v.device, "All tensors must be on the same device."
    assert q.dtype == k.dtype == v.dtype, "All tensors must have the same dtype."
    if qk_quant_gran == "per_thread" and pv_f16:
        raise NotImplementedError("qk_quant_gran='per_thread' is not available with pv_f16")

    # launch on the tensors' device, as the reference's set_device workaround does (core.py:168-174)
    with torch.cuda.device(v.device):
        layout_flag = 0 if tensor_layout == "NHD" else 1
        head_dim_og = q.size(-1)
        if head_dim_og < 64:
            pad = 64 - head_dim_og
        elif 64 < head_dim_og < 128:
            pad = 128 - head_dim_og
        elif head_dim_og > 128:
            raise ValueError(f"Unsupported head_dim: {head_dim_og}")
        else:
            pad = 0
        if pad:
            q = torch.nn.functional.pad(q, (0, pad))
            k = torch.nn.functional.pad(k, (0, pad))
            v = torch.nn.functional.pad(v, (0, pad))
        assert q.stride(-1) == 1 and k.stride(-1) == 1 and v.stride(-1) == 1, "Last dim of qkv must be contiguous."
        if sm_scale is None:
            sm_scale = head_dim_og ** -0.5
        seq_dim = 1 if layout_flag == 0 else 2
        km = k.mean(dim=seq_dim, keepdim=True) if smooth_k else None
        if qk_quant_gran == "per_thread":
            # (core.py:204-205 of the reference pairs per-block scales, softmax scale folded in, with the kernel's
            # per-thread path, whose shape check rejects them; here the scales are made at that granularity)
            q_int8, q_scale, k_int8, k_scale = per_thread_int8(q, k, km, tensor_layout=tensor_layout)
        else:
            q_int8, q_scale, k_int8, k_scale = per_warp_int8_cuda(q, k, km, BLKQ=64, WARPQ=32, BLKK=64,
                                                                  tensor_layout=tensor_layout)
        o = torch.empty(q.size(), dtype=dtype, device=q.device)
        lse = qattn.qk_int8_sv_f16_accum_f16_attn(q_int8, k_int8, v, o, q_scale, k_scale, layout_flag,
                                                  1 if is_causal else 0, 3 if qk_quant_gran == "per_thread" else 2,
                                                  sm_scale, 1 if return_lse else 0,
                                                  sparse, smooth_v=smooth_v, exact_exp=exact_exp,
                                                  two_waves=two_waves, pv_f16=pv_f16)
        o = o[..., :head_dim_og]
        if return_lse:
            lse = lse / 1.44269504
            if km is not None:
                # the kernel saw K - km: every score of row i is lower by sm_scale * q_i . km, which the softmax
                # does not notice but the log-sum-exp does; put it back, so that lse is that of the scores of q
                # and k as given (what a caller that merges partial results over key ranges needs)
                groups = q.size(2 if layout_flag == 0 else 1) // km.size(2 if layout_flag == 0 else 1)
                if layout_flag == 0:   # q [B,N,H,D], km [B,1,Hkv,D]
                    kmh = km.float().repeat_interleave(groups, dim=2)
                    corr = torch.stack([(q[b].float() * kmh[b]).sum(-1).transpose(0, 1) for b in range(q.size(0))])
                else:                  # q [B,H,N,D], km [B,Hkv,1,D]
                    kmh = km.float().repeat_interleave(groups, dim=1)
                    corr = torch.stack([torch.bmm(q[b].float(), kmh[b].transpose(1, 2)).squeeze(-1)
                                        for b in range(q.size(0))])
                lse = lse + corr * sm_scale
            return o, lse
        return o
