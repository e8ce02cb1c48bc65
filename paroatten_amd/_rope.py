"""Mirror of the reference's prototype `paroattention._rope` extension
(csrc/rope/pybind.cpp:5-8, csrc/rope/rope.cu:14-48, csrc/rope/rope.cuh:9-96).

rope_permutation(Q, K, freq, permutation) -> (QO, KO): Q, K float16 [bs, H, W, dim]; freq float32
[128] holding (cos, sin) pairs that every token and every 128-channel slice shares; each channel
pair (x, y) becomes (c*x - s*y, c*y + s*x); with `permutation` the (H, W) token grid is written
transposed.  Outputs float16 [bs, H*W, dim].  The reference's permuting kernel writes into its
INPUTS and leaves the outputs uninitialised (rope.cuh:49-50); this implements what its signature
promises: inputs untouched, results in the outputs.
"""
from __future__ import annotations

import torch

from . import _lib
from ._lib import ptr, stream_of


def rope_permutation(Q: torch.Tensor, K: torch.Tensor, freq: torch.Tensor, permutation: bool):
    for t, n in ((Q, "Q"), (K, "K"), (freq, "freq")):
        _lib.require_gpu(t, n)
    if Q.dtype != torch.float16 or K.dtype != torch.float16:
        raise RuntimeError("expected scalar type Half")
    if freq.dtype != torch.float32 or freq.numel() != 128:
        raise RuntimeError("freq must be float32 with 128 entries")
    if Q.dim() != 4 or Q.shape != K.shape or not Q.is_contiguous() or not K.is_contiguous():
        raise RuntimeError("Q and K must be contiguous [bs, H, W, dim] tensors of the same shape")
    bs, H, W, dim = Q.shape
    if dim % 128 != 0:
        raise ValueError(f"Unsupported head dim: {dim} (must be a multiple of 128)")
    heads, n = dim // 128, H * W
    cs = freq.view(64, 2)
    cos = cs[:, 0].repeat_interleave(2).expand(n, 128).contiguous()
    sin = cs[:, 1].repeat_interleave(2).expand(n, 128).contiguous()
    orders = torch.full((heads,), 1 if permutation else 0, dtype=torch.int32, device=Q.device)
    QO = torch.empty((bs, n, dim), dtype=torch.float16, device=Q.device)
    KO = torch.empty((bs, n, dim), dtype=torch.float16, device=Q.device)
    # [bs, n, heads, 128] seen as (batch, head, token, channel) through strides
    _lib.on(Q).paro_rope_permute_fwd(
        ptr(Q), ptr(K), None, ptr(QO), ptr(KO), None, _lib.DTYPE_CODE[torch.float16], ptr(cos), ptr(sin),
        ptr(orders), bs, heads, n, 128, 0, 1, H, W, n * dim, 128, dim, n * dim, 128, dim, stream_of(Q))
    return QO, KO
