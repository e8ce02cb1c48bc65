"""Mirror of the reference's `paroattention._fused` extension module
(csrc/fused/pybind.cpp:21-33, csrc/fused/fused.h:19-76): same function names, positional
arguments, preallocated outputs, `None` return, and the same validation order and messages
(csrc/utils.cuh:20-38, csrc/dispatch_utils.h:23-112).  Every function lands in the C ABI of
libparoatten_hip.so; there is no torch fallback.
"""
from __future__ import annotations

import torch

from . import _lib
from ._lib import ptr, stream_of

_HALF = (torch.float16, torch.bfloat16)


def _chk(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _check_cuda(t, name):
    _chk(t.is_cuda, f"Tensor {name} must be on CUDA")


def _layout_dims(t, tensor_layout):
    """-> (num_tokens, num_heads, stride_seq, stride_h) as the reference hosts extract them."""
    if tensor_layout == 0:
        return t.size(1), t.size(2), t.stride(1), t.stride(2)
    return t.size(2), t.size(1), t.stride(2), t.stride(1)


def _quant(input, mean, output, scale, group, n_groups_fn, tensor_layout, sm_scale, fn_name):
    for t, n in ((input, "input"), (output, "output"), (scale, "scale")):
        _check_cuda(t, n)
    if mean is not None:
        _check_cuda(mean, "mean")
    _chk(output.dtype == torch.int8, "Tensor output must have dtype (torch::kInt8)")
    _chk(scale.dtype == torch.float32, "Tensor scale must have dtype (torch::kFloat)")
    _chk(input.dim() == 4, "Tensor input must have dimension number (4)")
    _chk(input.stride(-1) == 1, "Tensor input must be contiguous at the last dimension")
    _chk(output.is_contiguous(), "Tensor output must be contiguous")
    _chk(scale.is_contiguous(), "Tensor scale must be contiguous")
    _chk(output.dim() == 4, "Tensor output must have dimension number (4)")
    _chk(scale.dim() == 3, "Tensor scale must have dimension number (3)")
    if mean is not None:
        _chk(mean.stride(-1) == 1, "Tensor mean must be contiguous at the last dimension")
        _chk(mean.dim() == 3, "Tensor mean must have dimension number (3)")
    if input.dtype not in _HALF:
        raise RuntimeError(f"{fn_name} failed to dispatch data type {input.dtype}")
    if mean is not None:
        _chk(mean.dtype == input.dtype, "Tensor mean must have dtype (input_dtype)")
    B, D = input.size(0), input.size(3)
    N, H, xs_n, xs_h = _layout_dims(input, tensor_layout)
    _, _, os_n, os_h = _layout_dims(output, tensor_layout)
    n_groups = n_groups_fn(N)  # raises ValueError on an unsupported block size
    if D not in (64, 128):
        raise ValueError(f"Unsupported head dim: {D}")
    _chk(tuple(output.shape) == tuple(input.shape),
         "Tensor output must have shape (input.size(0), input.size(1), input.size(2), input.size(3))")
    _chk(tuple(scale.shape) == (B, H, n_groups), "Tensor scale must have shape (batch_size, num_heads, num_groups)")
    if mean is not None:
        _chk(tuple(mean.shape) == (B, H, D), "Tensor mean must have shape (batch_size, num_heads, head_dim)")
    ms_b, ms_h = (mean.stride(0), mean.stride(1)) if mean is not None else (0, 0)
    _lib.on(input).paro_quant_int8(
        ptr(input), _lib.DTYPE_CODE[input.dtype], ptr(mean), ptr(output), ptr(scale),
        B, H, N, D, input.stride(0), xs_h, xs_n, ms_b, ms_h, output.stride(0), os_h, os_n,
        scale.stride(0), scale.stride(1), group, n_groups,
        0 if sm_scale is None else 1, 0.0 if sm_scale is None else float(sm_scale), stream_of(input))


def _block_groups(block_size):
    if block_size not in (64, 128):
        raise ValueError(f"Unsupported block_size {int(block_size)}")
    return lambda n: (n + block_size - 1) // block_size


def quant_per_block_int8_cuda(input, output, scale, *args):
    """Both overloads of the reference (csrc/fused/fused.cu:429-510 and :512-592):
    (input, output, scale, sm_scale, block_size, tensor_layout) or
    (input, output, scale, block_size, tensor_layout)."""
    if len(args) == 3:
        sm_scale, block_size, tensor_layout = args
    elif len(args) == 2:
        sm_scale = None
        block_size, tensor_layout = args
    else:
        raise TypeError("quant_per_block_int8_cuda(): incompatible function arguments")
    _quant(input, None, output, scale, block_size, _block_groups(block_size), tensor_layout, sm_scale,
           "quant_per_block_int8_cuda")


def quant_per_block_int8_fuse_sub_mean_cuda(input, mean, output, scale, block_size, tensor_layout):
    """csrc/fused/fused.cu:594-682."""
    _quant(input, mean, output, scale, block_size, _block_groups(block_size), tensor_layout, None,
           "quant_per_block_int8_fuse_sub_mean_cuda")


def quant_per_warp_int8_cuda(input, output, scale, block_size, warp_block_size, tensor_layout):
    """csrc/fused/fused.cu:685-768: one scale per `warp_block_size` tokens, the scale tensor
    holds ceil(N/block_size) * (block_size/warp_block_size) of them."""
    if block_size not in (64, 128):
        raise ValueError(f"Unsupported block_size {int(block_size)}")
    if warp_block_size not in (16, 32):
        raise ValueError(f"Unsupported warp_block_size {int(warp_block_size)}")
    groups = lambda n: (n + block_size - 1) // block_size * (block_size // warp_block_size)
    _quant(input, None, output, scale, warp_block_size, groups, tensor_layout, None, "quant_per_warp_int8_cuda")


def sub_mean_cuda(input, mean, output, tensor_layout):
    """csrc/fused/fused.cu:770-848: output(fp16) = input - mean."""
    for t, n in ((input, "input"), (mean, "mean"), (output, "output")):
        _check_cuda(t, n)
    _chk(output.dtype == torch.float16, "Tensor output must have dtype (torch::kHalf)")
    _chk(input.dim() == 4, "Tensor input must have dimension number (4)")
    _chk(mean.dim() == 3, "Tensor mean must have dimension number (3)")
    _chk(output.dim() == 4, "Tensor output must have dimension number (4)")
    _chk(input.stride(-1) == 1, "Tensor input must be contiguous at the last dimension")
    _chk(mean.stride(-1) == 1, "Tensor mean must be contiguous at the last dimension")
    _chk(output.stride(-1) == 1, "Tensor output must be contiguous at the last dimension")
    if input.dtype not in _HALF:
        raise RuntimeError(f"sub_mean_cuda failed to dispatch data type {input.dtype}")
    _chk(mean.dtype == input.dtype, "Tensor mean must have dtype (input_dtype)")
    B, D = input.size(0), input.size(3)
    N, H, vs_n, vs_h = _layout_dims(input, tensor_layout)
    _, _, os_n, os_h = _layout_dims(output, tensor_layout)
    _chk(tuple(mean.shape) == (B, H, D), "Tensor mean must have shape (batch_size, num_heads, head_dim)")
    _chk(tuple(output.shape) == tuple(input.shape),
         "Tensor output must have shape (input.size(0), input.size(1), input.size(2), input.size(3))")
    _lib.on(input).paro_sub_mean(ptr(input), _lib.DTYPE_CODE[input.dtype], ptr(mean), ptr(output), B, H, N, D,
                               input.stride(0), vs_h, vs_n, mean.stride(0), mean.stride(1),
                               output.stride(0), os_h, os_n, stream_of(input))


_NV_LAYOUT = (
    "{name} writes V in the register-fragment order of NVIDIA's fp8 mma "
    "(csrc/fused/fused.cu:287-291); that order has no meaning on gfx950 and nothing consumes it. "
    "Use paroatten_amd.quant.per_channel_fp8, which produces FP8 V in this library's MFMA tile order."
)


def transpose_pad_permute_cuda(input, output, tensor_layout):
    raise NotImplementedError(_NV_LAYOUT.format(name="transpose_pad_permute_cuda"))


def scale_fuse_quant_cuda(input, output, scale, num_tokens, scale_max, tensor_layout):
    raise NotImplementedError(_NV_LAYOUT.format(name="scale_fuse_quant_cuda"))


def mean_scale_fuse_quant_cuda(input, output, mean, scale, num_tokens, scale_max, tensor_layout):
    raise NotImplementedError(_NV_LAYOUT.format(name="mean_scale_fuse_quant_cuda"))
