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


def transpose_pad_permute_cuda(input, output, tensor_layout):
    """csrc/fused/fused.cu:850-923: input [B,H,N,D] (layout 1) or [B,N,H,D] (layout 0) ->
    output [B,H,D,ceil64(N)] or [B,D,H,ceil64(N)], tokens >= N zero, tokens inside every group of 16
    in the order 0,1,8,9,2,3,10,11,4,5,12,13,6,7,14,15 (the operand order of NVIDIA's fp8 mma; this
    library's attention kernel reads the tiles of quant.per_channel_fp8 instead)."""
    _check_cuda(input, "input")
    _check_cuda(output, "output")
    _chk(input.stride(-1) == 1, "Tensor input must be contiguous at the last dimension")
    _chk(output.is_contiguous(), "Tensor output must be contiguous")
    _chk(input.dim() == 4, "Tensor input must have dimension number (4)")
    _chk(output.dim() == 4, "Tensor output must have dimension number (4)")
    B, D = input.size(0), input.size(3)
    N, H, is_n, is_h = _layout_dims(input, tensor_layout)
    padded = (N + 63) // 64 * 64
    if tensor_layout == 0:
        _chk(tuple(output.shape) == (B, D, H, padded),
             "Tensor output must have shape (batch_size, head_dim, num_heads, padded_num_tokens)")
        os_d, os_h = output.stride(1), output.stride(2)
    else:
        _chk(tuple(output.shape) == (B, H, D, padded),
             "Tensor output must have shape (batch_size, num_heads, head_dim, padded_num_tokens)")
        os_d, os_h = output.stride(2), output.stride(1)
    _chk(input.dtype == output.dtype, "Input and output must have the same data type")
    if input.dtype not in _HALF:
        raise RuntimeError(f"transpose_pad_permute_cuda failed to dispatch data type {input.dtype}")
    if D not in (64, 128):
        raise ValueError(f"Unsupported head dim: {D}")
    _lib.on(input).paro_transpose_pad_permute(ptr(input), ptr(output), _lib.DTYPE_CODE[input.dtype], B, H, N, D,
                                            input.stride(0), is_h, is_n, output.stride(0), os_h, os_d,
                                            stream_of(input))


def _channel_quant(input, output, mean, scale, num_tokens, scale_max, tensor_layout, fn_name):
    tensors = [(input, "input"), (output, "output")] + ([(mean, "mean")] if mean is not None else []) + [(scale, "scale")]
    for t, n in tensors:
        _check_cuda(t, n)
    if mean is not None:
        _chk(mean.dtype == torch.float32, "Tensor mean must have dtype (torch::kFloat)")
    _chk(scale.dtype == torch.float32, "Tensor scale must have dtype (torch::kFloat)")
    for t, n in tensors:
        _chk(t.is_contiguous(), f"Tensor {n} must be contiguous")
    _chk(input.dim() == 4, "Tensor input must have dimension number (4)")
    _chk(output.dim() == 4, "Tensor output must have dimension number (4)")
    if mean is not None:
        _chk(mean.dim() == 3, "Tensor mean must have dimension number (3)")
    _chk(scale.dim() == 3, "Tensor scale must have dimension number (3)")
    B, row_len = input.size(0), input.size(3)
    if tensor_layout == 0:
        H, D, d_dim, h_dim = input.size(2), input.size(1), 1, 2
    else:
        H, D, d_dim, h_dim = input.size(1), input.size(2), 2, 1
    _chk(tuple(output.shape) == tuple(input.shape),
         "Tensor output must have shape (input.size(0), input.size(1), input.size(2), input.size(3))")
    if mean is not None:
        _chk(tuple(mean.shape) == (B, H, D), "Tensor mean must have shape (batch_size, num_heads, head_dim)")
    _chk(tuple(scale.shape) == (B, H, D), "Tensor scale must have shape (batch_size, num_heads, head_dim)")
    if input.dtype not in _HALF:
        raise RuntimeError(f"{fn_name} failed to dispatch data type {input.dtype}")
    # the reference leaves the output dtype unchecked (a commented-out int8 check): one byte per entry
    _chk(output.element_size() == 1, "Tensor output must have a one-byte dtype (torch.float8_e4m3fn)")
    ms_b, ms_h = (mean.stride(0), mean.stride(1)) if mean is not None else (0, 0)
    _lib.on(input).paro_channel_quant_fp8(
        ptr(input), _lib.DTYPE_CODE[input.dtype], ptr(output), ptr(mean), ptr(scale), B, H, D, int(num_tokens), row_len,
        float(scale_max), input.stride(0), input.stride(h_dim), input.stride(d_dim),
        output.stride(0), output.stride(h_dim), output.stride(d_dim), ms_b, ms_h,
        scale.stride(0), scale.stride(1), stream_of(input))


def scale_fuse_quant_cuda(input, output, scale, num_tokens, scale_max, tensor_layout):
    """csrc/fused/fused.cu:925-1000: per (batch, head, channel) row of the transposed V:
    scale = max|x[:ceil16(num_tokens)]| / scale_max, output = e4m3(x * scale_max / max|x|)."""
    _channel_quant(input, output, None, scale, num_tokens, scale_max, tensor_layout, "scale_fuse_quant_cuda")


def mean_scale_fuse_quant_cuda(input, output, mean, scale, num_tokens, scale_max, tensor_layout):
    """csrc/fused/fused.cu:1002-1083: as scale_fuse_quant_cuda after subtracting the row mean
    (sum over the first ceil16(num_tokens) entries divided by that count, fused.cu:335,381)."""
    _channel_quant(input, output, mean, scale, num_tokens, scale_max, tensor_layout, "mean_scale_fuse_quant_cuda")
