"""Rotary tables in the form the fused RoPE+permutation kernel reads: fp32 cos / sin of shape
[F*H*W, D], the frequency of every channel pair repeated over the pair.

CogVideoX: the (cos, sin) pair diffusers hands to the attention processor as `image_rotary_emb`
already has this form (paroattention/cogvideox.py:167-172 of the reference); `rope_table_cog`
builds it for synthetic runs in diffusers' documented convention (channels split t/h/w = D/4,
3D/8, 3D/8).  Wan: the reference carries complex128 frequencies [1,1,N,D/2]
(paroattention/wan.py:482-522) and multiplies in float64 (wan.py:161-167); `complex_to_real_tables`
converts such a tensor, `rope_table_wan_real` builds it directly (t/h/w = D-4*(D//6), 2*(D//6),
2*(D//6) channels).  The kernel rotates in fp32: results agree with the float64 form to 1 ulp of
the 16-bit output.
"""
from __future__ import annotations

from typing import Sequence, Tuple

import torch


def _angles_1d(dim: int, length: int, theta: float, device) -> torch.Tensor:
    inv = 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float64, device=device)[: dim // 2] / dim))
    return torch.outer(torch.arange(length, dtype=torch.float64, device=device), inv)


def _tables(dims: Sequence[int], grid: Sequence[int], theta: float, device) -> Tuple[torch.Tensor, torch.Tensor]:
    F, Hh, W = grid
    af = _angles_1d(dims[0], F, theta, device).view(F, 1, 1, -1).expand(F, Hh, W, -1)
    ah = _angles_1d(dims[1], Hh, theta, device).view(1, Hh, 1, -1).expand(F, Hh, W, -1)
    aw = _angles_1d(dims[2], W, theta, device).view(1, 1, W, -1).expand(F, Hh, W, -1)
    ang = torch.cat([af, ah, aw], dim=-1).reshape(F * Hh * W, -1).repeat_interleave(2, dim=1)
    return ang.cos().float().contiguous(), ang.sin().float().contiguous()


def rope_table_cog(head_dim: int, grid: Sequence[int], theta: float = 10000.0, device="cpu"):
    return _tables((head_dim // 4, head_dim // 8 * 3, head_dim // 8 * 3), grid, theta, device)


def rope_table_wan_real(head_dim: int, grid: Sequence[int], theta: float = 10000.0, device="cpu"):
    hw = 2 * (head_dim // 6)
    return _tables((head_dim - 2 * hw, hw, hw), grid, theta, device)


def complex_to_real_tables(freqs: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """complex [.., N, D/2] (Wan's `rotary_emb`) -> (cos, sin) fp32 [N, D]."""
    f = freqs.reshape(-1, freqs.shape[-1])
    cos = f.real.float().repeat_interleave(2, dim=1).contiguous()
    sin = f.imag.float().repeat_interleave(2, dim=1).contiguous()
    return cos, sin
