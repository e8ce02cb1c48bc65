"""Seeded synthetic inputs in the shapes the PAROAttention path runs on.

There are no calibrated plan files or captured activations to load offline, so tests and
the benchmark build their own: Q/K/V ~ N(0,1) with a per-(head, channel) bias on K (which
is what K mean-smoothing exists for), 64x64-block masks made of the diagonal, a +-2 band
and uniformly random extra blocks up to an exact per-head count, and a permute plan that
gives every head one of the six F/H/W orders.  Formats follow the reference's plan files
(example/pipeline_cogvideox.py:37-63 of the reference): `permute_plan = {'permute':
int[L,H], 'empty': bool[L,H]}`, masks bool [H, nb, nb] in the permuted token order.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Tuple

import torch

BLOCK = 64


@dataclass(frozen=True)
class Workload:
    name: str
    B: int
    H: int
    D: int
    grid: Tuple[int, int, int]
    n_text: int
    dtype: torch.dtype

    @property
    def N(self) -> int:
        return self.n_text + self.grid[0] * self.grid[1] * self.grid[2]

    @property
    def nb(self) -> int:
        return (self.N + BLOCK - 1) // BLOCK


WORKLOADS = {
    "cfg0_plumbing": Workload("cfg0_plumbing", 1, 2, 64, (16, 16, 16), 0, torch.float16),
    "cogvideox5b": Workload("cogvideox5b", 2, 48, 64, (13, 30, 45), 226, torch.float16),
    "cogvideox5b_rope": Workload("cogvideox5b_rope", 2, 48, 64, (13, 30, 45), 226, torch.bfloat16),
    "wan14b_480p": Workload("wan14b_480p", 1, 40, 128, (21, 30, 52), 0, torch.bfloat16),
    "wan14b_720p": Workload("wan14b_720p", 1, 40, 128, (21, 45, 80), 0, torch.bfloat16),
}


def make_qkv(B, H, N, D, dtype, seed=0, k_bias_std=3.0, device="cpu"):
    """Q, K, V ~ N(0,1); K += bias[h, d], bias ~ N(0, k_bias_std)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    q = torch.randn(B, H, N, D, generator=g)
    k = torch.randn(B, H, N, D, generator=g)
    v = torch.randn(B, H, N, D, generator=g)
    bias = torch.randn(1, H, 1, D, generator=g) * k_bias_std
    k = k + bias
    return q.to(dtype).to(device), k.to(dtype).to(device), v.to(dtype).to(device)


def make_qkv_device(B, H, N, D, dtype, seed=0, k_bias_std=3.0, device="cuda"):
    """Same distribution, generated on `device` (different stream than make_qkv; for
    benchmark-sized tensors where a CPU generator would take minutes)."""
    g = torch.Generator(device=device).manual_seed(seed)
    q = torch.randn(B, H, N, D, generator=g, device=device, dtype=torch.float32).to(dtype)
    k = torch.randn(B, H, N, D, generator=g, device=device, dtype=torch.float32)
    v = torch.randn(B, H, N, D, generator=g, device=device, dtype=torch.float32).to(dtype)
    bias = torch.randn(1, H, 1, D, generator=g, device=device) * k_bias_std
    k = (k + bias).to(dtype)
    return q, k, v


def make_block_mask(H, nb, density, seed=0, band=2, device="cpu"):
    """bool [H, nb, nb]: diagonal and |i-j| <= band always kept, then uniformly random
    extra blocks until each head holds exactly round(density * nb^2) kept blocks (or the
    band alone if that is already more)."""
    g = torch.Generator(device=device).manual_seed(seed)
    target = int(round(density * nb * nb))
    idx = torch.arange(nb, device=device)
    in_band = (idx[:, None] - idx[None, :]).abs() <= band
    score = torch.rand(H, nb, nb, generator=g, device=device)
    score = torch.where(in_band[None], torch.full_like(score, -1.0), score)
    target = max(target, int(in_band.sum()))
    flat = score.reshape(H, nb * nb)
    kth = torch.topk(flat, target, dim=1, largest=False, sorted=True).values[:, -1:]
    # ties at the threshold are measure-zero for float32 uniforms; keep exactly `target`
    mask = flat <= kth
    extra = mask.sum(dim=1) - target
    if int(extra.max()) > 0:  # pragma: no cover - only on an exact float tie
        for h in range(H):
            e = int(extra[h])
            if e > 0:
                tie = torch.nonzero(flat[h] == kth[h, 0]).flatten()[:e]
                mask[h, tie] = False
    return mask.reshape(H, nb, nb)


def make_window_mask(H, nb, density, device="cpu"):
    """bool [H, nb, nb]: every q-block keeps one contiguous run of round(density * nb) k-blocks
    centred on the diagonal (clipped at the ends): the shape the masks of a permuted head have, as
    opposed to the uniformly scattered extra blocks of make_block_mask."""
    w = max(1, min(nb, int(round(density * nb))))
    i = torch.arange(nb, device=device)
    lo = (i - w // 2).clamp(0, nb - w)
    j = i[None, :]
    m = (j >= lo[:, None]) & (j < lo[:, None] + w)
    return m[None].expand(H, nb, nb).contiguous()


def make_permute_plan(n_layers, H, seed=0):
    """{'permute': int64 [L,H] in 0..5, 'empty': bool [L,H]} (all heads non-empty)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    return {
        "permute": torch.randint(0, 6, (n_layers, H), generator=g),
        "empty": torch.zeros(n_layers, H, dtype=torch.bool),
    }


def attention_ops(mask: torch.Tensor, D: int) -> float:
    """Executed MFMA work: 4*64*64*D per kept block (2*D*64^2 for QK^T + 2*D*64^2 for PV)."""
    return 4.0 * BLOCK * BLOCK * D * float(mask.sum())


def dense_equiv_ops(B, H, N, D) -> float:
    """The reference's FLOP count (bench/bench.py:57 of the reference): 4*H*B*D*N^2."""
    return 4.0 * H * B * D * float(N) * float(N)
