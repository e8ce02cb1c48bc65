"""Plan files either side of the hot path: the per-head permutation plan and the block-sparse plan.

Formats (example/pipeline_cogvideox.py:37-63,72-103; example/pipeline_wan.py:75-108):
  permute_plan.pth : {'permute': int [L,H] with values 0..5, 'empty': bool [L,H]}
  sparse_plan.pth  : {'sparse': [T,L,H,nb_img,nb_img] (0/1), 'dense_rate': [T,L,H]}
with T mask timesteps, L transformer blocks, H heads.  The masks are expressed in the permuted
token order of each head.  Files are read with torch.load(weights_only=True) only.
"""
from __future__ import annotations

import os
from typing import Dict, Tuple

import torch


def _load(path, map_location="cpu"):
    return torch.load(os.fspath(path), map_location=map_location, weights_only=True)


def check_permute_plan(plan: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    if not isinstance(plan, dict) or "permute" not in plan:
        raise ValueError("permute plan must be a dict with key 'permute' ([L,H] integers in 0..5)")
    p = torch.as_tensor(plan["permute"])
    if p.dim() != 2 or p.is_floating_point() and not torch.equal(p, p.round()):
        raise ValueError("permute plan 'permute' must be an integer [L,H] tensor")
    if p.numel() and (int(p.min()) < 0 or int(p.max()) > 5):
        raise ValueError("permute plan entries must be in 0..5")
    out = {"permute": p.to(torch.int64)}
    empty = plan.get("empty")
    out["empty"] = torch.zeros(p.shape, dtype=torch.bool) if empty is None else torch.as_tensor(empty).bool()
    if out["empty"].shape != p.shape:
        raise ValueError("permute plan 'empty' must have the shape of 'permute'")
    return out


def load_permute_plan(path, map_location="cpu") -> Dict[str, torch.Tensor]:
    return check_permute_plan(_load(path, map_location))


def load_sparse_plan(path) -> Dict[str, torch.Tensor]:
    """Always to host memory: the Wan 720p plan is 8.9 GB as bool (pipeline_wan.py:75-79)."""
    plan = _load(path, "cpu")
    if not isinstance(plan, dict) or "sparse" not in plan:
        raise ValueError("sparse plan must be a dict with key 'sparse' ([T,L,H,nb,nb])")
    s = plan["sparse"]
    if s.dim() != 5 or s.shape[-1] != s.shape[-2]:
        raise ValueError(f"sparse plan 'sparse' must be [T,L,H,nb,nb], got {tuple(s.shape)}")
    out = {"sparse": s.bool()}
    if "dense_rate" in plan:
        out["dense_rate"] = plan["dense_rate"]
    return out


def cog_kernel_mask(sparse: torch.Tensor, n_text_blocks: int = 4) -> torch.Tensor:
    """[T,L,H,nb_img,nb_img] -> [T,L,H,nb,nb] with nb = nb_img + n_text_blocks as the kernel indexes it
    (pipeline_cogvideox.py:80,99-100): n_text_blocks rows and columns of ones in front (CogVideoX:
    226 text tokens + the first 30 image tokens = 4 blocks of 64), last row and column forced True."""
    m = torch.nn.functional.pad(sparse.bool(), (n_text_blocks, 0, n_text_blocks, 0), mode="constant", value=True)
    m[..., :, -1] = True
    m[..., -1, :] = True
    return m


def wan_kernel_mask(sparse: torch.Tensor) -> torch.Tensor:
    """Wan has no text tokens in self-attention: only the last row/column rule (pipeline_wan.py:104-105)."""
    m = sparse.bool().clone()
    m[..., :, -1] = True
    m[..., -1, :] = True
    return m


def write_synthetic_plans(directory, T: int, L: int, H: int, nb_img: int, density: float, seed: int = 0,
                          band: int = 2) -> Tuple[str, str]:
    """Writes permute_plan.pth and sparse_plan.pth of the formats above with random contents (per-head
    order uniform in 0..5; masks = diagonal band plus uniformly random blocks up to `density`).  There
    are no calibrated plans offline; this makes end-to-end runs and tests possible."""
    from . import synth

    os.makedirs(directory, exist_ok=True)
    g = torch.Generator().manual_seed(seed)
    permute = torch.randint(0, 6, (L, H), generator=g)
    empty = torch.zeros(L, H, dtype=torch.bool)
    sparse = torch.empty(T, L, H, nb_img, nb_img, dtype=torch.bool)
    for t in range(T):
        for l in range(L):
            sparse[t, l] = synth.make_block_mask(H, nb_img, density, seed=seed + 1 + t * L + l, band=band)
    dense_rate = sparse.float().mean(dim=(-1, -2))
    p_path = os.path.join(directory, "permute_plan.pth")
    s_path = os.path.join(directory, "sparse_plan.pth")
    torch.save({"permute": permute, "empty": empty}, p_path)
    torch.save({"sparse": sparse, "dense_rate": dense_rate}, s_path)
    return p_path, s_path
