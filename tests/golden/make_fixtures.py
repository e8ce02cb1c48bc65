"""Writes tests/golden/path_small.npz: one small, seeded instance of the whole hot path with every
intermediate result, computed by the CPU oracle (oracle/paro_oracle.py).

    python tests/golden/make_fixtures.py

The reference holds no golden vectors for this path and cannot run here (CUDA/PTX only), so these
vectors freeze the ORACLE, which is pinned independently in tests/test_oracle_*.py (closed forms,
library routines, brute force, the hand-derivable input of the reference's bench/test.py:5-14).  Tests
on the CPU check that the oracle still reproduces the file; tests on the GPU check the HIP kernels
against it.  16-bit floats are stored as their bit patterns (uint16), FP8 as bytes.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import paro_oracle as O  # noqa: E402
from paroatten_amd import synth  # noqa: E402

B, H, D = 1, 2, 64
GRID, N_TEXT = (2, 5, 12), 16
N = N_TEXT + GRID[0] * GRID[1] * GRID[2]          # 136 = 2 blocks of 64 + a tail of 8
DTYPE = torch.float16


def bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def build():
    q, k, v = synth.make_qkv(B, H, N, D, DTYPE, seed=2024)
    nb = (N + 63) // 64
    mask = synth.make_block_mask(H, nb, 0.7, seed=2025, band=0)
    plan = {"permute": torch.tensor([[4, 2]]), "empty": torch.zeros(1, H, dtype=torch.bool)}
    cos, sin = O.rope_table_cog(D, GRID)
    out = {"q": bits(q), "k": bits(k), "v": bits(v), "mask": mask.numpy(), "permute": plan["permute"].numpy(),
           "cos": cos.numpy(), "sin": sin.numpy(), "grid": np.array(GRID), "n_text": np.array(N_TEXT)}
    # RoPE (image tokens only), then the per-head permutation
    qr, kr = q.clone(), k.clone()
    qr[:, :, N_TEXT:] = O.rope_apply_cog(q[:, :, N_TEXT:], cos, sin)
    kr[:, :, N_TEXT:] = O.rope_apply_cog(k[:, :, N_TEXT:], cos, sin)
    qp, kp, vp = O.permute_qk(qr, kr, v, plan, 0, GRID, N_TEXT)
    out.update(q_rope=bits(qr), k_rope=bits(kr), q_perm=bits(qp), k_perm=bits(kp), v_perm=bits(vp))
    out["index_map"] = np.stack([O.permute_index_map(GRID, int(p)).numpy() for p in plan["permute"][0]])
    # INT8 quantisation, K mean-smoothed with the mean rounded to the input type
    km = kp.float().mean(dim=2, keepdim=True).to(DTYPE)
    q8, qs, k8, ks = O.per_warp_int8(qp, kp, km=km, BLKQ=64, WARPQ=32, BLKK=64)
    out.update(km=bits(km), q8=q8.numpy(), q_scale=qs.numpy(), k8=k8.numpy(), k_scale=ks.numpy())
    # exact integer scores of head 0
    out["s_int32_head0"] = O.qk_int32(q8, k8)[0, 0].numpy().astype(np.int32)
    # V -> e4m3 (token-major bytes), per-channel scale and mean
    v8, vsc, vm = O.per_channel_fp8(vp)
    out.update(v8=v8.view(torch.uint8).numpy(), v_scale=vsc.numpy(), v_mean=vm.numpy())
    # attention in float64 on the quantised Q/K and the 16-bit V, then the inverse permutation
    o, lse = O.sparse_attention(q8, k8, vp, qs, ks, mask[None], D ** -0.5, out_dtype=torch.float32,
                                compute_dtype=torch.float64)
    out.update(o_perm=o.numpy(), lse_base2=lse.numpy())
    out["o"] = O.permute_attn_out(o, plan, 0, GRID, N_TEXT).numpy()
    return out


if __name__ == "__main__":
    path = os.path.join(HERE, "path_small.npz")
    np.savez_compressed(path, **build())
    print(path, os.path.getsize(path), "bytes")
