"""GPU parity of the attention's accuracy mode (PARO_ATTN_PV_F16: float16 P.V product, what the reference's
qk_int8_sv_f16_accum_f16_attn computes, csrc/qattn/qk_int_sv_f16_cuda_sm80.cu:263-391) against the oracle.

The oracle attention takes the same INT8 Q/K and the unquantised V with P in fp32; what separates the kernel from it
is float16 rounding of P (2^-11) and fp32 accumulation order, so the bar here is FLAT and an order of magnitude
below the benchmark's atol 2e-2, also on rows that one key dominates, where the FP8 default needs its relative
bound."""
import numpy as np
import pytest
import torch

from conftest import cosine
from oracle import paro_oracle as O
from paroatten_amd import synth

pytestmark = pytest.mark.gpu

ATOL16 = 4e-3     # float16 output rounding (2^-11 of |o| <= 4) plus P's float16 rounding; measured ~1e-3
COS16 = 0.99999


def test_v_f16_tiles_are_in_the_documented_order(dev):
    """paro_v_f16_pack against the index law stated in include/paroatten.h, float16 (bit-exact copy) and
    bfloat16 (converted, exact for these magnitudes), ragged token count, both head sizes, strided input."""
    from paroatten_amd import _qattn_sm80 as qattn
    for D, dtype, N in ((64, torch.float16, 200), (128, torch.bfloat16, 130), (64, torch.bfloat16, 64)):
        B, H = 2, 3
        g = torch.Generator().manual_seed(N + D)
        v = torch.randn(B, N, H, D, generator=g).to(dtype)            # NHD storage: a strided HND view
        tiles = qattn.v_f16_tiles(v.to(dev).transpose(1, 2)).cpu().view(torch.float16)
        nb = (N + 63) // 64
        tiles = tiles.reshape(B, H, nb, D // 32, 4, 64, 8)
        vp = torch.zeros(B, H, nb * 64, D, dtype=torch.float16)
        vp[:, :, :N] = v.transpose(1, 2).to(torch.float16)
        dt, s, lane, e = np.meshgrid(np.arange(D // 32), np.arange(4), np.arange(64), np.arange(8), indexing="ij")
        tok = 32 * (s // 2) + 16 * (s % 2) + 8 * (e // 4) + 4 * (lane // 32) + e % 4
        ch = 32 * dt + lane % 32
        for kb in range(nb):
            want = vp[:, :, kb * 64 + torch.from_numpy(tok), torch.from_numpy(ch)]
            assert torch.equal(tiles[:, :, kb], want), (D, dtype, N, kb)


def _case(B, H, N, D, dtype, seed, Hkv=None, density=0.4, smooth_k=True, mask=None):
    Hkv = Hkv or H
    q, _, _ = synth.make_qkv(B, H, N, D, dtype, seed=seed)
    _, k, v = synth.make_qkv(B, Hkv, N, D, dtype, seed=seed + 1)
    nb = (N + 63) // 64
    if mask is None:
        mask = synth.make_block_mask(H, nb, density, seed=seed + 2)
    return q, k, v, mask


def _oracle(q, k, v, mask, D, causal, smooth_k):
    km = k.float().mean(dim=2, keepdim=True).to(k.dtype) if smooth_k else None
    q8, qs, k8, ks = O.per_warp_int8(q, k, km=km, BLKQ=64, WARPQ=32, BLKK=64)
    B = q.size(0)
    mask_b = mask[None].expand(B, *mask.shape).contiguous()
    # the kernel multiplies by V in float16: for bfloat16 inputs that conversion is exact at these magnitudes
    o_ref, lse_ref = O.sparse_attention(q8, k8, v, qs, ks, mask_b, D ** -0.5, is_causal=causal, out_dtype=torch.float32)
    lse_ref = lse_ref / O.LOG2E
    if smooth_k:   # the operator returns the log-sum-exp of the scores of q and k as given (K - km + km)
        H, Hkv = q.size(1), k.size(1)
        lse_ref = lse_ref + torch.einsum("bhnd,bhd->bhn", q.float(),
                                         km.float().squeeze(2).repeat_interleave(H // Hkv, dim=1)) * D ** -0.5
    return o_ref, lse_ref


@pytest.mark.parametrize("D,dtype,N,Hkv,causal", [
    (64, torch.float16, 1000, None, False),
    (64, torch.bfloat16, 2048, None, False),
    (128, torch.float16, 1000, None, False),
    (128, torch.bfloat16, 777, None, False),
    (64, torch.float16, 700, 2, True),
    (128, torch.float16, 640, 2, True),
])
def test_accuracy_mode_against_the_oracle(dev, D, dtype, N, Hkv, causal):
    """Outputs within a flat 4e-3 of the oracle and cosine >= 0.99999, log-sum-exp as the other kernels' (the
    INT8 stage is the same); with and without lse the same output bits."""
    import paroatten_amd as P
    B, H = 2, 4
    nb = (N + 63) // 64
    mask = torch.ones(H, nb, nb, dtype=torch.bool) if causal else None
    q, k, v, mask = _case(B, H, N, D, dtype, seed=N + D, Hkv=Hkv, mask=mask)
    o_ref, lse_ref = _oracle(q, k, v, mask, D, causal, True)
    args = (q.to(dev), k.to(dev), v.to(dev), mask.to(dev))
    o, lse = P.paroattn_qk_int8_pv_fp16_cuda(*args, is_causal=causal, smooth_k=True, return_lse=True, pv_f16=True)
    o2 = P.paroattn_qk_int8_pv_fp16_cuda(*args, is_causal=causal, smooth_k=True, pv_f16=True)
    assert torch.equal(o, o2)
    o, lse = o.cpu(), lse.cpu()
    err = (o.float() - o_ref).abs().max().item()
    assert err <= ATOL16 + 2 ** -9 * o_ref.abs().max().item(), err       # + output rounding in bfloat16
    assert cosine(o, o_ref) >= COS16
    assert torch.allclose(lse, lse_ref, atol=2e-3, rtol=1e-4)
    # and it is the more accurate of the two products
    o8 = P.paroattn_qk_int8_pv_fp16_cuda(*args, is_causal=causal, smooth_k=True).cpu()
    assert err < (o8.float() - o_ref).abs().max().item()


def test_accuracy_mode_on_rows_that_one_key_dominates(dev):
    """Spiky scores (a handful of keys carry each row): the FP8 default leaves the flat atol 2e-2 there, by up to
    6 % of the output; the float16 product holds a flat bound ten times tighter than the benchmark's."""
    import paroatten_amd as P
    from test_gpu_attention import _ramp_case
    for D in (64, 128):
        B, H, N = 1, 2, 1024 - 19
        nb = (N + 63) // 64
        q, k, v = _ramp_case(B, H, N, D, torch.float16, 7 + D, "spike")
        v = v * 8          # outputs of several units, so that a relative error of 2^-4 is far above 2e-2
        mask = synth.make_block_mask(H, nb, 0.5, seed=5)
        q8, qs, k8, ks = O.per_warp_int8(q, k, BLKQ=64, WARPQ=32, BLKK=64)
        o_ref, _ = O.sparse_attention(q8, k8, v, qs, ks, mask[None], D ** -0.5, out_dtype=torch.float32)
        args = (q.to(dev), k.to(dev), v.to(dev), mask.to(dev))
        o16 = P.paroattn_qk_int8_pv_fp16_cuda(*args, smooth_k=False, pv_f16=True).cpu()
        o8 = P.paroattn_qk_int8_pv_fp16_cuda(*args, smooth_k=False).cpu()
        e16 = (o16.float() - o_ref).abs().max().item()
        e8 = (o8.float() - o_ref).abs().max().item()
        scale = o_ref.abs().max().item()
        assert scale > 4.0, scale                       # the case does what it is meant to
        assert e8 > 2e-2, e8                            # FP8 leaves the flat bound here ...
        assert e16 <= 2e-3 * scale, (e16, scale)        # ... float16 stays at its own rounding error
        assert e16 <= 2e-2, e16


def test_prepacked_tiles_and_the_unpermuting_store(dev):
    """The kernel on operands packed beforehand (paro_v_f16_pack + paro_attn_sparse_fwd with the flag) gives the
    bits of the one-call entry point; with the unpermuting store, the rows land where permute_attn_out would put
    them."""
    from paroatten_amd import _qattn_sm80 as qattn, quant as Q, permute as PM
    B, H, D = 1, 3, 64
    grid, n_text = (3, 4, 8), 20
    N = n_text + grid[0] * grid[1] * grid[2]
    q, k, v, mask = _case(B, H, N, D, torch.float16, seed=31)
    qd, kd, vd, md = q.to(dev), k.to(dev), v.to(dev), mask.to(dev)
    q8, qs, k8, ks = Q.per_warp_int8(qd, kd, None, BLKQ=64, WARPQ=32, BLKK=64)
    out = torch.empty_like(qd)
    qattn.qk_int8_sv_f16_accum_f16_attn(q8, k8, vd, out, qs, ks, 1, 0, 2, D ** -0.5, 0, md, pv_f16=True)
    tiles = qattn.v_f16_tiles(vd)
    out2 = torch.empty_like(qd)
    qattn.attn_sparse_prepacked(q8, k8, tiles, None, None, out2, qs, ks, D ** -0.5, md, pv_f16=True)
    assert torch.equal(out, out2)
    orders = torch.tensor([0, 3, 5], dtype=torch.int32, device=dev)
    token_major = torch.empty((B, N, H, D), dtype=torch.float16, device=dev)
    qattn.attn_sparse_prepacked(q8, k8, tiles, None, None, token_major.transpose(1, 2), qs, ks, D ** -0.5, md,
                                unpermute=(orders, grid, n_text), pv_f16=True)
    want = PM.permute_inverse(out, orders, grid, n_text)
    assert torch.equal(token_major.transpose(1, 2), want)


def test_flag_is_checked(dev):
    """Score dump and float16 product do not combine; a workspace sized for FP8 tiles is too small for float16 ones."""
    from paroatten_amd import _qattn_sm80 as qattn, quant as Q
    B, H, N, D = 1, 1, 256, 64
    q, k, v, mask = _case(B, H, N, D, torch.float16, seed=3)
    qd, kd, vd, md = q.to(dev), k.to(dev), v.to(dev), mask.to(dev)
    q8, qs, k8, ks = Q.per_warp_int8(qd, kd, None, BLKQ=64, WARPQ=32, BLKK=64)
    small = torch.empty(qattn.workspace_bytes(B, H, N, D) // 2, dtype=torch.uint8, device=dev)
    assert qattn.workspace_bytes(B, H, N, D, pv_f16=True) >= 2 * N * D
    with pytest.raises(RuntimeError):
        qattn.qk_int8_sv_f16_accum_f16_attn(q8, k8, vd, torch.empty_like(qd), qs, ks, 1, 0, 2, D ** -0.5, 0, md,
                                            pv_f16=True, workspace=small)
