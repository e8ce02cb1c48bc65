"""Per-thread scale granularity (qk_quant_gran 3 of the reference's attention kernel,
csrc/qattn/qk_int_sv_f16_cuda_sm80.cu:112-116, 129-133, shapes :1034-1038): the quantiser bit for bit against the
oracle, the attention against the oracle with the same scales.  Inputs whose token magnitudes differ by up to 8x from
token to token, so that the eight q scales of a 32-row group and the four k scales of a block differ by factors
and a wrong scale index shows as an error far outside the tolerance."""
import pytest
import torch

from conftest import assert_attention_close
from oracle import paro_oracle as O
from paroatten_amd import synth

pytestmark = pytest.mark.gpu


def _inputs(B, H, Hkv, N, D, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H, N, D, generator=g) * (0.25 + 1.75 * torch.rand(B, H, N, 1, generator=g))
    k = torch.randn(B, Hkv, N, D, generator=g) * (0.25 + 1.75 * torch.rand(B, Hkv, N, 1, generator=g)) + \
        torch.randn(1, Hkv, 1, D, generator=g)
    v = torch.randn(B, Hkv, N, D, generator=g)
    return q.to(dtype), k.to(dtype), v.to(dtype)


@pytest.mark.parametrize("D,N,dtype,layout,smooth", [
    (64, 1000, torch.float16, "HND", True), (128, 333, torch.bfloat16, "NHD", False),
    (64, 64, torch.bfloat16, "HND", False), (128, 31, torch.float16, "HND", True), (64, 2113, torch.float16, "NHD", True)])
def test_per_thread_quantiser_bitexact(dev, D, N, dtype, layout, smooth):
    from paroatten_amd import quant as Q
    q, k, _ = _inputs(2, 3, 3, N, D, dtype, seed=N + D)
    km = k.float().mean(dim=2, keepdim=True).to(dtype) if smooth else None
    want = O.per_thread_int8(q, k, km=km)
    tr = (lambda t: t) if layout == "HND" else (lambda t: t.transpose(1, 2).contiguous())
    kmd = None if km is None else (km.to(dev) if layout == "HND" else km.transpose(1, 2).contiguous().to(dev))
    got = Q.per_thread_int8(tr(q.to(dev)), tr(k.to(dev)), kmd, tensor_layout=layout)
    nb = (N + 63) // 64
    assert got[1].shape == (2, 3, nb * 16) and got[3].shape == (2, 3, nb * 4)
    assert torch.equal(tr(got[0].cpu()) if layout == "NHD" else got[0].cpu(), want[0])
    assert torch.equal(got[1].cpu(), want[1])
    assert torch.equal(tr(got[2].cpu()) if layout == "NHD" else got[2].cpu(), want[2])
    assert torch.equal(got[3].cpu(), want[3])
    # the scales inside a group really differ (otherwise the test would not see a wrong index)
    if N >= 64:
        assert float(want[1][0, 0, :8].max() / want[1][0, 0, :8].min()) > 1.05


@pytest.mark.parametrize("B,H,Hkv,N,D,dtype,density,causal,lse_on,exact", [
    (2, 3, 3, 1000, 64, torch.float16, 0.4, False, True, False),     # (lse: true exponentials)
    (1, 4, 2, 700, 64, torch.bfloat16, 1.0, True, False, False),     # fast construction of the weights
    (1, 2, 2, 2048, 128, torch.bfloat16, 0.3, False, False, False),
    (1, 2, 2, 2048, 128, torch.bfloat16, 0.3, False, False, True),   # true exponentials without lse
    (2, 2, 1, 333, 128, torch.float16, 0.6, True, True, False),
    (1, 2, 2, 63, 64, torch.float16, 1.0, False, True, False),
    (1, 3, 3, 1500, 64, torch.float16, 0.3, False, False, True),
])
def test_per_thread_attention_against_oracle(dev, B, H, Hkv, N, D, dtype, density, causal, lse_on, exact):
    import paroatten_amd as P
    q, k, v = _inputs(B, H, Hkv, N, D, dtype, seed=N)
    nb = (N + 63) // 64
    mask = synth.make_block_mask(H, nb, density, seed=N + 2) if density < 1 else torch.ones(H, nb, nb, dtype=torch.bool)
    if density < 1:
        mask[0, nb // 2] = False                       # an empty row
    mask_b = mask[None].expand(B, H, nb, nb).contiguous()
    km = k.float().mean(dim=2, keepdim=True).to(dtype)
    q8, qs, k8, ks = O.per_thread_int8(q, k, km=km)
    o_ref, lse_ref = O.sparse_attention(q8, k8, v, qs, ks, mask_b, D ** -0.5, is_causal=causal, out_dtype=dtype, per_thread=True)
    a_ref, _ = O.sparse_attention(q8, k8, v.abs(), qs, ks, mask_b, D ** -0.5, is_causal=causal, out_dtype=torch.float32,
                                  per_thread=True)
    out = P.paroattn_qk_int8_pv_fp16_cuda(q.to(dev), k.to(dev), v.to(dev), mask.to(dev), is_causal=causal,
                                          qk_quant_gran="per_thread", smooth_k=True, return_lse=lse_on, exact_exp=exact)
    o, lse = out if lse_on else (out, None)
    assert_attention_close(o.cpu(), o_ref, a_ref, 0.999, what="per_thread")
    if lse_on:
        lr = lse_ref / O.LOG2E + torch.einsum("bhnd,bhd->bhn", q.float(),
                                              km.float().squeeze(2).repeat_interleave(H // Hkv, dim=1)) * D ** -0.5
        assert torch.equal(torch.isinf(lse.cpu()), torch.isinf(lr))
        keep = ~torch.isinf(lr)
        assert torch.allclose(lse.cpu()[keep], lr[keep], atol=2e-3, rtol=1e-4)
    # the same scale tensors read with the per-warp law (every 8th / 4th entry) are far away: the index law matters
    o_wrong, _ = O.sparse_attention(q8, k8, v, qs[:, :, ::8].contiguous(), ks[:, :, ::4].contiguous(), mask_b, D ** -0.5,
                                    is_causal=causal, out_dtype=dtype)
    if N >= 256:
        assert float((o_wrong.float() - o_ref.float()).abs().max()) > 0.05


def test_per_thread_with_group_constant_scales_is_the_per_warp_kernel(dev):
    """scales constant over every 32-row / 64-key group: the per-thread path returns bit for bit what the two-wave
    kernel returns for the per-warp scales with true exponentials"""
    from paroatten_amd import _qattn_sm80 as qattn, quant as Q
    B, H, N, D = 1, 3, 900, 128
    q, k, v = (t.to(dev) for t in _inputs(B, H, H, N, D, torch.bfloat16, seed=1))
    nb = (N + 63) // 64
    mask = synth.make_block_mask(H, nb, 0.5, seed=4).to(dev)
    q8, qs, k8, ks = Q.per_warp_int8(q, k, BLKQ=64, WARPQ=32, BLKK=64)
    a, b = torch.empty_like(q), torch.empty_like(q)
    la = qattn.qk_int8_sv_f16_accum_f16_attn(q8, k8, v, a, qs, ks, 1, 0, 2, D ** -0.5, 1, mask)
    lb = qattn.qk_int8_sv_f16_accum_f16_attn(q8, k8, v, b, qs.repeat_interleave(8, dim=2).contiguous(),
                                             ks.repeat_interleave(4, dim=2).contiguous(), 1, 0, 3, D ** -0.5, 1, mask)
    assert torch.equal(a, b) and torch.equal(la, lb)
    # and without lse: the fast construction of the weights on both sides
    qattn.qk_int8_sv_f16_accum_f16_attn(q8, k8, v, a, qs, ks, 1, 0, 2, D ** -0.5, 0, mask, two_waves=True)
    qattn.qk_int8_sv_f16_accum_f16_attn(q8, k8, v, b, qs.repeat_interleave(8, dim=2).contiguous(),
                                        ks.repeat_interleave(4, dim=2).contiguous(), 1, 0, 3, D ** -0.5, 0, mask)
    assert torch.equal(a, b)


def test_per_thread_paced_launch_is_bit_identical(dev):
    """the paced launch form with per-thread scales (more q-blocks per XCD than resident workgroups, so the generation
    counters are in use): the same bits as the plain launch"""
    from paroatten_amd import _qattn_sm80 as qattn, quant as Q
    B, H, N, D = 2, 12, 3104, 128
    q, k, v = (t.to(dev) for t in _inputs(B, H, H, N, D, torch.bfloat16, seed=3))
    nb = (N + 63) // 64
    mask = synth.make_block_mask(H, nb, 0.4, seed=5).to(dev)
    q8, qs, k8, ks = Q.per_thread_int8(q, k)
    outs = []
    for pacing in (False, True):
        o = torch.empty_like(q)
        qattn.qk_int8_sv_f16_accum_f16_attn(q8, k8, v, o, qs, ks, 1, 0, 3, D ** -0.5, 0, mask, pacing=pacing)
        outs.append(o)
    assert torch.equal(outs[0], outs[1]) and bool(torch.isfinite(outs[0].float()).all())


def test_per_thread_argument_checks(dev):
    from paroatten_amd import _qattn_sm80 as qattn, quant as Q
    import paroatten_amd as P
    B, H, N, D = 1, 2, 256, 64
    q, k, v = (t.to(dev) for t in _inputs(B, H, H, N, D, torch.float16, seed=2))
    mask = torch.ones(H, 4, 4, dtype=torch.bool, device=dev)
    q8, qs, k8, ks = Q.per_thread_int8(q, k)
    o = torch.empty_like(q)
    with pytest.raises(RuntimeError, match=r"Tensor key_scale must have shape .*\* 4"):
        qattn.qk_int8_sv_f16_accum_f16_attn(q8, k8, v, o, qs, ks[:, :, :4].contiguous(), 1, 0, 3, 0.125, 0, mask)
    with pytest.raises(NotImplementedError):
        qattn.qk_int8_sv_f16_accum_f16_attn(q8, k8, v, o, qs, ks, 1, 0, 3, 0.125, 0, mask, pv_f16=True)
    with pytest.raises(NotImplementedError):
        P.paroattn_qk_int8_pv_fp16_cuda(q, k, v, mask, qk_quant_gran="per_thread", pv_f16=True)
    with pytest.raises(ValueError, match="Unsupported head dim"):
        Q.per_thread_int8(q[..., :32], k[..., :32])
