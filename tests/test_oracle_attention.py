"""Pins oracle.qk_int32 and oracle.sparse_attention by what they must reduce to: an int64 einsum,
torch's own softmax/SDPA on dequantised operands, and the invariants of the intended semantics
(kept blocks form the softmax support; an all-masked row gives 0)."""

import pytest
import torch

from oracle import paro_oracle as O
from paroatten_amd import synth


def _inputs(B, H, N, D, seed, Hkv=None):
    q, _, _ = synth.make_qkv(B, H, N, D, torch.float16, seed=seed)
    _, k, v = synth.make_qkv(B, Hkv or H, N, D, torch.float16, seed=seed + 1)
    q8, qs, k8, ks = O.per_warp_int8(q, k, BLKQ=64, WARPQ=32, BLKK=64)
    return q, k, v, q8, qs, k8, ks


def test_qk_int32_is_integer_matmul():
    g = torch.Generator().manual_seed(0)
    q8 = torch.randint(-128, 128, (1, 2, 70, 128), generator=g, dtype=torch.int8)
    k8 = torch.randint(-128, 128, (1, 2, 90, 128), generator=g, dtype=torch.int8)
    s = O.qk_int32(q8, k8)
    ref = torch.einsum("bhid,bhjd->bhij", q8.long(), k8.long())
    assert s.dtype == torch.int32 and torch.equal(s.long(), ref)
    # extreme values stay exact: 128 channels of (-128)*(-128)
    e = torch.full((1, 1, 1, 128), -128, dtype=torch.int8)
    assert int(O.qk_int32(e, e)) == 128 * 128 * 128


def _library_reference(q8, qs, k8, ks, v, mask, sm_scale, causal=False):
    """softmax(mask(S)) @ V with torch library calls in float64 on dequantised operands."""
    B, H, N, D = q8.shape
    Hk = k8.shape[1]
    qd = q8.double() * qs.double().repeat_interleave(32, dim=-1)[..., :N, None]
    kd = k8.double() * ks.double().repeat_interleave(64, dim=-1)[..., : k8.shape[2], None]
    kd = kd.repeat_interleave(H // Hk, dim=1)
    vd = v.to(torch.float16).double().repeat_interleave(H // Hk, dim=1)
    s = torch.einsum("bhid,bhjd->bhij", qd, kd) * sm_scale
    keep = O.expand_block_mask(mask, N, k8.shape[2])
    if causal:
        keep = keep & torch.tril(torch.ones(N, N, dtype=torch.bool))
    s = s.masked_fill(~keep, float("-inf"))
    p = torch.softmax(s, dim=-1)
    p = torch.nan_to_num(p, nan=0.0)  # all-masked rows
    lse = torch.logsumexp(s, dim=-1)
    return p @ vd, lse


@pytest.mark.parametrize("N,density", [(300, 0.5), (256, 1.0), (200, 0.3)])
def test_reduces_to_library_softmax(N, density):
    B, H, D = 1, 2, 64
    q, k, v, q8, qs, k8, ks = _inputs(B, H, N, D, seed=N)
    nb = (N + 63) // 64
    mask = synth.make_block_mask(H, nb, density, seed=1)[None]
    o, lse2 = O.sparse_attention(q8, k8, v, qs, ks, mask, D ** -0.5, out_dtype=torch.float32,
                                 compute_dtype=torch.float64)
    ref, lse = _library_reference(q8, qs, k8, ks, v, mask, D ** -0.5)
    assert torch.allclose(o.double(), ref, atol=1e-6, rtol=1e-6)
    assert torch.allclose(lse2.double() / O.LOG2E, lse, atol=1e-5, rtol=1e-6)
    # fp32 compute path (the one timed as CPU baseline) agrees to fp32 accuracy
    o32, _ = O.sparse_attention(q8, k8, v, qs, ks, mask, D ** -0.5, out_dtype=torch.float32)
    assert torch.allclose(o32.double(), ref, atol=2e-5, rtol=1e-4)


def test_dense_equals_sdpa_on_dequantised():
    B, H, N, D = 1, 2, 192, 64
    q, k, v, q8, qs, k8, ks = _inputs(B, H, N, D, seed=9)
    mask = torch.ones(1, H, 3, 3, dtype=torch.bool)
    o, _ = O.sparse_attention(q8, k8, v, qs, ks, mask, D ** -0.5, out_dtype=torch.float32)
    qd = q8.float() * qs.repeat_interleave(32, dim=-1)[..., :N, None]
    kd = k8.float() * ks.repeat_interleave(64, dim=-1)[..., :N, None]
    ref = torch.nn.functional.scaled_dot_product_attention(qd, kd, v.half().float())
    assert torch.allclose(o, ref, atol=2e-5, rtol=1e-4)
    # and it is close to attention on the unquantised inputs (int8 noise only)
    full = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    assert torch.nn.functional.cosine_similarity(o.flatten(), full.flatten(), dim=0) > 0.99


def test_causal_and_gqa_reduce_to_library():
    B, H, Hkv, N, D = 1, 4, 2, 150, 64
    q, k, v, q8, qs, k8, ks = _inputs(B, H, N, D, seed=11, Hkv=Hkv)
    mask = torch.ones(1, H, 3, 3, dtype=torch.bool)
    o, lse2 = O.sparse_attention(q8, k8, v, qs, ks, mask, 0.2, is_causal=True, out_dtype=torch.float32,
                                 compute_dtype=torch.float64)
    ref, lse = _library_reference(q8, qs, k8, ks, v, mask, 0.2, causal=True)
    assert torch.allclose(o.double(), ref, atol=1e-6, rtol=1e-6)
    assert torch.allclose(lse2.double() / O.LOG2E, lse, atol=1e-5)


def test_empty_rows_single_block_and_tail_columns():
    B, H, N, D = 1, 1, 64 * 3 - 7, 64
    q, k, v, q8, qs, k8, ks = _inputs(B, H, N, D, seed=13)
    mask = torch.zeros(1, 1, 3, 3, dtype=torch.bool)
    mask[0, 0, 0, 2] = True  # q-block 0 sees only the (partial) last k-block
    mask[0, 0, 2, 1] = True
    o, lse2 = O.sparse_attention(q8, k8, v, qs, ks, mask, D ** -0.5, out_dtype=torch.float32)
    assert torch.count_nonzero(o[0, 0, 64:128]) == 0 and torch.isinf(lse2[0, 0, 64:128]).all()
    # local attention over exactly the kept block, tail columns >= N excluded
    qd = q8.float() * qs.repeat_interleave(32, dim=-1)[..., :N, None]
    kd = k8.float() * ks.repeat_interleave(64, dim=-1)[..., :N, None]
    loc = torch.softmax(qd[0, 0, :64] @ kd[0, 0, 128:N].T * D ** -0.5, dim=-1) @ v.half().float()[0, 0, 128:N]
    assert torch.allclose(o[0, 0, :64], loc, atol=2e-5, rtol=1e-4)


def test_k_smoothing_invariance_and_output_dtype():
    """softmax(q (k - km)^T) = softmax(q k^T): with exact arithmetic the smoothed path changes
    nothing; with int8 operands it changes the quantisation noise only."""
    B, H, N, D = 1, 2, 256, 64
    q, k, v = synth.make_qkv(B, H, N, D, torch.float16, seed=17)
    mask = torch.ones(1, H, 4, 4, dtype=torch.bool)
    km = k.float().mean(dim=2, keepdim=True).half()
    full = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    outs = []
    for mean in (None, km):
        q8, qs, k8, ks = O.per_warp_int8(q, k, km=mean, BLKQ=64, WARPQ=32, BLKK=64)
        o, _ = O.sparse_attention(q8, k8, v, qs, ks, mask, D ** -0.5, out_dtype=torch.bfloat16)
        assert o.dtype == torch.bfloat16
        outs.append(torch.nn.functional.cosine_similarity(o.float().flatten(), full.flatten(), dim=0).item())
    assert outs[1] >= outs[0] - 1e-4 and outs[1] > 0.995  # smoothing helps (K carries a large bias)


def test_paro_path_equals_unpermuted_attention_when_mask_is_dense():
    """Permuting tokens, attending densely and un-permuting is the identity on the result up to
    quantisation-group noise: pins the chaining (permute -> quant -> attention -> inverse)."""
    B, H, D, grid, n_text = 1, 2, 64, (2, 4, 8), 0
    N = 64
    q, k, v = synth.make_qkv(B, H, N, D, torch.float16, seed=19)
    plan = {"permute": torch.tensor([[2, 5]]), "empty": torch.zeros(1, 2, dtype=torch.bool)}
    mask = torch.ones(1, H, 1, 1, dtype=torch.bool)
    o = O.paro_path(q, k, v, mask, plan, 0, grid, n_text)
    full = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    assert torch.nn.functional.cosine_similarity(o.float().flatten(), full.flatten(), dim=0) > 0.995


def test_per_thread_scales_reduce_to_per_warp_and_to_rowwise_dequantisation():
    """sparse_attention(per_thread=True): (i) with scales that are constant over each 32-row / 64-key group it
    is the per-warp result bit for bit; (ii) with distinct scales it is fp64 softmax attention on Q and K
    dequantised row by row with the scale the reference kernel's lanes read for that row (enumerated lane by
    lane in test_oracle_quant, not taken from the oracle's index law)."""
    from test_oracle_quant import _lane_enumeration
    g = torch.Generator().manual_seed(11)
    B, H, Hk, N, D = 1, 4, 2, 200, 64
    q = torch.randn(B, H, N, D, generator=g).to(torch.float16)
    k = torch.randn(B, Hk, N, D, generator=g).to(torch.float16)
    v = torch.randn(B, Hk, N, D, generator=g).to(torch.float16)
    nb = (N + 63) // 64
    mask = synth.make_block_mask(H, nb, 0.6, seed=3)[None].contiguous()
    q8, qs, k8, ks = O.per_warp_int8(q, k, BLKQ=64, WARPQ=32, BLKK=64)
    o2, l2 = O.sparse_attention(q8, k8, v, qs, ks, mask, D ** -0.5)
    o3, l3 = O.sparse_attention(q8, k8, v, qs.repeat_interleave(8, dim=2), ks.repeat_interleave(4, dim=2), mask,
                                D ** -0.5, per_thread=True)
    assert torch.equal(o2, o3) and torch.equal(l2, l3)

    q8, qs, k8, ks = O.per_thread_int8(q, k)
    assert qs.shape == (B, H, nb * 16) and ks.shape == (B, Hk, nb * 4)
    assert len(torch.unique(qs[0, 0, :8])) == 8 and len(torch.unique(ks[0, 0, :4])) == 4   # distinct scales
    o, lse = O.sparse_attention(q8, k8, v, qs, ks, mask, D ** -0.5, per_thread=True, compute_dtype=torch.float64)
    qi, ki = _lane_enumeration(N, False), _lane_enumeration(N, True)
    qd = q8.double() * qs.double()[:, :, qi].unsqueeze(-1)
    kd = (k8.double() * ks.double()[:, :, ki].unsqueeze(-1)).repeat_interleave(H // Hk, dim=1)
    s = qd @ kd.transpose(-1, -2) * D ** -0.5
    keep = O.expand_block_mask(mask, N, N)
    s = s.masked_fill(~keep, float("-inf"))
    want = torch.softmax(s, dim=-1) @ v.double().repeat_interleave(H // Hk, dim=1)
    assert torch.allclose(o.double(), want, atol=2e-3, rtol=0)   # fp16 rounding of the output
    assert torch.allclose(lse.double(), torch.logsumexp(s, dim=-1) * O.LOG2E, atol=1e-4, rtol=1e-6)
    # and it is not what per-warp indexing of the same scale tensors would give
    o_wrong, _ = O.sparse_attention(q8, k8, v, qs[:, :, ::8].contiguous(), ks[:, :, ::4].contiguous(), mask, D ** -0.5)
    assert (o_wrong.float() - o.float()).abs().max() > 1e-2
