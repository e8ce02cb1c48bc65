"""The one-pass preparation (RoPE + permutation + INT8 Q/K + FP8 V) against the oracle and against the
chain of separate kernels it replaces: INT8 tensors and their scales bit for bit; the V statistics
are summed in source-token order instead of permuted order, so the mean may differ in the last fp32
bit and, through it, an FP8 code here and there by one step.  v_mean is the offset the attention
epilogue adds back: the channel mean plus the mean rounding residual of the channel's own codes."""
import pytest
import torch

from conftest import untile_v8, v8_offset_expected
from oracle import paro_oracle as O
from paroatten_amd import synth

pytestmark = pytest.mark.gpu


def _case(dev, B, H, D, grid, n_text, dtype, seed, rope_kind):
    from paroatten_amd import rope
    N = n_text + grid[0] * grid[1] * grid[2]
    q, k, v = synth.make_qkv(B, H, N, D, dtype, seed=seed)
    plan = synth.make_permute_plan(1, H, seed=seed + 1)
    cos = sin = None
    if rope_kind == "cog":
        cos, sin = rope.rope_table_cog(D, grid)
    elif rope_kind == "wan":
        cos, sin = rope.rope_table_wan_real(D, grid)
    return q, k, v, plan, cos, sin, N


def _same_v(got, v8_chain, vsc_chain, vm_chain):
    assert torch.allclose(got.v_scale, vsc_chain, atol=0, rtol=1e-6)
    # each side's offset belongs to its own codes: a code that differs by one step (at most 32 scaled
    # units, at most 1e-3 of the codes) moves the mean residual by that step / N
    assert bool(((got.v_mean - vm_chain).abs() <= 1e-6 + 0.032 * got.v_scale).all())
    a = got.v8.view(torch.uint8).flatten().int()
    b = v8_chain.view(torch.uint8).flatten().int()
    diff = (a - b).abs()
    assert int(diff.max()) <= 1 and float((diff != 0).float().mean()) <= 1e-3


def _chain(dev, q, k, v, orders, grid, n_text, cos, sin, km):
    from paroatten_amd import permute as PM
    from paroatten_amd import quant as Q
    qp, kp, vp = PM.rope_permute(q, k, v, orders, grid, n_text, cos, sin)
    q8, qs, k8, ks = Q.per_warp_int8(qp, kp, km, BLKQ=64, WARPQ=32, BLKK=64)
    v8, vsc, vm = Q.per_channel_fp8(vp)
    return q8, qs, k8, ks, v8, vsc, vm


@pytest.mark.parametrize("B,H,D,grid,n_text,dtype,rope_kind,smooth_k", [
    (2, 4, 64, (4, 8, 12), 32, torch.float16, "cog", True),     # text + image, multiple of 64
    (1, 7, 64, (3, 5, 7), 226, torch.bfloat16, "cog", False),   # ragged tail (331 = 5*64 + 11: an empty Q group)
    (1, 3, 128, (3, 6, 16), 0, torch.bfloat16, "wan", True),    # Wan layout
    (2, 2, 128, (2, 5, 9), 17, torch.float16, None, False),     # no rotation, tail of 43
    (1, 13, 64, (2, 3, 4), 8, torch.float16, "cog", True),      # one block, more heads than orders
])
def test_fused_prep_matches_oracle_and_chain(dev, B, H, D, grid, n_text, dtype, rope_kind, smooth_k):
    from paroatten_amd import permute as PM
    q, k, v, plan, cos, sin, N = _case(dev, B, H, D, grid, n_text, dtype, 3, rope_kind)
    orders = PM.head_orders(plan, 0, dev)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    cd = None if cos is None else cos.to(dev)
    sd = None if sin is None else sin.to(dev)

    # oracle: rotate, permute, quantise
    qr, kr = q.clone(), k.clone()
    if cos is not None:
        qr[:, :, n_text:] = O.rope_apply_cog(q[:, :, n_text:], cos, sin)
        kr[:, :, n_text:] = O.rope_apply_cog(k[:, :, n_text:], cos, sin)
    rq, rk, rv = O.permute_qk(qr, kr, v, plan, 0, grid, n_text)
    km = None
    if smooth_k:
        km_dev = PM.rope_k_mean(kd, grid, n_text, cd, sd)
        want = rk.float().mean(dim=2, keepdim=True)
        ulp = want.abs().clamp_min(1e-3) * (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10)
        assert km_dev.shape == (B, H, 1, D) and km_dev.dtype == dtype
        assert bool(((km_dev.cpu().float() - want).abs() <= ulp).all())
        km = km_dev.cpu()       # the same rounded mean on both sides
    o8 = O.per_warp_int8(rq, rk, km=km, BLKQ=64, WARPQ=32, BLKK=64)
    ov8, ovs, ovm = O.per_channel_fp8(rv)

    got = PM.rope_permute_quant(qd, kd, vd, orders, grid, n_text, cd, sd, km=None if km is None else km.to(dev))
    assert torch.equal(got.q8.cpu(), o8[0]) and torch.equal(got.q_scale.cpu(), o8[1])
    assert torch.equal(got.k8.cpu(), o8[2]) and torch.equal(got.k_scale.cpu(), o8[3])

    # the separate kernels (each checked against the oracle in its own test)
    ch = _chain(dev, qd, kd, vd, orders, grid, n_text, cd, sd, None if km is None else km.to(dev))
    assert torch.equal(got.q8, ch[0]) and torch.equal(got.q_scale, ch[1])
    assert torch.equal(got.k8, ch[2]) and torch.equal(got.k_scale, ch[3])
    _same_v(got, ch[4], ch[5], ch[6])
    # V statistics against the oracle (mean: fp32 sum in another order); the offset = the oracle's mean
    # plus the mean rounding residual of the codes the kernel wrote, which stays a small fraction of a step
    assert torch.allclose(got.v_scale.cpu(), ovs, atol=0, rtol=1e-5)
    want = v8_offset_expected(rv, untile_v8(got.v8, B, H, N, D), got.v_scale)
    assert torch.allclose(got.v_mean.cpu().double(), want, atol=1e-5, rtol=1e-5)
    assert bool(((got.v_mean.cpu() - ovm).abs() <= 1e-6 + 16.0 * ovs).all())   # never more than half the widest rounding cell


def test_fused_prep_token_major_views_and_attention(dev):
    """inputs as the processors have them ([B,N,H*D] projections viewed [B,H,N,D]); the attention
    kernel on the fused operands returns exactly what the chain returns."""
    from paroatten_amd import _qattn_sm80 as qattn
    from paroatten_amd import permute as PM
    from paroatten_amd import rope
    B, H, D, grid, n_text = 2, 3, 64, (4, 6, 10), 16
    N = n_text + 240
    g = torch.Generator().manual_seed(5)
    proj = [torch.randn(B, N, H * D, generator=g).to(dev, torch.bfloat16) for _ in range(3)]
    q, k, v = (p.view(B, N, H, D).transpose(1, 2) for p in proj)
    plan = synth.make_permute_plan(1, H, seed=6)
    orders = PM.head_orders(plan, 0, dev)
    cos, sin = (t.to(dev) for t in rope.rope_table_cog(D, grid))
    nb = (N + 63) // 64
    mask = synth.make_block_mask(H, nb, 0.6, seed=7).to(dev)

    got = PM.rope_permute_quant(q, k, v, orders, grid, n_text, cos, sin)
    out_f = torch.empty((B, H, N, D), dtype=torch.bfloat16, device=dev)
    qattn.attn_sparse_prepacked(got.q8, got.k8, got.v8, got.v_scale, got.v_mean, out_f, got.q_scale, got.k_scale,
                                D ** -0.5, mask)

    ch = _chain(dev, q, k, v, orders, grid, n_text, cos, sin, None)
    qp, kp, vp = PM.rope_permute(q, k, v, orders, grid, n_text, cos, sin)
    out_c = torch.empty_like(out_f)
    qattn.qk_int8_sv_f16_accum_f16_attn(ch[0], ch[2], vp, out_c, ch[1], ch[3], 1, 0, 2, D ** -0.5, 0, mask)
    assert torch.equal(got.q8, ch[0]) and torch.equal(got.k8, ch[2])
    assert torch.allclose(out_f.float(), out_c.float(), atol=2e-3, rtol=1e-2)   # V mean: last-bit differences


def test_fused_prep_full_cogvideox_shape(dev):
    """B=2, H=48, N=17776, D=64, bf16 with RoPE: fused == chain on every INT8 byte and scale."""
    from paroatten_amd import permute as PM
    from paroatten_amd import rope
    wl = synth.WORKLOADS["cogvideox5b_rope"]
    q, k, v = synth.make_qkv_device(wl.B, wl.H, wl.N, wl.D, wl.dtype, seed=8, device=dev)
    plan = synth.make_permute_plan(1, wl.H, seed=9)
    orders = PM.head_orders(plan, 0, dev)
    cos, sin = (t.to(dev) for t in rope.rope_table_cog(wl.D, wl.grid))
    km = PM.rope_k_mean(k, wl.grid, wl.n_text, cos, sin)
    got = PM.rope_permute_quant(q, k, v, orders, wl.grid, wl.n_text, cos, sin, km=km)
    ch = _chain(dev, q, k, v, orders, wl.grid, wl.n_text, cos, sin, km)
    assert torch.equal(got.q8, ch[0]) and torch.equal(got.q_scale, ch[1])
    assert torch.equal(got.k8, ch[2]) and torch.equal(got.k_scale, ch[3])
    _same_v(got, ch[4], ch[5], ch[6])


@pytest.mark.parametrize("B,H,same_order", [(36, 64, True), (5, 33, False)])
def test_fused_prep_many_batch_head_pairs(dev, B, H, same_order):
    """long lists of (batch, head) pairs per workgroup (2304 pairs of one order: the head split is
    raised so that a workgroup's list fits) and pair counts that do not divide by the split."""
    from paroatten_amd import permute as PM
    from paroatten_amd import rope
    D, grid, n_text = 64, (2, 4, 8), 5
    N = n_text + 64
    q, k, v = (t.to(dev) for t in synth.make_qkv(B, H, N, D, torch.bfloat16, seed=31))
    if same_order:
        orders = torch.full((H,), 4, dtype=torch.int32, device=dev)
    else:
        orders = PM.head_orders(synth.make_permute_plan(1, H, seed=32), 0, dev)
    cos, sin = (t.to(dev) for t in rope.rope_table_cog(D, grid))
    km = PM.rope_k_mean(k, grid, n_text, cos, sin)
    got = PM.rope_permute_quant(q, k, v, orders, grid, n_text, cos, sin, km=km)
    ch = _chain(dev, q, k, v, orders, grid, n_text, cos, sin, km)
    assert torch.equal(got.q8, ch[0]) and torch.equal(got.q_scale, ch[1])
    assert torch.equal(got.k8, ch[2]) and torch.equal(got.k_scale, ch[3])
    _same_v(got, ch[4], ch[5], ch[6])


def test_fused_prep_rejects_bad_arguments(dev):
    from paroatten_amd import permute as PM
    q = torch.zeros(1, 2, 128, 64, dtype=torch.float16, device=dev)
    orders = torch.zeros(2, dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError):
        PM.rope_permute_quant(q, q, q, orders, (2, 8, 9), 0)            # 144 != 128 tokens
    with pytest.raises(RuntimeError):
        PM.rope_permute_quant(q, q, q[:, :, :, :32], orders, (2, 8, 8), 0)
    with pytest.raises(RuntimeError):
        PM.rope_permute_quant(q, q, q, orders, (2, 8, 8), 0, km=torch.zeros(1, 2, 1, 64, device=dev))  # dtype


@pytest.mark.parametrize("D,grid,n_text,dtype", [(64, (4, 6, 10), 16, torch.float16), (128, (3, 5, 9), 0, torch.bfloat16),
                                                 (64, (3, 5, 7), 226, torch.bfloat16)])
def test_attention_with_folded_inverse_permutation(dev, D, grid, n_text, dtype):
    """paro_attn_sparse_unpermute_fwd == attention followed by the inverse permutation, bit for bit,
    into a token-major buffer; an empty mask row still writes its zeros at the unpermuted places."""
    from paroatten_amd import _qattn_sm80 as qattn
    from paroatten_amd import permute as PM
    B, H = 2, 5
    N = n_text + grid[0] * grid[1] * grid[2]
    q, k, v = (t.to(dev) for t in synth.make_qkv(B, H, N, D, dtype, seed=21))
    plan = synth.make_permute_plan(1, H, seed=22)
    orders = PM.head_orders(plan, 0, dev)
    nb = (N + 63) // 64
    mask = synth.make_block_mask(H, nb, 0.6, seed=23).to(dev)
    mask[1, nb - 1, :] = False
    ops = PM.rope_permute_quant(q, k, v, orders, grid, n_text)
    plain = torch.empty((B, H, N, D), dtype=dtype, device=dev)
    qattn.attn_sparse_prepacked(ops.q8, ops.k8, ops.v8, ops.v_scale, ops.v_mean, plain, ops.q_scale, ops.k_scale,
                                D ** -0.5, mask)
    want = PM.permute_inverse(plain, orders, grid, n_text)
    token_major = torch.full((B, N, H, D), 7.0, dtype=dtype, device=dev)
    qattn.attn_sparse_prepacked(ops.q8, ops.k8, ops.v8, ops.v_scale, ops.v_mean, token_major.transpose(1, 2),
                                ops.q_scale, ops.k_scale, D ** -0.5, mask, unpermute=(orders, grid, n_text))
    assert torch.equal(token_major.transpose(1, 2), want)
    # with the log-sum-exp (exact exponentials): lse stays in q-row order, the output is unpermuted
    lse_p = qattn.attn_sparse_prepacked(ops.q8, ops.k8, ops.v8, ops.v_scale, ops.v_mean, plain, ops.q_scale,
                                        ops.k_scale, D ** -0.5, mask, return_lse=1)
    lse_u = qattn.attn_sparse_prepacked(ops.q8, ops.k8, ops.v8, ops.v_scale, ops.v_mean, token_major.transpose(1, 2),
                                        ops.q_scale, ops.k_scale, D ** -0.5, mask, return_lse=1,
                                        unpermute=(orders, grid, n_text))
    assert torch.equal(lse_p, lse_u)
    assert torch.equal(token_major.transpose(1, 2), PM.permute_inverse(plain, orders, grid, n_text))
    with pytest.raises(RuntimeError):
        qattn.attn_sparse_prepacked(ops.q8, ops.k8, ops.v8, ops.v_scale, ops.v_mean, plain, ops.q_scale, ops.k_scale,
                                    D ** -0.5, mask, unpermute=(orders, (grid[0], grid[1], grid[2] + 1), n_text))


@pytest.mark.parametrize("B,H,D,grid,n_text,dtype,rope_kind", [
    (2, 5, 64, (3, 10, 11), 35, torch.float16, "cog"),      # a text prefix inside the first chunk, ragged last chunk
    (1, 6, 128, (4, 9, 31), 0, torch.bfloat16, "wan"),
    (1, 3, 64, (2, 8, 8), 0, torch.bfloat16, None),         # no rotation, fewer heads than a head group
])
def test_k_mean_inside_the_preparation_call(dev, B, H, D, grid, n_text, dtype, rope_kind):
    """km="mean" (paro_rope_k_mean_permute_quant_fwd: the K sums and the V statistics in one launch, their
    second steps in another) against rope_k_mean followed by rope_permute_quant with that mean: every output
    bit for bit, the mean included."""
    from paroatten_amd import permute as PM
    q, k, v, plan, cos, sin, N = _case(dev, B, H, D, grid, n_text, dtype, 41, rope_kind)
    q, k, v = q.to(dev), k.to(dev), v.to(dev)
    k = k + 2.0     # a mean worth subtracting
    cos, sin = (None, None) if cos is None else (cos.to(dev), sin.to(dev))
    orders = PM.head_orders(plan, 0, dev)
    km = PM.rope_k_mean(k, grid, n_text, cos, sin)
    two = PM.rope_permute_quant(q, k, v, orders, grid, n_text, cos, sin, km=km)
    one = PM.rope_permute_quant(q, k, v, orders, grid, n_text, cos, sin, km="mean")
    assert two.k_mean is None and one.k_mean is not None
    assert torch.equal(one.k_mean.view(torch.int16), km.view(torch.int16))
    for name in ("q8", "q_scale", "k8", "k_scale", "v8", "v_scale", "v_mean"):
        a, b = getattr(one, name), getattr(two, name)
        assert torch.equal(a.view(torch.uint8) if a.dtype != torch.float32 else a, b.view(torch.uint8) if b.dtype != torch.float32 else b), name
    assert float(km.float().abs().mean()) > 0.5
