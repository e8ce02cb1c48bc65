"""GPU parity of the block-sparse attention kernel against the oracle.

Integer stage: the raw int32 Q.K^T accumulators dumped by the kernel are bit-exact.
Floating-point stage: outputs within atol 2e-2 of the oracle and cosine >= 0.999 (the tolerance
the FP8 P.V product is specified to; the oracle keeps P and V in 16/32-bit)."""
import pytest
import torch

from conftest import assert_attention_close, cosine
from oracle import paro_oracle as O
from paroatten_amd import synth

pytestmark = pytest.mark.gpu

ATOL = 2e-2
COS = 0.999


def _run(dev, B, H, N, D, dtype, density, seed, Hkv=None, causal=False, smooth_k=True, return_lse=True,
         mask=None, batch_mask=False, exact_exp=False):
    import paroatten_amd as P
    Hkv = Hkv or H
    q, _, _ = synth.make_qkv(B, H, N, D, dtype, seed=seed)
    _, k, v = synth.make_qkv(B, Hkv, N, D, dtype, seed=seed + 1)
    nb = (N + 63) // 64
    if mask is None:
        mask = synth.make_block_mask(H, nb, density, seed=seed + 2)
    mask_b = mask[None].expand(B, H, nb, nb).contiguous() if mask.dim() == 3 else mask
    km = k.float().mean(dim=2, keepdim=True).to(dtype) if smooth_k else None
    q8, qs, k8, ks = O.per_warp_int8(q, k, km=km, BLKQ=64, WARPQ=32, BLKK=64)
    o_ref, lse_ref = O.sparse_attention(q8, k8, v, qs, ks, mask_b, D ** -0.5, is_causal=causal, out_dtype=dtype)
    a_ref, _ = O.sparse_attention(q8, k8, v.abs(), qs, ks, mask_b, D ** -0.5, is_causal=causal, out_dtype=torch.float32)
    m_dev = (mask_b if batch_mask else mask).to(dev)
    out = P.paroattn_qk_int8_pv_fp16_cuda(q.to(dev), k.to(dev), v.to(dev), m_dev, is_causal=causal,
                                          smooth_k=smooth_k, return_lse=return_lse, exact_exp=exact_exp)
    o, lse = out if return_lse else (out, None)
    lse_ref = lse_ref / O.LOG2E
    if smooth_k:
        # the operator returns the log-sum-exp of the scores of q and k as given: the oracle's, taken on K - km,
        # plus sm_scale * q . km per row
        lse_ref = lse_ref + torch.einsum("bhnd,bhd->bhn", q.float(),
                                         km.float().squeeze(2).repeat_interleave(H // Hkv, dim=1)) * D ** -0.5
    return o.cpu(), (None if lse is None else lse.cpu()), (o_ref, a_ref), lse_ref, mask_b


def _assert_close(o, ref, baseline_shape=False):
    """ref = (o_ref, a_ref) as _run returns them: the one rule of conftest.assert_attention_close
    (|o - o_ref| <= 2e-2 + 2^-3 * sum_j p_ij |v_j|, all but 1e-3 within 2e-2 + 2^-4 * that, cosine >= 0.999); at a benchmark shape additionally the
    flat atol 2e-2 the benchmark states."""
    o_ref, a_ref = ref
    assert_attention_close(o, o_ref, a_ref, COS)
    if baseline_shape:
        err = (o.float() - o_ref.float()).abs().max().item()
        assert err <= ATOL, f"max abs err {err} > {ATOL}"


def test_cfg0_plumbing(dev):
    """benchmark configuration 0: B=1,H=2,D=64,fp16,N=4096, density 0.5, K bias.  With lse the kernel
    evaluates exact exponentials; without, its default fast path builds the e4m3 weights directly."""
    o, lse, o_ref, lse_ref, _ = _run(dev, 1, 2, 4096, 64, torch.float16, 0.5, seed=0)
    _assert_close(o, o_ref, baseline_shape=True)
    assert torch.allclose(lse, lse_ref, atol=2e-3, rtol=1e-4)
    for h in range(2):
        assert cosine(o[:, h], o_ref[0][:, h]) >= COS
    for exact in (False, True):
        o2, _, o_ref2, _, _ = _run(dev, 1, 2, 4096, 64, torch.float16, 0.5, seed=0, return_lse=False,
                                   exact_exp=exact)
        _assert_close(o2, o_ref2, baseline_shape=True)
        for h in range(2):
            assert cosine(o2[:, h], o_ref2[0][:, h]) >= COS
    assert torch.equal(o2, o)  # exact_exp without lse == the lse instantiation


@pytest.mark.parametrize("D,dtype", [(64, torch.bfloat16), (128, torch.float16), (128, torch.bfloat16)])
@pytest.mark.parametrize("N", [1000, 2048])
def test_shapes_and_tails(dev, D, dtype, N):
    o, lse, o_ref, lse_ref, _ = _run(dev, 2, 3, N, D, dtype, 0.4, seed=N + D, batch_mask=(N == 1000))
    _assert_close(o, o_ref)
    assert torch.allclose(lse, lse_ref, atol=2e-3, rtol=1e-4)
    o, _, o_ref, _, _ = _run(dev, 2, 3, N, D, dtype, 0.4, seed=N + D, batch_mask=(N == 1000), return_lse=False)
    _assert_close(o, o_ref)  # default fast exponential


def test_dense_equals_masked_all_true(dev):
    nb = 9
    mask = torch.ones(2, nb, nb, dtype=torch.bool)
    for lse_on in (True, False):
        o, lse, o_ref, lse_ref, _ = _run(dev, 1, 2, 64 * nb - 13, 64, torch.float16, 1.0, seed=4, mask=mask,
                                         return_lse=lse_on)
        _assert_close(o, o_ref)


def test_empty_rows_and_single_block(dev):
    """A q-block with no kept k-block outputs exactly 0 (lse = -inf); one kept block = local
    attention."""
    nb = 6
    mask = torch.zeros(2, nb, nb, dtype=torch.bool)
    mask[0, 0, 3] = True
    mask[0, 2, 2] = True
    mask[1] = torch.eye(nb, dtype=torch.bool)
    mask[1, 4, 4] = False
    o, lse, o_ref, lse_ref, _ = _run(dev, 1, 2, 64 * nb - 5, 64, torch.float16, 0.0, seed=8, mask=mask)
    _assert_close(o, o_ref)
    assert torch.count_nonzero(o[0, 0, 64:128]) == 0
    assert torch.count_nonzero(o[0, 1, 256:320]) == 0
    assert torch.isinf(lse[0, 1, 256:320]).all() and (lse[0, 1, 256:320] < 0).all()
    keep = ~torch.isinf(lse_ref)
    assert torch.equal(torch.isinf(lse), torch.isinf(lse_ref))
    assert torch.allclose(lse[keep], lse_ref[keep], atol=2e-3, rtol=1e-4)


def test_lse_with_k_smoothing_is_that_of_the_unsmoothed_scores(dev):
    """K smoothing lowers every score of row i by sm_scale * q_i . km: invisible to the softmax, not to the
    log-sum-exp.  The operator puts it back: its lse with smooth_k=True agrees with the lse of the same call without
    smoothing up to the INT8 rounding of the two different K tensors, and with the oracle's lse of unsmoothed
    quantised scores; left out, the difference would be of order 1 (the K of the synthetic inputs carries a bias)."""
    import paroatten_amd as P
    B, H, Hkv, N, D = 1, 4, 2, 900, 64
    q, _, _ = synth.make_qkv(B, H, N, D, torch.float16, seed=21)
    _, k, v = synth.make_qkv(B, Hkv, N, D, torch.float16, seed=22)
    nb = (N + 63) // 64
    mask = synth.make_block_mask(H, nb, 0.5, seed=23)
    qd, kd, vd, md = q.to(dev), k.to(dev), v.to(dev), mask.to(dev)
    lse_s = P.paroattn_qk_int8_pv_fp16_cuda(qd, kd, vd, md, smooth_k=True, return_lse=True)[1].cpu()
    lse_u = P.paroattn_qk_int8_pv_fp16_cuda(qd, kd, vd, md, smooth_k=False, return_lse=True)[1].cpu()
    tr = lambda t: t.transpose(1, 2).contiguous()
    lse_n = P.paroattn_qk_int8_pv_fp16_cuda(tr(qd), tr(kd), tr(vd), md, tensor_layout="NHD", smooth_k=True,
                                            return_lse=True)[1].cpu()
    q8, qs, k8, ks = O.per_warp_int8(q, k, km=None, BLKQ=64, WARPQ=32, BLKK=64)
    _, lse_o = O.sparse_attention(q8, k8, v, qs, ks, mask[None], D ** -0.5)
    # (the unsmoothed K spends most of its INT8 range on the bias: its scores carry a rounding noise of a few 1e-2)
    for other in (lse_u, lse_o / O.LOG2E):
        d = (lse_s - other).abs()
        assert float(d.max()) < 0.2 and float(d.mean()) < 0.03, (float(d.max()), float(d.mean()))
    assert torch.allclose(lse_n, lse_s, atol=1e-4, rtol=1e-5)      # the correction is summed in another order
    corr = torch.einsum("bhnd,bhd->bhn", q.float(), k.float().mean(dim=2).repeat_interleave(H // Hkv, dim=1)) * D ** -0.5
    assert float(corr.abs().mean()) > 0.3      # what an uncorrected lse would be off by


def test_causal_and_gqa(dev):
    o, lse, o_ref, lse_ref, _ = _run(dev, 1, 4, 700, 64, torch.float16, 1.0, seed=12, Hkv=2, causal=True,
                                     mask=torch.ones(4, 11, 11, dtype=torch.bool))
    _assert_close(o, o_ref)
    assert torch.allclose(lse, lse_ref, atol=2e-3, rtol=1e-4)
    o, _, o_ref, _, _ = _run(dev, 1, 4, 700, 64, torch.float16, 1.0, seed=12, Hkv=2, causal=True,
                             mask=torch.ones(4, 11, 11, dtype=torch.bool), return_lse=False)
    _assert_close(o, o_ref)


def test_no_smoothing_paths(dev):
    import paroatten_amd as P
    B, H, N, D = 1, 2, 512, 64
    q, k, v = synth.make_qkv(B, H, N, D, torch.float16, seed=21)
    mask = synth.make_block_mask(H, 8, 0.6, seed=22)
    q8, qs, k8, ks = O.per_warp_int8(q, k, BLKQ=64, WARPQ=32, BLKK=64)
    o_ref, _ = O.sparse_attention(q8, k8, v, qs, ks, mask[None], D ** -0.5)
    a_ref, _ = O.sparse_attention(q8, k8, v.abs(), qs, ks, mask[None], D ** -0.5, out_dtype=torch.float32)
    o = P.paroattn_qk_int8_pv_fp16_cuda(q.to(dev), k.to(dev), v.to(dev), mask.to(dev), smooth_k=False,
                                        smooth_v=False).cpu()
    _assert_close(o, (o_ref, a_ref))


def test_head_dim_padding(dev):
    import paroatten_amd as P
    B, H, N, D = 1, 2, 320, 96
    q, k, v = synth.make_qkv(B, H, N, D, torch.bfloat16, seed=31)
    mask = synth.make_block_mask(H, 5, 0.7, seed=32)
    pad = lambda t: torch.nn.functional.pad(t, (0, 128 - D))
    q8, qs, k8, ks = O.per_warp_int8(pad(q), pad(k), BLKQ=64, WARPQ=32, BLKK=64)
    o_ref, _ = O.sparse_attention(q8, k8, pad(v), qs, ks, mask[None], D ** -0.5, out_dtype=torch.bfloat16)
    a_ref, _ = O.sparse_attention(q8, k8, pad(v).abs(), qs, ks, mask[None], D ** -0.5, out_dtype=torch.float32)
    o = P.paroattn_qk_int8_pv_fp16_cuda(q.to(dev), k.to(dev), v.to(dev), mask.to(dev)).cpu()
    assert o.shape == (B, H, N, D)
    _assert_close(o, (o_ref[..., :D], a_ref[..., :D]))


@pytest.mark.parametrize("D", [64, 128])
def test_int32_qk_accumulators_bitexact(dev, D):
    """The kernel's own MFMA path, dumped block by block, equals the integer matmul exactly."""
    import paroatten_amd._lib as L
    from paroatten_amd.quant import per_channel_fp8
    B, H, N = 1, 2, 333
    nb = (N + 63) // 64
    q, k, v = synth.make_qkv(B, H, N, D, torch.float16, seed=41 + D)
    q8, qs, k8, ks = O.per_warp_int8(q, k, BLKQ=64, WARPQ=32, BLKK=64)
    mask = synth.make_block_mask(H, nb, 0.5, seed=43)[None].contiguous()
    s_ref = O.qk_int32(q8, k8)
    lib = L.load()
    v8, vsc, vm = per_channel_fp8(v.to(dev))
    out = torch.empty(B, H, N, D, dtype=torch.float16, device=dev)
    dump = torch.full((B, H, nb * 64, nb * 64), -(2 ** 31), dtype=torch.int32, device=dev)
    q8d, k8d, qsd, ksd, md = q8.to(dev), k8.to(dev), qs.to(dev), ks.to(dev), mask.to(dev)
    L.check(lib.paro_attn_sparse_fwd(
        L.ptr(q8d), L.ptr(k8d), L.ptr(v8), L.ptr(qsd), L.ptr(ksd), L.ptr(vsc), L.ptr(vm), L.ptr(md), md.stride(0),
        L.ptr(out), 0, None, L.ptr(dump), B, H, H, N, N, D,
        q8d.stride(0), q8d.stride(1), q8d.stride(2), k8d.stride(0), k8d.stride(1), k8d.stride(2),
        out.stride(0), out.stride(1), out.stride(2), D ** -0.5, 0, 0, L.stream_of(out)))
    dump = dump.cpu()
    keep = O.expand_block_mask(mask, nb * 64, nb * 64)
    # computed blocks: exact on the real rows/columns; skipped blocks: untouched
    assert torch.equal(dump[..., :N, :N][keep[..., :N, :N]], s_ref[keep[..., :N, :N]])
    assert (dump[~keep] == -(2 ** 31)).all()
    # (rows/columns past N inside computed blocks hold products with a re-read last row; the
    # kernel masks those columns out of the softmax and never stores those rows)


def test_nhd_layout_and_paroattn_entry(dev):
    """tensor_layout="NHD" ([B,N,H,D]) gives exactly the HND result; `paroattn` with sparse=None is the
    all-true mask (core.py:13-85 of the reference documents both and can run neither)."""
    import paroatten_amd as P
    B, H, N, D = 2, 3, 700, 64
    q, k, v = synth.make_qkv(B, H, N, D, torch.float16, seed=31)
    nb = (N + 63) // 64
    mask = synth.make_block_mask(H, nb, 0.5, seed=32).to(dev)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    o_hnd, lse_hnd = P.paroattn_qk_int8_pv_fp16_cuda(qd, kd, vd, mask, return_lse=True)
    qn, kn, vn = (t.transpose(1, 2).contiguous() for t in (qd, kd, vd))
    o_nhd, lse_nhd = P.paroattn_qk_int8_pv_fp16_cuda(qn, kn, vn, mask, tensor_layout="NHD", return_lse=True)
    assert o_nhd.shape == (B, N, H, D)
    assert torch.equal(o_nhd.transpose(1, 2), o_hnd) and torch.equal(lse_nhd, lse_hnd)
    dense = P.paroattn(qd, kd, vd, smooth_k=True)
    full = P.paroattn_qk_int8_pv_fp16_cuda(qd, kd, vd, torch.ones(H, nb, nb, dtype=torch.bool, device=dev),
                                           smooth_k=True)
    assert torch.equal(dense, full)
    # against attention on the UNQUANTISED tensors: INT8 Q/K (K smoothed) and FP8 P/V together
    ref = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    assert cosine(dense.cpu(), ref) >= 0.998


def _ramp_case(B, H, N, D, dtype, seed, pattern):
    """Scores that climb along the key axis, so that later kept blocks exceed the running row maximum by
    more than the FP8 headroom (3.75 octaves) again and again: "ramp" adds a common direction w to every
    query and b*w*step to the keys of block b (each block ~4.3 octaves above the one before); "spike" puts
    single keys 12 and 25 octaves above the rest into late blocks."""
    q, k, v = synth.make_qkv(B, H, N, D, dtype, seed=seed, k_bias_std=0.0)
    g = torch.Generator().manual_seed(seed + 100)
    w = torch.randn(D, generator=g)
    w = w / w.norm()
    qf, kf = q.float() * 0.3 + 4.0 * w, k.float() * 0.3
    blk = torch.arange(N) // 64
    sm = D ** -0.5
    if pattern == "ramp":
        kf = kf + (3.0 * blk.float() / (4.0 * sm))[None, None, :, None] * w     # +3 nats per block
    else:
        for j, nats in ((N // 2 + 5, 8.0), (N - 70, 17.0)):
            kf[:, :, j] += (nats / (4.0 * sm)) * w
    return qf.to(dtype), kf.to(dtype), v


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("pattern,causal,density", [("ramp", False, 1.0), ("ramp", False, 0.5), ("ramp", True, 1.0),
                                                    ("spike", False, 0.5), ("spike", True, 1.0)])
def test_fast_path_maximum_recovery(dev, D, pattern, causal, density):
    """The default (fast) softmax path computes a block's weights against the running maximum as it is
    and only afterwards notices, from a NaN in the row sums of the bytes it built, that a score was more
    than the FP8 headroom above it; it then refreshes the maximum and recomputes the block.  Here that happens in
    block after block (every row, dense, sparse and causal masks): the output must be finite and match
    both the oracle and the exact-exponential path."""
    import paroatten_amd as P
    B, H, N = 1, 2, 1024 - 19
    nb = (N + 63) // 64
    q, k, v = _ramp_case(B, H, N, D, torch.float16, 7 + D, pattern)
    mask = (torch.ones(H, nb, nb, dtype=torch.bool) if density == 1.0
            else synth.make_block_mask(H, nb, density, seed=5))
    q8, qs, k8, ks = O.per_warp_int8(q, k, BLKQ=64, WARPQ=32, BLKK=64)
    o_ref, _ = O.sparse_attention(q8, k8, v, qs, ks, mask[None], D ** -0.5, is_causal=causal, out_dtype=torch.float32)
    # rows that one or a few keys dominate: the error is FP8's relative rounding error on each product
    # p*v (at most 2^-4 for V's code and for P's), so the elementwise bound is relative to sum_j p_ij |v_j| (conftest.assert_attention_close)
    a_ref, _ = O.sparse_attention(q8, k8, v.abs(), qs, ks, mask[None], D ** -0.5, is_causal=causal,
                                  out_dtype=torch.float32)

    def close(a, b):
        # (every row of this case hangs on one or two keys: two roundings coincide on about 1 % of the elements)
        assert_attention_close(a, b, a_ref, COS, frac_one_step=2e-2)
    # the case does what it is meant to: block maxima climb by more than the headroom many times per row
    s = O.qk_int32(q8, k8)[0, 0].double() * qs[0, 0].double().repeat_interleave(32)[:N, None] \
        * ks[0, 0].double().repeat_interleave(64)[None, :N] * (D ** -0.5) * O.LOG2E
    keep = O.expand_block_mask(mask[0], N, N)
    if causal:
        keep = keep & (torch.arange(N)[None, :] <= torch.arange(N)[:, None])
    s = s.masked_fill(~keep, float("-inf"))
    pad = torch.full((N, nb * 64 - N), float("-inf"), dtype=s.dtype)
    blockmax = torch.cat([s, pad], dim=1).reshape(N, nb, 64).amax(dim=-1)
    run = torch.cummax(blockmax, dim=1).values
    jumps = ((blockmax[:, 1:] - run[:, :-1]) > 3.75).sum(dim=1)
    assert int(jumps.max()) >= (1 if pattern == "spike" else 4), int(jumps.max())
    kw = dict(is_causal=causal, smooth_k=False)
    o_fast = P.paroattn_qk_int8_pv_fp16_cuda(q.to(dev), k.to(dev), v.to(dev), mask.to(dev), **kw).cpu()
    o_exact = P.paroattn_qk_int8_pv_fp16_cuda(q.to(dev), k.to(dev), v.to(dev), mask.to(dev), exact_exp=True, **kw).cpu()
    assert torch.isfinite(o_fast.float()).all() and torch.isfinite(o_exact.float()).all()
    close(o_fast, o_ref)
    close(o_exact, o_ref)
    close(o_fast, o_exact)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("row", [3, 20, 37, 59])
def test_fast_path_overflow_of_a_single_row(dev, D, row):
    """One q-row of one q-block alone meets a key far above its running maximum, late in its row: the row sits
    in the lower or upper half of either wave's 32 rows (the row sums of rows j and j + 16 share a lane of the
    row-sum product, and the overflow test has to see each of them).  Every other row must be untouched by
    the refresh that this row forces on its wave (same result as the exact path to the usual tolerance)."""
    import paroatten_amd as P
    B, H, N = 1, 1, 640
    nb = N // 64
    q, k, v = synth.make_qkv(B, H, N, D, torch.float16, seed=row, k_bias_std=0.0)
    g = torch.Generator().manual_seed(1000 + row)
    w = torch.randn(D, generator=g)
    w = w / w.norm()
    qf, kf = q.float() * 0.3, k.float() * 0.3
    qrow, key = 64 * 3 + row, 64 * 8 + 11            # q-block 3, key block 8 of 10
    sm = D ** -0.5
    qf[0, 0, qrow] = 4.0 * w
    kf[0, 0, key] = (14.0 / (4.0 * sm)) * w            # 14 nats = 20 octaves above the rest, for this row only
    q, k = qf.to(torch.float16), kf.to(torch.float16)
    mask = torch.ones(H, nb, nb, dtype=torch.bool)
    q8, qs, k8, ks = O.per_warp_int8(q, k, BLKQ=64, WARPQ=32, BLKK=64)
    o_ref, _ = O.sparse_attention(q8, k8, v, qs, ks, mask[None], sm, out_dtype=torch.float32)
    a_ref, _ = O.sparse_attention(q8, k8, v.abs(), qs, ks, mask[None], sm, out_dtype=torch.float32)
    kw = dict(smooth_k=False)
    o_fast = P.paroattn_qk_int8_pv_fp16_cuda(q.to(dev), k.to(dev), v.to(dev), mask.to(dev), **kw).cpu()
    o_exact = P.paroattn_qk_int8_pv_fp16_cuda(q.to(dev), k.to(dev), v.to(dev), mask.to(dev), exact_exp=True, **kw).cpu()
    assert torch.isfinite(o_fast.float()).all()
    for got in (o_fast, o_exact):
        assert_attention_close(got, o_ref, a_ref, COS)
    # the row itself is dominated by the one key: its output is that key's V row to FP8 accuracy
    dom = o_fast[0, 0, qrow].float()
    assert cosine(dom, v[0, 0, key].float()) >= 0.995
    # and the other rows of its q-block agree with the exact path like any other row
    others = [r for r in range(64 * 3, 64 * 4) if r != qrow]
    assert cosine(o_fast[0, 0, others], o_exact[0, 0, others]) >= COS


@pytest.mark.parametrize("D,H,N", [(128, 8, 16384), (64, 16, 12352)])
def test_paced_launch_is_bit_identical(dev, D, H, N, monkeypatch):
    """PARO_ATTN_PACED (resident workgroups per XCD that take their q-blocks generation by generation)
    against PARO_ATTN_UNPACED: the launch form may not change a single bit, whether the workgroups wait
    for each other (default: for all but a share of the generation), for all, for next to none, or never
    (a spin limit of zero, forced through the environment: the meeting point only paces).  Shapes with more q-blocks per XCD than workgroups fit on it, so that the
    paced kernel really runs several generations; checked against the oracle on one head."""
    from paroatten_amd import _qattn_sm80 as qattn
    from paroatten_amd import quant as Q
    B = 1
    nb = (N + 63) // 64
    q, k, v = synth.make_qkv_device(B, H, N, D, torch.bfloat16, seed=5, device=dev)
    mask = synth.make_block_mask(H, nb, 0.25, seed=6, device=dev)
    mask[1, 7] = False     # an empty row in the middle of a generation
    q8, qs, k8, ks = Q.per_warp_int8(q, k, None, BLKQ=64, WARPQ=32, BLKK=64)
    v8, vsc, vm = Q.per_channel_fp8(v)
    outs = []
    # (spin limit, arrivals a generation does not wait for): the library's defaults, no waiting at all, a short
    # limit, waiting for every workgroup, waiting for next to none
    for pacing, spins, slack in ((False, None, None), (True, None, None), (True, "0", None), (True, "3", None),
                                 (True, None, "0"), (True, None, "100000"), (True, "5", "7")):
        for name, val in (("PARO_ATTN_PACE_SPINS", spins), ("PARO_ATTN_PACE_SLACK", slack)):
            if val is None:
                monkeypatch.delenv(name, raising=False)
            else:
                monkeypatch.setenv(name, val)
        out = torch.full_like(q, float("nan"))
        lse = qattn.attn_sparse_prepacked(q8, k8, v8, vsc, vm, out, qs, ks, D ** -0.5, mask, return_lse=1, pacing=pacing)
        outs.append((out, lse))
    for o, l in outs[1:]:
        assert torch.equal(o.view(torch.int16), outs[0][0].view(torch.int16)) and torch.equal(l, outs[0][1])
    assert torch.count_nonzero(outs[0][0][0, 1, 7 * 64:8 * 64]) == 0
    h = 3
    o_ref, _ = O.sparse_attention(q8[:, h:h + 1].cpu(), k8[:, h:h + 1].cpu(), v[:, h:h + 1].cpu(), qs[:, h:h + 1].cpu(),
                                  ks[:, h:h + 1].cpu(), mask[None, h:h + 1].cpu(), D ** -0.5, out_dtype=torch.float32)
    a_ref, _ = O.sparse_attention(q8[:, h:h + 1].cpu(), k8[:, h:h + 1].cpu(), v[:, h:h + 1].cpu().abs(), qs[:, h:h + 1].cpu(),
                                  ks[:, h:h + 1].cpu(), mask[None, h:h + 1].cpu(), D ** -0.5, out_dtype=torch.float32)
    _assert_close(outs[1][0][:, h:h + 1].cpu(), (o_ref, a_ref), baseline_shape=True)
    # the fast-exponential instantiation and the folded inverse permutation go through the same launch code
    a = torch.empty_like(q)
    b = torch.empty_like(q)
    qattn.attn_sparse_prepacked(q8, k8, v8, vsc, vm, a, qs, ks, D ** -0.5, mask, pacing=False)
    qattn.attn_sparse_prepacked(q8, k8, v8, vsc, vm, b, qs, ks, D ** -0.5, mask, pacing=True)
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))


def test_paced_launches_that_overlap_on_two_streams(dev):
    """Two paced launches in flight at once on one GPU (two streams, as a caller that runs the two halves of a
    classifier-free-guidance batch side by side would have them): each takes its own set of the library's pacing
    counters, so neither zeroes the other's; the resident workgroups of the second cannot all be co-resident with
    the first, so its generations stop waiting after one bounded wait.  Results bit-identical to the launches run
    one after the other, and the pair takes no longer than 1.2 x the two alone plus one wait limit."""
    import time
    from paroatten_amd import _qattn_sm80 as qattn
    from paroatten_amd import quant as Q
    B, H, N, D = 1, 8, 16384, 128
    nb = N // 64
    cases = []
    for seed in (11, 12):
        q, k, v = synth.make_qkv_device(B, H, N, D, torch.bfloat16, seed=seed, device=dev)
        mask = synth.make_block_mask(H, nb, 0.25, seed=seed + 20, device=dev)
        q8, qs, k8, ks = Q.per_warp_int8(q, k, None, BLKQ=64, WARPQ=32, BLKK=64)
        v8, vsc, vm = Q.per_channel_fp8(v)
        cases.append((q8, k8, v8, vsc, vm, qs, ks, mask, torch.empty_like(q), torch.empty_like(q)))

    def launch(c, out):
        qattn.attn_sparse_prepacked(c[0], c[1], c[2], c[3], c[4], out, c[5], c[6], D ** -0.5, c[7], pacing=True)

    for c in cases:          # one after the other, on the current stream
        launch(c, c[8])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        for c in cases:
            launch(c, c[8])
    torch.cuda.synchronize()
    serial = (time.perf_counter() - t0) / 5
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for rep in range(6):     # (the first repetition warms the streams up and is not timed)
        if rep == 1:
            torch.cuda.synchronize()
            t0 = time.perf_counter()
        for c, s in zip(cases, streams):
            with torch.cuda.stream(s):
                launch(c, c[9])
    torch.cuda.synchronize()
    overlapped = (time.perf_counter() - t0) / 5
    for c in cases:
        assert torch.equal(c[8].view(torch.int16), c[9].view(torch.int16))
        assert torch.isfinite(c[9].float()).all()
    wait_limit = 128 * 2e-6      # nb / 2 rounds of one to two microseconds
    assert overlapped <= 1.2 * serial + wait_limit, (overlapped, serial)
