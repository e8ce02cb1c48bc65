"""GPU parity at the benchmark shapes.  The kernels run on the full (B, H) extent where the memory of
the test is bounded, the oracle checks whole heads of it (every head is independent), and
size-independent properties cover the rest: permutation round trips, bit-exact re-quantisation,
all-true masks against dense attention, zero rows for empty mask rows."""
import pytest
import torch

from conftest import assert_attention_close, cosine
from oracle import paro_oracle as O
from paroatten_amd import synth

pytestmark = pytest.mark.gpu
ATOL, COS = 2e-2, 0.999


def _check_heads(dev, wl, density, heads, seed, n_heads_total=None, with_rope=False):
    """Run the path (permute [+ RoPE] -> quant (K smoothed) -> sparse attention -> inverse permute)
    on `n_heads_total` heads of workload `wl` and compare the listed heads with the oracle.

    Without RoPE (what benchmark configurations 2-4 describe: N(0,1) Q/K/V, a per-channel bias on K that the
    mean smoothing removes) attention is diffuse and the bar is atol 2e-2 / cosine 0.999 on every
    element.  With RoPE the rotated K bias makes rows that one to three tokens dominate; there the
    absolute error is FP8's relative rounding error times an output of order 0.5, so the elementwise
    bound is the general rule of conftest.assert_attention_close (2e-2 plus two e4m3 steps of the |V|-weighted
    sum behind the element; cosine 0.999 stays)."""
    import paroatten_amd as P
    from paroatten_amd import permute as PM
    from paroatten_amd import rope
    H = n_heads_total or len(heads)
    B, N, D, nb = 1, wl.N, wl.D, wl.nb
    if H > 8:   # a full extent: generated on the device, the heads to check copied back
        q, k, v = (t.cpu() for t in synth.make_qkv_device(B, H, N, D, wl.dtype, seed=seed, device=dev))
        mask = synth.make_block_mask(H, nb, density, seed=seed + 1, device=dev).cpu()
    else:
        q, k, v = synth.make_qkv(B, H, N, D, wl.dtype, seed=seed)
        mask = synth.make_block_mask(H, nb, density, seed=seed + 1)
    plan = synth.make_permute_plan(1, H, seed=seed + 2)
    cos = sin = None
    if with_rope:
        cos, sin = (rope.rope_table_cog if wl.n_text else rope.rope_table_wan_real)(D, wl.grid)
    orders = PM.head_orders(plan, 0, dev)
    qp, kp, vp = PM.rope_permute(q.to(dev), k.to(dev), v.to(dev), orders, wl.grid, wl.n_text,
                                 None if cos is None else cos.to(dev), None if sin is None else sin.to(dev))
    o = P.paroattn_qk_int8_pv_fp16_cuda(qp, kp, vp, mask.to(dev), smooth_k=True)
    o = PM.permute_inverse(o.contiguous(), orders, wl.grid, wl.n_text).cpu()
    assert torch.isfinite(o.float()).all()
    for h in heads:
        sub_plan = {"permute": plan["permute"][:, h:h + 1], "empty": plan["empty"][:, h:h + 1]}
        ref = O.paro_path(q[:, h:h + 1], k[:, h:h + 1], v[:, h:h + 1], mask[None, h:h + 1], sub_plan, 0,
                          wl.grid, wl.n_text, cos, sin)
        err = (o[:, h:h + 1].float() - ref.float()).abs().max().item()
        c = cosine(o[:, h:h + 1], ref)
        assert c >= COS, f"head {h}: cosine {c}"
        if with_rope:
            a_ref = O.paro_path(q[:, h:h + 1], k[:, h:h + 1], v[:, h:h + 1].abs(), mask[None, h:h + 1], sub_plan, 0,
                                wl.grid, wl.n_text, cos, sin)
            assert_attention_close(o[:, h:h + 1], ref, a_ref, COS, what=f"head {h}")
        else:
            assert err <= ATOL, f"head {h}: max abs err {err}"


@pytest.mark.parametrize("density", [0.5, 0.3, 0.2])
def test_cfg2_cogvideox_heads(dev, density):
    """config 2: D=64, fp16, N=17776 (226 text + 13x30x45), K bias; 4 heads run, 2 checked in full."""
    _check_heads(dev, synth.WORKLOADS["cogvideox5b"], density, heads=[0, 3], seed=int(density * 100), n_heads_total=4)


def test_cfg2_whole_path_with_rope(dev):
    """the processors' whole sequence on the CogVideoX shape, RoPE included"""
    _check_heads(dev, synth.WORKLOADS["cogvideox5b"], 0.3, heads=[1], seed=77, n_heads_total=2, with_rope=True)


def test_cfg3_wan480p_full_extent(dev):
    """config 3 at its full extent: B=1, H=40, D=128, bf16, N=32760 (21x30x52), density 0.3; two of
    the 40 heads checked in full against the oracle."""
    wl = synth.WORKLOADS["wan14b_480p"]
    _check_heads(dev, wl, 0.3, heads=[7, 39], seed=33, n_heads_total=wl.H)


def test_cfg0_whole_path_with_permutation(dev):
    """config 0 as the benchmark list states it: B=1, H=2, D=64, fp16, a 16x16x16 grid (N=4096), K bias,
    density 0.5, a random F/H/W order per head applied before the attention and inverted after."""
    _check_heads(dev, synth.WORKLOADS["cfg0_plumbing"], 0.5, heads=[0, 1], seed=0)


def test_cfg1_rope_permute_full_shape(dev):
    """config 1: B=2, H=48, D=64, bf16, 226 + 13x30x45 tokens: inverse(forward) = identity on V, bit-exact
    index law per head, and Q/K of two heads against the oracle."""
    from paroatten_amd import permute as PM
    from paroatten_amd import rope
    wl = synth.WORKLOADS["cogvideox5b_rope"]
    B, H, N, D = wl.B, wl.H, wl.N, wl.D
    g = torch.Generator(device=dev).manual_seed(5)
    q = torch.randn(B, H, N, D, generator=g, device=dev, dtype=torch.float32).to(wl.dtype)
    k = torch.randn(B, H, N, D, generator=g, device=dev, dtype=torch.float32).to(wl.dtype)
    v = torch.randn(B, H, N, D, generator=g, device=dev, dtype=torch.float32).to(wl.dtype)
    plan = synth.make_permute_plan(1, H, seed=6)
    orders = PM.head_orders(plan, 0, dev)
    cos, sin = rope.rope_table_cog(D, wl.grid)
    qo, ko, vo = PM.rope_permute(q, k, v, orders, wl.grid, wl.n_text, cos.to(dev), sin.to(dev))
    assert torch.equal(PM.permute_inverse(vo, orders, wl.grid, wl.n_text), v)
    idx = PM.permute_index_map(orders, wl.grid).cpu()
    for h in (0, 17, 47):
        assert torch.equal(idx[h].long(), O.permute_index_map(wl.grid, int(plan["permute"][0, h])))
        # the permuted V rows are exactly the source rows at the mapped positions
        assert torch.equal(vo[1, h, wl.n_text:].cpu()[idx[h].long()], v[1, h, wl.n_text:].cpu())
        qh, kh = q[:, h:h + 1].cpu(), k[:, h:h + 1].cpu()
        qr, kr = qh.clone(), kh.clone()
        qr[:, :, wl.n_text:] = O.rope_apply_cog(qh[:, :, wl.n_text:], cos, sin)
        kr[:, :, wl.n_text:] = O.rope_apply_cog(kh[:, :, wl.n_text:], cos, sin)
        sub = {"permute": plan["permute"][:, h:h + 1], "empty": plan["empty"][:, h:h + 1]}
        rq, rk, _ = O.permute_qk(qr, kr, kr, sub, 0, wl.grid, wl.n_text)
        assert torch.equal(qo[:, h:h + 1].cpu(), rq) and torch.equal(ko[:, h:h + 1].cpu(), rk)


def test_cfg2_full_extent_properties(dev):
    """config 2 at its full extent (B=2, H=48): quantisation is bit-exact against the oracle on sampled
    heads, an empty mask row gives zeros, and the all-true mask of a sampled head matches torch's dense
    attention on the dequantised operands."""
    import paroatten_amd as P
    from paroatten_amd import quant as Q
    wl = synth.WORKLOADS["cogvideox5b"]
    B, H, N, D, nb = wl.B, wl.H, wl.N, wl.D, wl.nb
    q, k, v = synth.make_qkv_device(B, H, N, D, wl.dtype, seed=11, device=dev)
    km = k.mean(dim=2, keepdim=True)
    q8, qs, k8, ks = Q.per_warp_int8(q, k, km, BLKQ=64, WARPQ=32, BLKK=64)
    for b, h in ((0, 0), (1, 31)):
        r = O.per_warp_int8(q[b:b + 1, h:h + 1].cpu(), k[b:b + 1, h:h + 1].cpu(), km=km[b:b + 1, h:h + 1].cpu(),
                            BLKQ=64, WARPQ=32, BLKK=64)
        assert torch.equal(q8[b, h].cpu(), r[0][0, 0]) and torch.equal(qs[b, h].cpu(), r[1][0, 0])
        assert torch.equal(k8[b, h].cpu(), r[2][0, 0]) and torch.equal(ks[b, h].cpu(), r[3][0, 0])
    mask = synth.make_block_mask(H, nb, 0.2, seed=12, device=dev)
    mask[5, 100, :] = False   # an empty row
    mask[7] = True            # a dense head
    o = P.paroattn_qk_int8_pv_fp16_cuda(q, k, v, mask, smooth_k=True)
    assert torch.isfinite(o.float()).all()
    assert torch.count_nonzero(o[:, 5, 6400:6464]) == 0
    qd = q8[0, 7].float() * qs[0, 7].repeat_interleave(32)[:N, None]
    kd = k8[0, 7].float() * ks[0, 7].repeat_interleave(64)[:N, None]
    ref = torch.nn.functional.scaled_dot_product_attention(qd[None], kd[None], v[0, 7].float()[None])[0]
    assert (o[0, 7].float() - ref).abs().max().item() <= ATOL
    assert cosine(o[0, 7].cpu(), ref.cpu()) >= COS


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_cfg4_wan720p_full_extent(dev, dtype):
    """config 4 at its full extent: B=1, H=40, D=128, N=75600 (21x45x80), density 0.2 and the dense mask,
    in the configuration's own dtype (bfloat16) and in float16.  All 40 heads run; for three of them
    the oracle checks three whole q-blocks (rows are independent): atol 2e-2 and cosine >= 0.999.

    With i.i.d. V the output of a row that averages n keys is of size |v|/sqrt(n_eff), 5e-3..1e-2 here,
    far below atol, so the cosine is the measure that bites: it holds because the per-channel mean
    rounding residual of the FP8 codes (which does not shrink with n, and which the 8-significant-bit
    lattice of bfloat16 makes ~3e-4 |v|) is folded into the offset the epilogue adds back."""
    from paroatten_amd import _qattn_sm80 as qattn
    from paroatten_amd import permute as PM
    from paroatten_amd import quant as Q
    wl = synth.WORKLOADS["wan14b_720p"]
    H, N, D, nb = wl.H, wl.N, wl.D, wl.nb
    q, k, v = synth.make_qkv_device(1, H, N, D, dtype, seed=44, device=dev)
    plan = synth.make_permute_plan(1, H, seed=45)
    orders = PM.head_orders(plan, 0, dev)
    qp, kp, vp = PM.rope_permute(q, k, v, orders, wl.grid, 0)
    del q, k, v
    # the same rounded K mean on both sides (a one-ulp difference of a 16-bit mean would give two
    # different, equally valid int8 quantisations, whose difference is not what this test measures)
    km = kp.float().mean(dim=2, keepdim=True).to(dtype)
    g8 = Q.per_warp_int8(qp, kp, km, BLKQ=64, WARPQ=32, BLKK=64)
    heads, blocks = [0, 17, 39], [0, 500, 1180]
    rows = torch.cat([torch.arange(64 * b, 64 * b + 64) for b in blocks])
    refs = {}
    for h in heads:
        rq, rk, rv = qp[:, h:h + 1].cpu(), kp[:, h:h + 1].cpu(), vp[:, h:h + 1].cpu()
        q8, qs, k8, ks = O.per_warp_int8(rq, rk, km=km[:, h:h + 1].cpu(), BLKQ=64, WARPQ=32, BLKK=64)
        assert torch.equal(g8[0][:, h:h + 1].cpu(), q8) and torch.equal(g8[2][:, h:h + 1].cpu(), k8)
        assert torch.equal(g8[1][:, h:h + 1].cpu(), qs) and torch.equal(g8[3][:, h:h + 1].cpu(), ks)
        refs[h] = (q8[:, :, rows], k8, rv, torch.cat([qs[:, :, 2 * b:2 * b + 2] for b in blocks], dim=-1), ks)
    for density in (0.2, 1.0):
        mask = (synth.make_block_mask(H, nb, density, seed=46, device=dev) if density < 1
                else torch.ones(H, nb, nb, dtype=torch.bool, device=dev))
        o = torch.empty_like(qp)
        qattn.qk_int8_sv_f16_accum_f16_attn(g8[0], g8[2], vp, o, g8[1], g8[3], 1, 0, 2, D ** -0.5, 0, mask)
        assert torch.isfinite(o.float()).all()
        for h in heads:
            q8r, k8, rv, qs_sel, ks = refs[h]
            ref, _ = O.sparse_attention(q8r, k8, rv, qs_sel, ks, mask[None, h:h + 1][:, :, blocks].cpu(), D ** -0.5,
                                        out_dtype=torch.float32)
            got = o[:, h:h + 1][:, :, rows].cpu().float()
            err = (got - ref).abs().max().item()
            assert err <= ATOL, (density, h, err)
            assert cosine(got, ref) >= COS, (density, h, cosine(got, ref))


def test_cfg2_peaked_rows_fast_and_exact_exponential(dev, record_property):
    """Peaked rows at the CogVideoX shape (RoPE turns the per-channel K bias into rows that one to three
    keys dominate, outputs up to ~0.9 instead of ~0.05): what the default (fast) and the exact
    exponential each deliver there.  Measured: both keep cosine >= 0.999 (fast 0.99921, exact 0.99935)
    and both leave atol 2e-2 on a few 1e-5 of the elements (max |err| 0.05-0.09 on outputs of ~0.9: the
    6 % worst-case relative rounding of an e4m3 V entry or P weight that a dominating key carries); the
    fast path's share of that is the smaller one.  So on such rows neither FP8 path holds a FLAT atol 2e-2;
    the bound that holds for both is the general rule of conftest.assert_attention_close.  The accuracy mode
    (pv_f16=True: the float16 P.V product the reference's kernel computes) holds the flat atol 2e-2 on every
    element here, with a tenth of it to spare."""
    import paroatten_amd as P
    from paroatten_amd import permute as PM
    from paroatten_amd import rope
    wl = synth.WORKLOADS["cogvideox5b"]
    H, N, D, nb = 2, wl.N, wl.D, wl.nb
    q, k, v = synth.make_qkv(1, H, N, D, wl.dtype, seed=78)
    mask = synth.make_block_mask(H, nb, 0.3, seed=79)
    plan = synth.make_permute_plan(1, H, seed=80)
    cos, sin = rope.rope_table_cog(D, wl.grid)
    orders = PM.head_orders(plan, 0, dev)
    qp, kp, vp = PM.rope_permute(q.to(dev), k.to(dev), v.to(dev), orders, wl.grid, wl.n_text, cos.to(dev), sin.to(dev))
    ref = O.paro_path(q, k, v, mask[None], plan, 0, wl.grid, wl.n_text, cos, sin)
    a_ref = O.paro_path(q, k, v.abs(), mask[None], plan, 0, wl.grid, wl.n_text, cos, sin)
    assert ref.float().abs().max().item() > 0.5       # the rows are peaked: i.i.d. inputs give ~0.05
    res = {}
    for name, exact in (("fast", False), ("exact", True)):
        o = P.paroattn_qk_int8_pv_fp16_cuda(qp, kp, vp, mask.to(dev), smooth_k=True, exact_exp=exact)
        o = PM.permute_inverse(o.contiguous(), orders, wl.grid, wl.n_text).cpu()
        e = (o.float() - ref.float()).abs()
        res[name] = (e.max().item(), (e > ATOL).float().mean().item(), cosine(o, ref))
        record_property(f"{name}_max_abs_err", res[name][0])
        record_property(f"{name}_frac_above_atol", res[name][1])
        record_property(f"{name}_cosine", res[name][2])
        assert res[name][2] >= COS, (name, res[name])
        assert_attention_close(o, ref, a_ref, COS, what=name)
        assert res[name][1] <= 2e-4, (name, res[name])          # atol 2e-2 holds on all but ~1e-5..1e-4 of the elements
    assert res["exact"][2] >= res["fast"][2] - 1e-5              # the exact exponential is the (slightly) more accurate one
    o = P.paroattn_qk_int8_pv_fp16_cuda(qp, kp, vp, mask.to(dev), smooth_k=True, pv_f16=True)
    o = PM.permute_inverse(o.contiguous(), orders, wl.grid, wl.n_text).cpu()
    e16 = (o.float() - ref.float()).abs().max().item()
    record_property("pv_f16_max_abs_err", e16)
    record_property("pv_f16_cosine", cosine(o, ref))
    assert e16 <= 2e-3, e16                                      # flat, a tenth of the benchmark's atol
    assert cosine(o, ref) >= 0.99999
