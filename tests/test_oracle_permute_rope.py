"""Pins the permutation index law, the reshape/permute restatements and the RoPE functions of the
oracle against torch library routines, the reference's literal tables and mathematical identities."""
import itertools

import pytest
import torch

from oracle import paro_oracle as O


def test_literal_tables_match_reference_source():
    # paroattention/cogvideox.py:38-45 and :85-92, held as literals here
    assert O.PERMUTATIONS == ((0, 1, 2), (0, 2, 1), (1, 2, 0), (1, 0, 2), (2, 1, 0), (2, 0, 1))
    assert O.PERMUTATIONS_INV == ((0, 1, 2), (0, 2, 1), (2, 0, 1), (1, 0, 2), (2, 1, 0), (1, 2, 0))
    # the inverse table really holds the inverse orders, and all six orders are distinct
    for p, pinv in zip(O.PERMUTATIONS, O.PERMUTATIONS_INV):
        assert tuple(p[i] for i in pinv) == (0, 1, 2)
    assert set(O.PERMUTATIONS) == set(itertools.permutations(range(3)))


@pytest.mark.parametrize("grid", [(2, 3, 5), (3, 3, 3), (13, 30, 45), (21, 30, 52)])
def test_index_law_equals_torch_permute(grid):
    F, H, W = grid
    n = F * H * W
    ar = torch.arange(n).reshape(F, H, W)
    for oid, p in enumerate(O.PERMUTATIONS):
        new_of_old = O.permute_index_map(grid, oid)
        old_of_new = ar.permute(*p).reshape(-1)  # library routine: out[new] = in[old_of_new[new]]
        assert torch.equal(new_of_old[old_of_new], torch.arange(n))
        assert sorted(new_of_old.tolist()) == list(range(n))  # a bijection


def test_permute_qk_gather_form_and_inverse():
    grid, n_text, B, H, D = (3, 4, 5), 7, 2, 6, 8
    n_img = 60
    g = torch.Generator().manual_seed(0)
    q = torch.randn(B, H, n_text + n_img, D, generator=g)
    k, v = q + 1, q + 2
    plan = {"permute": torch.tensor([[0, 1, 2, 3, 4, 5]]), "empty": torch.zeros(1, 6, dtype=torch.bool)}
    pq, pk, pv = O.permute_qk(q, k, v, plan, 0, grid, n_text)
    for h in range(H):
        m = O.permute_index_map(grid, h)
        exp = torch.empty_like(q[:, h, n_text:])
        exp[:, m] = q[:, h, n_text:]  # out[new] = in[old]
        assert torch.equal(pq[:, h, n_text:], exp)
        assert torch.equal(pq[:, h, :n_text], q[:, h, :n_text])  # text tokens are fixed points
    assert torch.equal(pk, pq + 1) and torch.equal(pv, pq + 2)
    assert torch.equal(O.permute_attn_out(pq, plan, 0, grid, n_text), q)  # inverse o forward = id
    assert not q.data_ptr() == pq.data_ptr() and torch.equal(k, q + 1)  # inputs untouched


def test_rope_is_a_rotation():
    g = torch.Generator().manual_seed(1)
    D, grid = 64, (2, 3, 4)
    x = torch.randn(1, 2, 24, D, generator=g, dtype=torch.float64)
    cos, sin = O.rope_table_cog(D, grid)
    y = O.rope_apply_cog(x, cos.double(), sin.double())
    # norm of every channel pair is preserved; position (0,0,0) is the identity
    assert torch.allclose(y.reshape(1, 2, 24, -1, 2).norm(dim=-1), x.reshape(1, 2, 24, -1, 2).norm(dim=-1))
    assert torch.allclose(y[:, :, 0], x[:, :, 0])
    # agrees with the complex form: (x0 + i x1) * exp(i theta)
    ang = torch.atan2(sin.double(), cos.double())[:, 0::2]
    yc = torch.view_as_real(torch.view_as_complex(x.reshape(1, 2, 24, -1, 2).contiguous()) * torch.polar(torch.ones_like(ang), ang)).flatten(-2)
    assert torch.allclose(y, yc)


def test_rope_cog_table_closed_form():
    """The CogVideoX rotary TABLE (the pair the reference consumes at cogvideox.py:167-172) in the
    documented get_3d_rotary_pos_embed convention, checked against closed forms evaluated here in
    Python floats: a wrong t/h/w split, concatenated instead of interleaved pairs, or an exponent
    over D instead of over the group's own dimension each fail it."""
    import math

    D, grid, theta = 64, (13, 30, 45), 10000.0
    F, Hh, W = grid
    cos, sin = O.rope_table_cog(D, grid, theta)
    assert cos.shape == sin.shape == (F * Hh * W, D) and cos.dtype == sin.dtype == torch.float32
    assert torch.allclose(cos.double() ** 2 + sin.double() ** 2, torch.ones(F * Hh * W, D, dtype=torch.float64), atol=1e-6)
    c3, s3 = cos.reshape(F, Hh, W, D), sin.reshape(F, Hh, W, D)
    # channel groups 16 / 24 / 24 (t / h / w = D/4, 3D/8, 3D/8); each depends on ONE grid axis only
    groups = ((0, 16, 0, F), (16, 40, 1, Hh), (40, 64, 2, W))
    for lo, hi, axis, _ in groups:
        for other in ((1, 7, 11), (12, 29, 44), (5, 0, 31)):
            for pos in (0, 1, 5):
                a = [other[0], other[1], other[2]]
                b = [0, 0, 0]
                a[axis] = b[axis] = pos
                assert torch.equal(c3[a[0], a[1], a[2], lo:hi], c3[b[0], b[1], b[2], lo:hi])
                assert torch.equal(s3[a[0], a[1], a[2], lo:hi], s3[b[0], b[1], b[2], lo:hi])
    # inside a group of dim_g channels: angle[pos, 2i] = angle[pos, 2i+1] = pos * theta^(-2i/dim_g)
    for lo, hi, axis, length in groups:
        dim_g = hi - lo
        for pos in (1, 2, 7, length - 1):
            idx = [0, 0, 0]
            idx[axis] = pos
            for i in (0, 1, 2, dim_g // 2 - 1):
                ang = pos * theta ** (-2.0 * i / dim_g)
                for ch in (lo + 2 * i, lo + 2 * i + 1):      # interleaved: the pair shares its frequency
                    assert float(c3[idx[0], idx[1], idx[2], ch]) == pytest.approx(math.cos(ang), abs=2e-7)
                    assert float(s3[idx[0], idx[1], idx[2], ch]) == pytest.approx(math.sin(ang), abs=2e-7)
        # first frequency of each group is theta^0 = 1 rad per position; the second is NOT (rules out a
        # concatenated [f0, f1, ..., f0, f1, ...] layout, where channel lo + 1 would hold f1's neighbour f0 ... )
        one = [0, 0, 0]
        one[axis] = 1
        assert float(s3[one[0], one[1], one[2], lo]) == pytest.approx(math.sin(1.0), abs=2e-7)
        assert float(s3[one[0], one[1], one[2], lo + 1]) == pytest.approx(math.sin(1.0), abs=2e-7)
        assert float(s3[one[0], one[1], one[2], lo + 2]) == pytest.approx(math.sin(theta ** (-2.0 / dim_g)), abs=2e-7)
        # ... and an exponent over D (64) instead of dim_g would put theta^(-2/64) there
        assert abs(float(s3[one[0], one[1], one[2], lo + 2]) - math.sin(theta ** (-2.0 / D))) > 1e-2
    # the last channel of the t group and the first of the h group belong to different axes
    assert float(s3[1, 0, 0, 16]) == 0.0 and float(s3[0, 1, 0, 15]) == 0.0 and float(s3[0, 1, 0, 16]) == pytest.approx(math.sin(1.0), abs=2e-7)
    assert float(s3[0, 0, 1, 39]) == 0.0 and float(s3[0, 0, 1, 40]) == pytest.approx(math.sin(1.0), abs=2e-7)


def test_rope_cog_table_of_the_package_is_the_oracles():
    """paroatten_amd.rope.rope_table_cog is independent code (one concatenation, then one
    repeat_interleave, float64 angles): bit for bit the oracle's table at the CogVideoX-5b grid."""
    from paroatten_amd.rope import rope_table_cog

    for D, grid in ((64, (13, 30, 45)), (128, (3, 4, 5))):
        co, so = O.rope_table_cog(D, grid)
        cp, sp = rope_table_cog(D, grid)
        assert torch.equal(co, cp) and torch.equal(so, sp)


def test_rope_wan_composition_and_split():
    D, grid = 128, (3, 4, 5)
    f = O.rope_table_wan(D, grid)
    assert f.shape == (1, 1, 60, 64) and f.dtype == torch.complex128
    assert torch.allclose(f.abs(), torch.ones(1, 1, 60, 64, dtype=torch.float64))
    ang = torch.angle(f[0, 0]).reshape(3, 4, 5, 64)
    # channel split 22 / 21 / 21 complex pairs (44/42/42 channels): each group depends on one axis only
    assert torch.allclose(ang[:, 0, 0, :22], ang[:, 2, 3, :22]) and torch.allclose(ang[0, :, 0, 22:43], ang[1, :, 4, 22:43])
    assert torch.allclose(ang[0, 0, :, 43:], ang[2, 3, :, 43:])
    # first frequency of each group is theta^0 = 1 rad per position: R(a)R(b) = R(a+b)
    assert torch.allclose(f[0, 0].reshape(3, 4, 5, 64)[2, 0, 0, 0], f[0, 0].reshape(3, 4, 5, 64)[1, 0, 0, 0] ** 2)
    assert float(ang[1, 0, 0, 0]) == pytest.approx(1.0) and float(ang[0, 1, 0, 22]) == pytest.approx(1.0)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(1, 2, 60, D, generator=g).bfloat16()
    y = O.rope_apply_wan(x, f)
    assert y.dtype == torch.bfloat16
    assert torch.allclose(y.float().reshape(1, 2, 60, -1, 2).norm(dim=-1), x.float().reshape(1, 2, 60, -1, 2).norm(dim=-1), rtol=2e-2, atol=1e-2)


def test_per_channel_fp8_against_library_cast():
    g = torch.Generator().manual_seed(3)
    v = (torch.randn(1, 2, 100, 64, generator=g) + 0.5).half()
    v8, sc, vm = O.per_channel_fp8(v)
    assert v8.dtype == torch.float8_e4m3fn and sc.shape == (1, 2, 64) and vm.shape == (1, 2, 64)
    assert torch.allclose(vm, v.float().mean(dim=2))
    centred = v.float() - vm.unsqueeze(2)
    assert torch.allclose(sc * 448, centred.abs().amax(dim=2))
    deq = v8.float() * sc.unsqueeze(2)
    rel = (deq - centred).abs() / centred.abs().clamp_min(1e-3)
    assert float(rel.max()) <= 0.0625 + 1e-3 or float(((deq - centred).abs()).max()) < 2e-2  # 3 mantissa bits
    assert float(v8.float().abs().max()) == 448.0


def test_transpose_pad_permute_order_is_stated_twice_by_the_reference():
    """the kernel's formula (fused.cu:287-291) and the docstring's literal list (quant.py:231-234) agree,
    and the oracle is torch.transpose + pad with that order"""
    for r in range(16):
        assert O.V_SHUFFLE16[O.shuffle16_position_of(r)] == r
    assert sorted(O.V_SHUFFLE16) == list(range(16))
    g = torch.Generator().manual_seed(0)
    v = torch.randn(2, 3, 100, 64, generator=g).to(torch.float16)
    out = O.transpose_pad_permute(v)
    assert out.shape == (2, 3, 64, 128) and (out[..., 112:] == 0).all()
    for n in (0, 1, 2, 8, 17, 50, 99):
        pos = (n // 16) * 16 + O.shuffle16_position_of(n % 16)
        assert torch.equal(out[..., pos], v[:, :, n, :])
    # tokens 100..111 share a group of 16 with real tokens: zero, at their shuffled positions
    assert (out[..., [96 + O.shuffle16_position_of(r) for r in range(4, 16)]] == 0).all()


def test_channel_quant_fp8_reduces_to_per_channel_fp8_and_keeps_the_quirk():
    g = torch.Generator().manual_seed(1)
    v = (torch.randn(1, 2, 128, 64, generator=g) + 0.7).to(torch.bfloat16)
    x = v.transpose(2, 3).contiguous()
    codes, sc, mean = O.channel_quant_fp8(x, 128)
    v8, vs, vm = O.per_channel_fp8(v)            # pinned by its own tests
    assert torch.allclose(mean, vm, atol=1e-6) and torch.allclose(sc, vs, rtol=1e-5)
    same = (codes.view(torch.uint8) == v8.transpose(2, 3).view(torch.uint8)).float().mean()
    assert same >= 0.999                          # a last-bit difference of the mean flips a tie here and there
    # 100 real tokens in rows padded to 128: statistics over the first 112, mean divides by 112
    xp = x.clone()
    xp[..., 100:] = 0
    codes, sc, mean = O.channel_quant_fp8(xp, 100)
    assert codes.shape[-1] == 128
    assert torch.allclose(mean, xp[..., :100].float().sum(-1) / 112, atol=1e-6)
    cen = xp[..., :112].float() - mean[..., None]
    assert torch.allclose(sc, cen.abs().amax(-1) / 448.0, rtol=1e-6)
    deq = codes.float() * sc[..., None] + mean[..., None]
    assert ((deq - xp.float()).abs() <= sc[..., None] * 16.0 + 1e-6).all()     # half the widest e4m3 cell
    assert (codes.float().abs().amax(-1) == 448.0).all()                          # the extreme maps to +-448
    # without the mean: symmetric scale, zeros stay zero codes
    codes, sc, none = O.channel_quant_fp8(xp, 100, sub_mean=False)
    assert none is None and torch.allclose(sc, xp[..., :112].float().abs().amax(-1) / 448.0, rtol=1e-6)
    assert (codes[..., 100:].float() == 0).all()
    # a constant row gives zero codes, not NaN
    codes, sc, mean = O.channel_quant_fp8(torch.full((1, 1, 2, 64), 3.0, dtype=torch.float16), 64)
    assert (codes.float() == 0).all() and (sc == 0).all() and torch.allclose(mean, torch.full((1, 1, 2), 3.0))
