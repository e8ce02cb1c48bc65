"""GPU parity of the fused RoPE + permutation kernels against the oracle: bit-exact index maps,
bit-exact permutation of values, rotation bit-exact against the fp32 formula (Cog form) and within
1 ulp of the output dtype against the float64 complex form (Wan)."""
import pytest
import torch

from oracle import paro_oracle as O
from paroatten_amd import synth

pytestmark = pytest.mark.gpu


def _ulp_diff(a: torch.Tensor, b: torch.Tensor) -> int:
    """max distance in representable 16-bit values (monotone integer encoding)."""
    def key(t):
        i = t.view(torch.int16).to(torch.int32)
        return torch.where(i < 0, -(i & 0x7FFF), i)
    return int((key(a) - key(b)).abs().max())


@pytest.mark.parametrize("grid", [(2, 3, 5), (4, 4, 4), (13, 30, 45), (21, 30, 52)])
def test_index_map_bitexact(dev, grid):
    from paroatten_amd.permute import permute_index_map
    orders = torch.arange(6, dtype=torch.int32)
    idx = permute_index_map(orders.to(dev), grid).cpu()
    for o in range(6):
        assert torch.equal(idx[o].long(), O.permute_index_map(grid, o))


@pytest.mark.parametrize("dtype,D,grid,n_text,B,H", [
    (torch.bfloat16, 64, (3, 5, 7), 11, 2, 6),
    (torch.float16, 128, (4, 6, 5), 0, 1, 7),
    (torch.bfloat16, 64, (13, 30, 45), 226, 1, 3),
])
def test_rope_permute_cog_and_inverse(dev, dtype, D, grid, n_text, B, H):
    from paroatten_amd import permute as PM
    n_img = grid[0] * grid[1] * grid[2]
    N = n_text + n_img
    q, k, v = synth.make_qkv(B, H, N, D, dtype, seed=N)
    plan = synth.make_permute_plan(2, H, seed=N + 1)
    plan["permute"][1, : min(H, 6)] = torch.arange(min(H, 6))  # every order appears
    cos, sin = O.rope_table_cog(D, grid)
    qr, kr = q.clone(), k.clone()
    qr[:, :, n_text:] = O.rope_apply_cog(q[:, :, n_text:], cos, sin)
    kr[:, :, n_text:] = O.rope_apply_cog(k[:, :, n_text:], cos, sin)
    rq, rk, rv = O.permute_qk(qr, kr, v, plan, 1, grid, n_text)
    orders = PM.head_orders(plan, 1, dev)
    gq, gk, gv = PM.rope_permute(q.to(dev), k.to(dev), v.to(dev), orders, grid, n_text, cos.to(dev), sin.to(dev))
    assert torch.equal(gv.cpu(), rv)  # pure data movement
    assert torch.equal(gq.cpu(), rq)  # fp32 products and sum rounded as torch does
    assert torch.equal(gk.cpu(), rk)
    # permutation only
    pq, pk, pv = PM.rope_permute(q.to(dev), None, v.to(dev), orders, grid, n_text)
    oq, _, _ = O.permute_qk(q, k, v, plan, 1, grid, n_text)
    assert pk is None and torch.equal(pq.cpu(), oq) and torch.equal(pv.cpu(), rv)
    # inverse
    back = PM.permute_inverse(gv, orders, grid, n_text)
    assert torch.equal(back.cpu(), v)
    assert torch.equal(PM.permute_inverse(gq, orders, grid, n_text).cpu(), O.permute_attn_out(rq, plan, 1, grid, n_text))
    # in-place drop-ins
    q2, k2, v2 = q.to(dev).clone(), k.to(dev).clone(), v.to(dev).clone()
    PM.permute_qk(q2, k2, v2, plan, 1, grid, n_text)
    assert torch.equal(q2.cpu(), oq) and torch.equal(v2.cpu(), rv)
    PM.permute_attn_out(v2, plan, 1, grid, n_text)
    assert torch.equal(v2.cpu(), v)


def test_rope_wan_within_one_ulp(dev):
    from paroatten_amd import permute as PM
    D, grid, B, H = 128, (3, 6, 8), 1, 5
    N = grid[0] * grid[1] * grid[2]
    q, k, v = synth.make_qkv(B, H, N, D, torch.bfloat16, seed=77)
    freqs = O.rope_table_wan(D, grid)
    rq = O.rope_apply_wan(q, freqs)
    ang = torch.angle(freqs[0, 0])
    cos = ang.cos().float().repeat_interleave(2, dim=1).contiguous()
    sin = ang.sin().float().repeat_interleave(2, dim=1).contiguous()
    orders = torch.zeros(H, dtype=torch.int32, device=dev)
    gq, _, _ = PM.rope_permute(q.to(dev), None, None, orders, grid, 0, cos.to(dev), sin.to(dev))
    assert _ulp_diff(gq.cpu(), rq) <= 1


def test_rope_prototype_module(dev):
    """_rope.rope_permutation: token-independent (cos, sin) pairs, optional (H,W) transpose."""
    from paroatten_amd import _rope
    bs, H, W, dim = 2, 5, 7, 256
    g = torch.Generator().manual_seed(5)
    Q = (torch.randn(bs, H, W, dim, generator=g) * 0.5).half()
    K = (torch.randn(bs, H, W, dim, generator=g) * 0.5).half()
    freq = torch.randn(128, generator=g) * 0.5
    c = freq.view(64, 2)[:, 0].repeat(dim // 128)
    s = freq.view(64, 2)[:, 1].repeat(dim // 128)

    def ref(x):
        xr, xi = x.float().reshape(bs, H, W, dim // 2, 2).unbind(-1)
        return torch.stack([c * xr - s * xi, c * xi + s * xr], dim=-1).flatten(-2).half()

    for perm in (False, True):
        QO, KO = _rope.rope_permutation(Q.to(dev), K.to(dev), freq.to(dev), perm)
        rq, rk = ref(Q), ref(K)
        if perm:
            rq, rk = rq.transpose(1, 2), rk.transpose(1, 2)
        assert _ulp_diff(QO.cpu(), rq.reshape(bs, H * W, dim).contiguous()) <= 1
        assert _ulp_diff(KO.cpu(), rk.reshape(bs, H * W, dim).contiguous()) <= 1


def test_out_of_range_order_on_device_is_identity(dev):
    """the order table lives on the device, so the C ABI cannot validate it: a value outside 0..5 is
    treated as order 0 (no out-of-bounds index can be formed from it) by every kernel that reads it."""
    from paroatten_amd import permute as PM
    grid, n_text, D = (2, 3, 4), 8, 64
    N = n_text + 24
    g = torch.Generator().manual_seed(0)
    x = torch.randn(1, 2, N, D, generator=g).to(dev, torch.float16)
    bad = torch.tensor([9, -3], dtype=torch.int32, device=dev)
    zero = torch.zeros(2, dtype=torch.int32, device=dev)
    assert torch.equal(PM.permute_index_map(bad, grid), PM.permute_index_map(zero, grid))
    _, _, v_bad = PM.rope_permute(None, None, x, bad, grid, n_text)
    assert torch.equal(v_bad, x)
    assert torch.equal(PM.permute_inverse(x, bad, grid, n_text), x)
    a, b = PM.rope_permute_quant(x, x, x, bad, grid, n_text), PM.rope_permute_quant(x, x, x, zero, grid, n_text)
    assert torch.equal(a.q8, b.q8) and torch.equal(a.k_scale, b.k_scale) and torch.equal(a.v8, b.v8)
