"""paro_rope_k_mean_static: the rotated K mean through the library's built-in work buffer, for callers
that cannot allocate.  Called through the C ABI and compared bit for bit with paro_rope_k_mean (which
takes the caller's workspace), on two calls in a row, the second with a smaller input: the buffer is
shared by every call on the GPU and keeps what the previous call left in it."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(dev, B, H, D, grid, n_text, dtype, seed, with_rope):
    import paroatten_amd._lib as L
    from paroatten_amd import rope
    lib = L.load()
    N = n_text + grid[0] * grid[1] * grid[2]
    g = torch.Generator(device=dev).manual_seed(seed)
    k = (torch.randn(B, H, N, D, generator=g, device=dev) + 2.0 * torch.randn(1, H, 1, D, generator=g, device=dev)).to(dtype)
    cos = sin = None
    if with_rope:
        cos, sin = (t.to(dev) for t in rope.rope_table_cog(D, grid))
    n_chunks = (N + 255) // 256
    ws = torch.empty(B * H * n_chunks * D, dtype=torch.float32, device=dev)
    want = torch.full((B, H, 1, D), float("nan"), dtype=dtype, device=dev)
    got = torch.full((B, H, 1, D), float("nan"), dtype=dtype, device=dev)
    common = (B, H, N, D, n_text, grid[0], grid[1], grid[2], k.stride(0), k.stride(1), k.stride(2),
              want.stride(0), want.stride(1), L.stream_of(k))
    L.check(lib.paro_rope_k_mean(L.ptr(k), L.DTYPE_CODE[dtype], L.ptr(cos), L.ptr(sin), L.ptr(want), L.ptr(ws),
                                 ws.numel() * 4, *common))
    L.check(lib.paro_rope_k_mean_static(L.ptr(k), L.DTYPE_CODE[dtype], L.ptr(cos), L.ptr(sin), L.ptr(got), *common))
    torch.cuda.synchronize()
    assert torch.isfinite(want.float()).all()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    # and the mean is the mean (text rows unrotated, image rows rotated), to one ulp of the 16-bit type
    kr = k.float()
    if with_rope:
        x = kr[:, :, n_text:].reshape(B, H, -1, D // 2, 2)
        c, s_ = cos.reshape(1, 1, -1, D // 2, 2), sin.reshape(1, 1, -1, D // 2, 2)
        rot = torch.stack((x[..., 0] * c[..., 0] - x[..., 1] * s_[..., 0], x[..., 1] * c[..., 1] + x[..., 0] * s_[..., 1]), dim=-1)
        kr = torch.cat((kr[:, :, :n_text], rot.reshape(B, H, -1, D).to(dtype).float()), dim=2)
    ref = kr.mean(dim=2, keepdim=True)
    ulp = ref.abs().clamp_min(1e-3) * (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10)
    assert bool(((got.float() - ref).abs() <= ulp).all())


def test_static_scratch_entry_matches_workspace_entry_twice(dev):
    # the CogVideoX-5b shape (0.43 M partial sums of the 2 M the buffer holds), then a small ragged one
    _both(dev, 2, 48, 64, (13, 30, 45), 226, torch.float16, 1, True)
    _both(dev, 1, 3, 128, (3, 5, 7), 17, torch.bfloat16, 2, False)
    _both(dev, 1, 5, 64, (2, 3, 4), 0, torch.float16, 3, True)


def test_static_scratch_entry_rejects_what_does_not_fit(dev):
    import paroatten_amd._lib as L
    lib = L.load()
    p = ctypes.c_void_p(256)   # never dereferenced: the size check comes first
    # B*H*ceil(N/256)*D = 64*64*40*128 = 20 971 520 floats > 2 097 152
    rc = lib.paro_rope_k_mean_static(p, 0, None, None, p, 64, 64, 10240, 128, 0, 10, 32, 32,
                                     64 * 10240 * 128, 10240 * 128, 128, 64 * 128, 128, None)
    assert rc == L.PARO_ERR_RUNTIME and b"exceed the built-in work buffer" in lib.paro_last_error()
    assert lib.paro_rope_k_mean_static(p, 0, None, None, p, 1, 1, 64, 96, 0, 4, 4, 4, 64 * 96, 64 * 96, 96, 96, 96,
                                       None) == L.PARO_ERR_INVALID_VALUE
