"""GPU parity of the INT8 quantisation kernel (through the C ABI) against the oracle: bit-exact
int8 tensors and fp32 scales."""
import pytest
import torch

from oracle import paro_oracle as O
from paroatten_amd import synth

pytestmark = pytest.mark.gpu


def _q():
    import paroatten_amd.quant as Q
    return Q


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D,N", [(64, 4096), (64, 1000), (128, 2072), (64, 65), (128, 31)])
def test_per_warp_int8_bitexact(dev, dtype, D, N):
    q, k, v = synth.make_qkv(2, 3, N, D, dtype, seed=N + D)
    km = k.float().mean(dim=2, keepdim=True).to(dtype)
    for kmean in (None, km):
        rq8, rqs, rk8, rks = O.per_warp_int8(q, k, km=kmean, BLKQ=64, WARPQ=32, BLKK=64)
        q8, qs, k8, ks = _q().per_warp_int8(q.to(dev), k.to(dev), None if kmean is None else kmean.to(dev),
                                            BLKQ=64, WARPQ=32, BLKK=64)
        assert qs.shape == rqs.shape and ks.shape == rks.shape
        assert torch.equal(q8.cpu(), rq8)
        assert torch.equal(k8.cpu(), rk8)
        assert torch.equal(qs.cpu(), rqs)
        assert torch.equal(ks.cpu(), rks)


@pytest.mark.parametrize("BLKQ,BLKK", [(128, 64), (64, 128), (128, 128)])
def test_per_block_int8_bitexact(dev, BLKQ, BLKK):
    q, k, v = synth.make_qkv(1, 2, 777, 64, torch.float16, seed=5)
    km = k.float().mean(dim=2, keepdim=True).to(k.dtype)
    r = O.per_block_int8(q, k, km=km, BLKQ=BLKQ, BLKK=BLKK, sm_scale=0.11)
    g = _q().per_block_int8(q.to(dev), k.to(dev), km.to(dev), BLKQ=BLKQ, BLKK=BLKK, sm_scale=0.11)
    for a, b in zip(g, r):
        assert torch.equal(a.cpu(), b)


def test_per_warp_int8_warp16_and_nhd(dev):
    q, k, v = synth.make_qkv(2, 4, 300, 128, torch.bfloat16, seed=9)
    rq8, rqs, rk8, rks = O.per_warp_int8(q, k, BLKQ=128, WARPQ=16, BLKK=64)
    # NHD: [B,N,H,D]
    qn, kn = q.transpose(1, 2).contiguous().to(dev), k.transpose(1, 2).contiguous().to(dev)
    q8, qs, k8, ks = _q().per_warp_int8(qn, kn, BLKQ=128, WARPQ=16, BLKK=64, tensor_layout="NHD")
    assert torch.equal(q8.transpose(1, 2).cpu(), rq8)
    assert torch.equal(k8.transpose(1, 2).cpu(), rk8)
    assert torch.equal(qs.cpu(), rqs) and torch.equal(ks.cpu(), rks)


def test_known_answer_rows(dev):
    """bench/test.py:5-14 of the reference: rows -256..255 repeated over 64 channels (bf16)."""
    rows = torch.arange(-256, 256, dtype=torch.bfloat16).unsqueeze(1)
    q = rows.repeat(1, 64)[None, None]
    q8, qs, k8, ks = _q().per_warp_int8(q.to(dev), q.to(dev), BLKQ=64, WARPQ=32, BLKK=64)
    for g in range(16):
        lo, hi = -256 + 32 * g, -225 + 32 * g
        amax = max(abs(lo), abs(hi))
        assert abs(float(qs[0, 0, g]) - amax / 127.0) <= 1e-6 * amax
        vals = torch.arange(lo, hi + 1, dtype=torch.float32)
        exp = torch.round(vals * (torch.tensor(127.0) / torch.tensor(float(amax)))).to(torch.int8)
        assert torch.equal(q8[0, 0, 32 * g:32 * g + 32, 0].cpu(), exp)


def test_sub_mean(dev):
    q, k, v = synth.make_qkv(1, 2, 130, 64, torch.bfloat16, seed=3)
    vs, vm = _q().sub_mean(v.to(dev))
    ref_vm = v.to(dev).mean(dim=2)
    ref = (v.to(dev) - ref_vm.unsqueeze(2)).to(torch.float16)  # bf16 subtraction, then fp16
    assert torch.equal(vs, ref)


@pytest.mark.parametrize("layout,D,N,dtype", [("HND", 64, 200, torch.float16), ("NHD", 128, 333, torch.bfloat16),
                                              ("HND", 128, 64, torch.float16), ("HND", 64, 17776, torch.bfloat16)])
def test_reference_format_v_preparation(dev, layout, D, N, dtype):
    """transpose_pad_permute_cuda, mean_scale_fuse_quant_cuda and scale_fuse_quant_cuda of
    paroattention._fused (csrc/fused/pybind.cpp:29-33) against the oracle: the transposed, padded and
    reordered tensor bit for bit; scales and means to fp32 summation order; codes equal except where the
    mean's last bit moves a value across a rounding boundary."""
    from paroatten_amd import _fused
    B, H = 2, 3
    g = torch.Generator().manual_seed(N + D)
    v = (torch.randn(B, H, N, D, generator=g) * 1.5 + torch.randn(1, H, 1, D, generator=g)).to(dtype)
    want_t = O.transpose_pad_permute(v)                               # [B,H,D,padded]
    padded = want_t.shape[-1]
    vd = v.to(dev)
    flag = 1
    if layout == "NHD":
        vd = vd.transpose(1, 2).contiguous()                          # [B,N,H,D]
        flag = 0
        out = torch.full((B, D, H, padded), float("nan"), dtype=dtype, device=dev)
    else:
        out = torch.full((B, H, D, padded), float("nan"), dtype=dtype, device=dev)
    _fused.transpose_pad_permute_cuda(vd, out, flag)
    got_t = out.transpose(1, 2) if layout == "NHD" else out
    assert torch.equal(got_t.cpu().view(torch.int16), want_t.view(torch.int16))
    for smooth in (True, False):
        codes = torch.zeros(out.shape, dtype=torch.float8_e4m3fn, device=dev)
        scale = torch.empty(B, H, D, dtype=torch.float32, device=dev)
        mean = torch.empty(B, H, D, dtype=torch.float32, device=dev)
        if smooth:
            _fused.mean_scale_fuse_quant_cuda(out, codes, mean, scale, N, 448.0, flag)
        else:
            _fused.scale_fuse_quant_cuda(out, codes, scale, N, 448.0, flag)
        wc, ws, wm = O.channel_quant_fp8(want_t, N, sub_mean=smooth)
        gc = (codes.transpose(1, 2) if layout == "NHD" else codes).cpu().view(torch.uint8)
        assert torch.allclose(scale.cpu(), ws, rtol=2e-6, atol=0)
        if smooth:
            assert torch.allclose(mean.cpu(), wm, rtol=1e-5, atol=1e-6)
        diff = (gc.int() - wc.view(torch.uint8).int()).abs()
        assert int(diff.max()) <= 1 and float((diff != 0).float().mean()) <= (1e-3 if smooth else 0.0)


def test_per_channel_fp8_reference_order(dev):
    """quant.per_channel_fp8(tile_order=False) = the reference's own sequence of the three calls
    (paroattention/quant.py:266-293)"""
    g = torch.Generator().manual_seed(9)
    v = torch.randn(1, 2, 150, 64, generator=g).to(torch.float16)
    v8, vs, vm = _q().per_channel_fp8(v.to(dev), tile_order=False)
    assert v8.shape == (1, 2, 64, 192) and v8.dtype == torch.float8_e4m3fn
    wc, ws, wm = O.channel_quant_fp8(O.transpose_pad_permute(v), 150)
    assert torch.allclose(vs.cpu(), ws, rtol=2e-6) and torch.allclose(vm.cpu(), wm, rtol=1e-5, atol=1e-6)
    diff = (v8.cpu().view(torch.uint8).int() - wc.view(torch.uint8).int()).abs()
    assert int(diff.max()) <= 1 and float((diff != 0).float().mean()) <= 1e-3
    v8n, vsn, none = _q().per_channel_fp8(v.to(dev), smooth_v=False, tile_order=False, scale_max=224.0)
    assert none is None and torch.allclose(vsn.cpu(), v.float().abs().amax(dim=2) / 224.0, rtol=2e-6)
