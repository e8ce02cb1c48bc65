"""tests/golden/path_small.npz (written by tests/golden/make_fixtures.py): the oracle must still
reproduce it (CPU), and the HIP path must match it (GPU): bit-exact for indices, INT8, scales, int32
scores, 16-bit RoPE results and FP8 bytes; within the stated tolerance for the attention output."""
import os

import numpy as np
import pytest
import torch

from conftest import assert_attention_close, cosine, untile_v8, v8_offset_expected
from oracle import paro_oracle as O

FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "path_small.npz")
DTYPE = torch.float16


@pytest.fixture(scope="module")
def fx():
    with np.load(FIX, allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def _f16(a):
    return torch.from_numpy(a.view(np.int16).copy()).view(DTYPE)


def _plan(fx):
    return {"permute": torch.from_numpy(fx["permute"]), "empty": torch.zeros(fx["permute"].shape, dtype=torch.bool)}


def test_oracle_reproduces_the_fixture(fx):
    grid, n_text = tuple(int(x) for x in fx["grid"]), int(fx["n_text"])
    q, k, v = _f16(fx["q"]), _f16(fx["k"]), _f16(fx["v"])
    cos, sin = torch.from_numpy(fx["cos"]), torch.from_numpy(fx["sin"])
    plan = _plan(fx)
    D = q.shape[-1]
    c2, s2 = O.rope_table_cog(D, grid)
    assert torch.equal(c2, cos) and torch.equal(s2, sin)
    qr, kr = q.clone(), k.clone()
    qr[:, :, n_text:] = O.rope_apply_cog(q[:, :, n_text:], cos, sin)
    kr[:, :, n_text:] = O.rope_apply_cog(k[:, :, n_text:], cos, sin)
    assert torch.equal(qr, _f16(fx["q_rope"])) and torch.equal(kr, _f16(fx["k_rope"]))
    qp, kp, vp = O.permute_qk(qr, kr, v, plan, 0, grid, n_text)
    assert torch.equal(qp, _f16(fx["q_perm"])) and torch.equal(kp, _f16(fx["k_perm"])) and torch.equal(vp, _f16(fx["v_perm"]))
    for h in range(q.shape[1]):
        assert np.array_equal(O.permute_index_map(grid, int(fx["permute"][0, h])).numpy(), fx["index_map"][h])
    km = _f16(fx["km"])
    assert torch.equal(kp.float().mean(dim=2, keepdim=True).to(DTYPE), km)
    q8, qs, k8, ks = O.per_warp_int8(qp, kp, km=km, BLKQ=64, WARPQ=32, BLKK=64)
    assert np.array_equal(q8.numpy(), fx["q8"]) and np.array_equal(k8.numpy(), fx["k8"])
    assert np.array_equal(qs.numpy(), fx["q_scale"]) and np.array_equal(ks.numpy(), fx["k_scale"])
    assert np.array_equal(O.qk_int32(q8, k8)[0, 0].numpy().astype(np.int32), fx["s_int32_head0"])
    v8, vsc, vm = O.per_channel_fp8(vp)
    assert np.array_equal(v8.view(torch.uint8).numpy(), fx["v8"])
    assert np.array_equal(vsc.numpy(), fx["v_scale"]) and np.array_equal(vm.numpy(), fx["v_mean"])
    o, lse = O.sparse_attention(q8, k8, vp, qs, ks, torch.from_numpy(fx["mask"])[None], D ** -0.5,
                                out_dtype=torch.float32, compute_dtype=torch.float64)
    assert np.allclose(o.numpy(), fx["o_perm"], atol=1e-6, rtol=1e-6)
    assert np.allclose(lse.numpy(), fx["lse_base2"], atol=1e-5, rtol=1e-6)
    assert np.allclose(O.permute_attn_out(o, plan, 0, grid, n_text).numpy(), fx["o"], atol=1e-6, rtol=1e-6)


def test_fixture_internal_consistency(fx):
    """what the file must satisfy whoever wrote it: the permuted tensors are the rotated ones at the
    mapped positions, |q8| <= 127 with a +-127 in every group, scores = integer products."""
    n_text = int(fx["n_text"])
    qr, qp = fx["q_rope"], fx["q_perm"]
    for h in range(qr.shape[1]):
        idx = fx["index_map"][h]
        assert np.array_equal(qp[0, h, n_text:][idx], qr[0, h, n_text:])
        assert np.array_equal(qp[0, h, :n_text], qr[0, h, :n_text])
        assert sorted(idx.tolist()) == list(range(len(idx)))
    q8 = fx["q8"].astype(np.int32)
    assert np.abs(q8).max() <= 127
    N = q8.shape[2]
    for g in range((N + 31) // 32):
        assert np.abs(q8[0, 0, 32 * g:32 * g + 32]).max() == 127
    s = q8[0, 0].astype(np.int64) @ fx["k8"][0, 0].astype(np.int64).T
    assert np.array_equal(s, fx["s_int32_head0"].astype(np.int64))


@pytest.mark.gpu
def test_hip_path_matches_the_fixture(fx, dev):
    import paroatten_amd._lib as L
    from paroatten_amd import _qattn_sm80 as qattn
    from paroatten_amd import permute as PM
    from paroatten_amd import quant as Q
    grid, n_text = tuple(int(x) for x in fx["grid"]), int(fx["n_text"])
    q, k, v = (_f16(fx[n]).to(dev) for n in ("q", "k", "v"))
    cos, sin = torch.from_numpy(fx["cos"]).to(dev), torch.from_numpy(fx["sin"]).to(dev)
    plan = _plan(fx)
    B, H, N, D = q.shape
    orders = PM.head_orders(plan, 0, dev)
    assert np.array_equal(PM.permute_index_map(orders, grid).cpu().numpy(), fx["index_map"])
    qp, kp, vp = PM.rope_permute(q, k, v, orders, grid, n_text, cos, sin)
    assert torch.equal(qp.cpu(), _f16(fx["q_perm"])) and torch.equal(kp.cpu(), _f16(fx["k_perm"]))
    assert torch.equal(vp.cpu(), _f16(fx["v_perm"]))
    km = _f16(fx["km"]).to(dev)
    q8, qs, k8, ks = Q.per_warp_int8(qp, kp, km, BLKQ=64, WARPQ=32, BLKK=64)
    for got, name in ((q8, "q8"), (qs, "q_scale"), (k8, "k8"), (ks, "k_scale")):
        assert np.array_equal(got.cpu().numpy(), fx[name]), name
    # the one-pass preparation gives the same INT8 tensors straight from q, k, v
    ops = PM.rope_permute_quant(q, k, v, orders, grid, n_text, cos, sin, km=km)
    for got, name in ((ops.q8, "q8"), (ops.q_scale, "q_scale"), (ops.k8, "k8"), (ops.k_scale, "k_scale")):
        assert np.array_equal(got.cpu().numpy(), fx[name]), "fused " + name
    # FP8 V: scale bit-exact, mean to fp32 summation order, bytes (un-tiled) equal except where the
    # mean's last bit moves a value across a rounding boundary
    v8, vsc, vm = Q.per_channel_fp8(vp)
    assert np.array_equal(vsc.cpu().numpy(), fx["v_scale"])
    tok = untile_v8(v8, B, H, N, D)
    assert (tok[:, :, N:] == 0).all()
    diff = np.abs(tok[:, :, :N].numpy().astype(np.int32) - fx["v8"].astype(np.int32))
    assert diff.max() <= 1 and (diff != 0).mean() <= 1e-3
    # the offset the epilogue adds back: the fixture's mean plus the mean rounding residual of these codes
    want = v8_offset_expected(_f16(fx["v_perm"]), tok, vsc)
    assert np.allclose(vm.cpu().double().numpy(), want.numpy(), atol=1e-5, rtol=1e-5)
    assert (np.abs(vm.cpu().numpy() - fx["v_mean"]) <= 1e-6 + 16.0 * fx["v_scale"]).all()
    # integer scores through the debug dump of the attention kernel
    mask = torch.from_numpy(fx["mask"]).to(dev)
    nb = (N + 63) // 64
    lib = L.load()
    dump = torch.zeros((B, H, nb * 64, nb * 64), dtype=torch.int32, device=dev)
    out = torch.empty((B, H, N, D), dtype=DTYPE, device=dev)
    ones = torch.ones_like(mask)
    L.check(lib.paro_attn_sparse_fwd(
        L.ptr(q8), L.ptr(k8), L.ptr(v8), L.ptr(qs), L.ptr(ks), L.ptr(vsc), L.ptr(vm), L.ptr(ones), 0,
        L.ptr(out), L.DTYPE_CODE[DTYPE], None, L.ptr(dump), B, H, H, N, N, D,
        q8.stride(0), q8.stride(1), q8.stride(2), k8.stride(0), k8.stride(1), k8.stride(2),
        out.stride(0), out.stride(1), out.stride(2), D ** -0.5, 0, 0, L.stream_of(out)))
    assert np.array_equal(dump[0, 0, :N, :N].cpu().numpy(), fx["s_int32_head0"])
    # attention output and log-sum-exp; tolerance: the one rule of conftest.assert_attention_close (2e-2 plus
    # two e4m3 steps of the |V|-weighted sum the element is built on), cosine >= 0.999; lse within 1e-3 (fp32 sums)
    lse = qattn.qk_int8_sv_f16_accum_f16_attn(q8, k8, vp, out, qs, ks, 1, 0, 2, D ** -0.5, 1, mask)
    ref = torch.from_numpy(fx["o_perm"])
    a_ref, _ = O.sparse_attention(q8.cpu(), k8.cpu(), vp.cpu().abs(), qs.cpu(), ks.cpu(), mask.cpu()[None], D ** -0.5,
                                  out_dtype=torch.float32)
    assert_attention_close(out.cpu(), ref, a_ref)
    assert np.allclose(lse.cpu().numpy(), fx["lse_base2"], atol=1e-3, rtol=1e-4)
    o = PM.permute_inverse(out, orders, grid, n_text).cpu()
    assert cosine(o, torch.from_numpy(fx["o"])) >= 0.999
