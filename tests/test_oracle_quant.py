"""Pins oracle.quant_int8 and its wrappers without retyping its formula: a hand-derivable
known-answer case (the reference's own smoke input, bench/test.py:5-14), invariants every correct
symmetric int8 quantiser obeys, and an independent scalar re-implementation in Python floats
rounded through numpy float32."""
import numpy as np
import pytest
import torch

from oracle import paro_oracle as O


def test_known_answer_rows_bench_test_py():
    rows = torch.arange(-256, 256, dtype=torch.bfloat16).unsqueeze(1)
    q = rows.repeat(1, 64)[None, None]
    q8, qs, k8, ks = O.per_warp_int8(q, q, BLKQ=64, WARPQ=32, BLKK=64)
    assert qs.shape == (1, 1, 16) and ks.shape == (1, 1, 8)
    # group 0 of Q: rows -256..-225 -> amax 256, row -256 -> -127, row -225 -> round(-225*127/256) = -112
    assert float(qs[0, 0, 0]) == pytest.approx(256 / 127, rel=1e-7)
    assert q8[0, 0, 0, 0] == -127 and q8[0, 0, 31, 0] == -112
    # group 8: rows 0..31 -> amax 31: row 0 -> 0, row 31 -> 127, row 16 -> round(16*127/31) = 66
    assert float(qs[0, 0, 8]) == pytest.approx(31 / 127, rel=1e-7)
    assert q8[0, 0, 256, 0] == 0 and q8[0, 0, 287, 0] == 127 and q8[0, 0, 272, 0] == 66
    # K block 0: rows -256..-193 -> amax 256; block 7: rows 192..255 -> amax 255 -> row 255 -> 127
    assert float(ks[0, 0, 0]) == pytest.approx(256 / 127, rel=1e-7)
    assert float(ks[0, 0, 7]) == pytest.approx(255 / 127, rel=1e-7)
    assert k8[0, 0, 511, 0] == 127 and k8[0, 0, 448, 0] == round(192 * 127 / 255)
    # all 64 channels of a row are equal
    assert (q8 == q8[..., :1]).all()


def _scalar_quant(block: np.ndarray):
    """independent scalar path: python loop, numpy float32 scalars"""
    amax = np.float32(1e-7)
    for x in block.flat:
        amax = max(amax, np.float32(abs(np.float32(x))))
    inv = np.float32(127.0) / amax
    out = np.empty(block.shape, dtype=np.int8)
    for i, x in enumerate(block.flat):
        r = np.float32(x) * inv
        out.flat[i] = int(np.clip(np.rint(r), -128, 127))  # rint = ties to even
    return out, amax / np.float32(127.0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_against_scalar_reimplementation(dtype):
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(1, 2, 50, 64, generator=g) * 3).to(dtype)
    q8, sc = O.quant_int8(x, 32)
    assert sc.shape == (1, 2, 2)
    xf = x.float().numpy()
    for h in range(2):
        for gi in range(2):
            blk = xf[0, h, gi * 32:min(50, gi * 32 + 32)]
            rq, rs = _scalar_quant(blk)
            assert np.array_equal(q8[0, h, gi * 32:gi * 32 + blk.shape[0]].numpy(), rq)
            assert np.float32(sc[0, h, gi]) == rs


def test_invariants_and_edge_cases():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(2, 3, 200, 128, generator=g).half()
    q8, sc = O.quant_int8(x, 64)
    assert sc.shape == (2, 3, 4)
    deq = q8.float() * sc.repeat_interleave(64, dim=-1)[..., :200, None]
    # half a quantisation step, plus the few-ulp slack of scale * (127/amax) not being exactly 1
    assert ((deq - x.float()).abs() <= sc.repeat_interleave(64, dim=-1)[..., :200, None] * 0.5 + 1e-6 * x.float().abs()).all()
    assert q8.abs().max() <= 127
    # the largest element of every group maps to +-127
    xg = torch.nn.functional.pad(x.float(), (0, 0, 0, 56)).reshape(2, 3, 4, -1)
    qg = torch.nn.functional.pad(q8, (0, 0, 0, 56)).reshape(2, 3, 4, -1)
    pos = xg.abs().argmax(dim=-1, keepdim=True)
    assert (qg.gather(-1, pos).abs() == 127).all()
    # all-zero group: scale 1e-7/127, zeros out
    z = torch.zeros(1, 1, 64, 64, dtype=torch.float16)
    q0, s0 = O.quant_int8(z, 64)
    assert (q0 == 0).all() and float(s0) == pytest.approx(1e-7 / 127, rel=1e-6)
    # groups wholly past the end exist (ceil(N/BLKQ)*(BLKQ/WARPQ) scales) and are "zero" groups
    x2 = torch.randn(1, 1, 70, 64, generator=g).half()
    q8b, qs, _, _ = O.per_warp_int8(x2, x2, BLKQ=128, WARPQ=32, BLKK=64)
    assert qs.shape == (1, 1, 4) and float(qs[0, 0, 3]) == pytest.approx(1e-7 / 127, rel=1e-6)
    assert q8b.shape == x2.shape


def test_mean_subtraction_and_sm_scale_fold():
    g = torch.Generator().manual_seed(5)
    k = (torch.randn(1, 2, 128, 64, generator=g) + 3).half()
    km = k.float().mean(dim=2, keepdim=True).half()
    a8, asc = O.quant_int8(k, 64, mean=km.reshape(1, 2, 64))
    centred = k.float() - km.float()  # exact in fp32: both operands are fp16 values
    b8, bsc = O.quant_int8(centred, 64)  # fp32 input passes through .to(float32) unchanged
    assert torch.equal(a8, b8) and torch.equal(asc, bsc)
    # per_block_int8 folds sm_scale*log2e into Q before the amax
    q = torch.randn(1, 2, 128, 64, generator=g).half()
    q8, qs, _, _ = O.per_block_int8(q, k, BLKQ=128, BLKK=64, sm_scale=0.125)
    f = torch.tensor(0.125 * 1.44269504, dtype=torch.float32)
    c8, cs = O.quant_int8(q.float() * f, 128)
    assert torch.equal(q8, c8) and torch.equal(qs, cs)


def test_ties_round_to_even():
    # amax 127 -> factor exactly 1: x.5 values must round to even
    x = torch.tensor([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5] + [0.0] * 56, dtype=torch.float16)
    x = x.reshape(1, 1, 1, 64).repeat(1, 1, 16, 1)
    q8, sc = O.quant_int8(x, 16)
    assert q8[0, 0, 0, :8].tolist() == [127, 0, 2, 2, 0, -2, -2, 4]
    assert float(sc) == 1.0


def _lane_enumeration(n, is_key):
    """Scale index per token from an enumeration of the reference kernel's accumulator lanes, the way its
    per-thread branch reads them (csrc/qattn/qk_int_sv_f16_cuda_sm80.cu:112-116: q_scale_idx = ... +
    warp_idx_q * 8 + lane_id / 4, :129-133: k_scale_idx = ... + lane_id % 4, advancing by 4 per 64-key block):
    lane l of a warp holds, in every m16n8 tile, rows l/4 and l/4 + 8 and columns 2*(l%4), 2*(l%4) + 1."""
    idx = [-1] * n
    if is_key:
        for block in range((n + 63) // 64):
            for lane in range(32):
                for tile in range(8):              # 8-column tiles of the 64-key block
                    for e in range(2):
                        c = block * 64 + tile * 8 + 2 * (lane % 4) + e
                        if c < n:
                            idx[c] = block * 4 + lane % 4
    else:
        for warp in range((n + 31) // 32):
            for lane in range(32):
                for tile in range(2):              # 16-row tiles of the 32-row warp
                    for half in range(2):
                        r = warp * 32 + tile * 16 + lane // 4 + 8 * half
                        if r < n:
                            idx[r] = warp * 8 + lane // 4
    assert min(idx) >= 0
    return torch.tensor(idx)


@pytest.mark.parametrize("n", [1, 31, 64, 100, 257])
def test_per_thread_scale_index_matches_the_lane_enumeration(n):
    assert torch.equal(O.per_thread_scale_index(n, False), _lane_enumeration(n, False))
    assert torch.equal(O.per_thread_scale_index(n, True), _lane_enumeration(n, True))
    # the values a wrong law would give differ: plain 8-row groups, or pairs of 16 consecutive keys
    if n >= 64:
        assert not torch.equal(O.per_thread_scale_index(n, False), torch.arange(n) // 4)
        assert not torch.equal(O.per_thread_scale_index(n, True), torch.arange(n) // 16)


@pytest.mark.parametrize("is_key", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_per_thread_quantiser_is_quant_int8_on_regrouped_tokens(is_key, dtype):
    """Tokens sorted so that every per-thread group is contiguous turn the per-thread quantiser into the
    pinned group quantiser (groups of 4 query tokens / 16 key tokens); a ragged length equals its zero-padded
    self on the tokens that exist."""
    g = torch.Generator().manual_seed(5)
    B, H, N, D = 2, 3, 192, 64
    x = (torch.randn(B, H, N, D, generator=g) * torch.rand(1, 1, N, 1, generator=g) * 3).to(dtype)
    mean = x.float().mean(dim=2).to(dtype) if is_key else None
    q8, sc = O.quant_int8_per_thread(x, is_key, mean=mean)
    idx = _lane_enumeration(N, is_key)
    order = torch.argsort(idx, stable=True)                   # tokens of scale 0, then of scale 1, ...
    per = 16 if is_key else 4
    assert torch.equal(idx[order], torch.arange(N // per).repeat_interleave(per))
    q8_ref, sc_ref = O.quant_int8(x[:, :, order], per, mean=mean)
    assert torch.equal(sc, sc_ref)
    assert torch.equal(q8[:, :, order], q8_ref)
    assert sc.shape == (B, H, N // 64 * (4 if is_key else 16))
    # ragged
    n = 150
    q8r, scr = O.quant_int8_per_thread(x[:, :, :n], is_key, mean=mean)
    xz = x.clone()
    if mean is not None:
        xz[:, :, n:] = mean[:, :, None, :]                    # x - mean = 0 exactly there
    else:
        xz[:, :, n:] = 0
    q8z, scz = O.quant_int8_per_thread(xz, is_key, mean=mean)
    assert torch.equal(q8r, q8z[:, :, :n]) and torch.equal(scr, scz)
