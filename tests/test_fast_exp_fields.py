"""CPU model of the arithmetic behind the attention kernel's default softmax weights
(paroatten_amd/csrc/attn_sparse.hip, "fast path"): the e4m3 byte of 2^t is built as
round(8*(t + 7) - 0.35) from one fma with a [0,1] clamp, a conversion to a 16-bit normalised integer
field and a shift-or that interleaves four fields into a word.  Checked here against torch's own
float8_e4m3fn decoding: the byte decodes to within 8 % of 2^t (3.3 % RMS: the linear mantissa is at most
6 % off, rounding to 3 mantissa bits adds up to 3 %) over the whole range the kernel allows, is
monotonic, never reaches the NaN code while the input is inside the headroom, and every input more than
0.11 octaves beyond the headroom yields a field above 126, which is what the kernel's refresh test looks
for (in between, the field is 126 = 448, within 4.5 % of the true weight)."""
import numpy as np
import torch

P_EXP_OFFSET, P_HEADROOM, SHIFT = 5.0, 3.75, -0.35
S_MAGIC = 12582912.0


def fields(s_int, c, m):
    """fp32 model: s (integer score, biased by 1.5*2^23 as the MFMA accumulator holds it) -> 16-bit field.
    c = q_scale*k_scale*sm_scale*log2e; m = running maximum (log2 domain)."""
    f32 = np.float32
    s = (f32(S_MAGIC) + s_int.astype(np.float32)).astype(np.float32)          # exact: |s_int| < 2^22
    c8 = f32(f32(8.0) / f32(32767.0)) * f32(c)
    m_off8 = f32((f32(8.0) * (f32(P_EXP_OFFSET) + f32(7.0) - f32(m)) + f32(SHIFT)) * f32(1.0 / 32767.0))
    bias8 = f32(np.float64(-S_MAGIC) * np.float64(c8) + np.float64(m_off8))    # fmaf: one rounding
    u = (s.astype(np.float64) * np.float64(c8) + np.float64(bias8)).astype(np.float32)   # v_fma_f32
    u = np.clip(u, f32(0), f32(1))                                             # clamp output modifier
    return np.rint(u.astype(np.float64) * 32767.0).astype(np.int64)            # v_cvt_pknorm_i16_f32 (RNE)


def decode_e4m3(b):
    return torch.from_numpy(b.astype(np.uint8)).view(torch.float8_e4m3fn).float().numpy()


def test_fields_inside_the_headroom_decode_to_two_to_the_t():
    c = 3.1e-4
    m = 11.3
    # t = S*c - m + OFFSET over [-9, OFFSET + HEADROOM]
    t_want = np.linspace(-9.0, P_EXP_OFFSET + P_HEADROOM, 20001)
    s_int = np.rint((t_want + m - P_EXP_OFFSET) / c)
    t = s_int * c - m + P_EXP_OFFSET
    f = fields(s_int, c, m)
    assert f.max() <= 126 and f.min() == 0
    assert (np.diff(f) >= 0).all()
    val = decode_e4m3(f)
    normal = t >= -6.0 + 0.1          # e4m3 normals start at 2^-6
    rel = val[normal] / np.exp2(t[normal]) - 1.0
    assert np.abs(rel).max() <= 0.08, np.abs(rel).max()
    assert np.sqrt((rel ** 2).mean()) <= 0.035, np.sqrt((rel ** 2).mean())
    assert abs(rel.mean()) <= 0.01    # centred by the -0.35 shift
    # below 2^-6 the byte's mantissa-only codes fall off linearly to 0 at t = -7: absolute error below
    # 2^-7 * 1.1, i.e. 2e-5 of the largest weight
    assert (val[t < -7.0] == 0).all()
    sub = ~normal
    assert np.abs(val[sub] - np.exp2(t[sub])).max() <= 2.0 ** -7 * 1.1


def test_scores_beyond_the_headroom_are_detected():
    c, m = 7.7e-4, -3.2
    t_want = np.linspace(P_EXP_OFFSET + P_HEADROOM + 0.11, 200.0, 5001)
    s_int = np.rint((t_want + m - P_EXP_OFFSET) / c)
    f = fields(s_int, c, m)
    assert f.min() > 126 and f.max() <= 0x7FFF       # never negative, never more than 15 bits
    # just past the headroom the field is still 126 (= 448), within 4.5 % of the true weight
    t_edge = np.linspace(P_EXP_OFFSET + P_HEADROOM, P_EXP_OFFSET + P_HEADROOM + 0.1, 101)
    s_edge = np.rint((t_edge + m - P_EXP_OFFSET) / c)
    fe = fields(s_edge, c, m)
    assert ((fe == 126) | (fe == 127)).all()
    ok = fe == 126
    assert np.abs(448.0 / np.exp2(s_edge[ok] * c - m + P_EXP_OFFSET) - 1.0).max() <= 0.045
    # and as half-precision bit patterns, compared the way v_pk_maximum3_f16 compares them (denormals
    # kept), they order like the integers, NaN patterns (0x7C01..) reading as "large"
    legal = np.arange(0, 127, dtype=np.uint16).view(np.float16).astype(np.float64)
    for x in (127, 128, 255, 256, 1023, 1024, 0x7BFF, 0x7C00):
        assert np.array([x], dtype=np.uint16).view(np.float16).astype(np.float64)[0] > legal.max()
    assert np.isnan(np.array([0x7C01, 0x7FFF], dtype=np.uint16).view(np.float16)).all()


def test_four_fields_interleave_into_bytes_without_spilling():
    rng = np.random.default_rng(0)
    f = rng.integers(0, 127, size=(1000, 4))
    lo = f[:, 0] | (f[:, 2] << 16)           # v_cvt_pknorm_i16_f32(u0, u2)
    hi = f[:, 1] | (f[:, 3] << 16)           # v_cvt_pknorm_i16_f32(u1, u3)
    w = ((hi << 8) | lo) & 0xFFFFFFFF        # v_lshl_or_b32
    for i in range(4):
        assert np.array_equal((w >> (8 * i)) & 0xFF, f[:, i])
