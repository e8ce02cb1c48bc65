"""CPU model of the arithmetic behind the attention kernel's default softmax weights
(paroatten_amd/csrc/attn_sparse.hip, "fast path"): the e4m3 byte of 2^t is built as
b = round(8*(t + 7) - 0.35) from one fma with a [0,1] clamp that yields (b + 0.5) * 256 / 32767, a
conversion to a 16-bit normalised integer field (round(u * 32767), whose HIGH byte is then round(b)) and
a byte permute that gathers the high bytes of four fields into a word.  Checked here against torch's own
float8_e4m3fn decoding: the byte decodes to within 8 % of 2^t (3.3 % RMS: the linear mantissa is at most
6 % off, rounding to 3 mantissa bits adds up to 3 %) over the whole range the kernel allows, is
monotonic, never reaches the NaN code while the input is inside the headroom, and EVERY input more than
0.11 octaves beyond the headroom, however far, yields exactly the byte 0x7F, the e4m3 NaN, which the
kernel's row sums expose (in between, the byte is 126 = 448, within 4.5 % of the true weight).  No byte
ever has its sign bit set and no field reaches into a neighbouring byte."""
import numpy as np
import torch

P_EXP_OFFSET, P_HEADROOM, SHIFT = 5.0, 3.75, -0.35
S_MAGIC = 12582912.0
FIELD_SCALE = np.float32(256.0) / np.float32(32767.0)


def fields(s_int, c, m):
    """fp32 model: s (integer score, biased by 1.5*2^23 as the MFMA accumulator holds it) -> 16-bit field.
    c = q_scale*k_scale*sm_scale*log2e; m = running maximum (log2 domain)."""
    f32 = np.float32
    s = (f32(S_MAGIC) + s_int.astype(np.float32)).astype(np.float32)          # exact: |s_int| < 2^22
    c8 = f32(f32(8.0) * FIELD_SCALE) * f32(c)
    m_off8 = f32((f32(8.0) * (f32(P_EXP_OFFSET) + f32(7.0) - f32(m)) + f32(SHIFT) + f32(0.5)) * FIELD_SCALE)
    bias8 = f32(np.float64(-S_MAGIC) * np.float64(c8) + np.float64(m_off8))    # fmaf: one rounding
    u = (s.astype(np.float64) * np.float64(c8) + np.float64(bias8)).astype(np.float32)   # v_fma_f32
    u = np.clip(u, f32(0), f32(1))                                             # clamp output modifier
    return np.rint(u.astype(np.float64) * 32767.0).astype(np.int64)            # v_cvt_pknorm_i16_f32 (RNE)


def byte_of(field):
    return field >> 8


def decode_e4m3(b):
    return torch.from_numpy(b.astype(np.uint8)).view(torch.float8_e4m3fn).float().numpy()


def test_bytes_inside_the_headroom_decode_to_two_to_the_t():
    c = 3.1e-4
    m = 11.3
    # t = S*c - m + OFFSET over [-9, OFFSET + HEADROOM]
    t_want = np.linspace(-9.0, P_EXP_OFFSET + P_HEADROOM, 20001)
    s_int = np.rint((t_want + m - P_EXP_OFFSET) / c)
    t = s_int * c - m + P_EXP_OFFSET
    f = fields(s_int, c, m)
    assert f.max() <= 0x7FFF and f.min() >= 0
    b = byte_of(f)
    assert b.max() <= 126 and b.min() == 0
    assert (np.diff(b) >= 0).all()
    # the high byte of the field IS the rounded real-valued byte (ties aside, which sit 1/512 of a byte off)
    want = 8.0 * (t + 7.0) + SHIFT
    inside = want > 0.0
    assert np.abs(b[inside] - want[inside]).max() <= 0.5 + 1.0 / 256
    val = decode_e4m3(b)
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


def test_scores_beyond_the_headroom_become_the_nan_byte():
    c, m = 7.7e-4, -3.2
    t_want = np.concatenate([np.linspace(P_EXP_OFFSET + P_HEADROOM + 0.11, 200.0, 5001), [1e3, 1e4]])
    s_int = np.rint((t_want + m - P_EXP_OFFSET) / c)
    s_int = np.minimum(s_int, 2.0 ** 22 - 1)          # what an int8 x int8 accumulator can hold at D <= 128
    b = byte_of(fields(s_int, c, m))
    assert (b == 0x7F).all()                            # exactly the NaN code: never a sign bit, never a spill
    assert np.isnan(decode_e4m3(b)).all()
    # with no maximum yet (m = -1e30, the state before the first block) everything is the NaN byte as well
    assert (byte_of(fields(np.array([-(2.0 ** 22) + 1, 0.0, 12345.0]), c, -1e30)) == 0x7F).all()
    # just past the headroom the byte is still 126 (= 448), within 4.5 % of the true weight
    t_edge = np.linspace(P_EXP_OFFSET + P_HEADROOM, P_EXP_OFFSET + P_HEADROOM + 0.1, 101)
    s_edge = np.rint((t_edge + m - P_EXP_OFFSET) / c)
    be = byte_of(fields(s_edge, c, m))
    assert ((be == 126) | (be == 127)).all()
    ok = be == 126
    assert np.abs(448.0 / np.exp2(s_edge[ok] * c - m + P_EXP_OFFSET) - 1.0).max() <= 0.045


def test_masked_and_far_below_scores_are_zero_bytes():
    c, m = 2.0e-4, 4.0
    s_int = np.array([-(2.0 ** 22) + 1, -3.0e6, -1.0e5])
    assert (byte_of(fields(s_int, c, m)) == 0).all()
    # a masked score (-inf in place of the biased score) leaves the fma as -inf and the clamp as 0
    f32 = np.float32
    u = np.clip(f32(-np.inf) * f32(1e-6) + f32(3.0), f32(0), f32(1))
    assert u == 0


def test_four_high_bytes_gather_into_a_word():
    rng = np.random.default_rng(0)
    f = rng.integers(0, 0x8000, size=(1000, 4))        # any field the conversion can produce
    lo = f[:, 0] | (f[:, 2] << 16)           # v_cvt_pknorm_i16_f32(u0, u2)
    hi = f[:, 1] | (f[:, 3] << 16)           # v_cvt_pknorm_i16_f32(u1, u3)

    def perm(s0, s1, sel):                   # v_perm_b32: bytes 0-3 of s1, 4-7 of s0
        src = (s0.astype(np.uint64) << np.uint64(32)) | s1.astype(np.uint64)
        out = np.zeros_like(s1, dtype=np.uint64)
        for i in range(4):
            k = (sel >> (8 * i)) & 0xFF
            out |= ((src >> np.uint64(8 * k)) & np.uint64(0xFF)) << np.uint64(8 * i)
        return out

    w = perm(hi, lo, 0x07030501)
    for i in range(4):
        assert np.array_equal((w >> np.uint64(8 * i)) & np.uint64(0xFF), (f[:, i] >> 8).astype(np.uint64))
        assert (((w >> np.uint64(8 * i)) & np.uint64(0x80)) == 0).all()
