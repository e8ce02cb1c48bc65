// Device helpers shared by the permutation kernels and the V -> FP8 kernels (gfx950 only).
#pragma once
#include "paro_common.hpp"

namespace paro {

// tokens per workgroup of the two statistics passes.  Measured: the V statistics (three values per
// channel to reduce and write) want long chunks, 1024 beats 256 by 7 %; the K mean, launched per group
// of heads, runs out of workgroups beyond 256.
constexpr int V_CHUNK = 1024;  // per-channel V statistics
constexpr int K_CHUNK = 256;   // rotated K mean

// strides of the (f,h,w) coordinates in the permuted order `order`
// (0 FHW, 1 FWH, 2 HWF, 3 HFW, 4 WHF, 5 WFH).  Written as selects: a switch that assigns through the
// three references made the compiler keep them in scratch memory, 12 bytes written per lane and use.
__device__ __forceinline__ void order_strides(int order, int F, int Hh, int W, int& sf, int& sh, int& sw) {
  if ((unsigned)order > 5u) order = 0;  // the table lives on the device and cannot be checked by the host
  sf = (order <= 1) ? Hh * W : (order == 3 ? W : (order == 5 ? Hh : 1));
  sh = (order == 2 || order == 3) ? W * F : (order == 0 ? W : (order == 4 ? F : 1));
  sw = (order >= 4) ? Hh * F : (order == 1 ? Hh : (order == 2 ? F : 1));
}

// image index in permuted order -> image index in source (F,H,W row-major) order
__device__ __forceinline__ int unpermute_index(int di, int order, int F, int Hh, int W) {
  // axes in the permuted order, slowest first (cogvideox.py:38-45)
  int s1, s2, a0, a1, a2;  // sizes of the two faster axes; which source axis each position is
  switch (order) {
    default:
    case 0: a0 = 0; a1 = 1; a2 = 2; break;
    case 1: a0 = 0; a1 = 2; a2 = 1; break;
    case 2: a0 = 1; a1 = 2; a2 = 0; break;
    case 3: a0 = 1; a1 = 0; a2 = 2; break;
    case 4: a0 = 2; a1 = 1; a2 = 0; break;
    case 5: a0 = 2; a1 = 0; a2 = 1; break;
  }
  const int S[3] = {F, Hh, W};
  s1 = S[a1];
  s2 = S[a2];
  int c[3];
  c[a2] = di % s2;
  const int r = di / s2;
  c[a1] = r % s1;
  c[a0] = r / s1;
  return (c[0] * Hh + c[1]) * W + c[2];
}

// two floats -> two 16-bit values (round to nearest even), `lo` in bits 0..15: one instruction on gfx950
template <int DT>
__device__ __forceinline__ unsigned pack2_from_f32(float lo, float hi) {
  unsigned w;
  if constexpr (DT == PARO_DTYPE_F16) asm("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(w) : "v"(lo), "v"(hi));
  else asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(w) : "v"(lo), "v"(hi));
  return w;
}
template <int DT>
__device__ __forceinline__ float lo16_to_f32(unsigned w) {
  if constexpr (DT == PARO_DTYPE_BF16) return __uint_as_float(w << 16);
  else return F16x<DT>::to_f32((unsigned short)(w & 0xffffu));
}
template <int DT>
__device__ __forceinline__ float hi16_to_f32(unsigned w) {
  if constexpr (DT == PARO_DTYPE_BF16) return __uint_as_float(w & 0xffff0000u);
  else return F16x<DT>::to_f32((unsigned short)(w >> 16));
}
// element j (0..7) of a 16-byte piece
template <int DT>
__device__ __forceinline__ float elem16_to_f32(const v4i& raw, int j) {
  const unsigned w = (unsigned)raw[j >> 1];
  return (j & 1) ? hi16_to_f32<DT>(w) : lo16_to_f32<DT>(w);
}

// rotation of 8 consecutive channels (4 pairs) of one token; cs/sn: that token's table entries
template <int DT>
__device__ __forceinline__ v4i rotate8(const v4i raw, const float* cs, const float* sn) {
  v4i o;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const float x0 = lo16_to_f32<DT>((unsigned)raw[j]);
    const float x1 = hi16_to_f32<DT>((unsigned)raw[j]);
    const float o0 = __fsub_rn(__fmul_rn(x0, cs[2 * j]), __fmul_rn(x1, sn[2 * j]));
    const float o1 = __fadd_rn(__fmul_rn(x1, cs[2 * j + 1]), __fmul_rn(x0, sn[2 * j + 1]));
    o[j] = (int)pack2_from_f32<DT>(o0, o1);
  }
  return o;
}

__device__ __forceinline__ void* uniform_ptr(const void* ptr) {
  // the address is the same in every lane; say so, so that the descriptor lives in scalar registers
  const unsigned long long a = reinterpret_cast<unsigned long long>(ptr);
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)a);
  const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32));
  return reinterpret_cast<void*>(((unsigned long long)hi << 32) | lo);
}

// the same rotation (or none, ROT = false) with the result left in fp32: the values are those the
// 16-bit result holds, so arithmetic on them equals arithmetic on a stored and reloaded tensor
template <int DT>
__device__ __forceinline__ void rotate8_f32(const v4i raw, bool rot, const float* cs, const float* sn, float* out) {
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const float x0 = lo16_to_f32<DT>((unsigned)raw[j]);
    const float x1 = hi16_to_f32<DT>((unsigned)raw[j]);
    out[2 * j] = x0;
    out[2 * j + 1] = x1;
    if (rot) {
      const float o0 = __fsub_rn(__fmul_rn(x0, cs[2 * j]), __fmul_rn(x1, sn[2 * j]));
      const float o1 = __fadd_rn(__fmul_rn(x1, cs[2 * j + 1]), __fmul_rn(x0, sn[2 * j + 1]));
      const unsigned w = pack2_from_f32<DT>(o0, o1);
      out[2 * j] = lo16_to_f32<DT>(w);
      out[2 * j + 1] = hi16_to_f32<DT>(w);
    }
  }
}

// four values y (|y| <= 127.5, not yet rounded) -> four int8 = rint(y) packed in a word.  Adding
// 1.5*2^23 rounds to the nearest integer, ties to even, exactly as rintf does (the sum lies in
// [2^23, 2^24), where floats are the integers), and leaves the two's-complement byte in bits 0..7.
__device__ __forceinline__ unsigned pack4_rint_i8(float y0, float y1, float y2, float y3) {
  constexpr float M = 12582912.0f;
  const unsigned a0 = __float_as_uint(__fadd_rn(y0, M)), a1 = __float_as_uint(__fadd_rn(y1, M));
  const unsigned a2 = __float_as_uint(__fadd_rn(y2, M)), a3 = __float_as_uint(__fadd_rn(y3, M));
  const unsigned lo = __builtin_amdgcn_perm(a1, a0, 0x0c0c0400u);  // [a0.b0, a1.b0, 0, 0]
  const unsigned hi = __builtin_amdgcn_perm(a3, a2, 0x0c0c0400u);
  return lo | (hi << 16);
}

// One 64-token V tile held in LDS as 16-bit rows (row pitch PITCH elements) -> (v - mean) * recp as
// e4m3 in the fragment order of the P.V MFMA: 16-byte piece c = (dt, mt, lane) holds channel
// 32*dt + lane%32 of tokens 32*mt + 8*g + 4*(lane/32) + q, byte 4*g + q.  recp = 448 / max|v - mean|
// (0 for a constant channel), as MeanScaleKernel of the reference forms it
// (csrc/fused/fused.cu:399,414).  256 threads.  SWZ: rows are unpadded (PITCH = D) and 16-byte chunk c
// of row r sits at chunk position c ^ 4*((r >> 2) & 1).
// resid[n] (n < D/64): the rounding residual sum over the 32 tokens of row tile mt = wave%2 of
// (v - mean)*recp - e4m3(that), for channel 32*(wave/2 + 2n) + lane%32, the same value in lanes l and
// l^32.  Its mean over all tokens, times the scale, is what the codes of a channel are off by on
// average: the attention epilogue adds it back together with the channel mean.
template <int DT, int D, int PITCH, bool SWZ = false>
__device__ __forceinline__ void pack_v_tile(const unsigned short* tile, uint8_t* ob, const float* v_recp,
                                            const float* v_mean, int tok0, int N, int t, float* resid) {
  const bool full = tok0 + 64 <= N;    // uniform: only the last tile of a sequence checks its rows
#pragma unroll
  for (int n = 0; n < D / 64; n++) {   // 4*D pieces, 256 threads
    const int c = t + 256 * n;
    const int lane = c & 63, mt = (c >> 6) & 1, dt = c >> 7;
    const int ch = 32 * dt + (lane & 31);
    const float mean = v_mean ? v_mean[ch] : 0.f;
    const float rc = v_recp[ch];
    int w[4];
    float es = 0.f;
#pragma unroll
    for (int g = 0; g < 4; g++) {
      float f[4];
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const int r = 32 * mt + 8 * g + 4 * (lane >> 5) + q;
        const int at = SWZ ? r * PITCH + ((((ch >> 3) ^ (((r >> 2) & 1) << 2)) << 3) | (ch & 7)) : r * PITCH + ch;
        const float x = F16x<DT>::to_f32(tile[at]);
        f[q] = (full || tok0 + r < N) ? (x - mean) * rc : 0.f;
      }
      int p = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], 0, false);
      p = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], p, true);
      w[g] = p;
      es += ((f[0] - __builtin_amdgcn_cvt_f32_fp8(p, 0)) + (f[1] - __builtin_amdgcn_cvt_f32_fp8(p, 1))) +
            ((f[2] - __builtin_amdgcn_cvt_f32_fp8(p, 2)) + (f[3] - __builtin_amdgcn_cvt_f32_fp8(p, 3)));
    }
    __builtin_nontemporal_store(v4i{w[0], w[1], w[2], w[3]}, reinterpret_cast<v4i*>(ob + (int64_t)c * 16));
    float a, b;
    with_lane_xor32(es, a, b);
    resid[n] = a + b;
  }
}

// residual sums of pack_v_tile: [B*Hkv][nb][2 row tiles][D] floats behind the statistics partials
__host__ __device__ inline int64_t v_resid_offset(int64_t BH, int n_chunks, int D) { return BH * n_chunks * 3 * D; }

// where v_fp8_stats leaves recp[b,h,:] inside the partial-sum workspace
__host__ __device__ inline int64_t v_recp_offset(int64_t bh, int n_chunks, int D) { return bh * n_chunks * 3 * D; }

// per-(batch, head, channel) statistics of V: v_scale = max|v - mean| / 448, v_mean = mean over the
// N tokens (0 if !smooth), and recp = 448 / max|v - mean| at partial[v_recp_offset(bh, ...) + ch];
// two launches on `st` (defined in v_fp8.hip)
int v_fp8_stats(const void* v, int dtype, float* v_scale, float* v_mean, float* partial, int B, int Hkv, int N,
                int D, int64_t vs_b, int64_t vs_h, int64_t vs_n, int smooth, hipStream_t st);
// v_mean[b,h,ch] += v_scale[b,h,ch] * (sum of the channel's residual sums) / N, in a fixed order (one launch)
int v_fp8_add_residual(const float* resid, const float* v_scale, float* v_mean, int B, int Hkv, int N, int D,
                       hipStream_t st);

}  // namespace paro
