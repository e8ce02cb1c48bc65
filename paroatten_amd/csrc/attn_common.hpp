// Shared by the two attention kernels of this library (attn_sparse.hip: two waves per 64-row q-block, any head
// size and variant; attn_sparse_w64.hip: one wave per q-block, D = 64): launch parameters, the constants of the
// softmax-weight arithmetic and small device helpers.  gfx950 only.
#pragma once
#include "paro_device.hpp"
#include <type_traits>

namespace paro {

struct AttnParams {
  const int8_t* q8;
  const int8_t* k8;
  const uint8_t* v8;
  const float* q_scale;
  const float* k_scale;
  const float* v_scale;
  const float* v_mean;
  const uint8_t* sparse;
  void* out;
  float* lse;
  int32_t* s_dump;
  int64_t sparse_bs;
  int64_t qs_b, qs_h, qs_n;
  int64_t ks_b, ks_h, ks_n;
  int64_t os_b, os_h, os_n;
  int B, H, Hkv, Nq, Nk, nbq, nbk;
  int total;  // B*H*nbq workgroups that have work
  float sm_scale_log2e;
  // optional inverse permutation on the way out: q-row r of head h is stored at token
  // n_text + unpermute(r - n_text, orders[h]) (rows below n_text stay); orders == nullptr: row r
  const int* orders;
  int n_text, F, Hh, W;
  int pacing;  // +1: paced launch asked for, -1: plain launch asked for, 0: the library chooses
};

// P~ = 2^(S*c - m + P_EXP_OFFSET).  m is the running row maximum, refreshed lazily: only when a
// block's maximum exceeds it by more than P_HEADROOM are m, O and the row sums rescaled, so that
// P~ <= 2^(P_EXP_OFFSET + P_HEADROOM) = 2^8.75 < 448, the largest e4m3 value.
constexpr float P_EXP_OFFSET = 5.0f;
constexpr float P_HEADROOM = 3.75f;
constexpr int S_MAGIC_BITS = 0x4B400000;  // float 1.5 * 2^23
constexpr float S_MAGIC_F = 12582912.0f;
constexpr int FP8_ONES = 0x38383838;  // four e4m3 1.0
constexpr float FAST_EXP_SHIFT = -0.35f;  // centres the linear-mantissa error of the fast exponential
// fast path: the real-valued byte b becomes the 16-bit field round((b + 0.5) * 256), whose HIGH byte is
// round(b); the field is bounded by 0x7FFF, so the byte is bounded by 0x7F
constexpr float FAST_FIELD_SCALE = 256.0f / 32767.0f;

__device__ __forceinline__ float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// two floats -> two e4m3 bytes in the low (HI = false) or high half of a word; the other half of the
// destination is left as it is, so a full word takes one call of each kind
template <bool HI>
__device__ __forceinline__ void cvt_pk_fp8(int& w, float a, float b) {
  if constexpr (HI) asm("v_cvt_pk_fp8_f32 %0, %1, %2 op_sel:[0,0,1]" : "+v"(w) : "v"(a), "v"(b));
  else asm("v_cvt_pk_fp8_f32 %0, %1, %2" : "=v"(w) : "v"(a), "v"(b));  // upper half: don't care, overwritten next
}

// a*b + c clamped to [0,1] (the clamp is an output modifier: no extra instruction)
__device__ __forceinline__ float fma_clamp01(float a, float b, float c) {
  float r;
  asm("v_fma_f32 %0, %1, %2, %3 clamp" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// two floats in [0,1] -> round(x * 32767) as two 16-bit fields (never negative, at most 0x7FFF)
__device__ __forceinline__ int cvt_pknorm_i16(float a, float b) {
  // (the builtin, not inline assembly: between two assembly statements the compiler assumes the worst
  // hazard and pads with s_nop)
  return __builtin_bit_cast(int, __builtin_amdgcn_cvt_pknorm_i16(a, b));
}

__device__ __forceinline__ float partner_max(float x) {
  // max of own value and that of lane ^ 32: v_permlane32_swap exchanges the upper half of its
  // first operand with the lower half of its second
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return max3(__uint_as_float(r[0]), __uint_as_float(r[1]), __uint_as_float(r[1]));
}

__device__ __forceinline__ v4i buffer_load16(__amdgpu_buffer_rsrc_t rsrc, int voffset, int soffset) {
  // out-of-range bytes read as 0 (raw buffer, bounds-checked by the hardware)
  return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voffset, soffset, 0));
}

// LDS-DMA: 16 bytes per lane from a buffer straight into LDS at lds_base + lane*16; no registers, no
// ds_write; completion is counted by vmcnt
// IMM (a compile-time constant below 4096) is added to BOTH the memory offset and the LDS address: the
// pieces of one tile share one LDS base register (M0) and differ in IMM only
template <int IMM>
__device__ __forceinline__ void buffer_load16_lds(__amdgpu_buffer_rsrc_t rsrc, uint8_t* lds_base, int voffset,
                                                  int soffset) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)lds_base, 16, voffset,
                                           soffset, IMM, 0);
}

// The one-wave-per-q-block kernel (D = 64, no lse, no score dump, plain launch).  out_dtype: PARO_DTYPE_*.
int launch_attn_w64(const AttnParams& p, int out_dtype, bool causal, bool exact, hipStream_t st);

// The kernel with a float16 P.V product (attn_sparse_pv16.hip): p.v8 points at paro_v_f16_pack's tiles, p.v_scale
// and p.v_mean may be null.  Either head size, with or without lse, plain launch.
int launch_attn_pv16(const AttnParams& p, int D, int out_dtype, bool causal, hipStream_t st);

}  // namespace paro
