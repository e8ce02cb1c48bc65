// Shared host/device helpers of libparoatten_hip (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include "../../include/paroatten.h"

namespace paro {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned short v8u16 __attribute__((ext_vector_type(8)));

// thread-local error text, set by PARO_FAIL
void set_error(const char* fmt, ...);

#define PARO_FAIL(code, ...)          \
  do {                                \
    ::paro::set_error(__VA_ARGS__);   \
    return (code);                    \
  } while (0)

#define PARO_CHECK(cond, code, ...)   \
  do {                                \
    if (!(cond)) PARO_FAIL(code, __VA_ARGS__); \
  } while (0)

#define PARO_HIP(expr)                                                          \
  do {                                                                          \
    hipError_t e__ = (expr);                                                    \
    if (e__ != hipSuccess)                                                      \
      PARO_FAIL(PARO_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e__));  \
  } while (0)

// ---- 16-bit float <-> fp32, bit level (identical on host and device) -------------------
template <int DT> struct F16x;  // DT = PARO_DTYPE_F16 / PARO_DTYPE_BF16

template <> struct F16x<PARO_DTYPE_F16> {
  static __device__ __forceinline__ float to_f32(unsigned short u) {
    return __half2float(__ushort_as_half(u));
  }
  static __device__ __forceinline__ unsigned short from_f32(float f) {
    return __half_as_ushort(__float2half_rn(f));
  }
};
template <> struct F16x<PARO_DTYPE_BF16> {
  static __device__ __forceinline__ float to_f32(unsigned short u) {
    return __uint_as_float(((unsigned)u) << 16);
  }
  static __device__ __forceinline__ unsigned short from_f32(float f) {
    // round-to-nearest-even; NaN kept quiet
    unsigned x = __float_as_uint(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((x >> 16) | 0x40);
    x += 0x7fffu + ((x >> 16) & 1u);
    return (unsigned short)(x >> 16);
  }
};

// ---- cross-lane exchange without the LDS crossbar ----------------------------------------------
// value of another lane of the same 16-lane row: DPP control 0xB1 = lane ^ 1, 0x4E = lane ^ 2,
// 0x124 / 0x128 = four / eight lanes further round the row
template <int CTRL> __device__ __forceinline__ float row_dpp(float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, false));
}
// {own value, value of lane ^ 16} resp. {.., lane ^ 32} in some order: the swaps exchange the odd
// rows (upper half) of their first operand with the even rows (lower half) of their second
__device__ __forceinline__ void with_lane_xor16(float x, float& a, float& b) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  a = __uint_as_float(r[0]);
  b = __uint_as_float(r[1]);
}
__device__ __forceinline__ void with_lane_xor32(float x, float& a, float& b) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  a = __uint_as_float(r[0]);
  b = __uint_as_float(r[1]);
}

__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, row_dpp<0xB1>(v));
  v = fmaxf(v, row_dpp<0x4E>(v));
  v = fmaxf(v, row_dpp<0x124>(v));
  v = fmaxf(v, row_dpp<0x128>(v));
  float a, b;
  with_lane_xor16(v, a, b);
  v = fmaxf(a, b);
  with_lane_xor32(v, a, b);
  return fmaxf(a, b);
}

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// batch and head counts become the y / z dimensions of a launch grid (at most 65535 each)
constexpr int MAX_GRID_YZ = 65535;

}  // namespace paro
