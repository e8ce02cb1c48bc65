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

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// batch and head counts become the y / z dimensions of a launch grid (at most 65535 each)
constexpr int MAX_GRID_YZ = 65535;

}  // namespace paro
