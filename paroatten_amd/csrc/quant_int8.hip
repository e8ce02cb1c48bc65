// Per-group symmetric INT8 quantisation of Q / K (HBM-bound).
//
// One 64-lane wave owns one group of G tokens x D channels: every lane holds G*D/64 values in
// registers (16-byte loads, consecutive lanes on consecutive addresses), the group maximum is a
// wave reduction, and the int8 result leaves as 8-byte stores.  Nothing goes through LDS.
// Arithmetic follows QuantInt8Kernel of the reference (csrc/fused/fused.cu:64-198) in IEEE fp32:
// this file is compiled without fast-math and with fp contraction off.
#include "paro_device.hpp"

namespace paro {

template <int DT, int D, int G, bool MEAN, bool SMS>
__global__ void __launch_bounds__(256) quant_int8_kernel(
    const unsigned short* __restrict__ x, const unsigned short* __restrict__ mean,
    int8_t* __restrict__ out, float* __restrict__ scale, int N, int n_groups,
    int64_t xs_b, int64_t xs_h, int64_t xs_n, int64_t ms_b, int64_t ms_h,
    int64_t os_b, int64_t os_h, int64_t os_n, int64_t ss_b, int64_t ss_h, float sm_scale) {
  constexpr int LPR = D / 8;          // lanes per token row (16-byte chunks)
  constexpr int CH = G * D / 512;     // 16-byte chunks per lane
  constexpr int ROWS_PER_IT = 64 / LPR;
  const int lane = threadIdx.x & 63;
  const int g = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (g >= n_groups) return;
  const int h = blockIdx.y, b = blockIdx.z;
  const int col = (lane % LPR) * 8;
  const int row0 = lane / LPR;

  float mv[8];
  if constexpr (MEAN) {
    const v4i m = *reinterpret_cast<const v4i*>(mean + b * ms_b + h * ms_h + col);
#pragma unroll
    for (int j = 0; j < 4; j++) {
      mv[2 * j] = F16x<DT>::to_f32((unsigned short)(m[j] & 0xffff));
      mv[2 * j + 1] = F16x<DT>::to_f32((unsigned short)((unsigned)m[j] >> 16));
    }
  }

  const unsigned short* xb = x + b * xs_b + h * xs_h + col;
  v4i raw[CH];
#pragma unroll
  for (int i = 0; i < CH; i++) {
    const int tok = g * G + i * ROWS_PER_IT + row0;
    raw[i] = (tok < N) ? __builtin_nontemporal_load(reinterpret_cast<const v4i*>(xb + (int64_t)tok * xs_n))
                       : v4i{0, 0, 0, 0};
  }

  // value of element (chunk i, slot j) after mean subtraction / scaling; recomputed in the
  // second pass instead of being kept, so that only the packed input stays in registers
  auto value = [&](int i, int j) -> float {
    float f = elem16_to_f32<DT>(raw[i], j);
    if constexpr (MEAN) f -= mv[j];
    if constexpr (SMS) f *= sm_scale;
    return f;
  };

  float amax = 0.0000001f;
#pragma unroll
  for (int i = 0; i < CH; i++) {
    const int tok = g * G + i * ROWS_PER_IT + row0;
    if (tok < N) {  // rows past the end read as zero, whatever the mean
#pragma unroll
      for (int j = 0; j < 8; j++) amax = fmaxf(amax, fabsf(value(i, j)));
    }
  }
  amax = wave_max(amax);
  if (lane == 0) scale[b * ss_b + h * ss_h + g] = amax / 127.0f;
  const float inv = 127.0f / amax;

  int8_t* ob = out + b * os_b + h * os_h + col;
#pragma unroll
  for (int i = 0; i < CH; i++) {
    const int tok = g * G + i * ROWS_PER_IT + row0;
    // |value * (127/amax)| <= 127 up to rounding: the reference's clamp to [-128,127] never acts
    float y[8];
#pragma unroll
    for (int j = 0; j < 8; j++) y[j] = value(i, j) * inv;
    if (tok < N)
      __builtin_nontemporal_store(
          v2i{(int)pack4_rint_i8(y[0], y[1], y[2], y[3]), (int)pack4_rint_i8(y[4], y[5], y[6], y[7])},
          reinterpret_cast<v2i*>(ob + (int64_t)tok * os_n));
  }
}

// The same arithmetic on the per-thread groups of qk_quant_gran 3: a wave owns 64 tokens and their 16 (Q: two
// 32-token groups of 8) or 4 (K) scales.  Token row r of the 64 belongs to group
//   Q: (r / 32) * 8 + r % 8        K: (r % 8) / 2
// A lane's chunks sit in rows row0 + i * ROWS_PER_IT; every group maximum is a full wave reduction of the
// lanes' contributions to that group (the kernel is bound by HBM, not by these).
template <int DT, int D, bool KEY, bool MEAN>
__global__ void __launch_bounds__(256) quant_int8_per_thread_kernel(
    const unsigned short* __restrict__ x, const unsigned short* __restrict__ mean, int8_t* __restrict__ out,
    float* __restrict__ scale, int N, int n_blocks, int64_t xs_b, int64_t xs_h, int64_t xs_n, int64_t ms_b,
    int64_t ms_h, int64_t os_b, int64_t os_h, int64_t os_n) {
  constexpr int LPR = D / 8;
  constexpr int CH = 64 * D / 512;
  constexpr int ROWS_PER_IT = 64 / LPR;
  constexpr int NG = KEY ? 4 : 16;
  const int lane = threadIdx.x & 63;
  const int w = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= n_blocks) return;
  const int h = blockIdx.y, b = blockIdx.z, H = gridDim.y;
  const int col = (lane % LPR) * 8;
  const int row0 = lane / LPR;
  auto group_of = [](int r) { return KEY ? (r % 8) / 2 : (r / 32) * 8 + r % 8; };

  float mv[8];
  if constexpr (MEAN) {
    const v4i m = *reinterpret_cast<const v4i*>(mean + b * ms_b + h * ms_h + col);
#pragma unroll
    for (int j = 0; j < 4; j++) {
      mv[2 * j] = F16x<DT>::to_f32((unsigned short)(m[j] & 0xffff));
      mv[2 * j + 1] = F16x<DT>::to_f32((unsigned short)((unsigned)m[j] >> 16));
    }
  }
  const unsigned short* xb = x + b * xs_b + h * xs_h + col;
  v4i raw[CH];
#pragma unroll
  for (int i = 0; i < CH; i++) {
    const int tok = w * 64 + i * ROWS_PER_IT + row0;
    raw[i] = (tok < N) ? __builtin_nontemporal_load(reinterpret_cast<const v4i*>(xb + (int64_t)tok * xs_n))
                       : v4i{0, 0, 0, 0};
  }
  auto value = [&](int i, int j) -> float {
    float f = elem16_to_f32<DT>(raw[i], j);
    if constexpr (MEAN) f -= mv[j];
    return f;
  };
  // this lane's maximum per chunk, then per group over the wave
  float cmax[CH];
#pragma unroll
  for (int i = 0; i < CH; i++) {
    const int tok = w * 64 + i * ROWS_PER_IT + row0;
    cmax[i] = 0.f;
    if (tok < N) {
#pragma unroll
      for (int j = 0; j < 8; j++) cmax[i] = fmaxf(cmax[i], fabsf(value(i, j)));
    }
  }
  float inv[CH];
#pragma unroll
  for (int g = 0; g < NG; g++) {
    float a = 0.0000001f;
#pragma unroll
    for (int i = 0; i < CH; i++)
      if (group_of(i * ROWS_PER_IT + row0) == g) a = fmaxf(a, cmax[i]);
    a = wave_max(a);
    if (lane == 0) scale[((int64_t)b * H + h) * ((int64_t)n_blocks * NG) + (int64_t)w * NG + g] = a / 127.0f;
#pragma unroll
    for (int i = 0; i < CH; i++)
      if (group_of(i * ROWS_PER_IT + row0) == g) inv[i] = 127.0f / a;
  }
  int8_t* ob = out + b * os_b + h * os_h + col;
#pragma unroll
  for (int i = 0; i < CH; i++) {
    const int tok = w * 64 + i * ROWS_PER_IT + row0;
    float y[8];
#pragma unroll
    for (int j = 0; j < 8; j++) y[j] = value(i, j) * inv[i];
    if (tok < N)
      __builtin_nontemporal_store(
          v2i{(int)pack4_rint_i8(y[0], y[1], y[2], y[3]), (int)pack4_rint_i8(y[4], y[5], y[6], y[7])},
          reinterpret_cast<v2i*>(ob + (int64_t)tok * os_n));
  }
}

template <int DT, int D, int G>
static int launch_quant(const void* x, const void* mean, int8_t* out, float* scale, int B, int H, int N,
                        int n_groups, int64_t xs_b, int64_t xs_h, int64_t xs_n, int64_t ms_b, int64_t ms_h,
                        int64_t os_b, int64_t os_h, int64_t os_n, int64_t ss_b, int64_t ss_h,
                        int has_sm_scale, float sm_scale, hipStream_t st) {
  dim3 grid(ceil_div(n_groups, 4), H, B), block(256);
  const unsigned short* xp = (const unsigned short*)x;
  const unsigned short* mp = (const unsigned short*)mean;
#define PARO_Q_LAUNCH(M, S)                                                                          \
  hipLaunchKernelGGL((quant_int8_kernel<DT, D, G, M, S>), grid, block, 0, st, xp, mp, out, scale, N, \
                     n_groups, xs_b, xs_h, xs_n, ms_b, ms_h, os_b, os_h, os_n, ss_b, ss_h, sm_scale)
  if (mean && has_sm_scale) PARO_Q_LAUNCH(true, true);
  else if (mean) PARO_Q_LAUNCH(true, false);
  else if (has_sm_scale) PARO_Q_LAUNCH(false, true);
  else PARO_Q_LAUNCH(false, false);
#undef PARO_Q_LAUNCH
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}

template <int DT, int D>
static int dispatch_group(int group, const void* x, const void* mean, int8_t* out, float* scale, int B, int H,
                          int N, int n_groups, int64_t xs_b, int64_t xs_h, int64_t xs_n, int64_t ms_b,
                          int64_t ms_h, int64_t os_b, int64_t os_h, int64_t os_n, int64_t ss_b, int64_t ss_h,
                          int has_sm_scale, float sm_scale, hipStream_t st) {
#define PARO_G(GV)                                                                                          \
  case GV:                                                                                                  \
    return launch_quant<DT, D, GV>(x, mean, out, scale, B, H, N, n_groups, xs_b, xs_h, xs_n, ms_b, ms_h,    \
                                   os_b, os_h, os_n, ss_b, ss_h, has_sm_scale, sm_scale, st)
  switch (group) {
    PARO_G(16);
    PARO_G(32);
    PARO_G(64);
    PARO_G(128);
    default:
      PARO_FAIL(PARO_ERR_INVALID_VALUE, "Unsupported block size: %d", group);
  }
#undef PARO_G
}

}  // namespace paro

extern "C" int paro_quant_int8(const void* x, int dtype, const void* mean, int8_t* out, float* scale, int B,
                               int H, int N, int D, int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_n,
                               int64_t mean_stride_b, int64_t mean_stride_h, int64_t out_stride_b,
                               int64_t out_stride_h, int64_t out_stride_n, int64_t scale_stride_b,
                               int64_t scale_stride_h, int group, int n_groups, int has_sm_scale,
                               float sm_scale, void* stream) {
  using namespace paro;
  PARO_CHECK(x && out && scale, PARO_ERR_RUNTIME, "paro_quant_int8: null tensor pointer");
  PARO_CHECK(B > 0 && H > 0 && N > 0 && n_groups > 0, PARO_ERR_RUNTIME, "paro_quant_int8: empty shape");
  PARO_CHECK(B <= MAX_GRID_YZ && H <= MAX_GRID_YZ, PARO_ERR_RUNTIME, "paro_quant_int8: batch or head count exceeds %d",
             MAX_GRID_YZ);
  PARO_CHECK(D == 64 || D == 128, PARO_ERR_INVALID_VALUE, "Unsupported head dim: %d", D);
  PARO_CHECK(dtype == PARO_DTYPE_F16 || dtype == PARO_DTYPE_BF16, PARO_ERR_RUNTIME,
             "Unsupported input dtype (expect float16 or bfloat16)");
  PARO_CHECK((int64_t)n_groups * group >= N, PARO_ERR_RUNTIME,
             "paro_quant_int8: %d groups of %d tokens do not cover %d tokens", n_groups, group, N);
  PARO_CHECK(x_stride_n % 8 == 0 && x_stride_h % 8 == 0 && x_stride_b % 8 == 0 && ((uintptr_t)x % 16) == 0,
             PARO_ERR_RUNTIME, "Tensor input must be 16-byte aligned with strides that are multiples of 8");
  PARO_CHECK(out_stride_n % 8 == 0 && out_stride_h % 8 == 0 && out_stride_b % 8 == 0 && ((uintptr_t)out % 8) == 0,
             PARO_ERR_RUNTIME, "Tensor output must be 8-byte aligned with strides that are multiples of 8");
  if (mean)
    PARO_CHECK(mean_stride_h % 8 == 0 && mean_stride_b % 8 == 0 && ((uintptr_t)mean % 16) == 0, PARO_ERR_RUNTIME,
               "Tensor mean must be 16-byte aligned with strides that are multiples of 8");
  hipStream_t st = (hipStream_t)stream;
#define PARO_D(DTV, DV)                                                                                        \
  return dispatch_group<DTV, DV>(group, x, mean, out, scale, B, H, N, n_groups, x_stride_b, x_stride_h,        \
                                 x_stride_n, mean_stride_b, mean_stride_h, out_stride_b, out_stride_h,         \
                                 out_stride_n, scale_stride_b, scale_stride_h, has_sm_scale, sm_scale, st)
  if (dtype == PARO_DTYPE_F16) {
    if (D == 64) PARO_D(PARO_DTYPE_F16, 64);
    PARO_D(PARO_DTYPE_F16, 128);
  } else {
    if (D == 64) PARO_D(PARO_DTYPE_BF16, 64);
    PARO_D(PARO_DTYPE_BF16, 128);
  }
#undef PARO_D
}

extern "C" int paro_quant_int8_per_thread(const void* x, int dtype, const void* mean, int8_t* out, float* scale, int B,
                                          int H, int N, int D, int64_t x_stride_b, int64_t x_stride_h,
                                          int64_t x_stride_n, int64_t mean_stride_b, int64_t mean_stride_h,
                                          int64_t out_stride_b, int64_t out_stride_h, int64_t out_stride_n,
                                          int is_key, void* stream) {
  using namespace paro;
  PARO_CHECK(x && out && scale, PARO_ERR_RUNTIME, "paro_quant_int8_per_thread: null tensor pointer");
  PARO_CHECK(B > 0 && H > 0 && N > 0, PARO_ERR_RUNTIME, "paro_quant_int8_per_thread: empty shape");
  PARO_CHECK(B <= MAX_GRID_YZ && H <= MAX_GRID_YZ, PARO_ERR_RUNTIME,
             "paro_quant_int8_per_thread: batch or head count exceeds %d", MAX_GRID_YZ);
  PARO_CHECK(D == 64 || D == 128, PARO_ERR_INVALID_VALUE, "Unsupported head dim: %d", D);
  PARO_CHECK(dtype == PARO_DTYPE_F16 || dtype == PARO_DTYPE_BF16, PARO_ERR_RUNTIME,
             "Unsupported input dtype (expect float16 or bfloat16)");
  PARO_CHECK(is_key == 0 || is_key == 1, PARO_ERR_INVALID_VALUE, "is_key must be 0 or 1");
  PARO_CHECK(x_stride_n % 8 == 0 && x_stride_h % 8 == 0 && x_stride_b % 8 == 0 && ((uintptr_t)x % 16) == 0,
             PARO_ERR_RUNTIME, "Tensor input must be 16-byte aligned with strides that are multiples of 8");
  PARO_CHECK(out_stride_n % 8 == 0 && out_stride_h % 8 == 0 && out_stride_b % 8 == 0 && ((uintptr_t)out % 8) == 0,
             PARO_ERR_RUNTIME, "Tensor output must be 8-byte aligned with strides that are multiples of 8");
  if (mean)
    PARO_CHECK(mean_stride_h % 8 == 0 && mean_stride_b % 8 == 0 && ((uintptr_t)mean % 16) == 0, PARO_ERR_RUNTIME,
               "Tensor mean must be 16-byte aligned with strides that are multiples of 8");
  hipStream_t st = (hipStream_t)stream;
  const int n_blocks = ceil_div(N, 64);
  dim3 grid(ceil_div(n_blocks, 4), H, B), block(256);
  const unsigned short* xp = (const unsigned short*)x;
  const unsigned short* mp = (const unsigned short*)mean;
#define PARO_QT(DTV, DV, KV, MV)                                                                                  \
  hipLaunchKernelGGL((quant_int8_per_thread_kernel<DTV, DV, KV, MV>), grid, block, 0, st, xp, mp, out, scale, N, \
                     n_blocks, x_stride_b, x_stride_h, x_stride_n, mean_stride_b, mean_stride_h, out_stride_b,   \
                     out_stride_h, out_stride_n)
#define PARO_QT_KM(DTV, DV)                                  \
  do {                                                       \
    if (is_key && mean) PARO_QT(DTV, DV, true, true);        \
    else if (is_key) PARO_QT(DTV, DV, true, false);          \
    else if (mean) PARO_QT(DTV, DV, false, true);            \
    else PARO_QT(DTV, DV, false, false);                     \
  } while (0)
  if (dtype == PARO_DTYPE_F16) {
    if (D == 64) PARO_QT_KM(PARO_DTYPE_F16, 64); else PARO_QT_KM(PARO_DTYPE_F16, 128);
  } else {
    if (D == 64) PARO_QT_KM(PARO_DTYPE_BF16, 64); else PARO_QT_KM(PARO_DTYPE_BF16, 128);
  }
#undef PARO_QT_KM
#undef PARO_QT
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}
