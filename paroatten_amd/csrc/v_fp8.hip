// V -> FP8 (e4m3fn) per-channel quantisation with mean smoothing, written in the fragment order
// of the P.V MFMA (v_mfma_f32_32x32x64_f8f6f4) so that the attention kernel's K-loop copies V
// tiles straight from HBM to LDS and reads each A operand as one contiguous 16-byte piece per lane.
//
// Three launches, all HBM-bound and deterministic (no float atomics):
//   v_stats    : per V_CHUNK-token chunk, per channel: sum, min, max      (reads V once)
//   v_finalize : per (b,h,channel): mean = sum/N, amax = max(max-mean, mean-min), scale = amax/448,
//                recp = 448/amax
//   v_pack     : per 64-token tile: (v-mean)*recp -> e4m3, fragment order  (reads V once more), and the
//                tile's rounding residual sums per channel
//   v_residual : per (b,h,channel): v_mean += scale * (sum of residuals) / N
// The last step removes the mean error of the codes: rounding (v-mean)/scale to e4m3 is unbiased only if
// the values are spread evenly over the rounding cells, and 16-bit inputs (bfloat16 above all, with its 8
// significant bits) are a lattice that is not; what is left, ~3e-4 of max|v| per channel, does not
// average out over the keys of an attention row, whereas the rounding noise does.
// max|v-mean| over tokens equals max(max-mean, mean-min) exactly because fp32 subtraction is
// monotonic, so no second reduction pass is needed.
// Arithmetic follows MeanScaleKernel of the reference (csrc/fused/fused.cu:316-427) except that the
// mean divides by the true token count.
#include "stats_device.hpp"

namespace paro {

template <int DT, int D>
__global__ void __launch_bounds__(256) v_stats_kernel(const unsigned short* __restrict__ v,
                                                      float* __restrict__ partial, int N, int n_chunks,
                                                      int64_t vs_b, int64_t vs_h, int64_t vs_n) {
  v_stats_body<DT, D>(v, partial, N, n_chunks, vs_b, vs_h, vs_n, blockIdx.x, blockIdx.y, blockIdx.z, gridDim.y);
}

template <int D>
__global__ void __launch_bounds__(1024) v_finalize_kernel(float* partial, float* __restrict__ v_scale,
                                                          float* __restrict__ v_mean, int N, int n_chunks,
                                                          int smooth) {
  v_finalize_body<D>(partial, v_scale, v_mean, N, n_chunks, smooth, blockIdx.x);
}

template <int DT, int D>
__global__ void __launch_bounds__(256) v_pack_kernel(const unsigned short* __restrict__ v,
                                                     uint8_t* __restrict__ v8,
                                                     const float* __restrict__ v_recp,
                                                     const float* __restrict__ v_mean, float* __restrict__ resid,
                                                     int N, int nb, int n_chunks,
                                                     int64_t vs_b, int64_t vs_h, int64_t vs_n) {
  constexpr int LPR = D / 8;
  constexpr int ROWS = 256 / LPR;
  constexpr int PITCH = D + 8;  // 16-bit elements; +16 bytes keeps rows on different banks
  __shared__ unsigned short tile[64 * PITCH];
  const int t = threadIdx.x;
  const int kb = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int64_t bh = (int64_t)b * gridDim.y + h;
  const int col = (t % LPR) * 8;
  const unsigned short* vb = v + b * vs_b + h * vs_h + col;
#pragma unroll
  for (int r = t / LPR; r < 64; r += ROWS) {
    const int tok = kb * 64 + r;
    const v4i raw = (tok < N) ? __builtin_nontemporal_load(reinterpret_cast<const v4i*>(vb + (int64_t)tok * vs_n))
                              : v4i{0, 0, 0, 0};
    *reinterpret_cast<v4i*>(&tile[r * PITCH + col]) = raw;
  }
  __syncthreads();
  float rs[D / 64];
  pack_v_tile<DT, D, PITCH>(tile, v8 + (bh * nb + kb) * (int64_t)(64 * D), v_recp + v_recp_offset(bh, n_chunks, D),
                            v_mean ? v_mean + bh * D : nullptr, kb * 64, N, t, rs);
  if (resid != nullptr && (t & 63) < 32) {
    const int wave = t >> 6;
#pragma unroll
    for (int n = 0; n < D / 64; n++)
      resid[((bh * nb + kb) * 2 + (wave & 1)) * D + 32 * ((wave >> 1) + 2 * n) + (t & 31)] = rs[n];
  }
}

// v_mean += v_scale * (sum over tiles and row tiles of the residual sums) / N.  A thread takes four
// channels of every SL-th row (16-byte loads, all independent), the SL partial sums per channel are
// combined through LDS in a fixed order.
template <int D>
__global__ void __launch_bounds__(1024) v_residual_kernel(const float* __restrict__ resid,
                                                          const float* __restrict__ v_scale,
                                                          float* __restrict__ v_mean, int N, int n_rows) {
  constexpr int C4 = D / 4;          // threads per row
  constexpr int SL = 1024 / C4;      // rows in flight per pass
  __shared__ v4f red[SL][C4];
  const int c4 = threadIdx.x % C4, sl = threadIdx.x / C4;
  const int64_t bh = blockIdx.x;
  const v4f* p = reinterpret_cast<const v4f*>(resid + bh * n_rows * D) + c4;
  v4f s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int r = sl; r < n_rows; r += SL) s += p[(int64_t)r * C4];
  red[sl][c4] = s;
  __syncthreads();
  if (threadIdx.x < D) {
    const int ch = threadIdx.x;
    float t = 0.f;
    for (int i = 0; i < SL; i++) t += red[i][ch >> 2][ch & 3];
    v_mean[bh * D + ch] += v_scale[bh * D + ch] * (t / (float)N);
  }
}

int v_fp8_add_residual(const float* resid, const float* v_scale, float* v_mean, int B, int Hkv, int N, int D,
                       hipStream_t st) {
  const int n_rows = ceil_div(N, 64) * 2;
  if (D == 64)
    hipLaunchKernelGGL((v_residual_kernel<64>), dim3(B * Hkv), dim3(1024), 0, st, resid, v_scale, v_mean, N, n_rows);
  else
    hipLaunchKernelGGL((v_residual_kernel<128>), dim3(B * Hkv), dim3(1024), 0, st, resid, v_scale, v_mean, N, n_rows);
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}

template <int DT, int D>
static int run_v_stats(const void* v, float* v_scale, float* v_mean, float* partial, int B, int Hkv, int N,
                       int64_t vs_b, int64_t vs_h, int64_t vs_n, int smooth, hipStream_t st) {
  const int n_chunks = ceil_div(N, V_CHUNK);
  hipLaunchKernelGGL((v_stats_kernel<DT, D>), dim3(n_chunks, Hkv, B), dim3(256), 0, st, (const unsigned short*)v,
                     partial, N, n_chunks, vs_b, vs_h, vs_n);
  PARO_HIP(hipGetLastError());
  hipLaunchKernelGGL((v_finalize_kernel<D>), dim3(B * Hkv), dim3(1024), 0, st, partial, v_scale, v_mean, N,
                     n_chunks, smooth);
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}

int v_fp8_stats(const void* v, int dtype, float* v_scale, float* v_mean, float* partial, int B, int Hkv, int N,
                int D, int64_t vs_b, int64_t vs_h, int64_t vs_n, int smooth, hipStream_t st) {
  if (dtype == PARO_DTYPE_F16) {
    if (D == 64) return run_v_stats<PARO_DTYPE_F16, 64>(v, v_scale, v_mean, partial, B, Hkv, N, vs_b, vs_h, vs_n, smooth, st);
    return run_v_stats<PARO_DTYPE_F16, 128>(v, v_scale, v_mean, partial, B, Hkv, N, vs_b, vs_h, vs_n, smooth, st);
  }
  if (D == 64) return run_v_stats<PARO_DTYPE_BF16, 64>(v, v_scale, v_mean, partial, B, Hkv, N, vs_b, vs_h, vs_n, smooth, st);
  return run_v_stats<PARO_DTYPE_BF16, 128>(v, v_scale, v_mean, partial, B, Hkv, N, vs_b, vs_h, vs_n, smooth, st);
}

template <int DT, int D>
static int run_v_pack(const void* v, uint8_t* v8, float* partial, float* v_scale, float* v_mean, int B, int Hkv,
                      int N, int64_t vs_b, int64_t vs_h, int64_t vs_n, hipStream_t st) {
  const int nb = ceil_div(N, 64), n_chunks = ceil_div(N, V_CHUNK);
  // without smoothing there is no mean to correct
  float* resid = v_mean ? partial + v_resid_offset((int64_t)B * Hkv, n_chunks, D) : nullptr;
  hipLaunchKernelGGL((v_pack_kernel<DT, D>), dim3(nb, Hkv, B), dim3(256), 0, st, (const unsigned short*)v, v8,
                     partial, v_mean, resid, N, nb, n_chunks, vs_b, vs_h, vs_n);
  PARO_HIP(hipGetLastError());
  if (resid) return v_fp8_add_residual(resid, v_scale, v_mean, B, Hkv, N, D, st);
  return PARO_OK;
}

// out_f16 = fp16(v - mean): SubMeanKernel of the reference (csrc/fused/fused.cu:200-260); for bf16
// input the subtraction is rounded to bf16 before the conversion to fp16, as there.
template <int DT, int D>
__global__ void __launch_bounds__(256) sub_mean_kernel(const unsigned short* __restrict__ v,
                                                       const unsigned short* __restrict__ mean,
                                                       unsigned short* __restrict__ out, int N, int64_t vs_b,
                                                       int64_t vs_h, int64_t vs_n, int64_t ms_b, int64_t ms_h,
                                                       int64_t os_b, int64_t os_h, int64_t os_n) {
  constexpr int LPR = D / 8;
  const int t = threadIdx.x;
  const int tok = blockIdx.x * (256 / LPR) + t / LPR;
  if (tok >= N) return;
  const int h = blockIdx.y, b = blockIdx.z, col = (t % LPR) * 8;
  const v4i raw = *reinterpret_cast<const v4i*>(v + b * vs_b + h * vs_h + (int64_t)tok * vs_n + col);
  const v4i mr = *reinterpret_cast<const v4i*>(mean + b * ms_b + h * ms_h + col);
  v4i o;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    unsigned short r2[2];
#pragma unroll
    for (int q = 0; q < 2; q++) {
      const unsigned short xv = (unsigned short)(((unsigned)raw[j] >> (16 * q)) & 0xffffu);
      const unsigned short mv = (unsigned short)(((unsigned)mr[j] >> (16 * q)) & 0xffffu);
      float d = F16x<DT>::to_f32(xv) - F16x<DT>::to_f32(mv);
      if constexpr (DT == PARO_DTYPE_BF16) d = F16x<PARO_DTYPE_BF16>::to_f32(F16x<PARO_DTYPE_BF16>::from_f32(d));
      r2[q] = F16x<PARO_DTYPE_F16>::from_f32(d);
    }
    o[j] = (int)((unsigned)r2[0] | ((unsigned)r2[1] << 16));
  }
  *reinterpret_cast<v4i*>(out + b * os_b + h * os_h + (int64_t)tok * os_n + col) = o;
}

}  // namespace paro

extern "C" int64_t paro_v_fp8_bytes(int B, int Hkv, int N, int D) {
  return (int64_t)B * Hkv * paro::ceil_div(N, 64) * 64 * D;
}
extern "C" int64_t paro_v_fp8_partial_floats(int B, int Hkv, int N, int D) {
  // statistics partials (sum, min, max per chunk and channel), then the residual sums per row tile
  return (int64_t)B * Hkv * ((int64_t)paro::ceil_div(N, paro::V_CHUNK) * 3 + (int64_t)paro::ceil_div(N, 64) * 2) * D;
}

extern "C" int paro_v_fp8_pack(const void* v, int dtype, uint8_t* v8, float* v_scale, float* v_mean,
                               float* partial, int B, int Hkv, int N, int D, int64_t v_stride_b,
                               int64_t v_stride_h, int64_t v_stride_n, int smooth, void* stream) {
  using namespace paro;
  PARO_CHECK(v && v8 && v_scale && partial, PARO_ERR_RUNTIME, "paro_v_fp8_pack: null tensor pointer");
  PARO_CHECK(!smooth || v_mean, PARO_ERR_RUNTIME, "paro_v_fp8_pack: smoothing needs a v_mean buffer");
  PARO_CHECK(B > 0 && Hkv > 0 && N > 0, PARO_ERR_RUNTIME, "paro_v_fp8_pack: empty shape");
  PARO_CHECK(B <= MAX_GRID_YZ && Hkv <= MAX_GRID_YZ, PARO_ERR_RUNTIME, "paro_v_fp8_pack: batch or head count exceeds %d",
             MAX_GRID_YZ);
  PARO_CHECK(D == 64 || D == 128, PARO_ERR_INVALID_VALUE, "Unsupported head dim: %d", D);
  PARO_CHECK(dtype == PARO_DTYPE_F16 || dtype == PARO_DTYPE_BF16, PARO_ERR_RUNTIME,
             "Unsupported input dtype (expect float16 or bfloat16)");
  PARO_CHECK(v_stride_n % 8 == 0 && v_stride_h % 8 == 0 && v_stride_b % 8 == 0 && ((uintptr_t)v % 16) == 0,
             PARO_ERR_RUNTIME, "Tensor value must be 16-byte aligned with strides that are multiples of 8");
  PARO_CHECK(((uintptr_t)v8 % 16) == 0, PARO_ERR_RUNTIME, "paro_v_fp8_pack: v8 must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (int rc = v_fp8_stats(v, dtype, v_scale, v_mean, partial, B, Hkv, N, D, v_stride_b, v_stride_h, v_stride_n,
                           smooth, st))
    return rc;
  float* mean = smooth ? v_mean : nullptr;
  if (dtype == PARO_DTYPE_F16) {
    if (D == 64) return run_v_pack<PARO_DTYPE_F16, 64>(v, v8, partial, v_scale, mean, B, Hkv, N, v_stride_b, v_stride_h, v_stride_n, st);
    return run_v_pack<PARO_DTYPE_F16, 128>(v, v8, partial, v_scale, mean, B, Hkv, N, v_stride_b, v_stride_h, v_stride_n, st);
  }
  if (D == 64) return run_v_pack<PARO_DTYPE_BF16, 64>(v, v8, partial, v_scale, mean, B, Hkv, N, v_stride_b, v_stride_h, v_stride_n, st);
  return run_v_pack<PARO_DTYPE_BF16, 128>(v, v8, partial, v_scale, mean, B, Hkv, N, v_stride_b, v_stride_h, v_stride_n, st);
}

extern "C" int paro_sub_mean(const void* v, int dtype, const void* mean, void* out_f16, int B, int H, int N,
                             int D, int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_n,
                             int64_t mean_stride_b, int64_t mean_stride_h, int64_t out_stride_b,
                             int64_t out_stride_h, int64_t out_stride_n, void* stream) {
  using namespace paro;
  PARO_CHECK(v && mean && out_f16, PARO_ERR_RUNTIME, "paro_sub_mean: null tensor pointer");
  PARO_CHECK(B > 0 && H > 0 && N > 0 && B <= MAX_GRID_YZ && H <= MAX_GRID_YZ, PARO_ERR_RUNTIME,
             "paro_sub_mean: empty shape, or batch or head count above %d", MAX_GRID_YZ);
  PARO_CHECK(D == 64 || D == 128, PARO_ERR_INVALID_VALUE, "Unsupported head dim: %d", D);
  PARO_CHECK(dtype == PARO_DTYPE_F16 || dtype == PARO_DTYPE_BF16, PARO_ERR_RUNTIME,
             "Unsupported input dtype (expect float16 or bfloat16)");
  PARO_CHECK(v_stride_n % 8 == 0 && v_stride_h % 8 == 0 && v_stride_b % 8 == 0 && out_stride_n % 8 == 0 &&
                 out_stride_h % 8 == 0 && out_stride_b % 8 == 0 && mean_stride_b % 8 == 0 && mean_stride_h % 8 == 0 &&
                 ((uintptr_t)v % 16) == 0 && ((uintptr_t)out_f16 % 16) == 0 && ((uintptr_t)mean % 16) == 0,
             PARO_ERR_RUNTIME, "paro_sub_mean: tensors must be 16-byte aligned with strides that are multiples of 8");
  hipStream_t st = (hipStream_t)stream;
  const int rows = 256 / (D / 8);
  dim3 grid(ceil_div(N, rows), H, B), block(256);
#define PARO_SM(DTV, DV)                                                                                      \
  hipLaunchKernelGGL((sub_mean_kernel<DTV, DV>), grid, block, 0, st, (const unsigned short*)v,                \
                     (const unsigned short*)mean, (unsigned short*)out_f16, N, v_stride_b, v_stride_h,        \
                     v_stride_n, mean_stride_b, mean_stride_h, out_stride_b, out_stride_h, out_stride_n)
  if (dtype == PARO_DTYPE_F16) {
    if (D == 64) PARO_SM(PARO_DTYPE_F16, 64); else PARO_SM(PARO_DTYPE_F16, 128);
  } else {
    if (D == 64) PARO_SM(PARO_DTYPE_BF16, 64); else PARO_SM(PARO_DTYPE_BF16, 128);
  }
#undef PARO_SM
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}
