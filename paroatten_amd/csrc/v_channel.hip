// V preparation in the reference's own storage format (HBM-bound, gfx950):
//   transpose_pad_permute : V [.,N,D] -> [.,D,ceil64(N)], tokens >= N zero, and inside every group of 16
//                           tokens the order 0,1,8,9,2,3,10,11,4,5,12,13,6,7,14,15
//   channel_quant_fp8     : per (batch, head, channel) row of that tensor: (mean,) scale, e4m3 codes
// They stand in for TransposePadPermuteKernel and MeanScaleKernel of the reference
// (csrc/fused/fused.cu:262-313, 316-427) behind paroattention._fused's transpose_pad_permute_cuda,
// scale_fuse_quant_cuda and mean_scale_fuse_quant_cuda (fused.cu:850-1083), quirks included: statistics
// over the first ceil16(num_tokens) entries of a row (the zero padding takes part in min, max and the
// mean's divisor), codes written for the first ceil64(num_tokens) entries.  The token order inside a
// group of 16 is the operand order of NVIDIA's fp8 mma; nothing on gfx950 consumes it (this library's
// attention kernel reads the tiles of paro_v_fp8_pack), the functions exist so that callers of the
// reference's extension module find them.
#include "paro_device.hpp"

namespace paro {

// position inside a group of 16 -> token inside the group that is stored there (the inverse of
// fused.cu:287-291, which sends token r to position (r/8)*2 + ((r/2)%4)*4 + r%2)
__device__ __forceinline__ int shuffle16_token_at(int pos) { return ((pos >> 1) & 1) * 8 + (pos >> 2) * 2 + (pos & 1); }

template <int D>
__global__ void __launch_bounds__(256) transpose_pad_permute_kernel(const unsigned short* __restrict__ in,
                                                                    unsigned short* __restrict__ out, int N,
                                                                    int64_t is_b, int64_t is_h, int64_t is_n,
                                                                    int64_t os_b, int64_t os_h, int64_t os_d) {
  constexpr int LPR = D / 8;          // 16-byte pieces per token row
  constexpr int ROWS = 256 / LPR;
  constexpr int PITCH = D + 2;        // 16-bit elements: rows 8 apart land on different banks
  __shared__ unsigned short tile[64 * PITCH];
  const int t = threadIdx.x;
  const int kb = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const unsigned short* ib = in + b * is_b + h * is_h + (t % LPR) * 8;
#pragma unroll
  for (int r = t / LPR; r < 64; r += ROWS) {
    const int tok = kb * 64 + r;
    const v4i raw = tok < N ? __builtin_nontemporal_load(reinterpret_cast<const v4i*>(ib + (int64_t)tok * is_n))
                            : v4i{0, 0, 0, 0};
    // rows are 4-byte aligned only (PITCH is even, not a multiple of 8): four 4-byte stores
    unsigned* dst = reinterpret_cast<unsigned*>(&tile[r * PITCH + (t % LPR) * 8]);
#pragma unroll
    for (int j = 0; j < 4; j++) dst[j] = (unsigned)raw[j];
  }
  __syncthreads();
  unsigned short* ob = out + b * os_b + h * os_h + (int64_t)kb * 64;
#pragma unroll
  for (int n = 0; n < D / 32; n++) {   // D rows of 8 pieces of 8 tokens
    const int piece = t + 256 * n;
    const int d = piece >> 3, c8 = piece & 7;
    unsigned w[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int p0 = c8 * 8 + 2 * j, p1 = p0 + 1;
      const int r0 = (p0 & ~15) + shuffle16_token_at(p0 & 15), r1 = (p1 & ~15) + shuffle16_token_at(p1 & 15);
      w[j] = (unsigned)tile[r0 * PITCH + d] | ((unsigned)tile[r1 * PITCH + d] << 16);
    }
    __builtin_nontemporal_store(v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]},
                                reinterpret_cast<v4i*>(ob + d * os_d + c8 * 8));
  }
}

// sum / min / max of the 256 threads' values, combined in a fixed order (wave trees, then the four waves)
struct Stats { float s, mn, mx; };
__device__ __forceinline__ Stats block_stats(Stats v, float (*red)[4]) {
  auto step = [&](auto&& other) {
    Stats o = other(v);
    v.s += o.s; v.mn = fminf(v.mn, o.mn); v.mx = fmaxf(v.mx, o.mx);
  };
  step([](Stats x) { return Stats{row_dpp<0xB1>(x.s), row_dpp<0xB1>(x.mn), row_dpp<0xB1>(x.mx)}; });
  step([](Stats x) { return Stats{row_dpp<0x4E>(x.s), row_dpp<0x4E>(x.mn), row_dpp<0x4E>(x.mx)}; });
  step([](Stats x) { return Stats{row_dpp<0x124>(x.s), row_dpp<0x124>(x.mn), row_dpp<0x124>(x.mx)}; });
  step([](Stats x) { return Stats{row_dpp<0x128>(x.s), row_dpp<0x128>(x.mn), row_dpp<0x128>(x.mx)}; });
  float a, b;
  with_lane_xor16(v.s, a, b);  v.s = a + b;
  with_lane_xor16(v.mn, a, b); v.mn = fminf(a, b);
  with_lane_xor16(v.mx, a, b); v.mx = fmaxf(a, b);
  with_lane_xor32(v.s, a, b);  v.s = a + b;
  with_lane_xor32(v.mn, a, b); v.mn = fminf(a, b);
  with_lane_xor32(v.mx, a, b); v.mx = fmaxf(a, b);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) { red[0][wave] = v.s; red[1][wave] = v.mn; red[2][wave] = v.mx; }
  __syncthreads();
  return Stats{(red[0][0] + red[0][1]) + (red[0][2] + red[0][3]),
               fminf(fminf(red[1][0], red[1][1]), fminf(red[1][2], red[1][3])),
               fmaxf(fmaxf(red[2][0], red[2][1]), fmaxf(red[2][2], red[2][3]))};
}

template <int DT, bool SUB_MEAN>
__global__ void __launch_bounds__(256) channel_quant_fp8_kernel(const unsigned short* __restrict__ in,
                                                                uint8_t* __restrict__ out, float* __restrict__ mean,
                                                                float* __restrict__ scale, int num_tokens,
                                                                float scale_max, int64_t is_b, int64_t is_h,
                                                                int64_t is_d, int64_t os_b, int64_t os_h,
                                                                int64_t os_d, int64_t ms_b, int64_t ms_h,
                                                                int64_t ss_b, int64_t ss_h) {
  __shared__ float red[3][4];
  const int t = threadIdx.x;
  const int d = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const unsigned short* row = in + b * is_b + h * is_h + d * is_d;
  const int n16 = (num_tokens + 15) / 16 * 16, n64 = (num_tokens + 63) / 64 * 64;
  // the reference starts its running extremes at -/+1e6 (fused.cu:347-348)
  Stats st{0.f, 1000000.0f, -1000000.0f};
  for (int i = t * 8; i < n16; i += 2048) {
    const v4i raw = *reinterpret_cast<const v4i*>(row + i);   // read again below: ordinary load
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const float x = elem16_to_f32<DT>(raw, j);
      st.mx = fmaxf(st.mx, x);
      st.mn = fminf(st.mn, x);
      if constexpr (SUB_MEAN) st.s += x;
    }
  }
  st = block_stats(st, red);
  const float mean_v = SUB_MEAN ? st.s / (float)n16 : 0.f;
  const float amax = fmaxf(fabsf(st.mx - mean_v), fabsf(st.mn - mean_v));
  if (t == 0) {
    if constexpr (SUB_MEAN) mean[b * ms_b + h * ms_h + d] = mean_v;
    scale[b * ss_b + h * ss_h + d] = amax / scale_max;
  }
  // a constant row: the reference divides by zero here and writes NaN codes; this writes zeros
  const float recp = amax > 0.f ? scale_max / amax : 0.f;
  uint8_t* orow = out + b * os_b + h * os_h + d * os_d;
  for (int i = t * 8; i < n64; i += 2048) {
    const v4i raw = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(row + i));
    float f[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
      // e4m3 conversion saturates to the largest finite value (cvt.rn.satfinite in the reference)
      const float y = (elem16_to_f32<DT>(raw, j) - mean_v) * recp;
      f[j] = fminf(fmaxf(y, -448.0f), 448.0f);
    }
    int lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], 0, false);
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], lo, true);
    int hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], 0, false);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], hi, true);
    __builtin_nontemporal_store(v2i{lo, hi}, reinterpret_cast<v2i*>(orow + i));
  }
}

}  // namespace paro

extern "C" int paro_transpose_pad_permute(const void* in, void* out, int dtype, int B, int H, int N, int D,
                                          int64_t in_stride_b, int64_t in_stride_h, int64_t in_stride_n,
                                          int64_t out_stride_b, int64_t out_stride_h, int64_t out_stride_d,
                                          void* stream) {
  using namespace paro;
  PARO_CHECK(in && out, PARO_ERR_RUNTIME, "paro_transpose_pad_permute: null tensor pointer");
  PARO_CHECK(B > 0 && H > 0 && N > 0 && B <= MAX_GRID_YZ && H <= MAX_GRID_YZ, PARO_ERR_RUNTIME,
             "paro_transpose_pad_permute: empty shape, or batch or head count above %d", MAX_GRID_YZ);
  PARO_CHECK(D == 64 || D == 128, PARO_ERR_INVALID_VALUE, "Unsupported head dim: %d", D);
  PARO_CHECK(dtype == PARO_DTYPE_F16 || dtype == PARO_DTYPE_BF16, PARO_ERR_RUNTIME,
             "Unsupported input dtype (expect float16 or bfloat16)");
  PARO_CHECK(((uintptr_t)in % 16) == 0 && ((uintptr_t)out % 16) == 0 && in_stride_b % 8 == 0 && in_stride_h % 8 == 0 &&
                 in_stride_n % 8 == 0 && out_stride_b % 8 == 0 && out_stride_h % 8 == 0 && out_stride_d % 8 == 0,
             PARO_ERR_RUNTIME, "paro_transpose_pad_permute: tensors must be 16-byte aligned with strides that are multiples of 8");
  const int nb = ceil_div(N, 64);
  PARO_CHECK(out_stride_d >= (int64_t)nb * 64, PARO_ERR_RUNTIME,
             "paro_transpose_pad_permute: an output row must hold ceil64(num_tokens) = %d entries", nb * 64);
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(nb, H, B), block(256);
  // a copy: the 16-bit type does not matter
  if (D == 64)
    hipLaunchKernelGGL((transpose_pad_permute_kernel<64>), grid, block, 0, st, (const unsigned short*)in,
                       (unsigned short*)out, N, in_stride_b, in_stride_h, in_stride_n, out_stride_b, out_stride_h,
                       out_stride_d);
  else
    hipLaunchKernelGGL((transpose_pad_permute_kernel<128>), grid, block, 0, st, (const unsigned short*)in,
                       (unsigned short*)out, N, in_stride_b, in_stride_h, in_stride_n, out_stride_b, out_stride_h,
                       out_stride_d);
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}

extern "C" int paro_channel_quant_fp8(const void* in, int dtype, uint8_t* out, float* mean, float* scale, int B, int H,
                                      int D, int num_tokens, int row_len, float scale_max, int64_t in_stride_b,
                                      int64_t in_stride_h, int64_t in_stride_d, int64_t out_stride_b,
                                      int64_t out_stride_h, int64_t out_stride_d, int64_t mean_stride_b,
                                      int64_t mean_stride_h, int64_t scale_stride_b, int64_t scale_stride_h,
                                      void* stream) {
  using namespace paro;
  PARO_CHECK(in && out && scale, PARO_ERR_RUNTIME, "paro_channel_quant_fp8: null tensor pointer");
  PARO_CHECK(B > 0 && H > 0 && D > 0 && num_tokens > 0 && B <= MAX_GRID_YZ && H <= MAX_GRID_YZ, PARO_ERR_RUNTIME,
             "paro_channel_quant_fp8: empty shape, or batch or head count above %d", MAX_GRID_YZ);
  PARO_CHECK(dtype == PARO_DTYPE_F16 || dtype == PARO_DTYPE_BF16, PARO_ERR_RUNTIME,
             "Unsupported input dtype (expect float16 or bfloat16)");
  PARO_CHECK(scale_max > 0.f, PARO_ERR_INVALID_VALUE, "paro_channel_quant_fp8: scale_max must be positive");
  PARO_CHECK((int64_t)ceil_div(num_tokens, 64) * 64 <= row_len, PARO_ERR_RUNTIME,
             "paro_channel_quant_fp8: rows of %d entries are shorter than ceil64(num_tokens = %d)", row_len, num_tokens);
  PARO_CHECK(((uintptr_t)in % 16) == 0 && ((uintptr_t)out % 8) == 0 && in_stride_b % 8 == 0 && in_stride_h % 8 == 0 &&
                 in_stride_d % 8 == 0 && out_stride_b % 8 == 0 && out_stride_h % 8 == 0 && out_stride_d % 8 == 0,
             PARO_ERR_RUNTIME, "paro_channel_quant_fp8: tensors must be 16-byte aligned with strides that are multiples of 8");
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(D, H, B), block(256);
#define PARO_CQ(DTV, SM)                                                                                          \
  hipLaunchKernelGGL((channel_quant_fp8_kernel<DTV, SM>), grid, block, 0, st, (const unsigned short*)in, out, mean, \
                     scale, num_tokens, scale_max, in_stride_b, in_stride_h, in_stride_d, out_stride_b,           \
                     out_stride_h, out_stride_d, mean_stride_b, mean_stride_h, scale_stride_b, scale_stride_h)
  if (dtype == PARO_DTYPE_F16) {
    if (mean) PARO_CQ(PARO_DTYPE_F16, true); else PARO_CQ(PARO_DTYPE_F16, false);
  } else {
    if (mean) PARO_CQ(PARO_DTYPE_BF16, true); else PARO_CQ(PARO_DTYPE_BF16, false);
  }
#undef PARO_CQ
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}
