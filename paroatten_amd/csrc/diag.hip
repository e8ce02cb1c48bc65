// Measurement aid: what the matrix pipe of this GPU sustains by itself.
//
// Back-to-back MFMAs of the two kinds the attention kernel issues (v_mfma_i32_32x32x32_i8 for Q.K^T,
// v_mfma_f32_32x32x64_f8f6f4 for P.V), four independent accumulators per wave, no memory traffic and no
// VALU work inside the loop, operands taken once from a caller-supplied buffer (random bytes or zeros: the
// shader clock under a power cap depends on how much the operands toggle).  bench.py --mfma-ceiling times
// it; the figure is the ceiling any kernel built on these instructions has on the box it runs on.
#include "paro_common.hpp"

namespace paro {

template <int KIND>
__global__ void __launch_bounds__(256) mfma_loop_kernel(const int* __restrict__ operands, float* __restrict__ sink,
                                                        int iters) {
  const int lane = threadIdx.x & 63;
  // 16 words per lane of operand data, the same for every wave (the buffer holds 64 lanes x 16 words)
  int w[16];
#pragma unroll
  for (int i = 0; i < 16; i++) w[i] = operands[lane * 16 + i];
  float total = 0.f;
  if constexpr (KIND == 0) {
    const v4i a0 = {w[0], w[1], w[2], w[3]}, a1 = {w[4], w[5], w[6], w[7]};
    const v4i b0 = {w[8], w[9], w[10], w[11]}, b1 = {w[12], w[13], w[14], w[15]};
    v16i c0 = {}, c1 = {}, c2 = {}, c3 = {};
    for (int it = 0; it < iters; it++) {
      c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, b0, c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, b0, c1, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, b1, c2, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, b1, c3, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 16; i++) total += (float)(c0[i] ^ c1[i] ^ c2[i] ^ c3[i]);
  } else {
    const v8i a0 = {w[0], w[1], w[2], w[3], w[4], w[5], w[6], w[7]};
    const v8i a1 = {w[4], w[5], w[6], w[7], w[0], w[1], w[2], w[3]};
    const v8i b0 = {w[8], w[9], w[10], w[11], w[12], w[13], w[14], w[15]};
    const v8i b1 = {w[12], w[13], w[14], w[15], w[8], w[9], w[10], w[11]};
    v16f c0 = {}, c1 = {}, c2 = {}, c3 = {};
    for (int it = 0; it < iters; it++) {
      c0 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a0, b0, c0, 0, 0, 0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a1, b0, c1, 0, 0, 0, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a0, b1, c2, 0, 0, 0, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a1, b1, c3, 0, 0, 0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 16; i++) total += (c0[i] + c1[i]) + (c2[i] + c3[i]);
  }
  // one value per wave, so that the loop cannot be removed
  if (lane == 0) sink[(blockIdx.x * blockDim.x + threadIdx.x) >> 6] = total;
}

}  // namespace paro

extern "C" int64_t paro_diag_mfma_loop_ops(int kind, int workgroups, int iters) {
  // four MFMAs per iteration and wave, four waves per workgroup; 2*32*32*K operations each
  const int64_t per_mfma = kind == 0 ? 2LL * 32 * 32 * 32 : 2LL * 32 * 32 * 64;
  return per_mfma * 4 * 4 * (int64_t)workgroups * iters;
}

extern "C" int paro_diag_mfma_loop(int kind, const void* operands, float* sink, int workgroups, int iters,
                                   void* stream) {
  using namespace paro;
  PARO_CHECK(kind == 0 || kind == 1, PARO_ERR_INVALID_VALUE, "paro_diag_mfma_loop: kind must be 0 (int8) or 1 (fp8)");
  PARO_CHECK(operands && sink && workgroups > 0 && iters > 0, PARO_ERR_RUNTIME, "paro_diag_mfma_loop: bad arguments");
  hipStream_t st = (hipStream_t)stream;
  if (kind == 0)
    hipLaunchKernelGGL((mfma_loop_kernel<0>), dim3(workgroups), dim3(256), 0, st, (const int*)operands, sink, iters);
  else
    hipLaunchKernelGGL((mfma_loop_kernel<1>), dim3(workgroups), dim3(256), 0, st, (const int*)operands, sink, iters);
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}
