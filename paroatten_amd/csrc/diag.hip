// Measurement aid: what the matrix pipe of this GPU sustains by itself.
//
// Back-to-back MFMAs of the two kinds the attention kernel issues (v_mfma_i32_32x32x32_i8 for Q.K^T,
// v_mfma_f32_32x32x64_f8f6f4 for P.V), four independent accumulators per wave, no memory traffic and no
// VALU work inside the loop, operands taken once from a caller-supplied buffer (random bytes or zeros: the
// shader clock under a power cap depends on how much the operands toggle).  bench.py --mfma-ceiling times
// it; the figure is the ceiling any kernel built on these instructions has on the box it runs on.
//
// Second aid: a proxy of the attention kernel's loop body at D = 64, built up in four levels, each adding
// one ingredient of the real loop to the same instruction mix per wave and iteration (4 x i32_32x32x32_i8,
// 2 x f32_32x32x64 f8, 1 x f32_16x16x128 f8; 32 fma with clamp, 16 v_cvt_pknorm_i16_f32, 8 v_perm_b32, 8 and):
//   0  operands in registers, the same every iteration
//   1  + K/V fragments read from LDS every iteration (8 x ds_read_b128, K rows swizzled as in the kernel: the
//        operands now change, full-range e4m3 bytes for V)
//   2  + the four LDS-DMA tile loads per wave and iteration, tiles visited in a scattered order taken from a
//        block list in LDS, from a buffer that stays in the L2
//   3  + one barrier per iteration
// Workgroups of two waves, three waves per SIMD, as the kernel.  bench.py --proxy-ceiling times the levels:
// what separates the kernel from the matrix pipe's own ceiling is found where the figure drops.
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

template <int LEVEL>
__global__ void __launch_bounds__(128, 3) attn_proxy_kernel(const int* __restrict__ operands,
                                                            const uint8_t* __restrict__ tiles,
                                                            float* __restrict__ sink, int iters, int ntiles) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];   // 3 stages x (4 KB K + 4 KB V), then the block list
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int l32 = lane & 31, lh = lane >> 5;
  // LDS starts out with random bytes (e4m3 NaN codes 0x7f / 0xff avoided: bit 0 cleared where bits 1..6 are set)
  for (int i = t; i < 24576 / 4; i += 128) {
    int w = operands[i & 16383];
    w &= ~((w >> 1) & (w >> 2) & (w >> 3) & (w >> 4) & (w >> 5) & (w >> 6) & 0x01010101);
    reinterpret_cast<int*>(smem)[i] = w;
  }
  // the order in which this workgroup visits the tiles: scattered, as a kept-block list is
  unsigned short* klist = reinterpret_cast<unsigned short*>(smem + 24576);
  for (int i = t; i < 512; i += 128) klist[i] = (unsigned short)((i * 37 + blockIdx.x * 11) % ntiles);
  __syncthreads();
  v4i ka[4], qb[2];
  v8i va[2], pf, ones;
#pragma unroll
  for (int j = 0; j < 4; j++)
#pragma unroll
    for (int i = 0; i < 4; i++) ka[j][i] = operands[(t * 4 + i + j * 256) & 16383];
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int i = 0; i < 4; i++) qb[j][i] = operands[(4096 + t * 4 + i + j * 64) & 16383];
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int i = 0; i < 8; i++) va[j][i] = operands[(8192 + t * 8 + i + j * 512) & 16383] & 0x3f3f3f3f;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    pf[i] = operands[(12000 + t * 8 + i) & 16383] & 0x3f3f3f3f;
    ones[i] = 0x38383838;
  }
  v16i magic;
#pragma unroll
  for (int i = 0; i < 16; i++) magic[i] = 0x4B400000;
  asm volatile("" : "+v"(magic));
  v16i acc[2] = {magic, magic};
  v16f o[2] = {};
  v4f d = {0.f, 0.f, 0.f, 0.f};
  const float c8 = 1.0e-9f, bias = 0.3f;
  // K fragment (ks, mt): row 32*mt + lane%32, 16-byte chunk 2*ks + lane/32 at its swizzled position, as the kernel
  int kr_off[4];
#pragma unroll
  for (int ks = 0; ks < 2; ks++)
#pragma unroll
    for (int mt = 0; mt < 2; mt++) {
      const int row = 32 * mt + l32;
      kr_off[ks * 2 + mt] = row * 64 + (((2 * ks + lh) ^ ((row >> 2) & 3)) * 16);
    }
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)tiles, 0, ntiles * 8192, 0x00020000);
  int tile = __builtin_amdgcn_readfirstlane((int)klist[0]);
  int st = 0;
  for (int it = 0; it < iters; it++) {
    int next_v = 0;
    if constexpr (LEVEL >= 2) {   // each wave moves half of a K and of a V tile (2 x 1 KB each) into stage st + 2
      uint8_t* dst = smem + ((st + 2) % 3) * 8192 + wave * 2048;
      const int vo = lane * 16 + wave * 2048;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dst, 16, vo, tile * 8192, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dst, 16, vo, tile * 8192, 1024, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(dst + 4096), 16, vo + 4096, tile * 8192, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(dst + 4096), 16, vo + 4096, tile * 8192, 1024, 0);
      next_v = (int)klist[(it + 1) & 511];
    }
#pragma unroll
    for (int r = 0; r < 8; r++) {
      const int mt = r >> 2, i0 = 4 * (r & 3);
      float u0, u1, u2, u3;
      asm volatile("v_fma_f32 %0, %1, %2, %3 clamp" : "=v"(u0) : "v"(__int_as_float(acc[mt][i0])), "v"(c8), "v"(bias));
      asm volatile("v_fma_f32 %0, %1, %2, %3 clamp" : "=v"(u1) : "v"(__int_as_float(acc[mt][i0 + 1])), "v"(c8), "v"(bias));
      asm volatile("v_fma_f32 %0, %1, %2, %3 clamp" : "=v"(u2) : "v"(__int_as_float(acc[mt][i0 + 2])), "v"(c8), "v"(bias));
      asm volatile("v_fma_f32 %0, %1, %2, %3 clamp" : "=v"(u3) : "v"(__int_as_float(acc[mt][i0 + 3])), "v"(c8), "v"(bias));
      int lo, hi, w;
      asm volatile("v_cvt_pknorm_i16_f32 %0, %1, %2" : "=v"(lo) : "v"(u0), "v"(u2));
      asm volatile("v_cvt_pknorm_i16_f32 %0, %1, %2" : "=v"(hi) : "v"(u1), "v"(u3));
      asm volatile("v_perm_b32 %0, %1, %2, %3" : "=v"(w) : "v"(hi), "v"(lo), "v"(0x07030501));
      pf[r] = w & 0x3f3f3f3f;
    }
    __builtin_amdgcn_sched_barrier(0);
    v4f d_new = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ones, pf, d, 0, 0, 0, 0, 0, 0);
    if constexpr (LEVEL >= 1) {   // K and V fragments of stage st (8 x 16 B per lane)
#pragma unroll
      for (int j = 0; j < 4; j++) ka[j] = *reinterpret_cast<const v4i*>(smem + st * 8192 + kr_off[j]);
      const uint8_t* vb = smem + st * 8192 + 4096 + lane * 16;
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const v4i x = *reinterpret_cast<const v4i*>(vb + (2 * j) * 1024);
        const v4i y = *reinterpret_cast<const v4i*>(vb + (2 * j + 1) * 1024);
        va[j] = v8i{x[0], x[1], x[2], x[3], y[0], y[1], y[2], y[3]};
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    // the kernel's overflow test on the row sums (never taken here: the weights are kept finite)
    if (__ballot(d_new[0] != d_new[0]) != 0ull) d_new[0] = 0.f;
    d = d_new;
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
      for (int ks = 0; ks < 2; ks++)
        acc[mt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ka[ks * 2 + mt], qb[ks], ks == 0 ? magic : acc[mt], 0, 0, 0);
#pragma unroll
    for (int j = 0; j < 2; j++) o[j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(va[j], pf, o[j], 0, 0, 0, 0, 0, 0);
    if constexpr (LEVEL >= 2) {
      tile = __builtin_amdgcn_readfirstlane(next_v);
      asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory");
    }
    if constexpr (LEVEL >= 3) __builtin_amdgcn_s_barrier();
    st = st == 2 ? 0 : st + 1;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  float s = d[0] + d[1];
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int i = 0; i < 16; i++) s += o[j][i];
#pragma unroll
  for (int i = 0; i < 16; i++) s += (float)(acc[0][i] + acc[1][i]);
  sink[blockIdx.x * 128 + t] = s;
}

}  // namespace paro

extern "C" int64_t paro_diag_attn_proxy_ops(int workgroups, int iters) {
  // counted like the attention kernel counts a block: 4 int8 products of 2*32*32*32 and 2 fp8 products of
  // 2*32*32*64 operations per wave and iteration (the row-sum product is not counted), two waves per workgroup
  return (4LL * 65536 + 2LL * 131072) * 2 * (int64_t)workgroups * iters;
}

extern "C" int paro_diag_attn_proxy(int level, const void* operands, const void* tiles, float* sink, int workgroups,
                                    int iters, int ntiles, void* stream) {
  using namespace paro;
  PARO_CHECK(level >= 0 && level <= 3, PARO_ERR_INVALID_VALUE, "paro_diag_attn_proxy: level must be 0..3");
  PARO_CHECK(operands && tiles && sink && workgroups > 0 && iters > 0 && ntiles >= 4, PARO_ERR_RUNTIME,
             "paro_diag_attn_proxy: bad arguments");
  hipStream_t st = (hipStream_t)stream;
#define PARO_PROXY(L)                                                                                             \
  hipLaunchKernelGGL((attn_proxy_kernel<L>), dim3(workgroups), dim3(128), 24576 + 1024, st, (const int*)operands,        \
                     (const uint8_t*)tiles, sink, iters, ntiles)
  if (level == 0) PARO_PROXY(0);
  else if (level == 1) PARO_PROXY(1);
  else if (level == 2) PARO_PROXY(2);
  else PARO_PROXY(3);
#undef PARO_PROXY
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}

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
