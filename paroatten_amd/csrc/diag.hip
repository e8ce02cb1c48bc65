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
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <type_traits>
#include "../../include/paroatten_diag.h"

namespace paro {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

static thread_local char g_diag_err[256] = "";
static int diag_fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_diag_err, sizeof(g_diag_err), fmt, ap);
  va_end(ap);
  return code;
}
#define DIAG_CHECK(cond, code, ...) do { if (!(cond)) return ::paro::diag_fail(code, __VA_ARGS__); } while (0)
#define DIAG_HIP(expr) do { hipError_t e__ = (expr); if (e__ != hipSuccess) return ::paro::diag_fail(-4, "%s failed: %s", #expr, hipGetErrorString(e__)); } while (0)

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

// Third aid: the same instruction mix arranged as the one-wave-per-q-block kernel arranges it (attn_sparse_w64.hip):
// one-wave workgroups, two per SIMD, each owning two 32-row halves A and B that are software-pipelined against
// each other (the matrix products of one half are issued between the words of weights of the other), K and V
// fragments read once per block and used by both halves, whole tiles moved by the wave through a two-stage ring.
//   LDS = false            operands constant in registers
//   LDS, READS             the 8 fragment reads per block (every read feeds two products)
//   LDS, DMA               the 8 LDS-DMA tile loads per block, two blocks ahead, scattered tile order
// V_DIRECT: V fragments (already in fragment order in memory) by buffer_load_dwordx4 straight into a second
// register set one block ahead instead of through LDS.
// clk[0], clk[1]: shader-clock cycles and 100 MHz ticks that workgroup 777 spent in its loop.
template <bool LDS, bool DMA, bool READS, bool V_DIRECT>
__global__ void __launch_bounds__(64, 2) attn_proxy_w64_kernel(const int* __restrict__ operands,
                                                                const uint8_t* __restrict__ tiles,
                                                                float* __restrict__ sink, int iters, int ntiles,
                                                                long long* __restrict__ clk) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];   // K stages 2 x 4 KB, V stages 2 x 4 KB, block list
  const int lane = threadIdx.x;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)tiles, 0, ntiles * 8192, 0x00020000);
  for (int i = lane; i < 16384 / 4; i += 64) {
    int w = operands[i & 16383];
    w &= ~((w >> 1) & (w >> 2) & (w >> 3) & (w >> 4) & (w >> 5) & (w >> 6) & 0x01010101);   // no e4m3 NaN codes
    reinterpret_cast<int*>(smem)[i] = w;
  }
  unsigned short* klist = reinterpret_cast<unsigned short*>(smem + 16384);
  for (int i = lane; i < 512; i += 64) klist[i] = (unsigned short)((i * 37 + blockIdx.x * 11) % ntiles);
  __syncthreads();
  v4i ka[4], va[2][4], qA[2], qB[2];
  v8i pfA, pfB, ones;
#pragma unroll
  for (int j = 0; j < 4; j++)
#pragma unroll
    for (int i = 0; i < 4; i++) {
      ka[j][i] = operands[(lane * 4 + i + j * 256) & 16383];
      va[0][j][i] = operands[(8192 + lane * 4 + i + j * 256) & 16383] & 0x3f3f3f3f;
      va[1][j][i] = operands[(9216 + lane * 4 + i + j * 256) & 16383] & 0x3f3f3f3f;
    }
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int i = 0; i < 4; i++) {
      qA[j][i] = operands[(4096 + lane * 4 + i + j * 64) & 16383];
      qB[j][i] = operands[(5000 + lane * 4 + i + j * 64) & 16383];
    }
#pragma unroll
  for (int i = 0; i < 8; i++) {
    pfA[i] = operands[(12000 + lane * 8 + i) & 16383] & 0x3f3f3f3f;
    pfB[i] = operands[(13000 + lane * 8 + i) & 16383] & 0x3f3f3f3f;
    ones[i] = 0x38383838;
  }
  v16i magic;
#pragma unroll
  for (int i = 0; i < 16; i++) magic[i] = 0x4B400000;
  asm volatile("" : "+v"(magic));
  v16i accA[2] = {magic, magic}, accB[2] = {magic, magic};
  v16f oA[2] = {}, oB[2] = {};
  v4f dA = {0.f, 0.f, 0.f, 0.f}, dB = {0.f, 0.f, 0.f, 0.f};
  const float c8 = 1.0e-9f, bias = 0.3f;
  const int l32 = lane & 31, lh = lane >> 5;
  int kr_off[4];
#pragma unroll
  for (int ks = 0; ks < 2; ks++)
#pragma unroll
    for (int mt = 0; mt < 2; mt++) {
      const int row = 32 * mt + l32;
      kr_off[ks * 2 + mt] = row * 64 + (((2 * ks + lh) ^ ((row >> 2) & 3)) * 16);
    }
  int t1 = __builtin_amdgcn_readfirstlane((int)klist[0]), t2 = __builtin_amdgcn_readfirstlane((int)klist[1]);
  int t3 = __builtin_amdgcn_readfirstlane((int)klist[2]);

  auto word = [&](const v16i (&acc)[2], v8i& pf, int r) {   // four weights: 4 fma with clamp, 2 pknorm, 1 perm
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
  };
  // S_new = K.Q (4 int8 products into accN), O += V.P (2 fp8 products with pfO) between the words of accW -> pfW
  auto phase = [&](const v4i (&vf)[4], const v4i (&q)[2], v16i (&accN)[2], v16f (&o)[2], const v8i& pfO,
                   const v16i (&accW)[2], v8i& pfW, v4f& dW) {
    accN[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ka[0], q[0], magic, 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0); word(accW, pfW, 0); __builtin_amdgcn_sched_barrier(0);
    accN[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ka[1], q[0], magic, 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0); word(accW, pfW, 1); __builtin_amdgcn_sched_barrier(0);
    accN[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ka[2], q[1], accN[0], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0); word(accW, pfW, 2); __builtin_amdgcn_sched_barrier(0);
    accN[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ka[3], q[1], accN[1], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0); word(accW, pfW, 3); __builtin_amdgcn_sched_barrier(0);
    o[0] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
        v8i{vf[0][0], vf[0][1], vf[0][2], vf[0][3], vf[1][0], vf[1][1], vf[1][2], vf[1][3]}, pfO, o[0], 0, 0, 0, 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0); word(accW, pfW, 4); word(accW, pfW, 5); __builtin_amdgcn_sched_barrier(0);
    o[1] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
        v8i{vf[2][0], vf[2][1], vf[2][2], vf[2][3], vf[3][0], vf[3][1], vf[3][2], vf[3][3]}, pfO, o[1], 0, 0, 0, 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0); word(accW, pfW, 6); word(accW, pfW, 7); __builtin_amdgcn_sched_barrier(0);
    dW = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ones, pfW, dW, 0, 0, 0, 0, 0, 0);
    if (__ballot(dW[0] != dW[0]) != 0ull) dW[0] = 0.f;   // the kernel's overflow test (never taken: the weights stay finite)
  };
  // one block; CUR: register set that holds V(i), the other one receives V(i+1) when V comes straight from memory
  auto body = [&](int it, auto curc) {
    constexpr int CUR = decltype(curc)::value, NXT = V_DIRECT ? 1 - CUR : CUR;
    const int s_new = it & 1;
    constexpr int NDMA = (LDS && DMA) ? (V_DIRECT ? 4 : 8) : 0;
    if constexpr (V_DIRECT) {   // (issued first: waited for at the end of this block, the DMA two blocks later)
#pragma unroll
      for (int j = 0; j < 4; j++)
        va[NXT][j] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane * 16 + 4096 + j * 1024, t1 * 8192, 0));
    }
    if constexpr (LDS && DMA) {
      uint8_t* dk = smem + s_new * 4096;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dk, 16, lane * 16, t3 * 8192, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dk, 16, lane * 16, t3 * 8192, 1024, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dk, 16, lane * 16, t3 * 8192, 2048, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dk, 16, lane * 16, t3 * 8192, 3072, 0);
      if constexpr (!V_DIRECT) {
        uint8_t* dv = smem + 8192 + s_new * 4096;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dv, 16, lane * 16 + 4096, t2 * 8192, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dv, 16, lane * 16 + 4096, t2 * 8192, 1024, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dv, 16, lane * 16 + 4096, t2 * 8192, 2048, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dv, 16, lane * 16 + 4096, t2 * 8192, 3072, 0);
      }
    }
    const int next_t = (int)klist[(it + 3) & 511];
    __builtin_amdgcn_sched_barrier(0);
    phase(va[CUR], qA, accA, oA, pfA, accB, pfB, dB);
    __builtin_amdgcn_sched_barrier(0);
    phase(va[CUR], qB, accB, oB, pfB, accA, pfA, dA);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (NDMA > 0 || V_DIRECT) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NDMA) : "memory");
    if constexpr (LDS && READS) {
#pragma unroll
      for (int j = 0; j < 4; j++) ka[j] = *reinterpret_cast<const v4i*>(smem + (s_new ^ 1) * 4096 + kr_off[j]);
      if constexpr (!V_DIRECT) {
#pragma unroll
        for (int j = 0; j < 4; j++)
          va[NXT][j] = *reinterpret_cast<const v4i*>(smem + 8192 + (s_new ^ 1) * 4096 + lane * 16 + j * 1024);
      }
    }
    t1 = t2; t2 = t3; t3 = __builtin_amdgcn_readfirstlane(next_t);
    if constexpr (LDS && READS) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };
  const long long c0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; it += 2) {
    body(it, std::integral_constant<int, 0>{});
    body(it + 1, std::integral_constant<int, V_DIRECT ? 1 : 0>{});
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  float s = dA[0] + dA[1] + dB[0] + dB[1];
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int i = 0; i < 16; i++) s += oA[j][i] + oB[j][i];
#pragma unroll
  for (int i = 0; i < 16; i++) s += (float)(accA[0][i] + accA[1][i] + accB[0][i] + accB[1][i]);
  sink[blockIdx.x * 64 + lane] = s;
  if (lane == 0 && blockIdx.x == (gridDim.x > 777 ? 777 : 0)) {
    clk[0] = clock64() - c0;
    clk[1] = wall_clock64() - w0;
  }
}

}  // namespace paro

extern "C" const char* paro_diag_last_error(void) { return paro::g_diag_err; }

extern "C" int64_t paro_diag_attn_proxy_ops(int workgroups, int iters) {
  // counted like the attention kernel counts a block: 4 int8 products of 2*32*32*32 and 2 fp8 products of
  // 2*32*32*64 operations per wave and iteration (the row-sum product is not counted), two waves per workgroup
  return (4LL * 65536 + 2LL * 131072) * 2 * (int64_t)workgroups * iters;
}

extern "C" int paro_diag_attn_proxy(int level, const void* operands, const void* tiles, float* sink, int workgroups,
                                    int iters, int ntiles, void* stream) {
  using namespace paro;
  DIAG_CHECK(level >= 0 && level <= 3, -1, "paro_diag_attn_proxy: level must be 0..3");
  DIAG_CHECK(operands && tiles && sink && workgroups > 0 && iters > 0 && ntiles >= 4, -2,
             "paro_diag_attn_proxy: bad arguments");
  // block list entries are 16 bits, and the tiles are addressed through a 32-bit buffer descriptor
  DIAG_CHECK(ntiles <= 65535 && workgroups <= 1 << 20 && iters <= 1 << 24, -1,
             "paro_diag_attn_proxy: at most 65535 tiles, 2^20 workgroups, 2^24 iterations");
  hipStream_t st = (hipStream_t)stream;
#define PARO_PROXY(L)                                                                                             \
  hipLaunchKernelGGL((attn_proxy_kernel<L>), dim3(workgroups), dim3(128), 24576 + 1024, st, (const int*)operands,        \
                     (const uint8_t*)tiles, sink, iters, ntiles)
  if (level == 0) PARO_PROXY(0);
  else if (level == 1) PARO_PROXY(1);
  else if (level == 2) PARO_PROXY(2);
  else PARO_PROXY(3);
#undef PARO_PROXY
  DIAG_HIP(hipGetLastError());
  return 0;
}

extern "C" int64_t paro_diag_attn_proxy_w64_ops(int workgroups, int iters) {
  // one wave per workgroup, both 32-row halves per iteration: 8 int8 and 4 fp8 products counted
  return (8LL * 65536 + 4LL * 131072) * (int64_t)workgroups * iters;
}

extern "C" int paro_diag_attn_proxy_w64(int variant, const void* operands, const void* tiles, float* sink,
                                        int64_t* clk, int workgroups, int iters, int ntiles, void* stream) {
  using namespace paro;
  DIAG_CHECK(variant >= 0 && variant <= 4, -1, "paro_diag_attn_proxy_w64: variant must be 0..4");
  DIAG_CHECK(operands && tiles && sink && clk && workgroups > 0 && iters > 0 && (iters & 1) == 0 && ntiles >= 4, -2,
             "paro_diag_attn_proxy_w64: bad arguments (iters must be even)");
  DIAG_CHECK(ntiles <= 65535 && workgroups <= 1 << 20 && iters <= 1 << 24, -1,
             "paro_diag_attn_proxy_w64: at most 65535 tiles, 2^20 workgroups, 2^24 iterations");
  hipStream_t st = (hipStream_t)stream;
#define PARO_PROXY64(...)                                                                                        \
  hipLaunchKernelGGL((attn_proxy_w64_kernel<__VA_ARGS__>), dim3(workgroups), dim3(64), 16384 + 1024, st,          \
                     (const int*)operands, (const uint8_t*)tiles, sink, iters, ntiles, (long long*)clk)
  if (variant == 0) PARO_PROXY64(false, false, false, false);       // operands in registers
  else if (variant == 1) PARO_PROXY64(true, false, true, false);    // + fragment reads
  else if (variant == 2) PARO_PROXY64(true, true, false, false);    // + tile DMA (no reads)
  else if (variant == 3) PARO_PROXY64(true, true, true, false);     // + both
  else PARO_PROXY64(true, true, true, true);                        // K through LDS, V straight into registers
#undef PARO_PROXY64
  DIAG_HIP(hipGetLastError());
  return 0;
}

extern "C" int64_t paro_diag_mfma_loop_ops(int kind, int workgroups, int iters) {
  // four MFMAs per iteration and wave, four waves per workgroup; 2*32*32*K operations each
  const int64_t per_mfma = kind == 0 ? 2LL * 32 * 32 * 32 : 2LL * 32 * 32 * 64;
  return per_mfma * 4 * 4 * (int64_t)workgroups * iters;
}

extern "C" int paro_diag_mfma_loop(int kind, const void* operands, float* sink, int workgroups, int iters,
                                   void* stream) {
  using namespace paro;
  DIAG_CHECK(kind == 0 || kind == 1, -1, "paro_diag_mfma_loop: kind must be 0 (int8) or 1 (fp8)");
  DIAG_CHECK(operands && sink && workgroups > 0 && iters > 0, -2, "paro_diag_mfma_loop: bad arguments");
  hipStream_t st = (hipStream_t)stream;
  if (kind == 0)
    hipLaunchKernelGGL((mfma_loop_kernel<0>), dim3(workgroups), dim3(256), 0, st, (const int*)operands, sink, iters);
  else
    hipLaunchKernelGGL((mfma_loop_kernel<1>), dim3(workgroups), dim3(256), 0, st, (const int*)operands, sink, iters);
  DIAG_HIP(hipGetLastError());
  return 0;
}
