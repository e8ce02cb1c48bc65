/* libparoatten_diag.so: measurement aids for bench.py (--mfma-ceiling, --proxy-ceiling).
 *
 * NOT part of the drop-in boundary: nothing here has a counterpart in the reference, and the product library
 * (libparoatten_hip.so, include/paroatten.h) neither contains nor needs it.  gfx950 only.  Same conventions as
 * paroatten.h: device pointers, a hipStream_t as void*, return 0 or a negative code (-1 bad value, -2 bad
 * argument, -4 HIP error); paro_diag_last_error() gives the message of the calling thread's last failure.
 */
#ifndef PAROATTEN_DIAG_H
#define PAROATTEN_DIAG_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

const char* paro_diag_last_error(void);

/* ---------------------------------------------------------------------------------------------
 * `workgroups` workgroups of four waves each issue
 * `iters` x 4 back-to-back MFMAs of the kind the attention kernel uses (kind 0: v_mfma_i32_32x32x32_i8,
 * kind 1: v_mfma_f32_32x32x64_f8f6f4 on e4m3 operands) with nothing else in the loop.  operands: 4 KiB of
 * device memory (64 lanes x 16 words) that every wave takes its A / B registers from (random bytes or
 * zeros); sink: one float per wave (workgroups * 4).  paro_diag_mfma_loop_ops() = operations one launch
 * executes.  Timed by the caller, it gives what the matrix pipe sustains on the GPU at hand.
 * ------------------------------------------------------------------------------------------- */
int64_t paro_diag_mfma_loop_ops(int kind, int workgroups, int iters);
int paro_diag_mfma_loop(int kind, const void* operands, float* sink, int workgroups, int iters, void* stream);

/* A proxy of the attention loop body at D = 64 (the same
 * matrix and vector instructions per wave and iteration, workgroups of two waves) at four levels: 0 operands in
 * registers, 1 + K/V fragments read from LDS every iteration, 2 + the four LDS-DMA tile loads per wave and
 * iteration, 3 + one barrier per iteration.  operands: 16384 int32 of device memory (random bytes); tiles:
 * ntiles * 8192 bytes (random e4m3 bytes other than the NaN codes), ntiles <= 65535; sink: workgroups * 128 floats.
 * paro_diag_attn_proxy_ops() = operations one launch is credited with, counted as the attention kernel counts
 * a block.  Used by bench.py --proxy-ceiling. */
int64_t paro_diag_attn_proxy_ops(int workgroups, int iters);
int paro_diag_attn_proxy(int level, const void* operands, const void* tiles, float* sink, int workgroups, int iters,
                         int ntiles, void* stream);

/* The same instruction mix arranged as the one-wave-per-q-block kernel arranges it (attn_sparse_w64.hip): one-wave
 * workgroups, two per SIMD, two 32-row halves per wave software-pipelined against each other, every K / V fragment
 * read feeding two products.  variant: 0 operands in registers, 1 + the 8 fragment reads per block, 2 + the 8 LDS-DMA
 * tile loads per block instead (no reads), 3 + both, 4 as 3 with V straight from memory into registers (no LDS
 * round trip for V).  iters even.  sink: workgroups * 64 floats.  clk: two int64 on the device, shader-clock cycles
 * and 100 MHz ticks one workgroup spent in its loop (their ratio is the shader clock under this load).
 * Used by bench.py --proxy-ceiling. */
int64_t paro_diag_attn_proxy_w64_ops(int workgroups, int iters);
int paro_diag_attn_proxy_w64(int variant, const void* operands, const void* tiles, float* sink, int64_t* clk,
                             int workgroups, int iters, int ntiles, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PAROATTEN_DIAG_H */
