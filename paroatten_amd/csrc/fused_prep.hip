// One pass from the projections to the attention kernel's operands (HBM-bound):
//   Q, K : RoPE -> per-head token permutation -> per-group INT8 (Q: 32 tokens, K: 64 tokens, K
//          optionally mean-smoothed)                               -> q8, q_scale, k8, k_scale
//   V    : per-head token permutation -> (v - mean)/scale as e4m3 in P.V fragment order -> v8
// It replaces the chain rope_permute -> quant_int8 (twice) -> v_fp8_pack.  INT8 tensors and scales are
// bit-identical to the chain's: the rotated values are rounded to the 16-bit input type before
// quantisation exactly as if the permuted tensors had been written out, but they never are.  V's
// per-channel statistics are order-independent except for the fp32 summation order of the mean
// (taken here over the unpermuted tensor).  Per (batch, head) the pass saves one write and one read
// of Q and K and one write and one read of V.
//
// Ownership is by DESTINATION: a workgroup owns one 64-token block of the permuted sequence (= one K
// scale group, two Q scale groups, one V tile), so the group maxima are workgroup-local.  All heads
// that share a permutation order gather the same source rows, hence the same rotary-table rows: the
// workgroup is launched per (block, order), each lane keeps the table entries of its 16-byte pieces
// in registers and the workgroup walks over the (batch, head) pairs that use its order.
//
// Reference for the arithmetic: the RoPE + permute_qk sequence of the processors
// (paroattention/cogvideox.py:167-186), QuantInt8Kernel (csrc/fused/fused.cu:64-198) and
// MeanScaleKernel (csrc/fused/fused.cu:316-427).
#include "paro_device.hpp"

namespace paro {

template <int DT, int D>
__global__ void __launch_bounds__(256) rope_permute_quant_kernel(
    const unsigned short* __restrict__ q_in, const unsigned short* __restrict__ k_in,
    const unsigned short* __restrict__ v_in, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ orders, const unsigned short* __restrict__ k_mean, int8_t* __restrict__ q8,
    float* __restrict__ q_scale, int8_t* __restrict__ k8, float* __restrict__ k_scale, uint8_t* __restrict__ v8,
    const float* __restrict__ v_recp, const float* __restrict__ v_mean, int BH, int H, int N, int nb, int n_text,
    int F, int Hh, int W, int head_split, int64_t qs_b, int64_t qs_h, int64_t qs_n, int64_t ks_b, int64_t ks_h,
    int64_t ks_n, int64_t vs_b, int64_t vs_h, int64_t vs_n, int64_t ms_b, int64_t ms_h) {
  constexpr int LPR = D / 8;            // lanes per token row (16-byte pieces)
  constexpr int RPI = 64 / LPR;         // rows one wave covers per load instruction
  constexpr int PC = 16 / RPI;          // pieces per lane: a wave owns 16 rows of the block
  constexpr int PITCH = D + 8;          // V tile row pitch in 16-bit elements
  __shared__ int s_src[64];             // source token of each destination row, -1 past the end
  __shared__ __attribute__((aligned(16))) unsigned short s_tile[64 * PITCH];
  __shared__ float s_amax[2][4];        // [q|k][wave]

  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int kb = blockIdx.x;
  const int order = blockIdx.y % 6, split = blockIdx.y / 6;
  const bool rope = cos_t != nullptr;

  if (t < 64) {
    const int d = kb * 64 + t;
    int src = -1;
    if (d < N) src = d < n_text ? d : n_text + unpermute_index(d - n_text, order, F, Hh, W);
    s_src[t] = src;
  }
  __syncthreads();

  // this lane's pieces: rows 16*wave + i*RPI + lane/LPR of the block, channels col..col+7; their
  // rotary-table entries stay in registers for every (batch, head) the workgroup walks over
  const int col = (lane % LPR) * 8;
  const int row0 = 16 * wave + lane / LPR;
  int src[PC];
  float cs[PC][8], sn[PC][8];
#pragma unroll
  for (int i = 0; i < PC; i++) {
    src[i] = s_src[row0 + i * RPI];
    if (rope && src[i] >= n_text) {
      const int64_t o = (int64_t)(src[i] - n_text) * D + col;
      const v4f c0 = *reinterpret_cast<const v4f*>(cos_t + o), c1 = *reinterpret_cast<const v4f*>(cos_t + o + 4);
      const v4f s0 = *reinterpret_cast<const v4f*>(sin_t + o), s1 = *reinterpret_cast<const v4f*>(sin_t + o + 4);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        cs[i][j] = c0[j]; cs[i][4 + j] = c1[j];
        sn[i][j] = s0[j]; sn[i][4 + j] = s1[j];
      }
    }
  }

  const int n_chunks = (N + V_CHUNK - 1) / V_CHUNK;
  int n_match = 0;
  for (int bh = 0; bh < BH; bh++) {
    const int b = bh / H, head = bh - b * H;
    const int head_order = (unsigned)orders[head] > 5u ? 0 : orders[head];   // as order_strides treats it
    if (head_order != order) continue;                    // uniform over the workgroup
    if ((n_match++ % head_split) != split) continue;
    float mv[8];
    if (k_mean) {
      const v4i m = *reinterpret_cast<const v4i*>(k_mean + b * ms_b + head * ms_h + col);
#pragma unroll
      for (int j = 0; j < 8; j++) mv[j] = elem16_to_f32<DT>(m, j);
    } else {
#pragma unroll
      for (int j = 0; j < 8; j++) mv[j] = 0.f;
    }

    // ---- gather; rotate Q and K and round them to the input type (kept packed); V to the tile ----
    v4i rq[PC], rk[PC];
#pragma unroll
    for (int i = 0; i < PC; i++) {
      v4i rv = {0, 0, 0, 0};
      rq[i] = rv;
      rk[i] = rv;
      if (src[i] >= 0) {
        // read once: non-temporal, the L2 keeps the rotary tables and the V statistics instead
        rq[i] = __builtin_nontemporal_load(
            reinterpret_cast<const v4i*>(q_in + b * qs_b + head * qs_h + (int64_t)src[i] * qs_n + col));
        rk[i] = __builtin_nontemporal_load(
            reinterpret_cast<const v4i*>(k_in + b * ks_b + head * ks_h + (int64_t)src[i] * ks_n + col));
        rv = __builtin_nontemporal_load(
            reinterpret_cast<const v4i*>(v_in + b * vs_b + head * vs_h + (int64_t)src[i] * vs_n + col));
      }
      *reinterpret_cast<v4i*>(&s_tile[(row0 + i * RPI) * PITCH + col]) = rv;
    }
    float aq = 0.0000001f, ak = 0.0000001f;
#pragma unroll
    for (int i = 0; i < PC; i++) {
      if (rope && src[i] >= n_text) {
        rq[i] = rotate8<DT>(rq[i], cs[i], sn[i]);
        rk[i] = rotate8<DT>(rk[i], cs[i], sn[i]);
      }
      if (src[i] >= 0) {  // rows past the end count as zero, whatever the mean
#pragma unroll
        for (int j = 0; j < 8; j++) {
          aq = fmaxf(aq, fabsf(elem16_to_f32<DT>(rq[i], j)));
          ak = fmaxf(ak, fabsf(elem16_to_f32<DT>(rk[i], j) - mv[j]));
        }
      }
    }
    aq = wave_max(aq);
    ak = wave_max(ak);
    if (lane == 0) {
      s_amax[0][wave] = aq;
      s_amax[1][wave] = ak;
    }
    __syncthreads();

    // ---- group maxima: Q per 32 rows (two waves), K per 64 rows (the workgroup) --------------
    aq = fmaxf(s_amax[0][wave & 2], s_amax[0][(wave & 2) + 1]);
    ak = fmaxf(fmaxf(s_amax[1][0], s_amax[1][1]), fmaxf(s_amax[1][2], s_amax[1][3]));
    if (lane == 0 && (wave & 1) == 0) q_scale[(int64_t)bh * (nb * 2) + kb * 2 + (wave >> 1)] = aq / 127.0f;
    if (t == 0) k_scale[(int64_t)bh * nb + kb] = ak / 127.0f;
    const float inv_q = 127.0f / aq, inv_k = 127.0f / ak;
#pragma unroll
    for (int i = 0; i < PC; i++) {
      // |x * (127/amax)| <= 127 up to rounding: the reference's clamp to [-128,127] never acts
      float yq[8], yk[8];
#pragma unroll
      for (int j = 0; j < 8; j++) {
        yq[j] = elem16_to_f32<DT>(rq[i], j) * inv_q;
        yk[j] = (elem16_to_f32<DT>(rk[i], j) - mv[j]) * inv_k;
      }
      if (src[i] >= 0) {
        const int64_t o = ((int64_t)bh * N + kb * 64 + row0 + i * RPI) * D + col;
        __builtin_nontemporal_store(v2i{(int)pack4_rint_i8(yq[0], yq[1], yq[2], yq[3]),
                                        (int)pack4_rint_i8(yq[4], yq[5], yq[6], yq[7])},
                                    reinterpret_cast<v2i*>(q8 + o));
        __builtin_nontemporal_store(v2i{(int)pack4_rint_i8(yk[0], yk[1], yk[2], yk[3]),
                                        (int)pack4_rint_i8(yk[4], yk[5], yk[6], yk[7])},
                                    reinterpret_cast<v2i*>(k8 + o));
      }
    }

    // ---- V tile -> e4m3 fragments -------------------------------------------------------------
    pack_v_tile<DT, D, PITCH>(s_tile, v8 + ((int64_t)bh * nb + kb) * (int64_t)(64 * D),
                              v_recp + v_recp_offset(bh, n_chunks, D), v_mean ? v_mean + (int64_t)bh * D : nullptr,
                              kb * 64, N, t);
    __syncthreads();  // the tile and s_amax are reused by the next (batch, head)
  }
}

// K mean over tokens AFTER the rotation (the permutation does not change a mean): partial sums per
// 256-token chunk, then one workgroup per (batch, head) adds them in a fixed order.  A thread keeps
// the table entries of its token piece while it walks over a group of (batch, head) pairs.
constexpr int KM_GROUP = 8;
template <int DT, int D>
__global__ void __launch_bounds__(256) rope_k_sum_kernel(const unsigned short* __restrict__ k,
                                                         const float* __restrict__ cos_t,
                                                         const float* __restrict__ sin_t,
                                                         float* __restrict__ partial, int BH, int H, int N,
                                                         int n_text, int n_chunks, int64_t ks_b, int64_t ks_h,
                                                         int64_t ks_n) {
  constexpr int LPR = D / 8;
  constexpr int ROWS = 256 / LPR;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int chunk = blockIdx.x;
  const int bh0 = blockIdx.y * KM_GROUP;
  const int col = (t % LPR) * 8;
  float s[KM_GROUP][8];
#pragma unroll
  for (int g = 0; g < KM_GROUP; g++)
#pragma unroll
    for (int j = 0; j < 8; j++) s[g][j] = 0.f;
  for (int r = t / LPR; r < V_CHUNK; r += ROWS) {
    const int tok = chunk * V_CHUNK + r;
    if (tok >= N) break;
    const bool rot = cos_t != nullptr && tok >= n_text;
    float cs[8], sn[8];
    if (rot) {
      const int64_t o = (int64_t)(tok - n_text) * D + col;
      const v4f c0 = *reinterpret_cast<const v4f*>(cos_t + o), c1 = *reinterpret_cast<const v4f*>(cos_t + o + 4);
      const v4f s0 = *reinterpret_cast<const v4f*>(sin_t + o), s1 = *reinterpret_cast<const v4f*>(sin_t + o + 4);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        cs[j] = c0[j]; cs[4 + j] = c1[j];
        sn[j] = s0[j]; sn[4 + j] = s1[j];
      }
    }
#pragma unroll
    for (int g = 0; g < KM_GROUP; g++) {
      const int bh = bh0 + g;
      if (bh < BH) {
        const int b = bh / H, h = bh - b * H;
        // ordinary load: K was just written by the projection and is read again by the preparation
        // pass, so it should stay in the last-level cache
        v4i raw = *reinterpret_cast<const v4i*>(k + b * ks_b + h * ks_h + (int64_t)tok * ks_n + col);
        if (rot) raw = rotate8<DT>(raw, cs, sn);
#pragma unroll
        for (int j = 0; j < 8; j++) s[g][j] += elem16_to_f32<DT>(raw, j);
      }
    }
  }
  __shared__ float red[4][KM_GROUP][D];
#pragma unroll
  for (int g = 0; g < KM_GROUP; g++) {
#pragma unroll
    for (int o = 32; o >= LPR; o >>= 1)
#pragma unroll
      for (int j = 0; j < 8; j++) s[g][j] += __shfl_xor(s[g][j], o, 64);
    if (lane < LPR) {
#pragma unroll
      for (int j = 0; j < 8; j++) red[wave][g][col + j] = s[g][j];
    }
  }
  __syncthreads();
  for (int i = t; i < KM_GROUP * D; i += 256) {
    const int g = i / D, ch = i % D;
    if (bh0 + g < BH)
      partial[((int64_t)(bh0 + g) * n_chunks + chunk) * D + ch] =
          (red[0][g][ch] + red[1][g][ch]) + (red[2][g][ch] + red[3][g][ch]);
  }
}

template <int DT, int D>
__global__ void __launch_bounds__(1024) k_mean_finalize_kernel(const float* __restrict__ partial,
                                                               unsigned short* __restrict__ k_mean, int N,
                                                               int n_chunks, int64_t ms_b, int64_t ms_h, int H) {
  constexpr int SL = 1024 / D;
  __shared__ float red[SL][D];
  const int ch = threadIdx.x % D, sl = threadIdx.x / D;
  const int64_t bh = blockIdx.x;
  const float* p = partial + bh * n_chunks * D;
  float s = 0.f;
  for (int c = sl; c < n_chunks; c += SL) s += p[c * D + ch];
  red[sl][ch] = s;
  __syncthreads();
  if (sl == 0) {
    for (int i = 1; i < SL; i++) s += red[i][ch];
    const int b = (int)(bh / H), h = (int)(bh % H);
    k_mean[b * ms_b + h * ms_h + ch] = (unsigned short)(pack2_from_f32<DT>(s / (float)N, 0.f) & 0xffffu);
  }
}

static int check_prep(const char* fn, int dtype, int B, int H, int N, int D, int n_text, int F, int Hh, int W,
                      int64_t s_b, int64_t s_h, int64_t s_n) {
  PARO_CHECK(B > 0 && H > 0 && N > 0, PARO_ERR_RUNTIME, "%s: empty shape", fn);
  PARO_CHECK(D == 64 || D == 128, PARO_ERR_INVALID_VALUE, "Unsupported head dim: %d", D);
  PARO_CHECK(dtype == PARO_DTYPE_F16 || dtype == PARO_DTYPE_BF16, PARO_ERR_RUNTIME,
             "Unsupported input dtype (expect float16 or bfloat16)");
  PARO_CHECK(n_text >= 0 && F > 0 && Hh > 0 && W > 0 && (int64_t)n_text + (int64_t)F * Hh * W == N,
             PARO_ERR_RUNTIME, "%s: n_text + F*H*W = %d + %d*%d*%d does not equal the token count %d", fn, n_text, F,
             Hh, W, N);
  PARO_CHECK(s_b % 8 == 0 && s_h % 8 == 0 && s_n % 8 == 0, PARO_ERR_RUNTIME,
             "%s: strides must be multiples of 8 elements", fn);
  return PARO_OK;
}

}  // namespace paro

extern "C" int64_t paro_prep_workspace_bytes(int B, int H, int N, int D) {
  // per-chunk partials of the V statistics (sum, min, max); the K mean needs a third of that
  return paro_v_fp8_partial_floats(B, H, N, D) * 4;
}

extern "C" int paro_rope_k_mean(const void* k, int dtype, const float* cos, const float* sin, void* k_mean,
                                void* workspace, int64_t workspace_bytes, int B, int H, int N, int D, int n_text,
                                int F, int Hh, int W, int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_n,
                                int64_t mean_stride_b, int64_t mean_stride_h, void* stream) {
  using namespace paro;
  if (int rc = check_prep("paro_rope_k_mean", dtype, B, H, N, D, n_text, F, Hh, W, k_stride_b, k_stride_h, k_stride_n))
    return rc;
  PARO_CHECK(k && k_mean && workspace, PARO_ERR_RUNTIME, "paro_rope_k_mean: null pointer");
  PARO_CHECK((cos == nullptr) == (sin == nullptr), PARO_ERR_RUNTIME, "paro_rope_k_mean: cos and sin must be given together");
  PARO_CHECK(((uintptr_t)k % 16) == 0 && ((uintptr_t)cos % 16) == 0 && ((uintptr_t)sin % 16) == 0 &&
                 ((uintptr_t)workspace % 16) == 0,
             PARO_ERR_RUNTIME, "paro_rope_k_mean: tensors must be 16-byte aligned");
  const int n_chunks = ceil_div(N, V_CHUNK);
  PARO_CHECK(workspace_bytes >= (int64_t)B * H * n_chunks * D * 4, PARO_ERR_RUNTIME,
             "paro_rope_k_mean: workspace of %lld bytes is too small", (long long)workspace_bytes);
  hipStream_t st = (hipStream_t)stream;
  float* partial = (float*)workspace;
#define PARO_KM(DTV, DV)                                                                                        \
  do {                                                                                                          \
    hipLaunchKernelGGL((rope_k_sum_kernel<DTV, DV>), dim3(n_chunks, ceil_div(B * H, KM_GROUP)), dim3(256), 0,   \
                       st, (const unsigned short*)k, cos, sin, partial, B * H, H, N, n_text, n_chunks,          \
                       k_stride_b, k_stride_h, k_stride_n);                                                     \
    hipLaunchKernelGGL((k_mean_finalize_kernel<DTV, DV>), dim3(B * H), dim3(1024), 0, st, (const float*)partial, \
                       (unsigned short*)k_mean, N, n_chunks, mean_stride_b, mean_stride_h, H);                  \
  } while (0)
  if (dtype == PARO_DTYPE_F16) {
    if (D == 64) PARO_KM(PARO_DTYPE_F16, 64); else PARO_KM(PARO_DTYPE_F16, 128);
  } else {
    if (D == 64) PARO_KM(PARO_DTYPE_BF16, 64); else PARO_KM(PARO_DTYPE_BF16, 128);
  }
#undef PARO_KM
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}

extern "C" int paro_rope_permute_quant_fwd(const void* q, const void* k, const void* v, int dtype, const float* cos,
                                           const float* sin, const int32_t* orders, const void* k_mean,
                                           int8_t* q8, float* q_scale, int8_t* k8, float* k_scale, uint8_t* v8,
                                           float* v_scale, float* v_mean, void* workspace, int64_t workspace_bytes,
                                           int B, int H, int N, int D, int n_text, int F, int Hh, int W,
                                           int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_n,
                                           int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_n,
                                           int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_n,
                                           int64_t mean_stride_b, int64_t mean_stride_h, int smooth_v,
                                           void* stream) {
  using namespace paro;
  if (int rc = check_prep("paro_rope_permute_quant_fwd", dtype, B, H, N, D, n_text, F, Hh, W, q_stride_b,
                          q_stride_h, q_stride_n))
    return rc;
  PARO_CHECK(k_stride_b % 8 == 0 && k_stride_h % 8 == 0 && k_stride_n % 8 == 0 && v_stride_b % 8 == 0 &&
                 v_stride_h % 8 == 0 && v_stride_n % 8 == 0,
             PARO_ERR_RUNTIME, "paro_rope_permute_quant_fwd: strides must be multiples of 8 elements");
  PARO_CHECK(q && k && v && orders && q8 && q_scale && k8 && k_scale && v8 && v_scale && workspace, PARO_ERR_RUNTIME,
             "paro_rope_permute_quant_fwd: null pointer");
  PARO_CHECK(!smooth_v || v_mean, PARO_ERR_RUNTIME, "paro_rope_permute_quant_fwd: smoothing needs a v_mean buffer");
  PARO_CHECK((cos == nullptr) == (sin == nullptr), PARO_ERR_RUNTIME,
             "paro_rope_permute_quant_fwd: cos and sin must be given together");
  const void* ptrs[9] = {q, k, v, cos, sin, k_mean, q8, k8, v8};
  for (int i = 0; i < 9; i++)
    PARO_CHECK(((uintptr_t)ptrs[i] % 16) == 0, PARO_ERR_RUNTIME,
               "paro_rope_permute_quant_fwd: tensors must be 16-byte aligned");
  PARO_CHECK(!k_mean || (mean_stride_b % 8 == 0 && mean_stride_h % 8 == 0), PARO_ERR_RUNTIME,
             "Tensor mean must be 16-byte aligned with strides that are multiples of 8");
  PARO_CHECK(workspace_bytes >= paro_prep_workspace_bytes(B, H, N, D) && ((uintptr_t)workspace % 16) == 0,
             PARO_ERR_RUNTIME, "paro_rope_permute_quant_fwd: workspace of %lld bytes is too small or misaligned",
             (long long)workspace_bytes);
  hipStream_t st = (hipStream_t)stream;
  // V statistics do not depend on the token order: taken on the unpermuted tensor
  if (int rc = v_fp8_stats(v, dtype, v_scale, v_mean, (float*)workspace, B, H, N, D, v_stride_b, v_stride_h,
                           v_stride_n, smooth_v, st))
    return rc;
  const int nb = ceil_div(N, 64);
  // every order gets `head_split` workgroups per block, each walking over its share of the (batch,
  // head) pairs with that order: enough workgroups to fill the chip, few enough that the table rows a
  // workgroup holds are reused
  int head_split = 1;
  while (head_split < 8 && (int64_t)nb * 6 * head_split < 2048 && head_split * 2 <= B * H) head_split *= 2;
  dim3 grid(nb, 6 * head_split), block(256);
#define PARO_PREP(DTV, DV)                                                                                      \
  hipLaunchKernelGGL((rope_permute_quant_kernel<DTV, DV>), grid, block, 0, st, (const unsigned short*)q,        \
                     (const unsigned short*)k, (const unsigned short*)v, cos, sin, (const int*)orders,          \
                     (const unsigned short*)k_mean, q8, q_scale, k8, k_scale, v8, (const float*)workspace,      \
                     (const float*)(smooth_v ? v_mean : nullptr), B * H, H, N, nb, n_text, F, Hh, W, head_split, \
                     q_stride_b, q_stride_h, q_stride_n, k_stride_b, k_stride_h, k_stride_n, v_stride_b,        \
                     v_stride_h, v_stride_n, mean_stride_b, mean_stride_h)
  if (dtype == PARO_DTYPE_F16) {
    if (D == 64) PARO_PREP(PARO_DTYPE_F16, 64); else PARO_PREP(PARO_DTYPE_F16, 128);
  } else {
    if (D == 64) PARO_PREP(PARO_DTYPE_BF16, 64); else PARO_PREP(PARO_DTYPE_BF16, 128);
  }
#undef PARO_PREP
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}
