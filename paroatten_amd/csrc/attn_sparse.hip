// Block-sparse quantised attention for gfx950 (MI355X).
//
//   S^T = K8 . Q8^T      v_mfma_i32_32x32x32_i8       exact int32
//   P~  = 2^(S*c - m + 8) online base-2 softmax in fp32, rounded to FP8 e4m3 (OCP)
//   O^T += V8^T . P~^T   v_mfma_f32_32x32x64_f8f6f4   fp32 accumulation
//
// One workgroup = one 64-row q-block of one (batch, head); its two 64-lane waves own 32 q-rows
// each (= one q-scale group).  The transposed products make the accumulator fragment of S^T (a lane
// holds 32 kv-values of ONE q-row) directly the B operand of the P.V MFMA; the kv-order inside a
// block that this implies is absorbed by the tile order V8 is stored in (see v_fp8.hip), so no
// cross-lane data movement is needed between the two matrix products and the row maximum / row sum
// need one exchange with the partner lane (lane ^ 32) only.
//
// k-blocks: the workgroup turns its row of the bool mask into a compact list in LDS and loops over
// the kept blocks only; a skipped block costs neither loads nor MFMA issue.  K8 (row-major, XOR
// swizzled against bank conflicts) and V8 (already in fragment order) tiles are double-buffered in
// LDS: the global loads of block i+1 are in flight while block i is computed.
//
// Workgroups are renumbered so that each of the 8 XCDs walks a contiguous range of (batch, head,
// q-block): the K8/V8 of the one or two heads an XCD is working on stay resident in its own L2.
//
// Semantics follow qk_int_sv_f16_attn_kernel of the reference
// (csrc/qattn/qk_int_sv_f16_cuda_sm80.cu:44-726) as instantiated by its host (:1022-1048):
// scale indexing :100-133, mask indexing :222/:268, out-of-range columns attn_utils.cuh:355-381,
// softmax recurrence attn_utils.cuh:383-488, normalisation :786-840, lse = log2(d) + m (:711-723).
#include "paro_common.hpp"

namespace paro {

struct AttnParams {
  const int8_t* q8;
  const int8_t* k8;
  const uint8_t* v8;
  const float* q_scale;
  const float* k_scale;
  const float* v_scale;
  const float* v_mean;
  const uint8_t* sparse;
  void* out;
  float* lse;
  int32_t* s_dump;
  int64_t sparse_bs;
  int64_t qs_b, qs_h, qs_n;
  int64_t ks_b, ks_h, ks_n;
  int64_t os_b, os_h, os_n;
  int B, H, Hkv, Nq, Nk, nbq, nbk;
  int total;  // B*H*nbq workgroups that have work
  float sm_scale_log2e;
};

constexpr float P_EXP_OFFSET = 8.0f;  // P~ = 2^8 * P <= 256 < 448 = max e4m3
constexpr int S_MAGIC_BITS = 0x4B400000;  // float 1.5 * 2^23
constexpr float S_MAGIC_F = 12582912.0f;
constexpr int FP8_ONES = 0x38383838;  // four e4m3 1.0

template <int D>
__device__ __forceinline__ int k_swizzle(int row, int chunk) {
  if constexpr (D == 64) return chunk ^ (((row >> 1) ^ (row >> 3)) & 3);
  else return chunk ^ ((row ^ (row >> 3)) & 7);
}

__device__ __forceinline__ float partner_max(float x) {
  // max of own value and that of lane ^ 32: v_permlane32_swap exchanges the upper half of its
  // first operand with the lower half of its second
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

template <int D, int OUT_DT, bool CAUSAL, bool DUMP, bool LSE>
__global__ void __launch_bounds__(128) attn_sparse_kernel(const AttnParams p) {
  constexpr int KS = D / 32;        // k-steps of the QK MFMA (32 channels each)
  constexpr int DT_TILES = D / 32;  // 32-channel tiles of O^T
  constexpr int NLD = D / 32;       // 16-byte pieces per thread per K (or V) tile
  constexpr int TILE = 64 * D;      // bytes of one K8 or V8 tile
  constexpr int CPR = D / 16;       // 16-byte chunks per K row

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint8_t* lds_k = smem;                   // [2][TILE]
  uint8_t* lds_v = smem + 2 * TILE;        // [2][TILE]
  unsigned short* klist = reinterpret_cast<unsigned short*>(smem + 4 * TILE);  // [nbk]
  __shared__ int s_cnt;

  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int l32 = lane & 31, lh = lane >> 5;

  // XCD-aware renumbering: hardware deals workgroup ids round-robin to the 8 XCDs
  const int per = gridDim.x >> 3;
  const int vid = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
  if (vid >= p.total) return;
  const int qb = vid % p.nbq;
  const int bh = vid / p.nbq;
  const int h = bh % p.H, b = bh / p.H;
  const int hk = h / (p.H / p.Hkv);
  const int64_t bhk = (int64_t)b * p.Hkv + hk;

  // ---- compact list of kept k-blocks ------------------------------------------------------
  const int kmax = CAUSAL ? min(p.nbk, qb + 1) : p.nbk;
  if (wave == 0) {
    const uint8_t* mrow = p.sparse + b * p.sparse_bs + ((int64_t)h * p.nbq + qb) * p.nbk;
    int cnt = 0;
    for (int base = 0; base < kmax; base += 256) {
      uint8_t m[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int j = base + u * 64 + lane;
        m[u] = (j < kmax) ? mrow[j] : (uint8_t)0;
      }
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const bool keep = m[u] != 0;
        const unsigned long long bal = __ballot(keep);
        if (keep) klist[cnt + __popcll(bal & ((1ull << lane) - 1ull))] = (unsigned short)(base + u * 64 + lane);
        cnt += __popcll(bal);
      }
    }
    if (lane == 0) s_cnt = cnt;
  }

  // ---- Q fragments (B operand: column = q-row, 16 channels per lane and k-step) -----------
  const int qrow = qb * 64 + wave * 32 + l32;
  v4i qf[KS];
  {
    const int8_t* qp = p.q8 + b * p.qs_b + h * p.qs_h + (int64_t)qrow * p.qs_n + 16 * lh;
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
      qf[ks] = (qrow < p.Nq) ? *reinterpret_cast<const v4i*>(qp + 32 * ks) : v4i{0, 0, 0, 0};
  }
  const float qsc = p.q_scale[((int64_t)b * p.H + h) * (p.nbq * 2) + qb * 2 + wave] * p.sm_scale_log2e;
  const float* ksc_base = p.k_scale + bhk * p.nbk;

  __syncthreads();
  const int cnt = s_cnt;

  using OutT = F16x<OUT_DT>;
  unsigned short* outp = reinterpret_cast<unsigned short*>(p.out) + b * p.os_b + h * p.os_h + (int64_t)qrow * p.os_n;

  if (cnt == 0) {  // no kept block: the row outputs 0 (reference: m = -5e6, d = 1, O = 0)
    if (qrow < p.Nq) {
#pragma unroll
      for (int c = 0; c < D / 16; c++) *reinterpret_cast<v4i*>(outp + (lh * (D / 16) + c) * 8) = v4i{0, 0, 0, 0};
      if (p.lse && lh == 0) p.lse[((int64_t)b * p.H + h) * p.Nq + qrow] = -INFINITY;
    }
    return;
  }

  // ---- tile movers ------------------------------------------------------------------------
  const int8_t* kg = p.k8 + b * p.ks_b + hk * p.ks_h;
  const uint8_t* vg = p.v8 + bhk * p.nbk * (int64_t)TILE;
  v4i kst[NLD], vst[NLD];
  auto load_tile = [&](int kb) {
#pragma unroll
    for (int i = 0; i < NLD; i++) {
      const int c = t + 128 * i;
      const int row = c / CPR, cc = c % CPR;
      const int kvrow = kb * 64 + row;
      kst[i] = (kvrow < p.Nk) ? *reinterpret_cast<const v4i*>(kg + (int64_t)kvrow * p.ks_n + cc * 16)
                              : v4i{0, 0, 0, 0};
      vst[i] = *reinterpret_cast<const v4i*>(vg + (int64_t)kb * TILE + c * 16);
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < NLD; i++) {
      const int c = t + 128 * i;
      const int row = c / CPR, cc = c % CPR;
      *reinterpret_cast<v4i*>(lds_k + buf * TILE + row * D + k_swizzle<D>(row, cc) * 16) = kst[i];
      *reinterpret_cast<v4i*>(lds_v + buf * TILE + c * 16) = vst[i];
    }
  };

  // ---- state ------------------------------------------------------------------------------
  v16f o_acc[DT_TILES];
#pragma unroll
  for (int dt = 0; dt < DT_TILES; dt++)
#pragma unroll
    for (int i = 0; i < 16; i++) o_acc[dt][i] = 0.f;
  // every row of this 32x32 tile ends up holding the row sums of P~ (only element 0 is read)
  v16f d_acc;
#pragma unroll
  for (int i = 0; i < 16; i++) d_acc[i] = 0.f;
  const v8i ones = {FP8_ONES, FP8_ONES, FP8_ONES, FP8_ONES, FP8_ONES, FP8_ONES, FP8_ONES, FP8_ONES};
  float m_i = -1e30f;
  float d_exact = 0.f;  // LSE only: sum of the unrounded P~ of this lane's 32 kv-columns per block

  load_tile(klist[0]);
  store_tile(0);
  __syncthreads();

  for (int it = 0; it < cnt; it++) {
    const int kb = __builtin_amdgcn_readfirstlane((int)klist[it]);
    const int buf = it & 1;
    const bool more = it + 1 < cnt;
    if (more) load_tile(__builtin_amdgcn_readfirstlane((int)klist[it + 1]));

    // S^T tile: 64 kv-rows (2 MFMA row tiles) x 32 q-columns.  The accumulators start at the
    // bit pattern of 1.5*2^23: the int32 result then READS as the float 12582912 + S exactly
    // (|S| <= 127*127*128 < 2^22), which saves the int->float conversions.
    v16i acc[2];
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[mt][i] = S_MAGIC_BITS;
    const uint8_t* kt = lds_k + buf * TILE;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
#pragma unroll
      for (int mt = 0; mt < 2; mt++) {
        const int row = 32 * mt + l32;
        const v4i kf = *reinterpret_cast<const v4i*>(kt + row * D + k_swizzle<D>(row, 2 * ks + lh) * 16);
        acc[mt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf, qf[ks], acc[mt], 0, 0, 0);
      }
    }
    if constexpr (DUMP) {
      if (p.s_dump) {
        int32_t* sd = p.s_dump + (((int64_t)b * p.H + h) * (p.nbq * 64) + qrow) * (int64_t)(p.nbk * 64) + kb * 64;
#pragma unroll
        for (int mt = 0; mt < 2; mt++)
#pragma unroll
          for (int i = 0; i < 16; i++) sd[32 * mt + 8 * (i >> 2) + 4 * lh + (i & 3)] = acc[mt][i] - S_MAGIC_BITS;
      }
    }

    float s[2][16];
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
      for (int i = 0; i < 16; i++) s[mt][i] = __int_as_float(acc[mt][i]);

    // columns past the end of K (last block) or above the diagonal (causal) leave the softmax
    const bool edge = (kb == p.nbk - 1 && (p.Nk & 63) != 0) || (CAUSAL && kb == qb);
    if (edge) {
#pragma unroll
      for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const int j = kb * 64 + 32 * mt + 8 * (i >> 2) + 4 * lh + (i & 3);
          const bool dead = (j >= p.Nk) || (CAUSAL && j > qrow);
          if (dead) s[mt][i] = -INFINITY;
        }
    }

    float smax = fmaxf(s[0][0], s[0][1]);
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
      for (int i = (mt == 0 ? 2 : 0); i < 16; i += 2) smax = fmaxf(fmaxf(smax, s[mt][i]), s[mt][i + 1]);
    smax = partner_max(smax) - S_MAGIC_F;  // exact: both are integers below 2^24

    const float c = qsc * ksc_base[kb];
    const float m_new = fmaxf(m_i, smax * c);
    const float alpha = __builtin_amdgcn_exp2f(m_i - m_new);
    m_i = m_new;
    const float bias = fmaf(-S_MAGIC_F, c, P_EXP_OFFSET - m_new);

    v8i pf;
    float rs = 0.f;
#pragma unroll
    for (int r = 0; r < 8; r++) {
      const int mt = r >> 2, i0 = 4 * (r & 3);
      const float p0 = __builtin_amdgcn_exp2f(fmaf(s[mt][i0 + 0], c, bias));
      const float p1 = __builtin_amdgcn_exp2f(fmaf(s[mt][i0 + 1], c, bias));
      const float p2 = __builtin_amdgcn_exp2f(fmaf(s[mt][i0 + 2], c, bias));
      const float p3 = __builtin_amdgcn_exp2f(fmaf(s[mt][i0 + 3], c, bias));
      if constexpr (LSE) rs += (p0 + p1) + (p2 + p3);
      int w = __builtin_amdgcn_cvt_pk_fp8_f32(p0, p1, 0, false);
      w = __builtin_amdgcn_cvt_pk_fp8_f32(p2, p3, w, true);
      pf[r] = w;
    }
    if constexpr (LSE) d_exact = d_exact * alpha + rs;
    if (__ballot(alpha != 1.0f) != 0ull) {
      d_acc[0] *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT_TILES; dt++)
#pragma unroll
        for (int i = 0; i < 16; i++) o_acc[dt][i] *= alpha;
    }

    // O^T += V8^T . P~^T ; the row sums of the ROUNDED P~ come from one more MFMA against ones
    const uint8_t* vt = lds_v + buf * TILE;
#pragma unroll
    for (int dt = 0; dt < DT_TILES; dt++) {
      const v4i a0 = *reinterpret_cast<const v4i*>(vt + ((dt * 2 + 0) * 64 + lane) * 16);
      const v4i a1 = *reinterpret_cast<const v4i*>(vt + ((dt * 2 + 1) * 64 + lane) * 16);
      const v8i a = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
      o_acc[dt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, pf, o_acc[dt], 0, 0, 0, 0, 0, 0);
    }
    d_acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ones, pf, d_acc, 0, 0, 0, 0, 0, 0);

    if (more) store_tile(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: O = O~/d * v_scale + v_mean ------------------------------------------------
  const float d_tot = d_acc[0];
  const float inv = 1.0f / d_tot;
  if (qrow < p.Nq) {
    const float* vsc = p.v_scale + bhk * D;
    const float* vmn = p.v_mean ? p.v_mean + bhk * D : nullptr;
#pragma unroll
    for (int dt = 0; dt < DT_TILES; dt++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int ch = 32 * dt + 8 * g + 4 * lh;
        const v4f sc = *reinterpret_cast<const v4f*>(vsc + ch);
        v4f mn = {0.f, 0.f, 0.f, 0.f};
        if (vmn) mn = *reinterpret_cast<const v4f*>(vmn + ch);
        unsigned short r[4];
#pragma unroll
        for (int q = 0; q < 4; q++) r[q] = OutT::from_f32(fmaf(o_acc[dt][4 * g + q] * inv, sc[q], mn[q]));
        *reinterpret_cast<v2i*>(outp + ch) =
            v2i{(int)((unsigned)r[0] | ((unsigned)r[1] << 16)), (int)((unsigned)r[2] | ((unsigned)r[3] << 16))};
      }
    }
  }
  if constexpr (LSE) {
    // the log-sum-exp uses the exact fp32 row sum, not the sum of the FP8-rounded weights
    const float d_full = d_exact + __shfl_xor(d_exact, 32, 64);
    if (p.lse && qrow < p.Nq && lh == 0)
      p.lse[((int64_t)b * p.H + h) * p.Nq + qrow] = m_i + __builtin_amdgcn_logf(d_full) - P_EXP_OFFSET;
  }
}

template <int D, int OUT_DT, bool CAUSAL, bool DUMP, bool LSE>
static int launch_attn(const AttnParams& p, hipStream_t st) {
  const int grid = ((p.total + 7) / 8) * 8;
  const size_t smem = 4 * 64 * D + (((size_t)p.nbk * 2 + 15) & ~(size_t)15);
  auto kern = attn_sparse_kernel<D, OUT_DT, CAUSAL, DUMP, LSE>;
  if (smem > 48 * 1024)
    PARO_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
  hipLaunchKernelGGL(kern, dim3(grid), dim3(128), smem, st, p);
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}

template <int D, int OUT_DT>
static int dispatch_attn(const AttnParams& p, int is_causal, bool dump, hipStream_t st) {
  const bool lse = p.lse != nullptr;
  if (dump) {  // debug path: one instantiation per causal mode, always with the exact row sum
    if (is_causal) return launch_attn<D, OUT_DT, true, true, true>(p, st);
    return launch_attn<D, OUT_DT, false, true, true>(p, st);
  }
  if (is_causal) return lse ? launch_attn<D, OUT_DT, true, false, true>(p, st) : launch_attn<D, OUT_DT, true, false, false>(p, st);
  return lse ? launch_attn<D, OUT_DT, false, false, true>(p, st) : launch_attn<D, OUT_DT, false, false, false>(p, st);
}

}  // namespace paro

extern "C" int paro_attn_sparse_fwd(const int8_t* q8, const int8_t* k8, const uint8_t* v8, const float* q_scale,
                                    const float* k_scale, const float* v_scale, const float* v_mean,
                                    const uint8_t* sparse, int64_t sparse_batch_stride, void* out, int out_dtype,
                                    float* lse, int32_t* s_dump, int B, int H, int Hkv, int Nq, int Nk, int D,
                                    int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_n, int64_t k_stride_b,
                                    int64_t k_stride_h, int64_t k_stride_n, int64_t o_stride_b, int64_t o_stride_h,
                                    int64_t o_stride_n, float sm_scale, int is_causal, void* stream) {
  using namespace paro;
  PARO_CHECK(q8 && k8 && v8 && q_scale && k_scale && v_scale && sparse && out, PARO_ERR_RUNTIME,
             "paro_attn_sparse_fwd: null tensor pointer");
  PARO_CHECK(B > 0 && H > 0 && Hkv > 0 && Nq > 0 && Nk > 0, PARO_ERR_RUNTIME, "paro_attn_sparse_fwd: empty shape");
  PARO_CHECK(D == 64 || D == 128, PARO_ERR_INVALID_VALUE, "Unsupported head dim: %d", D);
  PARO_CHECK(H % Hkv == 0, PARO_ERR_INVALID_VALUE, "num_qo_heads (%d) must be divisible by num_kv_heads (%d)", H, Hkv);
  PARO_CHECK(is_causal == 0 || is_causal == 1, PARO_ERR_INVALID_VALUE, "Unsupported causal mode: %d", is_causal);
  PARO_CHECK(!is_causal || Nq == Nk, PARO_ERR_RUNTIME, "causal attention needs qo_len == kv_len (%d vs %d)", Nq, Nk);
  PARO_CHECK(out_dtype == PARO_DTYPE_F16 || out_dtype == PARO_DTYPE_BF16, PARO_ERR_RUNTIME,
             "Unsupported output dtype (expect float16 or bfloat16)");
  PARO_CHECK(((uintptr_t)q8 % 16) == 0 && ((uintptr_t)k8 % 16) == 0 && ((uintptr_t)v8 % 16) == 0 &&
                 q_stride_b % 16 == 0 && q_stride_h % 16 == 0 && q_stride_n % 16 == 0 && k_stride_b % 16 == 0 &&
                 k_stride_h % 16 == 0 && k_stride_n % 16 == 0,
             PARO_ERR_RUNTIME, "Tensor query/key must be 16-byte aligned with strides that are multiples of 16");
  PARO_CHECK(((uintptr_t)out % 16) == 0 && o_stride_b % 8 == 0 && o_stride_h % 8 == 0 && o_stride_n % 8 == 0,
             PARO_ERR_RUNTIME, "Tensor output must be 16-byte aligned with strides that are multiples of 8");
  PARO_CHECK(((uintptr_t)v_scale % 16) == 0 && ((uintptr_t)v_mean % 16) == 0, PARO_ERR_RUNTIME,
             "paro_attn_sparse_fwd: v_scale / v_mean must be 16-byte aligned");
  const int nbq = ceil_div(Nq, 64), nbk = ceil_div(Nk, 64);
  PARO_CHECK(nbk <= 65535, PARO_ERR_RUNTIME, "kv_len %d exceeds 65535 blocks of 64", Nk);
  PARO_CHECK((int64_t)B * H * nbq < (int64_t)1 << 31, PARO_ERR_RUNTIME, "paro_attn_sparse_fwd: too many q-blocks");
  AttnParams p;
  p.q8 = q8; p.k8 = k8; p.v8 = v8; p.q_scale = q_scale; p.k_scale = k_scale; p.v_scale = v_scale; p.v_mean = v_mean;
  p.sparse = sparse; p.out = out; p.lse = lse; p.s_dump = s_dump; p.sparse_bs = sparse_batch_stride;
  p.qs_b = q_stride_b; p.qs_h = q_stride_h; p.qs_n = q_stride_n;
  p.ks_b = k_stride_b; p.ks_h = k_stride_h; p.ks_n = k_stride_n;
  p.os_b = o_stride_b; p.os_h = o_stride_h; p.os_n = o_stride_n;
  p.B = B; p.H = H; p.Hkv = Hkv; p.Nq = Nq; p.Nk = Nk; p.nbq = nbq; p.nbk = nbk;
  p.total = B * H * nbq;
  p.sm_scale_log2e = sm_scale * 1.4426950408889634f;
  hipStream_t st = (hipStream_t)stream;
  const bool dump = s_dump != nullptr;
  if (D == 64) {
    if (out_dtype == PARO_DTYPE_F16) return dispatch_attn<64, PARO_DTYPE_F16>(p, is_causal, dump, st);
    return dispatch_attn<64, PARO_DTYPE_BF16>(p, is_causal, dump, st);
  }
  if (out_dtype == PARO_DTYPE_F16) return dispatch_attn<128, PARO_DTYPE_F16>(p, is_causal, dump, st);
  return dispatch_attn<128, PARO_DTYPE_BF16>(p, is_causal, dump, st);
}

extern "C" int64_t paro_attn_workspace_bytes(int B, int Hkv, int Nk, int D) {
  auto al = [](int64_t x) { return (x + 255) & ~(int64_t)255; };
  return al(paro_v_fp8_bytes(B, Hkv, Nk, D)) + 2 * al((int64_t)B * Hkv * D * 4) +
         al(paro_v_fp8_partial_floats(B, Hkv, Nk, D) * 4);
}

extern "C" int paro_qk_int8_sv_f16_attn(const int8_t* q8, const int8_t* k8, const void* v, int v_dtype, void* out,
                                        int out_dtype, const float* q_scale, const float* k_scale,
                                        const uint8_t* sparse, int64_t sparse_batch_stride, float* lse,
                                        void* workspace, int64_t workspace_bytes, int B, int H, int Hkv, int Nq,
                                        int Nk, int D, int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_n,
                                        int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_n,
                                        int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_n,
                                        int64_t o_stride_b, int64_t o_stride_h, int64_t o_stride_n,
                                        int tensor_layout, int is_causal, int qk_quant_gran, float sm_scale,
                                        int smooth_v, void* stream) {
  using namespace paro;
  PARO_CHECK(tensor_layout == 0 || tensor_layout == 1, PARO_ERR_INVALID_VALUE, "tensor_layout must be 0 or 1");
  PARO_CHECK(qk_quant_gran == 2 || qk_quant_gran == 3, PARO_ERR_INVALID_VALUE, "Unsupported quantization granularity: %d",
             qk_quant_gran);
  PARO_CHECK(qk_quant_gran == 2, PARO_ERR_UNSUPPORTED,
             "qk_quant_gran=3 (per_thread) is not implemented: quantise with per_warp (gran 2)");
  PARO_CHECK(workspace && ((uintptr_t)workspace % 256) == 0, PARO_ERR_RUNTIME,
             "paro_qk_int8_sv_f16_attn: workspace must be a 256-byte aligned device buffer");
  PARO_CHECK(B > 0 && Hkv > 0 && Nk > 0 && (D == 64 || D == 128), PARO_ERR_INVALID_VALUE,
             "Unsupported shape or head dim: B=%d Hkv=%d Nk=%d D=%d", B, Hkv, Nk, D);
  PARO_CHECK(workspace_bytes >= paro_attn_workspace_bytes(B, Hkv, Nk, D), PARO_ERR_RUNTIME,
             "paro_qk_int8_sv_f16_attn: workspace of %lld bytes is smaller than the %lld needed",
             (long long)workspace_bytes, (long long)paro_attn_workspace_bytes(B, Hkv, Nk, D));
  auto al = [](int64_t x) { return (x + 255) & ~(int64_t)255; };
  uint8_t* ws = (uint8_t*)workspace;
  uint8_t* v8 = ws;
  ws += al(paro_v_fp8_bytes(B, Hkv, Nk, D));
  float* v_scale = (float*)ws;
  ws += al((int64_t)B * Hkv * D * 4);
  float* v_mean = (float*)ws;
  ws += al((int64_t)B * Hkv * D * 4);
  float* partial = (float*)ws;
  int rc = paro_v_fp8_pack(v, v_dtype, v8, v_scale, v_mean, partial, B, Hkv, Nk, D, v_stride_b, v_stride_h,
                           v_stride_n, smooth_v, stream);
  if (rc) return rc;
  return paro_attn_sparse_fwd(q8, k8, v8, q_scale, k_scale, v_scale, smooth_v ? v_mean : nullptr, sparse,
                              sparse_batch_stride, out, out_dtype, lse, nullptr, B, H, Hkv, Nq, Nk, D, q_stride_b,
                              q_stride_h, q_stride_n, k_stride_b, k_stride_h, k_stride_n, o_stride_b, o_stride_h,
                              o_stride_n, sm_scale, is_causal, stream);
}
