// Block-sparse quantised attention with a 16-bit P.V product (PARO_ATTN_PV_F16), gfx950.
//
//   S^T = K8 . Q8^T      v_mfma_i32_32x32x32_i8      exact int32 (as in attn_sparse.hip)
//   P~  = 2^(S*c - m + 5) true exponentials, rounded to float16 (round to nearest even)
//   O^T += V16^T . P~^T  v_mfma_f32_32x32x16_f16     fp32 accumulation, V in float16 as given (no scale, no mean)
//   d   = sum_j P~       fp32, on the vector pipe
//
// This is the accuracy mode: what the reference's kernel of the same name computes, a float16 P.V product
// (csrc/qattn/qk_int_sv_f16_cuda_sm80.cu:263-391, attn_utils.cuh:383-488), where the default kernels of this
// library round P and V to FP8 e4m3.  An e4m3 code is up to 2^-4 off its value, and a q-row that one to three
// keys dominate carries that error undiluted; float16 is 2^-11.  The matrix pipe runs float16 at half the FP8
// rate and the weights need true exponentials, so this kernel is the slower one and is written for clarity, not
// tuned: two waves per 64-row q-block (32 q-rows each), a two-stage ring of K8 (int8) and V16 (float16) tiles
// moved by LDS-DMA one block ahead, one barrier per block, no software pipelining.  Mask semantics, scale
// indexing, the lazily refreshed maximum, edge columns, causal masking, the unpermuting store and the log-sum-exp
// are those of attn_sparse.hip.
//
// V16 tiles (paro_v_f16_pack): per (batch, kv-head, 64-token block) D/32 x 4 pieces of 1 KB; halfword e (0..7)
// of lane l of piece (dt, s) is token 64*kb + 32*(s/2) + 16*(s%2) + 8*(e/4) + 4*(l/32) + e%4, channel
// 32*dt + l%32: the A-operand fragment of v_mfma_f32_32x32x16_f16 under the kv-order that the S^T accumulator
// fragment imposes on the B operand (a lane's weights 8*(s%2) .. 8*(s%2)+7 of row tile s/2 are its B fragment of
// step s), so that no data moves between lanes from one product to the next.  Tokens past the end are 0.
#include "attn_common.hpp"

namespace paro {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));

template <int D> struct Pv16Lds {
  static constexpr int NST = 2;
  static constexpr int KTILE = 64 * D;        // int8, 16-byte chunks XOR-swizzled as in attn_sparse.hip
  static constexpr int VTILE = 64 * D * 2;    // float16, fragment order as in memory
  static constexpr int V_OFF = NST * KTILE;
  static constexpr int LIST_OFF = NST * (KTILE + VTILE);
  static constexpr int LIST_PAD = 8;
  static __device__ __forceinline__ int swz(int row) {
    if constexpr (D == 64) return (row >> 2) & 3;
    else return (row ^ (row >> 3)) & 7;
  }
};

template <int D, int OUT_DT>
__global__ void __launch_bounds__(128, 2) attn_sparse_pv16_kernel(const AttnParams p, const int causal) {
  using Lds = Pv16Lds<D>;
  constexpr int KS = D / 32;         // k-steps of the QK MFMA
  constexpr int DT_TILES = D / 32;   // 32-channel tiles of O^T
  constexpr int KPW = D / 32;        // 1 KB pieces of a K tile per wave (half a tile)
  constexpr int VPW = D / 16;        // 1 KB pieces of a V tile per wave
  constexpr int CPR = D / 16;        // 16-byte chunks per K row

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  float* clist = reinterpret_cast<float*>(smem + Lds::LIST_OFF);
  unsigned short* klist = reinterpret_cast<unsigned short*>(clist + p.nbk + Lds::LIST_PAD + 1);

  // XCD-aware renumbering: each XCD walks a contiguous range of (batch, head, q-block)
  const int per = gridDim.x >> 3;
  const int vid = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
  if (vid >= p.total) return;

  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int l32 = lane & 31, lh = lane >> 5;
  const int qb = vid % p.nbq, bh = vid / p.nbq;
  const int h = bh % p.H, b = bh / p.H;
  const int hk = h / (p.H / p.Hkv);
  const int64_t bhk = (int64_t)b * p.Hkv + hk;
  const int order_h = p.orders != nullptr ? p.orders[h] : 0;

  // ---- compact list of the kept key blocks and their scales (both waves build the same lists) ----
  const float* ksc_base = p.k_scale + bhk * p.nbk;
  const int kmax = causal ? min(p.nbk, qb + 1) : p.nbk;
  const uint8_t* mrow = p.sparse + b * p.sparse_bs + ((int64_t)h * p.nbq + qb) * p.nbk;
  const int trash = p.nbk + Lds::LIST_PAD;   // entries that are not kept go to this spare slot
  int cnt = 0;
  for (int base = 0; base < kmax; base += 64) {
    const int j = base + lane;
    const int jj = min(j, kmax - 1);
    const bool keep = mrow[jj] != 0 && j < kmax;
    const float sc = ksc_base[jj];
    const unsigned long long bal = __ballot(keep);
    const int pos = keep ? cnt + __popcll(bal & ((1ull << lane) - 1ull)) : trash;
    klist[pos] = (unsigned short)j;
    clist[pos] = sc;
    cnt += __popcll(bal);
  }
  if (cnt > 0 && lane < Lds::LIST_PAD) {   // the loop looks one block ahead without a branch
    klist[cnt + lane] = klist[cnt - 1];
    clist[cnt + lane] = clist[cnt - 1];
  }

  // ---- Q fragments and scale of this wave's 32 rows ----
  const int qrow = qb * 64 + wave * 32 + l32;
  v4i qf[KS];
  {
    const int8_t* qp = p.q8 + b * p.qs_b + h * p.qs_h + (int64_t)min(qrow, p.Nq - 1) * p.qs_n + 16 * lh;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[ks] = *reinterpret_cast<const v4i*>(qp + 32 * ks);
  }
  const float qsc = p.q_scale[((int64_t)b * p.H + h) * (p.nbq * 2) + qb * 2 + wave] * p.sm_scale_log2e;
  __syncthreads();

  using OutT = F16x<OUT_DT>;
  auto out_row_ptr = [&]() {
    int drow = qrow;
    if (p.orders != nullptr && qrow >= p.n_text && qrow < p.Nq)
      drow = p.n_text + unpermute_index(qrow - p.n_text, order_h, p.F, p.Hh, p.W);
    return reinterpret_cast<unsigned short*>(p.out) + b * p.os_b + h * p.os_h + (int64_t)drow * p.os_n;
  };
  if (cnt == 0) {  // no kept block: the row outputs 0 (reference: m = -5e6, d = 1, O = 0)
    if (qrow < p.Nq) {
      unsigned short* outp = out_row_ptr();
#pragma unroll
      for (int c = 0; c < D / 16; c++) *reinterpret_cast<v4i*>(outp + (lh * (D / 16) + c) * 8) = v4i{0, 0, 0, 0};
      if (p.lse && lh == 0) p.lse[((int64_t)b * p.H + h) * p.Nq + qrow] = -INFINITY;
    }
    return;
  }

  // ---- tile movers: each wave moves half of every tile, 1 KB per instruction ----
  const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      uniform_ptr(p.k8 + b * p.ks_b + hk * p.ks_h), 0, (int)((int64_t)(p.Nk - 1) * p.ks_n + D), 0x00020000);
  const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      uniform_ptr(p.v8 + bhk * p.nbk * (int64_t)Lds::VTILE), 0, p.nbk * Lds::VTILE, 0x00020000);
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  int k_goff[KPW];
#pragma unroll
  for (int i = 0; i < KPW; i++) {
    const int pos = (wave_u * KPW + i) * 1024 + lane * 16;   // byte position inside the LDS tile
    const int row = pos / D, cpos = (pos % D) / 16;
    k_goff[i] = row * (int)p.ks_n + ((cpos ^ Lds::swz(row)) * 16);
  }
  const int k_blk_stride = 64 * (int)p.ks_n;
  auto load_k = [&](int kb, int st) {   // rows >= Nk read as 0
#pragma unroll
    for (int i = 0; i < KPW; i++)
      buffer_load16_lds<0>(k_rsrc, smem + st * Lds::KTILE + (wave_u * KPW + i) * 1024, k_goff[i], kb * k_blk_stride);
  };
  auto load_v = [&](int kb, int st) {
#pragma unroll
    for (int i = 0; i < VPW; i++)
      buffer_load16_lds<0>(v_rsrc, smem + Lds::V_OFF + st * Lds::VTILE + (wave_u * VPW + i) * 1024, lane * 16,
                           kb * Lds::VTILE + (wave_u * VPW + i) * 1024);
  };

  // K fragment (ks, mt): row 32*mt + l32, chunk 2*ks + lh at its swizzled position
  int kr_off[2 * KS];
#pragma unroll
  for (int ks = 0; ks < KS; ks++)
#pragma unroll
    for (int mt = 0; mt < 2; mt++) {
      const int row = 32 * mt + l32;
      kr_off[ks * 2 + mt] = row * D + (((2 * ks + lh) ^ Lds::swz(row)) * 16);
    }

  // ---- state ----
  v16f o_acc[DT_TILES];
#pragma unroll
  for (int dt = 0; dt < DT_TILES; dt++)
#pragma unroll
    for (int i = 0; i < 16; i++) o_acc[dt][i] = 0.f;
  v16i magic;
#pragma unroll
  for (int i = 0; i < 16; i++) magic[i] = S_MAGIC_BITS;   // the int32 scores then read as floats 1.5*2^23 + S
  float m_i = -1e30f, m_thr = -1e30f, m_off = 0.f;
  float d_sum = 0.f;   // sum of this lane's weights (32 of the 64 columns of every block); partner lane: the rest

  load_k((int)klist[0], 0);
  load_v((int)klist[0], 0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  for (int it = 0; it < cnt; it++) {
    const int st = it & 1;
    const int kb = __builtin_amdgcn_readfirstlane((int)klist[it]);
    const int kb_next = __builtin_amdgcn_readfirstlane((int)klist[it + 1]);
    // the other stage was read during the previous iteration, whose closing barrier every wave has passed
    load_k(kb_next, st ^ 1);
    load_v(kb_next, st ^ 1);
    const float c = qsc * clist[it];

    // -- S^T = K . Q^T
    v16i acc[2];
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
#pragma unroll
      for (int mt = 0; mt < 2; mt++) {
        const v4i kf = *reinterpret_cast<const v4i*>(smem + st * Lds::KTILE + kr_off[ks * 2 + mt]);
        acc[mt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf, qf[ks], ks == 0 ? magic : acc[mt], 0, 0, 0);
      }
    float s[2][16];
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
      for (int i = 0; i < 16; i++) s[mt][i] = __int_as_float(acc[mt][i]);

    // -- columns past the end of K (last block) or above the diagonal (causal) leave the softmax
    const bool edge = (kb == p.nbk - 1 && (p.Nk & 63) != 0) || (causal && kb == qb);
    if (edge) {
      int thr = p.Nk - kb * 64 - 4 * lh;
      if (causal) thr = min(thr, qrow + 1 - kb * 64 - 4 * lh);
#pragma unroll
      for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const int cidx = 32 * mt + 8 * (i >> 2) + (i & 3);
          if (cidx >= thr) s[mt][i] = -INFINITY;
        }
    }

    // -- running maximum, refreshed only when a weight would exceed 2^(OFFSET + HEADROOM)
    // (four interleaved v_max3 chains; the values are integers read as floats: no NaN to canonicalise)
    float mx0 = max3(s[0][0], s[0][1], s[0][2]), mx1 = max3(s[0][8], s[0][9], s[0][10]);
    float mx2 = max3(s[1][0], s[1][1], s[1][2]), mx3 = max3(s[1][8], s[1][9], s[1][10]);
#pragma unroll
    for (int i = 3; i < 7; i += 2) {
      mx0 = max3(mx0, s[0][i], s[0][i + 1]);
      mx1 = max3(mx1, s[0][i + 8], s[0][i + 9]);
      mx2 = max3(mx2, s[1][i], s[1][i + 1]);
      mx3 = max3(mx3, s[1][i + 8], s[1][i + 9]);
    }
    mx0 = max3(mx0, s[0][7], s[0][15]);
    mx2 = max3(mx2, s[1][7], s[1][15]);
    const float smax = max3(max3(mx0, mx1, mx2), mx3, mx3);
    const float m_blk = fmaf(partner_max(smax), c, -S_MAGIC_F * c);
    if (__ballot(m_blk > m_thr) != 0ull) {
      const float m_new = fmaxf(m_i, m_blk);
      const float alpha = __builtin_amdgcn_exp2f(m_i - m_new);
      m_i = m_new;
      m_thr = m_new + P_HEADROOM;
      m_off = P_EXP_OFFSET - m_new;
      d_sum *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT_TILES; dt++)
#pragma unroll
        for (int i = 0; i < 16; i++) o_acc[dt][i] *= alpha;
    }
    const float bias = fmaf(-S_MAGIC_F, c, m_off);   // t = S*c - m + OFFSET from the biased score

    // -- weights: float16 pairs, in the order the B fragments of the four steps take them
    v2h pw[16];
    float rs = 0.f;
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
      for (int i = 0; i < 16; i += 2) {
        const float p0 = __builtin_amdgcn_exp2f(fmaf(s[mt][i], c, bias));
        const float p1 = __builtin_amdgcn_exp2f(fmaf(s[mt][i + 1], c, bias));
        rs += p0 + p1;
        v2h w;
        w[0] = (_Float16)p0;
        w[1] = (_Float16)p1;
        pw[mt * 8 + i / 2] = w;
      }
    d_sum += rs;

    // -- O^T += V^T . P~^T: step s = (row tile s/2, weights 8*(s%2) .. 8*(s%2)+7 of it)
#pragma unroll
    for (int sidx = 0; sidx < 4; sidx++) {
      v8h bfrag;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        bfrag[2 * j] = pw[4 * sidx + j][0];
        bfrag[2 * j + 1] = pw[4 * sidx + j][1];
      }
#pragma unroll
      for (int dt = 0; dt < DT_TILES; dt++) {
        const v8h afrag = *reinterpret_cast<const v8h*>(smem + Lds::V_OFF + st * Lds::VTILE + (dt * 4 + sidx) * 1024 +
                                                        lane * 16);
        o_acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afrag, bfrag, o_acc[dt], 0, 0, 0);
      }
    }

    // -- the next block's tiles have to have landed before the barrier publishes them; the barrier also says
    //    that every wave is done reading this stage
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
  }

  // ---- epilogue: O = O~ / d (times v_scale plus v_mean when the caller gives them) ----
  const float d_tot = d_sum + __shfl_xor(d_sum, 32, 64);
  const float inv = 1.0f / d_tot;
  if (qrow < p.Nq) {
    unsigned short* outp = out_row_ptr();
    const float* vsc = p.v_scale ? p.v_scale + bhk * D : nullptr;
    const float* vmn = p.v_mean ? p.v_mean + bhk * D : nullptr;
#pragma unroll
    for (int dt = 0; dt < DT_TILES; dt++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int ch = 32 * dt + 8 * g + 4 * lh;
        v4f sc = {1.f, 1.f, 1.f, 1.f}, mn = {0.f, 0.f, 0.f, 0.f};
        if (vsc) sc = *reinterpret_cast<const v4f*>(vsc + ch);
        if (vmn) mn = *reinterpret_cast<const v4f*>(vmn + ch);
        unsigned short r[4];
#pragma unroll
        for (int q = 0; q < 4; q++) r[q] = OutT::from_f32(fmaf(o_acc[dt][4 * g + q] * inv, sc[q], mn[q]));
        *reinterpret_cast<v2i*>(outp + ch) =
            v2i{(int)((unsigned)r[0] | ((unsigned)r[1] << 16)), (int)((unsigned)r[2] | ((unsigned)r[3] << 16))};
      }
    }
    if (p.lse && lh == 0)
      p.lse[((int64_t)b * p.H + h) * p.Nq + qrow] = m_i + __builtin_amdgcn_logf(d_tot) - P_EXP_OFFSET;
  }
}

template <int D, int OUT_DT>
static int launch_pv16(const AttnParams& p, bool causal, hipStream_t st) {
  const size_t smem = Pv16Lds<D>::LIST_OFF + (((size_t)(p.nbk + Pv16Lds<D>::LIST_PAD + 1) * 6 + 15) & ~(size_t)15);
  PARO_CHECK(smem <= 160 * 1024, PARO_ERR_RUNTIME, "kv_len %d: the list of %d key blocks does not fit the local data share",
             p.Nk, p.nbk);
  const int grid = ((p.total + 7) / 8) * 8;
  auto kern = attn_sparse_pv16_kernel<D, OUT_DT>;
  if (smem > 48 * 1024)
    PARO_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
  hipLaunchKernelGGL(kern, dim3(grid), dim3(128), smem, st, p, causal ? 1 : 0);
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}

int launch_attn_pv16(const AttnParams& p, int D, int out_dtype, bool causal, hipStream_t st) {
  if (D == 64) {
    if (out_dtype == PARO_DTYPE_F16) return launch_pv16<64, PARO_DTYPE_F16>(p, causal, st);
    return launch_pv16<64, PARO_DTYPE_BF16>(p, causal, st);
  }
  if (out_dtype == PARO_DTYPE_F16) return launch_pv16<128, PARO_DTYPE_F16>(p, causal, st);
  return launch_pv16<128, PARO_DTYPE_BF16>(p, causal, st);
}

// ---- V -> float16 tiles in fragment order ---------------------------------------------------------------
// One workgroup per (batch, kv-head, 64-token block): the block goes through LDS row by row (16-byte loads) and
// leaves as D/32 x 4 pieces of 1 KB (16 bytes per lane).
template <int DT, int D>
__global__ void __launch_bounds__(256) v_f16_pack_kernel(const unsigned short* __restrict__ v, unsigned short* __restrict__ out,
                                                         int Hkv, int N, int nb, int64_t sb, int64_t sh, int64_t sn) {
  __shared__ __attribute__((aligned(16))) unsigned short tile[64 * (D + 8)];   // rows padded by 16 bytes
  const int kb = blockIdx.x % nb, bh = blockIdx.x / nb;
  const int b = bh / Hkv, hk = bh % Hkv;
  const unsigned short* src = v + b * sb + hk * sh;
  constexpr int CPR = D / 8;   // 16-byte chunks per row
  for (int c = threadIdx.x; c < 64 * CPR; c += 256) {
    const int row = c / CPR, ch = c % CPR;
    const int tok = kb * 64 + row;
    v4i x = {0, 0, 0, 0};
    if (tok < N) x = *reinterpret_cast<const v4i*>(src + (int64_t)tok * sn + ch * 8);
    *reinterpret_cast<v4i*>(tile + row * (D + 8) + ch * 8) = x;
  }
  __syncthreads();
  unsigned short* dst = out + ((int64_t)bh * nb + kb) * (64 * D);
  for (int pl = threadIdx.x; pl < (D / 32) * 4 * 64; pl += 256) {
    const int lane = pl & 63, piece = pl >> 6;
    const int dt = piece >> 2, s = piece & 3;
    const int chn = 32 * dt + (lane & 31);
    unsigned short r[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const int row = 32 * (s >> 1) + 16 * (s & 1) + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
      const unsigned short raw = tile[row * (D + 8) + chn];
      r[e] = DT == PARO_DTYPE_F16 ? raw : F16x<PARO_DTYPE_F16>::from_f32(F16x<PARO_DTYPE_BF16>::to_f32(raw));
    }
    *reinterpret_cast<v4i*>(dst + (int64_t)pl * 8) =
        v4i{(int)(r[0] | ((unsigned)r[1] << 16)), (int)(r[2] | ((unsigned)r[3] << 16)),
            (int)(r[4] | ((unsigned)r[5] << 16)), (int)(r[6] | ((unsigned)r[7] << 16))};
  }
}

}  // namespace paro

extern "C" int64_t paro_v_f16_bytes(int B, int Hkv, int N, int D) {
  return (int64_t)B * Hkv * ((N + 63) / 64) * 64 * D * 2;
}

extern "C" int paro_v_f16_pack(const void* v, int dtype, void* v16, int B, int Hkv, int N, int D, int64_t v_stride_b,
                               int64_t v_stride_h, int64_t v_stride_n, void* stream) {
  using namespace paro;
  PARO_CHECK(v && v16, PARO_ERR_RUNTIME, "paro_v_f16_pack: null tensor pointer");
  PARO_CHECK(B > 0 && Hkv > 0 && N > 0, PARO_ERR_RUNTIME, "paro_v_f16_pack: empty shape");
  PARO_CHECK(D == 64 || D == 128, PARO_ERR_INVALID_VALUE, "Unsupported head dim: %d", D);
  PARO_CHECK(dtype == PARO_DTYPE_F16 || dtype == PARO_DTYPE_BF16, PARO_ERR_RUNTIME,
             "Unsupported input dtype (expect float16 or bfloat16)");
  PARO_CHECK(((uintptr_t)v % 16) == 0 && ((uintptr_t)v16 % 16) == 0 && v_stride_b % 8 == 0 && v_stride_h % 8 == 0 &&
                 v_stride_n % 8 == 0,
             PARO_ERR_RUNTIME, "Tensor value must be 16-byte aligned with strides that are multiples of 8");
  const int nb = (N + 63) / 64;
  PARO_CHECK((int64_t)B * Hkv * nb < (int64_t)1 << 31, PARO_ERR_RUNTIME, "paro_v_f16_pack: too many blocks");
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)(B * Hkv * nb));
#define PARO_V16(DTC, DD)                                                                                          \
  hipLaunchKernelGGL((v_f16_pack_kernel<DTC, DD>), grid, dim3(256), 0, st, (const unsigned short*)v,                \
                     (unsigned short*)v16, Hkv, N, nb, v_stride_b, v_stride_h, v_stride_n)
  if (dtype == PARO_DTYPE_F16) {
    if (D == 64) PARO_V16(PARO_DTYPE_F16, 64); else PARO_V16(PARO_DTYPE_F16, 128);
  } else {
    if (D == 64) PARO_V16(PARO_DTYPE_BF16, 64); else PARO_V16(PARO_DTYPE_BF16, 128);
  }
#undef PARO_V16
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}
