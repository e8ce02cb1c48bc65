// Block-sparse quantised attention for gfx950, head size 64: ONE wave per 64-row q-block.
//
// Same arithmetic as attn_sparse.hip (S^T = K8.Q8^T on v_mfma_i32_32x32x32_i8, base-2 online softmax with
// weights rounded to e4m3, O^T += V8^T.P~^T on v_mfma_f32_32x32x64_f8f6f4, row sums of the rounded weights from
// v_mfma_f32_16x16x128_f8f6f4), and bit-identical results.  What differs is who does it.  There, two waves
// share a q-block (32 q-rows each) and every K and V fragment read from LDS feeds one matrix instruction.
// Here one wave owns both 32-row halves A and B of the q-block, so every fragment it reads feeds two; the
// workgroup is a single wave, and nothing in the loop needs a barrier.  On this GPU the kernel's speed is set
// by the energy one kept block costs (the shader clock falls as the data movement per product rises), and
// halving the LDS reads per product is worth more than the third wave per SIMD that the narrower kernel has.
//
// The two halves are software-pipelined against each other inside the wave, so that matrix and vector
// instructions that do not depend on each other alternate in its instruction stream:
//   phase 1 of block i:  S_A(i+1) = K(i+1).Q_A,  O_A += V(i).P_A(i)   between the words of  P_B(i)   = weights of S_B(i)
//   phase 2 of block i:  S_B(i+1) = K(i+1).Q_B,  O_B += V(i).P_B(i)   between the words of  P_A(i+1) = weights of S_A(i+1)
// K8 and V8 tiles come in by LDS-DMA through two stages each (the wave moves whole tiles, two blocks ahead);
// their fragments are read once per block, right after the last product that used the previous ones.
//
// Semantics: qk_int_sv_f16_attn_kernel of the reference (csrc/qattn/qk_int_sv_f16_cuda_sm80.cu:44-726) as its
// host instantiates it (:1022-1048); see attn_sparse.hip for the line-by-line correspondence.
#include "attn_common.hpp"
#include <stdlib.h>

namespace paro {

struct W64Lds {
  static constexpr int D = 64;
  static constexpr int KTILE = 64 * D;   // 64 rows of D bytes, 16-byte chunks XOR-swizzled (as attn_sparse.hip)
  static constexpr int VTILE = 64 * D;   // fragment order, as in HBM
  static constexpr int V_OFF = 2 * KTILE;
  static constexpr int EPI_OFF = 2 * (KTILE + VTILE);
  static constexpr int EPI_BYTES = 2 * D * 4;   // v_scale and v_mean of the head
  static constexpr int LIST_OFF = EPI_OFF + EPI_BYTES;
  static constexpr int LIST_PAD = 8;
  static __device__ __forceinline__ int swz(int row) { return (row >> 2) & 3; }
};

template <int N> using IC = std::integral_constant<int, N>;

// The lane number, computed where it is needed.  (The rare paths of the loop and the epilogue derive half a
// dozen values from it; taken from threadIdx they would all be kept in registers across the loop, which has
// none to spare.  Opaque to the compiler so that it is not hoisted back.)
__device__ __forceinline__ int lane_here() {
  int x;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(x));
  return x;
}

template <int OUT_DT, bool CAUSAL, bool EXACT>
__device__ __forceinline__ void attn_qblock_w64(const AttnParams& p, const int vid) {
  using Lds = W64Lds;
  constexpr int D = 64;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  float* clist = reinterpret_cast<float*>(smem + Lds::LIST_OFF);  // [nbk + LIST_PAD + 1] k_scale of kept blocks
  unsigned short* klist = reinterpret_cast<unsigned short*>(clist + p.nbk + Lds::LIST_PAD + 1);  // their indices

  const int lane = threadIdx.x;
  const int l32 = lane & 31, lh = lane >> 5;
  const int qb = vid % p.nbq;
  const int bh = vid / p.nbq;
  const int h = bh % p.H, b = bh / p.H;
  const int hk = h / (p.H / p.Hkv);
  const int64_t bhk = (int64_t)b * p.Hkv + hk;

  // ---- everything the q-block needs from memory before its first tile, requested in one go ------------
  const int order_h = p.orders != nullptr ? p.orders[h] : 0;
  const float* ksc_base = p.k_scale + bhk * p.nbk;
  const int kmax = CAUSAL ? min(p.nbk, qb + 1) : p.nbk;
  const uint8_t* mrow = p.sparse + b * p.sparse_bs + ((int64_t)h * p.nbq + qb) * p.nbk;
  constexpr int MU = 8;   // 64 x MU blocks per pass
  uint8_t m[MU];
  float msc[MU];
  auto list_load = [&](int base) {
#pragma unroll
    for (int u = 0; u < MU; u++) {
      const int j = min(base + u * 64 + lane, kmax - 1);   // past the end: the last entry again
      m[u] = mrow[j];
      msc[u] = ksc_base[j];
    }
  };
  const int trash = p.nbk + Lds::LIST_PAD;   // spare slot for entries that are not kept
  int cnt = 0;
  auto list_take = [&](int base) {
#pragma unroll
    for (int u = 0; u < MU; u++) {
      const int j = base + u * 64 + lane;
      const bool keep = m[u] != 0 && j < kmax;
      const unsigned long long bal = __ballot(keep);
      const int pos = keep ? cnt + __popcll(bal & ((1ull << lane) - 1ull)) : trash;
      klist[pos] = (unsigned short)j;
      clist[pos] = msc[u];
      cnt += __popcll(bal);
    }
  };
  list_load(0);

  // Q fragments of both halves (B operand: column = q-row, 16 channels per lane and k-step)
  int qrow[2];
  v4i qf[2][2];
  float qsc[2];
#pragma unroll
  for (int hf = 0; hf < 2; hf++) {
    qrow[hf] = qb * 64 + hf * 32 + l32;
    // rows past the end re-read the last row; their results are never stored
    const int8_t* qp = p.q8 + b * p.qs_b + h * p.qs_h + (int64_t)min(qrow[hf], p.Nq - 1) * p.qs_n + 16 * lh;
#pragma unroll
    for (int ks = 0; ks < 2; ks++) qf[hf][ks] = *reinterpret_cast<const v4i*>(qp + 32 * ks);
    qsc[hf] = p.q_scale[((int64_t)b * p.H + h) * (p.nbq * 2) + qb * 2 + hf] * p.sm_scale_log2e;
  }
  float* epi = reinterpret_cast<float*>(smem + Lds::EPI_OFF);   // [2][D]: v_scale, v_mean
  const float epi_sc = p.v_scale[bhk * D + lane];
  const float epi_mn = p.v_mean ? p.v_mean[bhk * D + lane] : 0.f;

  list_take(0);
  for (int base = 64 * MU; base < kmax; base += 64 * MU) {
    list_load(base);
    list_take(base);
  }
  // the loop requests tiles up to 3 blocks ahead without branching: pad with the last kept block
  if (cnt > 0 && lane < Lds::LIST_PAD) {
    klist[cnt + lane] = klist[cnt - 1];
    clist[cnt + lane] = clist[cnt - 1];
  }
  epi[lane] = epi_sc;
  epi[D + lane] = epi_mn;
  __syncthreads();   // (one wave: orders the LDS writes above before the reads below)

  using OutT = F16x<OUT_DT>;
  auto out_row_ptr = [&](int row) {
    int drow = row;
    if (p.orders != nullptr && row >= p.n_text && row < p.Nq)
      drow = p.n_text + unpermute_index(row - p.n_text, order_h, p.F, p.Hh, p.W);
    return reinterpret_cast<unsigned short*>(p.out) + b * p.os_b + h * p.os_h + (int64_t)drow * p.os_n;
  };

  if (cnt == 0) {  // no kept block: the rows output 0 (reference: m = -5e6, d = 1, O = 0)
#pragma unroll
    for (int hf = 0; hf < 2; hf++)
      if (qrow[hf] < p.Nq) {
        unsigned short* outp = out_row_ptr(qrow[hf]);
#pragma unroll
        for (int c = 0; c < D / 16; c++) *reinterpret_cast<v4i*>(outp + (lh * (D / 16) + c) * 8) = v4i{0, 0, 0, 0};
      }
    return;
  }

  // ---- tile movers: the wave moves whole tiles, 1 KB per LDS-DMA instruction ---------------------------
  const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      uniform_ptr(p.k8 + b * p.ks_b + hk * p.ks_h), 0, (int)((int64_t)(p.Nk - 1) * p.ks_n + D), 0x00020000);
  const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      uniform_ptr(p.v8 + bhk * p.nbk * (int64_t)Lds::VTILE), 0, p.nbk * Lds::VTILE, 0x00020000);
  // LDS byte position i * 1024 + lane * 16 of a K tile is row 16 * i + lane / 4, chunk position lane % 4, which
  // holds chunk (lane % 4) ^ swz(row); swz(row) = (lane / 16) % 4 whatever i is, so the four pieces of a tile share
  // one per-lane offset and differ by 16 rows less the immediate 1024 that the instruction adds on both sides
  const int k_goff = (lane >> 2) * (int)p.ks_n + (((lane & 3) ^ Lds::swz(lane >> 2)) * 16);
  const int k_piece_stride = 16 * (int)p.ks_n - 1024;
  const int v_goff = lane * 16;
  const int k_blk_stride = 64 * (int)p.ks_n;
  auto load_k = [&](int kb, int ST) {  // rows >= Nk read as 0
    uint8_t* base = smem + ST * Lds::KTILE;
    buffer_load16_lds<0>(k_rsrc, base, k_goff, kb * k_blk_stride);
    buffer_load16_lds<1024>(k_rsrc, base, k_goff, kb * k_blk_stride + k_piece_stride);
    buffer_load16_lds<2048>(k_rsrc, base, k_goff, kb * k_blk_stride + 2 * k_piece_stride);
    buffer_load16_lds<3072>(k_rsrc, base, k_goff, kb * k_blk_stride + 3 * k_piece_stride);
  };
  auto load_v = [&](int kb, int ST) {
    uint8_t* base = smem + Lds::V_OFF + ST * Lds::VTILE;
    buffer_load16_lds<0>(v_rsrc, base, v_goff, kb * Lds::VTILE);
    buffer_load16_lds<1024>(v_rsrc, base, v_goff, kb * Lds::VTILE);
    buffer_load16_lds<2048>(v_rsrc, base, v_goff, kb * Lds::VTILE);
    buffer_load16_lds<3072>(v_rsrc, base, v_goff, kb * Lds::VTILE);
  };
  // one 1 KB piece of a tile (the loop spreads its eight DMA instructions over the block's matrix products: a wave
  // that issues them in one batch sits behind the CU's address unit, 16 cycles per instruction, for their duration)
  auto load_k_piece = [&](int kb, int ST, auto ic) {
    constexpr int I = decltype(ic)::value;
    buffer_load16_lds<I * 1024>(k_rsrc, smem + ST * Lds::KTILE, k_goff, kb * k_blk_stride + I * k_piece_stride);
  };
  auto load_v_piece = [&](int kb, int ST, auto ic) {
    constexpr int I = decltype(ic)::value;
    buffer_load16_lds<I * 1024>(v_rsrc, smem + Lds::V_OFF + ST * Lds::VTILE, v_goff, kb * Lds::VTILE);
  };
  constexpr int LOADS_PER_IT = 8;  // DMA instructions per block

  // ---- fragments ------------------------------------------------------------------------------------
  v4i kfrag[4];       // (ks, mt) at ks*2 + mt: row 32*mt + l32, chunk 2*ks + lh at its swizzled position
  v4i vfrag[2][2];    // (dt, mt)
  // row 32*mt + l32 has the swizzle of row l32; chunk 2*ks + lh sits at position (2*ks + lh) ^ swz: the two k-steps
  // differ in bit 1 of the position (32 bytes), the two row tiles by 2048 bytes (an immediate offset)
  const int kr_0 = l32 * D + ((lh ^ Lds::swz(l32)) * 16);
  const int kr_1 = kr_0 ^ 32;
  const int vr_base = Lds::V_OFF + lane * 16;
  auto read_k_frags = [&](int ST) {
#pragma unroll
    for (int i = 0; i < 4; i++)
      kfrag[i] = *reinterpret_cast<const v4i*>(smem + ST * Lds::KTILE + ((i >> 1) ? kr_1 : kr_0) + (i & 1) * 2048);
  };
  auto read_v_frags = [&](int ST) {
#pragma unroll
    for (int dt = 0; dt < 2; dt++)
#pragma unroll
      for (int mt = 0; mt < 2; mt++)
        vfrag[dt][mt] = *reinterpret_cast<const v4i*>(smem + ST * Lds::VTILE + vr_base + (dt * 2 + mt) * 1024);
  };

  // S^T accumulators start at the bit pattern of 1.5*2^23: the int32 result READS as the float 12582912 + S
  v16i magic;
#pragma unroll
  for (int i = 0; i < 16; i++) magic[i] = S_MAGIC_BITS;
  asm volatile("" : "+v"(magic));   // resident constant block
  v16i acc[2][2];                   // [half][row tile of the 64 kv-rows]
  auto qk_one = [&](auto hfc, int idx) {   // idx = 0..3: (mt, ks) = (idx & 1, idx >> 1)
    constexpr int hf = decltype(hfc)::value;
    const int mt = idx & 1, ks = idx >> 1;
    if (ks == 0) acc[hf][mt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kfrag[mt], qf[hf][0], magic, 0, 0, 0);
    else acc[hf][mt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kfrag[2 + mt], qf[hf][1], acc[hf][mt], 0, 0, 0);
  };

  // ---- state ------------------------------------------------------------------------------------------
  v16f o_acc[2][2];   // [half][32-channel tile]
#pragma unroll
  for (int hf = 0; hf < 2; hf++)
#pragma unroll
    for (int dt = 0; dt < 2; dt++)
#pragma unroll
      for (int i = 0; i < 16; i++) o_acc[hf][dt][i] = 0.f;
  // row sums of the rounded weights: selector operand as in attn_sparse.hip (lanes 0..15 get the sums of
  // q-rows lane and lane + 16 of the half in [0] and [1])
  v4f d_acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  v4f d_new[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};   // sums including the newest block, not yet accepted
  const int sel_word = ((lane & 15) == ((lane >> 4) & 1)) ? FP8_ONES : 0;
  v8i ones = {sel_word, sel_word, sel_word, sel_word, sel_word, sel_word, sel_word, sel_word};
  asm volatile("" : "+v"(ones));
  float m_i[2] = {-1e30f, -1e30f};
  float m_thr[2] = {-1e30f, -1e30f}, m_off[2] = {0.f, 0.f}, m_off8[2] = {0.f, 0.f};
  v8i pf[2];   // the weights of the newest block of each half, eight words of four e4m3 values

  auto pv_one = [&](auto hfc, int dt) {
    constexpr int hf = decltype(hfc)::value;
    const v8i a = {vfrag[dt][0][0], vfrag[dt][0][1], vfrag[dt][0][2], vfrag[dt][0][3],
                   vfrag[dt][1][0], vfrag[dt][1][1], vfrag[dt][1][2], vfrag[dt][1][3]};
    o_acc[hf][dt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, pf[hf], o_acc[hf][dt], 0, 0, 0, 0, 0, 0);
  };
  auto row_sums = [&](auto hfc) {
    constexpr int hf = decltype(hfc)::value;
    d_new[hf] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ones, pf[hf], d_acc[hf], 0, 0, 0, 0, 0, 0);
  };

  // columns past the end of K (last block) or above the diagonal (causal) leave the softmax: their scores
  // become -inf in place (one threshold per lane; the element of row tile mt, register i is column
  // kb*64 + 4*lh + 32*mt + 8*(i/4) + i%4)
  auto mask_edge = [&](auto hfc, int kb) {
    constexpr int hf = decltype(hfc)::value;
    const bool edge = (kb == p.nbk - 1 && (p.Nk & 63) != 0) || (CAUSAL && kb == qb);
    if (edge) {
      int kb_e = kb;
      asm volatile("" : "+s"(kb_e));   // opaque: otherwise 32 lane masks are hoisted into scalar registers
      const int ln = lane_here();
      int thr = p.Nk - kb_e * 64 - 4 * (ln >> 5);
      if constexpr (CAUSAL) thr = min(thr, qb * 64 + hf * 32 + (ln & 31) + 1 - kb_e * 64 - 4 * (ln >> 5));
#pragma unroll
      for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const int cidx = 32 * mt + 8 * (i >> 2) + (i & 3);
          if (cidx >= thr) acc[hf][mt][i] = (int)0xFF800000u;
        }
    }
  };
  // row maximum of the scores in acc[hf] as a log2-domain value (c: the block's scale)
  auto block_max = [&](auto hfc, float c) {
    constexpr int hf = decltype(hfc)::value;
    auto S = [&](int mt, int i) { return __int_as_float(acc[hf][mt][i]); };
    float mx0 = max3(S(0, 0), S(0, 1), S(0, 2)), mx1 = max3(S(0, 8), S(0, 9), S(0, 10));
    float mx2 = max3(S(1, 0), S(1, 1), S(1, 2)), mx3 = max3(S(1, 8), S(1, 9), S(1, 10));
#pragma unroll
    for (int i = 3; i < 7; i += 2) {
      mx0 = max3(mx0, S(0, i), S(0, i + 1));
      mx1 = max3(mx1, S(0, i + 8), S(0, i + 9));
      mx2 = max3(mx2, S(1, i), S(1, i + 1));
      mx3 = max3(mx3, S(1, i + 8), S(1, i + 9));
    }
    mx0 = max3(mx0, S(0, 7), S(0, 15));
    mx2 = max3(mx2, S(1, 7), S(1, 15));
    float smax = max3(mx0, mx1, mx2);
    smax = max3(smax, mx3, mx3);
    return fmaf(partner_max(smax), c, -S_MAGIC_F * c);
  };
  // refresh of the running maximum of one half: O and the accepted row sums are rescaled on the spot
  auto apply_refresh = [&](auto hfc, float m_blk) {
    constexpr int hf = decltype(hfc)::value;
    const float m_new = fmaxf(m_i[hf], m_blk);
    const float alpha = __builtin_amdgcn_exp2f(m_i[hf] - m_new);
    m_i[hf] = m_new;
    m_thr[hf] = m_new + P_HEADROOM;
    m_off[hf] = P_EXP_OFFSET - m_new;
    m_off8[hf] = (8.0f * (P_EXP_OFFSET + 7.0f - m_new) + FAST_EXP_SHIFT + 0.5f) * FAST_FIELD_SCALE;
    d_acc[hf][0] *= alpha;                                    // lanes 0..15: q-row lane
    d_acc[hf][1] *= __shfl(alpha, (lane_here() & 15) + 16, 64);   // and q-row lane + 16
#pragma unroll
    for (int dt = 0; dt < 2; dt++)
#pragma unroll
      for (int i = 0; i < 16; i++) o_acc[hf][dt][i] *= alpha;
  };
  // word r (0..7) of the weights of half hf: word r%4 of row tile r/4.  Fast path: the e4m3 byte is built
  // directly (attn_sparse.hip describes the field arithmetic); a weight above 448 comes out as the NaN byte.
  auto word_fma = [&](auto hfc, float (&ub)[2][4], int r, float cs, float bs) {   // cs, bs: the affine map
    constexpr int hf = decltype(hfc)::value;
    const int mt = r >> 2, i0 = 4 * (r & 3);
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const float s = __int_as_float(acc[hf][mt][i0 + q]);
      if constexpr (EXACT) ub[r & 1][q] = __builtin_amdgcn_exp2f(fmaf(s, cs, bs));
      else ub[r & 1][q] = fma_clamp01(s, cs, bs);
    }
  };
  auto word_pack = [&](auto hfc, float (&ub)[2][4], int r) {
    constexpr int hf = decltype(hfc)::value;
    const float* u = ub[r & 1];
    if constexpr (EXACT) {
      int w;
      cvt_pk_fp8<false>(w, u[0], u[1]);
      cvt_pk_fp8<true>(w, u[2], u[3]);
      pf[hf][r] = w;
    } else {
      const int lo = cvt_pknorm_i16(u[0], u[2]);
      const int hi = cvt_pknorm_i16(u[1], u[3]);
      pf[hf][r] = (int)__builtin_amdgcn_perm((unsigned)hi, (unsigned)lo, 0x07030501u);
    }
  };
  // scale and offset of the affine map score -> exponent (exact) or -> byte field (fast) for block scale c
  auto affine = [&](auto hfc, float c, float& cs, float& bs) {
    constexpr int hf = decltype(hfc)::value;
    if constexpr (EXACT) {
      cs = c;
      bs = fmaf(-S_MAGIC_F, c, m_off[hf]);
    } else {
      cs = (8.0f * FAST_FIELD_SCALE) * c;
      bs = fmaf(-S_MAGIC_F, cs, m_off8[hf]);
    }
  };
  // all eight words and their row sums at once (first block of a half, and the rare second pass)
  auto all_words = [&](auto hfc, float c) {
    float cs, bs;
    float ub[2][4];
    affine(hfc, c, cs, bs);
    word_fma(hfc, ub, 0, cs, bs);
#pragma unroll
    for (int r = 0; r < 8; r++) {
      if (r + 1 < 8) word_fma(hfc, ub, r + 1, cs, bs);
      word_pack(hfc, ub, r);
    }
    row_sums(hfc);
  };

  int kb_c = __builtin_amdgcn_readfirstlane((int)klist[0]);
  int kb_1 = __builtin_amdgcn_readfirstlane((int)klist[1]);
  int kb_2 = __builtin_amdgcn_readfirstlane((int)klist[2]);
  int kb_3 = __builtin_amdgcn_readfirstlane((int)klist[3]);
  // (the q scales are the same in every lane: scalar registers from here on)
  qsc[0] = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(qsc[0])));
  qsc[1] = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(qsc[1])));

  // One phase.  X: the half whose products are issued (S_X of the next block, O_X of this one); Y = 1 - X: the
  // half whose weights are computed, from the scores of block list entry `yi` (block number kb_y).  xi: list
  // entry of the block whose weights pf[X] are waiting to be accepted.  LAST: no next block.  (The first block's
  // maxima are taken in the prologue: no phase has to ask whether it is the first.)
  // after_qk / after_pv: hooks that read the next fragments once the products using the old ones are issued.
  auto phase = [&](auto xc, auto lastc, int xi, int yi, int kb_y, auto&& after_qk, auto&& after_pv,
                   auto&& piece) {
    constexpr int X = decltype(xc)::value, Y = 1 - X;
    constexpr bool LAST = decltype(lastc)::value != 0;
    constexpr bool WEIGHTS = !(LAST && X == 1);   // the last phase of a q-block has no weights left to compute
    const IC<Y> yc;
    float cs = 0.f, bs = 0.f;
    float ub[2][4];
    if constexpr (WEIGHTS) {
      const float c = qsc[Y] * clist[yi];
      mask_edge(yc, kb_y);
      if constexpr (EXACT) {
        const float m_blk = block_max(yc, c);
        if (__ballot(m_blk > m_thr[Y]) != 0ull) apply_refresh(yc, m_blk);
      }
      affine(yc, c, cs, bs);
      word_fma(yc, ub, 0, cs, bs);
      word_fma(yc, ub, 1, cs, bs);
      word_pack(yc, ub, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    // accept the weights of half X (fast path: unless one of them overflowed e4m3, seen as a NaN row sum; then
    // the maximum is refreshed and the words are computed again: the scores are still in acc[X])
    if constexpr (!EXACT) {
      if (__ballot(__builtin_isunordered(d_new[X][0], d_new[X][1])) != 0ull) {
        const float cx = qsc[X] * clist[xi];
        apply_refresh(xc, block_max(xc, cx));
        all_words(xc, cx);
      }
    }
    d_acc[X] = d_new[X];
    __builtin_amdgcn_sched_barrier(0);
    // matrix and vector instructions alternate: a word is 7 instructions (9.5 with true exponentials)
    if constexpr (!LAST) {
      qk_one(xc, 0);
      piece(IC<0>{});
      __builtin_amdgcn_sched_barrier(0);
      word_fma(yc, ub, 2, cs, bs); word_pack(yc, ub, 1);
      __builtin_amdgcn_sched_barrier(0);
      qk_one(xc, 1);
      piece(IC<1>{});
      __builtin_amdgcn_sched_barrier(0);
      word_fma(yc, ub, 3, cs, bs); word_pack(yc, ub, 2);
      __builtin_amdgcn_sched_barrier(0);
      qk_one(xc, 2);
      piece(IC<2>{});
      __builtin_amdgcn_sched_barrier(0);
      word_fma(yc, ub, 4, cs, bs); word_pack(yc, ub, 3);
      __builtin_amdgcn_sched_barrier(0);
      qk_one(xc, 3);
      piece(IC<3>{});
      __builtin_amdgcn_sched_barrier(0);
      after_qk();
      word_fma(yc, ub, 5, cs, bs); word_pack(yc, ub, 4);
      __builtin_amdgcn_sched_barrier(0);
      pv_one(xc, 0);
      __builtin_amdgcn_sched_barrier(0);
      word_fma(yc, ub, 6, cs, bs); word_pack(yc, ub, 5);
      __builtin_amdgcn_sched_barrier(0);
      pv_one(xc, 1);
      __builtin_amdgcn_sched_barrier(0);
      after_pv();
      word_fma(yc, ub, 7, cs, bs); word_pack(yc, ub, 6);
      word_pack(yc, ub, 7);
      __builtin_amdgcn_sched_barrier(0);
      row_sums(yc);
    } else {
      pv_one(xc, 0);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (WEIGHTS) {
#pragma unroll
        for (int r = 2; r < 5; r++) { word_fma(yc, ub, r, cs, bs); word_pack(yc, ub, r - 1); }
      }
      __builtin_amdgcn_sched_barrier(0);
      pv_one(xc, 1);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (WEIGHTS) {
#pragma unroll
        for (int r = 5; r < 8; r++) { word_fma(yc, ub, r, cs, bs); word_pack(yc, ub, r - 1); }
        word_pack(yc, ub, 7);
        __builtin_amdgcn_sched_barrier(0);
        row_sums(yc);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  auto nothing = [&]() {};
  auto no_piece = [&](auto) {};

  // ---- prologue ---------------------------------------------------------------------------------------------
  // stage of block j is j % 2 for K and for V.  Block `it` enters its iteration with K(it+1) and V(it) in
  // registers, S_B(it) in acc[1], the weights P_A(it) in pf[0] with their row sums waiting in d_new[0], and
  // K(it+2) on its way into stage it % 2; the iteration requests K(it+3) and V(it+2).
  load_k(kb_c, 0);
  load_k(kb_1, 1);
  load_v(kb_c, 0);
  load_v(kb_1, 1);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  read_k_frags(0);
#pragma unroll
  for (int i = 0; i < 4; i++) qk_one(IC<0>{}, i);
#pragma unroll
  for (int i = 0; i < 4; i++) qk_one(IC<1>{}, i);
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // K(0) is in registers: its stage may be refilled
  load_k(kb_2, 0);
  read_k_frags(1);
  read_v_frags(0);
  {
    // the first block gives both halves their first maximum (the fast path does not search one again unless a
    // weight overflows); half A's weights of it are due before the loop
    const float ks0 = clist[0];
    mask_edge(IC<0>{}, kb_c);
    mask_edge(IC<1>{}, kb_c);
    apply_refresh(IC<0>{}, block_max(IC<0>{}, qsc[0] * ks0));
    if constexpr (!EXACT) apply_refresh(IC<1>{}, block_max(IC<1>{}, qsc[1] * ks0));
    all_words(IC<0>{}, qsc[0] * ks0);
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");

  // One block that has a successor.  ST = it % 2.
  auto body = [&](auto stc, int it) {
    constexpr int ST = decltype(stc)::value;
    const int kidx_v = (int)klist[it + 4];
    __builtin_amdgcn_sched_barrier(0);
    phase(IC<0>{}, IC<0>{}, it, it, kb_c, nothing, nothing,
          [&](auto ic) { load_k_piece(kb_3, ST ^ 1, ic); });   // K(it+3) into the stage K(it+1) has left
    phase(IC<1>{}, IC<0>{}, it, it + 1, kb_1,
          [&]() {   // K(it+2) and V(it+1) have landed: everything older than the last eight requests has
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LOADS_PER_IT) : "memory");
            read_k_frags(ST);
          },
          [&]() { read_v_frags(ST ^ 1); },
          [&](auto ic) { load_v_piece(kb_2, ST, ic); });       // V(it+2) into the stage V(it) has left
    const int kb_4 = __builtin_amdgcn_readfirstlane(kidx_v);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    kb_c = kb_1; kb_1 = kb_2; kb_2 = kb_3; kb_3 = kb_4;
  };

  const int last = cnt - 1;
  for (int it = 0; it < last; it += 2) {
    body(IC<0>{}, it);
    if (it + 1 >= last) break;
    body(IC<1>{}, it + 1);
  }
  // the last kept block: O += V.P of both halves and the weights of half B
  phase(IC<0>{}, IC<1>{}, last, last, kb_c, nothing, nothing, no_piece);
  phase(IC<1>{}, IC<1>{}, last, last, kb_c, nothing, nothing, no_piece);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // DMA of the padded tail blocks: nobody reads it

  // ---- epilogue: O = O~/d * v_scale + v_mean ------------------------------------------------------------
  const int ln = lane_here(), e32 = ln & 31, eh = ln >> 5;
#pragma unroll
  for (int hf = 0; hf < 2; hf++) {
    const float d_lo = __shfl(d_acc[hf][0], e32 & 15, 64), d_hi = __shfl(d_acc[hf][1], e32 & 15, 64);
    const float inv = 1.0f / (e32 < 16 ? d_lo : d_hi);
    const int row = qb * 64 + hf * 32 + e32;
    if (row < p.Nq) {
      unsigned short* outp = out_row_ptr(row);
#pragma unroll
      for (int dt = 0; dt < 2; dt++) {
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const int ch = 32 * dt + 8 * g + 4 * eh;
          const v4f sc = *reinterpret_cast<const v4f*>(epi + ch);
          const v4f mn = *reinterpret_cast<const v4f*>(epi + D + ch);
          unsigned short r[4];
#pragma unroll
          for (int q = 0; q < 4; q++) r[q] = OutT::from_f32(fmaf(o_acc[hf][dt][4 * g + q] * inv, sc[q], mn[q]));
          *reinterpret_cast<v2i*>(outp + ch) =
              v2i{(int)((unsigned)r[0] | ((unsigned)r[1] << 16)), (int)((unsigned)r[2] | ((unsigned)r[3] << 16))};
        }
      }
    }
  }
}

template <int OUT_DT, bool CAUSAL, bool EXACT>
__global__ void __launch_bounds__(64, 2) attn_sparse_w64_kernel(const AttnParams p) {
  // XCD-aware renumbering: hardware deals workgroup ids round-robin to the 8 XCDs; each XCD walks a contiguous
  // range of (batch, head, q-block), so the K8 / V8 of the head it is working on stay in its own L2
  const int per = gridDim.x >> 3;
  const int vid = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
  if (vid >= p.total) return;
  attn_qblock_w64<OUT_DT, CAUSAL, EXACT>(p, vid);
}

template <int OUT_DT, bool CAUSAL, bool EXACT>
static int launch_w64(const AttnParams& p, hipStream_t st) {
  const size_t smem = W64Lds::LIST_OFF + (((size_t)(p.nbk + W64Lds::LIST_PAD + 1) * 6 + 15) & ~(size_t)15);
  const int grid = ((p.total + 7) / 8) * 8;
  auto kern = attn_sparse_w64_kernel<OUT_DT, CAUSAL, EXACT>;
  if (smem > 48 * 1024)
    PARO_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64), smem, st, p);
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}

int launch_attn_w64(const AttnParams& p, int out_dtype, bool causal, bool exact, hipStream_t st) {
  if (out_dtype == PARO_DTYPE_F16) {
    if (causal) return exact ? launch_w64<PARO_DTYPE_F16, true, true>(p, st) : launch_w64<PARO_DTYPE_F16, true, false>(p, st);
    return exact ? launch_w64<PARO_DTYPE_F16, false, true>(p, st) : launch_w64<PARO_DTYPE_F16, false, false>(p, st);
  }
  if (causal) return exact ? launch_w64<PARO_DTYPE_BF16, true, true>(p, st) : launch_w64<PARO_DTYPE_BF16, true, false>(p, st);
  return exact ? launch_w64<PARO_DTYPE_BF16, false, true>(p, st) : launch_w64<PARO_DTYPE_BF16, false, false>(p, st);
}

}  // namespace paro
