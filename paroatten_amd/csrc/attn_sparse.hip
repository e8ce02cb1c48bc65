// Block-sparse quantised attention for gfx950 (MI355X).
//
//   S^T = K8 . Q8^T      v_mfma_i32_32x32x32_i8       exact int32
//   P~  = 2^(S*c - m + 5) online base-2 softmax in fp32, rounded to FP8 e4m3 (OCP)
//   O^T += V8^T . P~^T   v_mfma_f32_32x32x64_f8f6f4   fp32 accumulation
//   d   += sum_j P~      v_mfma_f32_16x16x128_f8f6f4  against a selector operand
//
// One workgroup = one 64-row q-block of one (batch, head); its two 64-lane waves own 32 q-rows
// each (= one q-scale group).  The transposed products make the accumulator fragment of S^T (a lane
// holds 32 kv-values of ONE q-row) directly the B operand of the P.V MFMA; the kv-order inside a
// block that this implies is absorbed by the tile order V8 is stored in (see v_fp8.hip), so no
// cross-lane data movement is needed between the two matrix products and the row maximum needs one
// exchange with the partner lane (lane ^ 32) only.
//
// k-blocks: the workgroup turns its row of the bool mask into a compact list in LDS and loops over
// the kept blocks only; a skipped block costs neither loads nor MFMA issue.  K8 (row-major, 16-byte
// chunks XOR-swizzled against bank conflicts) and V8 (already in fragment order) tiles come in by
// LDS-DMA through a ring of three (D = 64) or two (D = 128) stages, and the loop is software-
// pipelined: while the softmax weights of block i are computed on the VALU, the tiles of the next
// blocks are in flight; then the MFMAs of S^T(i+1) and P.V(i) are issued back to back and run on under
// the VALU phase of block i+1.  One barrier per block.
//
// Workgroups are renumbered so that each of the 8 XCDs walks a contiguous range of (batch, head,
// q-block): the K8/V8 of the one or two heads an XCD is working on stay resident in its own L2.
//
// Semantics follow qk_int_sv_f16_attn_kernel of the reference
// (csrc/qattn/qk_int_sv_f16_cuda_sm80.cu:44-726) as instantiated by its host (:1022-1048):
// scale indexing :100-133, mask indexing :222/:268, out-of-range columns attn_utils.cuh:355-381,
// softmax recurrence attn_utils.cuh:383-488, normalisation :786-840, lse = log2(d) + m (:711-723).
#include "attn_common.hpp"
#include <atomic>
#include <mutex>
#include <stdlib.h>

namespace paro {

template <int D> struct AttnLds {
  // LDS ring stages per operand.  D = 64: three, tiles are requested two iterations ahead.  D = 128:
  // two, requested one iteration ahead (an iteration is twice as long there), which keeps a workgroup
  // at 32 KB + lists so that four of them, the register-limited number, fit a CU's 160 KB.
  static constexpr int NST = D == 128 ? 2 : 3;
  static constexpr int KTILE = 64 * D;   // bytes of one K8 tile: 64 rows of D bytes, 16-byte chunks XOR-swizzled
  static constexpr int VTILE = 64 * D;   // bytes of one V8 tile (fragment order, as in HBM)
  static constexpr int V_OFF = NST * KTILE;
  static constexpr int EPI_OFF = NST * (KTILE + VTILE);
  // D = 64: v_scale and v_mean of the head (2 x D floats), fetched at the start so that the epilogue does not
  // wait for them.  (At D = 128 the 1 KB would cost Wan 720p its fourth workgroup per CU.)
  static constexpr int EPI_BYTES = D == 64 ? 2 * D * 4 : 0;
  static constexpr int LIST_OFF = EPI_OFF + EPI_BYTES;
  static constexpr int LIST_PAD = 8;     // list entries past the end that the prefetch may touch
  // chunk c of row `row` is stored at chunk position c ^ swz(row): makes the MFMA A-operand reads (32
  // rows x one 16-byte chunk per half-wave) conflict-free; measured on gfx950 for both row lengths
  static __device__ __forceinline__ int swz(int row) {
    if constexpr (D == 64) return (row >> 2) & 3;
    else return (row ^ (row >> 3)) & 7;
  }
};

// Waves per SIMD the register budget is set for: the D = 64 production variants fit 168 registers.
#define PARO_ATTN_WAVES_PER_SIMD ((D == 64 && !CAUSAL && !DUMP && !LSE) ? 3 : 2)

// One 64-row q-block `vid` (numbered over batch, head, q-block) by one workgroup of two waves.
//
// PT: the scales have the reference's per-thread granularity (qk_quant_gran 3, csrc/qattn/
// qk_int_sv_f16_cuda_sm80.cu:112-116 and :129-133): eight q scales per 32-row group, scale g for the rows
// r with r % 8 == g (the rows lane / 4 + 8 j that a thread of the reference's m16n8 accumulator tiles holds),
// and four k scales per 64-key block, scale j for the keys c with (c % 8) / 2 == j (the columns 2 (lane % 4),
// 2 (lane % 4) + 1 of every 8-wide tile).  Here a lane holds one q-row, so its q scale is its own, and of its
// 32 keys per block (offsets 4 lh + i % 4 within every group of 8) the even pair i % 4 < 2 has k scale 2 lh and
// the odd pair 2 lh + 1: two affine maps from score to exponent per block instead of one.
template <int D, int OUT_DT, bool CAUSAL, bool DUMP, bool LSE, bool EXACT, bool PT = false>
__device__ __forceinline__ void attn_qblock(const AttnParams& p, const int vid) {
  static_assert(!PT || !DUMP, "per-thread scales: no score dump");
  using Lds = AttnLds<D>;
  constexpr int CW = PT ? 4 : 1;    // k scales per key block
  constexpr int KS = D / 32;        // k-steps of the QK MFMA (32 channels each)
  constexpr int DT_TILES = D / 32;  // 32-channel tiles of O^T
  constexpr int NLD = D / 32;       // 16-byte pieces per thread per K (or V) tile
  constexpr int CPR = D / 16;       // 16-byte chunks per K row

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  float* clist = reinterpret_cast<float*>(smem + Lds::LIST_OFF);  // [nbk + LIST_PAD + 1] k_scale of kept blocks
  unsigned short* klist = reinterpret_cast<unsigned short*>(clist + (p.nbk + Lds::LIST_PAD + 1) * CW);  // their indices

  // (D = 64: opaque to the compiler.  In the paced kernel, which calls this in a loop, everything derived from
  // the lane number alone is otherwise computed once in front of that loop and kept in registers, 35 more than
  // the 168 that three waves per SIMD allow; at D = 128, with registers to spare, hoisting measured 2 % faster)
  int t = threadIdx.x;
  if constexpr (D == 64) asm volatile("" : "+v"(t));
  const int lane = t & 63, wave = t >> 6;
  const int l32 = lane & 31, lh = lane >> 5;

  const int qb = vid % p.nbq;
  const int bh = vid / p.nbq;
  const int h = bh % p.H, b = bh / p.H;
  const int hk = h / (p.H / p.Hkv);
  const int64_t bhk = (int64_t)b * p.Hkv + hk;

  // Everything the q-block needs from memory before its first tile is requested here in one go, without a
  // branch (Q, the mask row, the k scales, the epilogue constants, the permutation order as a scalar): a
  // workgroup lives for a few dozen block iterations only, and every dependent round trip to HBM in front
  // of or behind its loop costs two or three of them.  Loads behind a branch are waited for one by one, and
  // loads whose only use sits in a branch are moved into it; so both waves build the (identical) lists, and
  // entries that are not kept go to a spare slot instead of being skipped.
  const int order_h = p.orders != nullptr ? p.orders[h] : 0;
  const float* ksc_base = p.k_scale + bhk * p.nbk * CW;
  const int kmax = CAUSAL ? min(p.nbk, qb + 1) : p.nbk;
  const uint8_t* mrow = p.sparse + b * p.sparse_bs + ((int64_t)h * p.nbq + qb) * p.nbk;
  constexpr int MU = 8;   // 64 x MU blocks per pass: one pass up to 512 blocks
  uint8_t m[MU];
  float msc[MU];
  v4f msc4[PT ? MU : 1];
  auto list_load = [&](int base) {
#pragma unroll
    for (int u = 0; u < MU; u++) {
      const int j = min(base + u * 64 + lane, kmax - 1);   // past the end: the last entry again
      m[u] = mrow[j];
      if constexpr (PT) msc4[u] = *reinterpret_cast<const v4f*>(ksc_base + 4 * j);
      else msc[u] = ksc_base[j];
    }
  };
  const int trash = p.nbk + Lds::LIST_PAD;   // the spare slot
  int cnt = 0;
  auto list_take = [&](int base) {
#pragma unroll
    for (int u = 0; u < MU; u++) {
      const int j = base + u * 64 + lane;
      const bool keep = m[u] != 0 && j < kmax;
      const unsigned long long bal = __ballot(keep);
      const int pos = keep ? cnt + __popcll(bal & ((1ull << lane) - 1ull)) : trash;
      klist[pos] = (unsigned short)j;
      if constexpr (PT) *reinterpret_cast<v4f*>(clist + 4 * pos) = msc4[u];
      else clist[pos] = msc[u];
      cnt += __popcll(bal);
    }
  };
  list_load(0);

  // ---- Q fragments (B operand: column = q-row, 16 channels per lane and k-step) -----------
  const int qrow = qb * 64 + wave * 32 + l32;
  v4i qf[KS];
  {
    // rows past the end re-read the last row; their results are never stored
    const int8_t* qp = p.q8 + b * p.qs_b + h * p.qs_h + (int64_t)min(qrow, p.Nq - 1) * p.qs_n + 16 * lh;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[ks] = *reinterpret_cast<const v4i*>(qp + 32 * ks);
  }
  const int64_t qs_group = ((int64_t)b * p.H + h) * (p.nbq * 2) + qb * 2 + wave;
  const float qsc = (PT ? p.q_scale[qs_group * 8 + (l32 & 7)] : p.q_scale[qs_group]) * p.sm_scale_log2e;

  float* epi = reinterpret_cast<float*>(smem + Lds::EPI_OFF);   // [2][D]: v_scale, v_mean (D = 64)
  float epi_sc = 0.f, epi_mn = 0.f;
  if constexpr (Lds::EPI_BYTES != 0) {
    epi_sc = p.v_scale[bhk * D + lane];
    if (p.v_mean) epi_mn = p.v_mean[bhk * D + lane];
  }

  // ---- compact list of kept k-blocks (and of their k scales) ------------------------------
  list_take(0);
  for (int base = 64 * MU; base < kmax; base += 64 * MU) {
    list_load(base);
    list_take(base);
  }
  // the loop prefetches up to 4 blocks ahead without branching: pad with the last kept block (entry
  // cnt - 1 of the lists just written; LDS operations of one wave complete in order)
  if (cnt > 0 && lane < Lds::LIST_PAD) {
    klist[cnt + lane] = klist[cnt - 1];
    if constexpr (PT) *reinterpret_cast<v4f*>(clist + 4 * (cnt + lane)) = *reinterpret_cast<const v4f*>(clist + 4 * (cnt - 1));
    else clist[cnt + lane] = clist[cnt - 1];
  }
  if constexpr (Lds::EPI_BYTES != 0) {
    epi[lane] = epi_sc;
    epi[D + lane] = epi_mn;
  }

  __syncthreads();


  using OutT = F16x<OUT_DT>;
  // where this lane's q-row goes (evaluated where it is needed: nothing of it lives across the loop)
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

  // ---- tile movers: LDS-DMA buffer loads (scalar base + per-lane offset fixed for the whole loop +
  //      scalar per-block offset).  Each wave moves half of every tile, 1 KB (64 lanes x 16 bytes) per
  //      instruction; K8's chunk swizzle is applied on the global-address side. ---------------------
  const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      uniform_ptr(p.k8 + b * p.ks_b + hk * p.ks_h), 0, (int)((int64_t)(p.Nk - 1) * p.ks_n + D), 0x00020000);
  const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      uniform_ptr(p.v8 + bhk * p.nbk * (int64_t)Lds::VTILE), 0, p.nbk * Lds::VTILE, 0x00020000);
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  int k_goff[NLD], v_goff[NLD];
#pragma unroll
  for (int i = 0; i < NLD; i++) {
    const int pos = (wave_u * NLD + i) * 1024 + lane * 16;  // byte position inside the LDS tile
    const int row = pos / D, cpos = (pos % D) / 16;
    // (less the immediate offset i * 1024 that the instruction adds on both sides; row * ks_n >= i * 1024)
    k_goff[i] = row * (int)p.ks_n + ((cpos ^ Lds::swz(row)) * 16) - i * 1024;
    v_goff[i] = pos - i * 1024;
  }
  const int k_blk_stride = 64 * (int)p.ks_n;
  auto load_k = [&](int kb, int ST) {  // rows >= Nk read as 0
    uint8_t* base = smem + ST * Lds::KTILE + wave_u * NLD * 1024;
    buffer_load16_lds<0>(k_rsrc, base, k_goff[0], kb * k_blk_stride);
    buffer_load16_lds<1024>(k_rsrc, base, k_goff[1], kb * k_blk_stride);
    if constexpr (NLD == 4) {
      buffer_load16_lds<2048>(k_rsrc, base, k_goff[2], kb * k_blk_stride);
      buffer_load16_lds<3072>(k_rsrc, base, k_goff[3], kb * k_blk_stride);
    }
  };
  auto load_v = [&](int kb, int ST) {
    uint8_t* base = smem + Lds::V_OFF + ST * Lds::VTILE + wave_u * NLD * 1024;
    buffer_load16_lds<0>(v_rsrc, base, v_goff[0], kb * Lds::VTILE);
    buffer_load16_lds<1024>(v_rsrc, base, v_goff[1], kb * Lds::VTILE);
    if constexpr (NLD == 4) {
      buffer_load16_lds<2048>(v_rsrc, base, v_goff[2], kb * Lds::VTILE);
      buffer_load16_lds<3072>(v_rsrc, base, v_goff[3], kb * Lds::VTILE);
    }
  };
  constexpr int LOADS_PER_IT = 2 * NLD;  // DMA instructions one wave issues per block

  // ---- fragment movers and the two matrix products ---------------------------------------
  const int vr_base = Lds::V_OFF + lane * 16;        // V fragment (dt, mt): + (dt*2+mt)*1024
  v4i kfrag[2 * KS];
  // K fragment (ks, mt): row 32*mt + l32, chunk 2*ks + lh at its swizzled position
  int kr_off[2 * KS];
#pragma unroll
  for (int ks = 0; ks < KS; ks++)
#pragma unroll
    for (int mt = 0; mt < 2; mt++) {
      const int row = 32 * mt + l32;
      kr_off[ks * 2 + mt] = row * D + (((2 * ks + lh) ^ Lds::swz(row)) * 16);
    }
  auto read_k_frag = [&](int ST, int i) {
    kfrag[i] = *reinterpret_cast<const v4i*>(smem + ST * Lds::KTILE + kr_off[i]);
  };
  auto read_k_frags = [&](int ST) {
#pragma unroll
    for (int i = 0; i < 2 * KS; i++) read_k_frag(ST, i);
  };
  // S^T tile: 64 kv-rows (2 MFMA row tiles) x 32 q-columns.  The accumulators start at the bit
  // pattern of 1.5*2^23: the int32 result then READS as the float 12582912 + S exactly
  // (|S| <= 127*127*128 < 2^22), which saves the int->float conversions.
  v16i magic;
#pragma unroll
  for (int i = 0; i < 16; i++) magic[i] = S_MAGIC_BITS;
  // keep the constant block resident instead of rebuilding it per block (15 scalar + 8 vector moves)
  // (not in the D = 128 variants with exact exponentials, which have no 16 registers to spare)
  if constexpr (D == 64 || (!EXACT && !LSE && !DUMP)) asm volatile("" : "+v"(magic));
  v16i acc[2];
  // (a wave that issues MFMAs back to back sits blocked behind the matrix pipe for their whole duration;
  // the other waves of the SIMD run their VALU phases meanwhile, see step below)
  auto qk_one = [&](int idx) {
    const int mt = idx / KS, ks = idx % KS;  // idx = mt * KS + ks
    if (ks == 0) acc[mt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kfrag[mt], qf[0], magic, 0, 0, 0);
    else acc[mt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kfrag[ks * 2 + mt], qf[ks], acc[mt], 0, 0, 0);
  };
  auto qk_mfma = [&]() {
#pragma unroll
    for (int i = 0; i < 2 * KS; i++) qk_one(i);
  };
  auto dump_s = [&](int kb) {
    if constexpr (DUMP) {
      if (p.s_dump) {
        int32_t* sd = p.s_dump + (((int64_t)b * p.H + h) * (p.nbq * 64) + qrow) * (int64_t)(p.nbk * 64) + kb * 64;
#pragma unroll
        for (int mt = 0; mt < 2; mt++)
#pragma unroll
          for (int i = 0; i < 16; i++) sd[32 * mt + 8 * (i >> 2) + 4 * lh + (i & 3)] = acc[mt][i] - S_MAGIC_BITS;
      }
    }
  };

  // ---- state ------------------------------------------------------------------------------
  v16f o_acc[DT_TILES];
#pragma unroll
  for (int dt = 0; dt < DT_TILES; dt++)
#pragma unroll
    for (int i = 0; i < 16; i++) o_acc[dt][i] = 0.f;
  // Row sums of the ROUNDED P~ from the matrix pipe, on the cheapest shape that fits: in a
  // 16x16x128 product the B lanes 16g..16g+15 (g = lane/16) supply k-range 32g..32g+31 of columns
  // 0..15, and P~'s fragment has q-row lane%32 and kv-half lane/32 there, i.e. k-ranges 0 and 2 are
  // the two kv-halves of q-rows 0..15 and k-ranges 1 and 3 those of q-rows 16..31.  With A row 0 =
  // ones on k-ranges {0,2} and A row 1 = ones on {1,3} (A lane: row lane%16, k-range lane/16), lanes
  // 0..15 get d_acc[0] = row sum of q-row lane and d_acc[1] = that of q-row lane+16.
  v4f d_acc = {0.f, 0.f, 0.f, 0.f};
  const int sel_word = ((lane & 15) == ((lane >> 4) & 1)) ? FP8_ONES : 0;
  v8i ones = {sel_word, sel_word, sel_word, sel_word, sel_word, sel_word, sel_word, sel_word};
  asm volatile("" : "+v"(ones));  // same: resident constant operand
  float m_i = -1e30f;
  float m_thr = -1e30f, m_off = 0.f, m_off8 = 0.f;  // m + headroom and the m-dependent offsets (see step)
  float d_exact = 0.f;  // LSE only: sum of the unrounded P~ of this lane's 32 kv-columns per block

  // ---- prologue ------------------------------------------------------------------------------
  // K ring: stage j % NST holds the K tile of block j; V ring likewise.  One iteration per kept block, in
  // two phases that never mix:
  //   VALU phase   P~(i) = softmax weights of S(i) as e4m3 words (no matrix instruction in it)
  //   matrix phase S(i+1) = K(i+1).Q, then O += V(i).P~(i) and the row sums, issued back to back
  // The wave's own P.V products run on under the VALU phase of its next block (which needs S(i+1) only), and
  // the other waves of the SIMD take their turns on the matrix pipe meanwhile.  Measured against issuing
  // one product after every word of weights (the other natural schedule): the same kernel time to 0.1 %;
  // this form needs no deferred product and a single buffer of weights.
  //   D = 64  (three stages): iteration i requests K(i+3), V(i+2); what it requests is waited for at the
  //                           end of iteration i+1 (vmcnt keeps the newest LOADS_PER_IT in flight)
  //   D = 128 (two stages):   iteration i requests K(i+2), V(i+1) at its start and waits for them at its end
  int kb_c = __builtin_amdgcn_readfirstlane((int)klist[0]);
  int kb_1 = __builtin_amdgcn_readfirstlane((int)klist[1]);
  int kb_2 = __builtin_amdgcn_readfirstlane((int)klist[2]);
  int kb_3 = __builtin_amdgcn_readfirstlane((int)klist[3]);
  constexpr bool RING2 = Lds::NST == 2;
  load_k(kb_c, 0);
  load_k(kb_1, 1);
  load_v(kb_c, 0);
  if constexpr (!RING2) {
    load_k(kb_2, 2);
    load_v(kb_1, 1);
  }
  // (PT: the lane's two k scales of the block, for its even and its odd pairs of keys)
  // (everything the odd pairs need is declared for PT only in effect: without PT the names below are never read,
  // so the per-warp kernels are the instruction streams they were)
  float c_cur = qsc * clist[PT ? 2 * lh : 0];
  float cb_cur = 0.f;
  if constexpr (PT) cb_cur = qsc * clist[2 * lh + 1];
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  read_k_frags(0);
  qk_mfma();
  dump_s(kb_c);
  // stage 0 is the first one the loop refills: both waves must hold their K(0) fragments by then
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();

  // the product O^T += V8^T . P~^T, plus the row sums of the ROUNDED P~ from one more MFMA against the
  // selector operand; idx 0..DT_TILES-1 = output tiles, DT_TILES = row sums
  v4i vfrag[DT_TILES][2];
  auto pv_one = [&](const v8i& pf, int idx) {
    if (idx < DT_TILES) {
      const v8i a = {vfrag[idx][0][0], vfrag[idx][0][1], vfrag[idx][0][2], vfrag[idx][0][3],
                     vfrag[idx][1][0], vfrag[idx][1][1], vfrag[idx][1][2], vfrag[idx][1][3]};
      o_acc[idx] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, pf, o_acc[idx], 0, 0, 0, 0, 0, 0);
    } else {
      d_acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ones, pf, d_acc, 0, 0, 0, 0, 0, 0);
    }
  };
  auto read_v_frags = [&](int ST) {
#pragma unroll
    for (int dt = 0; dt < DT_TILES; dt++)
#pragma unroll
      for (int mt = 0; mt < 2; mt++)
        vfrag[dt][mt] = *reinterpret_cast<const v4i*>(smem + ST * Lds::VTILE + vr_base + (dt * 2 + mt) * 1024);
  };

  constexpr int N_PV = DT_TILES + 1;     // MFMAs of one P.V (+ row sums)
  // One block.  `acc` holds its S^T on entry and that of the next block on exit.  sk1: K stage of block
  // it+1; sv: V stage of block it; skn / svn: the stages this iteration's DMA refills.
  auto step = [&](int it, int sk1, int sv, int skn, int svn) {
    // -- memory traffic of this iteration, issued up front
    if constexpr (RING2) {
      load_k(kb_2, skn);   // K(it+2) into the stage K(it) has left
      load_v(kb_1, svn);   // V(it+1) into the stage V(it-1) has left
    } else {
      load_k(kb_3, skn);   // K(it+3) into the stage K(it) has left
      load_v(kb_2, svn);   // V(it+2) into the stage V(it-1) has left
    }
    const int kidx_v = (int)klist[it + 4];
    const float c_next = qsc * clist[(it + 1) * CW + (PT ? 2 * lh : 0)];
    float cb_next = 0.f;
    if constexpr (PT) cb_next = qsc * clist[(it + 1) * CW + 2 * lh + 1];
    // scale of this block and what follows from it and from the current maximum alone
    const float c = c_cur;
    const float cb = cb_cur;
    const float nmc = -S_MAGIC_F * c;
    const float c8 = (8.0f * FAST_FIELD_SCALE) * c;
    float bias = fmaf(-S_MAGIC_F, c, m_off);      // exact path:  t  = S*c - m + OFFSET
    float biasb = 0.f;
    if constexpr (PT) biasb = fmaf(-S_MAGIC_F, cb, m_off);
    float bias8 = fmaf(-S_MAGIC_F, c8, m_off8);   // fast path: field = (8*(t + 7) + shift + 0.5) * 256 / 32767
    const float c8b = (8.0f * FAST_FIELD_SCALE) * cb;
    float bias8b = 0.f;
    if constexpr (PT) bias8b = fmaf(-S_MAGIC_F, c8b, m_off8);

    float s[2][16];
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
      for (int i = 0; i < 16; i++) s[mt][i] = __int_as_float(acc[mt][i]);

    // columns past the end of K (last block) or above the diagonal (causal) leave the softmax
    const bool edge = (kb_c == p.nbk - 1 && (p.Nk & 63) != 0) || (CAUSAL && kb_c == qb);
    if (edge) {
      // One threshold per lane: the element of row tile mt, register i is column
      // kb*64 + 4*lh + cidx, cidx = 32*mt + 8*(i/4) + i%4, and it is dead from the first column past the end
      // of K (or above the diagonal) on.  (The block index is made opaque: from loop invariants the compiler
      // would evaluate the 32 lane masks in front of the loop and hold them in 64 scalar registers.)
      int kb_e = kb_c;
      asm volatile("" : "+s"(kb_e));
      int thr = p.Nk - kb_e * 64 - 4 * lh;
      if constexpr (CAUSAL) thr = min(thr, qrow + 1 - kb_e * 64 - 4 * lh);
#pragma unroll
      for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const int cidx = 32 * mt + 8 * (i >> 2) + (i & 3);
          if (cidx >= thr) s[mt][i] = -INFINITY;
        }
    }

    // Row maximum of the block (biased by 1.5*2^23 like the scores), as the log2-domain score m_blk
    auto block_max = [&]() {
      if constexpr (PT) {
        // the even and the odd pairs carry different scales: two maxima, scaled, then the larger one
        float ma = fmaxf(s[0][0], s[0][1]), mb = fmaxf(s[0][2], s[0][3]);
#pragma unroll
        for (int mt = 0; mt < 2; mt++)
#pragma unroll
          for (int g = mt == 0 ? 1 : 0; g < 4; g++) {
            ma = max3(ma, s[mt][4 * g], s[mt][4 * g + 1]);
            mb = max3(mb, s[mt][4 * g + 2], s[mt][4 * g + 3]);
          }
        return partner_max(fmaxf(fmaf(ma, c, nmc), fmaf(mb, cb, -S_MAGIC_F * cb)));
      }
      // four interleaved v_max3 chains (the values are integers read as floats: no NaN to canonicalise)
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
      float smax = max3(mx0, mx1, mx2);
      smax = max3(smax, mx3, mx3);
      return fmaf(partner_max(smax), c, nmc);
    };
    // Refresh of the running maximum.  Everything that depends on m only (threshold, offsets of the
    // affine maps) is state that changes here; O and the row sums hold every product up to the previous
    // block by now and are rescaled on the spot.
    auto apply_refresh = [&](float m_blk) {
      const float m_new = fmaxf(m_i, m_blk);
      const float alpha = __builtin_amdgcn_exp2f(m_i - m_new);
      m_i = m_new;
      m_thr = m_new + P_HEADROOM;
      m_off = P_EXP_OFFSET - m_new;
      m_off8 = (8.0f * (P_EXP_OFFSET + 7.0f - m_new) + FAST_EXP_SHIFT + 0.5f) * FAST_FIELD_SCALE;
      bias = fmaf(-S_MAGIC_F, c, m_off);
      if constexpr (PT) biasb = fmaf(-S_MAGIC_F, cb, m_off);
      bias8 = fmaf(-S_MAGIC_F, c8, m_off8);
      if constexpr (PT) bias8b = fmaf(-S_MAGIC_F, c8b, m_off8);
      if constexpr (LSE) d_exact *= alpha;
      d_acc[0] *= alpha;                                          // lanes 0..15: q-row lane
      d_acc[1] *= __shfl(alpha, (lane & 15) + 16, 64);            // and q-row lane+16
#pragma unroll
      for (int dt = 0; dt < DT_TILES; dt++)
#pragma unroll
        for (int i = 0; i < 16; i++) o_acc[dt][i] *= alpha;
    };

    // -- VALU phase: the softmax weights of this block as 8 words of four e4m3 values each
    v8i pf;
    constexpr bool OPTIMISTIC = !EXACT;
    if constexpr (OPTIMISTIC) {
      // Fast path: the e4m3 byte of 2^t is built directly: byte = round(8*(t + 7) + FAST_EXP_SHIFT), i.e.
      // exponent field floor(t)+7 and a mantissa that interpolates 2^frac(t) linearly between powers of
      // two (at most 6 % off, shifted to be centred).  Per word of four weights: four fmas (the affine
      // map scaled so that the byte lands in the HIGH half of a 16-bit field, result clamped to [0,1], which
      // sends masked and underflowing elements to 0 and bounds the field by 0x7FFF, the byte by 0x7F), two
      // v_cvt_pknorm_i16_f32 (each rounds two values to 16-bit fields) and one v_perm_b32 that gathers the
      // four high bytes.  Instead of fma + v_exp_f32 + half a packed FP8 conversion per weight.
      // Word r = word r%4 of row tile r/4.
      //
      // It is optimistic about the maximum: the weights are computed with the running maximum as it is.
      // A weight above 448, the largest e4m3 value (a score more than 3.8 octaves above the running
      // maximum), comes out as the byte 0x7F, which is the e4m3 NaN: the row sums, taken by the matrix pipe
      // from the same bytes BEFORE anything else uses them, turn NaN in that column, and only then is the
      // block maximum searched (17 v_max3 otherwise spent on every block), the maximum refreshed and the
      // eight words computed again (the scores are still in `acc`: the next block's S^T is issued below).
      // Nothing is spent on tracking in the common case, and O never sees a NaN.
      auto fast_words = [&]() {
        float u_cur[4], u_nxt[4];
#pragma unroll
        for (int q = 0; q < 4; q++)
          u_cur[q] = fma_clamp01(s[0][q], PT && q >= 2 ? c8b : c8, PT && q >= 2 ? bias8b : bias8);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < 8; r++) {
          // the fmas of the next word are issued between this word's conversions: every conversion
          // finds its input ready
          const int rn = r + 1, mtn = rn >> 2, in0 = 4 * (rn & 3);
          if (rn < 8) {
            u_nxt[0] = fma_clamp01(s[mtn][in0 + 0], c8, bias8);
            u_nxt[2] = fma_clamp01(s[mtn][in0 + 2], PT ? c8b : c8, PT ? bias8b : bias8);
          }
          const int lo = cvt_pknorm_i16(u_cur[0], u_cur[2]);
          __builtin_amdgcn_sched_barrier(0);
          if (rn < 8) {
            u_nxt[1] = fma_clamp01(s[mtn][in0 + 1], c8, bias8);
            u_nxt[3] = fma_clamp01(s[mtn][in0 + 3], PT ? c8b : c8, PT ? bias8b : bias8);
          }
          const int hi = cvt_pknorm_i16(u_cur[1], u_cur[3]);
          __builtin_amdgcn_sched_barrier(0);
          // bytes 1, 3 of lo (weights 0, 2) and of hi (weights 1, 3), in weight order
          pf[r] = (int)__builtin_amdgcn_perm((unsigned)hi, (unsigned)lo, 0x07030501u);
#pragma unroll
          for (int q = 0; q < 4; q++) u_cur[q] = u_nxt[q];
          __builtin_amdgcn_sched_barrier(0);
        }
      };
      fast_words();
      v4f d_new = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ones, pf, d_acc, 0, 0, 0, 0, 0, 0);
      // the fragment reads of the matrix phase are issued here: they cover the latency of the product above
      __builtin_amdgcn_sched_barrier(0);
      read_k_frags(sk1);
      if constexpr (D == 64) read_v_frags(sv);
      __builtin_amdgcn_sched_barrier(0);
      // (the first block has no maximum yet.  Lane j < 16 holds the sums of q-rows j and j + 16 in d_new[0]
      // and d_new[1]; a NaN byte of either row makes its own sum NaN whatever the hardware makes of 0 x NaN)
      if (it == 0 || __ballot(__builtin_isunordered(d_new[0], d_new[1])) != 0ull) {
        apply_refresh(block_max());
        fast_words();
        d_new = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ones, pf, d_acc, 0, 0, 0, 0, 0, 0);
      }
      d_acc = d_new;
    } else {
      // Exact path: lazy refresh decided up front from the block maximum (P~ <= 2^(OFFSET + HEADROOM)),
      // then P~ = e4m3_rne(2^(S*c - m + OFFSET)): hardware exponential and the packed FP8 conversion
      const float m_blk = block_max();
      if (__ballot(m_blk > m_thr) != 0ull) apply_refresh(m_blk);
      float rs = 0.f;
#pragma unroll
      for (int r = 0; r < 8; r++) {
        const int mt = r >> 2, i0 = 4 * (r & 3);
        const float p0 = __builtin_amdgcn_exp2f(fmaf(s[mt][i0 + 0], c, bias));
        const float p1 = __builtin_amdgcn_exp2f(fmaf(s[mt][i0 + 1], c, bias));
        const float p2 = __builtin_amdgcn_exp2f(fmaf(s[mt][i0 + 2], PT ? cb : c, PT ? biasb : bias));
        const float p3 = __builtin_amdgcn_exp2f(fmaf(s[mt][i0 + 3], PT ? cb : c, PT ? biasb : bias));
        if constexpr (LSE) rs += (p0 + p1) + (p2 + p3);
        int w;
        cvt_pk_fp8<false>(w, p0, p1);
        cvt_pk_fp8<true>(w, p2, p3);
        pf[r] = w;
      }
      if constexpr (LSE) d_exact += rs;
    }
    __builtin_amdgcn_sched_barrier(0);

    // -- matrix phase: S^T of the next block first (the next VALU phase waits for it alone), then this
    //    block's P.V and row sums, which run on under that VALU phase
    // (fetching the K fragments at the head of the iteration instead, so that they arrive under the VALU
    // phase, measured 2 % slower at D = 128, 7 % with the dense mask)
    if constexpr (EXACT) {   // (the fast path has issued these reads already)
      read_k_frags(sk1);
      if constexpr (D == 64) read_v_frags(sv);
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (D == 128) {
      // the V fragments are fetched while the S^T products issue: after the two products of k-step ks the K
      // fragments of that step are dead, and two V pieces take their place (+1-2 % against fetching all
      // eight pieces after the last product)
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        qk_one(0 * KS + ks);
        qk_one(1 * KS + ks);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int mt = 0; mt < 2; mt++)
          vfrag[ks][mt] = *reinterpret_cast<const v4i*>(smem + sv * Lds::VTILE + vr_base + (ks * 2 + mt) * 1024);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
      qk_mfma();
      __builtin_amdgcn_sched_barrier(0);
    }
    // (fast path: the row sums have been taken above)
#pragma unroll
    for (int i = 0; i < (EXACT ? N_PV : DT_TILES); i++) pv_one(pf, i);
    __builtin_amdgcn_sched_barrier(0);
    if (it + 1 < cnt) dump_s(kb_1);

    // -- what the ring needs next has to have landed before the barrier publishes it
    const int kb_4 = __builtin_amdgcn_readfirstlane(kidx_v);
    // (a bare s_barrier: __syncthreads() would add a fence that waits for ALL outstanding loads)
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(RING2 ? 0 : LOADS_PER_IT) : "memory");
    __builtin_amdgcn_s_barrier();
    kb_c = kb_1; kb_1 = kb_2; kb_2 = kb_3; kb_3 = kb_4;
    c_cur = c_next;
    if constexpr (PT) cb_cur = cb_next;
  };

  if constexpr (RING2) {
    // stage of block j is j % 2: iteration `it` reads K(it+1) from the other stage and V(it) from its own,
    // refills its own K stage with K(it+2) and the other V stage with V(it+1)
    for (int it = 0; it < cnt; it += 2) {
      step(it, 1, 0, 0, 1);
      if (it + 1 >= cnt) break;
      step(it + 1, 0, 1, 1, 0);
    }
  } else {
    // stage of block j is j % 3: with i = it % 3, iteration `it` reads K stage i+1 and V stage i, refills
    // K stage i with K(it+3) and V stage i+2 with V(it+2)
    // (unrolled by three: the stage numbers are constants and every LDS address an immediate offset)
    for (int it = 0; it < cnt; it += 3) {
      step(it, 1, 0, 0, 2);
      if (it + 1 >= cnt) break;
      step(it + 1, 2, 1, 1, 0);
      if (it + 2 >= cnt) break;
      step(it + 2, 0, 2, 2, 1);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // DMA of the padded tail blocks: nobody reads it

  // ---- epilogue: O = O~/d * v_scale + v_mean ------------------------------------------------
  const float d_lo = __shfl(d_acc[0], l32 & 15, 64), d_hi = __shfl(d_acc[1], l32 & 15, 64);
  const float d_tot = l32 < 16 ? d_lo : d_hi;
  const float inv = 1.0f / d_tot;
  if (qrow < p.Nq) {
    unsigned short* outp = out_row_ptr();
    const float* vsc = p.v_scale + bhk * D;
    const float* vmn = p.v_mean ? p.v_mean + bhk * D : nullptr;
#pragma unroll
    for (int dt = 0; dt < DT_TILES; dt++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int ch = 32 * dt + 8 * g + 4 * lh;
        v4f sc, mn = {0.f, 0.f, 0.f, 0.f};
        if constexpr (Lds::EPI_BYTES != 0) {
          sc = *reinterpret_cast<const v4f*>(epi + ch);
          mn = *reinterpret_cast<const v4f*>(epi + D + ch);
        } else {
          sc = *reinterpret_cast<const v4f*>(vsc + ch);
          if (vmn) mn = *reinterpret_cast<const v4f*>(vmn + ch);
        }
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

template <int D, int OUT_DT, bool CAUSAL, bool DUMP, bool LSE, bool EXACT, bool PT = false>
__global__ void __launch_bounds__(128, PARO_ATTN_WAVES_PER_SIMD) attn_sparse_kernel(const AttnParams p) {
  // XCD-aware renumbering: hardware deals workgroup ids round-robin to the 8 XCDs
  const int per = gridDim.x >> 3;
  const int vid = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
  if (vid >= p.total) return;
  attn_qblock<D, OUT_DT, CAUSAL, DUMP, LSE, EXACT, PT>(p, vid);
}

// The same work with a resident set of workgroups per XCD that take the XCD's q-blocks generation by
// generation: all of them start a q-block together and so walk the key blocks of the head roughly in step.
// For heads whose K8 + V8 exceed the XCD's L2 (Wan 720p: 19 MB against 4 MB): in the ordinary launch
// the workgroups of an XCD sit at unrelated positions of the key sequence, the L2 sees a uniform stream
// over the whole head and hits at (L2 size / head size); started together, neighbours in time are
// neighbours in the key sequence.  The meeting point between generations only paces: a workgroup that
// has waited `spin_limit` rounds goes on regardless, so the kernel finishes whatever the residency or
// the state of the counters (they are zeroed by a small launch in front of this one).
//
// A workgroup goes on when all but `slack` of the XCD's workgroups have arrived: the last arrivals of a
// generation do not hold the others up, and since those never wait themselves they do not fall further behind.
// What matters for the L2 is that the workgroups stay within the part of the head that it holds, not that they
// start in the same microsecond; and a generation that starts all at once also runs all its prologues and
// epilogues at once, with nothing else on the compute unit to cover them.  (Measured on a mask whose rows hold
// 154 +- 10 and 236 +- 14 kept blocks: waiting for all, 38.3 % / 38.9 % of the matrix peak at Wan 480p / 720p;
// for all but an eighth 39.6 % / 39.6 %; for all but a quarter 40.0 % / 39.2 %; for all but a half 39.6 % /
// 37.2 %, the L2 fills growing from 1.6 to 8.7 GB and from 29 to 75 GB per launch.  Building the generations from
// q-blocks of equal length, sorted by a pre-pass over the mask, changed nothing: a workgroup that waits leaves
// the matrix pipe to its neighbours on the compute unit, so the waiting itself costs little.)
constexpr int PACE_PAD = 32;   // counters 128 bytes apart: one per XCD
template <int D, int OUT_DT, bool CAUSAL, bool DUMP, bool LSE, bool EXACT, bool PT = false>
__global__ void __launch_bounds__(128, PARO_ATTN_WAVES_PER_SIMD)
    attn_sparse_paced_kernel(const AttnParams p, unsigned* __restrict__ counters, const int per, const int spin_limit,
                             const int slack) {
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, G = gridDim.x >> 3;
  const int first = xcd * per, last = min(first + per, p.total);
  unsigned arrivals = 0;
  bool waiting = true;   // a workgroup that has once waited in vain goes on without waiting for the rest of the launch
  for (int base = first; base < last; base += G) {
    const int vid = base + slot;
    if (vid < last) attn_qblock<D, OUT_DT, CAUSAL, DUMP, LSE, EXACT, PT>(p, vid);
    if (base + G >= last) break;
    // every workgroup of the XCD arrives once per generation, with or without a q-block of its own
    __syncthreads();   // also: both waves are done with this q-block's lists in LDS
    if (threadIdx.x == 0) {
      arrivals += (unsigned)G;
      unsigned* c = counters + xcd * PACE_PAD;
      __hip_atomic_fetch_add(c, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (waiting) {
        int spin = 0;
        for (; spin < spin_limit; spin++) {
          if (__hip_atomic_load(c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + (unsigned)slack >= arrivals) break;
          __builtin_amdgcn_s_sleep(32);
        }
        // its generation is not co-resident (another kernel holds compute units, or the counters are not this
        // launch's alone): waiting again at every generation would cost the spin limit each time
        if (spin >= spin_limit && spin_limit > 0) waiting = false;
      }
    }
    __syncthreads();
  }
}

__global__ void attn_pace_reset_kernel(unsigned* counters) { counters[threadIdx.x] = 0u; }

// Counters of the paced kernel: library-owned (looked up once per device), PACE_SETS sets of one counter per XCD.
// Consecutive paced launches of the process take the sets in turn, so that launches which overlap on one GPU
// (two streams, two threads) do not zero or count on each other's counters unless more than PACE_SETS of them are
// in flight at once; even then only the pacing suffers (a workgroup stops waiting after its first timeout).
constexpr int PACE_SETS = 8;
static __device__ __align__(256) unsigned g_pace_counters[PACE_SETS * 8 * PACE_PAD];
static std::atomic<unsigned> g_pace_launches{0};
constexpr int PACE_MAX_DEVICES = 64;
struct PaceDevice { unsigned* counters; int cus; };
static PaceDevice g_pace_dev[PACE_MAX_DEVICES];
static std::mutex g_pace_mu;

static int pace_device(PaceDevice* out) {
  int dev = -1;
  PARO_HIP(hipGetDevice(&dev));
  PARO_CHECK(dev >= 0 && dev < PACE_MAX_DEVICES, PARO_ERR_RUNTIME, "device ordinal %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_pace_mu);
  if (g_pace_dev[dev].counters == nullptr) {
    void* ptr = nullptr;
    PARO_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_pace_counters)));
    int cus = 0;
    PARO_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    g_pace_dev[dev].cus = cus;
    g_pace_dev[dev].counters = static_cast<unsigned*>(ptr);
  }
  *out = g_pace_dev[dev];
  return PARO_OK;
}

// The caller's flags decide (PARO_ATTN_PACED / PARO_ATTN_UNPACED); without either, the environment
// variable PARO_ATTN_PACING (0: never, 1: always) does, and without that the launch is paced when one
// head's K8 + V8 exceed the 4 MB L2 of an XCD.  PARO_ATTN_PACE_SPINS: rounds (about 1 us each) a workgroup
// waits for its generation at most (default: half the number of key blocks, between 64 and 4096).
// PARO_ATTN_PACE_SLACK: how many of an XCD's resident workgroups a generation does not wait for (default: half
// the share of the head's K8 + V8 that the L2 holds, at most a quarter of them).
static bool want_pacing(const AttnParams& p, int D) {
  if (p.pacing != 0) return p.pacing > 0;
  if (const char* e = getenv("PARO_ATTN_PACING")) return e[0] == '1';
  return (int64_t)p.nbk * 64 * D * 2 > (int64_t)4 << 20;
}

// bytes of the kept-block list in LDS: per key block a 16-bit index and its k scale (four with per-thread scales)
static size_t attn_list_bytes(int nbk, int list_pad, bool per_thread) {
  return (((size_t)(nbk + list_pad + 1) * (per_thread ? 18 : 6) + 15) & ~(size_t)15);
}

template <int D, int OUT_DT, bool CAUSAL, bool DUMP, bool LSE, bool EXACT, bool PT = false>
static int launch_attn(const AttnParams& p, hipStream_t st) {
  const size_t smem = AttnLds<D>::LIST_OFF + attn_list_bytes(p.nbk, AttnLds<D>::LIST_PAD, PT);
  // (per-thread scales make the list three times as long: where that costs a compute unit its fourth workgroup,
  // Wan 720p, the paced form with half the waves measured slower than the plain launch, 21.8 against 17.3 ms)
  if (!DUMP && want_pacing(p, D) && (!PT || smem <= 40 * 1024)) {
    auto kern = attn_sparse_paced_kernel<D, OUT_DT, CAUSAL, DUMP, LSE, EXACT, PT>;
    if (smem > 48 * 1024)
      PARO_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    PaceDevice pd;
    if (int rc = pace_device(&pd)) return rc;
    int per_cu = 0;
    PARO_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, 128, smem));
    const int G = per_cu * (pd.cus / 8);        // workgroups resident on one XCD
    const int per = (p.total + 7) / 8;          // q-blocks per XCD, a contiguous range of (batch, head, q-block)
    if (G > 0 && per > G) {                     // more than one generation: otherwise the plain launch is the same
      // rounds of about 1 us: a q-block of a dense mask takes about 1.3 us per key block, and there is no point in
      // waiting longer for a generation than half of that
      int spins = max(64, min(4096, p.nbk / 2));
      if (const char* e = getenv("PARO_ATTN_PACE_SPINS")) spins = atoi(e);
      // stragglers within half of the L2's share of the head still find their tiles: that many need not be waited
      // for (measured optimum on two boxes: about 32 of 128 at Wan 480p, 8.4 MB per head, and 8 to 16 at 720p,
      // 19.4 MB; beyond that the L2 fills grow quickly, 1.6 -> 8.7 GB per launch at 480p from 16 to 64)
      const int64_t head_bytes = (int64_t)p.nbk * 64 * D * 2;
      int slack = (int)min((int64_t)G / 4, (int64_t)G * ((int64_t)2 << 20) / head_bytes);
      if (const char* e = getenv("PARO_ATTN_PACE_SLACK")) slack = max(0, min(G - 1, atoi(e)));
      unsigned* counters = pd.counters + (g_pace_launches.fetch_add(1u) % PACE_SETS) * (8 * PACE_PAD);
      hipLaunchKernelGGL(attn_pace_reset_kernel, dim3(1), dim3(8 * PACE_PAD), 0, st, counters);
      hipLaunchKernelGGL(kern, dim3(8 * G), dim3(128), smem, st, p, counters, per, spins, slack);
      PARO_HIP(hipGetLastError());
      return PARO_OK;
    }
  }
  const int grid = ((p.total + 7) / 8) * 8;
  auto kern = attn_sparse_kernel<D, OUT_DT, CAUSAL, DUMP, LSE, EXACT, PT>;
  if (smem > 48 * 1024)
    PARO_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
  hipLaunchKernelGGL(kern, dim3(grid), dim3(128), smem, st, p);
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}

// per-thread scales (qk_quant_gran 3): the two-wave kernel
template <int D, int OUT_DT>
static int dispatch_attn_per_thread(const AttnParams& p, int is_causal, bool exact, hipStream_t st) {
  if (p.lse != nullptr)
    return is_causal ? launch_attn<D, OUT_DT, true, false, true, true, true>(p, st)
                     : launch_attn<D, OUT_DT, false, false, true, true, true>(p, st);
  if (exact)
    return is_causal ? launch_attn<D, OUT_DT, true, false, false, true, true>(p, st)
                     : launch_attn<D, OUT_DT, false, false, false, true, true>(p, st);
  return is_causal ? launch_attn<D, OUT_DT, true, false, false, false, true>(p, st)
                   : launch_attn<D, OUT_DT, false, false, false, false, true>(p, st);
}

template <int D, int OUT_DT>
static int dispatch_attn(const AttnParams& p, int is_causal, bool dump, bool exact, hipStream_t st) {
  // the log-sum-exp needs true exponentials; the debug dump rides on the same instantiation
  if (p.lse != nullptr || dump) {
    if (dump) return is_causal ? launch_attn<D, OUT_DT, true, true, true, true>(p, st)
                               : launch_attn<D, OUT_DT, false, true, true, true>(p, st);
    return is_causal ? launch_attn<D, OUT_DT, true, false, true, true>(p, st)
                     : launch_attn<D, OUT_DT, false, false, true, true>(p, st);
  }
  if (exact)
    return is_causal ? launch_attn<D, OUT_DT, true, false, false, true>(p, st)
                     : launch_attn<D, OUT_DT, false, false, false, true>(p, st);
  return is_causal ? launch_attn<D, OUT_DT, true, false, false, false>(p, st)
                   : launch_attn<D, OUT_DT, false, false, false, false>(p, st);
}

}  // namespace paro

namespace paro {
static int attn_sparse_impl(const int8_t* q8, const int8_t* k8, const uint8_t* v8, const float* q_scale,
                            const float* k_scale, const float* v_scale, const float* v_mean,
                            const uint8_t* sparse, int64_t sparse_batch_stride, void* out, int out_dtype,
                            float* lse, int32_t* s_dump, int B, int H, int Hkv, int Nq, int Nk, int D,
                            int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_n, int64_t k_stride_b,
                            int64_t k_stride_h, int64_t k_stride_n, int64_t o_stride_b, int64_t o_stride_h,
                            int64_t o_stride_n, float sm_scale, int is_causal, int flags, const int32_t* orders,
                            int n_text, int F, int Hh, int W, void* stream) {
  PARO_CHECK((flags & ~(PARO_ATTN_EXACT_EXP | PARO_ATTN_PACED | PARO_ATTN_UNPACED | PARO_ATTN_TWO_WAVES |
                        PARO_ATTN_PV_F16 | PARO_ATTN_QK_PER_THREAD)) == 0 &&
                 (flags & (PARO_ATTN_PACED | PARO_ATTN_UNPACED)) != (PARO_ATTN_PACED | PARO_ATTN_UNPACED),
             PARO_ERR_INVALID_VALUE, "Unsupported attention flags: %d", flags);
  const bool pv16 = (flags & PARO_ATTN_PV_F16) != 0;
  const bool per_thread = (flags & PARO_ATTN_QK_PER_THREAD) != 0;
  PARO_CHECK(!per_thread || (!pv16 && s_dump == nullptr), PARO_ERR_UNSUPPORTED,
             "per-thread scales (PARO_ATTN_QK_PER_THREAD) go with neither PARO_ATTN_PV_F16 nor the score dump");
  PARO_CHECK(!per_thread || ((uintptr_t)k_scale % 16) == 0, PARO_ERR_RUNTIME,
             "paro_attn_sparse_fwd: per-thread key scales must be 16-byte aligned");
  PARO_CHECK(q8 && k8 && v8 && q_scale && k_scale && (v_scale || pv16) && sparse && out, PARO_ERR_RUNTIME,
             "paro_attn_sparse_fwd: null tensor pointer");
  PARO_CHECK(!pv16 || s_dump == nullptr, PARO_ERR_UNSUPPORTED, "the score dump is not available with PARO_ATTN_PV_F16");
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
  // one (batch, kv-head) slice of K8 and of V8 is addressed through a buffer descriptor with 32-bit offsets
  PARO_CHECK(k_stride_n >= D && (int64_t)(Nk - 1) * k_stride_n + D < (int64_t)1 << 31 &&
                 (int64_t)nbk * 64 * D < (int64_t)1 << 31,
             PARO_ERR_RUNTIME, "paro_attn_sparse_fwd: one head of key/value spans 2 GiB or more (kv_len %d, stride %lld)",
             Nk, (long long)k_stride_n);
  // ring stages + the list of kept blocks (6 bytes each, 18 with per-thread scales) have to fit the 160 KB of LDS of one CU
  if (!pv16) {
    const int64_t ring = D == 128 ? 2 * 2 * 64 * 128 : 3 * 2 * 64 * 64;
    PARO_CHECK(ring + (per_thread ? ((int64_t)nbk + 9) * 18 + 1024 : ((int64_t)nbk + 8) * 6 + 64) <= 160 * 1024, PARO_ERR_RUNTIME,
               "kv_len %d: the list of %d key blocks does not fit the local data share", Nk, nbk);
  }
  AttnParams p;
  p.q8 = q8; p.k8 = k8; p.v8 = v8; p.q_scale = q_scale; p.k_scale = k_scale; p.v_scale = v_scale; p.v_mean = v_mean;
  p.sparse = sparse; p.out = out; p.lse = lse; p.s_dump = s_dump; p.sparse_bs = sparse_batch_stride;
  p.qs_b = q_stride_b; p.qs_h = q_stride_h; p.qs_n = q_stride_n;
  p.ks_b = k_stride_b; p.ks_h = k_stride_h; p.ks_n = k_stride_n;
  p.os_b = o_stride_b; p.os_h = o_stride_h; p.os_n = o_stride_n;
  p.B = B; p.H = H; p.Hkv = Hkv; p.Nq = Nq; p.Nk = Nk; p.nbq = nbq; p.nbk = nbk;
  p.total = B * H * nbq;
  p.sm_scale_log2e = sm_scale * 1.4426950408889634f;
  p.orders = orders; p.n_text = n_text; p.F = F; p.Hh = Hh; p.W = W;
  p.pacing = (flags & PARO_ATTN_PACED) ? 1 : ((flags & PARO_ATTN_UNPACED) ? -1 : 0);
  hipStream_t st = (hipStream_t)stream;
  const bool dump = s_dump != nullptr;
  const bool exact = (flags & PARO_ATTN_EXACT_EXP) != 0;
  // float16 P.V product: a kernel of its own (true exponentials, plain launch)
  if (pv16) return launch_attn_pv16(p, D, out_dtype, is_causal != 0, st);
  if (per_thread) {
    if (D == 64)
      return out_dtype == PARO_DTYPE_F16 ? dispatch_attn_per_thread<64, PARO_DTYPE_F16>(p, is_causal, exact, st)
                                         : dispatch_attn_per_thread<64, PARO_DTYPE_BF16>(p, is_causal, exact, st);
    return out_dtype == PARO_DTYPE_F16 ? dispatch_attn_per_thread<128, PARO_DTYPE_F16>(p, is_causal, exact, st)
                                       : dispatch_attn_per_thread<128, PARO_DTYPE_BF16>(p, is_causal, exact, st);
  }
  // D = 64 without lse or score dump: one wave per q-block (attn_sparse_w64.hip), unless the caller asks for the
  // two-wave kernel or the launch is to be paced (only the two-wave kernel has the paced form)
  if (D == 64 && lse == nullptr && !dump && (flags & PARO_ATTN_TWO_WAVES) == 0 && !want_pacing(p, D))
    return launch_attn_w64(p, out_dtype, is_causal != 0, exact, st);
  if (D == 64) {
    if (out_dtype == PARO_DTYPE_F16) return dispatch_attn<64, PARO_DTYPE_F16>(p, is_causal, dump, exact, st);
    return dispatch_attn<64, PARO_DTYPE_BF16>(p, is_causal, dump, exact, st);
  }
  if (out_dtype == PARO_DTYPE_F16) return dispatch_attn<128, PARO_DTYPE_F16>(p, is_causal, dump, exact, st);
  return dispatch_attn<128, PARO_DTYPE_BF16>(p, is_causal, dump, exact, st);
}
}  // namespace paro

extern "C" int paro_attn_sparse_fwd(const int8_t* q8, const int8_t* k8, const uint8_t* v8, const float* q_scale,
                                    const float* k_scale, const float* v_scale, const float* v_mean,
                                    const uint8_t* sparse, int64_t sparse_batch_stride, void* out, int out_dtype,
                                    float* lse, int32_t* s_dump, int B, int H, int Hkv, int Nq, int Nk, int D,
                                    int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_n, int64_t k_stride_b,
                                    int64_t k_stride_h, int64_t k_stride_n, int64_t o_stride_b, int64_t o_stride_h,
                                    int64_t o_stride_n, float sm_scale, int is_causal, int flags, void* stream) {
  return paro::attn_sparse_impl(q8, k8, v8, q_scale, k_scale, v_scale, v_mean, sparse, sparse_batch_stride, out,
                                out_dtype, lse, s_dump, B, H, Hkv, Nq, Nk, D, q_stride_b, q_stride_h, q_stride_n,
                                k_stride_b, k_stride_h, k_stride_n, o_stride_b, o_stride_h, o_stride_n, sm_scale,
                                is_causal, flags, nullptr, 0, 0, 0, 0, stream);
}

extern "C" int paro_attn_sparse_unpermute_fwd(const int8_t* q8, const int8_t* k8, const uint8_t* v8,
                                              const float* q_scale, const float* k_scale, const float* v_scale,
                                              const float* v_mean, const uint8_t* sparse,
                                              int64_t sparse_batch_stride, void* out, int out_dtype, float* lse,
                                              int B, int H, int Hkv, int Nq, int Nk, int D, int64_t q_stride_b,
                                              int64_t q_stride_h, int64_t q_stride_n, int64_t k_stride_b,
                                              int64_t k_stride_h, int64_t k_stride_n, int64_t o_stride_b,
                                              int64_t o_stride_h, int64_t o_stride_n, float sm_scale, int is_causal,
                                              int flags, const int32_t* orders, int n_text, int F, int Hh, int W,
                                              void* stream) {
  using namespace paro;
  PARO_CHECK(orders, PARO_ERR_RUNTIME, "paro_attn_sparse_unpermute_fwd: null orders");
  PARO_CHECK(n_text >= 0 && F > 0 && Hh > 0 && W > 0 && (int64_t)n_text + (int64_t)F * Hh * W == Nq, PARO_ERR_RUNTIME,
             "paro_attn_sparse_unpermute_fwd: n_text + F*H*W = %d + %d*%d*%d does not equal the token count %d",
             n_text, F, Hh, W, Nq);
  return attn_sparse_impl(q8, k8, v8, q_scale, k_scale, v_scale, v_mean, sparse, sparse_batch_stride, out, out_dtype,
                          lse, nullptr, B, H, Hkv, Nq, Nk, D, q_stride_b, q_stride_h, q_stride_n, k_stride_b,
                          k_stride_h, k_stride_n, o_stride_b, o_stride_h, o_stride_n, sm_scale, is_causal, flags,
                          orders, n_text, F, Hh, W, stream);
}

extern "C" int64_t paro_attn_workspace_bytes(int B, int Hkv, int Nk, int D) {
  auto al = [](int64_t x) { return (x + 255) & ~(int64_t)255; };
  return al(paro_v_fp8_bytes(B, Hkv, Nk, D)) + 2 * al((int64_t)B * Hkv * D * 4) +
         al(paro_v_fp8_partial_floats(B, Hkv, Nk, D) * 4);
}

extern "C" int64_t paro_attn_workspace_bytes_for(int B, int Hkv, int Nk, int D, int flags) {
  if (flags & PARO_ATTN_PV_F16) return (paro_v_f16_bytes(B, Hkv, Nk, D) + 255) & ~(int64_t)255;
  return paro_attn_workspace_bytes(B, Hkv, Nk, D);
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
                                        int smooth_v, int flags, void* stream) {
  using namespace paro;
  PARO_CHECK(tensor_layout == 0 || tensor_layout == 1, PARO_ERR_INVALID_VALUE, "tensor_layout must be 0 or 1");
  PARO_CHECK(qk_quant_gran == 2 || qk_quant_gran == 3, PARO_ERR_INVALID_VALUE, "Unsupported quantization granularity: %d",
             qk_quant_gran);
  if (qk_quant_gran == 3) flags |= PARO_ATTN_QK_PER_THREAD;
  PARO_CHECK(workspace && ((uintptr_t)workspace % 256) == 0, PARO_ERR_RUNTIME,
             "paro_qk_int8_sv_f16_attn: workspace must be a 256-byte aligned device buffer");
  PARO_CHECK(B > 0 && Hkv > 0 && Nk > 0 && (D == 64 || D == 128), PARO_ERR_INVALID_VALUE,
             "Unsupported shape or head dim: B=%d Hkv=%d Nk=%d D=%d", B, Hkv, Nk, D);
  PARO_CHECK(workspace_bytes >= paro_attn_workspace_bytes_for(B, Hkv, Nk, D, flags), PARO_ERR_RUNTIME,
             "paro_qk_int8_sv_f16_attn: workspace of %lld bytes is smaller than the %lld needed",
             (long long)workspace_bytes, (long long)paro_attn_workspace_bytes_for(B, Hkv, Nk, D, flags));
  if (flags & PARO_ATTN_PV_F16) {
    // float16 P.V product: V goes into float16 tiles as it is (no scale, no mean; smooth_v has nothing to act on)
    int rc = paro_v_f16_pack(v, v_dtype, workspace, B, Hkv, Nk, D, v_stride_b, v_stride_h, v_stride_n, stream);
    if (rc) return rc;
    return paro_attn_sparse_fwd(q8, k8, (const uint8_t*)workspace, q_scale, k_scale, nullptr, nullptr, sparse,
                                sparse_batch_stride, out, out_dtype, lse, nullptr, B, H, Hkv, Nq, Nk, D, q_stride_b,
                                q_stride_h, q_stride_n, k_stride_b, k_stride_h, k_stride_n, o_stride_b, o_stride_h,
                                o_stride_n, sm_scale, is_causal, flags, stream);
  }
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
                              o_stride_n, sm_scale, is_causal, flags, stream);
}
