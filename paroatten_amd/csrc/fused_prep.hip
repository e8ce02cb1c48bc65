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
#include "stats_device.hpp"
#include <stdlib.h>
#include <mutex>

namespace paro {

// Library-owned work buffer of paro_rope_k_mean_static (the per-chunk partial sums of the K mean), for
// callers that can neither allocate nor bring a workspace.  One copy per GPU, at its own address, held
// from the moment the code object is loaded on that GPU until the process ends.  In host code the
// array's name is only a handle for hipGetSymbolAddress; the address kernels get is looked up once per
// device (with that device current) and kept in g_kmean_scratch.
constexpr int64_t KMEAN_SCRATCH_FLOATS = PARO_ROPE_K_MEAN_STATIC_MAX_FLOATS;   // 8 MiB
static __device__ __align__(256) float scratch[KMEAN_SCRATCH_FLOATS];
constexpr int MAX_DEVICES = 64;
static float* g_kmean_scratch[MAX_DEVICES];
static std::mutex g_kmean_scratch_mu;

static int kmean_scratch_of_current_device(float** out) {
  int dev = -1;
  PARO_HIP(hipGetDevice(&dev));
  PARO_CHECK(dev >= 0 && dev < MAX_DEVICES, PARO_ERR_RUNTIME, "paro_rope_k_mean_static: device ordinal %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_kmean_scratch_mu);
  if (g_kmean_scratch[dev] == nullptr) {
    void* ptr = nullptr;
    PARO_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    PARO_CHECK(ptr != nullptr, PARO_ERR_HIP, "paro_rope_k_mean_static: no device address for the scratch array");
    g_kmean_scratch[dev] = static_cast<float*>(ptr);
  }
  *out = g_kmean_scratch[dev];
  return PARO_OK;
}

// LDS of the preparation kernel.  The gathered token rows never pass through registers on their way
// in: LDS-DMA buffer loads drop them into a ring of four 64-token tile slots, Q, K, V of one (batch,
// head) pair after the other, and the loads of the NEXT pair are issued while this one is rotated,
// reduced and quantised - three tiles are in flight per workgroup at any time.
template <int D> struct PrepLds {
  static constexpr int TILE = 64 * D * 2;          // one tile: 64 rows of D 16-bit values
  static constexpr int RING = 4;
  static constexpr int KM_OFF = RING * TILE;       // [2][256 B]  K mean row of this / the next pair
  static constexpr int ST_OFF = KM_OFF + 2 * 256;  // [2][1 KB]   V reciprocal scale and mean rows
  static constexpr int LIST_OFF = ST_OFF + 2 * 1024;
  static constexpr int MAX_PAIRS = 2048;           // (batch, head) pairs one workgroup walks over
  static constexpr int BYTES = LIST_OFF + MAX_PAIRS * 2;
  // 16-byte chunk c of tile row `row` sits at chunk position c ^ swz(row): rows r and r + 4, which
  // the two halves of a wave read together when the V tile is transposed, land on different banks
  static __device__ __forceinline__ int swz(int row) { return ((row >> 2) & 1) << 2; }
};

struct PrepParams {
  const unsigned short *q, *k, *v;
  const float *cos_t, *sin_t;
  const int* orders;
  const unsigned short* k_mean;
  int8_t* q8;
  float* q_scale;
  int8_t* k8;
  float* k_scale;
  uint8_t* v8;
  const float* v_stats;  // per (batch, head): D reciprocal scales, then D means, at v_recp_offset
  float* v_resid;        // rounding residual sums of the V codes, [B*H][nb][2][D] (nullptr: not wanted)
  int BH, H, N, nb, n_text, F, Hh, W, head_split;
  int64_t qs_b, qs_h, qs_n, ks_b, ks_h, ks_n, vs_b, vs_h, vs_n, ms_b, ms_h;
};

// out-of-range bytes of a raw buffer read as 0 and are not written: `bytes` = 0 switches a whole
// access off without a branch
__device__ __forceinline__ __amdgpu_buffer_rsrc_t raw_buffer(const void* base, int bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(base), 0, bytes, 0x00020000);
}

// LDS-DMA: 16 (or 4) bytes per lane from a buffer straight into LDS at lds + lane*16 (lane*4); no
// registers, no ds_write; completion is counted with the wave's other vector-memory operations.  The
// token rows are read once: non-temporal.
__device__ __forceinline__ void buffer_load16_lds_once(__amdgpu_buffer_rsrc_t rsrc, uint8_t* lds, int voffset) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)lds, 16, voffset, 0, 0, 2);
}
__device__ __forceinline__ void buffer_load16_lds(__amdgpu_buffer_rsrc_t rsrc, uint8_t* lds, int voffset) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)lds, 16, voffset, 0, 0, 0);
}
__device__ __forceinline__ void buffer_load4_lds(__amdgpu_buffer_rsrc_t rsrc, uint8_t* lds, int voffset) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)lds, 4, voffset, 0, 0, 0);
}

// waits until at most N of this wave's vector-memory operations are outstanding (they complete in
// issue order) and all of its LDS operations are done
template <int N> __device__ __forceinline__ void wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(N) : "memory");
}

template <int DT, int D>
__global__ void __launch_bounds__(256) rope_permute_quant_kernel(const PrepParams p) {
  using L = PrepLds<D>;
  constexpr int LPR = D / 8;            // lanes per token row (16-byte pieces)
  constexpr int RPI = 64 / LPR;         // rows one wave covers per load instruction
  constexpr int PC = 16 / RPI;          // pieces per lane and tile: a wave owns 16 rows of the block
  constexpr int NV = D == 128 ? 2 : 1;  // distinct channel offsets among a lane's pieces
  // vector-memory operations one wave issues per pair: PC per tile, two more with the K tile (mean
  // row, V statistics row), and ST stores that are issued unconditionally (q8, k8: PC each, v8 and its
  // residual sums: D/64 each)
  constexpr int ST = 2 * PC + 2 * (D / 64);
  constexpr int OOB = 0x7ffffff0;       // offset beyond any descriptor range

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  unsigned short* s_list = reinterpret_cast<unsigned short*>(smem + L::LIST_OFF);
  __shared__ int s_src[64];             // source token of each destination row, -1 past the end
  __shared__ float s_amax[2][4];        // [q|k][wave]
  __shared__ int s_npairs;

  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int kb = blockIdx.x;
  const int order = blockIdx.y % 6, split = blockIdx.y / 6;
  const bool rope = p.cos_t != nullptr;

  if (t < 64) {
    const int d = kb * 64 + t;
    int src = -1;
    if (d < p.N) src = d < p.n_text ? d : p.n_text + unpermute_index(d - p.n_text, order, p.F, p.Hh, p.W);
    s_src[t] = src;
  }
  if (wave == 1) {
    // the (batch, head) pairs whose head uses this workgroup's order, every head_split-th of them
    int cnt = 0;
    for (int base = 0; base < p.BH; base += 64) {
      const int bh = base + lane;
      bool match = false;
      if (bh < p.BH) {
        const int o = p.orders[bh % p.H];
        match = ((unsigned)o > 5u ? 0 : o) == order;   // as order_strides treats it
      }
      const unsigned long long bal = __ballot(match);
      const int idx = cnt + __popcll(bal & ((1ull << lane) - 1ull));
      if (match && idx % p.head_split == split) s_list[idx / p.head_split] = (unsigned short)bh;
      cnt += __popcll(bal);
    }
    if (lane == 0) s_npairs = cnt > split ? (cnt - split + p.head_split - 1) / p.head_split : 0;
  }
  __syncthreads();
  const int npairs = s_npairs;
  if (npairs == 0) return;

  // this lane's pieces: tile rows 16*wave + i*RPI + lane/LPR; LDS chunk position lane%LPR of such a
  // row holds channels col..col+7.  Their rotary-table entries stay in registers for every pair.
  int src[PC], col[NV], voq[PC], vok[PC], vov[PC];
  float cs[PC][8], sn[PC][8];
#pragma unroll
  for (int i = 0; i < PC; i++) {
    const int row = 16 * wave + i * RPI + lane / LPR;
    const int c = ((lane % LPR) ^ L::swz(row)) * 8;
    if (i < NV) col[i] = c;
    src[i] = s_src[row];
    voq[i] = vok[i] = vov[i] = OOB;
    if (src[i] >= 0) {
      voq[i] = (int)(((int64_t)src[i] * p.qs_n + c) * 2);
      vok[i] = (int)(((int64_t)src[i] * p.ks_n + c) * 2);
      vov[i] = (int)(((int64_t)src[i] * p.vs_n + c) * 2);
    }
  }
  const int n_chunks = (p.N + V_CHUNK - 1) / V_CHUNK;
  const int q_bytes = (int)((((int64_t)p.N - 1) * p.qs_n + D) * 2);
  const int k_bytes = (int)((((int64_t)p.N - 1) * p.ks_n + D) * 2);
  const int v_bytes = (int)((((int64_t)p.N - 1) * p.vs_n + D) * 2);

  // ---- tile movers: every wave fetches the 16 rows it will itself rotate and quantise, so Q and K
  //      need no barrier, only the wave's own wait; the V tile is read across waves -----------------
  auto load_tile = [&](const unsigned short* base, int bytes, const int* voff, int slot) {
    const __amdgpu_buffer_rsrc_t r = raw_buffer(base, bytes);
#pragma unroll
    for (int i = 0; i < PC; i++)
      buffer_load16_lds_once(r, smem + slot * L::TILE + (wave_u * PC + i) * 1024, voff[i]);
  };
  // the pair the loads are issued for: (batch nx_b, head nx_h), or none (nx_bh < 0): the loads are
  // still issued then (the wait counts stay the same) but fetch nothing
  int nx_bh, nx_b = 0, nx_h = 0;
  auto set_next = [&](int bh) {
    nx_bh = bh;
    if (bh >= 0) { nx_b = bh / p.H; nx_h = bh - nx_b * p.H; }
  };
  auto load_q = [&](int slot) {
    load_tile(p.q + nx_b * p.qs_b + nx_h * p.qs_h, nx_bh < 0 ? 0 : q_bytes, voq, slot);
  };
  auto load_k = [&](int slot, int par) {
    const int bh = nx_bh, b = nx_b, head = nx_h;
    load_tile(p.k + b * p.ks_b + head * p.ks_h, bh < 0 ? 0 : k_bytes, vok, slot);
    // the pair's K mean row (zeros without smoothing) and its V statistics: every wave fetches the
    // same bytes to the same place
    const bool km = bh >= 0 && p.k_mean != nullptr;
    const __amdgpu_buffer_rsrc_t rm = raw_buffer(km ? p.k_mean + b * p.ms_b + head * p.ms_h : p.k, km ? D * 2 : 0);
    buffer_load4_lds(rm, smem + L::KM_OFF + par * 256, lane * 4);
    const __amdgpu_buffer_rsrc_t rs =
        raw_buffer(bh < 0 ? p.v_stats : p.v_stats + v_recp_offset(bh, n_chunks, D), bh < 0 ? 0 : 2 * D * 4);
    buffer_load16_lds(rs, smem + L::ST_OFF + par * 1024, lane * 16);
  };
  auto load_v = [&](int slot) {
    load_tile(p.v + nx_b * p.vs_b + nx_h * p.vs_h, nx_bh < 0 ? 0 : v_bytes, vov, slot);
  };
  auto own_piece = [&](int slot, int i) {
    return *reinterpret_cast<const v4i*>(smem + slot * L::TILE + (wave_u * PC + i) * 1024 + lane * 16);
  };

  set_next(__builtin_amdgcn_readfirstlane((int)s_list[0]));
  load_q(0);
  load_k(1, 0);
  load_v(2);
  // the table entries are fetched behind the first pair's tiles and pinned down here, so that nothing
  // but the tile stream is outstanding once the loop runs
#pragma unroll
  for (int i = 0; i < PC; i++) {
    if (rope && src[i] >= p.n_text) {
      const int64_t o = (int64_t)(src[i] - p.n_text) * D + col[i % NV];
      const v4f c0 = *reinterpret_cast<const v4f*>(p.cos_t + o), c1 = *reinterpret_cast<const v4f*>(p.cos_t + o + 4);
      const v4f s0 = *reinterpret_cast<const v4f*>(p.sin_t + o), s1 = *reinterpret_cast<const v4f*>(p.sin_t + o + 4);
#pragma unroll
      for (int e = 0; e < 4; e++) {
        cs[i][e] = c0[e]; cs[i][4 + e] = c1[e];
        sn[i][e] = s0[e]; sn[i][4 + e] = s1[e];
      }
    }
  }
#pragma unroll
  for (int i = 0; i < PC; i++)
#pragma unroll
    for (int e = 0; e < 8; e++) asm volatile("" : "+v"(cs[i][e]), "+v"(sn[i][e]));
  int j = 0;  // ring position of the current pair's Q tile (tile number mod 4)
  for (int ip = 0; ip < npairs; ip++) {
    const int bh = nx_bh;
    set_next(ip + 1 < npairs ? __builtin_amdgcn_readfirstlane((int)s_list[ip + 1]) : -1);
    const int par = ip & 1;

    // ---- Q tile: wait for this wave's rows; the barrier says every wave has finished with the V
    //      tile of the previous pair, whose slot the next Q tile is fetched into -------------------
    if (ip == 0) wait_vm<2 * PC + 2>(); else wait_vm<2 * PC + 2 + ST>();
    __builtin_amdgcn_s_barrier();
    load_q((j + 3) & 3);
    // rotated values, rounded to the input type as the permuted tensors would hold them, kept in fp32
    float fq[PC][8], fk[PC][8];
    float aq = 0.0000001f, ak = 0.0000001f;
#pragma unroll
    for (int i = 0; i < PC; i++) {
      rotate8_f32<DT>(own_piece(j & 3, i), rope && src[i] >= p.n_text, cs[i], sn[i], fq[i]);
#pragma unroll
      for (int e = 0; e < 8; e++) aq = fmaxf(aq, fabsf(fq[i][e]));   // rows past the end are 0
    }
    aq = wave_max(aq);
    if (lane == 0) s_amax[0][wave] = aq;

    // ---- K tile (its slot's next tenant is fetched by the same wave into the same rows) ---------
    if (ip == 0) wait_vm<2 * PC>(); else wait_vm<2 * PC + ST>();
    load_k(j & 3, par ^ 1);
    float mv[NV][8];
#pragma unroll
    for (int n = 0; n < NV; n++) {
      const v4i m = *reinterpret_cast<const v4i*>(smem + L::KM_OFF + par * 256 + col[n] * 2);
#pragma unroll
      for (int e = 0; e < 8; e++) mv[n][e] = elem16_to_f32<DT>(m, e);
    }
#pragma unroll
    for (int i = 0; i < PC; i++) {
      rotate8_f32<DT>(own_piece((j + 1) & 3, i), rope && src[i] >= p.n_text, cs[i], sn[i], fk[i]);
      // the mean goes off here; rows past the end count as zero, whatever the mean
#pragma unroll
      for (int e = 0; e < 8; e++) {
        fk[i][e] = src[i] >= 0 ? fk[i][e] - mv[i % NV][e] : 0.f;
        ak = fmaxf(ak, fabsf(fk[i][e]));
      }
    }
    ak = wave_max(ak);
    if (lane == 0) s_amax[1][wave] = ak;

    // ---- V tile: landed in every wave, and the group maxima are visible ------------------------
    if (ip == 0) wait_vm<2 * PC + 2>(); else wait_vm<2 * PC + 2 + ST>();
    __builtin_amdgcn_s_barrier();
    load_v((j + 1) & 3);
    // group maxima: Q per 32 rows (two waves), K per 64 rows (the workgroup)
    aq = fmaxf(s_amax[0][wave & 2], s_amax[0][(wave & 2) + 1]);
    ak = fmaxf(fmaxf(s_amax[1][0], s_amax[1][1]), fmaxf(s_amax[1][2], s_amax[1][3]));
    if (lane == 0 && (wave & 1) == 0) p.q_scale[(int64_t)bh * (p.nb * 2) + kb * 2 + (wave >> 1)] = aq / 127.0f;
    if (t == 0) p.k_scale[(int64_t)bh * p.nb + kb] = ak / 127.0f;
    const float inv_q = 127.0f / aq, inv_k = 127.0f / ak;
    {
      // rows >= N fall outside the descriptor and are not written
      const __amdgpu_buffer_rsrc_t rq8 = raw_buffer(p.q8 + (int64_t)bh * p.N * D, p.N * D);
      const __amdgpu_buffer_rsrc_t rk8 = raw_buffer(p.k8 + (int64_t)bh * p.N * D, p.N * D);
#pragma unroll
      for (int i = 0; i < PC; i++) {
        // |x * (127/amax)| <= 127 up to rounding: the reference's clamp to [-128,127] never acts
        float yq[8], yk[8];
#pragma unroll
        for (int e = 0; e < 8; e++) {
          yq[e] = fq[i][e] * inv_q;
          yk[e] = fk[i][e] * inv_k;
        }
        const int o = (kb * 64 + 16 * wave + i * RPI + lane / LPR) * D + col[i % NV];
        __builtin_amdgcn_raw_buffer_store_b64(
            v2u{pack4_rint_i8(yq[0], yq[1], yq[2], yq[3]), pack4_rint_i8(yq[4], yq[5], yq[6], yq[7])}, rq8, o, 0, 2);
        __builtin_amdgcn_raw_buffer_store_b64(
            v2u{pack4_rint_i8(yk[0], yk[1], yk[2], yk[3]), pack4_rint_i8(yk[4], yk[5], yk[6], yk[7])}, rk8, o, 0, 2);
      }
    }
    // V tile -> e4m3 fragments
    const float* st = reinterpret_cast<const float*>(smem + L::ST_OFF + par * 1024);
    float rs[D / 64];
    pack_v_tile<DT, D, D, true>(reinterpret_cast<const unsigned short*>(smem + ((j + 2) & 3) * L::TILE),
                                p.v8 + ((int64_t)bh * p.nb + kb) * (int64_t)(64 * D), st, st + D, kb * 64, p.N, t, rs);
    {
      // lanes 0..31 hold the sums of row tile wave%2, channels 32*(wave/2 + 2n) + lane; the store is issued
      // by every wave whether wanted or not (a descriptor of 0 bytes drops it), so the wait counts hold
      const __amdgpu_buffer_rsrc_t rr =
          raw_buffer(p.v_resid ? p.v_resid + ((int64_t)bh * p.nb + kb) * (2 * D) : p.q_scale, p.v_resid ? 2 * D * 4 : 0);
#pragma unroll
      for (int n = 0; n < D / 64; n++)
        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(rs[n]), rr,
                                              lane < 32 ? ((wave & 1) * D + 32 * ((wave >> 1) + 2 * n) + lane) * 4 : OOB,
                                              0, 0);
    }
    j = (j + 3) & 3;
  }
  // the loads issued for the pair after the last one fetch nothing, but they do write LDS
  wait_vm<0>();
}

// K mean over tokens AFTER the rotation (the permutation does not change a mean) and the V statistics: the bodies
// live in stats_device.hpp.  Alone (paro_rope_k_mean), or both in ONE launch when the preparation smooths K
// itself: a workgroup takes a K chunk of a head group or a V chunk of a head, and one more launch finishes both.
template <int DT, int D, int KB>
__global__ void __launch_bounds__(256) rope_k_sum_kernel(const unsigned short* __restrict__ k,
                                                         const float* __restrict__ cos_t,
                                                         const float* __restrict__ sin_t,
                                                         float* __restrict__ partial, int BH, int H, int N,
                                                         int n_text, int n_chunks, int64_t ks_b, int64_t ks_h,
                                                         int64_t ks_n) {
  rope_k_sum_body<DT, D, KB>(k, cos_t, sin_t, partial, BH, H, N, n_text, n_chunks, ks_b, ks_h, ks_n, blockIdx.x);
}

template <int DT, int D>
__global__ void __launch_bounds__(1024) k_mean_finalize_kernel(const float* __restrict__ partial,
                                                               unsigned short* __restrict__ k_mean, int N,
                                                               int n_chunks, int64_t ms_b, int64_t ms_h, int H) {
  k_mean_finalize_body<DT, D>(partial, k_mean, N, n_chunks, ms_b, ms_h, H, blockIdx.x);
}

// workgroups of the K sums: XCD x takes the chunks 8*i + x, and for each of them all head groups
static inline int k_sum_blocks(int n_chunks, int BH) { return ceil_div(n_chunks, 8) * 8 * ceil_div(BH, KM_GROUP); }

struct KvStatsParams {
  const unsigned short* k; const unsigned short* v;
  const float* cos_t; const float* sin_t;
  float* k_partial; float* v_partial;
  unsigned short* k_mean; float* v_scale; float* v_mean;
  int B, H, N, n_text, k_chunks, v_chunks, k_blocks, smooth_v;
  int64_t ks_b, ks_h, ks_n, vs_b, vs_h, vs_n, ms_b, ms_h;
};

template <int DT, int D, int KB>
__global__ void __launch_bounds__(256) kv_stats_kernel(const KvStatsParams p) {
  if ((int)blockIdx.x < p.k_blocks) {
    rope_k_sum_body<DT, D, KB>(p.k, p.cos_t, p.sin_t, p.k_partial, p.B * p.H, p.H, p.N, p.n_text, p.k_chunks, p.ks_b,
                               p.ks_h, p.ks_n, blockIdx.x);
  } else {
    const int i = blockIdx.x - p.k_blocks;
    const int chunk = i % p.v_chunks, bh = i / p.v_chunks;
    v_stats_body<DT, D>(p.v, p.v_partial, p.N, p.v_chunks, p.vs_b, p.vs_h, p.vs_n, chunk, bh % p.H, bh / p.H, p.H);
  }
}

template <int DT, int D>
__global__ void __launch_bounds__(1024) kv_finalize_kernel(const KvStatsParams p) {
  const int BH = p.B * p.H;
  if ((int)blockIdx.x < BH)
    k_mean_finalize_body<DT, D>(p.k_partial, p.k_mean, p.N, p.k_chunks, p.ms_b, p.ms_h, p.H, blockIdx.x);
  else
    v_finalize_body<D>(p.v_partial, p.v_scale, p.v_mean, p.N, p.v_chunks, p.smooth_v, (int64_t)blockIdx.x - BH);
}

template <int DT, int D>
static int launch_prep(const PrepParams& p, dim3 grid, hipStream_t st) {
  auto kern = rope_permute_quant_kernel<DT, D>;
  constexpr int lds = PrepLds<D>::BYTES;
  if (lds > 48 * 1024)
    PARO_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
  hipLaunchKernelGGL(kern, grid, dim3(256), lds, st, p);
  return PARO_OK;
}

static int check_prep(const char* fn, int dtype, int B, int H, int N, int D, int n_text, int F, int Hh, int W,
                      int64_t s_b, int64_t s_h, int64_t s_n) {
  PARO_CHECK(B > 0 && H > 0 && N > 0, PARO_ERR_RUNTIME, "%s: empty shape", fn);
  PARO_CHECK((int64_t)B * H <= MAX_GRID_YZ, PARO_ERR_RUNTIME, "%s: batch * heads = %lld exceeds %d", fn,
             (long long)B * H, MAX_GRID_YZ);
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
  // per-chunk partials of the V statistics (sum, min, max) or of the K mean (sums), whichever is larger
  const int64_t v_part = paro_v_fp8_partial_floats(B, H, N, D);
  const int64_t k_part = (int64_t)B * H * paro::ceil_div(N, paro::K_CHUNK) * D;
  return (v_part > k_part ? v_part : k_part) * 4;
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
  const int n_chunks = ceil_div(N, K_CHUNK);
  PARO_CHECK(workspace_bytes >= (int64_t)B * H * n_chunks * D * 4, PARO_ERR_RUNTIME,
             "paro_rope_k_mean: workspace of %lld bytes is too small", (long long)workspace_bytes);
  hipStream_t st = (hipStream_t)stream;
  float* partial = (float*)workspace;
  // tokens per thread whose loads are requested together: 2 at D = 64, 1 at D = 128 (measured)
#define PARO_KM(DTV, DV)                                                                                        \
  do {                                                                                                          \
    hipLaunchKernelGGL((rope_k_sum_kernel<DTV, DV, (DV == 64 ? 2 : 1)>), dim3(k_sum_blocks(n_chunks, B * H)), dim3(256), 0, \
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

extern "C" int paro_rope_k_mean_static(const void* k, int dtype, const float* cos, const float* sin, void* k_mean,
                                       int B, int H, int N, int D, int n_text, int F, int Hh, int W,
                                       int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_n,
                                       int64_t mean_stride_b, int64_t mean_stride_h, void* stream) {
  using namespace paro;
  PARO_CHECK(B > 0 && H > 0 && N > 0 && (D == 64 || D == 128), PARO_ERR_INVALID_VALUE,
             "Unsupported shape or head dim: B=%d H=%d N=%d D=%d", B, H, N, D);
  const int64_t need = (int64_t)B * H * ceil_div(N, K_CHUNK) * D;
  PARO_CHECK(need <= KMEAN_SCRATCH_FLOATS, PARO_ERR_RUNTIME,
             "paro_rope_k_mean_static: B*H*ceil(N/%d)*D = %lld partial sums exceed the built-in work buffer of %lld "
             "floats; use paro_rope_k_mean with a workspace of its own",
             K_CHUNK, (long long)need, (long long)KMEAN_SCRATCH_FLOATS);
  float* ws = nullptr;
  if (int rc = kmean_scratch_of_current_device(&ws)) return rc;
  // every partial sum the second launch reads is written by the first: nothing of the buffer has to
  // start at zero, whatever the previous call left in it
  return paro_rope_k_mean(k, dtype, cos, sin, k_mean, ws, KMEAN_SCRATCH_FLOATS * 4, B, H, N, D, n_text, F, Hh, W,
                          k_stride_b, k_stride_h, k_stride_n, mean_stride_b, mean_stride_h, stream);
}

namespace paro {
// compute_k_mean: k_mean is an output (the mean of the rotated K, as paro_rope_k_mean gives it) that this call
// fills before it uses it; the K sums and the V statistics then share one launch, and so do their second steps.
static int prep_impl(bool compute_k_mean, const void* q, const void* k, const void* v, int dtype, const float* cos,
                                           const float* sin, const int32_t* orders, const void* k_mean,
                                           int8_t* q8, float* q_scale, int8_t* k8, float* k_scale, uint8_t* v8,
                                           float* v_scale, float* v_mean, void* workspace, int64_t workspace_bytes,
                                           int B, int H, int N, int D, int n_text, int F, int Hh, int W,
                                           int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_n,
                                           int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_n,
                                           int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_n,
                                           int64_t mean_stride_b, int64_t mean_stride_h, int smooth_v,
                                           void* stream) {
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
  PARO_CHECK(!compute_k_mean || k_mean, PARO_ERR_RUNTIME, "paro_rope_k_mean_permute_quant_fwd: null k_mean");
  PARO_CHECK(workspace_bytes >= (compute_k_mean ? paro_prep_smooth_workspace_bytes(B, H, N, D)
                                                : paro_prep_workspace_bytes(B, H, N, D)) &&
                 ((uintptr_t)workspace % 16) == 0,
             PARO_ERR_RUNTIME, "paro_rope_permute_quant_fwd: workspace of %lld bytes is too small or misaligned",
             (long long)workspace_bytes);
  // one (batch, head) slice of each input and of q8 / k8 is addressed through 32-bit buffer offsets
  PARO_CHECK(q_stride_n >= D && k_stride_n >= D && v_stride_n >= D &&
                 ((int64_t)N - 1) * q_stride_n + D < (int64_t)1 << 30 &&
                 ((int64_t)N - 1) * k_stride_n + D < (int64_t)1 << 30 &&
                 ((int64_t)N - 1) * v_stride_n + D < (int64_t)1 << 30,
             PARO_ERR_RUNTIME, "paro_rope_permute_quant_fwd: one head of q, k or v spans 2 GiB or more");
  hipStream_t st = (hipStream_t)stream;
  // V statistics do not depend on the token order: taken on the unpermuted tensor
  if (!compute_k_mean) {
    if (int rc = v_fp8_stats(v, dtype, v_scale, v_mean, (float*)workspace, B, H, N, D, v_stride_b, v_stride_h,
                             v_stride_n, smooth_v, st))
      return rc;
  } else {
    KvStatsParams sp;
    sp.k = (const unsigned short*)k; sp.v = (const unsigned short*)v; sp.cos_t = cos; sp.sin_t = sin;
    sp.v_partial = (float*)workspace;
    sp.k_partial = (float*)workspace + paro_v_fp8_partial_floats(B, H, N, D);   // behind the V partials
    sp.k_mean = (unsigned short*)k_mean; sp.v_scale = v_scale; sp.v_mean = v_mean;
    sp.B = B; sp.H = H; sp.N = N; sp.n_text = n_text; sp.k_chunks = ceil_div(N, K_CHUNK); sp.v_chunks = ceil_div(N, V_CHUNK);
    sp.k_blocks = k_sum_blocks(sp.k_chunks, B * H); sp.smooth_v = smooth_v;
    sp.ks_b = k_stride_b; sp.ks_h = k_stride_h; sp.ks_n = k_stride_n;
    sp.vs_b = v_stride_b; sp.vs_h = v_stride_h; sp.vs_n = v_stride_n; sp.ms_b = mean_stride_b; sp.ms_h = mean_stride_h;
    const int n_blocks = sp.k_blocks + sp.v_chunks * B * H;
#define PARO_KV(DTV, DV)                                                                                          \
  do {                                                                                                            \
    hipLaunchKernelGGL((kv_stats_kernel<DTV, DV, (DV == 64 ? 2 : 1)>), dim3(n_blocks), dim3(256), 0, st, sp);      \
    hipLaunchKernelGGL((kv_finalize_kernel<DTV, DV>), dim3(2 * B * H), dim3(1024), 0, st, sp);                    \
  } while (0)
    if (dtype == PARO_DTYPE_F16) {
      if (D == 64) PARO_KV(PARO_DTYPE_F16, 64); else PARO_KV(PARO_DTYPE_F16, 128);
    } else {
      if (D == 64) PARO_KV(PARO_DTYPE_BF16, 64); else PARO_KV(PARO_DTYPE_BF16, 128);
    }
#undef PARO_KV
    PARO_HIP(hipGetLastError());
  }
  const int nb = ceil_div(N, 64);
  // every order gets `head_split` workgroups per block, each walking over its share of the (batch,
  // head) pairs with that order: enough workgroups to fill the chip, few enough that the table rows a
  // workgroup holds are reused
  int head_split = 1;
  while (head_split < 8 && (int64_t)nb * 6 * head_split < 2048 && head_split * 2 <= B * H) head_split *= 2;
  while (ceil_div(B * H, head_split) > PrepLds<64>::MAX_PAIRS) head_split *= 2;   // the list a workgroup keeps in LDS
  PrepParams p;
  p.q = (const unsigned short*)q; p.k = (const unsigned short*)k; p.v = (const unsigned short*)v;
  p.cos_t = cos; p.sin_t = sin; p.orders = (const int*)orders; p.k_mean = (const unsigned short*)k_mean;
  p.q8 = q8; p.q_scale = q_scale; p.k8 = k8; p.k_scale = k_scale; p.v8 = v8; p.v_stats = (const float*)workspace;
  p.v_resid = smooth_v ? (float*)workspace + v_resid_offset((int64_t)B * H, ceil_div(N, V_CHUNK), D) : nullptr;
  p.BH = B * H; p.H = H; p.N = N; p.nb = nb; p.n_text = n_text; p.F = F; p.Hh = Hh; p.W = W; p.head_split = head_split;
  p.qs_b = q_stride_b; p.qs_h = q_stride_h; p.qs_n = q_stride_n;
  p.ks_b = k_stride_b; p.ks_h = k_stride_h; p.ks_n = k_stride_n;
  p.vs_b = v_stride_b; p.vs_h = v_stride_h; p.vs_n = v_stride_n;
  p.ms_b = mean_stride_b; p.ms_h = mean_stride_h;
  dim3 grid(nb, 6 * head_split);
#define PARO_PREP(DTV, DV) rc = launch_prep<DTV, DV>(p, grid, st)
  int rc;
  if (dtype == PARO_DTYPE_F16) {
    if (D == 64) PARO_PREP(PARO_DTYPE_F16, 64); else PARO_PREP(PARO_DTYPE_F16, 128);
  } else {
    if (D == 64) PARO_PREP(PARO_DTYPE_BF16, 64); else PARO_PREP(PARO_DTYPE_BF16, 128);
  }
#undef PARO_PREP
  if (rc) return rc;
  PARO_HIP(hipGetLastError());
  if (p.v_resid) return v_fp8_add_residual(p.v_resid, v_scale, v_mean, B, H, N, D, st);
  return PARO_OK;
}
}  // namespace paro

extern "C" int64_t paro_prep_smooth_workspace_bytes(int B, int H, int N, int D) {
  // the V partials and, behind them, the K partial sums: both are alive at the same time
  return (paro_v_fp8_partial_floats(B, H, N, D) + (int64_t)B * H * paro::ceil_div(N, paro::K_CHUNK) * D) * 4;
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
  return paro::prep_impl(false, q, k, v, dtype, cos, sin, orders, k_mean, q8, q_scale, k8, k_scale, v8, v_scale, v_mean,
                         workspace, workspace_bytes, B, H, N, D, n_text, F, Hh, W, q_stride_b, q_stride_h, q_stride_n,
                         k_stride_b, k_stride_h, k_stride_n, v_stride_b, v_stride_h, v_stride_n, mean_stride_b,
                         mean_stride_h, smooth_v, stream);
}

extern "C" int paro_rope_k_mean_permute_quant_fwd(const void* q, const void* k, const void* v, int dtype,
                                                  const float* cos, const float* sin, const int32_t* orders,
                                                  void* k_mean, int8_t* q8, float* q_scale, int8_t* k8,
                                                  float* k_scale, uint8_t* v8, float* v_scale, float* v_mean,
                                                  void* workspace, int64_t workspace_bytes, int B, int H, int N,
                                                  int D, int n_text, int F, int Hh, int W, int64_t q_stride_b,
                                                  int64_t q_stride_h, int64_t q_stride_n, int64_t k_stride_b,
                                                  int64_t k_stride_h, int64_t k_stride_n, int64_t v_stride_b,
                                                  int64_t v_stride_h, int64_t v_stride_n, int64_t mean_stride_b,
                                                  int64_t mean_stride_h, int smooth_v, void* stream) {
  return paro::prep_impl(true, q, k, v, dtype, cos, sin, orders, k_mean, q8, q_scale, k8, k_scale, v8, v_scale, v_mean,
                         workspace, workspace_bytes, B, H, N, D, n_text, F, Hh, W, q_stride_b, q_stride_h, q_stride_n,
                         k_stride_b, k_stride_h, k_stride_n, v_stride_b, v_stride_h, v_stride_n, mean_stride_b,
                         mean_stride_h, smooth_v, stream);
}
