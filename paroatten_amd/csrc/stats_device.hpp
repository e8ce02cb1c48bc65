// Statistics passes of the path as device functions, so that one launch can run several of them side by side:
// per-channel sum / min / max of V (for the FP8 scale and mean) and the mean of the rotated K (for K smoothing).
// The launches that use them: v_fp8.hip (V alone), fused_prep.hip (K alone, or K and V in one launch).
#pragma once
#include "paro_device.hpp"

namespace paro {

// Per-channel sum, minimum and maximum of one V_CHUNK-token chunk of one (batch, head): 256 threads.
template <int DT, int D>
__device__ __forceinline__ void v_stats_body(const unsigned short* __restrict__ v, float* __restrict__ partial, int N,
                                             int n_chunks, int64_t vs_b, int64_t vs_h, int64_t vs_n, int chunk, int h,
                                             int b, int H) {
  constexpr int LPR = D / 8;
  constexpr int ROWS = 256 / LPR;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int col = (t % LPR) * 8;
  const unsigned short* vb = v + b * vs_b + h * vs_h + col;
  float s[8], mn[8], mx[8];
#pragma unroll
  for (int j = 0; j < 8; j++) {
    s[j] = 0.f;
    mn[j] = INFINITY;
    mx[j] = -INFINITY;
  }
  auto take = [&](const v4i raw) {
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const float f = elem16_to_f32<DT>(raw, j);
      s[j] += f;
      mn[j] = fminf(mn[j], f);
      mx[j] = fmaxf(mx[j], f);
    }
  };
  const int tok0 = chunk * V_CHUNK + t / LPR;
  if (chunk * V_CHUNK + V_CHUNK <= N) {
    // full chunk (uniform): batches of VS_BATCH independent loads, then the arithmetic
    constexpr int VS_BATCH = 8;
    for (int r = 0; r < V_CHUNK; r += ROWS * VS_BATCH) {
      v4i raw[VS_BATCH];
#pragma unroll
      for (int u = 0; u < VS_BATCH; u++)
        // (non-temporal: measured 3-5 us faster per launch of the entry point and of the per-layer sequence
        // than ordinary loads, although the packing pass reads the same tensor right afterwards)
        raw[u] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(vb + (int64_t)(tok0 + r + u * ROWS) * vs_n));
#pragma unroll
      for (int u = 0; u < VS_BATCH; u++) take(raw[u]);
    }
  } else {
    for (int r = 0; r < V_CHUNK; r += ROWS) {
      const int tok = tok0 + r;
      if (tok < N) take(*reinterpret_cast<const v4i*>(vb + (int64_t)tok * vs_n));
    }
  }
  // lanes that share a column sit LPR apart: 8 lanes round the row (D = 64 only), then lane ^ 16, ^ 32
#pragma unroll
  for (int j = 0; j < 8; j++) {
    float a, b;
    if constexpr (LPR == 8) {
      s[j] += row_dpp<0x128>(s[j]);
      mn[j] = fminf(mn[j], row_dpp<0x128>(mn[j]));
      mx[j] = fmaxf(mx[j], row_dpp<0x128>(mx[j]));
    }
    with_lane_xor16(s[j], a, b);  s[j] = a + b;
    with_lane_xor16(mn[j], a, b); mn[j] = fminf(a, b);
    with_lane_xor16(mx[j], a, b); mx[j] = fmaxf(a, b);
    with_lane_xor32(s[j], a, b);  s[j] = a + b;
    with_lane_xor32(mn[j], a, b); mn[j] = fminf(a, b);
    with_lane_xor32(mx[j], a, b); mx[j] = fmaxf(a, b);
  }
  __shared__ float red[4][3][D];
  if (lane < LPR) {
#pragma unroll
    for (int j = 0; j < 8; j++) {
      red[wave][0][col + j] = s[j];
      red[wave][1][col + j] = mn[j];
      red[wave][2][col + j] = mx[j];
    }
  }
  __syncthreads();
  if (t < D) {
    const float ss = (red[0][0][t] + red[1][0][t]) + (red[2][0][t] + red[3][0][t]);
    const float mm = fminf(fminf(red[0][1][t], red[1][1][t]), fminf(red[2][1][t], red[3][1][t]));
    const float xx = fmaxf(fmaxf(red[0][2][t], red[1][2][t]), fmaxf(red[2][2][t], red[3][2][t]));
    float* p = partial + (((int64_t)(b * H + h) * n_chunks + chunk) * 3) * D;
    p[t] = ss;
    p[D + t] = mm;
    p[2 * D + t] = xx;
  }
}


// mean, scale and reciprocal scale of one (batch, head) from its chunk statistics: 1024 threads.
template <int D>
__device__ __forceinline__ void v_finalize_body(float* partial, float* __restrict__ v_scale, float* __restrict__ v_mean,
                                                int N, int n_chunks, int smooth, int64_t bh) {
  // 1024 / D slices of the chunk range per channel, combined through LDS in a fixed order
  constexpr int SL = 1024 / D;
  __shared__ float red[3][SL][D];
  const int ch = threadIdx.x % D, sl = threadIdx.x / D;
  const float* p = partial + bh * n_chunks * 3 * D;
  float s = 0.f, mn = INFINITY, mx = -INFINITY;
  for (int c = sl; c < n_chunks; c += SL) {
    s += p[(c * 3 + 0) * D + ch];
    mn = fminf(mn, p[(c * 3 + 1) * D + ch]);
    mx = fmaxf(mx, p[(c * 3 + 2) * D + ch]);
  }
  red[0][sl][ch] = s;
  red[1][sl][ch] = mn;
  red[2][sl][ch] = mx;
  __syncthreads();
  if (sl == 0) {
    for (int i = 1; i < SL; i++) {
      s += red[0][i][ch];
      mn = fminf(mn, red[1][i][ch]);
      mx = fmaxf(mx, red[2][i][ch]);
    }
    const float mean = smooth ? s / (float)N : 0.f;
    const float amax = fmaxf(mx - mean, mean - mn);
    v_scale[bh * D + ch] = amax / 448.0f;
    if (v_mean) v_mean[bh * D + ch] = mean;
    // every thread of this workgroup has read its partials before the barrier above: the head of the
    // region is free to carry the reciprocal, and behind it the mean, to the pack kernel
    partial[v_recp_offset(bh, n_chunks, D) + ch] = amax > 0.f ? 448.0f / amax : 0.f;
    partial[v_recp_offset(bh, n_chunks, D) + D + ch] = mean;
  }
}


// K mean over tokens AFTER the rotation (the permutation does not change a mean): partial sums per
// K_CHUNK-token chunk, then one workgroup per (batch, head) adds them in a fixed order.  A thread keeps
// the table entries of its token piece while it walks over a group of (batch, head) pairs.
constexpr int KM_GROUP = 4;   // measured: 4 beats 8 (too few workgroups at 40 heads) and 2 (tables re-read twice as often)
template <int DT, int D, int KB>
__device__ __forceinline__ void rope_k_sum_body(const unsigned short* __restrict__ k, const float* __restrict__ cos_t,
                                                const float* __restrict__ sin_t, float* __restrict__ partial, int BH,
                                                int H, int N, int n_text, int n_chunks, int64_t ks_b, int64_t ks_h,
                                                int64_t ks_n, int block) {
  constexpr int LPR = D / 8;
  constexpr int ROWS = 256 / LPR;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  // Workgroup ids are dealt round-robin to the 8 XCDs: XCD x takes the token chunks 8*i + x, and for each of
  // them all head groups one after the other, so that a chunk of the rotary tables (twice the bytes of the
  // K rows of one head) crosses the fabric once per launch and is served to the other head groups by that
  // XCD's L2.
  const int n_hg = (BH + KM_GROUP - 1) / KM_GROUP;
  const int xcd = block & 7, j = block >> 3;
  const int chunk = (j / n_hg) * 8 + xcd;
  if (chunk >= n_chunks) return;
  const int bh0 = (j % n_hg) * KM_GROUP;
  const int col = (t % LPR) * 8;
  float s[KM_GROUP][8];
#pragma unroll
  for (int g = 0; g < KM_GROUP; g++)
#pragma unroll
    for (int j = 0; j < 8; j++) s[g][j] = 0.f;
  // one step: the rows of one token of the group's heads (table entries first: they are shared by the heads)
  auto add_rows = [&](const v4i (&raw)[KM_GROUP], bool rot, const v4f& c0, const v4f& c1, const v4f& s0, const v4f& s1) {
    float cs[8], sn[8];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      cs[j] = c0[j]; cs[4 + j] = c1[j];
      sn[j] = s0[j]; sn[4 + j] = s1[j];
    }
#pragma unroll
    for (int g = 0; g < KM_GROUP; g++) {
      const v4i x = rot ? rotate8<DT>(raw[g], cs, sn) : raw[g];
#pragma unroll
      for (int j = 0; j < 8; j++) s[g][j] += elem16_to_f32<DT>(x, j);
    }
  };
  const int tok_first = chunk * K_CHUNK;
  const bool full = tok_first + K_CHUNK <= N && bh0 + KM_GROUP <= BH &&
                    (cos_t == nullptr || tok_first >= n_text);   // uniform: every row there, every row rotated alike
  if (full) {
    // batches of KB tokens per thread: their table pieces and K rows are all requested before the first is used
    // (ordinary loads for K: it was just written by the projection and is read again by the preparation pass)
    const bool rot = cos_t != nullptr;
    const unsigned short* kp[KM_GROUP];
#pragma unroll
    for (int g = 0; g < KM_GROUP; g++) {
      const int bh = bh0 + g, b = bh / H, h = bh - b * H;
      kp[g] = k + b * ks_b + h * ks_h + col;
    }
    for (int r = t / LPR; r < K_CHUNK; r += ROWS * KB) {
      v4f c0[KB], c1[KB], s0[KB], s1[KB];
      v4i raw[KB][KM_GROUP];
#pragma unroll
      for (int u = 0; u < KB; u++) {
        const int tok = tok_first + r + u * ROWS;
        if (rot) {
          const int64_t o = (int64_t)(tok - n_text) * D + col;
          c0[u] = *reinterpret_cast<const v4f*>(cos_t + o); c1[u] = *reinterpret_cast<const v4f*>(cos_t + o + 4);
          s0[u] = *reinterpret_cast<const v4f*>(sin_t + o); s1[u] = *reinterpret_cast<const v4f*>(sin_t + o + 4);
        }
#pragma unroll
        for (int g = 0; g < KM_GROUP; g++) raw[u][g] = *reinterpret_cast<const v4i*>(kp[g] + (int64_t)tok * ks_n);
      }
#pragma unroll
      for (int u = 0; u < KB; u++) add_rows(raw[u], rot, c0[u], c1[u], s0[u], s1[u]);
    }
  } else {
    for (int r = t / LPR; r < K_CHUNK; r += ROWS) {
      const int tok = tok_first + r;
      if (tok >= N) break;
      const bool rot = cos_t != nullptr && tok >= n_text;
      v4f c0 = {}, c1 = {}, s0 = {}, s1 = {};
      if (rot) {
        const int64_t o = (int64_t)(tok - n_text) * D + col;
        c0 = *reinterpret_cast<const v4f*>(cos_t + o); c1 = *reinterpret_cast<const v4f*>(cos_t + o + 4);
        s0 = *reinterpret_cast<const v4f*>(sin_t + o); s1 = *reinterpret_cast<const v4f*>(sin_t + o + 4);
      }
      v4i raw[KM_GROUP];
#pragma unroll
      for (int g = 0; g < KM_GROUP; g++) {
        const int bh = min(bh0 + g, BH - 1);   // (a group past the last head re-reads it; its sums are not stored)
        const int b = bh / H, h = bh - b * H;
        raw[g] = *reinterpret_cast<const v4i*>(k + b * ks_b + h * ks_h + (int64_t)tok * ks_n + col);
      }
      add_rows(raw, rot, c0, c1, s0, s1);
    }
  }
  __shared__ float red[4][KM_GROUP][D];
#pragma unroll
  for (int g = 0; g < KM_GROUP; g++) {
    // lanes that share a column sit LPR apart
#pragma unroll
    for (int j = 0; j < 8; j++) {
      float a, b;
      if constexpr (LPR == 8) s[g][j] += row_dpp<0x128>(s[g][j]);
      with_lane_xor16(s[g][j], a, b);
      s[g][j] = a + b;
      with_lane_xor32(s[g][j], a, b);
      s[g][j] = a + b;
    }
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

// k_mean[b,h,:] = (sum of the chunk sums, in a fixed order) / N, rounded to the input dtype: 1024 threads.
template <int DT, int D>
__device__ __forceinline__ void k_mean_finalize_body(const float* __restrict__ partial,
                                                     unsigned short* __restrict__ k_mean, int N, int n_chunks,
                                                     int64_t ms_b, int64_t ms_h, int H, int64_t bh) {
  constexpr int SL = 1024 / D;
  __shared__ float red[SL][D];
  const int ch = threadIdx.x % D, sl = threadIdx.x / D;
  const float* p = partial + bh * n_chunks * D;
  float s = 0.f;
  // (batches of independent loads: as a plain loop every load waited for the one before it)
  constexpr int FB = 8;
  int c = sl;
  for (; c + (FB - 1) * SL < n_chunks; c += FB * SL) {
    float x[FB];
#pragma unroll
    for (int u = 0; u < FB; u++) x[u] = p[(c + u * SL) * D + ch];
#pragma unroll
    for (int u = 0; u < FB; u++) s += x[u];
  }
  for (; c < n_chunks; c += SL) s += p[c * D + ch];
  red[sl][ch] = s;
  __syncthreads();
  if (sl == 0) {
    for (int i = 1; i < SL; i++) s += red[i][ch];
    const int b = (int)(bh / H), h = (int)(bh % H);
    k_mean[b * ms_b + h * ms_h + ch] = (unsigned short)(pack2_from_f32<DT>(s / (float)N, 0.f) & 0xffffu);
  }
}

}  // namespace paro
