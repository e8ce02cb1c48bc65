// Fused 3-D RoPE + per-head F/H/W token permutation, and the inverse permutation (HBM-bound).
//
// A thread owns one 16-byte piece (8 channels) of one SOURCE token and keeps that token's cos/sin
// fragment in registers while it walks over a group of (batch, head) pairs and the q, k, v tensors:
// the rotary tables are read once per head group instead of once per head, reads are sequential
// 16-byte pieces, and every store is a full token row (D 16-bit values = 128 or 256 bytes, written
// by D/8 adjacent lanes) at its permuted position.  The inverse walks destination tokens in order
// and gathers rows, so it, too, issues whole rows on both sides.
//
// Index law (permute_qk of the reference, paroattention/cogvideox.py:22-62): image token
// (f,h,w) of a head with order p goes to (c[p0]*S[p1] + c[p1])*S[p2] + c[p2].
// Rotation (diffusers apply_rotary_emb as called at paroattention/cogvideox.py:167-172): fp32
// products and sum, each rounded (this file is built with fp contraction off).
#include "paro_device.hpp"

namespace paro {

template <int DT, int D, bool INVERSE>
__global__ void __launch_bounds__(256) rope_permute_kernel(
    const unsigned short* __restrict__ q_in, const unsigned short* __restrict__ k_in,
    const unsigned short* __restrict__ v_in, unsigned short* __restrict__ q_out,
    unsigned short* __restrict__ k_out, unsigned short* __restrict__ v_out,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, const int* __restrict__ orders,
    int BH, int H, int N, int n_text, int F, int Hh, int W, int heads_per_wg,
    int64_t is_b, int64_t is_h, int64_t is_n, int64_t os_b, int64_t os_h, int64_t os_n) {
  constexpr int LPR = D / 8;
  constexpr int ROWS = 256 / LPR;
  const int t = threadIdx.x;
  const int tok = blockIdx.x * ROWS + t / LPR;
  if (tok >= N) return;
  const int col = (t % LPR) * 8;
  const bool img = tok >= n_text;
  int f = 0, hh = 0, w = 0;
  float cs[8], sn[8];
  const bool rope = img && cos_t != nullptr;
  if (img) {
    const int ti = tok - n_text;
    f = ti / (Hh * W);
    const int rem = ti - f * (Hh * W);
    hh = rem / W;
    w = rem - hh * W;
    if (rope) {
      const v4f c0 = *reinterpret_cast<const v4f*>(cos_t + (int64_t)ti * D + col);
      const v4f c1 = *reinterpret_cast<const v4f*>(cos_t + (int64_t)ti * D + col + 4);
      const v4f s0 = *reinterpret_cast<const v4f*>(sin_t + (int64_t)ti * D + col);
      const v4f s1 = *reinterpret_cast<const v4f*>(sin_t + (int64_t)ti * D + col + 4);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        cs[j] = c0[j]; cs[4 + j] = c1[j];
        sn[j] = s0[j]; sn[4 + j] = s1[j];
      }
    }
  }
  const int bh0 = blockIdx.y * heads_per_wg;
  const int bh1 = min(BH, bh0 + heads_per_wg);
  for (int bh = bh0; bh < bh1; bh++) {
    const int b = bh / H, head = bh - b * H;
    int mapped = tok;
    if (img) {
      int sf, sh, sw;
      order_strides(orders[head], F, Hh, W, sf, sh, sw);
      mapped = n_text + f * sf + hh * sh + w * sw;
    }
    const int src = INVERSE ? mapped : tok;
    const int dst = INVERSE ? tok : mapped;
    const int64_t io = b * is_b + head * is_h + (int64_t)src * is_n + col;
    const int64_t oo = b * os_b + head * os_h + (int64_t)dst * os_n + col;
    // streamed once in, once out: non-temporal on both sides keeps the rotary tables in the L2
    v4i rq, rk, rv;
    if (q_in) rq = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(q_in + io));
    if (k_in) rk = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(k_in + io));
    if (v_in) rv = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(v_in + io));
    if (rope) {
      if (q_in) rq = rotate8<DT>(rq, cs, sn);
      if (k_in) rk = rotate8<DT>(rk, cs, sn);
    }
    if (q_in) __builtin_nontemporal_store(rq, reinterpret_cast<v4i*>(q_out + oo));
    if (k_in) __builtin_nontemporal_store(rk, reinterpret_cast<v4i*>(k_out + oo));
    if (v_in) __builtin_nontemporal_store(rv, reinterpret_cast<v4i*>(v_out + oo));
  }
}

__global__ void permute_index_kernel(int* __restrict__ idx, const int* __restrict__ orders, int F, int Hh, int W) {
  const int n = F * Hh * W;
  const int head = blockIdx.y;
  const int old = blockIdx.x * blockDim.x + threadIdx.x;
  if (old >= n) return;
  const int f = old / (Hh * W), rem = old - f * (Hh * W), hh = rem / W, w = rem - hh * W;
  int sf, sh, sw;
  order_strides(orders[head], F, Hh, W, sf, sh, sw);
  idx[(int64_t)head * n + old] = f * sf + hh * sh + w * sw;
}

static int check_common(const char* fn, int dtype, int B, int H, int N, int D, int n_text, int F, int Hh, int W,
                        int64_t is_b, int64_t is_h, int64_t is_n, int64_t os_b, int64_t os_h, int64_t os_n) {
  PARO_CHECK(B > 0 && H > 0 && N > 0, PARO_ERR_RUNTIME, "%s: empty shape", fn);
  PARO_CHECK((int64_t)B * H <= MAX_GRID_YZ, PARO_ERR_RUNTIME, "%s: batch * heads = %lld exceeds %d", fn,
             (long long)B * H, MAX_GRID_YZ);
  PARO_CHECK(D == 64 || D == 128, PARO_ERR_INVALID_VALUE, "Unsupported head dim: %d", D);
  PARO_CHECK(dtype == PARO_DTYPE_F16 || dtype == PARO_DTYPE_BF16, PARO_ERR_RUNTIME,
             "Unsupported input dtype (expect float16 or bfloat16)");
  PARO_CHECK(n_text >= 0 && F > 0 && Hh > 0 && W > 0 && (int64_t)n_text + (int64_t)F * Hh * W == N,
             PARO_ERR_RUNTIME, "%s: n_text + F*H*W = %d + %d*%d*%d does not equal the token count %d", fn, n_text, F,
             Hh, W, N);
  PARO_CHECK(is_b % 8 == 0 && is_h % 8 == 0 && is_n % 8 == 0 && os_b % 8 == 0 && os_h % 8 == 0 && os_n % 8 == 0,
             PARO_ERR_RUNTIME, "%s: strides must be multiples of 8 elements", fn);
  return PARO_OK;
}

template <bool INVERSE>
static int launch_rp(const void* q_in, const void* k_in, const void* v_in, void* q_out, void* k_out, void* v_out,
                     int dtype, const float* cos_t, const float* sin_t, const int32_t* orders, int B, int H, int N,
                     int D, int n_text, int F, int Hh, int W, int64_t is_b, int64_t is_h, int64_t is_n,
                     int64_t os_b, int64_t os_h, int64_t os_n, hipStream_t st) {
  const int rows = 256 / (D / 8);
  const int BH = B * H;
  // (batch, head) pairs per workgroup: enough to amortise the rotary fragment (a table row is 8*D
  // bytes per token, twice a token row), few enough that the launch has many short workgroups.
  // Measured: D = 64 is fastest at 2..4 pairs (5.6-5.75 TB/s against 5.25 at 16), D = 128 at 16
  // (5.5 against 5.4 at 4).  Without tables there is nothing to amortise: one pair per workgroup.
  int hpw = cos_t ? (D == 64 ? 4 : 16) : 1;
  while (hpw > 1 && (int64_t)ceil_div(N, rows) * ceil_div(BH, hpw) < 3072) hpw >>= 1;
  dim3 grid(ceil_div(N, rows), ceil_div(BH, hpw)), block(256);
#define PARO_RP(DTV, DV)                                                                                          \
  hipLaunchKernelGGL((rope_permute_kernel<DTV, DV, INVERSE>), grid, block, 0, st, (const unsigned short*)q_in,    \
                     (const unsigned short*)k_in, (const unsigned short*)v_in, (unsigned short*)q_out,            \
                     (unsigned short*)k_out, (unsigned short*)v_out, cos_t, sin_t, (const int*)orders, BH, H, N,  \
                     n_text, F, Hh, W, hpw, is_b, is_h, is_n, os_b, os_h, os_n)
  if (dtype == PARO_DTYPE_F16) {
    if (D == 64) PARO_RP(PARO_DTYPE_F16, 64); else PARO_RP(PARO_DTYPE_F16, 128);
  } else {
    if (D == 64) PARO_RP(PARO_DTYPE_BF16, 64); else PARO_RP(PARO_DTYPE_BF16, 128);
  }
#undef PARO_RP
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}

}  // namespace paro

extern "C" int paro_rope_permute_fwd(const void* q_in, const void* k_in, const void* v_in, void* q_out,
                                     void* k_out, void* v_out, int dtype, const float* cos, const float* sin,
                                     const int32_t* orders, int B, int H, int N, int D, int n_text, int F, int Hh,
                                     int W, int64_t in_stride_b, int64_t in_stride_h, int64_t in_stride_n,
                                     int64_t out_stride_b, int64_t out_stride_h, int64_t out_stride_n,
                                     void* stream) {
  using namespace paro;
  int rc = check_common("paro_rope_permute_fwd", dtype, B, H, N, D, n_text, F, Hh, W, in_stride_b, in_stride_h,
                        in_stride_n, out_stride_b, out_stride_h, out_stride_n);
  if (rc) return rc;
  PARO_CHECK(orders, PARO_ERR_RUNTIME, "paro_rope_permute_fwd: null orders");
  PARO_CHECK(q_in || k_in || v_in, PARO_ERR_RUNTIME, "paro_rope_permute_fwd: no input tensor");
  PARO_CHECK((!q_in || q_out) && (!k_in || k_out) && (!v_in || v_out), PARO_ERR_RUNTIME,
             "paro_rope_permute_fwd: an input tensor has no output tensor");
  PARO_CHECK((cos == nullptr) == (sin == nullptr), PARO_ERR_RUNTIME,
             "paro_rope_permute_fwd: cos and sin must be given together");
  const void* ptrs[6] = {q_in, k_in, v_in, q_out, k_out, v_out};
  for (int i = 0; i < 6; i++)
    PARO_CHECK(((uintptr_t)ptrs[i] % 16) == 0, PARO_ERR_RUNTIME, "paro_rope_permute_fwd: tensors must be 16-byte aligned");
  PARO_CHECK(((uintptr_t)cos % 16) == 0 && ((uintptr_t)sin % 16) == 0, PARO_ERR_RUNTIME,
             "paro_rope_permute_fwd: cos/sin must be 16-byte aligned");
  return launch_rp<false>(q_in, k_in, v_in, q_out, k_out, v_out, dtype, cos, sin, orders, B, H, N, D, n_text, F, Hh,
                          W, in_stride_b, in_stride_h, in_stride_n, out_stride_b, out_stride_h, out_stride_n,
                          (hipStream_t)stream);
}

extern "C" int paro_permute_inv(const void* in, void* out, int dtype, const int32_t* orders, int B, int H, int N,
                                int D, int n_text, int F, int Hh, int W, int64_t in_stride_b, int64_t in_stride_h,
                                int64_t in_stride_n, int64_t out_stride_b, int64_t out_stride_h,
                                int64_t out_stride_n, void* stream) {
  using namespace paro;
  int rc = check_common("paro_permute_inv", dtype, B, H, N, D, n_text, F, Hh, W, in_stride_b, in_stride_h,
                        in_stride_n, out_stride_b, out_stride_h, out_stride_n);
  if (rc) return rc;
  PARO_CHECK(in && out && orders, PARO_ERR_RUNTIME, "paro_permute_inv: null pointer");
  PARO_CHECK(((uintptr_t)in % 16) == 0 && ((uintptr_t)out % 16) == 0, PARO_ERR_RUNTIME,
             "paro_permute_inv: tensors must be 16-byte aligned");
  return launch_rp<true>(nullptr, nullptr, in, nullptr, nullptr, out, dtype, nullptr, nullptr, orders, B, H, N, D,
                         n_text, F, Hh, W, in_stride_b, in_stride_h, in_stride_n, out_stride_b, out_stride_h,
                         out_stride_n, (hipStream_t)stream);
}

extern "C" int paro_permute_index_map(int32_t* idx, const int32_t* orders, int H, int F, int Hh, int W,
                                      void* stream) {
  using namespace paro;
  PARO_CHECK(idx && orders, PARO_ERR_RUNTIME, "paro_permute_index_map: null pointer");
  PARO_CHECK(H > 0 && F > 0 && Hh > 0 && W > 0, PARO_ERR_RUNTIME, "paro_permute_index_map: empty shape");
  PARO_CHECK(H <= MAX_GRID_YZ && (int64_t)F * Hh * W < (int64_t)1 << 31, PARO_ERR_RUNTIME,
             "paro_permute_index_map: head count or grid too large");
  const int n = F * Hh * W;
  hipLaunchKernelGGL(permute_index_kernel, dim3(ceil_div(n, 256), H), dim3(256), 0, (hipStream_t)stream, idx,
                     (const int*)orders, F, Hh, W);
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}
