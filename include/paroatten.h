/*
 * paroatten.h - C ABI of libparoatten_hip.so: the PAROAttention hot path for AMD MI355X (gfx950).
 *
 * Plain pointers and sizes only.  Every pointer argument is a DEVICE pointer unless it says
 * "host".  `stream` is a hipStream_t passed as void* (NULL = the null stream).  All strides
 * are in ELEMENTS of the tensor they belong to.  Functions are re-entrant, keep no state
 * between calls, never synchronise the device and never allocate; work buffers are passed in.
 * Return value: PARO_OK or a negative PARO_ERR_* code; paro_last_error() gives the message
 * of the last failure on the calling thread.
 *
 * Size limits, checked by every entry point they apply to (PARO_ERR_RUNTIME beyond them): batch and
 * head counts up to 65535 each (they are launch-grid dimensions; the permutation and preparation
 * entry points need batch * heads <= 65535); kernels that address one (batch, head) slice through a
 * 32-bit buffer descriptor (attention: K8 / V8; one-pass preparation: q, k, v, q8, k8) need that slice,
 * (N - 1) * token stride + D elements, below 2 GiB; the attention kernel keeps the list of kept key
 * blocks in the local data share, which bounds kv_len at about 1.4 million tokens.
 *
 * Each entry point names the interface of the reference (jamescsq47/PAROAtten) it stands in
 * for, as file:line relative to the reference tree.
 */
#ifndef PAROATTEN_H
#define PAROATTEN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PARO_OK 0
#define PARO_ERR_INVALID_VALUE (-1) /* bad layout / head_dim / flag: the reference throws std::invalid_argument (ValueError) */
#define PARO_ERR_RUNTIME (-2)       /* shape / dtype / contiguity check: the reference's TORCH_CHECK (RuntimeError)        */
#define PARO_ERR_UNSUPPORTED (-3)   /* a variant of the reference that this library does not implement                      */
#define PARO_ERR_HIP (-4)           /* a HIP runtime call failed                                                            */

#define PARO_DTYPE_F16 0
#define PARO_DTYPE_BF16 1

/* flags of the attention entry points */
#define PARO_ATTN_EXACT_EXP 1 /* P = e4m3(2^x) by hardware exponential + FP8 conversion instead of the fast
                                 direct construction of the e4m3 byte (see paro_attn_sparse_fwd) */
#define PARO_ATTN_PACED 2     /* launch form, results are bit-identical either way: a resident set of workgroups per
                                 XCD takes the q-blocks generation by generation, so that workgroups running
                                 together walk the key sequence together and share K8 / V8 tiles in the XCD's L2 */
#define PARO_ATTN_UNPACED 4   /* one workgroup per q-block, started as the hardware pleases.  With neither flag the
                                 library paces when one head's K8 + V8 exceed an XCD's 4 MB L2 (environment variable
                                 PARO_ATTN_PACING=0/1 overrides that default).  Scattered masks on long sequences gain
                                 (Wan 720p, uniformly random blocks: 26 -> 39 % of the MFMA peak, 4x fewer L2 fills);
                                 masks made of one contiguous run per row lose a few per cent.  A generation waits for
                                 all but a share of its workgroups (PARO_ATTN_PACE_SLACK; default half the L2's share
                                 of a head, at most a quarter of them) and at most PARO_ATTN_PACE_SPINS rounds. */
#define PARO_ATTN_TWO_WAVES 8 /* kernel form, results are bit-identical either way: two waves per 64-row q-block
                                 (32 q-rows each) also where the library would pick the one-wave-per-q-block
                                 kernel (head size 64, no lse, plain launch), which is the faster of the two there */
#define PARO_ATTN_PV_F16 16   /* accuracy mode: the P.V product in float16 with fp32 accumulation, as the reference's
                                 qk_int8_sv_f16_accum_f16_attn computes it (csrc/qattn/qk_int_sv_f16_cuda_sm80.cu:263-391),
                                 instead of FP8 e4m3 P and V.  True exponentials; V as given (no per-channel scale, no
                                 mean).  For paro_attn_sparse_fwd / _unpermute_fwd the `v8` argument then points at
                                 paro_v_f16_pack's tiles and v_scale / v_mean may be NULL; paro_qk_int8_sv_f16_attn
                                 packs them into its workspace itself (paro_attn_workspace_bytes_for).  Plain launch
                                 only; about half the speed of the default (the matrix pipe runs float16 at half the
                                 FP8 rate). */

#define PARO_ATTN_QK_PER_THREAD 32 /* q_scale / k_scale have the reference's per-thread granularity (qk_quant_gran 3,
                                 csrc/qattn/qk_int_sv_f16_cuda_sm80.cu:112-116, 129-133, shapes :1034-1038): q_scale
                                 [B,H,nbq*2*8], scale g of a 32-row group for its rows r with r % 8 == g; k_scale
                                 [B,Hkv,nbk*4] (16-byte aligned), scale j of a 64-key block for its keys c with
                                 (c % 8) / 2 == j.  Two-wave kernel; with
                                 neither PARO_ATTN_PV_F16 nor s_dump.  paro_quant_int8_per_thread makes such scales. */

/* Version of this ABI (bumped when a signature changes or an export leaves the library; currently 2). */
int paro_abi_version(void);
/* Message of the last error on this thread ("" if none). Host pointer, valid until the next call. */
const char* paro_last_error(void);
/* Architecture the device code was built for ("gfx950"). */
const char* paro_build_arch(void);

/* ---------------------------------------------------------------------------------------------
 * (1) Per-group symmetric INT8 quantisation of Q or K.
 * Stands in for QuantInt8Kernel and its four hosts: quant_per_block_int8_cuda (6- and 5-argument
 * overloads), quant_per_block_int8_fuse_sub_mean_cuda and quant_per_warp_int8_cuda
 * (csrc/fused/fused.cu:64-198, 429-510, 512-592, 594-682, 685-768; csrc/fused/fused.h:19-57).
 *
 * x [B,H,N,D] in 16-bit `dtype`, addressed by (stride_b, stride_h, stride_n), last dim contiguous.
 * For every group g of `group` consecutive tokens (g < n_groups, tokens >= N read as 0):
 *   v = float(x) - float(mean[b,h,:]) (if mean != NULL) ; v *= sm_scale (if has_sm_scale)
 *   amax = max(1e-7f, max|v|); scale[b,h,g] = amax / 127.f; out = sat_s8(rint(v * (127.f / amax)))
 * IEEE fp32 arithmetic, round-half-even.  D in {64,128}; group in {16,32,64,128}.
 * mean [B,H,D] in `dtype` (strides mean_stride_b/h); scale fp32 (strides scale_stride_b/h).
 * ------------------------------------------------------------------------------------------- */
int paro_quant_int8(const void* x, int dtype, const void* mean, int8_t* out, float* scale,
                    int B, int H, int N, int D,
                    int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_n,
                    int64_t mean_stride_b, int64_t mean_stride_h,
                    int64_t out_stride_b, int64_t out_stride_h, int64_t out_stride_n,
                    int64_t scale_stride_b, int64_t scale_stride_h,
                    int group, int n_groups, int has_sm_scale, float sm_scale, void* stream);

/* (1') The same arithmetic with the per-thread grouping of qk_quant_gran 3.  The reference declares that
 * granularity in its attention kernel (csrc/qattn/qk_int_sv_f16_cuda_sm80.cu:112-116, 129-133) and checks the
 * scale shapes (:1034-1038) but ships no quantiser for it (paroattention/core.py:204-205 calls the per-block
 * one, whose scales that check rejects); the grouping is the one the kernel's indexing implies.
 *   is_key == 0 (Q): eight scales per 32 tokens; group g of tokens 32 w + g + 8 j, j = 0..3;
 *                    scale [B,H, ceil(N/64)*2*8] at (w * 8 + g)
 *   is_key == 1 (K): four scales per 64 tokens; group j of tokens 64 w + 8 t + 2 j + e, t = 0..7, e = 0..1;
 *                    scale [B,H, ceil(N/64)*4] at (w * 4 + j)
 * Tokens >= N read as 0; groups that lie wholly past N get scale 1e-7 / 127.  scale contiguous. */
int paro_quant_int8_per_thread(const void* x, int dtype, const void* mean, int8_t* out, float* scale,
                               int B, int H, int N, int D,
                               int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_n,
                               int64_t mean_stride_b, int64_t mean_stride_h,
                               int64_t out_stride_b, int64_t out_stride_h, int64_t out_stride_n,
                               int is_key, void* stream);

/* ---------------------------------------------------------------------------------------------
 * (2a) V -> FP8 (e4m3fn) with per-(b,h,channel) mean smoothing and scale, written in the
 * MFMA-fragment tile order the attention kernel reads.
 * Stands in for transpose_pad_permute_cuda + mean_scale_fuse_quant_cuda / scale_fuse_quant_cuda
 * (csrc/fused/fused.cu:262-313, 316-427, 850-1083; paroattention/quant.py:224-293).  The
 * reference's within-16 token shuffle is an NVIDIA mma fragment order; this library uses its own.
 *
 * v [B,Hkv,N,D] 16-bit.  v_mean, v_scale: fp32 [B,Hkv,D] (contiguous).  v8: paro_v_fp8_bytes().
 *   mean = sum_n v / N (0 if !smooth) ; scale = max|v - mean| / 448 ; v8 = e4m3_rne((v-mean)/scale)
 *   v_mean = mean + sum_n (v - mean - scale * v8) / N   (if smooth)
 * i.e. v_mean is the offset the attention epilogue adds back: the channel mean plus the mean rounding
 * residual of the channel's codes (a few 1e-4 of max|v|; rounding 16-bit inputs to e4m3 is not unbiased,
 * and a per-channel bias does not average out over the keys of a row the way rounding noise does).
 * Tile order: v8[((b*Hkv+h)*nb + kb)*64*D + ((dt*2 + mt)*64 + lane)*16 + r] holds token
 * kb*64 + 32*mt + 8*(r/4) + 4*(lane/32) + r%4, channel 32*dt + lane%32 (tokens >= N are 0).
 * partial: fp32 work buffer of paro_v_fp8_partial_floats() floats.
 * ------------------------------------------------------------------------------------------- */
int64_t paro_v_fp8_bytes(int B, int Hkv, int N, int D);
int64_t paro_v_fp8_partial_floats(int B, int Hkv, int N, int D);
int paro_v_fp8_pack(const void* v, int dtype, uint8_t* v8, float* v_scale, float* v_mean, float* partial,
                    int B, int Hkv, int N, int D,
                    int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_n,
                    int smooth, void* stream);

/* ---------------------------------------------------------------------------------------------
 * (2a') V -> float16 tiles for the attention's accuracy mode (PARO_ATTN_PV_F16).  Stands in for the
 * float16 V operand the reference's kernel reads as it is (value.to(float16) in its callers,
 * paroattention/core.py:150-160): values unchanged (bfloat16 inputs converted to float16, round to nearest
 * even), no scale, no mean; only the order differs.
 * v [B,Hkv,N,D] 16-bit.  v16: paro_v_f16_bytes() bytes.  Tile order: halfword
 * v16[((b*Hkv+h)*nb + kb)*64*D + ((dt*4 + s)*64 + lane)*8 + e] holds token
 * kb*64 + 32*(s/2) + 16*(s%2) + 8*(e/4) + 4*(lane/32) + e%4, channel 32*dt + lane%32 (tokens >= N are 0).
 * ------------------------------------------------------------------------------------------- */
int64_t paro_v_f16_bytes(int B, int Hkv, int N, int D);
int paro_v_f16_pack(const void* v, int dtype, void* v16, int B, int Hkv, int N, int D,
                    int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_n, void* stream);

/* ---------------------------------------------------------------------------------------------
 * (2b) Block-sparse attention: INT8 Q.K^T on i8 MFMA (exact int32), online base-2 softmax,
 * FP8 P.V on fp8 MFMA with fp32 accumulation, k-blocks skipped per (head, 64-row q-block).
 * Stands in for qk_int_sv_f16_attn_kernel and the body of its host qk_int8_sv_f16_accum_f16_attn
 * (csrc/qattn/qk_int_sv_f16_cuda_sm80.cu:44-726, 905-1080), instantiated as the reference does:
 * 64-row q-blocks, 64-row k-blocks, q scales per 32 rows (:1022-1048).
 *
 * q8 [B,H,Nq,D], k8 [B,Hkv,Nk,D] int8 with element strides; q_scale fp32 [B,H,ceil(Nq/64)*2];
 * k_scale fp32 [B,Hkv,ceil(Nk/64)]; v8/v_scale/v_mean from paro_v_fp8_pack (v_mean may be NULL).
 * sparse: bool bytes [B,H,nbq,nbk] contiguous, nonzero = compute; if sparse_batch_stride == 0 the
 * same [H,nbq,nbk] mask serves every batch entry.  A kept block joins the softmax support, a
 * skipped one is as if masked with -inf; a row with no kept block outputs 0 (lse = -inf).
 * out [B,H,Nq,D] in `out_dtype`; lse (may be NULL) fp32 [B,H,Nq], base 2: log2 sum_j 2^(s_ij*log2e).
 * s_dump (may be NULL): int32 [B,H,nbq*64,nbk*64]; the raw Q.K^T accumulators of every computed
 * block are stored there (debug / parity of the integer stage; untouched where skipped).
 * D in {64,128}; is_causal in {0,1} (needs Nq == Nk).
 * flags: 0, or a combination of PARO_ATTN_EXACT_EXP and one of PARO_ATTN_PACED / PARO_ATTN_UNPACED.  The paced
 * launch keeps eight counters in a work buffer of the library (per GPU; cleared by a small launch in front of
 * the kernel); two paced launches that overlap on one GPU disturb each other's pacing, never their results,
 * and a workgroup never waits more than a bounded number of rounds.  By default the softmax weight 2^x is turned into its e4m3 byte
 * directly (exponent field from floor(x), mantissa by linear interpolation between powers of two,
 * round-to-nearest-even): at most 6 % from the exact weight, which the row normalisation (done with the
 * same rounded weights) absorbs; measured output error stays inside atol 2e-2 / cosine 0.999.  With
 * PARO_ATTN_EXACT_EXP, or whenever lse or s_dump is requested, 2^x is evaluated in fp32 and rounded.
 * ------------------------------------------------------------------------------------------- */
int paro_attn_sparse_fwd(const int8_t* q8, const int8_t* k8, const uint8_t* v8,
                         const float* q_scale, const float* k_scale,
                         const float* v_scale, const float* v_mean,
                         const uint8_t* sparse, int64_t sparse_batch_stride,
                         void* out, int out_dtype, float* lse, int32_t* s_dump,
                         int B, int H, int Hkv, int Nq, int Nk, int D,
                         int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_n,
                         int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_n,
                         int64_t o_stride_b, int64_t o_stride_h, int64_t o_stride_n,
                         float sm_scale, int is_causal, int flags, void* stream);

/* (2b') The same kernel with the inverse token permutation folded into its stores: q-row r of head
 * `head` is written at token n_text + old(r - n_text), old() = the inverse of the index law of (3)
 * below for order orders[head] (rows below n_text stay in place).  Stands in for the attention call
 * followed by permute_attn_out (paroattention/cogvideox.py:216-227; wan.py:276,300): with
 * out strides of a [B,N,H,D] buffer the result is token-major, ready for the output projection.
 * Requires Nq == n_text + F*Hh*W.  orders: int32 [H] on the device.  lse, if given, stays in the
 * order of the q-rows (the permuted order): only `out` is stored through the inverse permutation. */
int paro_attn_sparse_unpermute_fwd(const int8_t* q8, const int8_t* k8, const uint8_t* v8,
                                   const float* q_scale, const float* k_scale,
                                   const float* v_scale, const float* v_mean,
                                   const uint8_t* sparse, int64_t sparse_batch_stride,
                                   void* out, int out_dtype, float* lse,
                                   int B, int H, int Hkv, int Nq, int Nk, int D,
                                   int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_n,
                                   int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_n,
                                   int64_t o_stride_b, int64_t o_stride_h, int64_t o_stride_n,
                                   float sm_scale, int is_causal, int flags,
                                   const int32_t* orders, int n_text, int F, int Hh, int W,
                                   void* stream);

/* ---------------------------------------------------------------------------------------------
 * (2c) The reference's extension entry point in one call: V (fp16/bf16) -> FP8 tiles, then (2b).
 * Stands in for qk_int8_sv_f16_accum_f16_attn as bound at csrc/qattn/pybind_sm80.cpp:23 /
 * csrc/qattn/attn_cuda_sm80.h:19-31: same tensors, same integer flags (tensor_layout 0 = NHD,
 * 1 = HND; qk_quant_gran 2 = per_warp, 3 = per_thread: PARO_ATTN_QK_PER_THREAD is set), same checks.
 * workspace: paro_attn_workspace_bytes() bytes of device memory (256-byte aligned).
 * ------------------------------------------------------------------------------------------- */
int64_t paro_attn_workspace_bytes(int B, int Hkv, int Nk, int D);
/* The same for a call with the given flags (PARO_ATTN_PV_F16 needs float16 tiles of V instead). */
int64_t paro_attn_workspace_bytes_for(int B, int Hkv, int Nk, int D, int flags);
int paro_qk_int8_sv_f16_attn(const int8_t* q8, const int8_t* k8, const void* v, int v_dtype,
                             void* out, int out_dtype,
                             const float* q_scale, const float* k_scale,
                             const uint8_t* sparse, int64_t sparse_batch_stride,
                             float* lse, void* workspace, int64_t workspace_bytes,
                             int B, int H, int Hkv, int Nq, int Nk, int D,
                             int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_n,
                             int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_n,
                             int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_n,
                             int64_t o_stride_b, int64_t o_stride_h, int64_t o_stride_n,
                             int tensor_layout, int is_causal, int qk_quant_gran,
                             float sm_scale, int smooth_v, int flags, void* stream);

/* ---------------------------------------------------------------------------------------------
 * (3) Fused 3-D RoPE + per-head F/H/W token permutation, and the inverse permutation.
 * Stands in for the Python head loops permute_qk / permute_attn_out
 * (paroattention/cogvideox.py:22-62, 64-110; paroattention/wan.py:25-63, 65-111), the RoPE that
 * precedes them (cogvideox.py:167-172; wan.py:161-167) and the prototype rope_permutation
 * (csrc/rope/rope.cu:14-48, csrc/rope/rope.cuh:9-96).
 *
 * Tokens [0,n_text) are text: copied through.  Image token t = (f*Hh + h)*W + w of head `head`
 * moves to n_text + (c[p0]*S[p1] + c[p1])*S[p2] + c[p2], p = the order `orders[head]` in 0..5
 * (0 FHW, 1 FWH, 2 HWF, 3 HFW, 4 WHF, 5 WFH; any other value is treated as 0), S = (F,Hh,W), c = (f,h,w).
 * paro_rope_permute_fwd: for each of q, k (rotated if cos != NULL) and v (never rotated; any of
 * the three may be NULL): out[b,head,new] = rot(in[b,head,old]).  Rotation of channel pairs:
 *   o[2i] = x[2i]*cos[t,2i] - x[2i+1]*sin[t,2i] ; o[2i+1] = x[2i+1]*cos[t,2i+1] + x[2i]*sin[t,2i+1]
 * each product and the sum rounded to fp32 (no fused multiply-add), then to `dtype`.
 * cos, sin: fp32 [F*Hh*W, D].  orders: int32 [H] on the device.  in/out [B,H,N,D] 16-bit, must
 * not overlap.  paro_permute_inv: out[b,head,old] = in[b,head,new] (text copied through).
 * ------------------------------------------------------------------------------------------- */
int paro_rope_permute_fwd(const void* q_in, const void* k_in, const void* v_in,
                          void* q_out, void* k_out, void* v_out, int dtype,
                          const float* cos, const float* sin, const int32_t* orders,
                          int B, int H, int N, int D, int n_text, int F, int Hh, int W,
                          int64_t in_stride_b, int64_t in_stride_h, int64_t in_stride_n,
                          int64_t out_stride_b, int64_t out_stride_h, int64_t out_stride_n,
                          void* stream);
int paro_permute_inv(const void* in, void* out, int dtype, const int32_t* orders,
                     int B, int H, int N, int D, int n_text, int F, int Hh, int W,
                     int64_t in_stride_b, int64_t in_stride_h, int64_t in_stride_n,
                     int64_t out_stride_b, int64_t out_stride_h, int64_t out_stride_n,
                     void* stream);
/* new_of_old index map of every head: idx int32 [H, F*Hh*W] (parity of the integer index law). */
int paro_permute_index_map(int32_t* idx, const int32_t* orders, int H, int F, int Hh, int W, void* stream);

/* ---------------------------------------------------------------------------------------------
 * (3b) The whole preparation of the attention operands in one pass: RoPE + permutation + INT8
 * quantisation of Q and K + FP8 packing of the permuted V.  Same results as the chain
 * paro_rope_permute_fwd -> paro_quant_int8 (Q: groups of 32 tokens, K: groups of 64, optional
 * mean) -> paro_v_fp8_pack (INT8 tensors and scales bit-identical; V's mean is summed in source
 * order, so it may differ in the last fp32 bit), i.e. as what the processors do between the projections and the
 * attention call (paroattention/cogvideox.py:167-186 with quant.py:105-180 and, for V,
 * quant.py:224-293), without writing the permuted 16-bit tensors.
 * q, k, v: [B,H,N,D], each through its own three strides.  k_mean: NULL
 * or [B,H,D] in the input dtype through mean strides (subtracted from the rotated K before
 * quantisation).  Outputs, all contiguous: q8, k8 int8 [B,H,N,D]; q_scale f32 [B,H,2*ceil(N/64)];
 * k_scale f32 [B,H,ceil(N/64)]; v8 paro_v_fp8_bytes(); v_scale, v_mean f32 [B,H,D].
 * workspace: paro_prep_workspace_bytes() bytes.
 * paro_rope_k_mean: k_mean[b,h,:] = mean over tokens of the ROTATED K, rounded to the input dtype
 * (what `km = k.mean(dim=seq)` gives the reference's quantiser after the processor's RoPE).
 * ------------------------------------------------------------------------------------------- */
int64_t paro_prep_workspace_bytes(int B, int H, int N, int D);
int paro_rope_permute_quant_fwd(const void* q, const void* k, const void* v, int dtype,
                                const float* cos, const float* sin, const int32_t* orders,
                                const void* k_mean,
                                int8_t* q8, float* q_scale, int8_t* k8, float* k_scale,
                                uint8_t* v8, float* v_scale, float* v_mean,
                                void* workspace, int64_t workspace_bytes,
                                int B, int H, int N, int D, int n_text, int F, int Hh, int W,
                                int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_n,
                                int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_n,
                                int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_n,
                                int64_t mean_stride_b, int64_t mean_stride_h,
                                int smooth_v, void* stream);
int paro_rope_k_mean(const void* k, int dtype, const float* cos, const float* sin, void* k_mean,
                     void* workspace, int64_t workspace_bytes,
                     int B, int H, int N, int D, int n_text, int F, int Hh, int W,
                     int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_n,
                     int64_t mean_stride_b, int64_t mean_stride_h, void* stream);
/* paro_rope_k_mean followed by paro_rope_permute_quant_fwd with that mean, as one call: what a caller that
 * smooths K does per layer (the reference's quantiser takes `km = k.mean(dim=seq)`, paroattention/quant.py:105-180,
 * 174-176).  k_mean is an OUTPUT here ([B,H,D] in the input dtype through the mean strides), filled before it
 * is used; the results are bit-identical to the two calls.  The K sums and the V statistics, both plain
 * streaming passes, share one launch and their second steps another (four launches instead of six).
 * workspace: paro_prep_smooth_workspace_bytes() bytes (the K and V partial results are alive together). */
int64_t paro_prep_smooth_workspace_bytes(int B, int H, int N, int D);
int paro_rope_k_mean_permute_quant_fwd(const void* q, const void* k, const void* v, int dtype,
                                       const float* cos, const float* sin, const int32_t* orders,
                                       void* k_mean,
                                       int8_t* q8, float* q_scale, int8_t* k8, float* k_scale,
                                       uint8_t* v8, float* v_scale, float* v_mean,
                                       void* workspace, int64_t workspace_bytes,
                                       int B, int H, int N, int D, int n_text, int F, int Hh, int W,
                                       int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_n,
                                       int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_n,
                                       int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_n,
                                       int64_t mean_stride_b, int64_t mean_stride_h,
                                       int smooth_v, void* stream);

/* paro_rope_k_mean for callers that can neither allocate device memory nor bring a workspace (code under
 * HIP graph capture, serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  Same arguments and results as paro_rope_k_mean without the workspace: the per-chunk partial
 * sums go to a work buffer built into the library (a __device__ array of
 * PARO_ROPE_K_MEAN_STATIC_MAX_FLOATS floats = 8 MiB that every GPU the library runs on holds until the
 * process ends).  The call allocates and frees nothing.  B * H * ceil(N/256) * D must not exceed
 * PARO_ROPE_K_MEAN_STATIC_MAX_FLOATS (PARO_ERR_RUNTIME otherwise; CogVideoX-5b needs 0.43 M, Wan 720p
 * 1.5 M).  All calls on one GPU share that GPU's buffer: calls that may overlap on one GPU (different
 * streams, different threads) race; calls on one stream do not.  The first call on each device looks the
 * buffer's address up (hipGetSymbolAddress) and should therefore be made outside stream capture. */
#define PARO_ROPE_K_MEAN_STATIC_MAX_FLOATS (2 * 1024 * 1024)
int paro_rope_k_mean_static(const void* k, int dtype, const float* cos, const float* sin, void* k_mean,
                            int B, int H, int N, int D, int n_text, int F, int Hh, int W,
                            int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_n,
                            int64_t mean_stride_b, int64_t mean_stride_h, void* stream);

/* ---------------------------------------------------------------------------------------------
 * V helpers kept for API completeness of paroattention._fused (csrc/fused/fused.cu:200-260,
 * 770-848): out_f16[b,h,n,:] = fp16(v - mean[b,h,:]) (bf16 input: subtract in bf16 first).
 * ------------------------------------------------------------------------------------------- */
int paro_sub_mean(const void* v, int dtype, const void* mean, void* out_f16,
                  int B, int H, int N, int D,
                  int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_n,
                  int64_t mean_stride_b, int64_t mean_stride_h,
                  int64_t out_stride_b, int64_t out_stride_h, int64_t out_stride_n, void* stream);

/* ---------------------------------------------------------------------------------------------
 * V preparation in the reference's own storage format, for callers of paroattention._fused.
 * paro_transpose_pad_permute stands in for transpose_pad_permute_cuda (csrc/fused/fused.cu:262-313,
 * 850-923): in [B,H,N,D] 16-bit through (stride_b, stride_h, stride_n) -> out [B,H,D,ceil64(N)] through
 * (stride_b, stride_h, stride_d), last dim contiguous; tokens >= N are zero; inside every group of 16
 * tokens, position i holds token [0,1,8,9,2,3,10,11,4,5,12,13,6,7,14,15][i] (the operand order of NVIDIA's
 * fp8 mma, paroattention/quant.py:231-234; this library's attention kernel reads paro_v_fp8_pack's tiles
 * instead).  D in {64,128}.
 * paro_channel_quant_fp8 stands in for scale_fuse_quant_cuda (mean == NULL) and mean_scale_fuse_quant_cuda
 * (fused.cu:316-427, 925-1083): per row in[b,h,d,:] of row_len entries,
 *   n16 = ceil16(num_tokens); mean = sum(in[:n16]) / n16 (0 without `mean`)
 *   amax = max(|max(in[:n16]) - mean|, |min(in[:n16]) - mean|) ; scale = amax / scale_max
 *   out[:ceil64(num_tokens)] = e4m3_rne_satfinite((in - mean) * (scale_max / amax))
 * as the reference does it (the zero padding up to n16 takes part in the statistics).  A constant row
 * gives zero codes (the reference divides by zero there).  mean, scale: fp32 [B,H,D] through (stride_b,
 * stride_h).
 * ------------------------------------------------------------------------------------------- */
int paro_transpose_pad_permute(const void* in, void* out, int dtype, int B, int H, int N, int D,
                               int64_t in_stride_b, int64_t in_stride_h, int64_t in_stride_n,
                               int64_t out_stride_b, int64_t out_stride_h, int64_t out_stride_d, void* stream);
int paro_channel_quant_fp8(const void* in, int dtype, uint8_t* out, float* mean, float* scale,
                           int B, int H, int D, int num_tokens, int row_len, float scale_max,
                           int64_t in_stride_b, int64_t in_stride_h, int64_t in_stride_d,
                           int64_t out_stride_b, int64_t out_stride_h, int64_t out_stride_d,
                           int64_t mean_stride_b, int64_t mean_stride_h,
                           int64_t scale_stride_b, int64_t scale_stride_h, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Block-mask bit packing.  The sparse plan is the one operand of the path that is staged from the
 * host per layer (paroattention/prefetch_utils.py:34-59 keeps it as torch.bool on the CPU and
 * paroattention/cogvideox.py:188-213 copies one [H,nb,nb] slice per call); as bits it is 8x smaller
 * in pinned memory and on the wire.  Bit i of byte j = element 8j+i (numpy.packbits, bitorder
 * "little").  mask: n bytes of 0/1 (nonzero counts as 1 when packing); bits: paro_mask_bits_bytes(n)
 * bytes.  Both pointers 16-byte aligned, on the device.
 * ------------------------------------------------------------------------------------------- */
int64_t paro_mask_bits_bytes(int64_t n);
int paro_mask_pack(const uint8_t* mask, uint8_t* bits, int64_t n, void* stream);
int paro_mask_unpack(const uint8_t* bits, uint8_t* mask, int64_t n, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PAROATTEN_H */
