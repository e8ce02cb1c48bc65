// PyTorch-ROCm C++ extension over the C ABI of libparoatten_hip.so (include/paroatten.h).
//
// Host code only: no kernels here.  It registers, under one extension module, three submodules with the
// names, positional signatures, preallocated-output conventions and error behaviour of the reference's
// three CUDA extensions:
//   _qattn_sm80  csrc/qattn/pybind_sm80.cpp:21-27, csrc/qattn/attn_cuda_sm80.h:19-69
//   _fused       csrc/fused/pybind.cpp:21-33,      csrc/fused/fused.h:19-76
//   _rope        csrc/rope/pybind.cpp:5-8,         csrc/rope/rope.h:6
// Checks fail as the reference's do: TORCH_CHECK -> RuntimeError with the texts of csrc/utils.cuh:20-38,
// std::invalid_argument -> ValueError for unsupported layouts, head dims and flags
// (csrc/dispatch_utils.h:23-112).  Unlike the reference's launches (legacy default stream, no device
// guard: paroattention/core.py:168-174 works around it) every call runs under a guard for the tensors'
// device and on torch's current stream of that device.
#include <torch/extension.h>
#include <atomic>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include <stdexcept>
#include <string>

#include "../../include/paroatten.h"

namespace {

void check_rc(int rc) {
  if (rc == PARO_OK) return;
  const std::string msg = paro_last_error();
  if (rc == PARO_ERR_INVALID_VALUE) throw std::invalid_argument(msg);
  if (rc == PARO_ERR_UNSUPPORTED) {
    PyErr_SetString(PyExc_NotImplementedError, msg.c_str());
    throw py::error_already_set();
  }
  TORCH_CHECK(false, msg);
}

void on_gpu(const torch::Tensor& x, const char* name) { TORCH_CHECK(x.is_cuda(), "Tensor ", name, " must be on CUDA"); }
void contiguous(const torch::Tensor& x, const char* name) { TORCH_CHECK(x.is_contiguous(), "Tensor ", name, " must be contiguous"); }
void lastdim_contiguous(const torch::Tensor& x, const char* name) {
  TORCH_CHECK(x.stride(-1) == 1, "Tensor ", name, " must be contiguous at the last dimension");
}
void dims(const torch::Tensor& x, const char* name, int64_t n) {
  TORCH_CHECK(x.dim() == n, "Tensor ", name, " must have dimension number (", n, ")");
}
void dtype(const torch::Tensor& x, const char* name, at::ScalarType t, const char* tname) {
  TORCH_CHECK(x.scalar_type() == t, "Tensor ", name, " must have dtype (", tname, ")");
}
void shape(const torch::Tensor& x, const char* name, at::IntArrayRef want, const char* text) {
  TORCH_CHECK(x.sizes() == want, "Tensor ", name, " must have shape (", text, ")");
}
int half_code(const torch::Tensor& x, const char* fn) {
  if (x.scalar_type() == at::kHalf) return PARO_DTYPE_F16;
  if (x.scalar_type() == at::kBFloat16) return PARO_DTYPE_BF16;
  TORCH_CHECK(false, fn, " failed to dispatch data type ", x.scalar_type());
  return -1;
}
void* stream_of(const torch::Tensor& x) { return c10::hip::getCurrentHIPStream(x.device().index()).stream(); }

struct Layout { int64_t n_tokens, n_heads, stride_n, stride_h; };
Layout layout_of(const torch::Tensor& x, int tensor_layout) {
  if (tensor_layout == 0) return {x.size(1), x.size(2), x.stride(1), x.stride(2)};
  return {x.size(2), x.size(1), x.stride(2), x.stride(1)};
}

// ---- _qattn_sm80 ------------------------------------------------------------------------------------
// The reference's positional signature has no room for this library's attention flags (PARO_ATTN_* of
// include/paroatten.h: exact exponentials, the float16 P.V product, launch forms).  A process-wide default,
// set_attention_flags(), lets a caller of the compiled module choose them; 0 = the library's defaults.
static std::atomic<int> g_attention_flags{0};
void set_attention_flags(int flags) { g_attention_flags.store(flags); }
int get_attention_flags() { return g_attention_flags.load(); }

torch::Tensor qk_int8_sv_f16_accum_f16_attn(torch::Tensor query, torch::Tensor key, torch::Tensor value,
                                            torch::Tensor output, torch::Tensor query_scale,
                                            torch::Tensor key_scale, int tensor_layout, int is_causal,
                                            int qk_quant_gran, float sm_scale, int return_lse,
                                            torch::Tensor sparse) {
  on_gpu(query, "query"); on_gpu(key, "key"); on_gpu(value, "value"); on_gpu(output, "output");
  on_gpu(query_scale, "query_scale"); on_gpu(key_scale, "key_scale");
  contiguous(query, "query"); contiguous(key, "key");
  lastdim_contiguous(value, "value"); lastdim_contiguous(output, "output");
  contiguous(query_scale, "query_scale"); contiguous(key_scale, "key_scale");
  dtype(query, "query", at::kChar, "torch::kInt8"); dtype(key, "key", at::kChar, "torch::kInt8");
  // the reference takes float16 only; bfloat16 saves the caller's conversion
  TORCH_CHECK(value.scalar_type() == at::kHalf || value.scalar_type() == at::kBFloat16,
              "Tensor value must have dtype (torch::kHalf)");
  dtype(query_scale, "query_scale", at::kFloat, "torch::kFloat32");
  dtype(key_scale, "key_scale", at::kFloat, "torch::kFloat32");
  dims(query, "query", 4); dims(key, "key", 4); dims(value, "value", 4); dims(output, "output", 4);
  dims(query_scale, "query_scale", 3); dims(key_scale, "key_scale", 3);
  if (tensor_layout != 0 && tensor_layout != 1) throw std::invalid_argument("tensor_layout must be 0 or 1");
  const int sn = tensor_layout == 0 ? 1 : 2, sh = tensor_layout == 0 ? 2 : 1;
  const int64_t B = query.size(0), D = query.size(3), H = query.size(sh), Hkv = key.size(sh), Nq = query.size(sn),
                Nk = key.size(sn);
  if (tensor_layout == 0) {
    shape(key, "key", {B, Nk, Hkv, D}, "batch_size, kv_len, num_kv_heads, head_dim");
    shape(value, "value", {B, Nk, Hkv, D}, "batch_size, kv_len, num_kv_heads, head_dim");
  } else {
    shape(key, "key", {B, Hkv, Nk, D}, "batch_size, num_kv_heads, kv_len, head_dim");
    shape(value, "value", {B, Hkv, Nk, D}, "batch_size, num_kv_heads, kv_len, head_dim");
  }
  if (Hkv == 0 || H % Hkv != 0)
    throw std::invalid_argument("num_qo_heads (" + std::to_string(H) + ") must be divisible by num_kv_heads (" +
                                std::to_string(Hkv) + ")");
  if (D != 64 && D != 128) throw std::invalid_argument("Unsupported head dim: " + std::to_string(D));
  if (return_lse != 0 && return_lse != 1)
    throw std::invalid_argument("Unsupported causal mode: " + std::to_string(return_lse));   // sic, as the reference words it
  const int out_code = half_code(output, "qk_int8_sv_f16_accum_f16_attn");
  TORCH_CHECK(output.sizes() == query.sizes(), "Tensor output must have the shape of query");
  const int64_t nbq = (Nq + 63) / 64, nbk = (Nk + 63) / 64;
  if (qk_quant_gran == 2) {
    shape(query_scale, "query_scale", {B, H, nbq * 2},
          "batch_size, num_qo_heads, div_ceil(qo_len, CTA_Q) * (CTA_Q / WARP_Q)");
    shape(key_scale, "key_scale", {B, Hkv, nbk}, "batch_size, num_kv_heads, div_ceil(kv_len, CTA_K) * (CTA_K / WARP_K)");
  } else if (qk_quant_gran == 3) {   // per thread (csrc/qattn/qk_int_sv_f16_cuda_sm80.cu:1034-1038)
    shape(query_scale, "query_scale", {B, H, nbq * 2 * 8},
          "batch_size, num_qo_heads, div_ceil(qo_len, CTA_Q) * (CTA_Q / WARP_Q) * 8");
    shape(key_scale, "key_scale", {B, Hkv, nbk * 4},
          "batch_size, num_kv_heads, div_ceil(kv_len, CTA_K) * (CTA_K / WARP_K) * 4");
  }
  // the reference reads `sparse` through a raw pointer without any check
  on_gpu(sparse, "sparse"); contiguous(sparse, "sparse");
  TORCH_CHECK(sparse.scalar_type() == at::kBool || sparse.scalar_type() == at::kByte,
              "Tensor sparse must have dtype (torch::kBool)");
  int64_t sparse_bs = 0;
  if (sparse.dim() == 4) {
    shape(sparse, "sparse", {B, H, nbq, nbk}, "batch_size, num_qo_heads, num_q_blocks, num_k_blocks");
    sparse_bs = sparse.stride(0);
  } else {
    dims(sparse, "sparse", 3);
    shape(sparse, "sparse", {H, nbq, nbk}, "num_qo_heads, num_q_blocks, num_k_blocks");
  }
  const c10::DeviceGuard guard(query.device());
  torch::Tensor lse = torch::empty({0});
  if (return_lse) lse = torch::empty({B, H, Nq}, query.options().dtype(at::kFloat));
  const int flags = g_attention_flags.load();
  const int64_t ws_bytes = paro_attn_workspace_bytes_for((int)B, (int)Hkv, (int)Nk, (int)D, flags);
  torch::Tensor ws = torch::empty({ws_bytes}, query.options().dtype(at::kByte));
  check_rc(paro_qk_int8_sv_f16_attn(
      query.data_ptr<int8_t>(), key.data_ptr<int8_t>(), value.data_ptr(), half_code(value, "qk_int8_sv_f16_accum_f16_attn"),
      output.data_ptr(), out_code, query_scale.data_ptr<float>(), key_scale.data_ptr<float>(),
      static_cast<const uint8_t*>(sparse.data_ptr()), sparse_bs, return_lse ? lse.data_ptr<float>() : nullptr,
      ws.data_ptr(), ws_bytes, (int)B, (int)H, (int)Hkv, (int)Nq, (int)Nk, (int)D, query.stride(0), query.stride(sh),
      query.stride(sn), key.stride(0), key.stride(sh), key.stride(sn), value.stride(0), value.stride(sh), value.stride(sn),
      output.stride(0), output.stride(sh), output.stride(sn), tensor_layout, is_causal, qk_quant_gran, sm_scale,
      /*smooth_v=*/1, flags, stream_of(query)));
  return lse;
}

torch::Tensor prototype_variant(torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
                                int, int, int, float, int, torch::Tensor) {
  PyErr_SetString(PyExc_NotImplementedError,
                  "experimental variant of the reference (INT4 Q/K or INT8 P.V) without a working caller; "
                  "use qk_int8_sv_f16_accum_f16_attn");
  throw py::error_already_set();
}

// ---- _fused -----------------------------------------------------------------------------------------
void quant_int8(const char* fn, torch::Tensor input, const torch::Tensor* mean, torch::Tensor output, torch::Tensor scale,
                int group, int64_t groups_per_block, int block_size, int tensor_layout, bool has_sm_scale,
                float sm_scale) {
  on_gpu(input, "input"); on_gpu(output, "output"); on_gpu(scale, "scale");
  if (mean) on_gpu(*mean, "mean");
  dtype(output, "output", at::kChar, "torch::kInt8"); dtype(scale, "scale", at::kFloat, "torch::kFloat");
  dims(input, "input", 4);
  lastdim_contiguous(input, "input"); contiguous(output, "output"); contiguous(scale, "scale");
  dims(output, "output", 4); dims(scale, "scale", 3);
  if (mean) { lastdim_contiguous(*mean, "mean"); dims(*mean, "mean", 3); }
  const int code = half_code(input, fn);
  if (mean) TORCH_CHECK(mean->scalar_type() == input.scalar_type(), "Tensor mean must have dtype (input_dtype)");
  const int64_t B = input.size(0), D = input.size(3);
  const Layout in = layout_of(input, tensor_layout), out = layout_of(output, tensor_layout);
  if (block_size != 64 && block_size != 128) throw std::invalid_argument("Unsupported block_size " + std::to_string(block_size));
  if (D != 64 && D != 128) throw std::invalid_argument("Unsupported head dim: " + std::to_string(D));
  const int64_t n_groups = (in.n_tokens + block_size - 1) / block_size * groups_per_block;
  TORCH_CHECK(output.sizes() == input.sizes(),
              "Tensor output must have shape (input.size(0), input.size(1), input.size(2), input.size(3))");
  shape(scale, "scale", {B, in.n_heads, n_groups}, "batch_size, num_heads, num_groups");
  if (mean) shape(*mean, "mean", {B, in.n_heads, D}, "batch_size, num_heads, head_dim");
  const c10::DeviceGuard guard(input.device());
  check_rc(paro_quant_int8(input.data_ptr(), code, mean ? mean->data_ptr() : nullptr, output.data_ptr<int8_t>(),
                           scale.data_ptr<float>(), (int)B, (int)in.n_heads, (int)in.n_tokens, (int)D, input.stride(0),
                           in.stride_h, in.stride_n, mean ? mean->stride(0) : 0, mean ? mean->stride(1) : 0,
                           output.stride(0), out.stride_h, out.stride_n, scale.stride(0), scale.stride(1), group,
                           (int)n_groups, has_sm_scale ? 1 : 0, sm_scale, stream_of(input)));
}

void quant_per_block_int8_cuda_sm(torch::Tensor input, torch::Tensor output, torch::Tensor scale, float sm_scale,
                                  int block_size, int tensor_layout) {
  quant_int8("quant_per_block_int8_cuda", input, nullptr, output, scale, block_size, 1, block_size, tensor_layout, true, sm_scale);
}
void quant_per_block_int8_cuda(torch::Tensor input, torch::Tensor output, torch::Tensor scale, int block_size,
                               int tensor_layout) {
  quant_int8("quant_per_block_int8_cuda", input, nullptr, output, scale, block_size, 1, block_size, tensor_layout, false, 0.f);
}
void quant_per_block_int8_fuse_sub_mean_cuda(torch::Tensor input, torch::Tensor mean, torch::Tensor output,
                                             torch::Tensor scale, int block_size, int tensor_layout) {
  quant_int8("quant_per_block_int8_fuse_sub_mean_cuda", input, &mean, output, scale, block_size, 1, block_size,
             tensor_layout, false, 0.f);
}
void quant_per_warp_int8_cuda(torch::Tensor input, torch::Tensor output, torch::Tensor scale, int block_size,
                              int warp_block_size, int tensor_layout) {
  if (block_size != 64 && block_size != 128) throw std::invalid_argument("Unsupported block_size " + std::to_string(block_size));
  if (warp_block_size != 16 && warp_block_size != 32)
    throw std::invalid_argument("Unsupported warp_block_size " + std::to_string(warp_block_size));
  quant_int8("quant_per_warp_int8_cuda", input, nullptr, output, scale, warp_block_size, block_size / warp_block_size,
             block_size, tensor_layout, false, 0.f);
}

void sub_mean_cuda(torch::Tensor input, torch::Tensor mean, torch::Tensor output, int tensor_layout) {
  on_gpu(input, "input"); on_gpu(mean, "mean"); on_gpu(output, "output");
  dtype(output, "output", at::kHalf, "torch::kHalf");
  dims(input, "input", 4); dims(mean, "mean", 3); dims(output, "output", 4);
  lastdim_contiguous(input, "input"); lastdim_contiguous(mean, "mean"); lastdim_contiguous(output, "output");
  const int code = half_code(input, "sub_mean_cuda");
  TORCH_CHECK(mean.scalar_type() == input.scalar_type(), "Tensor mean must have dtype (input_dtype)");
  const int64_t B = input.size(0), D = input.size(3);
  const Layout in = layout_of(input, tensor_layout), out = layout_of(output, tensor_layout);
  shape(mean, "mean", {B, in.n_heads, D}, "batch_size, num_heads, head_dim");
  TORCH_CHECK(output.sizes() == input.sizes(),
              "Tensor output must have shape (input.size(0), input.size(1), input.size(2), input.size(3))");
  const c10::DeviceGuard guard(input.device());
  check_rc(paro_sub_mean(input.data_ptr(), code, mean.data_ptr(), output.data_ptr(), (int)B, (int)in.n_heads,
                         (int)in.n_tokens, (int)D, input.stride(0), in.stride_h, in.stride_n, mean.stride(0),
                         mean.stride(1), output.stride(0), out.stride_h, out.stride_n, stream_of(input)));
}

void transpose_pad_permute_cuda(torch::Tensor input, torch::Tensor output, int tensor_layout) {
  on_gpu(input, "input"); on_gpu(output, "output");
  lastdim_contiguous(input, "input"); contiguous(output, "output");
  dims(input, "input", 4); dims(output, "output", 4);
  const int64_t B = input.size(0), D = input.size(3);
  const Layout in = layout_of(input, tensor_layout);
  const int64_t padded = (in.n_tokens + 63) / 64 * 64;
  int64_t os_d, os_h;
  if (tensor_layout == 0) {
    shape(output, "output", {B, D, in.n_heads, padded}, "batch_size, head_dim, num_heads, padded_num_tokens");
    os_d = output.stride(1); os_h = output.stride(2);
  } else {
    shape(output, "output", {B, in.n_heads, D, padded}, "batch_size, num_heads, head_dim, padded_num_tokens");
    os_d = output.stride(2); os_h = output.stride(1);
  }
  TORCH_CHECK(input.scalar_type() == output.scalar_type(), "Input and output must have the same data type");
  const int code = half_code(input, "transpose_pad_permute_cuda");
  if (D != 64 && D != 128) throw std::invalid_argument("Unsupported head dim: " + std::to_string(D));
  const c10::DeviceGuard guard(input.device());
  check_rc(paro_transpose_pad_permute(input.data_ptr(), output.data_ptr(), code, (int)B, (int)in.n_heads, (int)in.n_tokens,
                                      (int)D, input.stride(0), in.stride_h, in.stride_n, output.stride(0), os_h, os_d,
                                      stream_of(input)));
}

void channel_quant(const char* fn, torch::Tensor input, torch::Tensor output, const torch::Tensor* mean, torch::Tensor scale,
                   int num_tokens, float scale_max, int tensor_layout) {
  on_gpu(input, "input"); on_gpu(output, "output");
  if (mean) on_gpu(*mean, "mean");
  on_gpu(scale, "scale");
  if (mean) dtype(*mean, "mean", at::kFloat, "torch::kFloat");
  dtype(scale, "scale", at::kFloat, "torch::kFloat");
  contiguous(input, "input"); contiguous(output, "output");
  if (mean) contiguous(*mean, "mean");
  contiguous(scale, "scale");
  dims(input, "input", 4); dims(output, "output", 4);
  if (mean) dims(*mean, "mean", 3);
  dims(scale, "scale", 3);
  const int64_t B = input.size(0), row_len = input.size(3);
  const int d_dim = tensor_layout == 0 ? 1 : 2, h_dim = tensor_layout == 0 ? 2 : 1;
  const int64_t H = input.size(h_dim), D = input.size(d_dim);
  TORCH_CHECK(output.sizes() == input.sizes(),
              "Tensor output must have shape (input.size(0), input.size(1), input.size(2), input.size(3))");
  if (mean) shape(*mean, "mean", {B, H, D}, "batch_size, num_heads, head_dim");
  shape(scale, "scale", {B, H, D}, "batch_size, num_heads, head_dim");
  const int code = half_code(input, fn);
  TORCH_CHECK(output.element_size() == 1, "Tensor output must have a one-byte dtype (torch.float8_e4m3fn)");
  const c10::DeviceGuard guard(input.device());
  check_rc(paro_channel_quant_fp8(input.data_ptr(), code, static_cast<uint8_t*>(output.data_ptr()),
                                  mean ? mean->data_ptr<float>() : nullptr, scale.data_ptr<float>(), (int)B, (int)H, (int)D,
                                  num_tokens, (int)row_len, scale_max, input.stride(0), input.stride(h_dim),
                                  input.stride(d_dim), output.stride(0), output.stride(h_dim), output.stride(d_dim),
                                  mean ? mean->stride(0) : 0, mean ? mean->stride(1) : 0, scale.stride(0), scale.stride(1),
                                  stream_of(input)));
}
void scale_fuse_quant_cuda(torch::Tensor input, torch::Tensor output, torch::Tensor scale, int num_tokens, float scale_max,
                           int tensor_layout) {
  channel_quant("scale_fuse_quant_cuda", input, output, nullptr, scale, num_tokens, scale_max, tensor_layout);
}
void mean_scale_fuse_quant_cuda(torch::Tensor input, torch::Tensor output, torch::Tensor mean, torch::Tensor scale,
                                int num_tokens, float scale_max, int tensor_layout) {
  channel_quant("mean_scale_fuse_quant_cuda", input, output, &mean, scale, num_tokens, scale_max, tensor_layout);
}

// ---- _rope ------------------------------------------------------------------------------------------
// rope_permutation(Q, K, freq, permutation) -> (QO, KO): Q, K float16 [bs, H, W, dim]; freq float32 [128]
// of (cos, sin) pairs shared by every token and every 128-channel slice; with `permutation` the (H, W) grid
// is written transposed.  The reference's permuting kernel overwrites its inputs and leaves its outputs
// uninitialised (csrc/rope/rope.cuh:49-50); here the inputs stay and the outputs hold the result.
std::vector<torch::Tensor> rope_permutation(torch::Tensor Q, torch::Tensor K, torch::Tensor freq, bool permutation) {
  on_gpu(Q, "Q"); on_gpu(K, "K"); on_gpu(freq, "freq");
  TORCH_CHECK(Q.scalar_type() == at::kHalf && K.scalar_type() == at::kHalf, "expected scalar type Half");
  TORCH_CHECK(freq.scalar_type() == at::kFloat && freq.numel() == 128, "freq must be float32 with 128 entries");
  TORCH_CHECK(Q.dim() == 4 && Q.sizes() == K.sizes() && Q.is_contiguous() && K.is_contiguous(),
              "Q and K must be contiguous [bs, H, W, dim] tensors of the same shape");
  const int64_t bs = Q.size(0), H = Q.size(1), W = Q.size(2), dim = Q.size(3);
  if (dim % 128 != 0) throw std::invalid_argument("Unsupported head dim: " + std::to_string(dim) + " (must be a multiple of 128)");
  const int64_t heads = dim / 128, n = H * W;
  const c10::DeviceGuard guard(Q.device());
  auto cs = freq.view({64, 2});
  auto cos = cs.select(1, 0).repeat_interleave(2).expand({n, 128}).contiguous();
  auto sin = cs.select(1, 1).repeat_interleave(2).expand({n, 128}).contiguous();
  auto orders = torch::full({heads}, permutation ? 1 : 0, Q.options().dtype(at::kInt));
  auto QO = torch::empty({bs, n, dim}, Q.options()), KO = torch::empty({bs, n, dim}, Q.options());
  // [bs, n, heads, 128] seen as (batch, head, token, channel) through strides
  check_rc(paro_rope_permute_fwd(Q.data_ptr(), K.data_ptr(), nullptr, QO.data_ptr(), KO.data_ptr(), nullptr, PARO_DTYPE_F16,
                                 cos.data_ptr<float>(), sin.data_ptr<float>(), orders.data_ptr<int32_t>(), (int)bs, (int)heads,
                                 (int)n, 128, 0, 1, (int)H, (int)W, n * dim, 128, dim, n * dim, 128, dim, stream_of(Q)));
  return {QO, KO};
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "paroattention's extension modules (_qattn_sm80, _fused, _rope) over libparoatten_hip.so (gfx950)";
  m.def("abi_version", &paro_abi_version);
  auto qattn = m.def_submodule("_qattn_sm80");
  qattn.def("qk_int8_sv_f16_accum_f16_attn", &qk_int8_sv_f16_accum_f16_attn, "QK int8 sv f16 accum f16 attn");
  qattn.def("set_attention_flags", &set_attention_flags,
            "process-wide PARO_ATTN_* flags of the attention entry point (1 exact exponentials, 16 float16 P.V product, ...)");
  qattn.def("get_attention_flags", &get_attention_flags);
  qattn.def("qk_int4_sv_f16_accum_f16_attn", &prototype_variant);
  qattn.def("qk_int4_sv_int8_accum_f16_attn", &prototype_variant);
  qattn.def("qk_int8_sv_int8_accum_f16_attn", &prototype_variant);
  auto fused = m.def_submodule("_fused");
  fused.def("quant_per_block_int8_cuda", &quant_per_block_int8_cuda_sm);
  fused.def("quant_per_block_int8_cuda", &quant_per_block_int8_cuda);
  fused.def("quant_per_block_int8_fuse_sub_mean_cuda", &quant_per_block_int8_fuse_sub_mean_cuda);
  fused.def("quant_per_warp_int8_cuda", &quant_per_warp_int8_cuda);
  fused.def("sub_mean_cuda", &sub_mean_cuda);
  fused.def("transpose_pad_permute_cuda", &transpose_pad_permute_cuda);
  fused.def("scale_fuse_quant_cuda", &scale_fuse_quant_cuda);
  fused.def("mean_scale_fuse_quant_cuda", &mean_scale_fuse_quant_cuda);
  auto rope = m.def_submodule("_rope");
  rope.def("rope_permutation", &rope_permutation, "RoPE op with permutation.");
}
