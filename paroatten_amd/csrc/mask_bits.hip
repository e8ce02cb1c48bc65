// Block-mask bit packing: bool bytes <-> 1 bit per block.
//
// The sparse plan is the only per-layer operand that lives on the host (the reference keeps it
// there as torch.bool and copies one [H,nb,nb] slice per layer, paroattention/prefetch_utils.py:34-59
// and paroattention/cogvideox.py:188-213).  Packed to bits it is 8x smaller in pinned memory and
// over PCIe; these two kernels convert on the device, on the stream of the copy.
// Bit i of byte j holds element 8j+i (numpy.packbits(..., bitorder="little")).
#include "paro_common.hpp"

namespace paro {

// One lane per 16 mask elements: 16 B of bool in, 2 B of bits out (and the reverse).
__global__ __launch_bounds__(256) void mask_pack_kernel(const uint8_t* __restrict__ mask,
                                                        uint8_t* __restrict__ bits, int64_t n) {
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t e0 = g * 16;
  if (e0 >= n) return;
  unsigned w = 0;
  if (e0 + 16 <= n) {
    const uint4 x = *reinterpret_cast<const uint4*>(mask + e0);
    const unsigned v[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int b = 0; b < 4; ++b) w |= (((v[i] >> (8 * b)) & 0xffu) != 0u ? 1u : 0u) << (4 * i + b);
    *reinterpret_cast<unsigned short*>(bits + 2 * g) = (unsigned short)w;
  } else {
    const int r = (int)(n - e0);
    for (int i = 0; i < r; ++i) w |= (mask[e0 + i] != 0 ? 1u : 0u) << i;
    bits[2 * g] = (uint8_t)(w & 0xff);
    if (r > 8) bits[2 * g + 1] = (uint8_t)(w >> 8);
  }
}

__global__ __launch_bounds__(256) void mask_unpack_kernel(const uint8_t* __restrict__ bits,
                                                          uint8_t* __restrict__ mask, int64_t n) {
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t e0 = g * 16;
  if (e0 >= n) return;
  if (e0 + 16 <= n) {
    const unsigned w = *reinterpret_cast<const unsigned short*>(bits + 2 * g);
    unsigned v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[i] = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) v[i] |= ((w >> (4 * i + b)) & 1u) << (8 * b);
    }
    *reinterpret_cast<uint4*>(mask + e0) = make_uint4(v[0], v[1], v[2], v[3]);
  } else {
    const int r = (int)(n - e0);
    unsigned w = bits[2 * g];
    if (r > 8) w |= (unsigned)bits[2 * g + 1] << 8;
    for (int i = 0; i < r; ++i) mask[e0 + i] = (uint8_t)((w >> i) & 1u);
  }
}

static int check_args(const void* a, const void* b, int64_t n, const char* fn) {
  PARO_CHECK(n >= 0 && n < ((int64_t)1 << 40), PARO_ERR_INVALID_VALUE, "%s: n = %lld out of range", fn, (long long)n);
  if (n == 0) return PARO_OK;
  PARO_CHECK(a && b, PARO_ERR_RUNTIME, "%s: null pointer", fn);
  PARO_CHECK(((uintptr_t)a % 16 == 0) && ((uintptr_t)b % 16 == 0), PARO_ERR_RUNTIME,
             "%s: mask and bits must be 16-byte aligned", fn);
  return PARO_OK;
}

}  // namespace paro

extern "C" int64_t paro_mask_bits_bytes(int64_t n) { return n < 0 ? 0 : (n + 7) / 8; }

extern "C" int paro_mask_pack(const uint8_t* mask, uint8_t* bits, int64_t n, void* stream) {
  using namespace paro;
  if (int rc = check_args(mask, bits, n, "paro_mask_pack")) return rc;
  if (n == 0) return PARO_OK;
  const int64_t groups = (n + 15) / 16;
  hipLaunchKernelGGL(mask_pack_kernel, dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     mask, bits, n);
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}

extern "C" int paro_mask_unpack(const uint8_t* bits, uint8_t* mask, int64_t n, void* stream) {
  using namespace paro;
  if (int rc = check_args(bits, mask, n, "paro_mask_unpack")) return rc;
  if (n == 0) return PARO_OK;
  const int64_t groups = (n + 15) / 16;
  hipLaunchKernelGGL(mask_unpack_kernel, dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     bits, mask, n);
  PARO_HIP(hipGetLastError());
  return PARO_OK;
}
