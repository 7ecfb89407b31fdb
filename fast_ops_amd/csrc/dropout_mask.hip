// The dropout keep-mask of the attention kernels as a tensor of its own (flash_attention_triton.py:669-717,
// _dropout_mask_kernel / triton_dropout_mask): what a caller needs to apply the very same mask in a reference
// computation. One byte per (batch, head, query, key): 1 = kept. HBM-bound (1 byte written per element).
#include "attn_common.hpp"
#include "common.hpp"

namespace fo {

// 16 consecutive elements per lane and store: one 16-byte write
__global__ void __launch_bounds__(256) dropout_mask_kernel(uint8_t* __restrict__ out, int64_t n, DropoutParams drop) {
  const int64_t first = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 16;
  if (first >= n) return;
  const uint32_t base = drop.offset + (uint32_t)first;     // 32-bit wrap-around, as the kernels index (:125)
  if (first + 16 <= n && (((uintptr_t)out) & 15u) == 0) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      w[i] = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) w[i] |= (dropout_keep(base + 4 * i + j, drop.seed, drop.threshold) ? 1u : 0u) << (8 * j);
    }
    typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
    u32x4 v = {w[0], w[1], w[2], w[3]};
    *(u32x4*)(out + first) = v;
  } else {
    for (int i = 0; i < 16 && first + i < n; ++i) out[first + i] = dropout_keep(base + i, drop.seed, drop.threshold) ? 1 : 0;
  }
}

}  // namespace fo

extern "C" int fo_dropout_mask(uint8_t* keep, int64_t n_elements, float dropout_p, uint32_t seed, uint64_t rng_offset, void* stream) {
  if (!keep) return FO_ERR_NULL_POINTER;
  if (n_elements < 0 || n_elements > (1ll << 40)) return FO_ERR_BAD_SHAPE;
  if (!(dropout_p >= 0.0f) || dropout_p >= 1.0f) return FO_ERR_BAD_SHAPE;
  if (n_elements == 0) return FO_OK;
  const int64_t blocks = (n_elements + 4095) / 4096;
  fo::dropout_mask_kernel<<<(unsigned)blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(keep, n_elements, fo::make_dropout(dropout_p, seed, rng_offset));
  return fo::launch_status();
}
