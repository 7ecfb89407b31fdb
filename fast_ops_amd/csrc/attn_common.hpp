// Helpers shared by the attention kernels (forward and backward) of libfastops_hip.so.
#pragma once
#include "common.hpp"

namespace fo {

#define FO_LDS __attribute__((address_space(3)))
#define FO_GLOBAL __attribute__((address_space(1)))

template <typename T> struct Ops;
template <> struct Ops<__bf16> {
  typedef bf16x8 vec8;
  static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};
template <> struct Ops<_Float16> {
  typedef f16x8 vec8;
  static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};

// swizzle of 16-byte chunks inside a tile row; `row` is the row inside the tile
template <int D>
__device__ __forceinline__ int swz(int row) {
  if constexpr (D == 128) return ((row & 3) << 2) | ((row >> 2) & 3);              // 16 chunks per 256-byte row
  else { const int R = row >> 1; return ((R & 1) << 2) | ((R >> 1) & 3); }          // 8 chunks per 128-byte row
}

__device__ __forceinline__ float half_swap(float x) {
  // value held by the lane 32 positions away
  auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(int, x), __builtin_bit_cast(int, x), false, false);
  return __builtin_bit_cast(float, (threadIdx.x & 32) ? r[0] : r[1]);
}

// 16 bytes per lane, global -> LDS without passing through registers. LDS receives the 64 lanes' pieces back to back
// starting at `dst` (wave-uniform); the global address is per lane.
// An LDS-DMA instruction reads M0 (the LDS destination) and needs one wait state after the scalar instruction that
// wrote it. The compiler adds that s_nop for its own builtin; inside an asm statement nobody does, so it is spelled out
// here, and the build's assembly check (asm_lint.py) verifies it for every kernel.
// (hipcc also parses device functions in its host pass, where GCN assembly cannot be checked: the bodies exist in the
// device pass only.)
__device__ __forceinline__ void dma16_uniform_base(const void* base, uint32_t byte_off, FO_LDS void* dst) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(__builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)dst)), "v"(byte_off), "s"(base) : "memory", "m0");
#endif
}
// ... with the LDS address as a wave-uniform register plus a constant: one scalar instruction forms it in M0
template <int IMM>
__device__ __forceinline__ void dma16_uniform_base_lds_imm(const void* base, uint32_t byte_off, uint32_t lds_base) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(byte_off), "s"(base), "n"(IMM) : "memory", "m0", "scc");
#endif
}
__device__ __forceinline__ void dma16_lane_ptr(const void* ptr, FO_LDS void* dst) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(__builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)dst)), "v"(ptr) : "memory", "m0");
#endif
}

// Sixteen zero bytes in device memory. A head_dim below the 64 or 128 columns a kernel is compiled for is handled by
// addresses alone: whatever would read columns past the true head_dim - a lane's piece of a tile copy, a fragment
// loaded from a row - reads these zeros instead, so the padded columns of every operand are zero (they add nothing to a
// product) and nothing is read past the end of a row; stores of such columns are skipped.
static __device__ __attribute__((aligned(16))) const uint32_t kZero16[4] = {0u, 0u, 0u, 0u};
template <typename T>
__device__ __forceinline__ const T* live_or_zero(const T* ptr, int col, int d) {
  return col < d ? ptr : (const T*)kZero16;
}

// Dropout of attention probabilities, as the reference defines it (flash_attention_triton.py:38-50,125,216-219): element
// (b*H + h, q, key) has the 32-bit index  offset + (b*H + h)*Sq*Sk + q*Sk + key  (all arithmetic modulo 2^32); the index,
// xored with the seed, goes through an integer hash, and the element is KEPT iff the hash exceeds
// uint32(fp32(p) * 2^32); kept probabilities are multiplied by 1 / (1 - p). Row sums (and so LSE) use the
// undropped probabilities.
struct DropoutParams {
  uint32_t seed;
  uint32_t threshold;     // uint32(fp32(p) * fp32(4294967295)), computed on the host
  uint32_t offset;        // low 32 bits of the generator offset
  float keep_scale;       // 1 / (1 - p) in fp32; 1 when dropout is off
};
__host__ __device__ __forceinline__ bool dropout_keep(uint32_t index, uint32_t seed, uint32_t threshold) {
  uint32_t a = index ^ seed;
  a ^= a >> 4;
  a = (a ^ 0xDEADBEEFu) + (a << 5);
  a ^= a >> 11;
  return a > threshold;
}
inline DropoutParams make_dropout(float p, uint32_t seed, uint64_t rng_offset) {
  DropoutParams d;
  d.seed = seed;
  d.threshold = (uint32_t)(p * 4294967296.0f);       // fp32 product; fp32(4294967295) is 2^32
  d.offset = (uint32_t)rng_offset;
  d.keep_scale = 1.0f / (1.0f - p);
  return d;
}

// Additive bias on the scaled scores (flash_attention_triton.py:176-198, attention_ref.py:50-51): element
// (b, h, q, key) at bias + b*strides[0] + h*strides[1] + q*strides[2] + key, a stride of 0 broadcasting that dimension
// (the reference's "vector" bias is strides[2] == 0); fp32 or the operand type.
struct BiasParams {
  const void* ptr;
  int64_t strides[3];
  int is_f32;
  int dma_ok;   // forward: base and the three strides are multiples of 16 bytes, tiles may be copied with 16-byte pieces
  int vec_ok;   // base and the three strides are multiples of 4 elements: 4 consecutive keys may be read with one load
};
template <typename T>
__device__ __forceinline__ float load_bias(const BiasParams& bp, int64_t at) {
  return bp.is_f32 ? ((const float*)bp.ptr)[at] : (float)((const T*)bp.ptr)[at];
}
// four consecutive elements of type E (float or the operand type) from an address that is a multiple of 4 elements
template <typename E>
__device__ __forceinline__ void load_bias4(const E* at, float* out) {
  typedef __attribute__((ext_vector_type(4))) E e4;
  const e4 t = *(const e4*)at;
#pragma unroll
  for (int u = 0; u < 4; ++u) out[u] = (float)t[u];
}

// the same with 4 bytes per lane (LDS receives 256 bytes)
__device__ __forceinline__ void dma4_lane_ptr(const void* ptr, FO_LDS void* dst) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(__builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)dst)), "v"(ptr) : "memory", "m0");
#endif
}
// ... from a wave-uniform base plus a per-lane byte offset
__device__ __forceinline__ void dma4_uniform_base(const void* base, uint32_t byte_off, FO_LDS void* dst) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(__builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)dst)), "v"(byte_off), "s"(base) : "memory", "m0");
#endif
}

}  // namespace fo
