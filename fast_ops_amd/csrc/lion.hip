// Fused Lion step for gfx950: fp32 parameters and gradients, bf16 momentum, one HBM pass (16 bytes per parameter:
// read p 4 + g 4 + m 2, write p 4 + m 2).
//
// Replaces lion_update_kernel / lion_update (fast_ops/lion/lion_update.cu:15-107,121-161) and the per-parameter launch
// loop of Lion.step (fast_ops/lion/lion_optimizer.py:64-76). Same fusion (decay, sign update, momentum decay in one
// pass, lion_update.cu:55-105), but the arithmetic keeps the fp32 rounding points of the Python formula
// (fast_ops/lion/lion_optimizer_ref.py:51,64,65,67) instead of computing in the half type.
//
// This file is compiled with -ffp-contract=off: the only fused multiply-add is the explicit one in the momentum update.
//
// Launch shape: one workgroup of 256 lanes per chunk of FO_LION_CHUNK (8192) elements, so a wave issues 1 KiB
// (p, g: 16 B per lane) or 512 B (m: 8 B per lane) fully coalesced requests. All of a chunk's loads are issued
// before the first dependent instruction (8 x 40 B in flight per lane), which is what keeps HBM busy; streaming
// (non-temporal) accesses keep 13 GB of single-use data from churning L2.
#include "common.hpp"

namespace fo {

struct LionC { float c_wd, c_b1, c_1b1, c_nlr, c_b2, c_1b2; };

__device__ __forceinline__ uint32_t bf16_rne_bits(float f) {
  // c10::BFloat16 rounding: NaN -> 0x7FC0, otherwise add 0x7FFF + lsb and truncate
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  uint32_t r = (u + (((u >> 16) & 1u) + 0x7FFFu)) >> 16;
  return (f != f) ? 0x7FC0u : r;
}
__device__ __forceinline__ float bf16_bits_f32(uint32_t b) { return __builtin_bit_cast(float, b << 16); }

// one element; returns the new parameter, writes the new momentum bits
__device__ __forceinline__ float lion_elem(float p, float g, uint32_t mbits, const LionC& c, uint32_t& mout) {
  const float mf = bf16_bits_f32(mbits);
  const float p1 = p * c.c_wd;                                       // ref :51
  const float t1 = bf16_bits_f32(bf16_rne_bits(mf * c.c_b1));        // ref :64 (bf16 tensor)
  const float t2 = g * c.c_1b1;                                      // ref :64
  const float u = t1 + t2;                                           // ref :64
  const float s = (u > 0.0f) ? 1.0f : ((u < 0.0f) ? -1.0f : 0.0f);   // ref :65 torch.sign (0 for zero and NaN)
  const float p2 = p1 + c.c_nlr * s;                                 // ref :65 (product exact)
  const float m1 = bf16_bits_f32(bf16_rne_bits(mf * c.c_b2));        // ref :67 mul_ rounds to bf16
  mout = bf16_rne_bits(__builtin_fmaf(c.c_1b2, g, m1));              // ref :67 add_(g, alpha) is fused
  return p2;
}

// Pointers that arrive through a descriptor in memory have no known address space and would compile to flat_*
// accesses; every buffer here is device memory, so they are cast to the global address space (global_* accesses).
#define FO_GLOBAL __attribute__((address_space(1)))
template <typename T>
__device__ __forceinline__ FO_GLOBAL T* as_global(T* p) { return (FO_GLOBAL T*)p; }

template <bool NT, typename T>
__device__ __forceinline__ T ld(const FO_GLOBAL T* p) {
  if constexpr (NT) return __builtin_nontemporal_load(p);
  else return *p;
}
template <bool NT, typename T>
__device__ __forceinline__ void st(FO_GLOBAL T* p, T v) {
  if constexpr (NT) __builtin_nontemporal_store(v, p);
  else *p = v;
}

constexpr int kThreads = 256;
constexpr int kVec = 4;                                   // elements per lane per access
constexpr int kRow = kThreads * kVec;                     // 1024 elements per workgroup access
constexpr int kIters = FO_LION_CHUNK / kRow;              // 8
static_assert(FO_LION_CHUNK % kRow == 0, "chunk must be a whole number of workgroup rows");

// four elements held by one lane: p/g as a 16-byte vector, m as two packed bf16 pairs
__device__ __forceinline__ void lion_vec4(const f32x4& pr, const f32x4& gr, const u32x2& mr, const LionC& c, f32x4& po, u32x2& mo) {
  uint32_t o0, o1, o2, o3;
  po[0] = lion_elem(pr[0], gr[0], mr[0] & 0xFFFFu, c, o0);
  po[1] = lion_elem(pr[1], gr[1], mr[0] >> 16, c, o1);
  po[2] = lion_elem(pr[2], gr[2], mr[1] & 0xFFFFu, c, o2);
  po[3] = lion_elem(pr[3], gr[3], mr[1] >> 16, c, o3);
  mo[0] = o0 | (o1 << 16);
  mo[1] = o2 | (o3 << 16);
}

// One chunk of n <= FO_LION_CHUNK elements, processed by a whole workgroup.
// UNROLL = how many 1024-element rows are loaded before the first is consumed (kIters % UNROLL == 0).
template <int UNROLL, bool NT_LD, bool NT_ST>
__device__ __forceinline__ void lion_chunk(float* __restrict__ p_, const float* __restrict__ g_, uint16_t* __restrict__ m_,
                                           const int n, const LionC& c) {
  FO_GLOBAL float* p = as_global(p_);
  const FO_GLOBAL float* g = as_global(g_);
  FO_GLOBAL uint16_t* m = as_global(m_);
  const int t = threadIdx.x;
  const bool aligned = ((reinterpret_cast<uintptr_t>(p_) | reinterpret_cast<uintptr_t>(g_)) & 15u) == 0 &&
                       (reinterpret_cast<uintptr_t>(m_) & 7u) == 0;
  if (!aligned) {
    // a view into a larger buffer whose offset breaks vector alignment: element-wise
    for (int e = t; e < n; e += kThreads) {
      uint32_t o;
      p[e] = lion_elem(p[e], g[e], m[e], c, o);
      m[e] = static_cast<uint16_t>(o);
    }
    return;
  }
  FO_GLOBAL f32x4* pv = (FO_GLOBAL f32x4*)p;
  const FO_GLOBAL f32x4* gv = (const FO_GLOBAL f32x4*)g;
  FO_GLOBAL u32x2* mv = (FO_GLOBAL u32x2*)m;
  if (n == FO_LION_CHUNK) {
#pragma unroll
    for (int i0 = 0; i0 < kIters; i0 += UNROLL) {
      f32x4 pr[UNROLL], gr[UNROLL];
      u32x2 mr[UNROLL];
#pragma unroll
      for (int j = 0; j < UNROLL; ++j) {
        const int idx = (i0 + j) * kThreads + t;
        pr[j] = ld<NT_LD>(pv + idx);
        gr[j] = ld<NT_LD>(gv + idx);
        mr[j] = ld<NT_LD>(mv + idx);
      }
#pragma unroll
      for (int j = 0; j < UNROLL; ++j) {
        const int idx = (i0 + j) * kThreads + t;
        f32x4 po;
        u32x2 mo;
        lion_vec4(pr[j], gr[j], mr[j], c, po, mo);
        st<NT_ST>(pv + idx, po);
        st<NT_ST>(mv + idx, mo);
      }
    }
    return;
  }
  // short chunk (a tensor's tail): whole vectors, then up to 3 single elements
  const int nvec = n / kVec;
  for (int idx = t; idx < nvec; idx += kThreads) {
    f32x4 po;
    u32x2 mo;
    const f32x4 pr = pv[idx], gr = gv[idx];
    const u32x2 mr = mv[idx];
    lion_vec4(pr, gr, mr, c, po, mo);
    pv[idx] = po;
    mv[idx] = mo;
  }
  const int e = nvec * kVec + t;
  if (e < n) {
    uint32_t o;
    p[e] = lion_elem(p[e], g[e], m[e], c, o);
    m[e] = static_cast<uint16_t>(o);
  }
}

// many tensors: workgroup b processes the chunk described by chunks[b]
template <int UNROLL, bool NT_LD, bool NT_ST>
__global__ void __launch_bounds__(kThreads) lion_chunks_kernel(const fo_lion_chunk* __restrict__ chunks, LionC c) {
  const fo_lion_chunk ch = chunks[blockIdx.x];
  lion_chunk<UNROLL, NT_LD, NT_ST>(ch.p, ch.g, ch.m, ch.n, c);
}

// one tensor, no descriptor table: workgroup b covers elements [b*CHUNK, (b+1)*CHUNK)
template <int UNROLL, bool NT_LD, bool NT_ST>
__global__ void __launch_bounds__(kThreads) lion_flat_kernel(float* __restrict__ p, const float* __restrict__ g,
                                                             uint16_t* __restrict__ m, int64_t numel, LionC c) {
  const int64_t base = static_cast<int64_t>(blockIdx.x) * FO_LION_CHUNK;
  const int64_t left = numel - base;
  const int n = left < FO_LION_CHUNK ? static_cast<int>(left) : FO_LION_CHUNK;
  lion_chunk<UNROLL, NT_LD, NT_ST>(p + base, g + base, m + base, n, c);
}

static LionC to_c(const fo_lion_consts* k) { return LionC{k->c_wd, k->c_b1, k->c_1b1, k->c_nlr, k->c_b2, k->c_1b2}; }

// variant = UNROLL index (0:1, 1:2, 2:4, 3:8) + 4 * (nontemporal loads) + 8 * (nontemporal stores)
constexpr int kLionDefaultVariant = 3 + 4 + 8;

template <int U>
static void launch_chunks(int nt, const fo_lion_chunk* chunks, unsigned blocks, LionC c, hipStream_t s) {
  switch (nt) {
    case 0: lion_chunks_kernel<U, false, false><<<blocks, kThreads, 0, s>>>(chunks, c); break;
    case 1: lion_chunks_kernel<U, true, false><<<blocks, kThreads, 0, s>>>(chunks, c); break;
    case 2: lion_chunks_kernel<U, false, true><<<blocks, kThreads, 0, s>>>(chunks, c); break;
    default: lion_chunks_kernel<U, true, true><<<blocks, kThreads, 0, s>>>(chunks, c); break;
  }
}
template <int U>
static void launch_flat(int nt, float* p, const float* g, uint16_t* m, int64_t n, unsigned blocks, LionC c, hipStream_t s) {
  switch (nt) {
    case 0: lion_flat_kernel<U, false, false><<<blocks, kThreads, 0, s>>>(p, g, m, n, c); break;
    case 1: lion_flat_kernel<U, true, false><<<blocks, kThreads, 0, s>>>(p, g, m, n, c); break;
    case 2: lion_flat_kernel<U, false, true><<<blocks, kThreads, 0, s>>>(p, g, m, n, c); break;
    default: lion_flat_kernel<U, true, true><<<blocks, kThreads, 0, s>>>(p, g, m, n, c); break;
  }
}

}  // namespace fo

using namespace fo;

extern "C" int fo_lion_make_consts(double lr, double beta1, double beta2, double weight_decay, fo_lion_consts* out) {
  if (!out) return FO_ERR_NULL_POINTER;
  out->c_wd = static_cast<float>(1.0 - lr * weight_decay);
  out->c_b1 = static_cast<float>(beta1);
  out->c_1b1 = static_cast<float>(1.0 - beta1);
  out->c_nlr = static_cast<float>(-lr);
  out->c_b2 = static_cast<float>(beta2);
  out->c_1b2 = static_cast<float>(1.0 - beta2);
  return FO_OK;
}

extern "C" int64_t fo_lion_fill_chunks(float* p, const float* g, uint16_t* m, int64_t numel, fo_lion_chunk* out) {
  if (numel <= 0) return 0;
  const int64_t n = (numel + FO_LION_CHUNK - 1) / FO_LION_CHUNK;
  if (!out) return n;
  for (int64_t i = 0; i < n; ++i) {
    const int64_t off = i * FO_LION_CHUNK;
    const int64_t left = numel - off;
    out[i].p = p + off;
    out[i].g = g + off;
    out[i].m = m + off;
    out[i].n = static_cast<int32_t>(left < FO_LION_CHUNK ? left : FO_LION_CHUNK);
    out[i].reserved = 0;
  }
  return n;
}

extern "C" int fo_lion_step(const fo_lion_chunk* chunks_dev, int64_t n_chunks, const fo_lion_consts* consts, void* stream) {
  if (!consts) return FO_ERR_NULL_POINTER;
  if (n_chunks < 0 || n_chunks > 0x7FFFFFFFll) return FO_ERR_BAD_SHAPE;
  if (n_chunks == 0) return FO_OK;
  if (!chunks_dev) return FO_ERR_NULL_POINTER;
  if (reinterpret_cast<uintptr_t>(chunks_dev) & 7u) return FO_ERR_MISALIGNED;
  const int v = g_lion_variant < 0 ? kLionDefaultVariant : g_lion_variant;
  const LionC c = to_c(consts);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned blocks = static_cast<unsigned>(n_chunks);
  switch (v & 3) {
    case 0: launch_chunks<1>(v >> 2, chunks_dev, blocks, c, s); break;
    case 1: launch_chunks<2>(v >> 2, chunks_dev, blocks, c, s); break;
    case 2: launch_chunks<4>(v >> 2, chunks_dev, blocks, c, s); break;
    default: launch_chunks<8>(v >> 2, chunks_dev, blocks, c, s); break;
  }
  return launch_status();
}

extern "C" int fo_lion_update(float* p, const float* g, uint16_t* m, int64_t numel, const fo_lion_consts* consts, void* stream) {
  if (!consts) return FO_ERR_NULL_POINTER;
  if (numel < 0) return FO_ERR_BAD_SHAPE;
  if (numel == 0) return FO_OK;
  if (!p || !g || !m) return FO_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(p) & 3u) || (reinterpret_cast<uintptr_t>(g) & 3u) || (reinterpret_cast<uintptr_t>(m) & 1u))
    return FO_ERR_MISALIGNED;
  const int64_t n_blocks = (numel + FO_LION_CHUNK - 1) / FO_LION_CHUNK;
  if (n_blocks > 0x7FFFFFFFll) return FO_ERR_BAD_SHAPE;
  const int v = g_lion_variant < 0 ? kLionDefaultVariant : g_lion_variant;
  const LionC c = to_c(consts);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned blocks = static_cast<unsigned>(n_blocks);
  switch (v & 3) {
    case 0: launch_flat<1>(v >> 2, p, g, m, numel, blocks, c, s); break;
    case 1: launch_flat<2>(v >> 2, p, g, m, numel, blocks, c, s); break;
    case 2: launch_flat<4>(v >> 2, p, g, m, numel, blocks, c, s); break;
    default: launch_flat<8>(v >> 2, p, g, m, numel, blocks, c, s); break;
  }
  return launch_status();
}
