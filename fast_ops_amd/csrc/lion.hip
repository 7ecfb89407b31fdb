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
// Launch shape: measured on MI355X, HBM sustains the mixed read/write stream best when the work is cut very fine:
// one 64-lane workgroup per 256 elements (each lane: 16 B of p, 16 B of g, 8 B of m, then the two stores), so that
// the workgroups in flight at any moment cover one compact, advancing window of each array. Larger per-workgroup
// pieces or persistent grid-stride loops lose 10-25 % of bandwidth. Streaming (non-temporal) loads and stores keep
// the single-use data from churning L2.
#include "common.hpp"

namespace fo {

struct LionC { float c_wd, c_b1, c_1b1, c_nlr, c_b2, c_1b2; };

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

// fp32 pair -> packed bf16 pair (low half = first), round-to-nearest-even, in one v_cvt_pk_bf16_f32. For every
// non-NaN fp32 bit pattern (all 2^32 were compared on the device) this equals c10::BFloat16's integer rounding,
// ((u + 0x7FFF + ((u >> 16) & 1)) >> 16), denormals, ties and infinities included. A NaN stays a quiet NaN; its payload
// bits are unspecified (torch's own conversions disagree there: 0x7FC0 in the scalar path, 0xFFFF in the vector path).
__device__ __forceinline__ uint32_t bf16x2_rne(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){a, b}, bf16x2));
}
__device__ __forceinline__ float bf16_lo_f32(uint32_t packed) { return __builtin_bit_cast(float, packed << 16); }
__device__ __forceinline__ float bf16_hi_f32(uint32_t packed) { return __builtin_bit_cast(float, packed & 0xFFFF0000u); }

// parameter part of one element: decay, then step by -lr * sign(u)
__device__ __forceinline__ float lion_param(float p, float t1, float g, const LionC& c) {
  const float p1 = p * c.c_wd;                                       // ref :51
  const float t2 = g * c.c_1b1;                                      // ref :64
  const float u = t1 + t2;                                           // ref :64 (t1 = bf16(m * beta1) as fp32)
  const float s = (u > 0.0f) ? 1.0f : ((u < 0.0f) ? -1.0f : 0.0f);   // ref :65 torch.sign: 0 for zero and for NaN
  return p1 + c.c_nlr * s;                                           // ref :65 (the product is exact)
}

// two neighbouring elements whose momenta share one 32-bit word
__device__ __forceinline__ void lion_pair(float& p0, float& p1, float g0, float g1, uint32_t& mm, const LionC& c) {
  const float m0 = bf16_lo_f32(mm), m1 = bf16_hi_f32(mm);
  const uint32_t t = bf16x2_rne(m0 * c.c_b1, m1 * c.c_b1);           // ref :64 exp_avg * beta1 is a bf16 tensor
  p0 = lion_param(p0, bf16_lo_f32(t), g0, c);
  p1 = lion_param(p1, bf16_hi_f32(t), g1, c);
  const uint32_t d = bf16x2_rne(m0 * c.c_b2, m1 * c.c_b2);           // ref :67 mul_ rounds to bf16
  mm = bf16x2_rne(__builtin_fmaf(c.c_1b2, g0, bf16_lo_f32(d)),       // ref :67 add_(grad, alpha) is one fused
                  __builtin_fmaf(c.c_1b2, g1, bf16_hi_f32(d)));      //         multiply-add, then rounds to bf16
}

// one element on its own (tails and unaligned tensors); same arithmetic as lion_pair
__device__ __forceinline__ float lion_elem(float p, float g, uint32_t mbits, const LionC& c, uint32_t& mout) {
  float p0 = p, p1 = 0.0f;
  uint32_t mm = mbits & 0xFFFFu;
  lion_pair(p0, p1, g, 0.0f, mm, c);
  mout = mm & 0xFFFFu;
  return p0;
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
// Streaming stores are written as inline assembly: with __builtin_nontemporal_store the compiler dropped the `nt`
// modifier on the scalar-base form of the store it selects for the main path, which costs ~15 % of bandwidth here.
// The compiler's hazard recogniser does not look inside inline assembly, so the wait states that gfx940-class
// hardware needs between a store of more than 64 bits and a VALU write to its data registers are spelled out.
template <bool NT>
__device__ __forceinline__ void st(FO_GLOBAL f32x4* p, f32x4 v) {
  if constexpr (NT) asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 2" ::"v"(p), "v"(v) : "memory");
  else *p = v;
}
template <bool NT>
__device__ __forceinline__ void st(FO_GLOBAL u32x2* p, u32x2 v) {
  if constexpr (NT) asm volatile("global_store_dwordx2 %0, %1, off nt" ::"v"(p), "v"(v) : "memory");
  else *p = v;
}

constexpr int kVec = 4;   // elements per lane per access (16 B of p and g, 8 B of m)

// four elements held by one lane: p/g as a 16-byte vector, m as two packed bf16 pairs
__device__ __forceinline__ void lion_vec4(const f32x4& pr, const f32x4& gr, const u32x2& mr, const LionC& c, f32x4& po, u32x2& mo) {
  po = pr;
  mo = mr;
  float a0 = po[0], a1 = po[1], a2 = po[2], a3 = po[3];
  uint32_t m01 = mo[0], m23 = mo[1];
  lion_pair(a0, a1, gr[0], gr[1], m01, c);
  lion_pair(a2, a3, gr[2], gr[3], m23, c);
  po[0] = a0; po[1] = a1; po[2] = a2; po[3] = a3;
  mo[0] = m01; mo[1] = m23;
}

// One piece of n <= THREADS*4*UNROLL elements, processed by a whole workgroup of THREADS lanes.
// UNROLL = how many (THREADS*4)-element rows are loaded before the first is consumed.
template <int THREADS, int UNROLL, bool NT_LD, bool NT_ST>
__device__ __forceinline__ void lion_piece(float* __restrict__ p_, const float* __restrict__ g_, uint16_t* __restrict__ m_,
                                           const int n, const LionC& c) {
  constexpr int PIECE = THREADS * kVec * UNROLL;
  FO_GLOBAL float* p = as_global(p_);
  const FO_GLOBAL float* g = as_global(g_);
  FO_GLOBAL uint16_t* m = as_global(m_);
  const int t = threadIdx.x;
  const bool aligned = ((reinterpret_cast<uintptr_t>(p_) | reinterpret_cast<uintptr_t>(g_)) & 15u) == 0 &&
                       (reinterpret_cast<uintptr_t>(m_) & 7u) == 0;
  if (!aligned) {
    // a view into a larger buffer whose offset breaks vector alignment: element-wise
    for (int e = t; e < n; e += THREADS) {
      uint32_t o;
      p[e] = lion_elem(p[e], g[e], m[e], c, o);
      m[e] = static_cast<uint16_t>(o);
    }
    return;
  }
  FO_GLOBAL f32x4* pv = (FO_GLOBAL f32x4*)p;
  const FO_GLOBAL f32x4* gv = (const FO_GLOBAL f32x4*)g;
  FO_GLOBAL u32x2* mv = (FO_GLOBAL u32x2*)m;
  if (n == PIECE) {
    f32x4 pr[UNROLL], gr[UNROLL];
    u32x2 mr[UNROLL];
#pragma unroll
    for (int j = 0; j < UNROLL; ++j) {
      const int idx = j * THREADS + t;
      pr[j] = ld<NT_LD>(pv + idx);
      gr[j] = ld<NT_LD>(gv + idx);
      mr[j] = ld<NT_LD>(mv + idx);
    }
#pragma unroll
    for (int j = 0; j < UNROLL; ++j) {
      const int idx = j * THREADS + t;
      f32x4 po;
      u32x2 mo;
      lion_vec4(pr[j], gr[j], mr[j], c, po, mo);
      st<NT_ST>(pv + idx, po);
      st<NT_ST>(mv + idx, mo);
    }
    return;
  }
  // short piece (a tensor's tail): whole vectors, then up to 3 single elements
  const int nvec = n / kVec;
  for (int idx = t; idx < nvec; idx += THREADS) {
    f32x4 po;
    u32x2 mo;
    const f32x4 pr = ld<NT_LD>(pv + idx), gr = ld<NT_LD>(gv + idx);
    const u32x2 mr = ld<NT_LD>(mv + idx);
    lion_vec4(pr, gr, mr, c, po, mo);
    st<NT_ST>(pv + idx, po);
    st<NT_ST>(mv + idx, mo);
  }
  const int e = nvec * kVec + t;
  if (e < n) {
    uint32_t o;
    p[e] = lion_elem(p[e], g[e], m[e], c, o);
    m[e] = static_cast<uint16_t>(o);
  }
}

// many tensors: a chunk descriptor covers up to FO_LION_CHUNK elements and is shared by FO_LION_CHUNK / PIECE
// consecutive workgroups, each of which processes one piece of it
template <int THREADS, int UNROLL, bool NT_LD, bool NT_ST>
__global__ void __launch_bounds__(THREADS) lion_chunks_kernel(const fo_lion_chunk* __restrict__ chunks, LionC c) {
  constexpr int PIECE = THREADS * kVec * UNROLL;
  constexpr int PER_CHUNK = FO_LION_CHUNK / PIECE;
  static_assert(FO_LION_CHUNK % PIECE == 0, "a chunk must be a whole number of pieces");
  const fo_lion_chunk ch = chunks[blockIdx.x / PER_CHUNK];
  const int off = (blockIdx.x % PER_CHUNK) * PIECE;
  const int left = ch.n - off;
  if (left <= 0) return;
  lion_piece<THREADS, UNROLL, NT_LD, NT_ST>(ch.p + off, ch.g + off, ch.m + off, left < PIECE ? left : PIECE, c);
}

// one tensor, no descriptor table: workgroup b covers elements [b*PIECE, (b+1)*PIECE)
template <int THREADS, int UNROLL, bool NT_LD, bool NT_ST>
__global__ void __launch_bounds__(THREADS) lion_flat_kernel(float* __restrict__ p, const float* __restrict__ g,
                                                            uint16_t* __restrict__ m, int64_t numel, LionC c) {
  constexpr int PIECE = THREADS * kVec * UNROLL;
  const int64_t base = static_cast<int64_t>(blockIdx.x) * PIECE;
  const int64_t left = numel - base;
  lion_piece<THREADS, UNROLL, NT_LD, NT_ST>(p + base, g + base, m + base, left < PIECE ? static_cast<int>(left) : PIECE, c);
}

static LionC to_c(const fo_lion_consts* k) { return LionC{k->c_wd, k->c_b1, k->c_1b1, k->c_nlr, k->c_b2, k->c_1b2}; }

// Launch shapes selectable through fo_tune_set("lion.variant", v): v = shape + 8 * (plain loads) + 16 * (plain stores)
// shapes (lanes per workgroup, rows per lane): 0 {64,1} 1 {64,2} 2 {128,1} 3 {256,1} 4 {256,2} 5 {256,8} 6 {512,1} 7 {1024,1}
constexpr int kLionDefaultVariant = 0;
constexpr int kLionVariants = 32;

template <int THREADS, int UNROLL>
static int launch_shape(int plain, const fo_lion_chunk* chunks, int64_t n_chunks, float* p, const float* g, uint16_t* m,
                        int64_t numel, LionC c, hipStream_t s) {
  constexpr int PIECE = THREADS * kVec * UNROLL;
  const int64_t blocks64 = chunks ? n_chunks * (FO_LION_CHUNK / PIECE) : (numel + PIECE - 1) / PIECE;
  if (blocks64 > 0x7FFFFFFFll) return FO_ERR_BAD_SHAPE;
  const unsigned blocks = static_cast<unsigned>(blocks64);
#define FO_LAUNCH(NTL, NTS)                                                                            \
  if (chunks) lion_chunks_kernel<THREADS, UNROLL, NTL, NTS><<<blocks, THREADS, 0, s>>>(chunks, c);     \
  else lion_flat_kernel<THREADS, UNROLL, NTL, NTS><<<blocks, THREADS, 0, s>>>(p, g, m, numel, c);
  switch (plain) {
    case 0: FO_LAUNCH(true, true) break;
    case 1: FO_LAUNCH(false, true) break;
    case 2: FO_LAUNCH(true, false) break;
    default: FO_LAUNCH(false, false) break;
  }
#undef FO_LAUNCH
  return launch_status();
}

static int launch_variant(int v, const fo_lion_chunk* chunks, int64_t n_chunks, float* p, const float* g, uint16_t* m,
                          int64_t numel, LionC c, hipStream_t s) {
  const int plain = (v >> 3) & 3;
  switch (v & 7) {
    case 0: return launch_shape<64, 1>(plain, chunks, n_chunks, p, g, m, numel, c, s);
    case 1: return launch_shape<64, 2>(plain, chunks, n_chunks, p, g, m, numel, c, s);
    case 2: return launch_shape<128, 1>(plain, chunks, n_chunks, p, g, m, numel, c, s);
    case 3: return launch_shape<256, 1>(plain, chunks, n_chunks, p, g, m, numel, c, s);
    case 4: return launch_shape<256, 2>(plain, chunks, n_chunks, p, g, m, numel, c, s);
    case 5: return launch_shape<256, 8>(plain, chunks, n_chunks, p, g, m, numel, c, s);
    case 6: return launch_shape<512, 1>(plain, chunks, n_chunks, p, g, m, numel, c, s);
    default: return launch_shape<1024, 1>(plain, chunks, n_chunks, p, g, m, numel, c, s);
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
  if (n_chunks < 0 || n_chunks > (0x7FFFFFFFll / 64)) return FO_ERR_BAD_SHAPE;
  if (n_chunks == 0) return FO_OK;
  if (!chunks_dev) return FO_ERR_NULL_POINTER;
  if (reinterpret_cast<uintptr_t>(chunks_dev) & 7u) return FO_ERR_MISALIGNED;
  const int tv = tune(g_lion_variant);
  const int v = (tv < 0 || tv >= kLionVariants) ? kLionDefaultVariant : tv;
  return launch_variant(v, chunks_dev, n_chunks, nullptr, nullptr, nullptr, 0, to_c(consts), static_cast<hipStream_t>(stream));
}

extern "C" int fo_lion_update(float* p, const float* g, uint16_t* m, int64_t numel, const fo_lion_consts* consts, void* stream) {
  if (!consts) return FO_ERR_NULL_POINTER;
  if (numel < 0) return FO_ERR_BAD_SHAPE;
  if (numel == 0) return FO_OK;
  if (!p || !g || !m) return FO_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(p) & 3u) || (reinterpret_cast<uintptr_t>(g) & 3u) || (reinterpret_cast<uintptr_t>(m) & 1u))
    return FO_ERR_MISALIGNED;
  const int tv = tune(g_lion_variant);
  const int v = (tv < 0 || tv >= kLionVariants) ? kLionDefaultVariant : tv;
  return launch_variant(v, nullptr, 0, p, g, m, numel, to_c(consts), static_cast<hipStream_t>(stream));
}
