// Fused Lion step for every combination of parameter/gradient dtype P and momentum dtype M in {fp32, fp16, bf16}.
//
// Covers what lion.hip (fp32 parameters + bf16 momentum, the tuned path) does not: the reference kernel's own case,
// all three tensors in one half type (fast_ops/lion/lion_update.cu:132-141), and fp32 or fp16 momenta. The arithmetic
// is, for every combination, that of the reference formula (fast_ops/lion/lion_optimizer_ref.py:51,64,65,67) under
// PyTorch's type promotion: every tensor-valued intermediate is computed in fp32 and rounded to the dtype the
// corresponding torch expression has,
//     p1 = rP(p * c_wd)                                  :51   p.mul_(1 - lr*wd)
//     t1 = rM(m * c_b1),  t2 = rP(g * c_1b1)             :64   exp_avg * beta1, grad * (1 - beta1)
//     u  = rR(t1 + t2),   R = P if P == M else fp32      :64
//     p2 = rP(p1 + c_nlr * sign(u))                      :65   sign(0) = sign(NaN) = 0
//     m2 = rM(fma(c_1b2, g, rM(m * c_b2)))               :67   mul_ then add_(grad, alpha)
// with the six constants prepared by fo_lion_make_consts_typed (when P == M is a half type, torch rounds the `alpha`
// of its two add_ calls, -lr and 1 - beta2, to that type first). The reference CUDA kernel itself rounds after every
// operation in the half type and uses sign(0) = -1 (lion_update.cu:10-13,38-41); the reference's test accepts either
// within 1e-2 (tests/test_lion_optimizer.py:44-51), and this library follows the formula, which is the oracle.
//
// Compiled with -ffp-contract=off: the only fused multiply-add is the explicit one.
//
// Launch shape as in lion.hip: one 64-lane workgroup per piece of 64 x VEC elements, VEC = 16 bytes of the parameter
// type per lane, streaming loads and stores.
#include <type_traits>

#include "common.hpp"

namespace fo {

struct LionCT { float c_wd, c_b1, c_1b1, c_nlr, c_b2, c_1b2; };

#define FO_GLOBAL __attribute__((address_space(1)))

template <typename T> __device__ __forceinline__ float to_f32(T x) { return static_cast<float>(x); }
// fp32 -> storage type. The empty statement makes the fp32 value opaque to the compiler: it would otherwise merge the
// multiply (or fused multiply-add) that produced it with the conversion into one mixed-precision instruction
// (v_fma_mixlo_f16), which rounds the exact result once instead of to fp32 first and then to fp16, and so differs from
// the two-step rounding of the formula whenever the fp32 value sits exactly between two fp16 values.
template <typename T> __device__ __forceinline__ T to_storage(float x) {
  if constexpr (std::is_same<T, float>::value) return x;
  else {
    asm volatile("" : "+v"(x));
    return static_cast<T>(x);
  }
}
// round to the storage type and come back: the value a torch tensor of that dtype would hold
template <typename T> __device__ __forceinline__ float rnd(float x) { return static_cast<float>(to_storage<T>(x)); }

template <typename P, typename M>
__device__ __forceinline__ void lion_elem_typed(P& p_io, P g_in, M& m_io, const LionCT& c) {
  typedef typename std::conditional<std::is_same<P, M>::value, P, float>::type R;
  const float p = to_f32(p_io), g = to_f32(g_in), m = to_f32(m_io);
  const float p1 = rnd<P>(p * c.c_wd);
  const float t1 = rnd<M>(m * c.c_b1);
  const float t2 = rnd<P>(g * c.c_1b1);
  const float u = rnd<R>(t1 + t2);
  const float s = (u > 0.0f) ? 1.0f : ((u < 0.0f) ? -1.0f : 0.0f);
  p_io = to_storage<P>(p1 + c.c_nlr * s);                // the product is exact: one fp32 rounding, then the storage type
  const float m1 = rnd<M>(m * c.c_b2);
  m_io = to_storage<M>(__builtin_fmaf(c.c_1b2, g, m1));
}

template <typename T, int N> struct VecOf { typedef __attribute__((ext_vector_type(N))) T type; };

// one piece of n <= 64 * VEC elements by one 64-lane workgroup
template <typename P, typename M>
__device__ __forceinline__ void lion_piece_typed(P* __restrict__ p_, const P* __restrict__ g_, M* __restrict__ m_, const int n,
                                                 const LionCT& c) {
  constexpr int VEC = 16 / sizeof(P);
  constexpr int PIECE = 64 * VEC;
  typedef typename VecOf<P, VEC>::type pvec;
  typedef typename VecOf<M, VEC>::type mvec;
  FO_GLOBAL P* p = (FO_GLOBAL P*)p_;
  const FO_GLOBAL P* g = (const FO_GLOBAL P*)g_;
  FO_GLOBAL M* m = (FO_GLOBAL M*)m_;
  const int t = threadIdx.x;
  const bool aligned = ((reinterpret_cast<uintptr_t>(p_) | reinterpret_cast<uintptr_t>(g_)) & 15u) == 0 &&
                       (reinterpret_cast<uintptr_t>(m_) & (sizeof(mvec) - 1)) == 0;
  if (aligned && n == PIECE) {
    pvec pv = __builtin_nontemporal_load((const FO_GLOBAL pvec*)p + t);
    const pvec gv = __builtin_nontemporal_load((const FO_GLOBAL pvec*)g + t);
    mvec mv = __builtin_nontemporal_load((const FO_GLOBAL mvec*)m + t);
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      P pe = pv[i];
      M me = mv[i];
      lion_elem_typed<P, M>(pe, gv[i], me, c);
      pv[i] = pe;
      mv[i] = me;
    }
    __builtin_nontemporal_store(pv, (FO_GLOBAL pvec*)p + t);
    __builtin_nontemporal_store(mv, (FO_GLOBAL mvec*)m + t);
    return;
  }
  // a tensor's tail, or a view whose offset breaks vector alignment: element by element
  for (int e = t; e < n; e += 64) {
    P pe = p[e];
    M me = m[e];
    lion_elem_typed<P, M>(pe, g[e], me, c);
    p[e] = pe;
    m[e] = me;
  }
}

// the chunk descriptor of fastops.h with untyped pointers (same layout)
struct ChunkAny { void* p; const void* g; void* m; int32_t n; int32_t reserved; };
static_assert(sizeof(ChunkAny) == sizeof(fo_lion_chunk), "descriptor layout");

template <typename P, typename M>
__global__ void __launch_bounds__(64) lion_chunks_typed_kernel(const ChunkAny* __restrict__ chunks, LionCT c) {
  constexpr int PIECE = 64 * (16 / (int)sizeof(P));
  constexpr int PER_CHUNK = FO_LION_CHUNK / PIECE;
  const ChunkAny ch = chunks[blockIdx.x / PER_CHUNK];
  const int off = (blockIdx.x % PER_CHUNK) * PIECE;
  const int left = ch.n - off;
  if (left <= 0) return;
  lion_piece_typed<P, M>((P*)ch.p + off, (const P*)ch.g + off, (M*)ch.m + off, left < PIECE ? left : PIECE, c);
}

template <typename P, typename M>
__global__ void __launch_bounds__(64) lion_flat_typed_kernel(P* __restrict__ p, const P* __restrict__ g, M* __restrict__ m,
                                                             int64_t numel, LionCT c) {
  constexpr int PIECE = 64 * (16 / (int)sizeof(P));
  const int64_t base = static_cast<int64_t>(blockIdx.x) * PIECE;
  const int64_t left = numel - base;
  lion_piece_typed<P, M>(p + base, g + base, m + base, left < PIECE ? static_cast<int>(left) : PIECE, c);
}

template <typename P, typename M>
static int launch_typed(const void* chunks, int64_t n_chunks, void* p, const void* g, void* m, int64_t numel, LionCT c, hipStream_t s) {
  constexpr int PIECE = 64 * (16 / (int)sizeof(P));
  const int64_t blocks64 = chunks ? n_chunks * (FO_LION_CHUNK / PIECE) : (numel + PIECE - 1) / PIECE;
  if (blocks64 > 0x7FFFFFFFll) return FO_ERR_BAD_SHAPE;
  const unsigned blocks = static_cast<unsigned>(blocks64);
  if (chunks) lion_chunks_typed_kernel<P, M><<<blocks, 64, 0, s>>>((const ChunkAny*)chunks, c);
  else lion_flat_typed_kernel<P, M><<<blocks, 64, 0, s>>>((P*)p, (const P*)g, (M*)m, numel, c);
  return launch_status();
}

template <typename P>
static int dispatch_m(int m_dtype, const void* chunks, int64_t n_chunks, void* p, const void* g, void* m, int64_t numel, LionCT c,
                      hipStream_t s) {
  switch (m_dtype) {
    case FO_DTYPE_F32: return launch_typed<P, float>(chunks, n_chunks, p, g, m, numel, c, s);
    case FO_DTYPE_F16: return launch_typed<P, _Float16>(chunks, n_chunks, p, g, m, numel, c, s);
    case FO_DTYPE_BF16: return launch_typed<P, __bf16>(chunks, n_chunks, p, g, m, numel, c, s);
    default: return FO_ERR_BAD_DTYPE;
  }
}

static int dispatch(int p_dtype, int m_dtype, const void* chunks, int64_t n_chunks, void* p, const void* g, void* m, int64_t numel,
                    const fo_lion_consts* k, hipStream_t s) {
  const LionCT c{k->c_wd, k->c_b1, k->c_1b1, k->c_nlr, k->c_b2, k->c_1b2};
  switch (p_dtype) {
    case FO_DTYPE_F32: return dispatch_m<float>(m_dtype, chunks, n_chunks, p, g, m, numel, c, s);
    case FO_DTYPE_F16: return dispatch_m<_Float16>(m_dtype, chunks, n_chunks, p, g, m, numel, c, s);
    case FO_DTYPE_BF16: return dispatch_m<__bf16>(m_dtype, chunks, n_chunks, p, g, m, numel, c, s);
    default: return FO_ERR_BAD_DTYPE;
  }
}

static int elem_size(int dtype) { return dtype == FO_DTYPE_F32 ? 4 : ((dtype == FO_DTYPE_F16 || dtype == FO_DTYPE_BF16) ? 2 : 0); }

// fp32 -> half type -> fp32 on the host, round-to-nearest-even (what static_cast<c10::Half / c10::BFloat16>(float) does)
static float host_round(float x, int dtype) {
  if (dtype == FO_DTYPE_F16) return static_cast<float>(static_cast<_Float16>(x));
  if (dtype == FO_DTYPE_BF16) {
    uint32_t u;
    __builtin_memcpy(&u, &x, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return x;
    u = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
    __builtin_memcpy(&x, &u, 4);
  }
  return x;
}

}  // namespace fo

using namespace fo;

extern "C" int fo_lion_make_consts_typed(double lr, double beta1, double beta2, double weight_decay, int p_dtype, int m_dtype,
                                         fo_lion_consts* out) {
  if (!out) return FO_ERR_NULL_POINTER;
  if (!elem_size(p_dtype) || !elem_size(m_dtype)) return FO_ERR_BAD_DTYPE;
  const int rc = fo_lion_make_consts(lr, beta1, beta2, weight_decay, out);
  if (rc != FO_OK) return rc;
  if (p_dtype == m_dtype && p_dtype != FO_DTYPE_F32) {
    // add_(other, alpha) between two tensors of one half type: torch converts alpha to that type first
    out->c_nlr = host_round(out->c_nlr, p_dtype);
    out->c_1b2 = host_round(out->c_1b2, p_dtype);
  }
  return FO_OK;
}

extern "C" int64_t fo_lion_fill_chunks_typed(void* p, const void* g, void* m, int64_t numel, int p_dtype, int m_dtype, fo_lion_chunk* out) {
  const int ps = elem_size(p_dtype), ms = elem_size(m_dtype);
  if (numel <= 0 || !ps || !ms) return 0;
  const int64_t n = (numel + FO_LION_CHUNK - 1) / FO_LION_CHUNK;
  if (!out) return n;
  ChunkAny* o = reinterpret_cast<ChunkAny*>(out);
  for (int64_t i = 0; i < n; ++i) {
    const int64_t off = i * FO_LION_CHUNK;
    const int64_t left = numel - off;
    o[i].p = static_cast<char*>(p) + off * ps;
    o[i].g = static_cast<const char*>(g) + off * ps;
    o[i].m = static_cast<char*>(m) + off * ms;
    o[i].n = static_cast<int32_t>(left < FO_LION_CHUNK ? left : FO_LION_CHUNK);
    o[i].reserved = 0;
  }
  return n;
}

extern "C" int fo_lion_step_typed(const fo_lion_chunk* chunks_dev, int64_t n_chunks, int p_dtype, int m_dtype,
                                  const fo_lion_consts* consts, void* stream) {
  if (!consts) return FO_ERR_NULL_POINTER;
  if (!elem_size(p_dtype) || !elem_size(m_dtype)) return FO_ERR_BAD_DTYPE;
  if (n_chunks < 0 || n_chunks > (0x7FFFFFFFll / 64)) return FO_ERR_BAD_SHAPE;
  if (n_chunks == 0) return FO_OK;
  if (!chunks_dev) return FO_ERR_NULL_POINTER;
  if (reinterpret_cast<uintptr_t>(chunks_dev) & 7u) return FO_ERR_MISALIGNED;
  if (p_dtype == FO_DTYPE_F32 && m_dtype == FO_DTYPE_BF16) return fo_lion_step(chunks_dev, n_chunks, consts, stream);
  return dispatch(p_dtype, m_dtype, chunks_dev, n_chunks, nullptr, nullptr, nullptr, 0, consts, static_cast<hipStream_t>(stream));
}

extern "C" int fo_lion_update_typed(void* p, const void* g, void* m, int64_t numel, int p_dtype, int m_dtype,
                                    const fo_lion_consts* consts, void* stream) {
  if (!consts) return FO_ERR_NULL_POINTER;
  const int ps = elem_size(p_dtype), ms = elem_size(m_dtype);
  if (!ps || !ms) return FO_ERR_BAD_DTYPE;
  if (numel < 0) return FO_ERR_BAD_SHAPE;
  if (numel == 0) return FO_OK;
  if (!p || !g || !m) return FO_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(p) & (ps - 1)) || (reinterpret_cast<uintptr_t>(g) & (ps - 1)) || (reinterpret_cast<uintptr_t>(m) & (ms - 1)))
    return FO_ERR_MISALIGNED;
  if (p_dtype == FO_DTYPE_F32 && m_dtype == FO_DTYPE_BF16)
    return fo_lion_update(static_cast<float*>(p), static_cast<const float*>(g), static_cast<uint16_t*>(m), numel, consts, stream);
  return dispatch(p_dtype, m_dtype, nullptr, 0, p, g, m, numel, consts, static_cast<hipStream_t>(stream));
}
