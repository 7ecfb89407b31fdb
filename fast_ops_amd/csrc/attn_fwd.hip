// FlashAttention forward for gfx950 (MI355X): O = softmax(scale * Q K^T + mask) V and LSE, fp16 / bf16 operands,
// fp32 scores and accumulators.
//
// Replaces flash_attn_fwd_kernel / flash_attn_fwd_cuda (fast_ops/flash_attention/flash_attention_fwd.cu:27-152,154-181),
// which is a skeleton; the loop structure its comments describe is kept (:37-47: queries outer and parallel over
// workgroups, keys inner; Q read once, O written once, running max and sum never leave the chip) and the numerics are
// those of the reference's Triton forward (flash_attention_triton.py:128-255): fp32 online softmax, P rounded to the
// operand type before P.V (:237), LSE = natural-log logsumexp of the scaled scores (:241-243,255), causal mask
// top-left aligned with whole key tiles skipped (:149,174-175).
//
// Design for CDNA4
//   * One workgroup = 4 waves = 128 query rows; each wave owns 32 rows. Two workgroups fit a CU (<= 256 VGPRs, 64 KiB
//     LDS each) so one's softmax (VALU) overlaps the other's MFMA.
//   * The scores are computed transposed, S^T = K Q^T (A operand = K tile from LDS, B operand = Q^T held in
//     registers for the whole kernel). In the 32x32 accumulator layout a lane then owns ONE query column and 16 of
//     the 32 keys, so the row max / row sum are in-lane reductions plus one exchange between the two half-waves,
//     and the accumulator registers are, as they stand, the B operand of O^T = V^T P^T. P never touches LDS.
//   * V^T as an A operand needs 8 keys per lane for one d: read from the row-major V tile with the gfx950
//     transposing LDS load (ds_read_b64_tr_b16).
//   * K/V tiles (64 keys) go global -> LDS with the direct-to-LDS loads (16 B per lane, no VGPR staging), double
//     buffered, one barrier per tile. 16-byte chunks are XOR-swizzled inside a row so that both the K reads
//     (32 rows x one chunk) and the V reads (4 rows x 4 chunks) are free of bank conflicts.
//   * Workgroup order: heads are dealt to the 8 XCDs (workgroup ids round-robin over XCDs), each XCD walks one head
//     at a time with its heaviest (last) causal query blocks first, so an XCD's L2 holds the K/V it is streaming.
#include "common.hpp"

namespace fo {

#define FO_LDS __attribute__((address_space(3)))
#define FO_GLOBAL __attribute__((address_space(1)))

constexpr int kWaves = 4;
constexpr int kBM = 32 * kWaves;   // query rows per workgroup
constexpr int kBN = 64;            // keys per tile

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

struct AttnParams {
  const void* q; const void* k; const void* v; void* o; float* lse;
  int B, H, Sq, Sk;
  int64_t qs[3], ks[3], vs[3], os[3];   // element strides: batch, head, sequence
  float scale_log2e;                    // softmax_scale * log2(e)
  int n_qblk;
};

__device__ __forceinline__ float half_swap(float x) {
  // value held by the lane 32 positions away
  auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(int, x), __builtin_bit_cast(int, x), false, false);
  return __builtin_bit_cast(float, (threadIdx.x & 32) ? r[0] : r[1]);
}

// 16 bytes per lane, global -> LDS without passing through registers. LDS receives the 64 lanes' pieces back to back
// starting at `dst` (wave-uniform); the global address is per lane.
// (hipcc also parses device functions in its host pass, where GCN assembly cannot be checked: the bodies exist in the
// device pass only.)
__device__ __forceinline__ void dma16_uniform_base(const void* base, uint32_t byte_off, FO_LDS void* dst) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"((uint32_t)(uintptr_t)dst), "v"(byte_off), "s"(base) : "memory", "m0");
#endif
}
__device__ __forceinline__ void dma16_lane_ptr(const void* ptr, FO_LDS void* dst) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"((uint32_t)(uintptr_t)dst), "v"(ptr) : "memory", "m0");
#endif
}

constexpr float kLazyLog2 = 8.0f;   // how far (in log2 units) a tile maximum may exceed the reference before a rescale

template <typename T, int D, bool CAUSAL, bool LAZY, int DBG>
__global__ void __launch_bounds__(kWaves * 64, 2) attn_fwd_kernel(const AttnParams prm) {
  typedef typename Ops<T>::vec8 vec8;
  constexpr int ROW_BYTES = D * 2;
  constexpr int CHUNKS = ROW_BYTES / 16;            // 16-byte chunks per row
  constexpr int TILE_BYTES = kBN * ROW_BYTES;       // one K or V tile
  constexpr int KSTEPS = D / 16;                    // MFMA k-steps of Q K^T
  constexpr int DBLK = D / 32;                      // 32-wide d blocks of O
  constexpr int DMA_PER_WAVE = TILE_BYTES / 1024 / kWaves;   // direct-to-LDS instructions per wave per tile
  constexpr int ROWS_PER_DMA = 1024 / ROW_BYTES;

  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  FO_LDS char* smem = (FO_LDS char*)smem_raw;
  // layout: K0 | K1 | V0 | V1
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);   // the same, known to the compiler as wave-uniform (DMA operands)
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int hh = lane >> 5;

  // ---- which (head, query block) this workgroup owns
  const int n_bh = prm.B * prm.H;
  int bh, qblk;
  {
    const int id = blockIdx.x;
    if ((n_bh & 7) == 0) {
      const int x = id & 7, j = id >> 3;          // XCD, position in that XCD's list
      bh = x + 8 * (j / prm.n_qblk);
      qblk = prm.n_qblk - 1 - (j % prm.n_qblk);
    } else {
      bh = id % n_bh;
      qblk = prm.n_qblk - 1 - id / n_bh;
    }
  }
  const int b = bh / prm.H, h = bh % prm.H;
  const int q0 = qblk * kBM;
  const int q0w = q0 + wave * 32;                  // first query row of this wave
  const int Sq = prm.Sq, Sk = prm.Sk;

  const T* __restrict__ qbase = (const T*)prm.q + b * prm.qs[0] + h * prm.qs[1];
  const T* __restrict__ kbase = (const T*)prm.k + b * prm.ks[0] + h * prm.ks[1];
  const T* __restrict__ vbase = (const T*)prm.v + b * prm.vs[0] + h * prm.vs[1];

  // ---- key tiles this workgroup walks
  int n_tiles;
  if constexpr (CAUSAL) {
    const int kend = min(Sk, q0 + kBM);
    n_tiles = (kend + kBN - 1) / kBN;
  } else {
    n_tiles = (Sk + kBN - 1) / kBN;
  }

  // ---- direct-to-LDS copy of one K and one V tile: per lane, DMA_PER_WAVE 16-byte pieces of each.
  // Piece i of this wave covers tile rows [(wave*DMA_PER_WAVE + i) * ROWS_PER_DMA, +ROWS_PER_DMA). LDS receives the
  // 64 lanes' pieces back to back, so the swizzle is applied by choosing which global chunk each lane fetches.
  // Per-lane byte offsets inside a tile are fixed; a tile's base pointer is wave-uniform.
  uint32_t k_off[DMA_PER_WAVE], v_off[DMA_PER_WAVE];
#pragma unroll
  for (int i = 0; i < DMA_PER_WAVE; ++i) {
    const int row = (wave_s * DMA_PER_WAVE + i) * ROWS_PER_DMA + lane / CHUNKS;
    const int col = ((lane % CHUNKS) ^ swz<D>(row)) * 8;     // logical chunk -> element offset in the row
    k_off[i] = (uint32_t)(row * (int)prm.ks[2] + col) * 2u;
    v_off[i] = (uint32_t)(row * (int)prm.vs[2] + col) * 2u;
  }
  // The copies are issued as inline assembly so that the compiler does not track them: with the builtin it makes every
  // later LDS read it cannot disambiguate wait for ALL outstanding copies (vmcnt(0) in the middle of a tile, i.e.
  // for the NEXT tile's data). Completion is awaited explicitly, once per tile, before the barrier at the loop top.
  // The loop contains no other vector-memory instruction, so no compiler-inserted vmcnt wait depends on these.
  auto issue_tile = [&](int tile, int buf) {
    const int key0 = tile * kBN;
    FO_LDS char* kdst = smem + buf * TILE_BYTES;
    FO_LDS char* vdst = smem + (2 + buf) * TILE_BYTES;
    if (key0 + kBN <= Sk) {
      const char* ktile = (const char*)(kbase + (int64_t)key0 * prm.ks[2]);
      const char* vtile = (const char*)(vbase + (int64_t)key0 * prm.vs[2]);
#pragma unroll
      for (int i = 0; i < DMA_PER_WAVE; ++i) {
        const int lds_off = (wave_s * DMA_PER_WAVE + i) * 1024;
        dma16_uniform_base(ktile, k_off[i], kdst + lds_off);
        dma16_uniform_base(vtile, v_off[i], vdst + lds_off);
      }
    } else {
      // last, partial tile: rows past the end re-read the last key (masked later). Runs at most once per workgroup;
      // the opaque copy of the lane id keeps its address arithmetic from being hoisted out of the tile loop, where
      // it would hold registers for the whole kernel.
      int lane_here = lane;
      asm volatile("" : "+v"(lane_here));
#pragma unroll
      for (int i = 0; i < DMA_PER_WAVE; ++i) {
        const int row = (wave_s * DMA_PER_WAVE + i) * ROWS_PER_DMA + lane_here / CHUNKS;
        const int col = ((lane_here % CHUNKS) ^ swz<D>(row)) * 8;
        const int key = min(key0 + row, Sk - 1);
        const int lds_off = (wave_s * DMA_PER_WAVE + i) * 1024;
        dma16_lane_ptr(kbase + (int64_t)key * prm.ks[2] + col, kdst + lds_off);
        dma16_lane_ptr(vbase + (int64_t)key * prm.vs[2] + col, vdst + lds_off);
      }
    }
  };

  issue_tile(0, 0);

  // ---- Q^T fragments (B operand): lane holds query row q0w + l32, d = 16*ks + 8*hh .. +7
  vec8 qf[KSTEPS];
  {
    const int qrow = min(q0w + l32, Sq - 1);
    const T* qp = qbase + (int64_t)qrow * prm.qs[2] + 8 * hh;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) qf[ks] = *(const vec8*)(qp + 16 * ks);
    // Consume the fragments here so that the compiler waits for these loads before the loop instead of inside it:
    // a vmcnt wait inside the loop would also wait for the direct-to-LDS copies in flight, which it does not see.
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) asm volatile("" ::"v"(qf[ks]));
  }

  f32x16 oacc[DBLK];
#pragma unroll
  for (int i = 0; i < DBLK; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[i][r] = 0.0f;
  float m_run = -INFINITY;   // reference maximum (raw, unscaled scores) of this lane's query row
  float l_run = 0.0f;        // running sum of this lane's half of the keys
  const float c = prm.scale_log2e;

  // per-lane LDS read offsets that do not depend on the tile
  //  K (ds_read_b128): row = 32*kb + l32, logical chunk = 2*ks + hh
  //  V (transposing 8-byte read): row = 16*t + 8*half + 4*hh + (lane%16)/4, d = 32*dblk + 16*((lane/16)%2) + 4*(lane%4)
  const int L16 = lane & 15;
  const int g16 = (lane >> 4) & 1;

  for (int tile = 0; tile < n_tiles; ++tile) {
    const int buf = tile & 1;
    const int key0 = tile * kBN;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this lane's pieces of tile `tile` have landed in LDS
    __syncthreads();                        // everyone's pieces have landed; everyone is done reading the other buffer
    if (tile + 1 < n_tiles && (!(DBG & 1) || tile < 1)) issue_tile(tile + 1, buf ^ 1);

    // waves whose rows are all above this tile's keys have nothing to do (causal)
    if (CAUSAL && key0 > q0w + 31) continue;

    FO_LDS const char* kt = smem + buf * TILE_BYTES;
    FO_LDS const char* vt = smem + (2 + buf) * TILE_BYTES;

    // ---- S^T = K Q^T : two 32-key blocks. K fragments are fetched from LDS one group (GK k-steps) ahead of the
    //      MFMAs that consume them, so LDS latency hides behind the previous group's matrix work.
    f32x16 sacc[2];
    {
      // a group = GK fragments = GK/2 k-steps of both key blocks; consecutive MFMAs alternate between the two
      // accumulators (a dependent MFMA issued back to back costs ~6 extra cycles on this hardware)
      constexpr int GK = 4;
      constexpr int NG = 2 * KSTEPS / GK;                   // groups per tile
      auto load_group = [&](int g, vec8* dst) {
#pragma unroll
        for (int i = 0; i < GK; ++i) {
          const int kb = i & 1, ks = g * (GK / 2) + (i >> 1);
          const int row = 32 * kb + l32;
          dst[i] = *(FO_LDS const vec8*)(kt + row * ROW_BYTES + (((2 * ks + hh) ^ swz<D>(row)) * 16));
        }
      };
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[kb][r] = 0.0f;
      vec8 fa[GK], fb[GK];
      load_group(0, fa);
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        vec8* cur = (g & 1) ? fb : fa;
        vec8* nxt = (g & 1) ? fa : fb;
        if (g + 1 < NG) load_group(g + 1, nxt);
#pragma unroll
        for (int i = 0; i < GK; ++i) sacc[i & 1] = Ops<T>::mfma(cur[i], qf[g * (GK / 2) + (i >> 1)], sacc[i & 1]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    // ---- mask: causal diagonal and keys past the end. Register r of block kb holds key
    //      key0 + 32*kb + 4*hh + koff(r), koff(r) = (r & 3) + 8 * (r >> 2); it is dead iff key > q or key >= Sk,
    //      i.e. iff lim + koff(r) > 0 with lim = max(key_base - q, key_base - Sk + 1): one compare against a constant.
    const bool need_mask = (CAUSAL && key0 + kBN - 1 > q0w) || (key0 + kBN > Sk);
    if (need_mask) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const int key_base = key0 + 32 * kb + 4 * hh;
        int lim = key_base - Sk + 1;
        if (CAUSAL) lim = max(lim, key_base - (q0w + l32));
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[kb][r] = (lim > -((r & 3) + 8 * (r >> 2))) ? -INFINITY : sacc[kb][r];
      }
    }

    // ---- online softmax (base-2 domain) with a lazily updated reference maximum.
    // exp2 is taken relative to m_run, which is only raised (and O, l rescaled) when some row's tile maximum exceeds it
    // by more than 2^kLazyLog2; until then P may reach 2^kLazyLog2 instead of 1, which fp32 accumulators and the
    // half-precision P hold without loss of relative precision. O / l and LSE = m + log(l) do not depend on the
    // reference, so the result is that of the exact recurrence (flash_attention_triton.py:200-213,241-243) up to rounding.
    float mloc = sacc[0][0];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) mloc = fmaxf(mloc, sacc[kb][r]);
    mloc = fmaxf(mloc, half_swap(mloc));
    const bool raise = LAZY ? (mloc * c > m_run * c + kLazyLog2) : (mloc > m_run);
    if (__builtin_amdgcn_ballot_w64(raise) != 0) {
      const float m_new = fmaxf(m_run, mloc);          // finite from the first tile on: key 0 is never masked
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * c);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int i = 0; i < DBLK; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] *= alpha;
    }
    const float mc = m_run * c;
    float psum = 0.0f;
    vec8 pf[4];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float p = (DBG & 2) ? sacc[kb][r] : __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][r], c, -mc));
        psum += p;                                     // summed in fp32 before rounding (flash_attention_triton.py:203)
        pf[kb * 2 + (r >> 3)][r & 7] = (T)p;           // rounded to the operand type for P.V (:237)
      }
    l_run += psum;

    // ---- O^T += V^T P^T : four 16-key steps x DBLK d-blocks, V^T fragments fetched one group ahead
    {
      constexpr int NGV = 4;                                // one group per 16-key step
      auto load_vgroup = [&](int t, s16x8* dst) {
        const int row0 = 16 * t + 4 * hh + (L16 >> 2);
        const int row1 = row0 + 8;
        const int sw0 = swz<D>(row0), sw1 = swz<D>(row1);
        const int sub = (L16 & 1) * 8;                      // byte offset inside the 16-byte chunk
#pragma unroll
        for (int db = 0; db < DBLK; ++db) {
          const int chunk = 4 * db + 2 * g16 + ((L16 & 3) >> 1);   // logical 16-byte chunk
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FO_LDS s16x4*)(vt + row0 * ROW_BYTES + ((chunk ^ sw0) * 16) + sub));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FO_LDS s16x4*)(vt + row1 * ROW_BYTES + ((chunk ^ sw1) * 16) + sub));
          dst[db] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
      };
      s16x8 va[DBLK], vb[DBLK];
      load_vgroup(0, va);
#pragma unroll
      for (int t = 0; t < NGV; ++t) {
        s16x8* cur = (t & 1) ? vb : va;
        s16x8* nxt = (t & 1) ? va : vb;
        if (t + 1 < NGV) load_vgroup(t + 1, nxt);
#pragma unroll
        for (int db = 0; db < DBLK; ++db) oacc[db] = Ops<T>::mfma(__builtin_bit_cast(vec8, cur[db]), pf[t], oacc[db]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // ---- epilogue: normalise, write O and LSE
  const float l_tot = l_run + half_swap(l_run);
  const float inv = 1.0f / l_tot;
  const int qi = q0w + l32;
  if (qi < Sq) {
    T* op = (T*)prm.o + b * prm.os[0] + h * prm.os[1] + (int64_t)qi * prm.os[2];
#pragma unroll
    for (int db = 0; db < DBLK; ++db)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        typedef __attribute__((ext_vector_type(4))) T vec4;
        vec4 o4;
#pragma unroll
        for (int j = 0; j < 4; ++j) o4[j] = (T)(oacc[db][rg * 4 + j] * inv);
        *(vec4*)(op + 32 * db + 8 * rg + 4 * hh) = o4;
      }
    if (prm.lse != nullptr && hh == 0) {
      // ln sum_j exp(scale*s_j) = ln2 * (m*scale*log2e + log2(l))
      prm.lse[(int64_t)bh * Sq + qi] = (m_run * c + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f;
    }
  }
}

template <typename T, int D, bool CAUSAL, bool LAZY, int DBG>
static int launch_one(const AttnParams& p, hipStream_t stream) {
  const size_t lds = 4 * (size_t)kBN * D * 2;
  const unsigned grid = (unsigned)(p.n_qblk * p.B * p.H);
  static const hipError_t attr = hipFuncSetAttribute((const void*)attn_fwd_kernel<T, D, CAUSAL, LAZY, DBG>,
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (attr != hipSuccess) return FO_ERR_LAUNCH;
  attn_fwd_kernel<T, D, CAUSAL, LAZY, DBG><<<grid, kWaves * 64, lds, stream>>>(p);
  return launch_status();
}

// variant bit 0: 1 = exact (eager) rescale instead of the lazy one. Variants 2..7 are timing ablations that produce
// WRONG results (bit 1: keep re-using the first tiles instead of copying new ones; bit 2: no exponentials).
template <typename T, int D>
static int launch(const AttnParams& p, bool causal, hipStream_t stream) {
  const int v = g_attn_variant < 0 ? 0 : g_attn_variant;
  if (D == 128 && causal && sizeof(T) == 2) {
    switch (v >> 1) {
      case 1: return launch_one<T, D, true, true, 1>(p, stream);
      case 2: return launch_one<T, D, true, true, 2>(p, stream);
      case 3: return launch_one<T, D, true, true, 3>(p, stream);
      default: break;
    }
  }
  const bool lazy = (v & 1) == 0;
  if (causal) return lazy ? launch_one<T, D, true, true, 0>(p, stream) : launch_one<T, D, true, false, 0>(p, stream);
  return lazy ? launch_one<T, D, false, true, 0>(p, stream) : launch_one<T, D, false, false, 0>(p, stream);
}

}  // namespace fo

using namespace fo;

extern "C" int fo_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
                           int B, int H, int Sq, int Sk, int D,
                           const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os,
                           float softmax_scale, int causal, int dtype, void* stream) {
  if (!q || !k || !v || !o || !qs || !ks || !vs || !os) return FO_ERR_NULL_POINTER;
  if (dtype != FO_DTYPE_F16 && dtype != FO_DTYPE_BF16) return FO_ERR_BAD_DTYPE;
  if (D != 64 && D != 128) return FO_ERR_BAD_HEAD_DIM;
  if (B <= 0 || H <= 0 || Sq <= 0 || Sk <= 0) return FO_ERR_BAD_SHAPE;
  const int64_t n_qblk = ((int64_t)Sq + kBM - 1) / kBM;
  if (n_qblk * B * H > 0x7FFFFFFFll || (int64_t)B * H * Sq > (1ll << 40)) return FO_ERR_BAD_SHAPE;
  const int64_t* all[4] = {qs, ks, vs, os};
  for (int t = 0; t < 4; ++t) {
    // rows start on 16-byte boundaries (8 elements); only K/V may repeat a head (stride 0 = multi-query)
    for (int i = 0; i < 3; ++i) {
      if (all[t][i] < 0 || (all[t][i] % 8) != 0) return FO_ERR_BAD_STRIDE;
    }
    if (all[t][2] < D) return FO_ERR_BAD_STRIDE;
  }
  if (os[0] == 0 && B > 1) return FO_ERR_BAD_STRIDE;
  if (os[1] == 0 && H > 1) return FO_ERR_BAD_STRIDE;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o) & 15u) return FO_ERR_MISALIGNED;
  if (lse && ((uintptr_t)lse & 3u)) return FO_ERR_MISALIGNED;
  if (!(softmax_scale > 0.0f) || softmax_scale > 3.0e38f) return FO_ERR_BAD_SHAPE;   // also rejects NaN

  AttnParams p;
  p.q = q; p.k = k; p.v = v; p.o = o; p.lse = lse;
  p.B = B; p.H = H; p.Sq = Sq; p.Sk = Sk;
  for (int i = 0; i < 3; ++i) { p.qs[i] = qs[i]; p.ks[i] = ks[i]; p.vs[i] = vs[i]; p.os[i] = os[i]; }
  p.scale_log2e = softmax_scale * 1.4426950408889634f;
  p.n_qblk = (int)n_qblk;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == FO_DTYPE_BF16) return D == 128 ? launch<__bf16, 128>(p, causal != 0, s) : launch<__bf16, 64>(p, causal != 0, s);
  return D == 128 ? launch<_Float16, 128>(p, causal != 0, s) : launch<_Float16, 64>(p, causal != 0, s);
}
