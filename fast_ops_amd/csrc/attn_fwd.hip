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
#include <type_traits>

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
    if (!(DBG & 4)) __syncthreads();        // everyone's pieces have landed; everyone is done reading the other buffer
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

// =====================================================================================================================
// Pipelined kernel: 8 waves x 32 query rows = 256 rows per workgroup, one workgroup per CU (two waves per SIMD, at
// most 256 VGPRs each, no AccVGPRs), K and V in four-slot LDS rings (128 KiB at D = 128) filled two tiles ahead.
// Inside a wave the work is cut into 32-key sub-tiles and software-pipelined so that the MFMA pipe and the VALU
// overlap within ONE wave instead of relying on the other wave's phase:
//     phase A(s):  S(s+1) = K Q^T  (8 MFMAs)   interleaved with   P(s) = exp2(S(s) c - m c), row sums   (VALU)
//     phase B(s):  O += V^T P(s)^T (8 MFMAs)   interleaved with   mask + row max of S(s+1)              (VALU)
// followed by the (rare) raise of the reference maximum. LDS fragments are fetched one batch (4 MFMAs) ahead through
// two register buffers, across phase and tile boundaries.
constexpr int kPipeBM = 256;
constexpr int kRing = 4;
constexpr int SG_VALU = 0x2, SG_MFMA = 0x8, SG_DS_READ = 0x100, SG_TRANS = 0x400;   // sched_group_barrier masks

// scheduling recipe for one batch: the LDS reads of the next batch first, then 4*NG x (1 MFMA, NV VALU, NT transcendental)
template <bool ON, int NG, int NDS, int NV, int NT>
__device__ __forceinline__ void sched_batch() {
  if constexpr (ON) {
    if constexpr (NDS > 0) __builtin_amdgcn_sched_group_barrier(SG_DS_READ, NDS, 0);
#pragma unroll
    for (int q = 0; q < 4 * NG; ++q) {
      __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
      if constexpr (NV > 0) __builtin_amdgcn_sched_group_barrier(SG_VALU, NV, 0);
      if constexpr (NT > 0) __builtin_amdgcn_sched_group_barrier(SG_TRANS, NT, 0);
    }
  }
  __builtin_amdgcn_sched_barrier(0);
}

template <typename T, int D, bool CAUSAL, int SCHED, int NG>
__global__ void __launch_bounds__(kPipeBM / (32 * NG) * 64) attn_fwd_pipe_kernel(const AttnParams prm) {
  constexpr int NWAVES = kPipeBM / (32 * NG);     // 8 waves x 32 rows, or 4 waves x 64 rows (two row groups per wave)
  typedef typename Ops<T>::vec8 vec8;
  constexpr int ROW_BYTES = D * 2;
  constexpr int CHUNKS = ROW_BYTES / 16;
  constexpr int TILE_BYTES = kBN * ROW_BYTES;
  constexpr int KSTEPS = D / 16;                 // MFMAs of one sub-tile's Q K^T
  constexpr int DBLK = D / 32;
  constexpr int NB = KSTEPS / 4;                 // batches (of 4 MFMAs) per phase: 2 at D = 128, 1 at D = 64
  constexpr int DMA_PER_WAVE = TILE_BYTES / 1024 / NWAVES;
  constexpr int ROWS_PER_DMA = 1024 / ROW_BYTES;
  static_assert(2 * DBLK == KSTEPS && DMA_PER_WAVE >= 1, "tile shape");

  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  FO_LDS char* smem = (FO_LDS char*)smem_raw;    // K ring (kRing tiles) | V ring (kRing tiles)
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int hh = lane >> 5;
  const int L16 = lane & 15;
  const int g16 = (lane >> 4) & 1;

  const int n_bh = prm.B * prm.H;
  int bh, qblk;
  {
    const int id = blockIdx.x;
    if ((n_bh & 7) == 0) {
      const int x = id & 7, j = id >> 3;
      bh = x + 8 * (j / prm.n_qblk);
      qblk = prm.n_qblk - 1 - (j % prm.n_qblk);
    } else {
      bh = id % n_bh;
      qblk = prm.n_qblk - 1 - id / n_bh;
    }
  }
  const int b = bh / prm.H, h = bh % prm.H;
  const int q0 = qblk * kPipeBM;
  const int q0w = q0 + wave_s * 32 * NG;
  const int Sq = prm.Sq, Sk = prm.Sk;
  const T* __restrict__ qbase = (const T*)prm.q + b * prm.qs[0] + h * prm.qs[1];
  const T* __restrict__ kbase = (const T*)prm.k + b * prm.ks[0] + h * prm.ks[1];
  const T* __restrict__ vbase = (const T*)prm.v + b * prm.vs[0] + h * prm.vs[1];

  int n_tiles, n_w;                       // tiles the workgroup walks / tiles in which this wave has unmasked keys
  if constexpr (CAUSAL) {
    n_tiles = (min(Sk, q0 + kPipeBM) + kBN - 1) / kBN;
    n_w = min(n_tiles, (q0w + 32 * NG - 1) / kBN + 1);
  } else {
    n_tiles = (Sk + kBN - 1) / kBN;
    n_w = n_tiles;
  }

  // ---- global -> LDS copies
  uint32_t k_off[DMA_PER_WAVE], v_off[DMA_PER_WAVE];
#pragma unroll
  for (int i = 0; i < DMA_PER_WAVE; ++i) {
    const int row = (wave_s * DMA_PER_WAVE + i) * ROWS_PER_DMA + lane / CHUNKS;
    const int col = ((lane % CHUNKS) ^ swz<D>(row)) * 8;
    k_off[i] = (uint32_t)(row * (int)prm.ks[2] + col) * 2u;
    v_off[i] = (uint32_t)(row * (int)prm.vs[2] + col) * 2u;
  }
  // one tile of K (ring 0) or V (ring 1) into slot tile % kRing
  auto issue = [&](const T* base, int64_t stride, const uint32_t* off, int tile, int ring) {
    const int key0 = tile * kBN;
    FO_LDS char* dst = smem + (kRing * ring + (tile & (kRing - 1))) * TILE_BYTES;
    if (key0 + kBN <= Sk) {
      const char* src = (const char*)(base + (int64_t)key0 * stride);
#pragma unroll
      for (int i = 0; i < DMA_PER_WAVE; ++i) dma16_uniform_base(src, off[i], dst + (wave_s * DMA_PER_WAVE + i) * 1024);
    } else {
      int lane_here = lane;                            // (opaque: keeps this rare path's address math inside it)
      asm volatile("" : "+v"(lane_here));
#pragma unroll
      for (int i = 0; i < DMA_PER_WAVE; ++i) {
        const int row = (wave_s * DMA_PER_WAVE + i) * ROWS_PER_DMA + lane_here / CHUNKS;
        const int col = ((lane_here % CHUNKS) ^ swz<D>(row)) * 8;
        const int key = min(key0 + row, Sk - 1);       // rows past the end re-read the last key (masked later)
        dma16_lane_ptr(base + (int64_t)key * stride + col, dst + (wave_s * DMA_PER_WAVE + i) * 1024);
      }
    }
  };
  // batch(t), issued at the top of tile t: K(t+3) and V(t+2). Returns the number of copies this lane issued.
  auto issue_batch = [&](int t) -> int {
    int n = 0;
    if (t + 3 < n_tiles && t + 3 >= 0) { issue(kbase, prm.ks[2], k_off, t + 3, 0); n += DMA_PER_WAVE; }
    if (t + 2 < n_tiles && t + 2 >= 0) { issue(vbase, prm.vs[2], v_off, t + 2, 1); n += DMA_PER_WAVE; }
    return n;
  };
  issue_batch(-3);
  issue_batch(-2);
  int last_batch = issue_batch(-1);

  // ---- Q^T fragments (B operand of S^T = K Q^T)
  vec8 qf[NG][KSTEPS];
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    const int qrow = min(q0w + 32 * g + l32, Sq - 1);
    const T* qp = qbase + (int64_t)qrow * prm.qs[2] + 8 * hh;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) qf[g][ks] = *(const vec8*)(qp + 16 * ks);
  }
#pragma unroll
  for (int g = 0; g < NG; ++g)
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) asm volatile("" ::"v"(qf[g][ks]));   // wait for Q here, never inside the loop

  f32x16 oacc[NG][DBLK];
#pragma unroll
  for (int g = 0; g < NG; ++g)
#pragma unroll
    for (int i = 0; i < DBLK; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[g][i][r] = 0.0f;
  f32x16 Sacc[NG];             // scores of the sub-tile being produced (MFMA accumulators)
  f32x16 sv[NG];               // scores of the sub-tile being consumed: copied out of Sacc, masked
  vec8 pf[NG][2];              // P of the sub-tile being multiplied with V (two 16-key steps)
  vec8 FB[2][4];               // LDS fragment batches: current and next (each fragment feeds NG MFMAs)
  float m_run[NG], l_run[NG], mloc[NG];
#pragma unroll
  for (int g = 0; g < NG; ++g) { m_run[g] = -INFINITY; l_run[g] = 0.0f; mloc[g] = -INFINITY; }
  const float c = prm.scale_log2e;

  // Held in registers for the whole kernel: 8 byte offsets for K (one per k-step) and 2 x DBLK for V^T; everything else
  // about a fragment address (ring slot, sub-tile half, 16-key step) is a wave-uniform or compile-time addend.
  uint32_t koffs[KSTEPS], voffs0[DBLK], voffs1[DBLK];
  {
    const int ksw = swz<D>(l32);
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) koffs[ks] = (uint32_t)(l32 * ROW_BYTES + (((2 * ks + hh) ^ ksw) * 16));
    const int vrow0 = 4 * hh + (L16 >> 2);
    const int vsw0 = swz<D>(vrow0), vsw1 = swz<D>(vrow0 + 8);
    const int vsub = (L16 & 1) * 8;
    const int vchunk = 2 * g16 + ((L16 & 3) >> 1);
#pragma unroll
    for (int db = 0; db < DBLK; ++db) {
      voffs0[db] = (uint32_t)(vrow0 * ROW_BYTES + vsub + (((4 * db + vchunk) ^ vsw0) * 16));
      voffs1[db] = (uint32_t)((vrow0 + 8) * ROW_BYTES + vsub + (((4 * db + vchunk) ^ vsw1) * 16));
    }
  }
  auto read_k4 = [&](vec8 (&dst)[4], FO_LDS const char* kt, int hf, int ks0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) dst[i] = *(FO_LDS const vec8*)(kt + hf * 32 * ROW_BYTES + koffs[ks0 + i]);
  };
  // four V^T fragments: batch bi of sub-tile half hf. At D = 128: t = 2*hf + bi, db = 0..3. At D = 64: t = 2*hf + i/2, db = i%2.
  auto read_v4 = [&](vec8 (&dst)[4], FO_LDS const char* vt, int hf, int bi) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int t = (DBLK == 4) ? 2 * hf + bi : 2 * hf + (i >> 1);
      const int db = (DBLK == 4) ? i : (i & 1);
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FO_LDS s16x4*)(vt + 16 * t * ROW_BYTES + voffs0[db]));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FO_LDS s16x4*)(vt + 16 * t * ROW_BYTES + voffs1[db]));
      dst[i] = __builtin_bit_cast(vec8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    }
  };
  auto k_slot = [&](int tile) -> FO_LDS const char* { return smem + (tile & (kRing - 1)) * TILE_BYTES; };
  auto v_slot = [&](int tile) -> FO_LDS const char* { return smem + (kRing + (tile & (kRing - 1))) * TILE_BYTES; };

  // ---- VALU pieces
  // exponentials of elements [e0, e1) of sv -> pf, psum
  auto exp_part = [&](const float (&mc)[NG], float (&psum)[NG], int e0, int e1) {
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
      for (int e = e0; e < e1; ++e) {
        const float x = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[g][e], c, -mc[g]));
        psum[g] += x;                              // summed in fp32 before rounding (flash_attention_triton.py:203)
        pf[g][e >> 3][e & 7] = (T)x;               // rounded to the operand type for P.V (:237)
      }
  };
  // elements [e0, e1) of the sub-tile just produced (half hf of tile): copy out of the accumulators, mask, fold into the
  // row max. The mask is applied unconditionally (two VALU operations per element, hidden behind phase B's MFMAs): a
  // branch on "this tile needs a mask" would split the straight-line block that the MFMA/VALU interleave relies on.
  // Register r holds key key_base + koff(r), koff(r) = (r & 3) + 8 * (r >> 2); it is dead iff key > q or key >= Sk,
  // i.e. iff lim + koff(r) > 0 with lim = max(key_base - q, key_base - Sk + 1).
  auto max_part = [&](int tile, int hf, int e0, int e1) {
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      const int key_base = tile * kBN + 32 * hf + 4 * hh;
      int lim = key_base - Sk + 1;
      if (CAUSAL) lim = max(lim, key_base - (q0w + 32 * g + l32));
#pragma unroll
      for (int r = e0; r < e1; ++r) sv[g][r] = (lim > -((r & 3) + 8 * (r >> 2))) ? -INFINITY : Sacc[g][r];
#pragma unroll
      for (int r = e0; r < e1; r += 2) mloc[g] = fmaxf(fmaxf(mloc[g], sv[g][r]), sv[g][r + 1]);
    }
  };
  // finish the row max, raise the reference maximum where needed (lazily), rescale O and l
  auto settle = [&]() {
    bool raise = false;
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      mloc[g] = fmaxf(mloc[g], half_swap(mloc[g]));
      raise = raise || (mloc[g] * c > m_run[g] * c + kLazyLog2);
    }
    if (__builtin_amdgcn_ballot_w64(raise) != 0) {
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const float m_new = fmaxf(m_run[g], mloc[g]);    // finite from the first sub-tile on: key 0 is never masked
        const float alpha = __builtin_amdgcn_exp2f((m_run[g] - m_new) * c);
        m_run[g] = m_new;
        l_run[g] *= alpha;
#pragma unroll
        for (int i = 0; i < DBLK; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) oacc[g][i][r] *= alpha;
      }
    }
#pragma unroll
    for (int g = 0; g < NG; ++g) mloc[g] = -INFINITY;
  };

  // ---- one full step. On entry FB[0] holds the first K batch of sub-tile (tq, hq).
  //   phase A: Sacc = K(tq, hq) Q^T       ||  P = exp2(sv c - m c)                 (sv = sub-tile (te, he), the previous one)
  //   phase B: O += V(te, he)^T P^T       ||  sv = mask(Sacc), row max
  //   then settle; on exit FB[0] holds the first K batch of the sub-tile after (tq, hq) (garbage past the end: unused).
  auto full_step = [&](int tq, int hq, int te, int he) {
    FO_LDS const char* kt = k_slot(tq);
    FO_LDS const char* vt = v_slot(te);
    FO_LDS const char* kt_next = hq ? k_slot(tq + 1) : kt;
    float mc[NG], psum[NG];
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      mc[g] = m_run[g] * c;
      psum[g] = 0.0f;
#pragma unroll
      for (int r = 0; r < 16; ++r) Sacc[g][r] = 0.0f;
    }
    // phase A
#pragma unroll
    for (int bi = 0; bi < NB; ++bi) {
      if (bi + 1 < NB) read_k4(FB[(bi + 1) & 1], kt, hq, 4 * (bi + 1));
      else read_v4(FB[(bi + 1) & 1], vt, he, 0);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int g = 0; g < NG; ++g) Sacc[g] = Ops<T>::mfma(FB[bi & 1][i], qf[g][4 * bi + i], Sacc[g]);
      exp_part(mc, psum, bi * (16 / NB), (bi + 1) * (16 / NB));
      if (bi + 1 < NB) sched_batch<SCHED != 0, NG, 4, (16 / NB) * 5 / 8 + 1, (16 / NB) / 4>();
      else sched_batch<SCHED != 0, NG, 8, (16 / NB) * 5 / 8 + 1, (16 / NB) / 4>();
    }
#pragma unroll
    for (int g = 0; g < NG; ++g) l_run[g] += psum[g];
    // phase B (fragment buffers continue to alternate: batch NB of this step sits in FB[NB & 1])
#pragma unroll
    for (int bi = 0; bi < NB; ++bi) {
      const int cur = (NB + bi) & 1;
      if (bi + 1 < NB) read_v4(FB[cur ^ 1], vt, he, bi + 1);
      else read_k4(FB[cur ^ 1], kt_next, hq ^ 1, 0);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int t = (DBLK == 4) ? bi : (i >> 1);       // 16-key step inside the sub-tile
        const int db = (DBLK == 4) ? i : (i & 1);
#pragma unroll
        for (int g = 0; g < NG; ++g) oacc[g][db] = Ops<T>::mfma(FB[cur][i], pf[g][t], oacc[g][db]);
      }
      max_part(tq, hq, bi * (16 / NB), (bi + 1) * (16 / NB));
      if (bi + 1 < NB) sched_batch<SCHED != 0, NG, 8, (16 / NB) * 5 / 8 + 1, 0>();
      else sched_batch<SCHED != 0, NG, 4, (16 / NB) * 5 / 8 + 1, 0>();
    }
    settle();
  };
  static_assert(NB == 2 || NB == 1, "fragment buffer parity below assumes one or two batches per phase");

  // ---- first sub-tile alone: Sacc = K(0, 0) Q^T, copy out, mask, max, settle; leaves the next K batch in FB[0]
  auto first_step = [&]() {
    FO_LDS const char* kt = k_slot(0);
    read_k4(FB[0], kt, 0, 0);
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
      for (int r = 0; r < 16; ++r) Sacc[g][r] = 0.0f;
#pragma unroll
    for (int bi = 0; bi < NB; ++bi) {
      if (bi + 1 < NB) read_k4(FB[(bi + 1) & 1], kt, 0, 4 * (bi + 1));
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int g = 0; g < NG; ++g) Sacc[g] = Ops<T>::mfma(FB[bi & 1][i], qf[g][4 * bi + i], Sacc[g]);
      __builtin_amdgcn_sched_barrier(0);
    }
    read_k4(FB[0], kt, 1, 0);
    max_part(0, 0, 0, 16);
    settle();
  };
  // ---- last sub-tile (te, he) of this wave alone: P = exp2(sv ...), O += V^T P^T
  auto last_step = [&](int te, int he) {
    FO_LDS const char* vt = v_slot(te);
    float mc[NG], psum[NG];
#pragma unroll
    for (int g = 0; g < NG; ++g) { mc[g] = m_run[g] * c; psum[g] = 0.0f; }
    read_v4(FB[0], vt, he, 0);
    exp_part(mc, psum, 0, 16);
#pragma unroll
    for (int g = 0; g < NG; ++g) l_run[g] += psum[g];
#pragma unroll
    for (int bi = 0; bi < NB; ++bi) {
      if (bi + 1 < NB) read_v4(FB[(bi + 1) & 1], vt, he, bi + 1);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int t = (DBLK == 4) ? bi : (i >> 1);
        const int db = (DBLK == 4) ? i : (i & 1);
#pragma unroll
        for (int g = 0; g < NG; ++g) oacc[g][db] = Ops<T>::mfma(FB[bi & 1][i], pf[g][t], oacc[g][db]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // ---- tile loop. Iteration j: [S(j,0) || P(j-1,1)] [PV(j-1,1) || max(j,0)] [S(j,1) || P(j,0)] [PV(j,0) || max(j,1)]
  // reads K(j), V(j-1), V(j). Batches up to (j-2) must have landed: K(j+1) and V(j) among them.
  for (int j = 0; j < n_tiles; ++j) {
    if (last_batch >= 2 * DMA_PER_WAVE) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * DMA_PER_WAVE) : "memory");
    else if (last_batch >= DMA_PER_WAVE) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(DMA_PER_WAVE) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    last_batch = issue_batch(j);
    if (j < n_w) {
      if (j == 0) first_step();
      else full_step(j, 0, j - 1, 1);
      full_step(j, 1, j, 0);
    } else if (j == n_w) {
      last_step(j - 1, 1);
    }
  }
  if (n_w == n_tiles) last_step(n_tiles - 1, 1);

  // ---- epilogue: normalise, write O and LSE
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    const float l_tot = l_run[g] + half_swap(l_run[g]);
    const float inv = 1.0f / l_tot;
    const int qi = q0w + 32 * g + l32;
    if (qi < Sq) {
      T* op = (T*)prm.o + b * prm.os[0] + h * prm.os[1] + (int64_t)qi * prm.os[2];
#pragma unroll
      for (int db = 0; db < DBLK; ++db)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          typedef __attribute__((ext_vector_type(4))) T vec4;
          vec4 o4;
#pragma unroll
          for (int u = 0; u < 4; ++u) o4[u] = (T)(oacc[g][db][rg * 4 + u] * inv);
          *(vec4*)(op + 32 * db + 8 * rg + 4 * hh) = o4;
        }
      if (prm.lse != nullptr && hh == 0)
        prm.lse[(int64_t)bh * Sq + qi] = (m_run[g] * c + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f;
    }
  }
}

template <typename T, int D, bool CAUSAL, int SCHED, int NG>
static int launch_pipe(AttnParams p, hipStream_t stream) {
  const size_t lds = 2 * (size_t)kRing * kBN * D * 2;
  p.n_qblk = (p.Sq + kPipeBM - 1) / kPipeBM;
  const unsigned grid = (unsigned)(p.n_qblk * p.B * p.H);
  static const hipError_t attr = hipFuncSetAttribute((const void*)attn_fwd_pipe_kernel<T, D, CAUSAL, SCHED, NG>,
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (attr != hipSuccess) return FO_ERR_LAUNCH;
  attn_fwd_pipe_kernel<T, D, CAUSAL, SCHED, NG><<<grid, kPipeBM / (32 * NG) * 64, lds, stream>>>(p);
  return launch_status();
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
  if (v == 16) return causal ? launch_pipe<T, D, true, 0, 1>(p, stream) : launch_pipe<T, D, false, 0, 1>(p, stream);
  if (v == 17) return causal ? launch_pipe<T, D, true, 1, 1>(p, stream) : launch_pipe<T, D, false, 1, 1>(p, stream);
  if (v == 18) return causal ? launch_pipe<T, D, true, 0, 2>(p, stream) : launch_pipe<T, D, false, 0, 2>(p, stream);
  if (v == 19) return causal ? launch_pipe<T, D, true, 1, 2>(p, stream) : launch_pipe<T, D, false, 1, 2>(p, stream);
  if (D == 128 && causal && sizeof(T) == 2) {
    switch (v >> 1) {
      case 1: return launch_one<T, D, true, true, 1>(p, stream);
      case 2: return launch_one<T, D, true, true, 2>(p, stream);
      case 3: return launch_one<T, D, true, true, 3>(p, stream);
      case 4: return launch_one<T, D, true, true, 5>(p, stream);
      case 5: return launch_one<T, D, true, true, 7>(p, stream);
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
