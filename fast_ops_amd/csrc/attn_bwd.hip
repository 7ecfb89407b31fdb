// FlashAttention backward for gfx950 (MI355X): dQ, dK, dV from Q, K, V, O, dO and the forward's logsumexp.
//
// Replaces the backward the reference leaves unimplemented behind its CUDA forward (fast_ops/flash_attention/
// flash_attention.py:40-45) with what its Triton backward computes (flash_attention_triton.py:273-315 delta pre-pass,
// :322-638 kernel, :832-958 host): with P = exp(scale * Q K^T - LSE) (masked entries 0),
//     delta_i = sum_d dO_id O_id      dV = P^T dO      dP = dO V^T      dS = P * (dP - delta) * scale
//     dQ = dS K                       dK = dS^T Q
// fp32 scores and accumulators; P and dS are rounded to the operand type before the second GEMMs, as the reference
// does (:515,:562-563).
//
// Two launches, no atomics, no scratch beyond the caller's [2, B, H, Sq] fp32 workspace (delta and -LSE / scale):
//   1. attn_bwd_dq_kernel: one workgroup per 128 query rows (4 waves x 32), walks the key tiles like the forward
//      kernel. Scores are computed transposed, S^T = K Q^T and dP^T = V dO^T (A operands = K / V rows from LDS, B
//      operands = Q^T / dO^T held in registers), so a lane owns one query: LSE and delta are per-lane scalars and
//      dS^T is, as it stands, the B operand of dQ^T = K^T dS^T (A operand via the transposing LDS read of the K tile).
//      It also computes delta (negated) from the dO fragments it holds and the same pieces of O, and stores it.
//   2. attn_bwd_dkdv_kernel: one workgroup per 128 keys (4 waves x 32), walks the query tiles. Here the scores are
//      computed untransposed, S = Q K^T and dP = dO V^T (A operands = Q / dO rows from LDS, B operands = K^T / V^T
//      held in registers), so a lane owns one key and P, dS are the B operands of dV^T = dO^T P and dK^T = Q^T dS
//      (A operands via the transposing LDS read of the dO and Q tiles); per-row LSE and delta come from LDS.
//      Without dropout and bias this runs as attn_bwd_dkdv_pipe_kernel, the same computation laid out by hand as a
//      software pipeline (described there); attn_bwd_dkdv_kernel is the plain, compiler-scheduled form.
// Both recompute the scores (seven GEMMs in total instead of the five of an atomics-based single pass). softmax_scale
// is applied once to the finished dQ and dK accumulators rather than to every dS.
// Tiles of 64 rows go global -> LDS with the direct-to-LDS loads, double buffered (three buffers in the pipelined
// kernel), one barrier per tile, 16-byte chunks XOR-swizzled inside a row (no bank conflicts), exactly as in the
// 128-row forward kernel.
#include <type_traits>

#include <mutex>

#include "attn_common.hpp"

namespace fo {

constexpr int kBwdWaves = 4;
constexpr int kBwdRows = 32 * kBwdWaves;   // rows (queries or keys) owned by a workgroup
constexpr int kBwdTile = 64;               // rows of a streamed tile

struct AttnBwdParams {
  const void *q, *k, *v, *o, *d_o;
  const float* lse;
  float* delta;
  float* nlse;        // [B, H, Sq]: -LSE / softmax_scale, written by the dQ kernel beside delta (see there)
  void *dq, *dk, *dv;
  int B, H, Sq, Sk;
  int d;                // true head_dim: a multiple of 8, at most the D the kernels are compiled for
  int64_t qs[3], ks[3], vs[3], os[3], dos[3], dqs[3], dks[3], dvs[3];   // element strides: batch, head, sequence
  float scale, scale_log2e, neg_inv_scale_log2e;   // softmax scale, scale * log2 e, -1 / (scale * log2 e)
  int head_group;       // heads per group in the order of the workgroups (see bwd_item)
  DropoutParams drop;   // used by the kernels instantiated with dropout only
  BiasParams bias;      // used by the kernels instantiated with bias only
};

// Which (head, block) a workgroup of the dQ or dK/dV kernel owns. Blocks are numbered in the order they should start:
// when causal, the heaviest first (the last query blocks, the first key blocks), so that the light ones fill the gaps
// at the end. Taking every head's block 0, then every head's block 1, ... walks through the operands of all heads
// once per block index; with many heads they no longer stay in the caches between two visits (512 heads of 2 MiB:
// the kernels become HBM-bound), so the heads are taken in groups of head_group, group after group.
__device__ inline void bwd_item(const AttnBwdParams& prm, int n_blk, int& bh, int& blk) {
  const int n_bh = prm.B * prm.H, per_group = prm.head_group * n_blk;
  const int grp = blockIdx.x / per_group, r = blockIdx.x - grp * per_group;
  const int heads = min(prm.head_group, n_bh - grp * prm.head_group);
  bh = grp * prm.head_group + r % heads;
  blk = r / heads;
}

constexpr float kLog2e = 1.4426950408889634f;

// acc += A B with the accumulator pinned in AGPRs. Left to the compiler, the 128 accumulator registers of dK and dV are
// kept elsewhere between uses and copied in and out around every MFMA (eight extra VALU instructions per MFMA). Inside
// an asm statement the compiler's hazard recognizer does not see the MFMA: no source may have been written by a VALU
// instruction (a register copy, say) in the two instructions before it, and nothing but such an MFMA may touch an
// accumulator before acc_fence(). The build checks the generated assembly for both (fast_ops_amd/asm_lint.py) and
// falls back to FO_MFMA_NOPS=1, the builtin, if it finds a violation.
#ifndef FO_MFMA_NOPS
#define FO_MFMA_NOPS 0
#endif
// pipelined dK/dV kernel: the copies of the tile after next are issued between the MFMAs of phase 4 (1) or in one batch
// at the hand-over (0)
#ifndef FO_BWD_SPREAD
#define FO_BWD_SPREAD 1
#endif
template <typename T>
__device__ __forceinline__ void mfma_acc_agpr(f32x16& acc, typename Ops<T>::vec8 a, typename Ops<T>::vec8 b) {
#if defined(__HIP_DEVICE_COMPILE__) && !FO_MFMA_NOPS
  if constexpr (std::is_same<T, __bf16>::value)
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
  else
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
#else
  acc = Ops<T>::mfma(a, b, acc);
#endif
}
// S / dP of the pipelined dK/dV kernel: result pinned in VGPRs (the softmax gradient reads it element by element; from
// AGPRs every read is an extra instruction); the accumulator is given its start values before the first call. A VALU
// instruction may read the result 11 wait states after the last MFMA was issued: the kernel's schedule sees to that.
template <typename T>
__device__ __forceinline__ void mfma_scores_vgpr(f32x16& acc, typename Ops<T>::vec8 a, typename Ops<T>::vec8 b) {
#if defined(__HIP_DEVICE_COMPILE__) && !FO_MFMA_NOPS
  if constexpr (std::is_same<T, __bf16>::value) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
  else asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
#else
  acc = Ops<T>::mfma(a, b, acc);
#endif
}
template <int N>
__device__ __forceinline__ void acc_fence(f32x16 (&acc)[N]) {
#if defined(__HIP_DEVICE_COMPILE__) && !FO_MFMA_NOPS
  asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");
#pragma unroll
  for (int i = 0; i < N; ++i) asm volatile("" : "+a"(acc[i]));
#endif
}

// ---------------------------------------------------------------------------------------------------------------------
// ---------------------------------------------------------------------------------------------------------------------
// Copy of a 64-row tile (rows row0 .. row0+63 of a [S, D] matrix with row stride `stride`) into LDS by the whole
// workgroup: per wave D/32 direct-to-LDS instructions. Each instruction fills 1 KiB of LDS with the 64 lanes' pieces
// back to back, so the swizzle is applied by choosing which global chunk a lane fetches. Rows past the end re-read
// the last row (callers mask them); columns from the true head_dim `d` on read zeros.
template <typename T, int D>
__device__ __forceinline__ void copy_tile64(const T* base, int64_t stride, int row0, int S, int d, FO_LDS char* dst, int wave_s, int lane_in) {
  // (an opaque copy of the lane index: this is the path of tiles that cross the end of the matrix, taken once per
  // workgroup at most; its address arithmetic must not be hoisted out of it into registers that live across the loop)
  int lane = lane_in;
  asm volatile("" : "+v"(lane));
  constexpr int ROW_BYTES = D * 2;
  constexpr int CHUNKS = ROW_BYTES / 16;
  constexpr int ROWS_PER_DMA = 1024 / ROW_BYTES;
  constexpr int DMA_PER_WAVE = kBwdTile * ROW_BYTES / 1024 / kBwdWaves;
#pragma unroll
  for (int i = 0; i < DMA_PER_WAVE; ++i) {
    const int row = (wave_s * DMA_PER_WAVE + i) * ROWS_PER_DMA + lane / CHUNKS;
    const int col = ((lane % CHUNKS) ^ swz<D>(row)) * 8;
    const int r = min(row0 + row, S - 1);
    dma16_lane_ptr(live_or_zero(base + (int64_t)r * stride + col, col, d), dst + (wave_s * DMA_PER_WAVE + i) * 1024);
  }
}

// The same copy for a tile that lies wholly inside the matrix, with the address split into a wave-uniform base (the
// tile's first row: scalar arithmetic, once per tile) and per-lane byte offsets that never change (TileLaneOffsets,
// computed once per kernel): two instructions per 1 KiB piece instead of a 64-bit multiply-add per lane and piece.
template <typename T, int D>
struct TileLaneOffsets {
  static constexpr int N = kBwdTile * D * 2 / 1024 / kBwdWaves;   // pieces per wave and tile
  uint32_t off[N];
  bool ok;                                                        // 32-bit offsets suffice for this row stride, and the rows have all D columns
  __device__ __forceinline__ void init(int64_t stride, int d, int wave_s, int lane) {
    constexpr int ROW_BYTES = D * 2, CHUNKS = ROW_BYTES / 16, ROWS_PER_DMA = 1024 / ROW_BYTES;
    ok = stride < (1 << 23) && d == D;
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int row = (wave_s * N + i) * ROWS_PER_DMA + lane / CHUNKS;
      const int col = ((lane % CHUNKS) ^ swz<D>(row)) * 8;
      off[i] = (uint32_t)(row * (int)stride + col) * 2u;
    }
  }
};
template <typename T, int D>
__device__ __forceinline__ void copy_tile64_inside(const T* base, int64_t stride, int row0, const TileLaneOffsets<T, D>& lo,
                                                   FO_LDS char* dst, int wave_s) {
  const char* tile = (const char*)(base + (int64_t)row0 * stride);
#pragma unroll
  for (int i = 0; i < TileLaneOffsets<T, D>::N; ++i) dma16_uniform_base(tile, lo.off[i], dst + (wave_s * TileLaneOffsets<T, D>::N + i) * 1024);
}

// The same offsets kept as two registers per matrix instead of one per piece, for a kernel that has none to spare: the
// byte offset of the lane's row of piece 0 and of its 16-byte chunk in that row. Piece i lies ROWS_PER_DMA * i rows
// further (added to the uniform base) and its rows' swizzle differs from piece 0's in fixed bits (i for 256-byte rows,
// 2 i for 128-byte rows: the bits of the row number that the swizzle takes and the piece index changes), so a piece's
// offset is an XOR with a constant and an addition.
template <typename T, int D>
struct TileLaneOffsetsCompact {
  static constexpr int N = kBwdTile * D * 2 / 1024 / kBwdWaves;
  static constexpr int ROW_BYTES = D * 2, CHUNKS = ROW_BYTES / 16, ROWS_PER_DMA = 1024 / ROW_BYTES;
  uint32_t row_bytes0, chunk_bytes0;
  bool ok;
  __device__ __forceinline__ void init(int64_t stride, int d, int wave_s, int lane) {
    ok = stride < (1 << 23) && d == D;
    const int row = (wave_s * N) * ROWS_PER_DMA + lane / CHUNKS;
    row_bytes0 = (uint32_t)(row * (int)stride) * 2u;
    chunk_bytes0 = (uint32_t)(((lane % CHUNKS) ^ swz<D>(row)) * 16);
  }
  static constexpr uint32_t flip(int i) { return (uint32_t)((D == 128 ? i : 2 * i) * 16); }
  // (wave_s * N is a multiple of N = 4 or 2, so the piece index occupies bits of the row number that are zero in piece 0)
  static_assert((D == 128 && N == 4) || (D == 64 && N == 2), "which bits of the swizzle a piece index changes");
};
// Two tiles (K and V) at once: every offset is computed before the first copy goes out. (Should the compiler have parked
// one of the four registers in scratch memory, its reload - which it waits for with vmcnt(0) - then comes before the
// copies and finds nothing in flight; between two copies it would wait for the first one to land.)
template <typename T, int D>
__device__ __forceinline__ void copy_two_tiles64_inside(const T* base_a, int64_t stride_a, const TileLaneOffsetsCompact<T, D>& lo_a, FO_LDS char* dst_a,
                                                        const T* base_b, int64_t stride_b, const TileLaneOffsetsCompact<T, D>& lo_b, FO_LDS char* dst_b,
                                                        int row0, int wave_s) {
  typedef TileLaneOffsetsCompact<T, D> L;
  const char* tile_a = (const char*)(base_a + (int64_t)row0 * stride_a);
  const char* tile_b = (const char*)(base_b + (int64_t)row0 * stride_b);
  uint32_t ra = lo_a.row_bytes0, ca = lo_a.chunk_bytes0, rb = lo_b.row_bytes0, cb = lo_b.chunk_bytes0;
  // (recomputed per tile: hoisted out of the loop they would be 2 N registers again)
  asm volatile("" : "+v"(ra), "+v"(ca), "+v"(rb), "+v"(cb));
  uint32_t off_a[L::N], off_b[L::N];
#pragma unroll
  for (int i = 0; i < L::N; ++i) {
    off_a[i] = ra + (ca ^ L::flip(i));
    off_b[i] = rb + (cb ^ L::flip(i));
    asm volatile("" : "+v"(off_a[i]), "+v"(off_b[i]));
  }
#pragma unroll
  for (int i = 0; i < L::N; ++i) {
    dma16_uniform_base(tile_a + (int64_t)i * L::ROWS_PER_DMA * stride_a * 2, off_a[i], dst_a + (wave_s * L::N + i) * 1024);
    dma16_uniform_base(tile_b + (int64_t)i * L::ROWS_PER_DMA * stride_b * 2, off_b[i], dst_b + (wave_s * L::N + i) * 1024);
  }
}

// A operand of a 32x32x16 MFMA from a row-major tile in LDS: lane = row l32 of block `blk`, 8 elements at
// column 16*ks + 8*hh
template <typename T, int D>
__device__ __forceinline__ typename Ops<T>::vec8 row_frag(FO_LDS const char* tile, int blk, int ks, int l32, int hh) {
  const int row = 32 * blk + l32;
  return *(FO_LDS const typename Ops<T>::vec8*)(tile + row * (D * 2) + (((2 * ks + hh) ^ swz<D>(row)) * 16));
}
// A operand = transpose of a tile block: M = 32 columns (d = 32*db ..), K = 16 rows of the tile in the order the 32x32
// accumulator layout hands them over as a B operand (rows 16*t + 4*hh + {0..3} and + 8)
template <typename T, int D>
__device__ __forceinline__ typename Ops<T>::vec8 col_frag(FO_LDS const char* tile, int t, int db, int lane) {
  const int hh = lane >> 5, L16 = lane & 15, g16 = (lane >> 4) & 1;
  const int row0 = 16 * t + 4 * hh + (L16 >> 2), row1 = row0 + 8;
  const int chunk = 4 * db + 2 * g16 + ((L16 & 3) >> 1);
  const int sub = (L16 & 1) * 8;
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FO_LDS s16x4*)(tile + row0 * (D * 2) + ((chunk ^ swz<D>(row0)) * 16) + sub));
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FO_LDS s16x4*)(tile + row1 * (D * 2) + ((chunk ^ swz<D>(row1)) * 16) + sub));
  return __builtin_bit_cast(typename Ops<T>::vec8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

// A wave's 32 finished gradient rows (accumulator layout: lane = row l32, registers 4*rg + u = columns
// 32*db + 8*rg + 4*hh + u) written to memory. Straight from the registers that is 8 bytes per lane to 32 different
// rows per instruction (4.3 us per workgroup for dK and dV, during which the workgroup's LDS and registers keep the
// next one waiting); instead the rows are rounded into LDS (`stage`, 32 rows padded by 16 bytes each, this wave's
// own) and leave as whole 16-byte pieces, 64 lanes covering consecutive rows. Rows from n_rows on and columns from the true head_dim `d` on are not written.
template <typename T, int D>
__device__ __forceinline__ void store_rows_via_lds(const f32x16 (&acc)[D / 32], float mul, FO_LDS char* stage, T* base, int64_t stride,
                                                   int row0, int n_rows, int d, int lane) {
  constexpr int ROW_BYTES = D * 2, OROW = ROW_BYTES + 16, CH = ROW_BYTES / 16;
  typedef __attribute__((ext_vector_type(4))) T vec4;
  typedef __attribute__((ext_vector_type(4))) int i32x4;
  const int l32 = lane & 31, hh = lane >> 5;
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
      vec4 o4;
#pragma unroll
      for (int u = 0; u < 4; ++u) o4[u] = (T)(acc[db][rg * 4 + u] * mul);
      *(FO_LDS vec4*)(stage + l32 * OROW + (32 * db + 8 * rg + 4 * hh) * 2) = o4;
    }
#pragma unroll
  for (int it = 0; it < 32 * CH / 64; ++it) {
    const int idx = it * 64 + lane, row = idx / CH, ch = idx % CH;
    const i32x4 piece = *(FO_LDS const i32x4*)(stage + row * OROW + ch * 16);
    if (row0 + row < n_rows && ch * 8 < d) *(i32x4*)(base + (int64_t)(row0 + row) * stride + ch * 8) = piece;
  }
}
constexpr int stage_bytes(int D) { return 32 * (D * 2 + 16); }   // per wave and matrix

// ---------------------------------------------------------------------------------------------------------------------
// KBIAS (without BIAS): a bias that is the same for every query (query stride 0), at no cost per score. Its 64
// values of a key tile, divided by softmax_scale, are what the accumulators of S^T start from - register r of a lane
// holds a key that depends on r and the half of the wave only - so that the MFMAs deliver S + b / scale and everything
// after them is the code without bias. Wave 0 fetches the values of tile t+2 while tile t is worked on (a plain load: it
// is waited for at the top of the next tile, where every copy in flight is waited for anyway), converts those of tile
// t+1 and puts them into LDS, where every wave reads them after the next barrier.
template <typename T, int D, bool CAUSAL, bool DROP, bool BIAS, bool KBIAS = false>
__global__ void __launch_bounds__(kBwdWaves * 64, 2) attn_bwd_dq_kernel(const AttnBwdParams prm) {
  static_assert(!(KBIAS && BIAS), "one bias form at a time");
  typedef typename Ops<T>::vec8 vec8;
  constexpr int TILE_BYTES = kBwdTile * D * 2;
  constexpr int KSTEPS = D / 16;
  constexpr int DBLK = D / 32;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  FO_LDS char* smem = (FO_LDS char*)smem_raw;   // K0 | K1 | V0 | V1 | bias of the tile's 64 keys, two buffers (BIAS)
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);
  const int lane = tid & 63, l32 = lane & 31, hh = lane >> 5;
  const int n_qblk = (prm.Sq + kBwdRows - 1) / kBwdRows;
  int bh, qblk;
  bwd_item(prm, n_qblk, bh, qblk);
  qblk = n_qblk - 1 - qblk;                          // heaviest causal blocks first
  const int b = bh / prm.H, h = bh % prm.H;
  const int q0 = qblk * kBwdRows, q0w = q0 + wave * 32;
  const int Sq = prm.Sq, Sk = prm.Sk;
  const T* kbase = (const T*)prm.k + b * prm.ks[0] + h * prm.ks[1];
  const T* vbase = (const T*)prm.v + b * prm.vs[0] + h * prm.vs[1];
  const int n_tiles = CAUSAL ? (min(Sk, q0 + kBwdRows) + kBwdTile - 1) / kBwdTile : (Sk + kBwdTile - 1) / kBwdTile;

  // (one register per piece where the kernel has them - head_dim 64, and the plain causal form at head_dim 128, which
  // were 0.4-0.6 % faster that way - and two per matrix where it would otherwise park some in scratch memory)
  constexpr bool ROOMY = D == 64 || (CAUSAL && !DROP && !BIAS && !KBIAS);
  typename std::conditional<ROOMY, TileLaneOffsets<T, D>, TileLaneOffsetsCompact<T, D>>::type klo, vlo;
  klo.init(prm.ks[2], prm.d, wave_s, lane);
  vlo.init(prm.vs[2], prm.d, wave_s, lane);
  // A bias that is the same for every query (query stride 0) is 64 values per key tile, the same for all lanes: wave 0
  // copies them into LDS with the tile (4 bytes per lane: one key in fp32, two in the operand type), and every lane
  // reads its registers' keys from there. (Loaded from global memory where they are used, the compiler waits for
  // them together with the tile copies in flight.) Keys past the end re-read the last ones and are masked below.
  FO_LDS char* bias_keys = smem + 4 * TILE_BYTES;
  bool bias_keys_staged = false;
  const char* bias_keys_src = nullptr;
  if constexpr (BIAS) {
    const int64_t at = b * prm.bias.strides[0] + h * prm.bias.strides[1];
    bias_keys_src = (const char*)prm.bias.ptr + at * (prm.bias.is_f32 ? 4 : 2);
    bias_keys_staged = prm.bias.strides[2] == 0 && ((uintptr_t)bias_keys_src % 4) == 0 && (prm.bias.is_f32 || Sk % 2 == 0);   // (pairs of keys: an even count)
  }
  auto issue = [&](int tile, int buf) {
    if constexpr (BIAS) {
      if (bias_keys_staged && wave_s == 0) {
        if (prm.bias.is_f32) dma4_lane_ptr(bias_keys_src + (int64_t)min(tile * kBwdTile + lane, Sk - 1) * 4, bias_keys + buf * 256);
        else if (lane < 32) dma4_lane_ptr(bias_keys_src + (int64_t)min(tile * kBwdTile + 2 * lane, Sk - 2) * 2, bias_keys + buf * 256);
      }
    }
    if (tile * kBwdTile + kBwdTile <= Sk && klo.ok && vlo.ok) {
      if constexpr (ROOMY) {
        copy_tile64_inside<T, D>(kbase, prm.ks[2], tile * kBwdTile, klo, smem + buf * TILE_BYTES, wave_s);
        copy_tile64_inside<T, D>(vbase, prm.vs[2], tile * kBwdTile, vlo, smem + (2 + buf) * TILE_BYTES, wave_s);
      } else {
        copy_two_tiles64_inside<T, D>(kbase, prm.ks[2], klo, smem + buf * TILE_BYTES, vbase, prm.vs[2], vlo, smem + (2 + buf) * TILE_BYTES,
                                      tile * kBwdTile, wave_s);
      }
    } else {
      copy_tile64<T, D>(kbase, prm.ks[2], tile * kBwdTile, Sk, prm.d, smem + buf * TILE_BYTES, wave_s, lane);
      copy_tile64<T, D>(vbase, prm.vs[2], tile * kBwdTile, Sk, prm.d, smem + (2 + buf) * TILE_BYTES, wave_s, lane);
    }
  };
  issue(0, 0);
  FO_LDS float* key_bias = (FO_LDS float*)(smem + 4 * TILE_BYTES);      // KBIAS: [2][64], bias / scale of the keys of a tile
  float key_bias_next = 0.0f;                                           // (wave 0) this lane's key of the tile after next
  // (wave-uniform, and told so: this kernel has no vector register to spare)
  const float per_scale = KBIAS ? __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, kLog2e / prm.scale_log2e))) : 0.0f;
  const int64_t key_bias_row = KBIAS ? b * prm.bias.strides[0] + h * prm.bias.strides[1] : 0;
  if constexpr (KBIAS) {
    if (wave_s == 0) {
      key_bias[lane] = load_bias<T>(prm.bias, key_bias_row + min(lane, Sk - 1)) * per_scale;
      key_bias_next = load_bias<T>(prm.bias, key_bias_row + min(kBwdTile + lane, Sk - 1));
    }
  }

  // B operands held for the whole kernel: Q^T and dO^T fragments of this lane's query row; its LSE and delta
  const int qrow = min(q0w + l32, Sq - 1);
  vec8 qf[KSTEPS], gf[KSTEPS];
  {
    const T* qp = (const T*)prm.q + b * prm.qs[0] + h * prm.qs[1] + (int64_t)qrow * prm.qs[2] + 8 * hh;
    const T* gp = (const T*)prm.d_o + b * prm.dos[0] + h * prm.dos[1] + (int64_t)qrow * prm.dos[2] + 8 * hh;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      qf[ks] = *(const vec8*)live_or_zero(qp + 16 * ks, 16 * ks + 8 * hh, prm.d);
      gf[ks] = *(const vec8*)live_or_zero(gp + 16 * ks, 16 * ks + 8 * hh, prm.d);
    }
  }
  const float lse2 = prm.lse[(int64_t)bh * Sq + qrow] * kLog2e;
  // delta_i = sum_d dO_id O_id (flash_attention_triton.py:273-315), negated: this lane holds half of its row's dO
  // already, so it reads the same pieces of O, and the two halves of the wave add up. Stored for the dK/dV kernel,
  // which runs after this one (a pass of its own over O and dO would be a launch more: 5 of 83 us at B=8 H=12 S=1024).
  float delta = 0.0f;
  {
    const T* op = (const T*)prm.o + b * prm.os[0] + h * prm.os[1] + (int64_t)qrow * prm.os[2] + 8 * hh;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const vec8 ov = *(const vec8*)live_or_zero(op + 16 * ks, 16 * ks + 8 * hh, prm.d);
#pragma unroll
      for (int e = 0; e < 8; ++e) delta -= (float)ov[e] * (float)gf[ks][e];
    }
    delta += half_swap(delta);
    if (hh == 0 && q0w + l32 < Sq) prm.delta[(int64_t)bh * Sq + q0w + l32] = delta;
  }
  // (consumed here so that the compiler waits for these loads before the loop: a vmcnt wait inside the loop would
  // also wait for the tile copies in flight, which it does not see)
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) asm volatile("" ::"v"(qf[ks]), "v"(gf[ks]));
  asm volatile("" ::"v"(lse2), "v"(delta));

  f32x16 acc[DBLK];
#pragma unroll
  for (int i = 0; i < DBLK; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
  const float c = prm.scale_log2e, scale = prm.scale;

  for (int tile = 0; tile < n_tiles; ++tile) {
    const int buf = tile & 1;
    const int key0 = tile * kBwdTile;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if constexpr (KBIAS) {
      // (the value fetched one tile ago is used before this tile's copies go out: the wait the compiler puts in front
      // of its use then finds nothing in flight)
      if (wave_s == 0) {
        asm volatile("" : "+v"(key_bias_next));                                  // (the use starts here, not earlier)
        key_bias[(buf ^ 1) * kBwdTile + lane] = key_bias_next * per_scale;       // tile + 1: read after the next barrier
      }
    }
    if (tile + 1 < n_tiles) issue(tile + 1, buf ^ 1);
    if constexpr (KBIAS) {
      if (wave_s == 0) key_bias_next = load_bias<T>(prm.bias, key_bias_row + min((tile + 2) * kBwdTile + lane, Sk - 1));
    }
    if (CAUSAL && key0 > q0w + 31) continue;
    FO_LDS const char* kt = smem + buf * TILE_BYTES;
    FO_LDS const char* vt = smem + (2 + buf) * TILE_BYTES;

    f32x16 sacc[2], dpacc[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) { sacc[kb][r] = 0.0f; dpacc[kb][r] = 0.0f; }
    if constexpr (KBIAS) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int jv = 0; jv < 4; ++jv) {
          const f32x4 b4 = *(FO_LDS const f32x4*)(key_bias + buf * kBwdTile + 32 * kb + 8 * jv + 4 * hh);
#pragma unroll
          for (int u = 0; u < 4; ++u) sacc[kb][4 * jv + u] = b4[u];
        }
    }
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        sacc[kb] = Ops<T>::mfma(row_frag<T, D>(kt, kb, ks, l32, hh), qf[ks], sacc[kb]);      // S^T = K Q^T
        dpacc[kb] = Ops<T>::mfma(row_frag<T, D>(vt, kb, ks, l32, hh), gf[ks], dpacc[kb]);    // dP^T = V dO^T
      }
    // register r of block kb holds key key0 + 32*kb + 4*hh + koff(r), koff(r) = (r & 3) + 8 * (r >> 2); dead iff
    // key > q or key >= Sk
    vec8 dsf[4];
    // dropout (flash_attention_triton.py:524-532,599): dP reaches only the kept probabilities, scaled by 1 / (1 - p_drop)
    const uint32_t drop_row = DROP ? prm.drop.offset + ((uint32_t)bh * (uint32_t)Sq + (uint32_t)(q0w + l32)) * (uint32_t)Sk + (uint32_t)key0 : 0u;
    // bias row of this lane's query (flash_attention_triton.py:497-509); keys past the end re-read the last one
    const int64_t bias_row = BIAS ? b * prm.bias.strides[0] + h * prm.bias.strides[1] + (int64_t)qrow * prm.bias.strides[2] : 0;
    // (the factor softmax_scale of dS is applied once, to the finished accumulators; tiles that no mask touches - most -
    // go without the comparisons)
    auto softmax_grad = [&](auto masked) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const int key_base = key0 + 32 * kb + 4 * hh;
        int lim = key_base - Sk + 1;
        if (CAUSAL) lim = max(lim, key_base - (q0w + l32));
        // registers 4*j .. 4*j + 3 (four consecutive keys), given their bias
        auto four = [&](int j, const float* b4) {
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int r = 4 * j + u;
            const bool dead = decltype(masked)::value && lim > -(u + 8 * j);
            float shift = -lse2;
            if constexpr (BIAS) shift = __builtin_fmaf(b4[u], kLog2e, -lse2);
            const float p = dead ? 0.0f : __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][r], c, shift));
            float dp = dpacc[kb][r];
            if constexpr (DROP) {
              const uint32_t idx = drop_row + (uint32_t)(32 * kb + 4 * hh + u + 8 * j);
              dp = dropout_keep(idx, prm.drop.seed, prm.drop.threshold) ? dp * prm.drop.keep_scale : 0.0f;
            }
            dsf[kb * 2 + (r >> 3)][r & 7] = (T)(p * (dp + delta));
          }
        };
        // The bias of four keys at a time (few values in flight: this kernel has no registers to spare). From the
        // per-key values staged in LDS; else with one load of four consecutive keys when the tile is complete and the
        // bias is laid out for it; else key by key. Every lane reads its own row, so a load instruction touches 32
        // cache lines either way, and fewer instructions is what counts. The bias type is decided around the loops.
        float b4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        if constexpr (!BIAS) {
#pragma unroll
          for (int j = 0; j < 4; ++j) four(j, b4);
        } else if (bias_keys_staged) {
          FO_LDS const char* bk = bias_keys + buf * 256;
          if (prm.bias.is_f32) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const f32x4 t4 = *(FO_LDS const f32x4*)(bk + (32 * kb + 4 * hh + 8 * j) * 4);
#pragma unroll
              for (int u = 0; u < 4; ++u) b4[u] = t4[u];
              four(j, b4);
            }
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              typedef __attribute__((ext_vector_type(4))) T vec4;
              const vec4 t4 = *(FO_LDS const vec4*)(bk + (32 * kb + 4 * hh + 8 * j) * 2);
#pragma unroll
              for (int u = 0; u < 4; ++u) b4[u] = (float)t4[u];
              four(j, b4);
            }
          }
        } else if (prm.bias.vec_ok && key0 + kBwdTile <= Sk) {
          if (prm.bias.is_f32) {
#pragma unroll
            for (int j = 0; j < 4; ++j) { load_bias4<float>((const float*)prm.bias.ptr + bias_row + key_base + 8 * j, b4); four(j, b4); }
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) { load_bias4<T>((const T*)prm.bias.ptr + bias_row + key_base + 8 * j, b4); four(j, b4); }
          }
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int u = 0; u < 4; ++u) b4[u] = load_bias<T>(prm.bias, bias_row + min(key_base + u + 8 * j, Sk - 1));
            four(j, b4);
          }
        }
      }
    };
    if (key0 + kBwdTile > Sk || (CAUSAL && key0 + kBwdTile - 1 > q0w)) softmax_grad(std::true_type{});
    else softmax_grad(std::false_type{});
    // dQ^T += K^T dS^T : four 16-key steps x DBLK d-blocks
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int db = 0; db < DBLK; ++db) acc[db] = Ops<T>::mfma(col_frag<T, D>(kt, t, db, lane), dsf[t], acc[db]);
  }

  // (straight from the registers, 8 bytes per lane: with two workgroups per CU the other one covers the time these
  // stores take, and staging the rows in LDS as the dK/dV kernels do made this kernel 5-10 % slower)
  const int qi = q0w + l32;
  if (qi < Sq) {
    // -LSE / softmax_scale for the dK/dV kernel, whose score accumulators start from it: P = exp2((QK^T - LSE / scale)
    // * scale * log2 e) is then one multiplication and the exponential per element. (Stored here, from the scaled LSE
    // the loop used, and not beside delta: every register is taken while the loop runs.)
    if (hh == 0) prm.nlse[(int64_t)bh * Sq + qi] = lse2 * prm.neg_inv_scale_log2e;
    T* op = (T*)prm.dq + b * prm.dqs[0] + h * prm.dqs[1] + (int64_t)qi * prm.dqs[2];
#pragma unroll
    for (int db = 0; db < DBLK; ++db)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        typedef __attribute__((ext_vector_type(4))) T vec4;
        vec4 o4;
#pragma unroll
        for (int u = 0; u < 4; ++u) o4[u] = (T)(acc[db][rg * 4 + u] * scale);
        if (32 * db + 8 * rg + 4 * hh < prm.d) *(vec4*)(op + 32 * db + 8 * rg + 4 * hh) = o4;
      }
  }
}

// ---------------------------------------------------------------------------------------------------------------------
template <typename T, int D, bool CAUSAL, bool DROP, bool BIAS>
__global__ void __launch_bounds__(kBwdWaves * 64) attn_bwd_dkdv_kernel(const AttnBwdParams prm) {
  typedef typename Ops<T>::vec8 vec8;
  constexpr int TILE_BYTES = kBwdTile * D * 2;
  constexpr int KSTEPS = D / 16;
  constexpr int DBLK = D / 32;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  FO_LDS char* smem = (FO_LDS char*)smem_raw;   // Q0 | Q1 | dO0 | dO1 | lse[2][64] | delta[2][64] | bias tiles (BIAS)
  FO_LDS float* rowvals = (FO_LDS float*)(smem + 4 * TILE_BYTES);
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);
  const int lane = tid & 63, l32 = lane & 31, hh = lane >> 5;
  int bh, kblk;                                       // key block 0 has the most queries when causal: heaviest first
  bwd_item(prm, (prm.Sk + kBwdRows - 1) / kBwdRows, bh, kblk);
  const int b = bh / prm.H, h = bh % prm.H;
  const int k0 = kblk * kBwdRows, k0w = k0 + wave * 32;
  const int Sq = prm.Sq, Sk = prm.Sk;
  const T* qbase = (const T*)prm.q + b * prm.qs[0] + h * prm.qs[1];
  const T* gbase = (const T*)prm.d_o + b * prm.dos[0] + h * prm.dos[1];
  const int n_qt = (Sq + kBwdTile - 1) / kBwdTile;
  const int qt0 = CAUSAL ? min(k0 / kBwdTile, n_qt) : 0;   // queries before the block's first key never attend it

  TileLaneOffsets<T, D> qlo, glo;
  qlo.init(prm.qs[2], prm.d, wave_s, lane);
  glo.init(prm.dos[2], prm.d, wave_s, lane);
  // ---- bias. A lane owns a key and its registers run over queries, so a bias that is the same for every query (query
  // stride 0) is one value per lane for the whole kernel. Otherwise the wave's 64 queries x 32 keys of a tile are
  // copied straight into LDS together with the tile (a load the compiler can see is waited for right where it is
  // issued, together with the tile copies in flight, which then no longer overlap the arithmetic): two buffers of
  // kBiasWaveBytes per wave. A row of the wave's part is 128 bytes (fp32) or 64 bytes (operand type), so one copy
  // instruction of 64 x 16 bytes holds 8 or 16 rows; inside it, row 4*hh + u (+ 8 for the second eight) sits in
  // slot 2*u + hh (+ 8), so that a lane reads register u at a fixed distance from its base and the two halves of
  // a wave, four rows apart, read different banks. Only complete tiles of suitably aligned tensors; the rest reads
  // the bias element by element.
  constexpr int kBiasWaveBytes = kBwdTile * 32 * 4;
  FO_LDS char* bias_lds = (FO_LDS char*)(rowvals + 4 * kBwdTile) + wave_s * 2 * kBiasWaveBytes;
  const bool bias_per_key = BIAS && prm.bias.strides[2] == 0;
  const bool bias_staged = BIAS && !bias_per_key && prm.bias.dma_ok && k0 + wave_s * 32 + 32 <= Sk &&
                           prm.bias.strides[2] > 0 && prm.bias.strides[2] < (1 << 24);   // (32-bit offsets inside a copy instruction)
  float bias_lane = 0.0f;
  if (bias_per_key) bias_lane = load_bias<T>(prm.bias, b * prm.bias.strides[0] + h * prm.bias.strides[1] + min(k0w + l32, Sk - 1)) * kLog2e;
  // (per lane: the byte offset of its piece inside the rows of one copy instruction, added to a uniform base per
  // instruction. Handing base and offset to the copy separately, as a scalar base plus a 32-bit lane offset, left the
  // GPU faulted in this kernel for a reason not found; the per-lane 64-bit pointer is the form that is tested.)
  uint32_t bias_lane_off = 0;
  const char* bias_src = nullptr;
  int64_t bias_row_bytes = 0;
  if (bias_staged) {
    const int elt = prm.bias.is_f32 ? 4 : 2;
    const int g = prm.bias.is_f32 ? lane >> 3 : lane >> 2, piece = prm.bias.is_f32 ? lane & 7 : lane & 3;
    const int row_in = 8 * (g >> 3) + 4 * (g & 1) + ((g >> 1) & 3);   // the row kept in slot g
    bias_row_bytes = prm.bias.strides[2] * elt;
    bias_lane_off = (uint32_t)(row_in * bias_row_bytes + piece * 16);
    bias_src = (const char*)prm.bias.ptr + (b * prm.bias.strides[0] + h * prm.bias.strides[1] + k0 + wave_s * 32) * elt;   // wave-uniform
  }
  auto issue_bias = [&](int qt, int buf) {
    if (!bias_staged || qt * kBwdTile + kBwdTile > Sq) return;
    const int rows_per_dma = prm.bias.is_f32 ? 8 : 16, n_dma = prm.bias.is_f32 ? 8 : 4;
    FO_LDS char* dst = bias_lds + buf * kBiasWaveBytes;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (i < n_dma) dma16_lane_ptr(bias_src + (int64_t)(qt * kBwdTile + i * rows_per_dma) * bias_row_bytes + bias_lane_off, dst + i * 1024);
  };
  auto issue = [&](int qt, int buf) {
    if constexpr (BIAS) issue_bias(qt, buf);
    if (qt * kBwdTile + kBwdTile <= Sq && qlo.ok && glo.ok) {
      copy_tile64_inside<T, D>(qbase, prm.qs[2], qt * kBwdTile, qlo, smem + buf * TILE_BYTES, wave_s);
      copy_tile64_inside<T, D>(gbase, prm.dos[2], qt * kBwdTile, glo, smem + (2 + buf) * TILE_BYTES, wave_s);
    } else {
      copy_tile64<T, D>(qbase, prm.qs[2], qt * kBwdTile, Sq, prm.d, smem + buf * TILE_BYTES, wave_s, lane);
      copy_tile64<T, D>(gbase, prm.dos[2], qt * kBwdTile, Sq, prm.d, smem + (2 + buf) * TILE_BYTES, wave_s, lane);
    }
    // per-row LSE and delta of the tile, 4 bytes per lane, also straight into LDS (a load the compiler can see would
    // make it wait for the tile copies as well); rows past the end re-read the last row and are masked below
    if (wave_s < 2) {
      const int64_t at = (int64_t)bh * Sq + min(qt * kBwdTile + lane, Sq - 1);
      dma4_lane_ptr((wave_s == 0 ? prm.lse : (const float*)prm.delta) + at, rowvals + (2 * wave_s + buf) * kBwdTile);
    }
  };
  if (qt0 < n_qt) issue(qt0, 0);

  // B operands held for the whole kernel: K^T and V^T fragments of this lane's key
  const int key = k0w + l32;
  const int krow = min(key, Sk - 1);
  vec8 kf[KSTEPS], vf[KSTEPS];
  {
    const T* kp = (const T*)prm.k + b * prm.ks[0] + h * prm.ks[1] + (int64_t)krow * prm.ks[2] + 8 * hh;
    const T* vp = (const T*)prm.v + b * prm.vs[0] + h * prm.vs[1] + (int64_t)krow * prm.vs[2] + 8 * hh;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      kf[ks] = *(const vec8*)live_or_zero(kp + 16 * ks, 16 * ks + 8 * hh, prm.d);
      vf[ks] = *(const vec8*)live_or_zero(vp + 16 * ks, 16 * ks + 8 * hh, prm.d);
    }
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) asm volatile("" ::"v"(kf[ks]), "v"(vf[ks]));
  }

  f32x16 dkacc[DBLK], dvacc[DBLK];
#pragma unroll
  for (int i = 0; i < DBLK; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) { dkacc[i][r] = 0.0f; dvacc[i][r] = 0.0f; }
  const float c = prm.scale_log2e, scale = prm.scale;

  for (int qt = qt0; qt < n_qt; ++qt) {
    const int buf = (qt - qt0) & 1;
    const int q0t = qt * kBwdTile;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (qt + 1 < n_qt) issue(qt + 1, buf ^ 1);
    FO_LDS const char* qtile = smem + buf * TILE_BYTES;
    FO_LDS const char* gtile = smem + (2 + buf) * TILE_BYTES;
    FO_LDS const float* lse_t = rowvals + buf * kBwdTile;
    FO_LDS const float* del_t = rowvals + (2 + buf) * kBwdTile;
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      if (CAUSAL && q0t + 32 * qb + 31 < k0w) continue;   // every query of the block is before every key of this wave
      f32x16 sacc, dpacc;
#pragma unroll
      for (int r = 0; r < 16; ++r) { sacc[r] = 0.0f; dpacc[r] = 0.0f; }
      // the staged bias of this block's 16 registers, read ahead of the MFMAs below (read where it is used, each
      // value is waited for on its own): row 32*qb + 8*j + 4*hh + u of the tile sits in copy instruction 4*qb + j
      // (fp32) or 2*qb + j/2 (operand type)
      float bias_reg[BIAS ? 16 : 1];
      const bool bias_from_lds = BIAS && bias_staged && q0t + kBwdTile <= Sq;
      if constexpr (BIAS) {
        if (bias_from_lds) {
          FO_LDS const char* bias_t = bias_lds + buf * kBiasWaveBytes + (prm.bias.is_f32 ? hh * 128 + l32 * 4 : hh * 64 + l32 * 2);
          // (one decision on the bias type around all 16 reads: decided per element, every read gets its own branch
          // and its own wait)
          if (prm.bias.is_f32) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
              for (int u = 0; u < 4; ++u) bias_reg[4 * j + u] = *(FO_LDS const float*)(bias_t + (4 * qb + j) * 1024 + u * 256);
          } else {
            T raw[16];
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
              for (int u = 0; u < 4; ++u) raw[4 * j + u] = *(FO_LDS const T*)(bias_t + (2 * qb + (j >> 1)) * 1024 + (j & 1) * 512 + u * 128);
#pragma unroll
            for (int r = 0; r < 16; ++r) bias_reg[r] = (float)raw[r];
          }
        }
      }
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        sacc = Ops<T>::mfma(row_frag<T, D>(qtile, qb, ks, l32, hh), kf[ks], sacc);      // S = Q K^T
        dpacc = Ops<T>::mfma(row_frag<T, D>(gtile, qb, ks, l32, hh), vf[ks], dpacc);    // dP = dO V^T
      }
      // register r holds query q0t + 32*qb + 4*hh + koff(r), koff(r) = (r & 3) + 8 * (r >> 2); dead iff key > query
      // or the query is past the end
      const int lim = CAUSAL ? key - (q0t + 32 * qb + 4 * hh) : 0;
      const int lim_end = Sq - (q0t + 32 * qb + 4 * hh);
      vec8 pf[2], dsf[2];
      // dropout index of (first query of this lane's register set, this lane's key); consecutive queries are Sk apart
      const uint32_t drop_base = DROP ? prm.drop.offset + ((uint32_t)bh * (uint32_t)Sq + (uint32_t)(q0t + 32 * qb + 4 * hh)) * (uint32_t)Sk + (uint32_t)key : 0u;
      // bias column of this lane's key; queries past the end re-read the last one
      const int64_t bias_col = BIAS ? b * prm.bias.strides[0] + h * prm.bias.strides[1] + krow : 0;
      // where the bias comes from: 0 global memory, element by element; 1 the lane's own value; 2 the staged tile
      auto softmax_grad = [&](auto masked, auto bias_mode) {
      constexpr int BM = decltype(bias_mode)::value;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const f32x4 l4 = *(FO_LDS const f32x4*)(lse_t + 32 * qb + 8 * j + 4 * hh);
        const f32x4 d4 = *(FO_LDS const f32x4*)(del_t + 32 * qb + 8 * j + 4 * hh);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int r = 4 * j + u;
          const bool dead = decltype(masked)::value && ((u + 8 * j) < lim || (u + 8 * j) >= lim_end);
          float shift = -l4[u] * kLog2e;
          if constexpr (BIAS && BM == 0) {
            const int qi = min(q0t + 32 * qb + 4 * hh + u + 8 * j, Sq - 1);
            shift = __builtin_fmaf(load_bias<T>(prm.bias, bias_col + (int64_t)qi * prm.bias.strides[2]), kLog2e, shift);
          }
          if constexpr (BIAS && BM == 1) shift += bias_lane;
          if constexpr (BIAS && BM == 2) shift = __builtin_fmaf(bias_reg[r], kLog2e, shift);
          const float p = dead ? 0.0f : __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[r], c, shift));
          float pd = p, dp = dpacc[r];
          if constexpr (DROP) {
            const bool keep = dropout_keep(drop_base + (uint32_t)(u + 8 * j) * (uint32_t)Sk, prm.drop.seed, prm.drop.threshold);
            pd = keep ? p * prm.drop.keep_scale : 0.0f;       // dV sees the dropped, rescaled probabilities (:551-552)
            dp = keep ? dp * prm.drop.keep_scale : 0.0f;
          }
          pf[r >> 3][r & 7] = (T)pd;
          dsf[r >> 3][r & 7] = (T)(p * (dp + d4[u]));   // (d4 = -delta) softmax_scale is applied to the finished dK
        }
      }
      };
      const bool needs_mask = q0t + 32 * qb + 32 > Sq || (CAUSAL && k0w + 31 > q0t + 32 * qb);
      typedef std::integral_constant<int, 0> BM0;
      typedef std::integral_constant<int, 1> BM1;
      typedef std::integral_constant<int, 2> BM2;
      if constexpr (!BIAS) {
        if (needs_mask) softmax_grad(std::true_type{}, BM0{}); else softmax_grad(std::false_type{}, BM0{});
      } else if (bias_per_key) {
        if (needs_mask) softmax_grad(std::true_type{}, BM1{}); else softmax_grad(std::false_type{}, BM1{});
      } else if (bias_from_lds) {
        if (needs_mask) softmax_grad(std::true_type{}, BM2{}); else softmax_grad(std::false_type{}, BM2{});
      } else {
        if (needs_mask) softmax_grad(std::true_type{}, BM0{}); else softmax_grad(std::false_type{}, BM0{});
      }
      // dV^T += dO^T P and dK^T += Q^T dS : two 16-query steps x DBLK d-blocks
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int db = 0; db < DBLK; ++db) {
          dvacc[db] = Ops<T>::mfma(col_frag<T, D>(gtile, 2 * qb + t, db, lane), pf[t], dvacc[db]);
          dkacc[db] = Ops<T>::mfma(col_frag<T, D>(qtile, 2 * qb + t, db, lane), dsf[t], dkacc[db]);
        }
    }
  }

  // (the tile buffers are free once every wave is past its last tile; dK, then dV, through the wave's own piece of them)
  __syncthreads();
  {
    FO_LDS char* stage = smem + wave_s * stage_bytes(D);
    const int k0w_s = k0 + wave_s * 32;
    store_rows_via_lds<T, D>(dkacc, scale, stage, (T*)prm.dk + b * prm.dks[0] + h * prm.dks[1], prm.dks[2], k0w_s, Sk, prm.d, lane);
    store_rows_via_lds<T, D>(dvacc, 1.0f, stage, (T*)prm.dv + b * prm.dvs[0] + h * prm.dvs[1], prm.dvs[2], k0w_s, Sk, prm.d, lane);
  }
}

// ---------------------------------------------------------------------------------------------------------------------
// The softmax-gradient jobs of one tile of the pipelined dK/dV kernel (see its tile_body): 48 slots, slot s = eight per
// half-phase from the second half of phase 1 on. stage 0 = A of element r (P = exp2(S c)), stage 1 = B of elements r and
// r + 1 (dS = P dP, both rounded) of query block qb.
struct SoftmaxGradJob { int stage, qb, r; };
constexpr SoftmaxGradJob softmax_grad_job(int s) {
  const int h = s / 8, u = s % 8;
  if (h == 0) return {0, 0, u};
  if (h == 1) return {0, 0, 8 + u};
  if (h == 2) return u < 4 ? SoftmaxGradJob{1, 0, 2 * u} : SoftmaxGradJob{0, 1, u - 4};
  if (h == 3) return u < 4 ? SoftmaxGradJob{1, 0, 8 + 2 * u} : SoftmaxGradJob{0, 1, u};
  if (h == 4) return u < 4 ? SoftmaxGradJob{1, 1, 2 * u} : SoftmaxGradJob{0, 1, 4 + u};
  return u < 4 ? SoftmaxGradJob{0, 1, 12 + u} : SoftmaxGradJob{1, 1, 8 + 2 * (u - 4)};
}
// Every element gets each stage once; a job runs behind the MFMA of its group, so stage A of block qb needs a group
// after the block's last S MFMA, stage B one after its last dP MFMA and a slot after the A jobs of its two elements, and
// the B operands of elements 8t .. 8t+7 must be complete in a group before the first gradient MFMA that reads them.
// (The wait states these distances need in instructions are checked on the generated code, fast_ops_amd/asm_lint.py.)
constexpr bool softmax_grad_jobs_fit(int nmf) {
  const int half = nmf / 2, ksteps = nmf / 2, spg = 48 / (3 * nmf);
  if (spg * 3 * nmf != 48) return false;
  int slot_a[2][16] = {}, slot_b[2][16] = {}, n_a[2][16] = {}, n_b[2][16] = {};
  for (int s = 0; s < 48; ++s) {
    const SoftmaxGradJob j = softmax_grad_job(s);
    if (j.qb < 0 || j.qb > 1 || j.r < 0 || j.r + j.stage > 15) return false;
    if (j.stage == 0) { slot_a[j.qb][j.r] = s; ++n_a[j.qb][j.r]; }
    else { slot_b[j.qb][j.r] = slot_b[j.qb][j.r + 1] = s; ++n_b[j.qb][j.r]; ++n_b[j.qb][j.r + 1]; }
  }
  for (int qb = 0; qb < 2; ++qb)
    for (int r = 0; r < 16; ++r) {
      if (n_a[qb][r] != 1 || n_b[qb][r] != 1) return false;
      const int ga = half + slot_a[qb][r] / spg, gb = half + slot_b[qb][r] / spg;     // the groups the jobs run in
      if (ga < qb * nmf + ksteps) return false;                                          // S complete
      if (gb < (qb + 1) * nmf || slot_b[qb][r] <= slot_a[qb][r]) return false;           // dP complete, P there
      if (gb >= (2 + qb) * nmf + (r / 8) * half) return false;                           // before its first reader
    }
  return true;
}
static_assert(softmax_grad_jobs_fit(16) && softmax_grad_jobs_fit(8), "head_dim 128 and 64");

// ---------------------------------------------------------------------------------------------------------------------
// dK/dV without dropout and bias, as a software pipeline. The accumulators of dK and dV, the K^T and V^T fragments and
// two blocks of scores leave room for one wave per SIMD only, and a lone wave issues in order: whatever arithmetic sits
// between two MFMAs keeps the matrix pipe waiting unless it is laid out to run beside them. A 64-query tile is two
// 32-query blocks and four phases of NMF MFMAs each:
//   1: S, then dP of block 0 | 2: S, then dP of block 1 | 3: dV, dK of block 0 | 4: dV, dK of block 1
// as micro-groups of one MFMA, the LDS read of the A operand needed kFragAhead groups later and a share of the tile's
// softmax-gradient arithmetic (see tile_body), fenced so that the compiler keeps the groups apart. The accumulators of
// S and dP do not start from zero but from -LSE / scale and -delta of their rows (written by the dQ kernel, read from
// LDS straight into the registers while they are idle), so that P = exp2((QK^T - LSE / scale) c) and dS = P (dP - delta)
// are two multiplications and the exponential.
// KBIAS: with a bias that is the same for every query (query stride 0): a lane owns a key, so the bias is one value per
// lane for the whole kernel, and P = exp2(S c + b log2 e) is a fused multiply-add where the form without bias multiplies.
template <typename T, int D, bool CAUSAL, bool KBIAS = false>
__global__ void __launch_bounds__(kBwdWaves * 64) attn_bwd_dkdv_pipe_kernel(const AttnBwdParams prm) {
  typedef typename Ops<T>::vec8 vec8;
  constexpr int TILE_BYTES = kBwdTile * D * 2;
  constexpr int KSTEPS = D / 16;
  constexpr int DBLK = D / 32;
  constexpr int NMF = 2 * KSTEPS;           // MFMAs per phase (= 4 * DBLK)
  static_assert(4 * DBLK == NMF, "phases of equal length");
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  constexpr int NBUF = 3;                   // tile buffers: see hand_over()
  FO_LDS char* smem = (FO_LDS char*)smem_raw;   // Q[NBUF] | dO[NBUF] | -LSE/scale[NBUF][64] | -delta[NBUF][64]
  FO_LDS float* rowvals = (FO_LDS float*)(smem + 2 * NBUF * TILE_BYTES);
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);
  const int lane = tid & 63, l32 = lane & 31, hh = lane >> 5;
  int bh, kblk;                                       // key block 0 has the most queries when causal: heaviest first
  bwd_item(prm, (prm.Sk + kBwdRows - 1) / kBwdRows, bh, kblk);
  const int b = bh / prm.H, h = bh % prm.H;
  const int k0 = kblk * kBwdRows, k0w = k0 + wave_s * 32;
  const int Sq = prm.Sq, Sk = prm.Sk;
  const T* qbase = (const T*)prm.q + b * prm.qs[0] + h * prm.qs[1];
  const T* gbase = (const T*)prm.d_o + b * prm.dos[0] + h * prm.dos[1];
  const int n_qt = (Sq + kBwdTile - 1) / kBwdTile;
  const int qt0 = CAUSAL ? min(k0 / kBwdTile, n_qt) : 0;     // queries before the block's first key never attend it
  const int ja = CAUSAL ? min(k0w / kBwdTile, n_qt) : 0;     // ... and this wave's keys start later still

  TileLaneOffsets<T, D> qlo, glo;
  qlo.init(prm.qs[2], prm.d, wave_s, lane);
  glo.init(prm.dos[2], prm.d, wave_s, lane);
  auto issue = [&](int qt, int buf) {
    if (qt * kBwdTile + kBwdTile <= Sq && qlo.ok && glo.ok) {
      copy_tile64_inside<T, D>(qbase, prm.qs[2], qt * kBwdTile, qlo, smem + buf * TILE_BYTES, wave_s);
      copy_tile64_inside<T, D>(gbase, prm.dos[2], qt * kBwdTile, glo, smem + (NBUF + buf) * TILE_BYTES, wave_s);
    } else {
      copy_tile64<T, D>(qbase, prm.qs[2], qt * kBwdTile, Sq, prm.d, smem + buf * TILE_BYTES, wave_s, lane);
      copy_tile64<T, D>(gbase, prm.dos[2], qt * kBwdTile, Sq, prm.d, smem + (NBUF + buf) * TILE_BYTES, wave_s, lane);
    }
    if (wave_s < 2) {
      const int64_t at = (int64_t)bh * Sq + min(qt * kBwdTile + lane, Sq - 1);
      dma4_lane_ptr((wave_s == 0 ? (const float*)prm.nlse : (const float*)prm.delta) + at, rowvals + (NBUF * wave_s + buf) * kBwdTile);
    }
  };
  if (qt0 < n_qt) issue(qt0, 0);
  // hand-over j, between phases 3 and 4 of tile j: tile j+1 (copy started one tile ago) has landed for everyone, and
  // since everyone is past phase 3 of tile j nobody reads tile j-1 any more, whose buffer - the third one - takes the
  // copy of tile j+2. Phase 4 still reads tile j, and already fetches the first fragments of tile j+1, so the fragment
  // pipeline never drains. Every wave runs hand-overs qt0-1 .. n_qt-2, each exactly once.
  auto hand_over = [&](int j) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    if (j + 2 < n_qt) issue(j + 2, (j + 2 - qt0) % NBUF);
  };

  // B operands held for the whole kernel: K^T and V^T fragments of this lane's key. The block's 128 rows of K and of V
  // come in like tiles - 16-byte pieces straight into LDS, into the buffers of the second and third tile, which are
  // still free - and each lane takes its row's pieces from there. (Read from global memory row by row, 32 rows per
  // instruction, this took 4.4 us, a quarter of a workgroup's time at 512 queries.) Rows past the end re-read the
  // last one, as the masks below expect. The barrier of the first hand-over comes after every wave has its fragments.
  vec8 kf[KSTEPS], vf[KSTEPS];
  {
    const T* kbase = (const T*)prm.k + b * prm.ks[0] + h * prm.ks[1];
    const T* vbase = (const T*)prm.v + b * prm.vs[0] + h * prm.vs[1];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      copy_tile64<T, D>(kbase, prm.ks[2], k0 + 64 * half, Sk, prm.d, smem + (1 + half) * TILE_BYTES, wave_s, lane);
      copy_tile64<T, D>(vbase, prm.vs[2], k0 + 64 * half, Sk, prm.d, smem + (NBUF + 1 + half) * TILE_BYTES, wave_s, lane);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    FO_LDS const char* kt = smem + (1 + (wave_s >> 1)) * TILE_BYTES;
    FO_LDS const char* vt = smem + (NBUF + 1 + (wave_s >> 1)) * TILE_BYTES;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) { kf[ks] = row_frag<T, D>(kt, wave_s & 1, ks, l32, hh); vf[ks] = row_frag<T, D>(vt, wave_s & 1, ks, l32, hh); }
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) asm volatile("" ::"v"(kf[ks]), "v"(vf[ks]));
  }
  const int key = k0w + l32;
  float bias_lane = 0.0f;
  if constexpr (KBIAS) {
    bias_lane = load_bias<T>(prm.bias, b * prm.bias.strides[0] + h * prm.bias.strides[1] + min(key, Sk - 1)) * kLog2e;
    asm volatile("" : "+v"(bias_lane));      // (waited for here, not inside the loops, where copies are in flight)
  }
  f32x16 dkacc[DBLK], dvacc[DBLK];
#pragma unroll
  for (int i = 0; i < DBLK; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) { dkacc[i][r] = 0.0f; dvacc[i][r] = 0.0f; }
  const float c = prm.scale_log2e, scale = prm.scale;

  // Per-lane byte offsets of the fragment reads inside a tile, swizzle included (what row_frag / col_frag compute; the
  // swizzle of a row does not depend on the 32-row block or 16-row step it is in). With the tile's base added once
  // per tile every read is register + immediate: block, step and the dO tiles (NBUF tiles behind the Q tiles) are
  // immediates.
  constexpr int ROW = D * 2;
  constexpr int G_OFF = NBUF * TILE_BYTES;
  uint32_t row_off[KSTEPS], col_off[DBLK][2];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) row_off[ks] = (uint32_t)(l32 * ROW + (((2 * ks + hh) ^ swz<D>(l32)) * 16));
  {
    const int L16 = lane & 15, g16 = (lane >> 4) & 1;
    const int r0 = 4 * hh + (L16 >> 2), r1 = r0 + 8, sub = (L16 & 1) * 8;
#pragma unroll
    for (int db = 0; db < DBLK; ++db) {
      const int chunk = 4 * db + 2 * g16 + ((L16 & 3) >> 1);
      col_off[db][0] = (uint32_t)(r0 * ROW + ((chunk ^ swz<D>(r0)) * 16) + sub);
      col_off[db][1] = (uint32_t)(r1 * ROW + ((chunk ^ swz<D>(r1)) * 16) + sub);
    }
  }
  // A operand of MFMA i of a scores phase (i < KSTEPS: Q rows for S, then dO rows for dP) / of a gradient phase (even i:
  // dO^T for dV, odd i: Q^T for dK); rq / cq = the offsets above plus the byte offset of the tile's Q buffer
  auto scores_frag_sd = [&](const uint32_t* rq, int qb, int i) -> vec8 {
    return *(FO_LDS const vec8*)(smem + rq[i % KSTEPS] + (i >= KSTEPS ? G_OFF : 0) + qb * 32 * ROW);
  };
  auto grads_frag = [&](const uint32_t (*cq)[2], int qb, int i) -> vec8 {
    const int tp = 2 * qb + i / (2 * DBLK), db = (i >> 1) % DBLK;
    const int imm = ((i & 1) ? 0 : G_OFF) + 16 * tp * ROW;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FO_LDS s16x4*)(smem + cq[db][0] + imm));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FO_LDS s16x4*)(smem + cq[db][1] + imm));
    return __builtin_bit_cast(vec8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  constexpr int kFragAhead = 4;
  static_assert((4 * NMF) % kFragAhead == 0, "the fragment ring runs on across tiles");
  vec8 fr[kFragAhead];         // A operands, fetched kFragAhead micro-groups ahead of their MFMA
  f32x16 sacc[2], dpacc[2];
  // P and dS as B operands: pairs of 16-bit values, kept as 32-bit words so that a finished pair can be pinned
  typedef __attribute__((ext_vector_type(4))) int i32x4;
  typedef __attribute__((ext_vector_type(2))) T vec2;
  i32x4 pf[2][2], dsf[2][2];

  const uint32_t lane4 = (uint32_t)lane * 4u;
  // One tile. `buf`: the tile's buffer, (j - qt0) % NBUF, which the caller counts along. `spread`: tile j+2 lies wholly
  // inside Q and dO (and the lane offsets fit): its copy is not issued in one batch at the hand-over but one instruction
  // at a time between the MFMAs of phase 4 (a batch of direct-to-LDS copies holds the wave's issue port for hundreds of
  // cycles while the matrix pipe runs dry; one copy per two MFMAs hides behind them).
  // The softmax-gradient arithmetic is spread evenly over the tile's micro-groups: a lone wave hides about five VALU
  // instructions behind a 32-cycle MFMA (an exponential counts as four) and pays in full for every further one, and with
  // a whole score element (multiply, exponential, multiply, rounding) beside each MFMA of phases 2 and 3 and nothing
  // beside those of phases 1 and 4, half of the groups ran at 1.7-2x the MFMA time. So the scores of a block come first
  // (S: KSTEPS MFMAs, then dP: KSTEPS MFMAs), an element is split into stage A (P = exp2(S c), needs S only) and stage B
  // (dS = P dP, both rounded to B operands; two elements at a time), and the 32 A and 16 B jobs of a tile fill 48 slots
  // laid over the groups from the middle of phase 1 to the middle of phase 4 (one slot per group at head_dim 128, two at
  // 64) in an order that meets every producer and consumer (dK/dV kernel: -12 % cycles, -5.5 % time at head_dim 128):
  //   half-phase   MFMAs            slots
  //   0            S0               -
  //   1            dP0              A0[0..7]
  //   2            S1               A0[8..15]
  //   3            dP1              B0[0..7], A1[0..3]
  //   4            dV0,dK0 (t=0)    B0[8..15], A1[4..7]
  //   5            dV0,dK0 (t=1)    B1[0..7], A1[8..11]
  //   6            dV1,dK1 (t=0)    A1[12..15], B1[8..15]
  //   7            dV1,dK1 (t=1)    -
  auto tile_body = [&](int j, int buf, auto masked, auto spread) __attribute__((always_inline)) {
    constexpr bool SPREAD = decltype(spread)::value;
    constexpr int HALF = NMF / 2, NG = 4 * NMF, SPG = 48 / (3 * NMF);      // groups per half-phase / per tile, slots per group
    static_assert(SPG * 3 * NMF == 48 && kFragAhead <= KSTEPS, "48 slots over the groups of six half-phases");
    const int nbuf = buf == NBUF - 1 ? 0 : buf + 1;
    const int q0t = j * kBwdTile;
    uint32_t rq[KSTEPS], cq[DBLK][2], rq_next[kFragAhead];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) { rq[ks] = row_off[ks] + (uint32_t)(buf * TILE_BYTES); asm volatile("" : "+v"(rq[ks])); }
#pragma unroll
    for (int db = 0; db < DBLK; ++db)
#pragma unroll
      for (int u = 0; u < 2; ++u) { cq[db][u] = col_off[db][u] + (uint32_t)(buf * TILE_BYTES); asm volatile("" : "+v"(cq[db][u])); }
#pragma unroll
    for (int ks = 0; ks < kFragAhead; ++ks) { rq_next[ks] = row_off[ks] + (uint32_t)(nbuf * TILE_BYTES); asm volatile("" : "+v"(rq_next[ks])); }
    auto frag = [&](int g) -> vec8 {
      const int ph = g / NMF, i = g % NMF;
      return ph < 2 ? scores_frag_sd(rq, ph, i) : grads_frag(cq, ph - 2, i);
    };
    auto refill = [&](int g) {
      fr[g % kFragAhead] = g + kFragAhead < NG ? frag(g + kFragAhead) : scores_frag_sd(rq_next, 0, g + kFragAhead - NG);
    };
    // an accumulator's start values, straight from LDS into its registers
    auto start_acc = [&](f32x16& acc, FO_LDS const float* rows, int qb) {
#pragma unroll
      for (int jv = 0; jv < 4; ++jv) {
        const f32x4 d4 = *(FO_LDS const f32x4*)(rows + 32 * qb + 8 * jv + 4 * hh);
#pragma unroll
        for (int u = 0; u < 4; ++u) acc[4 * jv + u] = d4[u];
      }
    };
    float pv[2][16];            // P of a block between its two stages
    auto stage_a = [&](int qb, int r) {
      const int koff = (r & 3) + 8 * (r >> 2);
      bool dead = false;
      if constexpr (decltype(masked)::value) {
        const int lim = CAUSAL ? key - (q0t + 32 * qb + 4 * hh) : 0;
        const int lim_end = Sq - (q0t + 32 * qb + 4 * hh);
        dead = koff < lim || koff >= lim_end;
      }
      pv[qb][r] = dead ? 0.0f : __builtin_amdgcn_exp2f(KBIAS ? __builtin_fmaf(sacc[qb][r], c, bias_lane) : sacc[qb][r] * c);
    };
    auto stage_b = [&](int qb, int r) {          // elements r and r + 1
      const float ds0 = pv[qb][r] * dpacc[qb][r], ds1 = pv[qb][r + 1] * dpacc[qb][r + 1];
      const vec2 p2 = {(T)pv[qb][r], (T)pv[qb][r + 1]}, ds2 = {(T)ds0, (T)ds1};
      int pw = __builtin_bit_cast(int, p2), dsw = __builtin_bit_cast(int, ds2);
      // (pinned to its micro-group: left alone, the compiler moves the multiplications and the rounding down to the MFMA
      // that reads them, which may not read a register that a VALU instruction has just written)
      asm volatile("" : "+v"(pw), "+v"(dsw));
      pf[qb][r >> 3][(r & 7) >> 1] = pw;
      dsf[qb][r >> 3][(r & 7) >> 1] = dsw;
    };
    auto slot = [&](int s) {
      const SoftmaxGradJob job = softmax_grad_job(s);      // (s is a constant once the loop is unrolled)
      if (job.stage == 0) stage_a(job.qb, job.r); else stage_b(job.qb, job.r);
    };
    const char* next_q = nullptr;
    const char* next_g = nullptr;
    const char* next_rows = nullptr;
    uint32_t next_q_dst = 0;
    FO_LDS char* next_rows_dst = nullptr;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      const int ph = g / NMF, i = g % NMF;
      if (g == 3 * NMF) {
        // the hand-over, between phases 3 and 4 (see hand_over)
        if constexpr (SPREAD) {
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          __builtin_amdgcn_s_barrier();
          const int b2 = buf == 0 ? NBUF - 1 : buf - 1, which = wave_s & 1;   // (waves 2 and 3 repeat the row values of waves 0 and 1)
          next_q = (const char*)(qbase + (int64_t)(j + 2) * kBwdTile * prm.qs[2]);
          next_g = (const char*)(gbase + (int64_t)(j + 2) * kBwdTile * prm.dos[2]);
          next_rows = (const char*)((which ? (const float*)prm.delta : (const float*)prm.nlse) + (int64_t)bh * Sq + (j + 2) * kBwdTile);
          next_q_dst = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(smem + b2 * TILE_BYTES + wave_s * (TileLaneOffsets<T, D>::N * 1024)));
          next_rows_dst = (FO_LDS char*)(rowvals + (NBUF * which + b2) * kBwdTile);
        } else {
          if (j + 1 < n_qt) hand_over(j);
        }
      }
      // (two wait states where an MFMA may follow the VALU instruction that wrote its B operand: behind the hand-over,
      // whose paths join here, and where the last B job of the tile ends right before its first reader)
      if (g == 3 * NMF || g == 3 * NMF + HALF) asm volatile("s_nop 1");
      if (ph < 2) {
        if (i < KSTEPS) mfma_scores_vgpr<T>(sacc[ph], fr[g % kFragAhead], kf[i]);
        else mfma_scores_vgpr<T>(dpacc[ph], fr[g % kFragAhead], vf[i - KSTEPS]);
      } else {
        const int t = i / (2 * DBLK), db = (i >> 1) % DBLK;
        if (i & 1) mfma_acc_agpr<T>(dkacc[db], fr[g % kFragAhead], __builtin_bit_cast(vec8, dsf[ph - 2][t]));
        else mfma_acc_agpr<T>(dvacc[db], fr[g % kFragAhead], __builtin_bit_cast(vec8, pf[ph - 2][t]));
      }
      refill(g);
      // start values of the accumulators while they are idle: block 1 of this tile, block 0 of the next (visible since
      // the hand-over; after the last tile: read, unused)
      if (g == 0) start_acc(dpacc[1], rowvals + (NBUF + buf) * kBwdTile, 1);
      if (g == 1) start_acc(sacc[1], rowvals + buf * kBwdTile, 1);
      if (g == 3 * NMF) start_acc(dpacc[0], rowvals + (NBUF + nbuf) * kBwdTile, 0);
      if (g == 3 * NMF + 1) start_acc(sacc[0], rowvals + nbuf * kBwdTile, 0);
      if constexpr (SPREAD) {
        if (ph == 3) {
          constexpr int N = TileLaneOffsets<T, D>::N, EVERY = NMF / (2 * N);
          static_assert(EVERY >= 1 && 2 * N * EVERY == NMF && 2 * N <= 8, "one copy per EVERY micro-groups");
          auto copy_piece = [&](auto pc) {
            constexpr int piece = decltype(pc)::value;
            if constexpr (piece < N) dma16_uniform_base_lds_imm<piece * 1024>(next_q, qlo.off[piece], next_q_dst);
            else if constexpr (piece < 2 * N) dma16_uniform_base_lds_imm<NBUF * TILE_BYTES + (piece - N) * 1024>(next_g, glo.off[piece - N], next_q_dst);
          };
          if (i % EVERY == EVERY - 1) {
            switch (i / EVERY) {      // (a constant once the loop is unrolled)
              case 0: copy_piece(std::integral_constant<int, 0>{}); break;
              case 1: copy_piece(std::integral_constant<int, 1>{}); break;
              case 2: copy_piece(std::integral_constant<int, 2>{}); break;
              case 3: copy_piece(std::integral_constant<int, 3>{}); break;
              case 4: copy_piece(std::integral_constant<int, 4>{}); break;
              case 5: copy_piece(std::integral_constant<int, 5>{}); break;
              case 6: copy_piece(std::integral_constant<int, 6>{}); break;
              default: copy_piece(std::integral_constant<int, 7>{}); break;
            }
          }
          if (i == 0) dma4_uniform_base(next_rows, lane4, next_rows_dst);
        }
      }
      if (g >= HALF && g < NG - HALF) {
        // (S of block 0 was finished by the MFMA before this group's: that one and four wait states cover the 11 its
        // result needs before a VALU instruction may read it; every later first read is several MFMAs behind)
        if (g == HALF) asm volatile("s_nop 3" : "+v"(sacc[0]));
#pragma unroll
        for (int u = 0; u < SPG; ++u) slot((g - HALF) * SPG + u);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  int j = qt0 - 1;
  for (; j <= min(ja, n_qt) - 1 && j <= n_qt - 2; ++j) hand_over(j);
  // Tiles that need the mask are a prefix (the causal diagonal) and possibly the last tile (queries past the end).
  // One loop per kind, each with a single body: with alternatives inside one loop the compiler moves the 128
  // accumulator registers between homes at every tile.
  auto needs_mask = [&](int jt) { return jt * kBwdTile + kBwdTile > Sq || (CAUSAL && k0w + 31 > jt * kBwdTile); };
  j = ja;
  if (j < n_qt) {
    const int buf = (j - qt0) % NBUF;
    uint32_t rq0[kFragAhead];
#pragma unroll
    for (int ks = 0; ks < kFragAhead; ++ks) rq0[ks] = row_off[ks < KSTEPS ? ks : 0] + (uint32_t)(buf * TILE_BYTES);
#pragma unroll
    for (int i = 0; i < kFragAhead; ++i) fr[i] = scores_frag_sd(rq0, 0, i);
    // (dP of the first tile's block 0 starts from -delta, as every later one does at the end of the tile before it)
#pragma unroll
    for (int jv = 0; jv < 4; ++jv) {
      const f32x4 d4 = *(FO_LDS const f32x4*)(rowvals + (NBUF + buf) * kBwdTile + 8 * jv + 4 * hh);
#pragma unroll
      for (int u = 0; u < 4; ++u) dpacc[0][4 * jv + u] = d4[u];
      const f32x4 n4 = *(FO_LDS const f32x4*)(rowvals + buf * kBwdTile + 8 * jv + 4 * hh);
#pragma unroll
      for (int u = 0; u < 4; ++u) sacc[0][4 * jv + u] = n4[u];
    }
  }
  int buf = j < n_qt ? (j - qt0) % NBUF : 0;
  auto next_buf = [&]() { buf = buf == NBUF - 1 ? 0 : buf + 1; };
  for (; j < n_qt && needs_mask(j); ++j, next_buf()) tile_body(j, buf, std::true_type{}, std::false_type{});
#if FO_BWD_SPREAD
  // (from here on only a last tile that crosses the end of Q needs the mask; tiles j with tile j+2 wholly inside Q)
  if (qlo.ok && glo.ok)
    for (const int end = Sq / kBwdTile - 2; j < end; ++j, next_buf()) tile_body(j, buf, std::false_type{}, std::true_type{});
#endif
  for (; j < n_qt && !needs_mask(j); ++j, next_buf()) tile_body(j, buf, std::false_type{}, std::false_type{});
  for (; j < n_qt; ++j, next_buf()) tile_body(j, buf, std::true_type{}, std::false_type{});

  acc_fence(dkacc);
  acc_fence(dvacc);
  // (the tile buffers are free once every wave is past its last tile; dK, then dV, through the wave's own piece of them)
  __syncthreads();
  {
    FO_LDS char* stage = smem + wave_s * stage_bytes(D);
    const int k0w_s = k0 + wave_s * 32;
    store_rows_via_lds<T, D>(dkacc, scale, stage, (T*)prm.dk + b * prm.dks[0] + h * prm.dks[1], prm.dks[2], k0w_s, Sk, prm.d, lane);
    store_rows_via_lds<T, D>(dvacc, 1.0f, stage, (T*)prm.dv + b * prm.dvs[0] + h * prm.dvs[1], prm.dvs[2], k0w_s, Sk, prm.d, lane);
  }
}

template <typename T, int D, bool CAUSAL, bool DROP, bool BIAS>
static int launch_bwd(const AttnBwdParams& p, hipStream_t s) {
  const int64_t n_bh = (int64_t)p.B * p.H;
  const int64_t g_dq = ((p.Sq + kBwdRows - 1) / kBwdRows) * n_bh;
  const int64_t g_dkdv = ((p.Sk + kBwdRows - 1) / kBwdRows) * n_bh;
  if (g_dq > 0x7FFFFFFFll || g_dkdv > 0x7FFFFFFFll) return FO_ERR_BAD_SHAPE;
  const size_t lds_tiles = 4 * (size_t)kBwdTile * D * 2;
  const size_t lds_dq = lds_tiles + (BIAS ? 512 : 0);   // + the per-key bias of two tiles (both bias forms)
  const size_t lds_dkdv = lds_tiles + 4 * kBwdTile * sizeof(float) + (BIAS ? kBwdWaves * 2 * kBwdTile * 32 * 4 : 0);   // + bias tiles
  static const hipError_t a1 = hipFuncSetAttribute((const void*)attn_bwd_dq_kernel<T, D, CAUSAL, DROP, BIAS>,
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_dq);
  static const hipError_t a2 = hipFuncSetAttribute((const void*)attn_bwd_dkdv_kernel<T, D, CAUSAL, DROP, BIAS>,
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_dkdv);
  const size_t lds_pipe = 6 * (size_t)kBwdTile * D * 2 + 6 * kBwdTile * sizeof(float);   // three tile buffers
  static const hipError_t a3 = hipFuncSetAttribute((const void*)attn_bwd_dkdv_pipe_kernel<T, D, CAUSAL>,
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_pipe);
  if (a1 != hipSuccess || a2 != hipSuccess || a3 != hipSuccess) return FO_ERR_LAUNCH;
  // a bias without a query stride: the forms of the dQ kernel and (without dropout) of the pipelined dK/dV kernel that
  // take it at no cost per score (attn_bwd.variant 0 keeps the general bias kernels, which tests compare them with)
  const bool key_bias = BIAS && p.bias.strides[2] == 0 && tune(g_attn_bwd_variant) != 0;
  if constexpr (BIAS) {
    static const hipError_t a4 = hipFuncSetAttribute((const void*)attn_bwd_dq_kernel<T, D, CAUSAL, DROP, false, true>,
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_dq);
    static const hipError_t a5 = hipFuncSetAttribute((const void*)attn_bwd_dkdv_pipe_kernel<T, D, CAUSAL, true>,
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_pipe);
    if (a4 != hipSuccess || a5 != hipSuccess) return FO_ERR_LAUNCH;
  }
  // one group while the Q, dO, K and V of all heads fit the memory-side cache (256 MiB), else groups of heads whose
  // operands stay within a quarter of it; multiples of 8 so that a head's workgroups keep landing on one XCD
  // (B=16 H=32 S=2048 D=128 causal: 2.61 ms in one group, 2.23 ms in groups of 32; the headline shape, 256 MiB: 1.80 ms
  // in one group, 1.90 ms in groups of 8)
  AttnBwdParams q = p;
  {
    const int64_t bytes_head = 2 * ((int64_t)p.Sq + p.Sk) * D * 2;
    const int order = tune(g_attn_bwd_order);
    int64_t group = order >= 0 ? order : bytes_head * n_bh <= (256ll << 20) ? n_bh : ((64ll << 20) / bytes_head) & ~7ll;
    if (order < 0 && group < 8) group = 8;
    if (group <= 0 || group > n_bh) group = n_bh;
    q.head_group = (int)group;
  }
  // (delta is computed by the dQ kernel, which the dK/dV kernel follows)
  if constexpr (BIAS) {
    if (key_bias) {
      attn_bwd_dq_kernel<T, D, CAUSAL, DROP, false, true><<<(unsigned)g_dq, kBwdWaves * 64, lds_dq, s>>>(q);
      if (!DROP && p.d == D) attn_bwd_dkdv_pipe_kernel<T, D, CAUSAL, true><<<(unsigned)g_dkdv, kBwdWaves * 64, lds_pipe, s>>>(q);
      else attn_bwd_dkdv_kernel<T, D, CAUSAL, DROP, BIAS><<<(unsigned)g_dkdv, kBwdWaves * 64, lds_dkdv, s>>>(q);
      return launch_status();
    }
  }
  attn_bwd_dq_kernel<T, D, CAUSAL, DROP, BIAS><<<(unsigned)g_dq, kBwdWaves * 64, lds_dq, s>>>(q);
  // attn_bwd.variant 0 selects the plain dK/dV kernel everywhere (tests compare the two)
  // (and every head_dim other than the two the kernels are compiled for)
  if (!DROP && !BIAS && p.d == D && tune(g_attn_bwd_variant) != 0) attn_bwd_dkdv_pipe_kernel<T, D, CAUSAL><<<(unsigned)g_dkdv, kBwdWaves * 64, lds_pipe, s>>>(q);
  else attn_bwd_dkdv_kernel<T, D, CAUSAL, DROP, BIAS><<<(unsigned)g_dkdv, kBwdWaves * 64, lds_dkdv, s>>>(q);
  return launch_status();
}

// every kernel of one operand type and head_dim behind one function, which one translation unit defines (see below)
template <typename T, int D>
int launch_bwd_of(const AttnBwdParams& p, bool causal, bool drop, bool has_bias, hipStream_t s) {
  if (has_bias) {
    if (drop) return causal ? launch_bwd<T, D, true, true, true>(p, s) : launch_bwd<T, D, false, true, true>(p, s);
    return causal ? launch_bwd<T, D, true, false, true>(p, s) : launch_bwd<T, D, false, false, true>(p, s);
  }
  if (drop) return causal ? launch_bwd<T, D, true, true, false>(p, s) : launch_bwd<T, D, false, true, false>(p, s);
  return causal ? launch_bwd<T, D, true, false, false>(p, s) : launch_bwd<T, D, false, false, false>(p, s);
}
// This file is compiled several times, in parallel: as it stands it is the C ABI and holds no kernel;
// attn_bwd_bf16_d64.hip ... attn_bwd_f16_d128.hip include it with FO_ATTN_UNIT set and instantiate launch_bwd_of<T, D>.
#ifndef FO_ATTN_UNIT
#define FO_ATTN_UNIT 0
#endif
#define FO_ATTN_LAUNCH(UNIT, T, D) \
  FO_ATTN_EXTERN_##UNIT template int launch_bwd_of<T, D>(const AttnBwdParams&, bool, bool, bool, hipStream_t);
#if FO_ATTN_UNIT == 1
#define FO_ATTN_EXTERN_1
#else
#define FO_ATTN_EXTERN_1 extern
#endif
#if FO_ATTN_UNIT == 2
#define FO_ATTN_EXTERN_2
#else
#define FO_ATTN_EXTERN_2 extern
#endif
#if FO_ATTN_UNIT == 3
#define FO_ATTN_EXTERN_3
#else
#define FO_ATTN_EXTERN_3 extern
#endif
#if FO_ATTN_UNIT == 4
#define FO_ATTN_EXTERN_4
#else
#define FO_ATTN_EXTERN_4 extern
#endif
FO_ATTN_LAUNCH(1, __bf16, 64)
FO_ATTN_LAUNCH(2, __bf16, 128)
FO_ATTN_LAUNCH(3, _Float16, 64)
FO_ATTN_LAUNCH(4, _Float16, 128)

}  // namespace fo

#if FO_ATTN_UNIT == 0
using namespace fo;

// ---- the same without a workspace argument and without any allocation: the workspace is a device array of this library.
// The array's name is only a host-side handle for the device symbol; its address on a device comes from
// hipGetSymbolAddress, asked once per device with that device current, and only that pointer is handed to the kernels.
constexpr int64_t kStaticDeltaFloats = FO_ATTN_BWD_STATIC_ROWS;
static __device__ __align__(256) float scratch[2 * kStaticDeltaFloats];   // two values per row: see AttnBwdParams
constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static float* g_scratch_ptr[kMaxDevices];   // per device; null until that device's first call

static int scratch_of_current_device(float** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return FO_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) return FO_ERR_LAUNCH;
    g_scratch_ptr[dev] = static_cast<float*>(ptr);
  }
  *out = g_scratch_ptr[dev];
  return FO_OK;
}

static int attn_bwd_impl(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                         float* delta_ws, void* dq, void* dk, void* dv, int B, int H, int Sq, int Sk, int D,
                         const int64_t* const* strides_host, float softmax_scale, int causal, int dtype, float dropout_p,
                         uint32_t seed, uint64_t rng_offset, const void* bias, const int64_t* bias_strides, int bias_dtype,
                         void* stream, bool static_ws = false) {
  // static_ws: delta_ws is ignored and the library's own per-device array takes its place (fo_attn_bwd_static_ws)
  if (!q || !k || !v || !o || !d_o || !lse || (!delta_ws && !static_ws) || !dq || !dk || !dv || !strides_host) return FO_ERR_NULL_POINTER;
  for (int t = 0; t < 8; ++t)
    if (!strides_host[t]) return FO_ERR_NULL_POINTER;
  if (dtype != FO_DTYPE_F16 && dtype != FO_DTYPE_BF16) return FO_ERR_BAD_DTYPE;
  if (D < 8 || D > 128 || D % 8 != 0) return FO_ERR_BAD_HEAD_DIM;
  if (B <= 0 || H <= 0 || Sq <= 0 || Sk <= 0 || (int64_t)B * H * Sq > (1ll << 40)) return FO_ERR_BAD_SHAPE;
  for (int t = 0; t < 8; ++t) {
    // rows start on 16-byte boundaries (8 elements); only the inputs K and V may repeat a head (stride 0 = multi-query)
    for (int i = 0; i < 3; ++i)
      if (strides_host[t][i] < 0 || (strides_host[t][i] % 8) != 0) return FO_ERR_BAD_STRIDE;
    if (strides_host[t][2] < D) return FO_ERR_BAD_STRIDE;
    const bool output = t >= 5;
    if (output && ((strides_host[t][0] == 0 && B > 1) || (strides_host[t][1] == 0 && H > 1))) return FO_ERR_BAD_STRIDE;
  }
  const uintptr_t all = (uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o | (uintptr_t)d_o | (uintptr_t)dq | (uintptr_t)dk | (uintptr_t)dv;
  if (all & 15u) return FO_ERR_MISALIGNED;
  if (((uintptr_t)lse | (static_ws ? 0 : (uintptr_t)delta_ws)) & 3u) return FO_ERR_MISALIGNED;
  if (!(softmax_scale > 0.0f) || softmax_scale > 3.0e38f) return FO_ERR_BAD_SHAPE;
  if (!(dropout_p >= 0.0f) || dropout_p >= 1.0f) return FO_ERR_BAD_SHAPE;
  if (bias) {
    if (!bias_strides) return FO_ERR_NULL_POINTER;
    if (bias_dtype != FO_DTYPE_F32 && bias_dtype != dtype) return FO_ERR_BAD_DTYPE;
    if (bias_strides[0] < 0 || bias_strides[1] < 0 || bias_strides[2] < 0) return FO_ERR_BAD_STRIDE;
    if ((uintptr_t)bias & (bias_dtype == FO_DTYPE_F32 ? 3u : 1u)) return FO_ERR_MISALIGNED;
  }
  if (static_ws) {
    // (after every argument check: a rejected call has made no HIP call)
    if ((int64_t)B * H * Sq > kStaticDeltaFloats) return FO_ERR_BAD_SHAPE;
    const int st = scratch_of_current_device(&delta_ws);
    if (st != FO_OK) return st;
  }

  AttnBwdParams p;
  p.q = q; p.k = k; p.v = v; p.o = o; p.d_o = d_o; p.lse = lse; p.delta = delta_ws; p.nlse = delta_ws + (int64_t)B * H * Sq; p.dq = dq; p.dk = dk; p.dv = dv;
  p.B = B; p.H = H; p.Sq = Sq; p.Sk = Sk; p.d = D;
  int64_t* dst[8] = {p.qs, p.ks, p.vs, p.os, p.dos, p.dqs, p.dks, p.dvs};
  for (int t = 0; t < 8; ++t)
    for (int i = 0; i < 3; ++i) dst[t][i] = strides_host[t][i];
  p.scale = softmax_scale;
  p.scale_log2e = softmax_scale * kLog2e;
  p.neg_inv_scale_log2e = -1.0f / p.scale_log2e;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool c = causal != 0, drop = dropout_p > 0.0f;
  p.drop = make_dropout(dropout_p, seed, rng_offset);
  p.bias.ptr = bias;
  for (int i = 0; i < 3; ++i) p.bias.strides[i] = bias ? bias_strides[i] : 0;
  p.bias.is_f32 = bias_dtype == FO_DTYPE_F32;
  {
    const uintptr_t elt = p.bias.is_f32 ? 4 : 2;
    // (dK/dV kernel: tiles of the bias are copied into LDS in 16-byte pieces)
    p.bias.dma_ok = bias && p.bias.strides[2] != 0 && ((uintptr_t)bias % 16) == 0 && (p.bias.strides[0] * elt) % 16 == 0 &&
                    (p.bias.strides[1] * elt) % 16 == 0 && (p.bias.strides[2] * elt) % 16 == 0;
    p.bias.vec_ok = bias && ((uintptr_t)bias % (4 * elt)) == 0 && p.bias.strides[0] % 4 == 0 && p.bias.strides[1] % 4 == 0 && p.bias.strides[2] % 4 == 0;
  }
  // kernels are compiled for 64 and 128 columns; a head_dim in between runs on the next one with zero columns
  const bool has_bias = bias != nullptr;
  if (dtype == FO_DTYPE_BF16) return D > 64 ? launch_bwd_of<__bf16, 128>(p, c, drop, has_bias, s) : launch_bwd_of<__bf16, 64>(p, c, drop, has_bias, s);
  return D > 64 ? launch_bwd_of<_Float16, 128>(p, c, drop, has_bias, s) : launch_bwd_of<_Float16, 64>(p, c, drop, has_bias, s);
}

extern "C" int fo_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                           float* delta_ws, void* dq, void* dk, void* dv, int B, int H, int Sq, int Sk, int D,
                           const int64_t* const* strides_host, float softmax_scale, int causal, int dtype, void* stream) {
  return attn_bwd_impl(q, k, v, o, d_o, lse, delta_ws, dq, dk, dv, B, H, Sq, Sk, D, strides_host, softmax_scale, causal, dtype,
                       0.0f, 0u, 0ull, nullptr, nullptr, 0, stream);
}

extern "C" int fo_attn_bwd_static_ws(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                                     void* dq, void* dk, void* dv, int B, int H, int Sq, int Sk, int D,
                                     const int64_t* const* strides_host, float softmax_scale, int causal, int dtype, void* stream) {
  // Every delta element the dK/dV kernel reads (rows below Sq of each head) is written by the dQ kernel of the same
  // call, so what an earlier call left in the array does not matter and nothing has to be cleared.
  return attn_bwd_impl(q, k, v, o, d_o, lse, nullptr, dq, dk, dv, B, H, Sq, Sk, D, strides_host, softmax_scale, causal, dtype,
                       0.0f, 0u, 0ull, nullptr, nullptr, 0, stream, true);
}

extern "C" int fo_attn_bwd_dropout(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                                   float* delta_ws, void* dq, void* dk, void* dv, int B, int H, int Sq, int Sk, int D,
                                   const int64_t* const* strides_host, float softmax_scale, int causal, int dtype,
                                   float dropout_p, uint32_t seed, uint64_t rng_offset, void* stream) {
  return attn_bwd_impl(q, k, v, o, d_o, lse, delta_ws, dq, dk, dv, B, H, Sq, Sk, D, strides_host, softmax_scale, causal, dtype,
                       dropout_p, seed, rng_offset, nullptr, nullptr, 0, stream);
}

extern "C" int fo_attn_bwd_ex(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                              float* delta_ws, void* dq, void* dk, void* dv, int B, int H, int Sq, int Sk, int D,
                              const int64_t* const* strides_host, float softmax_scale, int causal, int dtype,
                              const fo_attn_extras* extras, void* stream) {
  if (!extras)
    return attn_bwd_impl(q, k, v, o, d_o, lse, delta_ws, dq, dk, dv, B, H, Sq, Sk, D, strides_host, softmax_scale, causal, dtype,
                         0.0f, 0u, 0ull, nullptr, nullptr, 0, stream);
  return attn_bwd_impl(q, k, v, o, d_o, lse, delta_ws, dq, dk, dv, B, H, Sq, Sk, D, strides_host, softmax_scale, causal, dtype,
                       extras->dropout_p, extras->dropout_seed, extras->dropout_offset, extras->bias, extras->bias_strides,
                       extras->bias_dtype, stream);
}
#endif  // FO_ATTN_UNIT == 0
