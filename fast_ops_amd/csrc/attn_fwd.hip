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
// Two kernels. Common to both:
//   * The scores are computed transposed, S^T = K Q^T (A operand = K from LDS, B operand = Q^T held in registers for
//     the whole kernel). In the 32x32 accumulator layout a lane then owns ONE query column and 16 of the 32 keys, so
//     the row max / row sum are in-lane reductions plus one exchange between the two half-waves, and the accumulator
//     registers are, as they stand, the B operand of O^T = V^T P^T. P never touches LDS.
//   * V^T as an A operand needs 8 keys per lane for one d: read from the row-major V tile with the gfx950
//     transposing LDS load (ds_read_b64_tr_b16).
//   * K/V tiles (64 keys) go global -> LDS with the direct-to-LDS loads (16 B per lane, no VGPR staging).
//   * Workgroup order: heads are dealt to the 8 XCDs (workgroup ids round-robin over XCDs), each XCD walks one head
//     at a time, so an XCD's L2 holds the K/V it is streaming.
// attn_fwd_kernel (small or very long inputs; bias and dropout): one workgroup = 4 waves = 128 query
//   rows, two workgroups per CU, compiler-scheduled MFMA builtins, tiles double buffered with one barrier per tile,
//   16-byte chunks XOR-swizzled inside a row so that both the K reads (32 rows x one chunk) and the V reads (4 rows x
//   4 chunks) are free of bank conflicts; heaviest (last) causal query blocks first.
// attn_fwd_wide_kernel (the default once a shape gives every CU a workgroup): 256 query rows per workgroup, one
//   workgroup per CU (two fit for head_dim 64), MFMAs as inline assembly
//   with the accumulators of O and the fragments of Q in AGPRs, a three-deep software pipeline over 32-key sub-tiles
//   laid out as micro-groups of one MFMA plus its share of everything else; described where it is defined.
#include <type_traits>

#include "attn_common.hpp"

// This file is compiled several times, in parallel: as it stands it is the C ABI and the kernel choice, and holds no
// kernel; attn_fwd_bf16_d64.hip ... attn_fwd_f16_d128.hip include it with FO_ATTN_UNIT set and instantiate launch<T, D>,
// i.e. every kernel of one operand type and head_dim (the kernels are what takes the compiler's time).
#ifndef FO_ATTN_UNIT
#define FO_ATTN_UNIT 0
#endif

namespace fo {

constexpr int kWaves = 4;
constexpr int kBM = 32 * kWaves;   // query rows per workgroup
constexpr int kBN = 64;            // keys per tile

constexpr int kOrderTab = 128;

struct AttnParams {
  const void* q; const void* k; const void* v; void* o; float* lse;
  int B, H, Sq, Sk;
  int d;                                // true head_dim: a multiple of 8, at most the D the kernel is compiled for (128-row kernel only)
  int64_t qs[3], ks[3], vs[3], os[3];   // element strides: batch, head, sequence
  float scale_log2e;                    // softmax_scale * log2(e)
  int n_qblk;
  int heavy_first;                      // 128-row kernel, causal: heads per group in the order of an XCD's workgroups, 0 = head by head (see launch_one)
  int order_n;                          // 128-row kernel, causal: entries of order_tab in use, 0 = none
  int id_limit;                         // 256-row kernel: work items [0, id_limit) only (0 = all): the rest goes to a launch of the 128-row form
  int tail_base;                        // 128-row pipelined form, non-causal: > 0 = this launch takes the 256-row work items from tail_base on, two workgroups each
  int keep_on;                          // 256-row kernel without bias: non-zero = copy the next query block's first tiles during the last tiles of a block
  uint8_t order_tab[kOrderTab];         // position in an XCD's launch order -> rank of the workgroup (0 = heaviest) that runs there
  DropoutParams drop;                   // used by the kernels instantiated with dropout only
  BiasParams bias;                      // used by the kernels instantiated with bias only
};

constexpr int64_t kMaxRowStride = 1ll << 24;   // elements; see attn_fwd_impl
constexpr float kLazyLog2 = 8.0f;   // how far (in log2 units) a tile maximum may exceed the reference before a rescale

// KBIAS (without BIAS): a bias that is the same for every query (query stride 0) at no cost per score. The 64 values of a
// key tile, divided by softmax_scale, are what the score accumulators start from (register r of a lane holds a key that
// depends on r and the half of the wave only), so the MFMAs deliver S + b / scale and the rest is the code without bias.
// Wave 0 fetches the values of tile t+2 while tile t is worked on (a plain load, waited for at the top of the next tile,
// where every copy in flight is waited for anyway), converts those of tile t+1 and puts them into LDS for everyone.
template <typename T, int D, bool CAUSAL, bool LAZY, int DBG, bool DROP = false, bool BIAS = false, bool KBIAS = false>
__global__ void __launch_bounds__(kWaves * 64, 2) attn_fwd_kernel(const AttnParams prm) {
  static_assert(!(KBIAS && BIAS), "one bias form at a time");
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
      if (CAUSAL && prm.heavy_first > 0) {
        // groups of heavy_first heads; inside a group the heaviest query blocks of all its heads first
        const int n_bh_x = n_bh >> 3, per_group = prm.heavy_first * prm.n_qblk;
        const int grp = j / per_group;
        int r = j - grp * per_group;
        const int heads = min(prm.heavy_first, n_bh_x - grp * prm.heavy_first);
        if (prm.order_n > 0) r = prm.order_tab[r];      // (a launch whose workgroups are all resident at once: see launch_one)
        bh = x + 8 * (grp * prm.heavy_first + r % heads);
        qblk = prm.n_qblk - 1 - r / heads;
      } else {
        bh = x + 8 * (j / prm.n_qblk);
        qblk = prm.n_qblk - 1 - (j % prm.n_qblk);
      }
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
    if (key0 + kBN <= Sk && prm.d == D) {
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
      // it would hold registers for the whole kernel. Also every tile of a head_dim below D: columns from the true
      // head_dim on read zeros.
      int lane_here = lane;
      asm volatile("" : "+v"(lane_here));
#pragma unroll
      for (int i = 0; i < DMA_PER_WAVE; ++i) {
        const int row = (wave_s * DMA_PER_WAVE + i) * ROWS_PER_DMA + lane_here / CHUNKS;
        const int col = ((lane_here % CHUNKS) ^ swz<D>(row)) * 8;
        const int key = min(key0 + row, Sk - 1);
        const int lds_off = (wave_s * DMA_PER_WAVE + i) * 1024;
        dma16_lane_ptr(live_or_zero(kbase + (int64_t)key * prm.ks[2] + col, col, prm.d), kdst + lds_off);
        dma16_lane_ptr(live_or_zero(vbase + (int64_t)key * prm.vs[2] + col, col, prm.d), vdst + lds_off);
      }
    }
  };

  // ---- bias: the wave's 32 query rows x 64 keys of a tile, copied like K and V straight into LDS (a per-lane global
  // read of "my row" touches 64 cache lines per instruction). Two buffers of 8 KiB per wave behind the K/V tiles. A row
  // of the tile is 256 bytes (fp32) or 128 bytes (operand type) = 16 or 8 pieces of 16 bytes; piece s of LDS row r
  // holds the row's piece s ^ (r mod 16 or 8), so the reads below (32 rows x the same piece) are spread over the banks.
  // Only for complete tiles of suitably aligned tensors; everything else takes the per-element loads further down.
  constexpr int kBiasWaveBytes = 32 * kBN * 4;
  FO_LDS char* bias_lds = smem + 4 * TILE_BYTES + wave_s * kBiasWaveBytes;
  auto issue_bias = [&](int tile, int buf) {
    if (!prm.bias.dma_ok || tile * kBN + kBN > Sk) return;
    int lane_here = lane;                      // (opaque: this arithmetic is redone per tile rather than kept in registers)
    asm volatile("" : "+v"(lane_here));
    const int elt = prm.bias.is_f32 ? 4 : 2;
    const int pieces = prm.bias.is_f32 ? 16 : 8, rows_per_dma = 64 / pieces;
    const char* base = (const char*)prm.bias.ptr + (b * prm.bias.strides[0] + h * prm.bias.strides[1] + (int64_t)tile * kBN) * elt;
    FO_LDS char* dst = bias_lds + buf * kWaves * kBiasWaveBytes;
    const int n_dma = prm.bias.is_f32 ? 8 : 4;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (i < n_dma) {
        const int row = i * rows_per_dma + lane_here / pieces;
        const int piece = (lane_here % pieces) ^ (row & (pieces - 1));
        const int64_t q = min(q0w + row, Sq - 1);
        dma16_lane_ptr(base + q * prm.bias.strides[2] * elt + piece * 16, dst + i * 1024);
      }
    }
  };

  issue_tile(0, 0);
  if constexpr (BIAS) issue_bias(0, 0);
  FO_LDS float* key_bias = (FO_LDS float*)(smem + 4 * TILE_BYTES);      // KBIAS: [2][64], bias / scale of the keys of a tile
  float key_bias_next = 0.0f;                                           // (wave 0) this lane's key of the tile after next
  const float per_scale = KBIAS ? 1.4426950408889634f / prm.scale_log2e : 0.0f;
  const int64_t key_bias_row = KBIAS ? b * prm.bias.strides[0] + h * prm.bias.strides[1] : 0;
  if constexpr (KBIAS) {
    if (wave_s == 0) {
      key_bias[lane] = load_bias<T>(prm.bias, key_bias_row + min(lane, Sk - 1)) * per_scale;
      key_bias_next = load_bias<T>(prm.bias, key_bias_row + min(kBN + lane, Sk - 1));
    }
  }

  // ---- Q^T fragments (B operand): lane holds query row q0w + l32, d = 16*ks + 8*hh .. +7
  vec8 qf[KSTEPS];
  {
    const int qrow = min(q0w + l32, Sq - 1);
    const T* qp = qbase + (int64_t)qrow * prm.qs[2] + 8 * hh;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) qf[ks] = *(const vec8*)live_or_zero(qp + 16 * ks, 16 * ks + 8 * hh, prm.d);
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
  // with a bias the scores are turned into base-2 logits (score * scale * log2e + bias * log2e) right after the mask, and
  // everything downstream sees a scale of 1
  const float c = BIAS ? 1.0f : prm.scale_log2e;

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
    if constexpr (KBIAS) {
      // (the value fetched one tile ago is used before this tile's copies go out: the wait the compiler puts in front
      // of its use then finds nothing in flight)
      if (wave_s == 0) {
        asm volatile("" : "+v"(key_bias_next));
        key_bias[(buf ^ 1) * kBN + lane] = key_bias_next * per_scale;   // tile + 1: read after the next barrier
      }
    }
    if (tile + 1 < n_tiles && (!(DBG & 1) || tile < 1)) issue_tile(tile + 1, buf ^ 1);
    if constexpr (BIAS) { if (tile + 1 < n_tiles) issue_bias(tile + 1, buf ^ 1); }
    if constexpr (KBIAS) {
      if (wave_s == 0) key_bias_next = load_bias<T>(prm.bias, key_bias_row + min((tile + 2) * kBN + lane, Sk - 1));
    }

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
      if constexpr (KBIAS) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int jv = 0; jv < 4; ++jv) {
            const f32x4 b4 = *(FO_LDS const f32x4*)(key_bias + buf * kBN + 32 * kb + 8 * jv + 4 * hh);
#pragma unroll
            for (int u = 0; u < 4; ++u) sacc[kb][4 * jv + u] = b4[u];
          }
      }
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

    if constexpr (BIAS) {
      // qk * softmax_scale + bias (flash_attention_triton.py:198)
      if (prm.bias.dma_ok && key0 + kBN <= Sk) {
        // from the tile copied into LDS: register r = 4 j + u of block kb is key 32 kb + 8 j + 4 hh + u of row l32
        FO_LDS const char* bt = bias_lds + buf * kWaves * kBiasWaveBytes;
        // (the bias type is decided once around the unrolled loops: decided per element, every read gets a branch)
        if (prm.bias.is_f32) {
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const f32x4 bv = *(FO_LDS const f32x4*)(bt + l32 * 256 + (((8 * kb + 2 * j + hh) ^ (l32 & 15)) * 16));
#pragma unroll
              for (int u = 0; u < 4; ++u)
                sacc[kb][4 * j + u] = __builtin_fmaf(sacc[kb][4 * j + u], prm.scale_log2e, bv[u] * 1.4426950408889634f);
            }
        } else {
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              typedef __attribute__((ext_vector_type(4))) T vec4;
              const vec4 h4 = *(FO_LDS const vec4*)(bt + l32 * 128 + (((4 * kb + j) ^ (l32 & 7)) * 16) + hh * 8);
#pragma unroll
              for (int u = 0; u < 4; ++u)
                sacc[kb][4 * j + u] = __builtin_fmaf(sacc[kb][4 * j + u], prm.scale_log2e, (float)h4[u] * 1.4426950408889634f);
            }
        }
      } else {
        // loads from global memory: four consecutive keys per load when the tile is complete and the bias is laid out
        // for it, else key by key; rows and keys past the end re-read the last ones
        const int64_t brow = b * prm.bias.strides[0] + h * prm.bias.strides[1] + (int64_t)min(q0w + l32, Sq - 1) * prm.bias.strides[2];
        float bv[2][16];
        if (prm.bias.vec_ok && key0 + kBN <= Sk) {
          if (prm.bias.is_f32) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
              for (int j = 0; j < 4; ++j) load_bias4<float>((const float*)prm.bias.ptr + brow + key0 + 32 * kb + 4 * hh + 8 * j, bv[kb] + 4 * j);
          } else {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
              for (int j = 0; j < 4; ++j) load_bias4<T>((const T*)prm.bias.ptr + brow + key0 + 32 * kb + 4 * hh + 8 * j, bv[kb] + 4 * j);
          }
        } else if (prm.bias.is_f32) {
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) bv[kb][r] = ((const float*)prm.bias.ptr)[brow + min(key0 + 32 * kb + 4 * hh + (r & 3) + 8 * (r >> 2), Sk - 1)];
        } else {
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) bv[kb][r] = (float)((const T*)prm.bias.ptr)[brow + min(key0 + 32 * kb + 4 * hh + (r & 3) + 8 * (r >> 2), Sk - 1)];
        }
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) sacc[kb][r] = __builtin_fmaf(sacc[kb][r], prm.scale_log2e, bv[kb][r] * 1.4426950408889634f);
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
      const float alpha = ((BIAS || KBIAS) && m_new == -INFINITY) ? 1.0f : __builtin_amdgcn_exp2f((m_run - m_new) * c);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int i = 0; i < DBLK; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] *= alpha;
    }
    // a bias may mask every key seen so far (-inf, e.g. left padding): the reference then stays 0 until a key counts
    const float mc = ((BIAS || KBIAS) && m_run == -INFINITY) ? 0.0f : m_run * c;
    float psum = 0.0f;
    vec8 pf[4];
    // dropout: 32-bit index of this lane's query row at key 0 of the tile (flash_attention_triton.py:125,217)
    const uint32_t drop_row = DROP ? prm.drop.offset + ((uint32_t)bh * (uint32_t)Sq + (uint32_t)(q0w + l32)) * (uint32_t)Sk + (uint32_t)key0 : 0u;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float p = (DBG & 2) ? sacc[kb][r] : __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][r], c, -mc));
        psum += p;                                     // summed in fp32 before rounding and before dropout (flash_attention_triton.py:203)
        if constexpr (DROP) {
          const uint32_t idx = drop_row + (uint32_t)(32 * kb + 4 * hh + (r & 3) + 8 * (r >> 2));
          p = dropout_keep(idx, prm.drop.seed, prm.drop.threshold) ? p * prm.drop.keep_scale : 0.0f;   // :216-219
        }
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
        if (32 * db + 8 * rg + 4 * hh < prm.d) *(vec4*)(op + 32 * db + 8 * rg + 4 * hh) = o4;
      }
    if (prm.lse != nullptr && hh == 0) {
      // ln sum_j exp(scale*s_j) = ln2 * (m*scale*log2e + log2(l))
      prm.lse[(int64_t)bh * Sq + qi] = (m_run * c + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f;
    }
  }
}

// =====================================================================================================================
// Wide kernel: 4 waves x 64 query rows = 256 rows per workgroup, one workgroup per CU, ONE wave per SIMD with the
// whole register file (256 VGPRs for operands, scores and softmax state + the 128 accumulator registers of O^T in
// AGPRs). K and V tiles in four-slot LDS rings (128 KiB at D = 128) filled two tiles ahead.
//
// Measured on MI355X: a SIMD overlaps MFMA and VALU work only when the two alternate INSIDE a wave (about six plain
// VALU operations, or three transcendentals, issue for free behind each 32x32x16 MFMA); MFMA and VALU work of two
// different waves on one SIMD mostly serialise. So one wave per SIMD does everything, 64 rows wide (every K / V^T
// fragment read from LDS feeds two MFMAs, halving LDS traffic per flop), software-pipelined three deep over 32-key
// sub-tiles, with the instruction stream laid out as micro-groups of ONE MFMA plus its share of LDS reads and
// softmax arithmetic, fenced so that the compiler keeps that order:
//     step(s):   S(s+1) = K Q^T          16 MFMAs  \  alternating, 32 micro-groups at D = 128
//                O += V^T P(s-1)^T       16 MFMAs  /
//                row max of S(s), new reference maximum, P(s) = exp2(S(s) c - m c), row sums   (VALU, spread over all)
// The (rare) rescale of O by 2^(old reference - new reference) is applied at the end of the step, after P(s-1) V has
// been accumulated with the old reference and before P(s) V is.
//
// The MFMAs are issued as inline assembly with explicit register classes: accumulators of O^T updated in place in
// AGPRs, scores in VGPRs. (Left to choose, the compiler puts both in AGPRs, updates them out of place and copies.)
// Two hazards the compiler can no longer see are kept by construction. A VALU read of an MFMA result needs 11 wait
// states after an 8-pass MFMA: at least two further MFMAs (8 wait states each) or explicit s_nop separate the last
// write of a score or accumulator register from its first VALU read. An MFMA source register written by a VALU
// instruction (measured: also by v_accvgpr_read, which the compiler uses for values it parks in AGPRs) needs two wait
// states before the MFMA reads it: every MFMA carries them in front.
constexpr int kWideBM = 256;       // query rows per workgroup: 8 waves x 32 rows (QB = 1) or 4 waves x 64 rows (QB = 2)
constexpr int kRing = 4;
constexpr float kLargeRowSum = 4096.0f;   // a lane's 16-key row sum above this means some P exceeded 2^8: time to move the reference

typedef __attribute__((ext_vector_type(4))) int i32x4;

// NOP: two wait states in front of the MFMA (see above). FO_MFMA_NOPS = 1 puts them in front of every MFMA; with 0
// the MFMAs inside the tile loops go without, which is only correct if no VALU write of a source lands within two
// instructions before them: the build checks the generated assembly for that and falls back to 1 if it finds one.
#ifndef FO_MFMA_NOPS
#define FO_MFMA_NOPS 1
#endif
// Three layout choices of the pipelined kernel, each a bit mask over its forms (1: 256 rows as eight waves x 32 rows,
// 2: 256 rows as four waves x 64 rows, 4: 128 rows as four waves x 32 rows), kept as macros so that a build can measure
// them against each other:
// FO_PIN_MFMA  the MFMA of a micro-group is fenced to be its first instruction. A lone wave per SIMD issues in order: left
//              to the compiler, the MFMAs of two neighbouring groups end up back to back with all the other work after
//              them, and the second one stalls the wave for the 28 cycles the matrix pipe is still busy. Four-wave form:
//              -6 % cycles; eight-wave form +3 % (its second wave fills such gaps anyway).
// FO_SPREAD    the copies of a tile are issued one at a time between the MFMAs of its two steps instead of in one batch
//              behind the tile's barrier, where every wave of the workgroup queues up at the memory pipe at once (a
//              batch of 8 costs a lone wave ~390 cycles, spread ~110). Four-wave form -10 % cycles on top of the
//              pinning, eight-wave form -6 %, and the waves reach the barrier closer together (barrier 10 % -> 2.5 %).
// FO_STAGGER   eight-wave form without FO_SPREAD: the two waves of a SIMD issue the copies of both in turn (-4 % cycles).
#ifndef FO_PIN_MFMA
#define FO_PIN_MFMA 2
#endif
#ifndef FO_STAGGER
#define FO_STAGGER 0
#endif
#ifndef FO_SPREAD
#define FO_SPREAD 7
#endif
template <typename T, bool NOP> struct AsmMfma;
#if defined(__HIP_DEVICE_COMPILE__)
#define FO_MFMA_BODY(PRE, MNEMONIC)                                                                                     \
  /* acc (VGPRs) = a b, B operand in AGPRs */                                                                           \
  static __device__ __forceinline__ void v_init_ba(f32x16& acc, i32x4 a, i32x4 b) {                                     \
    asm volatile(PRE MNEMONIC " %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "a"(b));                                          \
  }                                                                                                                     \
  /* acc (VGPRs) += a b, B operand in AGPRs */                                                                          \
  static __device__ __forceinline__ void v_acc_ba(f32x16& acc, i32x4 a, i32x4 b) {                                      \
    asm volatile(PRE MNEMONIC " %0, %1, %2, %0" : "+v"(acc) : "v"(a), "a"(b));                                          \
  }                                                                                                                     \
  /* acc (AGPRs) += a b */                                                                                              \
  static __device__ __forceinline__ void a_acc(f32x16& acc, i32x4 a, i32x4 b) {                                         \
    asm volatile(PRE MNEMONIC " %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));                                          \
  }
#else
#define FO_MFMA_BODY(PRE, MNEMONIC)                                                                                     \
  static __device__ __forceinline__ void v_init_ba(f32x16&, i32x4, i32x4) {}                                            \
  static __device__ __forceinline__ void v_acc_ba(f32x16&, i32x4, i32x4) {}                                             \
  static __device__ __forceinline__ void a_acc(f32x16&, i32x4, i32x4) {}
#endif
template <> struct AsmMfma<__bf16, true> { FO_MFMA_BODY("s_nop 1\n\t", "v_mfma_f32_32x32x16_bf16") };
template <> struct AsmMfma<_Float16, true> { FO_MFMA_BODY("s_nop 1\n\t", "v_mfma_f32_32x32x16_f16") };
template <> struct AsmMfma<__bf16, false> { FO_MFMA_BODY("", "v_mfma_f32_32x32x16_bf16") };
template <> struct AsmMfma<_Float16, false> { FO_MFMA_BODY("", "v_mfma_f32_32x32x16_f16") };
#undef FO_MFMA_BODY

// Wait states for an MFMA result to become readable by VALU instructions the compiler places (see above). The values
// to be read are passed through empty volatile statements after the wait, so that no read can be moved above it.
template <int N>
__device__ __forceinline__ void mfma_result_fence_a(f32x16 (&acc)[N]) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");
#pragma unroll
  for (int i = 0; i < N; ++i) asm volatile("" : "+a"(acc[i]));
#endif
}
template <int N>
__device__ __forceinline__ void mfma_result_fence_v(f32x16 (&acc)[N]) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");
#pragma unroll
  for (int i = 0; i < N; ++i) asm volatile("" : "+v"(acc[i]));
#endif
}
// x *= a for an accumulator that lives in AGPRs, element by element in place through one VGPR (left to the compiler,
// every accumulator moves to VGPRs at once, at the cost of the whole kernel's register budget)
__device__ __forceinline__ void scale_acc(f32x16& acc, float a) {
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    float e = acc[r], tmp;
    asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 1\n\tv_accvgpr_write_b32 %0, %1" : "+a"(e), "=&v"(tmp) : "v"(a));
    acc[r] = e;
  }
#endif
}

// workgroups per head of the wide kernel
__host__ __device__ inline int wide_items(int n_qblk, bool causal) { return causal ? (n_qblk + 1) / 2 : n_qblk; }

// keys of a per-key bias the pipelined kernel keeps in LDS (fp32, beside the rings: 128 + 32 of the 160 KiB at head_dim 128)
constexpr int kVBiasKeys = 8192;
constexpr float kNoKeyYet = -1.0e30f;   // reference of a row all of whose keys so far a bias of -inf has removed

template <typename T, int D, bool CAUSAL, int QB, int DBG, int BM = kWideBM, bool VBIAS = false>
__global__ void __launch_bounds__(BM / (32 * QB) * 64, (BM == kWideBM || D == 128 || VBIAS) ? 1 : 2) attn_fwd_wide_kernel(const AttnParams prm_arg) {
  const AttnParams& prm = prm_arg;
  // VBIAS: an additive bias that is the same for every query of a head (query stride 0: the reference's "vector" bias,
  // flash_attention_triton.py:176-186, e.g. a key padding mask). The head's row of it, at most kVBiasKeys keys, is put
  // into LDS once per workgroup as fp32 divided by softmax_scale, so that (S + b / scale) * scale * log2 e is the biased
  // score in the base-2 domain and the running maximum, the lazily raised reference and LSE keep their meaning with
  // S + b / scale in the place of S. A step reads the 16 values of its 32 keys that a lane's registers hold (they
  // depend on the register and the half of the wave only) and adds them where the scores are scaled: one more VALU
  // instruction per score. A bias of -inf removes a key; a row whose keys so far are all removed has the reference
  // kNoKeyYet, a large negative number, against which removed keys give 0 and the first key that counts overflows the
  // row sum once (recovery path), which multiplies the row's empty O and l by 0 (left padding: one step per row).
  // BM = 256: the form described above. BM = 128 (QB = 1): the same pipeline with four waves x 32 rows, one query block
  // per workgroup in the 128-row kernel's order (heaviest causal blocks first), for shapes that give the chip too few
  // 256-row workgroups: a workgroup's time per key tile is what bounds those, and this pipeline's is less than half the
  // plain 128-row kernel's (which computes S, the softmax and P V of a tile one after the other).
  static_assert(BM == kWideBM || (BM == kBM && QB == 1), "forms of the pipelined kernel");
  constexpr bool PAIRED = CAUSAL && BM == kWideBM;   // a causal workgroup takes two query blocks
  constexpr int kWideWaves = BM / (32 * QB);
  typedef AsmMfma<T, true> Mfma;                  // outside the loops: always with wait states
  typedef __attribute__((ext_vector_type(2))) T vec2;
  constexpr int ROW_BYTES = D * 2;
  constexpr int TILE_BYTES = kBN * ROW_BYTES;
  constexpr int HALF_BYTES = TILE_BYTES / 2;     // one 32-key sub-tile
  constexpr int KSTEPS = D / 16;                 // K fragments of one sub-tile; each feeds QB MFMAs (one per 32-row query block)
  constexpr int DBLK = D / 32;
  constexpr int VFRAGS = 2 * DBLK;               // V^T fragments of one sub-tile (2 steps of 16 keys x D/32 blocks)
  constexpr int BLOCKS = TILE_BYTES / 1024;      // 1 KiB copy blocks per tile
  constexpr int DMA_PER_WAVE = BLOCKS / kWideWaves;
  static_assert(VFRAGS == KSTEPS && DMA_PER_WAVE >= 1 && KSTEPS >= 4, "tile shape");
  // Who issues the copies of a tile: every wave its own blocks (ISSUERS == 1), or the two waves of a SIMD in turn, each
  // the blocks of both (ISSUERS == 2: while one wave is held up at the memory pipe the other has the SIMD to itself).
  constexpr int FORM = BM == kWideBM ? QB : 4;   // bit of this form in the FO_PIN_MFMA / FO_SPREAD masks
  constexpr int ISSUERS = (FO_STAGGER && BM == kWideBM && QB == 1 && !(FO_SPREAD & FORM)) ? 2 : 1;
  constexpr int NBLK = DMA_PER_WAVE * ISSUERS;          // blocks a wave copies per matrix when it is its turn

  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  FO_LDS char* smem = (FO_LDS char*)smem_raw;    // K ring (kRing tiles) | V ring (kRing tiles)
  const int tid = threadIdx.x;
  const int wave_s = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int hh = lane >> 5;

  // A causal workgroup takes two query blocks, one after the other: block n-1-i (the heaviest left) and block i, so
  // that every workgroup has the same amount of work (n+1 tiles' worth) whatever i is. Non-causal: one block each.
  // (BM = 128: one block each, causal or not, heaviest blocks first as in attn_fwd_kernel.)
  // KEEP_ON (256 rows without bias): a workgroup may be given several work items, blockIdx.x, + gridDim.x,
  // ... (the launcher decides: one item per workgroup, or one workgroup per CU that walks its share), and while it is
  // in the last three tiles of a query block it already copies the first tiles of the next one - the second block of a
  // causal pair, or the next item's - into the ring slots the tiles behind the end would have taken, and fetches that
  // block's Q. The next block then starts without waiting for memory.
  constexpr bool KEEP_ON = BM == kWideBM && !VBIAS;
  const int n_bh = prm.B * prm.H;
  // (the tail of a launch of the 256-row kernel, taken over by this 128-row form: the 256-row blocks are what is dealt out)
  const bool tail_mode = BM != kWideBM && !CAUSAL && prm.tail_base > 0;
  const int n_items = PAIRED ? wide_items(prm.n_qblk, true) : tail_mode ? (prm.n_qblk + 1) / 2 : prm.n_qblk;
  const int n_ids = (BM == kWideBM && prm.id_limit > 0) ? min(n_items * n_bh, prm.id_limit) : n_items * n_bh;
  auto decode = [&](int id, int& bh_, int& item_) {
    int half = 0;
    if (tail_mode) {
      // workgroups 2 i and 2 i + 1 (16 j + x and 16 j + 8 + x where heads are dealt to XCDs, so that both stay on the
      // XCD of the item) take the two 128-row halves of 256-row item tail_base + i
      if ((n_bh & 7) == 0) { half = (id >> 3) & 1; id = prm.tail_base + ((id >> 4) << 3) + (id & 7); }
      else { half = id & 1; id = prm.tail_base + (id >> 1); }
    }
    if ((n_bh & 7) == 0) {
      const int x = id & 7, j = id >> 3;          // XCD, position in that XCD's list
      if (BM != kWideBM && CAUSAL && prm.heavy_first > 0) {
        // groups of heavy_first heads; inside a group the heaviest query blocks of all its heads first
        const int n_bh_x = n_bh >> 3, per_group = prm.heavy_first * prm.n_qblk;
        const int grp = j / per_group, r = j - grp * per_group;
        const int heads = min(prm.heavy_first, n_bh_x - grp * prm.heavy_first);
        bh_ = x + 8 * (grp * prm.heavy_first + r % heads);
        item_ = r / heads;
      } else {
        bh_ = x + 8 * (j / n_items);               // one head after the other
        item_ = j % n_items;
      }
    } else {
      bh_ = id % n_bh;
      item_ = id / n_bh;
    }
    if (BM != kWideBM && CAUSAL) item_ = prm.n_qblk - 1 - item_;   // heaviest first
    if (tail_mode) item_ = 2 * item_ + half;
  };
  int wg_id = blockIdx.x;
  int bh, item;
  decode(wg_id, bh, item);
  if (tail_mode && item * BM >= prm.Sq) return;        // (the second half of a last block that has only one)
  int pass = 0;
  bool first_block = true, prefetched = false;
  bool o_rows_whole = false;     // every row of the block before this one was stored (no store instruction may have been skipped)
  // Q^T fragments (B operand of S^T = K Q^T), QB blocks of 32 query rows, of the query block a pass works on. The
  // second pass's are fetched when the first pass has computed its last scores, so that they arrive while it
  // normalises and writes its O.
  i32x4 qf[QB][KSTEPS];
  auto load_q = [&](int of_bh, int for_qblk) {
    const T* qb_base = (const T*)prm.q + (of_bh / prm.H) * prm.qs[0] + (of_bh % prm.H) * prm.qs[1];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const int qrow = min(for_qblk * BM + wave_s * 32 * QB + 32 * qb + l32, prm.Sq - 1);
      const T* qp = qb_base + (int64_t)qrow * prm.qs[2] + 8 * hh;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) qf[qb][ks] = *(const i32x4*)(qp + 16 * ks);
    }
  };
  FO_LDS float* vbias = (FO_LDS float*)(smem + 2 * kRing * TILE_BYTES) + 4 * hh;   // (this lane's half: its registers' keys start 4 further)
  if constexpr (VBIAS) {
    const int64_t brow = (bh / prm.H) * prm.bias.strides[0] + (bh % prm.H) * prm.bias.strides[1];
    const float per_scale = 1.4426950408889634f / prm.scale_log2e;
    const int n_pad = (prm.Sk + kBN - 1) / kBN * kBN;                  // at most kVBiasKeys: the launcher checks
    for (int i = tid; i < n_pad; i += kWideWaves * 64)
      ((FO_LDS float*)(smem + 2 * kRing * TILE_BYTES))[i] = load_bias<T>(prm.bias, brow + min(i, prm.Sk - 1)) * per_scale;
    __syncthreads();
  }
  for (;;) {   // query blocks of this workgroup
#if defined(__HIP_DEVICE_COMPILE__)
  // (KEEP_ON: the kernel's arguments are read afresh for every block, through a copy of their address that the compiler
  // cannot see through. Otherwise everything derived from them is kept across the loop - far more than there are scalar
  // registers - and the moves to and from the lanes of spare vector registers cost a block about a microsecond.)
  // (prm_arg is the kernel's only argument: it sits at the start of the argument segment)
  typedef const __attribute__((address_space(4))) AttnParams* ArgPtr;
  ArgPtr args_here = (ArgPtr)__builtin_amdgcn_kernarg_segment_ptr();
  if constexpr (KEEP_ON) asm volatile("" : "+s"(args_here));
  decltype(auto) prm = [&]() -> decltype(auto) { if constexpr (KEEP_ON) return (*args_here); else return (prm_arg); }();
#else
  const AttnParams& prm = prm_arg;
#endif
  const int b = bh / prm.H, h = bh % prm.H;
  const int n_pass = (PAIRED && prm.n_qblk - 1 - item != item) ? 2 : 1;
  const int qblk = PAIRED ? (pass == 0 ? prm.n_qblk - 1 - item : item) : item;
  // the block after this one
  bool has_next = false;
  int next_bh = bh, next_item = item, next_qblk = item;       // (second pass of a pair: block `item` of the same head)
  if (pass + 1 < n_pass) has_next = true;
  else if (KEEP_ON && wg_id + (int)gridDim.x < n_ids) {
    decode(wg_id + (int)gridDim.x, next_bh, next_item);
    next_qblk = PAIRED ? prm.n_qblk - 1 - next_item : next_item;
    has_next = true;
  }
  if (!first_block && !prefetched) {
    // the other waves may still be reading the rings, and this wave's stores of O still count as memory operations in flight
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  }
  const int q0 = qblk * BM;
  const int q0w = q0 + wave_s * 32 * QB;
  const int Sq = prm.Sq, Sk = prm.Sk;
  const T* __restrict__ kbase = (const T*)prm.k + b * prm.ks[0] + h * prm.ks[1];
  const T* __restrict__ vbase = (const T*)prm.v + b * prm.vs[0] + h * prm.vs[1];

  int n_tiles, n_w;                       // tiles the workgroup walks / tiles in which this wave has unmasked keys
  if constexpr (CAUSAL) {
    n_tiles = (min(Sk, q0 + BM) + kBN - 1) / kBN;
    n_w = min(n_tiles, (q0w + 32 * QB - 1) / kBN + 1);
  } else {
    n_tiles = (Sk + kBN - 1) / kBN;
    n_w = n_tiles;
  }

  // ---- LDS layout of a tile: 1 KiB blocks, each written by ONE direct-to-LDS instruction (64 lanes x 16 bytes, lane
  // order) and laid out so that every fragment read of the inner loop is "lane base + compile-time offset" over
  // consecutive addresses - no swizzle arithmetic, no bank conflicts, one address register per matrix.
  //   K tile: block (hf, kp, r16) = rows 32 hf + 16 r16 .. +15 of the tile, 64 bytes (k-steps 2kp, 2kp+1) of each row,
  //     at ((hf * D/32 + kp) * 2 + r16) KiB; inside, the 16-byte piece (k-step 2kp + kk, half hh, row rr) sits at
  //     kk*512 + hh*256 + rr*16. The A-operand read of k-step ks (lane = row l32, half hh) is then
  //     (l32/16)*1024 + hh*256 + (l32%16)*16  +  hf*HALF_BYTES + (ks/2)*2048 + (ks%2)*512.
  //   V tile: block (hf, t, db) = rows 32 hf + 16 t .. +15, 64 bytes (d = 32 db .. +31) of each row, at
  //     (hf * D/16 + t * D/32 + db) KiB; inside, the two transposing reads (rows +0..7 / +8..15) each get 512
  //     consecutive bytes in the lane order of that read: lane*8  +  hf*HALF_BYTES + (t*D/32 + db)*1024 + half*512.
  // Which 16 bytes of global memory a copy lane fetches follows from that; per row the four lanes that fetch from it
  // cover 64 consecutive bytes.
  const int k_lane_row = lane & 15, k_lane_col = (lane >> 4) * 8;
  const int v_m = lane & 31;
  const int v_lane_row = 8 * (lane >> 5) + 4 * (v_m >> 4) + ((v_m & 7) >> 1), v_lane_col = 16 * ((v_m >> 3) & 1) + 8 * (v_m & 1);
  const uint32_t k_off = (uint32_t)(k_lane_row * (int)prm.ks[2] + k_lane_col) * 2u;
  const uint32_t v_off = (uint32_t)(v_lane_row * (int)prm.vs[2] + v_lane_col) * 2u;
  // block i of this wave's duty: its own DMA_PER_WAVE blocks, then (ISSUERS == 2) those of the other wave of its SIMD
  auto blk_of = [&](int i) -> int {
    if constexpr (ISSUERS == 1) return wave_s * DMA_PER_WAVE + i;
    else return ((wave_s & 3) + 4 * (i / DMA_PER_WAVE)) * DMA_PER_WAVE + i % DMA_PER_WAVE;
  };
  // batch t is this wave's to issue
  auto my_turn = [&](int t) -> bool { return ISSUERS == 1 || ((t + 4) & 1) == (wave_s >> 2); };
  // one tile of K (ring 0) or V (ring 1) into slot tile % kRing
  auto issue = [&](auto is_v, int tile, const T* base) {
    constexpr bool V = decltype(is_v)::value;
    const int64_t stride = V ? prm.vs[2] : prm.ks[2];
    const int key0 = tile * kBN;
    FO_LDS char* dst = smem + (kRing * (V ? 1 : 0) + (tile & (kRing - 1))) * TILE_BYTES;
#pragma unroll
    for (int i = 0; i < NBLK; ++i) {
      const int blk = blk_of(i);
      const int hf = blk / (BLOCKS / 2), in_half = blk % (BLOCKS / 2);
      // first row (in the tile) and first column of the block
      const int row0 = V ? 32 * hf + 16 * (in_half / DBLK) : 32 * hf + 16 * (in_half & 1);
      const int col0 = V ? 32 * (in_half % DBLK) : 32 * (in_half >> 1);
      if (key0 + kBN <= Sk) {
        const char* src = (const char*)(base + (int64_t)(key0 + row0) * stride + col0);
        dma16_uniform_base(src, V ? v_off : k_off, dst + blk * 1024);
      } else {
        int lane_here = lane;                            // (opaque: keeps this rare path's address math inside it)
        asm volatile("" : "+v"(lane_here));
        const int m = lane_here & 31;
        const int lrow = V ? 8 * (lane_here >> 5) + 4 * (m >> 4) + ((m & 7) >> 1) : (lane_here & 15);
        const int lcol = V ? 16 * ((m >> 3) & 1) + 8 * (m & 1) : (lane_here >> 4) * 8;
        const int key = min(key0 + row0 + lrow, Sk - 1);   // rows past the end re-read the last key (masked later)
        dma16_lane_ptr(base + (int64_t)key * stride + col0 + lcol, dst + blk * 1024);
      }
    }
  };
  // The common case, both tiles complete: this wave's blocks have fixed places inside a tile (pointers for tile 0
  // are loop-invariant scalars), and the tile's distance from tile 0 is added to the per-lane offset.
  const char* k_src0[NBLK];
  const char* v_src0[NBLK];
#pragma unroll
  for (int i = 0; i < NBLK; ++i) {
    const int blk = blk_of(i);
    const int hf = blk / (BLOCKS / 2), in_half = blk % (BLOCKS / 2);
    k_src0[i] = (const char*)(kbase + (int64_t)(32 * hf + 16 * (in_half & 1)) * prm.ks[2] + 32 * (in_half >> 1));
    v_src0[i] = (const char*)(vbase + (int64_t)(32 * hf + 16 * (in_half / DBLK)) * prm.vs[2] + 32 * (in_half % DBLK));
  }
  const uint32_t k_tile_bytes = (uint32_t)(kBN * (int)prm.ks[2]) * 2u, v_tile_bytes = (uint32_t)(kBN * (int)prm.vs[2]) * 2u;
  const int n_full = min(n_tiles, Sk / kBN);          // tiles below this one are complete
  // batch(t), issued at the top of tile t: K(t+3) and V(t+2). Returns the number of copies this lane issued.
  auto issue_batch = [&](int t) -> int {
    if (!my_turn(t)) return 0;
    if (t + 3 < n_full && t + 2 >= 0) {
      const uint32_t ko = k_off + (uint32_t)(t + 3) * k_tile_bytes, vo = v_off + (uint32_t)(t + 2) * v_tile_bytes;
      FO_LDS char* kdst = smem + ((t + 3) & (kRing - 1)) * TILE_BYTES;
      FO_LDS char* vdst = smem + (kRing + ((t + 2) & (kRing - 1))) * TILE_BYTES;
#pragma unroll
      for (int i = 0; i < NBLK; ++i) {
        dma16_uniform_base(k_src0[i], ko, kdst + blk_of(i) * 1024);
        dma16_uniform_base(v_src0[i], vo, vdst + blk_of(i) * 1024);
      }
      return 2 * NBLK;
    }
    int n = 0;
    if (t + 3 < n_tiles && t + 3 >= 0) { issue(std::false_type{}, t + 3, kbase); n += NBLK; }
    if (t + 2 < n_tiles && t + 2 >= 0) { issue(std::true_type{}, t + 2, vbase); n += NBLK; }
    return n;
  };
  // The first three batches of the NEXT block (t = -3, -2, -1: K(0) | K(1), V(0) | K(2), V(1)), issued at the tops of
  // this block's last three tiles. Its tile i goes to ring slot i % kRing, which is the slot this block's tile
  // n_tiles + i would have taken when n_tiles is a multiple of kRing - only then is there a prefetch.
  int next_tiles = 0;
  const T* next_kbase = kbase;
  const T* next_vbase = vbase;
  if (has_next) {
    next_tiles = CAUSAL ? (min(Sk, next_qblk * BM + BM) + kBN - 1) / kBN : n_tiles;
    next_kbase = (const T*)prm.k + (next_bh / prm.H) * prm.ks[0] + (next_bh % prm.H) * prm.ks[1];
    next_vbase = (const T*)prm.v + (next_bh / prm.H) * prm.vs[0] + (next_bh % prm.H) * prm.vs[1];
  }
  const bool prefetch_next = KEEP_ON && has_next && n_tiles >= kRing && (n_tiles & (kRing - 1)) == 0 && prm.keep_on != 0;
  auto issue_batch_next = [&](int t) -> int {
    int n = 0;
    if (t + 3 < next_tiles) { issue(std::false_type{}, t + 3, next_kbase); n += NBLK; }
    if (t + 2 < next_tiles && t + 2 >= 0) { issue(std::true_type{}, t + 2, next_vbase); n += NBLK; }
    return n;
  };
  int last_batch = 0;
  if (!prefetched) {
    issue_batch(-3);
    issue_batch(-2);
    last_batch = issue_batch(-1);
  }

  if (first_block) load_q(bh, qblk);
#pragma unroll
  for (int qb = 0; qb < QB; ++qb)
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) asm volatile("" : "+a"(qf[qb][ks]));   // wait for Q here, never inside the loop; held in AGPRs

  f32x16 oacc[DBLK][QB];       // O^T accumulators (AGPRs): d-block x query block
#pragma unroll
  for (int i = 0; i < DBLK; ++i)
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[i][qb][r] = 0.0f;
  f32x16 S[2][QB];             // scores: sub-tile s, query block qb live in S[s & 1][qb]
  i32x4 PF[2][QB][2];          // P of sub-tile s: PF[s & 1][qb][16-key step]
  // issue the copies of a tile between the MFMAs of its steps instead of at its top (in the loop of unmasked tiles whose
  // copies are all whole tiles; everywhere else they go out at the top)
  constexpr bool SPREAD_DMA = (DBG & 8) != 0 || (FO_SPREAD & FORM) != 0;
  constexpr int RD = QB == 2 ? 4 : 2;       // must divide the number of fragments of a sub-tile
  static_assert(KSTEPS % RD == 0, "fragment ring");
  i32x4 KF[RD], VF[RD];        // LDS fragment rings, refilled RD fragments ahead of use
  float m_run[QB], l_run[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) { m_run[qb] = -INFINITY; l_run[qb] = 0.0f; }
  const float c = prm.scale_log2e;

  const uint32_t k_lane = (uint32_t)((l32 >> 4) * 1024 + hh * 256 + (l32 & 15) * 16);
  const uint32_t v_lane = (uint32_t)(kRing * TILE_BYTES + lane * 8);
  // byte offset of sub-tile `sub` (tile sub/2, half sub%2) inside its ring
  auto sub_base = [&](int sub) -> uint32_t { return (uint32_t)(((sub >> 1) & (kRing - 1)) * TILE_BYTES + (sub & 1) * HALF_BYTES); };
  // K fragment ks / V^T fragment idx (16-key step idx / DBLK, d-block idx % DBLK) of the sub-tile whose base
  // (lane part included) is `base`. A sub-tile index past the end reads a valid but meaningless ring slot; such
  // fragments are never used.
  auto k_frag = [&](uint32_t base, int ks) -> i32x4 {
    return *(FO_LDS const i32x4*)(smem + base + (ks >> 1) * 2048 + (ks & 1) * 512);
  };
  auto v_frag = [&](uint32_t base, int idx) -> i32x4 {
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FO_LDS s16x4*)(smem + base + idx * 1024));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FO_LDS s16x4*)(smem + base + idx * 1024 + 512));
    return __builtin_bit_cast(i32x4, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  // ---- one pipeline step for sub-tile s (parity P = s & 1), as micro-groups of one MFMA each:
  //   HAS_QK: S[P^1] = K(s+1) Q^T;   HAS_PV: O += V(s-1)^T PF[P^1]^T;   always: S[P] -> PF[P] = exp2(S c - m c), row sums.
  // On entry KF holds K fragments 0..RD-1 of sub-tile s+1 and VF holds V^T fragments 0..RD-1 of sub-tile s-1; on exit
  // the same for the next step.
  //
  // The reference m of the exponentials is not the running row maximum but a stale one: the micro-groups compute no
  // maximum at all. P may therefore exceed 1; as long as it stays below 2^12 the fp32 accumulators and the
  // half-precision P lose no relative precision, and O / l and LSE = m + log(l) do not depend on the reference. At
  // the end of the step the row sums tell whether some P got large (or overflowed: the first step starts from
  // m = -inf); only then (rarely) the step's P is recomputed from the still intact scores against the true maximum,
  // and O and l are rescaled. The result is that of the exact recurrence (flash_attention_triton.py:200-213,241-243)
  // up to rounding.
  auto step = [&](int s_in, auto parity, auto has_qk, auto has_pv, auto masked, auto in_loop, auto spread, int dma_tile, auto... no_recovery) {
    // (an extra argument: the caller knows that no P of this step can be large, and the recovery path is left out)
    constexpr bool CAN_RECOVER = sizeof...(no_recovery) == 0;
    // inside the loops the MFMAs go without wait states in front unless the build asked for them (see above)
    typedef AsmMfma<T, !(decltype(in_loop)::value && !FO_MFMA_NOPS)> Mfma;
    constexpr int P = decltype(parity)::value;
    constexpr bool HAS_QK = decltype(has_qk)::value, HAS_PV = decltype(has_pv)::value, MASK = decltype(masked)::value;
    constexpr int NM = QB * KSTEPS;                                     // MFMAs of one kind
    constexpr int NMF = (HAS_QK ? NM : 0) + (HAS_PV ? NM : 0);          // micro-groups with an MFMA
    constexpr int NEL = 16 * QB;                                        // scores per lane
    // Group 0 only issues its MFMA: the scores of this sub-tile were written by MFMAs up to the last-but-one group of
    // the previous step. Then the mask (if any), then the exponentials.
    constexpr int GMASK = 1;
    constexpr int GE0 = MASK ? 2 : 1;                                   // first group that may read the scores
    constexpr int DA = 1;                                               // groups between an exponential and its use
    // (a step with few MFMAs - head_dim 64, first or last step - gets groups without one, so that the three stages of
    // the softmax arithmetic still have their places)
    constexpr int G = NMF > GE0 + 3 + DA ? NMF : GE0 + 3 + DA;          // micro-groups
    constexpr int NE = G - 1 - DA - GE0;                                // groups GE0+1 .. G-1-DA carry the exponentials
    static_assert(NE >= 2, "too few micro-groups");
    // (an opaque copy of the sub-tile index: the variants of this step are selected by branches, and identical address
    // arithmetic in two branches would otherwise be hoisted above them, out of its micro-group)
    int s = s_in;
    asm volatile("" : "+s"(s));
    const uint32_t kb1 = k_lane + sub_base(s + 1), kb2 = k_lane + sub_base(s + 2);
    const uint32_t vb0 = v_lane + sub_base(s - 1), vb1 = v_lane + sub_base(s);
    float mc[QB], psum[QB];
#pragma unroll
    for (int b2 = 0; b2 < QB; ++b2) { mc[b2] = m_run[b2] * c; psum[b2] = 0.0f; }
    // copies this step issues between its MFMAs (spread): the K blocks of tile dma_tile in the step of an even sub-tile,
    // the V blocks in that of an odd one
    constexpr bool SPREAD_HERE = decltype(spread)::value && HAS_QK && HAS_PV;
    uint32_t dma_off = 0;
    FO_LDS char* dma_dst = smem;
    if constexpr (SPREAD_HERE) {
      dma_off = (P == 0) ? k_off + (uint32_t)dma_tile * k_tile_bytes : v_off + (uint32_t)dma_tile * v_tile_bytes;
      dma_dst = smem + ((P == 0 ? 0 : kRing) + (dma_tile & (kRing - 1))) * TILE_BYTES + wave_s * DMA_PER_WAVE * 1024;
    }
    float ex[NEL];
    f32x4 bq[VBIAS ? 4 : 1];                 // bias / scale of the keys of registers 4 j .. 4 j + 3 (keys 32 s + 8 j + 4 hh ..)
    // score e of NEL: query block, accumulator register (the first 8 registers of every block first: they are the
    // first 16-key step of P V)
    auto el_qb = [](int e) { return QB == 2 ? (e >> 3) & 1 : 0; };
    auto el_reg = [](int e) { return QB == 2 ? 8 * (e >> 4) + (e & 7) : e; };
#pragma unroll
    for (int g = 0; g < G; ++g) {
      // -- the MFMA of this micro-group, and the LDS read that refills a fragment once every query block has used it
      const bool is_qk = HAS_QK && (!HAS_PV || (g & 1) == 0);
      const int i = (HAS_QK && HAS_PV) ? (g >> 1) : g;                 // index among the MFMAs of its kind
      const int f = i / QB, qb = i % QB;                               // fragment, query block
      if (g >= NMF) {
      } else if (is_qk) {
        if (f == 0) Mfma::v_init_ba(S[P ^ 1][qb], KF[f % RD], qf[qb][f]);
        else Mfma::v_acc_ba(S[P ^ 1][qb], KF[f % RD], qf[qb][f]);
        if (FO_PIN_MFMA & FORM) __builtin_amdgcn_sched_barrier(0);
        if (qb == QB - 1 && !(DBG & 4)) KF[f % RD] = (f + RD < KSTEPS) ? k_frag(kb1, f + RD) : k_frag(kb2, f + RD - KSTEPS);
      } else {
        Mfma::a_acc(oacc[f % DBLK][qb], VF[f % RD], PF[P ^ 1][qb][f / DBLK]);
        if (FO_PIN_MFMA & FORM) __builtin_amdgcn_sched_barrier(0);
        if (qb == QB - 1 && !(DBG & 4)) VF[f % RD] = (f + RD < VFRAGS) ? v_frag(vb0, f + RD) : v_frag(vb1, f + RD - VFRAGS);
      }
      if constexpr (!HAS_PV) {
        if (g < RD) VF[g] = v_frag(vb1, g);   // first step: the next one expects the first V^T fragments of sub-tile s
      }
      // -- this group's share of the tile copies (steps of even sub-tiles carry K, of odd ones V)
      if constexpr (SPREAD_HERE) {
        constexpr int SPACING = (G - 2) / DMA_PER_WAVE;
        if (g >= 2 && (g - 2) % SPACING == 0 && (g - 2) / SPACING < DMA_PER_WAVE) {
          const int i = (g - 2) / SPACING;
          dma16_uniform_base(P == 0 ? k_src0[i] : v_src0[i], dma_off, dma_dst + i * 1024);
        }
      }
      if constexpr (VBIAS) {
        // (the first eight registers of every block are used in the first half of the step, the others in the second)
        if (g == 0) { bq[0] = *(FO_LDS const f32x4*)(vbias + s * 32); bq[1] = *(FO_LDS const f32x4*)(vbias + s * 32 + 8); }
        if (g == (GE0 + 1 + NE / 2) - 3) { bq[2] = *(FO_LDS const f32x4*)(vbias + s * 32 + 16); bq[3] = *(FO_LDS const f32x4*)(vbias + s * 32 + 24); }
      }
      // -- this group's share of the softmax arithmetic
      if (MASK && g == GMASK) {
        // register r holds key key_base + koff(r), koff(r) = (r & 3) + 8 * (r >> 2); dead iff key > q or key >= Sk,
        // i.e. iff lim + koff(r) > 0 with lim = max(key_base - q, key_base - Sk + 1)
        const int key_base = s * 32 + 4 * hh;
#pragma unroll
        for (int b2 = 0; b2 < QB; ++b2) {
          int lim = key_base - Sk + 1;
          if (CAUSAL) lim = max(lim, key_base - (q0w + 32 * b2 + l32));
#pragma unroll
          for (int r = 0; r < 16; ++r) S[P][b2][r] = (lim > -((r & 3) + 8 * (r >> 2))) ? -INFINITY : S[P][b2][r];
        }
      }
      // Three stages, one micro-group apart, so that no instruction of a group waits for another one of the same
      // group: scale-and-shift of score e in group GE(e) - 1, its exponential in GE(e), the row sum and (for a finished
      // pair) the rounding to the operand type for P.V (flash_attention_triton.py:237) in GE(e) + 1.
#pragma unroll
      for (int e = 0; e < NEL; ++e) {
        const int ge = GE0 + 1 + (e * NE) / NEL;
        const int b2 = el_qb(e), r = el_reg(e);
        if (ge - 1 == g) {
          if constexpr (VBIAS) ex[e] = __builtin_fmaf(S[P][b2][r] + bq[r >> 2][r & 3], c, -mc[b2]);
          else ex[e] = (DBG & 2) ? S[P][b2][r] : __builtin_fmaf(S[P][b2][r], c, -mc[b2]);
          asm volatile("" : "+v"(ex[e]));                              // pins the instruction to this micro-group
        }
        if (ge == g) {
          if (!(DBG & 2)) ex[e] = __builtin_amdgcn_exp2f(ex[e]);
          asm volatile("" : "+v"(ex[e]));
        }
        if (ge + DA == g) {
          psum[b2] += ex[e];                                           // summed in fp32 before rounding (flash_attention_triton.py:203)
          asm volatile("" : "+v"(psum[b2]));
          if (e & 1) {
            const vec2 pk = {(T)ex[e - 1], (T)ex[e]};
            int pki = __builtin_bit_cast(int, pk);
            asm volatile("" : "+v"(pki));
            PF[P][b2][r >> 3][(r & 7) >> 1] = pki;
          }
        }
      }
      if (!(DBG & 128) || (g & 1)) __builtin_amdgcn_sched_barrier(0);
    }
    // -- end of step: did some P get large (or infinite, or NaN from a masked score against m = -inf)?
    bool redo = false;
#pragma unroll
    for (int b2 = 0; b2 < QB; ++b2) redo = redo || !(psum[b2] <= kLargeRowSum);
    if (CAN_RECOVER && __builtin_amdgcn_ballot_w64(redo) != 0 && !(DBG & 2)) {
      // rare: true row maxima of this sub-tile, new references, P and row sums again, O and l rescaled
#pragma unroll
      for (int d = 0; d < DBLK; ++d) mfma_result_fence_a(oacc[d]);
      if constexpr (VBIAS) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          f32x4 t4 = *(FO_LDS const f32x4*)(vbias + s * 32 + 8 * j);
          asm volatile("" : "+v"(t4));                                 // (four values at a time: no registers to spare here)
#pragma unroll
          for (int b2 = 0; b2 < QB; ++b2)
#pragma unroll
            for (int u = 0; u < 4; ++u) S[P][b2][4 * j + u] += t4[u];
        }
      }
#pragma unroll
      for (int b2 = 0; b2 < QB; ++b2) {
        float mloc = S[P][b2][0];
#pragma unroll
        for (int r = 1; r < 16; ++r) mloc = fmaxf(mloc, S[P][b2][r]);
        mloc = fmaxf(mloc, half_swap(mloc));
        const float m_new = fmaxf(m_run[b2], mloc);                    // finite: key 0 is never masked (a bias: see kNoKeyYet)
        const float alpha = __builtin_amdgcn_exp2f((m_run[b2] - m_new) * c);
        const float mcn = m_new * c;
        float ps = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(S[P][b2][r], c, -mcn));
          const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(S[P][b2][r + 1], c, -mcn));
          ps += p0;
          ps += p1;
          const vec2 pk = {(T)p0, (T)p1};
          PF[P][b2][r >> 3][(r & 7) >> 1] = __builtin_bit_cast(int, pk);
        }
        psum[b2] = ps;
        m_run[b2] = m_new;
        l_run[b2] *= alpha;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int d = 0; d < DBLK; ++d) scale_acc(oacc[d][b2], alpha);
      }
    }
#pragma unroll
    for (int b2 = 0; b2 < QB; ++b2) l_run[b2] += psum[b2];
  };
  using std::integral_constant;
  typedef integral_constant<int, 0> P0;
  typedef integral_constant<int, 1> P1;
  typedef std::true_type Y;
  typedef std::false_type N;

  // ---- tile loop. Tile j runs the steps of sub-tiles 2j and 2j+1; they read K(j), K(j+1), V(j-1), V(j).
  // At its top, copy batches up to (j-2) must have landed - K(j+1) and V(j) are among them - while batch (j-1) may still
  // be in flight; after the barrier every wave is done with tile j-1, so batch j may overwrite K(j-1) and V(j-2).
  auto tile_top = [&](int j, bool spread_this = false) -> bool {
    if (!(DBG & 32)) {
      // (as many copies may stay in flight as this wave issued in the batch before: 0, one matrix's or both)
      if (__builtin_expect(last_batch == 2 * NBLK, 1)) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NBLK) : "memory");
      else if (last_batch >= NBLK) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NBLK) : "memory");
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    // A bare barrier: __syncthreads() would first wait for every LDS read in flight, i.e. drain the fragment rings once
    // per tile. Nothing needs that wait: the reads in flight here target K(j) and V(j-1), not the slots batch j
    // overwrites, and copies are made visible by the vmcnt wait above (it covers this wave's own pieces; the barrier
    // extends that to everyone's).
    if (!(DBG & 64)) __builtin_amdgcn_s_barrier();
    if (spread_this) { last_batch = 2 * DMA_PER_WAVE; return true; }   // the steps of this tile issue them
    last_batch = (DBG & 1) ? 0 : issue_batch(j);
    if constexpr (KEEP_ON) {
      if (prefetch_next && j >= n_tiles - 3) last_batch += issue_batch_next(j - n_tiles);
    }
    return false;
  };
  // Tiles that need the mask (causal diagonal, keys past the end) are a suffix of the wave's tiles. The hot loops are
  // kept free of alternatives: unmasked tiles, then masked tiles, then the last tile, whose second step has no scores
  // left to compute; the first and last tiles always take the masking variant.
  int j_mask = n_w;                                   // first tile that needs the mask
  if (CAUSAL) j_mask = min(j_mask, (q0w + 1) / kBN);   // smallest j with 64 j + 63 > q0w
  if (Sk % kBN != 0) j_mask = min(j_mask, n_tiles - 1);

  // first tile: fill the pipeline - S(0) on its own, then a step that has nothing to multiply yet
  // (The code of the first tile is not the loops' code: whenever the compiler parks registers in scratch memory there,
  // every reload is waited for with a vmcnt wait that also covers the copies in flight. So all three batches issued
  // above land before it starts - K(0), K(1) and V(0) have to anyway - and batch 0, K(3) and V(2) into slots nobody
  // has used yet, goes out after it, in front of the loops.)
  // (A block whose tiles were copied ahead: its copies and its Q loads were issued before the stores of the previous
  // block's O, and memory operations complete in order - the last stores of O, one 32-row block's worth, may stay in
  // flight. They are counted, so only where none of them can have been skipped.)
  if (KEEP_ON && prefetched && o_rows_whole) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(32 * (ROW_BYTES / 16) / 64) : "memory");
  else if (!(DBG & 32)) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (!(DBG & 64)) __builtin_amdgcn_s_barrier();
  {
    const uint32_t kb0 = k_lane + sub_base(0), kb1 = k_lane + sub_base(1);
#pragma unroll
    for (int i = 0; i < RD; ++i) KF[i] = k_frag(kb0, i);
#pragma unroll
    for (int f = 0; f < KSTEPS; ++f) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        if (f == 0) Mfma::v_init_ba(S[0][qb], KF[f % RD], qf[qb][f]);
        else Mfma::v_acc_ba(S[0][qb], KF[f % RD], qf[qb][f]);
      }
      KF[f % RD] = (f + RD < KSTEPS) ? k_frag(kb0, f + RD) : k_frag(kb1, f + RD - KSTEPS);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  mfma_result_fence_v(S[0]);
  // The reference of the exponentials starts as the row maximum of the first sub-tile (dead keys left out as the step
  // will mask them: lim as there, sub-tile 0; key 0 is never dead, so the maximum is finite). Started from -inf, the
  // first step takes the recovery path - maxima, every exponential a second time, 64 accumulator registers rescaled -
  // once per query block, 1-2 us each time.
#pragma unroll
  for (int b2 = 0; b2 < QB; ++b2) {
    int lim = 4 * hh - Sk + 1;
    if (CAUSAL) lim = max(lim, 4 * hh - (q0w + 32 * b2 + l32));
    float mloc = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float sv = S[0][b2][r];
      if constexpr (VBIAS) sv += vbias[8 * (r >> 2) + (r & 3)];
      mloc = fmaxf(mloc, (lim > -((r & 3) + 8 * (r >> 2))) ? -INFINITY : sv);
    }
    m_run[b2] = fmaxf(mloc, half_swap(mloc));
    // (a bias may have removed every key of the sub-tile: the reference then starts from a large negative number
    // instead of -inf, so that a removed key gives exp2(-inf) = 0 and not exp2(-inf + inf); the first key that counts
    // overflows the row sum and the recovery path moves the reference to it, with O and l multiplied by exp2(-huge) = 0)
    if constexpr (VBIAS) m_run[b2] = fmaxf(m_run[b2], kNoKeyYet);
  }
  step(0, P0{}, Y{}, N{}, Y{}, N{}, N{}, -1, N{});   // (its reference is its own row maximum: every P <= 1, no recovery)
  if (n_w > 1) step(1, P1{}, Y{}, Y{}, Y{}, N{}, N{}, -1); else step(1, P1{}, N{}, Y{}, Y{}, N{}, N{}, -1);
  // Should the steps above have parked registers in scratch memory (they do not at present), wait here, visibly to
  // the compiler, for any reload still in flight: otherwise it guards the first use inside the loops with a vmcnt(0)
  // wait that executes on every iteration and also drains the copies in flight, which it does not see.
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0), nothing else
  last_batch = (DBG & 1) ? 0 : issue_batch(0);
  int j = 1;
  if constexpr (SPREAD_DMA) {
    // unmasked tiles whose copies (K three tiles, V two tiles ahead) are whole tiles: the steps issue them
    for (; j < min(min(j_mask, n_w - 1), n_full - 3); ++j) {
      tile_top(j, true);
      step(2 * j, P0{}, Y{}, Y{}, N{}, Y{}, Y{}, j + 3);
      step(2 * j + 1, P1{}, Y{}, Y{}, N{}, Y{}, Y{}, j + 2);
    }
  }
  for (; j < min(j_mask, n_w - 1); ++j) {
    tile_top(j);
    step(2 * j, P0{}, Y{}, Y{}, N{}, Y{}, N{}, -1);
    step(2 * j + 1, P1{}, Y{}, Y{}, N{}, Y{}, N{}, -1);
  }
  for (; j < n_w - 1; ++j) {
    tile_top(j);
    step(2 * j, P0{}, Y{}, Y{}, Y{}, Y{}, N{}, -1);
    step(2 * j + 1, P1{}, Y{}, Y{}, Y{}, Y{}, N{}, -1);
  }
  if (j < n_w) {
    tile_top(j);
    step(2 * j, P0{}, Y{}, Y{}, Y{}, N{}, N{}, -1);
    step(2 * j + 1, P1{}, N{}, Y{}, Y{}, N{}, N{}, -1);
    ++j;
  }
  {
    // drain: O += V(last)^T P(last)^T for this wave's last sub-tile (2*n_w - 1, odd parity); VF holds its first fragments
    const uint32_t vbl = v_lane + sub_base(2 * n_w - 1);
#pragma unroll
    for (int f = 0; f < VFRAGS; ++f) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) Mfma::a_acc(oacc[f % DBLK][qb], VF[f % RD], PF[1][qb][f / DBLK]);
      if (f + RD < VFRAGS) VF[f % RD] = v_frag(vbl, f + RD);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  // tiles in which this wave has nothing to do (causal): keep feeding the workgroup's rings
  for (; j < n_tiles; ++j) tile_top(j);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (has_next) load_q(next_bh, next_qblk);   // (they arrive while this block's O is written)

  // ---- epilogue: normalise, write O and LSE
#pragma unroll
  for (int d = 0; d < DBLK; ++d) mfma_result_fence_a(oacc[d]);
  // A lane holds 4 consecutive d of one query row per accumulator register group: written straight to memory that is
  // 8 bytes per lane, 16 per row and instruction. Instead the wave's rows are staged in LDS (the rings are free once
  // every wave is past its last tile; rows padded by 16 bytes against bank conflicts) and leave as whole 16-byte
  // pieces, 64 lanes covering four consecutive 256-byte rows per instruction.
  // (KEEP_ON: the first ring slots may already hold the next block's tiles. The rows are staged one 32-row block at a
  // time behind them, from the third slot of the V ring on - free once every wave is past its last tile - into the
  // 32 KiB after the rings.)
  __syncthreads();
  constexpr int CH = ROW_BYTES / 16;                    // 16-byte pieces per row
  constexpr int OROW = ROW_BYTES + 16;
  constexpr int STAGE_ROWS = KEEP_ON ? 32 : 32 * QB;    // rows a wave stages at a time
  // (eight waves at head_dim 128: seven of them fit there, the first one stages in the last slot of the K ring)
  constexpr bool STAGE_SPLIT = KEEP_ON && (kRing + 2) * TILE_BYTES + kWideWaves * STAGE_ROWS * OROW > 160 * 1024;
  FO_LDS char* stage = !KEEP_ON ? smem + wave_s * STAGE_ROWS * OROW
                     : (STAGE_SPLIT && wave_s == 0) ? smem + (kRing - 1) * TILE_BYTES
                     : smem + (kRing + 2) * TILE_BYTES + (wave_s - (STAGE_SPLIT ? 1 : 0)) * STAGE_ROWS * OROW;
  T* obase = (T*)prm.o + b * prm.os[0] + h * prm.os[1];
  auto write_rows = [&](int first_row, int rows) {      // staged rows [0, rows) are query rows q0w + first_row ..
#pragma unroll
    for (int it = 0; it < STAGE_ROWS * CH / 64; ++it) {
      const int idx = it * 64 + lane, row = idx / CH, ch = idx % CH;
      const i32x4 piece = *(FO_LDS const i32x4*)(stage + row * OROW + ch * 16);
      if (row < rows && q0w + first_row + row < Sq) *(i32x4*)(obase + (int64_t)(q0w + first_row + row) * prm.os[2] + ch * 8) = piece;
    }
  };
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const float l_tot = l_run[qb] + half_swap(l_run[qb]);
    const float inv = 1.0f / l_tot;
    const int qi = q0w + 32 * qb + l32;
    const int srow = KEEP_ON ? l32 : 32 * qb + l32;
#pragma unroll
    for (int db = 0; db < DBLK; ++db) {
      f32x16 t = oacc[db][qb];
      asm volatile("" : "+v"(t));                       // one accumulator at a time through VGPRs
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        typedef __attribute__((ext_vector_type(4))) T vec4;
        vec4 o4;
#pragma unroll
        for (int u = 0; u < 4; ++u) o4[u] = (T)(t[rg * 4 + u] * inv);
        *(FO_LDS vec4*)(stage + srow * OROW + (32 * db + 8 * rg + 4 * hh) * 2) = o4;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (qi < Sq && prm.lse != nullptr && hh == 0)
      prm.lse[(int64_t)bh * Sq + qi] = (m_run[qb] * c + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f;
    if constexpr (KEEP_ON) write_rows(32 * qb, 32);
  }
  if constexpr (!KEEP_ON) write_rows(0, 32 * QB);

  // ---- on to the next block, if there is one
  if (!has_next) break;
  prefetched = prefetch_next;
  o_rows_whole = q0w + 32 * QB <= Sq;
  first_block = false;
  if (pass + 1 < n_pass) ++pass;
  else { wg_id += (int)gridDim.x; bh = next_bh; item = next_item; pass = 0; }
  }   // query blocks
}

// heads per group in the causal order "heaviest query blocks of a group's heads first" of the kernels that take one
// 128-row query block per workgroup (see launch_one)
[[maybe_unused]] static int heavy_first_group(const AttnParams& p, int D) {   // (used by the launchers only: not in every unit)
  const int64_t kv_bytes_head = (int64_t)p.Sk * D * 2 * 2, n_bh_x = ((int64_t)p.B * p.H) >> 3;
  const int order = tune(g_attn_order);
  int64_t group = order >= 0 ? order : 8 * n_bh_x * kv_bytes_head <= (256ll << 20) ? n_bh_x : (64ll << 20) / (8 * kv_bytes_head);
  if (order < 0 && group < 1) group = 1;
  if (group > n_bh_x) group = n_bh_x;
  return (int)group;
}

// compute units of the current device (asked once per device; 256 where no device answers)
static int device_cus() {
  constexpr int kMaxDev = 64;
  static std::atomic<int> cached[kMaxDev];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev) return 256;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

template <typename T, int D, bool CAUSAL, int QB, int DBG = 0, int BM = kWideBM, bool VBIAS = false>
static int launch_wide(AttnParams p, hipStream_t stream) {
  constexpr bool KEEP_ON = BM == kWideBM && !VBIAS;      // (as in the kernel)
  // rings; bias row; or the rows of O staged behind the first six slots of the rings, 32 rows of D + 8 elements per wave
  // (eight waves at head_dim 128: seven of them there, see the kernel)
  constexpr int kWavesHere = BM / (32 * QB);
  constexpr size_t kStageAll = (size_t)(kRing + 2) * kBN * D * 2 + kWavesHere * 32 * (D * 2 + 16);
  const size_t lds = KEEP_ON ? (kStageAll > 160 * 1024 ? kStageAll - 32 * (D * 2 + 16) : kStageAll) : 2 * (size_t)kRing * kBN * D * 2 + (VBIAS ? kVBiasKeys * 4 : 0);
  if (VBIAS && (p.Sk + kBN - 1) / kBN * kBN > kVBiasKeys) return FO_ERR_UNSUPPORTED;
  p.n_qblk = (p.Sq + BM - 1) / BM;
  unsigned grid = (unsigned)((BM == kWideBM ? wide_items(p.n_qblk, CAUSAL) : p.n_qblk) * p.B * p.H);
  if (BM == kWideBM) { p.tail_base = 0; if (p.id_limit > 0 && grid > (unsigned)p.id_limit) grid = (unsigned)p.id_limit; }
  else { p.id_limit = 0; if (CAUSAL) p.tail_base = 0; }
  if (BM != kWideBM && p.tail_base > 0) grid = 2u * (unsigned)(wide_items((p.Sq + kWideBM - 1) / kWideBM, false) * p.B * p.H - p.tail_base);
  p.keep_on = 0;
  if (KEEP_ON) {
    // attn.keep_on: 0 = one work item per workgroup and no copies ahead for the next query block; 1 = copies ahead for
    // the second block of a causal pair; 2 (default) = also one workgroup per CU that walks its share of the items
    // (blockIdx.x, + gridDim.x, ...: a multiple of 8 apart, so that an XCD keeps its heads)
    const int asked = tune(g_attn_keep_on);
    const int mode = asked < 0 ? 2 : asked;
    p.keep_on = mode != 0;
    const unsigned wgs = (unsigned)(device_cus() / 8 * 8);
    if (mode == 2 && wgs >= 8 && grid > wgs) grid = wgs;
  }
  p.heavy_first = (CAUSAL && BM != kWideBM) ? heavy_first_group(p, D) : 0;
  p.order_n = 0;
  static const hipError_t attr = hipFuncSetAttribute((const void*)attn_fwd_wide_kernel<T, D, CAUSAL, QB, DBG, BM, VBIAS>,
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (attr != hipSuccess) return FO_ERR_LAUNCH;
  attn_fwd_wide_kernel<T, D, CAUSAL, QB, DBG, BM, VBIAS><<<grid, BM / (32 * QB) * 64, lds, stream>>>(p);
  return launch_status();
}

// The four-wave 256-row kernel, non-causal, whose last round of one workgroup per CU would be half empty or emptier:
// the work items of that round go to a second launch, of the 128-row pipelined form, two workgroups per item. A 128-row
// workgroup takes about two thirds of the time of a 256-row one, and that round is paid at that price instead of in
// full. Measured (the chip holds a power budget, so a round in which only half the CUs work is already cheaper than a full
// one): 12 heads x 8192 keys, 384 items on 256 CUs, 381 -> 363 us; 12 x 6144, 288 items, 290 -> 256; 33 x 4096, 528 items,
// 315 -> 295; 36 x 2048 108 -> 101; 4 x 40 heads x 1024 keys 96-98 -> 98: from 2048 keys on. (attn.tail 0 switches it off.)
template <typename T, int D, bool VBIAS>
static int launch_rows256_w4_noncausal(AttnParams p, hipStream_t stream) {
  p.id_limit = 0;
  p.tail_base = 0;
  const int n_cu = device_cus();
  const int64_t ids = (int64_t)((p.Sq + kWideBM - 1) / kWideBM) * p.B * p.H;
  const int64_t tail = ids % n_cu;
  if (D == 128 && tune(g_attn_tail) != 0 && (n_cu & 7) == 0 && ids > n_cu && tail > 0 && 2 * tail <= n_cu && p.Sk >= 2048) {
    AttnParams head = p, rest = p;
    head.id_limit = (int)(ids - tail);
    rest.tail_base = (int)(ids - tail);
    const int rc = launch_wide<T, D, false, 2, 0, kWideBM, VBIAS>(head, stream);
    if (rc != FO_OK) return rc;
    return launch_wide<T, D, false, 1, 0, kBM, VBIAS>(rest, stream);
  }
  return launch_wide<T, D, false, 2, 0, kWideBM, VBIAS>(p, stream);
}

template <typename T, int D, bool CAUSAL, bool LAZY, int DBG, bool DROP = false, bool BIAS = false, bool KBIAS = false>
static int launch_one(const AttnParams& p, hipStream_t stream) {
  const size_t lds_max = 4 * (size_t)kBN * D * 2 + (BIAS ? 2 * kWaves * 32 * kBN * 4 : 0) + (KBIAS ? 2 * kBN * 4 : 0);   // K, V tiles; bias tiles
  const size_t lds = 4 * (size_t)kBN * D * 2 + (BIAS && p.bias.dma_ok ? 2 * kWaves * 32 * kBN * 4 : 0) + (KBIAS ? 2 * kBN * 4 : 0);
  const unsigned grid = (unsigned)(p.n_qblk * p.B * p.H);
  static const hipError_t attr = hipFuncSetAttribute((const void*)attn_fwd_kernel<T, D, CAUSAL, LAZY, DBG, DROP, BIAS, KBIAS>,
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_max);
  if (attr != hipSuccess) return FO_ERR_LAUNCH;
  // Order of the workgroups of one XCD when causal: the heaviest query blocks of all its heads first, then the next
  // lighter ones, so that the light blocks fill the gaps at the end. (Head by head - each head's blocks from the
  // heaviest to the lightest - starts heavy blocks late: 25 % slower at S=1024..2048, 5 % at S=8192.) That walks
  // through the K and V of all those heads once per block index: when they do not all fit the memory-side cache
  // (256 MiB) the heads are taken in groups whose K and V (over the eight XCDs) stay within a quarter of it - with
  // 512 heads of 1 MiB in one group the kernel is bound by HBM (0.90 ms against 0.67 ms).
  AttnParams q = p;
  q.heavy_first = CAUSAL ? heavy_first_group(p, D) : 0;
  q.order_n = 0;
  if (CAUSAL && q.heavy_first > 0 && tune(g_attn_balance) != 0) {
    // When an XCD's workgroups are all resident at once (three per compute unit at head_dim 64, two at 128), they are
    // placed in launch order, one per unit in turn: unit m gets positions m, m + C, m + 2C of the XCD's list. In the
    // plain heaviest-first order that is the m-th heaviest of every layer, and the units' sums differ widely
    // (GPT-2-small shape, 96 workgroups per XCD on 32 units: 20 to 34 key tiles per unit). So the positions are filled
    // from a table: workgroups by falling size, each to the unit with the least work so far that still has a position
    // free (26 to 28 tiles per unit; 25.0 -> about 21 us). With more workgroups than fit at once the later ones start
    // wherever a slot frees, and the plain order is the better one.
    const int cus_x = device_cus() / 8, n_bh_x = (int)(((int64_t)p.B * p.H) >> 3);
    const int64_t n = (int64_t)n_bh_x * p.n_qblk;
    const int resident = (D == 64 && !DROP && !BIAS && !KBIAS) ? 3 : 2;      // workgroups per compute unit (registers)
    if (q.heavy_first == n_bh_x && cus_x > 0 && cus_x <= kOrderTab && n <= (int64_t)cus_x * resident && n <= kOrderTab && n > cus_x) {
      // (the table of the last shape is kept per host thread: filling it takes a few microseconds, a training loop
      // launches the same shape over and over)
      struct Memo { int n, n_bh_x, n_qblk, Sk, cus_x; uint8_t tab[kOrderTab]; };
      static thread_local Memo memo = {0, 0, 0, 0, 0, {0}};
      if (memo.n != (int)n || memo.n_bh_x != n_bh_x || memo.n_qblk != p.n_qblk || memo.Sk != p.Sk || memo.cus_x != cus_x) {
        int load[kOrderTab] = {0}, used[kOrderTab] = {0};
        for (int rank = 0; rank < (int)n; ++rank) {
          const int qblk = p.n_qblk - 1 - rank / n_bh_x;
          const int tiles = ((p.Sk < (qblk + 1) * kBM ? p.Sk : (qblk + 1) * kBM) + kBN - 1) / kBN;
          int best = -1;
          for (int m = 0; m < cus_x; ++m) {
            const int cap = (int)((n - m + cus_x - 1) / cus_x);      // positions m, m + C, ... below n
            if (used[m] < cap && (best < 0 || load[m] < load[best])) best = m;
          }
          memo.tab[used[best] * cus_x + best] = (uint8_t)rank;
          load[best] += tiles;
          used[best] += 1;
        }
        memo.n = (int)n; memo.n_bh_x = n_bh_x; memo.n_qblk = p.n_qblk; memo.Sk = p.Sk; memo.cus_x = cus_x;
      }
      for (int i = 0; i < (int)n; ++i) q.order_tab[i] = memo.tab[i];
      q.order_n = (int)n;
    }
  }
  attn_fwd_kernel<T, D, CAUSAL, LAZY, DBG, DROP, BIAS, KBIAS><<<grid, kWaves * 64, lds, stream>>>(q);
  return launch_status();
}

// Which kernel a call takes: FO_ATTN_KERNEL_ROWS128 / _ROWS128_EXACT (the 128-row kernel with the lazily raised or the
// exact running maximum), FO_ATTN_KERNEL_ROWS256_W8 / _W4 (the 256-row kernel, eight waves x 32 rows or four x 64).
// `forced` is the value of attn.variant (-1: the library's choice). Values from 256 on are timing ablations and exist
// only in a build with FO_ABLATIONS.
static int choose_kernel(const AttnParams& p, int D, bool causal, bool dropout, int forced) {
  // dropout, a bias with a query stride and head dims other than 64 and 128 run on the 128-row kernel; a bias that is
  // the same for every query (and short enough for the pipelined kernel to keep it in LDS) takes part in the choice
  const bool key_bias = p.bias.ptr != nullptr && p.bias.strides[2] == 0 && ((int64_t)p.Sk + kBN - 1) / kBN * kBN <= kVBiasKeys;
  if ((p.bias.ptr != nullptr && !key_bias) || dropout || p.d != D) return FO_ATTN_KERNEL_ROWS128;
  // The 256-row kernel addresses a head's keys with 32-bit byte offsets ...
  const bool wide_ok = (int64_t)p.Sk * (p.ks[2] > p.vs[2] ? p.ks[2] : p.vs[2]) * 2 < (1ll << 31);
  // ... and needs one 256-row workgroup (two query blocks each when causal) per CU to be worth it: below that the
  // 128-row kernel, with four times as many workgroups, fills the chip better
  const int n_cu = device_cus();
  const int64_t wide_wgs = (int64_t)wide_items((p.Sq + kWideBM - 1) / kWideBM, causal) * p.B * p.H;
  int v = forced;
  if (forced < 0) {
    const int keys = causal ? (p.Sq < p.Sk ? p.Sq : p.Sk) : p.Sk;
    // One workgroup per CU at a time: the launch runs in rounds, and a last round that is mostly empty is paid in full.
    // With the rounds filled to less than 80 % the 128-row kernel (two workgroups per CU, finer blocks, heaviest first)
    // was 1-5 % faster (B*H = 160-192 at 512-1024 keys, 48 heads x 4096 causal), from 83 % on the 256-row kernel 3-6 %.
    const int64_t rounds = (wide_wgs + n_cu - 1) / n_cu;
    // (non-causal at head_dim 128 a last round that is at most half full goes to a second launch of the 128-row form,
    // launch_rows256_w4_noncausal, and counts 0.6 of a round: 33 heads x 4096 keys, 528 items, 295 us that way against
    // 359 us on the 128-row kernel; 12 heads x 6144 keys, 288 items, 256 against 288 us)
    int64_t tenths = rounds * 10;
    {
      const int64_t tail = wide_wgs % n_cu;
      if (!causal && D == 128 && p.Sk >= 2048 && tune(g_attn_tail) != 0 && (n_cu & 7) == 0 && wide_wgs > n_cu && tail > 0 && 2 * tail <= n_cu)
        tenths = (rounds - 1) * 10 + 6;
    }
    bool wide = wide_ok && wide_wgs >= n_cu && wide_wgs * 100 >= tenths * n_cu * (D == 128 && keys >= 4096 ? 7 : 8);
    // (long rows of keys at head_dim 128: also with the rounds filled to 70-80 % - 12 heads x 8192 non-causal, 384
    // workgroups, 375 against 399 us - and with three quarters of a single round - 12 heads x 8192 causal 196 against 215 us,
    // 12 heads x 4096 non-causal 98 against 121 us)
    if (wide_ok && D == 128 && keys >= 4096 && wide_wgs < n_cu && wide_wgs * 4 >= (int64_t)n_cu * 3) wide = true;
    // head_dim 128, causal: from 1024 queries on (B*H = 128: 1024 queries -8 %, 1536 -16 %, 2048 -12 % against the
    // 128-row kernel; 512 and 768 queries +7 % and +18 %, a 256-row block being a large part of so small a triangle).
    if (D == 128 && causal && p.Sq < 1024) wide = false;
    // head_dim 64 (half the MFMAs per score, so the softmax weighs twice as much and the 128-row kernel's workgroups
    // sharing a CU hide it better): only for long rows of keys, and as four waves x 64 rows, which halves the LDS reads
    // per MFMA (on random operands this head_dim too runs at the clock the power budget leaves: all-zero operands take
    // 28 % less time). Four-wave form against the 128-row kernel: non-causal 1024 keys +2 %, 2048 -3 %, 4096 -6 %,
    // 8192 -6.5 %, 16384 -6 %; causal 2048 +3 %, 4096 -2 %, 8192 -5 %, 16384 -8 %. (The eight-wave form is 4-5 % behind
    // the four-wave form everywhere: non-causal 1024 keys +20 %, 4096 +0.6 %, 16384 -1.8 % against the 128-row kernel.)
    // Since the four-wave form's workgroups walk their items, without bias: non-causal 1024 keys +6 %, 2048 +2 %, 3072
    // -0.8 %, 4096 -1 %; causal 2048 +2 %, 4096 -8 %, 6144 -4.5 %, 8192 -6.5 %.
    if (D == 64 && keys < (causal && !key_bias ? 4096 : causal ? 8192 : 4096)) wide = false;
    v = wide ? FO_ATTN_KERNEL_ROWS256_W8 : FO_ATTN_KERNEL_ROWS128;
    // Few workgroups for the chip (12 heads of a tensor-parallel split, short batches): what bounds the launch then is
    // the time a workgroup takes per key tile, not throughput, and 128-row workgroups in the pipelined kernel take less
    // than the plain 128-row kernel (which runs S, the softmax and P V of a tile one after the other). Measured, plain
    // against pipelined, head_dim 128 causal: 12 heads x 2048 45 -> 36 us, x 4096 87 -> 66 us, 32 heads x 2048 56 -> 50;
    // non-causal 12 x 2048 46 -> 37, 8 x 4096 87 -> 72; head_dim 64 causal 12 x 4096 60 -> 50, 12 x 8192 139 -> 129. With
    // more 128-row workgroups than the chip holds at once (twice that when causal, the average block being half) the
    // other kernels are ahead again; below 1024 keys (2048 at head_dim 64) there is nothing to gain.
    if (!wide && wide_ok) {
      const int64_t wgs128 = ((int64_t)p.Sq + kBM - 1) / kBM * p.B * p.H;
      const int64_t slots = (int64_t)n_cu * (D == 64 ? 2 : 1) * (causal ? 2 : 1);
      if (wgs128 <= slots && keys >= (D == 64 ? 2048 : 1024)) v = FO_ATTN_KERNEL_ROWS128_PIPE;
    }
    // head_dim 128 with many key tiles per query block: four waves x 64 rows. Every K / V^T fragment read from LDS feeds two
    // MFMAs, which costs less energy (at full load the chip's clock is what its power budget leaves) but more cycles per
    // tile, and its longer pipeline fill and drain have to be spread over enough tiles. Measured on one box, new form
    // against the eight-wave form: non-causal 2048 keys -1.0 %, 4096 -2.3 %, 8192 -2.5 %; causal 3072 +3 %, 4096 +1 %,
    // 8192 -0.7 %, 16384 -1.8 %. With its workgroups walking their items (attn.keep_on), on one box: non-causal 512 keys
    // -4 %, 768 -2 %, 1024 -2.5 %, 1536 -1 %, 2048 -1.5 %; causal 2048 +3.5 %, 3072 +2 %, 4096 +1.7 %, 6144 +2.4 %,
    // 8192 -1 to -3 % (a causal block's diagonal costs the 64-row waves more than the 32-row ones).
    if (v == FO_ATTN_KERNEL_ROWS256_W8 && (D == 64 || keys >= (causal ? 8192 : 512))) v = FO_ATTN_KERNEL_ROWS256_W4;
  }
  if (v >= 256) return v;
  if (!wide_ok && v >= FO_ATTN_KERNEL_ROWS128_PIPE) v = FO_ATTN_KERNEL_ROWS128;
  if (key_bias) {
    // with a bias the pipelined kernel exists in two forms: 128 rows, and 256 rows as four waves
    if (v == FO_ATTN_KERNEL_ROWS256_W8) v = FO_ATTN_KERNEL_ROWS256_W4;
    if (v == FO_ATTN_KERNEL_ROWS128_EXACT) v = FO_ATTN_KERNEL_ROWS128;
  }
  return v;
}

template <typename T, int D>
int launch(const AttnParams& p, bool causal, bool dropout, hipStream_t stream) {
  if (p.bias.ptr != nullptr) {
    // A bias that is the same for every query has kernels of its own: the pipelined ones where choose_kernel says so, else
    // the per-key form of the 128-row kernel, with or without dropout. (attn.variant 1 keeps the general bias kernel,
    // which takes any strides: tests compare the two.)
    if (p.bias.strides[2] == 0 && tune(g_attn_variant) != FO_ATTN_KERNEL_ROWS128_EXACT) {
      if (!dropout) {
        const int v = choose_kernel(p, D, causal, dropout, tune(g_attn_variant));
        if (v >= 256) return FO_ERR_UNSUPPORTED;
        if (v == FO_ATTN_KERNEL_ROWS128_PIPE)
          return causal ? launch_wide<T, D, true, 1, 0, kBM, true>(p, stream) : launch_wide<T, D, false, 1, 0, kBM, true>(p, stream);
        if (v == FO_ATTN_KERNEL_ROWS256_W4)
          return causal ? launch_wide<T, D, true, 2, 0, kWideBM, true>(p, stream) : launch_rows256_w4_noncausal<T, D, true>(p, stream);
        return causal ? launch_one<T, D, true, true, 0, false, false, true>(p, stream) : launch_one<T, D, false, true, 0, false, false, true>(p, stream);
      }
      return causal ? launch_one<T, D, true, true, 0, true, false, true>(p, stream) : launch_one<T, D, false, true, 0, true, false, true>(p, stream);
    }
    if (dropout) return causal ? launch_one<T, D, true, true, 0, true, true>(p, stream) : launch_one<T, D, false, true, 0, true, true>(p, stream);
    return causal ? launch_one<T, D, true, true, 0, false, true>(p, stream) : launch_one<T, D, false, true, 0, false, true>(p, stream);
  }
  if (dropout) return causal ? launch_one<T, D, true, true, 0, true>(p, stream) : launch_one<T, D, false, true, 0, true>(p, stream);
  const int v = choose_kernel(p, D, causal, dropout, tune(g_attn_variant));
  if (v == FO_ATTN_KERNEL_ROWS256_W8) return causal ? launch_wide<T, D, true, 1>(p, stream) : launch_wide<T, D, false, 1>(p, stream);
  if (v == FO_ATTN_KERNEL_ROWS128_PIPE) return causal ? launch_wide<T, D, true, 1, 0, kBM>(p, stream) : launch_wide<T, D, false, 1, 0, kBM>(p, stream);
  if (v == FO_ATTN_KERNEL_ROWS256_W4) return causal ? launch_wide<T, D, true, 2>(p, stream) : launch_rows256_w4_noncausal<T, D, false>(p, stream);
#if defined(FO_ABLATIONS)
  // Timing ablations (WRONG results by design; bf16, head_dim 128 only). 256-row kernel, non-causal: 256 + bits for eight
  // waves, 512 + bits for four; bit 0 no global->LDS copies, 1 no exponentials, 2 no LDS fragment reads, 5 no wait for
  // copies, 6 no barrier. 128-row kernel, causal: 2..11.
  if constexpr (D == 128 && std::is_same<T, __bf16>::value) {
    if (v >= 256 && !causal) {
      switch (v) {
        case 256 + 1: return launch_wide<T, D, false, 1, 1>(p, stream);
        case 256 + 2: return launch_wide<T, D, false, 1, 2>(p, stream);
        case 256 + 4: return launch_wide<T, D, false, 1, 4>(p, stream);
        case 256 + 7: return launch_wide<T, D, false, 1, 7>(p, stream);
        case 256 + 64: return launch_wide<T, D, false, 1, 64>(p, stream);
        case 256 + 128: return launch_wide<T, D, false, 1, 128>(p, stream);
        case 512 + 128: return launch_wide<T, D, false, 2, 128>(p, stream);
        case 512 + 1: return launch_wide<T, D, false, 2, 1>(p, stream);
        case 512 + 2: return launch_wide<T, D, false, 2, 2>(p, stream);
        case 512 + 4: return launch_wide<T, D, false, 2, 4>(p, stream);
        case 512 + 64: return launch_wide<T, D, false, 2, 64>(p, stream);
        case 512 + 7: return launch_wide<T, D, false, 2, 7>(p, stream);
        case 512 + 8: return launch_wide<T, D, false, 2, 8>(p, stream);
        default: return FO_ERR_UNSUPPORTED;
      }
    }
    if (causal) {
      switch (v >> 1) {
        case 1: return launch_one<T, D, true, true, 1>(p, stream);
        case 2: return launch_one<T, D, true, true, 2>(p, stream);
        case 3: return launch_one<T, D, true, true, 3>(p, stream);
        case 4: return launch_one<T, D, true, true, 5>(p, stream);
        case 5: return launch_one<T, D, true, true, 7>(p, stream);
        default: break;
      }
    }
  }
#endif
  if (v != FO_ATTN_KERNEL_ROWS128 && v != FO_ATTN_KERNEL_ROWS128_EXACT) return FO_ERR_UNSUPPORTED;
  const bool lazy = v == FO_ATTN_KERNEL_ROWS128;
  if (causal) return lazy ? launch_one<T, D, true, true, 0>(p, stream) : launch_one<T, D, true, false, 0>(p, stream);
  return lazy ? launch_one<T, D, false, true, 0>(p, stream) : launch_one<T, D, false, false, 0>(p, stream);
}

// one translation unit per operand type and head_dim defines its launch<T, D>; the others see a declaration
#define FO_ATTN_LAUNCH(UNIT, T, D)                                                                  \
  FO_ATTN_EXTERN_##UNIT template int launch<T, D>(const AttnParams&, bool, bool, hipStream_t);
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

// The checks on sizes and strides that fo_attn_fwd and fo_attn_fwd_kernel share, so that the query answers "rejected"
// exactly where the call would.
static int check_sizes(int B, int H, int Sq, int Sk, int D) {
  if (D < 8 || D > 128 || D % 8 != 0) return FO_ERR_BAD_HEAD_DIM;
  if (B <= 0 || H <= 0 || Sq <= 0 || Sk <= 0) return FO_ERR_BAD_SHAPE;
  const int64_t n_qblk = ((int64_t)Sq + kBM - 1) / kBM;
  if (n_qblk * B * H > 0x7FFFFFFFll || (int64_t)B * H * Sq > (1ll << 40)) return FO_ERR_BAD_SHAPE;
  return FO_OK;
}
// three element strides (batch, head, sequence) of one operand: rows start on 16-byte boundaries (8 elements) and do not
// overlap; only K/V may repeat a head (stride 0 = multi-query), which the caller checks for the output. The kernels
// address the 64 rows of a key tile with 32-bit byte offsets (the 256-row kernel, whose offsets span a whole head, is
// chosen only where they fit): a K/V row stride must stay below 2^24 elements.
static int check_strides(const int64_t* st, int D, bool key_or_value) {
  for (int i = 0; i < 3; ++i) {
    if (st[i] < 0 || (st[i] % 8) != 0) return FO_ERR_BAD_STRIDE;
  }
  if (st[2] < D) return FO_ERR_BAD_STRIDE;
  if (key_or_value && st[2] >= kMaxRowStride) return FO_ERR_BAD_STRIDE;
  return FO_OK;
}

static int attn_fwd_impl(const void* q, const void* k, const void* v, void* o, float* lse,
                         int B, int H, int Sq, int Sk, int D,
                         const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os,
                         float softmax_scale, int causal, int dtype, float dropout_p, uint32_t seed, uint64_t rng_offset,
                         const void* bias, const int64_t* bias_strides, int bias_dtype, void* stream) {
  if (!q || !k || !v || !o || !qs || !ks || !vs || !os) return FO_ERR_NULL_POINTER;
  if (dtype != FO_DTYPE_F16 && dtype != FO_DTYPE_BF16) return FO_ERR_BAD_DTYPE;
  if (const int rc = check_sizes(B, H, Sq, Sk, D)) return rc;
  const int64_t n_qblk = ((int64_t)Sq + kBM - 1) / kBM;
  if (const int rc = check_strides(qs, D, false)) return rc;
  if (const int rc = check_strides(ks, D, true)) return rc;
  if (const int rc = check_strides(vs, D, true)) return rc;
  if (const int rc = check_strides(os, D, false)) return rc;
  if (os[0] == 0 && B > 1) return FO_ERR_BAD_STRIDE;
  if (os[1] == 0 && H > 1) return FO_ERR_BAD_STRIDE;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o) & 15u) return FO_ERR_MISALIGNED;
  if (lse && ((uintptr_t)lse & 3u)) return FO_ERR_MISALIGNED;
  if (!(softmax_scale > 0.0f) || softmax_scale > 3.0e38f) return FO_ERR_BAD_SHAPE;   // also rejects NaN
  if (!(dropout_p >= 0.0f) || dropout_p >= 1.0f) return FO_ERR_BAD_SHAPE;
  if (bias) {
    if (!bias_strides) return FO_ERR_NULL_POINTER;
    if (bias_dtype != FO_DTYPE_F32 && bias_dtype != dtype) return FO_ERR_BAD_DTYPE;
    if (bias_strides[0] < 0 || bias_strides[1] < 0 || bias_strides[2] < 0) return FO_ERR_BAD_STRIDE;
    if ((uintptr_t)bias & (bias_dtype == FO_DTYPE_F32 ? 3u : 1u)) return FO_ERR_MISALIGNED;
  }

  AttnParams p;
  p.q = q; p.k = k; p.v = v; p.o = o; p.lse = lse;
  p.B = B; p.H = H; p.Sq = Sq; p.Sk = Sk; p.d = D;
  for (int i = 0; i < 3; ++i) { p.qs[i] = qs[i]; p.ks[i] = ks[i]; p.vs[i] = vs[i]; p.os[i] = os[i]; }
  p.scale_log2e = softmax_scale * 1.4426950408889634f;
  p.n_qblk = (int)n_qblk;
  p.heavy_first = 0; p.order_n = 0; p.id_limit = 0; p.tail_base = 0; p.keep_on = 0;
  const bool drop = dropout_p > 0.0f;
  p.drop = make_dropout(dropout_p, seed, rng_offset);
  p.bias.ptr = bias;
  for (int i = 0; i < 3; ++i) p.bias.strides[i] = bias ? bias_strides[i] : 0;
  p.bias.is_f32 = bias_dtype == FO_DTYPE_F32;
  {
    const int64_t elt = p.bias.is_f32 ? 4 : 2;
    p.bias.vec_ok = bias && ((uintptr_t)bias % (4 * elt)) == 0 && p.bias.strides[0] % 4 == 0 && p.bias.strides[1] % 4 == 0 && p.bias.strides[2] % 4 == 0;
    // (a bias that is the same for every query - query stride 0 - is one row per tile: per-element loads of it are
    // broadcasts, and the kernel keeps its two workgroups per CU without the LDS for bias tiles)
    p.bias.dma_ok = bias && p.bias.strides[2] != 0 && ((uintptr_t)bias % 16) == 0 && (p.bias.strides[0] * elt) % 16 == 0 &&
                    (p.bias.strides[1] * elt) % 16 == 0 && (p.bias.strides[2] * elt) % 16 == 0;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  // kernels are compiled for 64 and 128 columns; a head_dim in between runs on the next one with zero columns
  if (dtype == FO_DTYPE_BF16) return D > 64 ? launch<__bf16, 128>(p, causal != 0, drop, s) : launch<__bf16, 64>(p, causal != 0, drop, s);
  return D > 64 ? launch<_Float16, 128>(p, causal != 0, drop, s) : launch<_Float16, 64>(p, causal != 0, drop, s);
}

extern "C" int fo_attn_fwd_kernel(int B, int H, int Sq, int Sk, int D, const int64_t* ks, const int64_t* vs,
                                  int causal, int has_bias, int has_dropout) {
  if (!ks || !vs) return FO_ERR_NULL_POINTER;
  if (const int rc = check_sizes(B, H, Sq, Sk, D)) return rc;
  if (const int rc = check_strides(ks, D, true)) return rc;
  if (const int rc = check_strides(vs, D, true)) return rc;
  AttnParams p = {};
  p.B = B; p.H = H; p.Sq = Sq; p.Sk = Sk; p.d = D;
  for (int i = 0; i < 3; ++i) { p.ks[i] = ks[i]; p.vs[i] = vs[i]; }
  p.bias.ptr = has_bias ? (const void*)ks : nullptr;   // (only tested against NULL)
  p.bias.strides[2] = has_bias == 2 ? 0 : 1;
  return choose_kernel(p, D > 64 ? 128 : 64, causal != 0, has_dropout != 0, tune(g_attn_variant));
}

extern "C" int fo_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
                           int B, int H, int Sq, int Sk, int D,
                           const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os,
                           float softmax_scale, int causal, int dtype, void* stream) {
  return attn_fwd_impl(q, k, v, o, lse, B, H, Sq, Sk, D, qs, ks, vs, os, softmax_scale, causal, dtype, 0.0f, 0u, 0ull, nullptr, nullptr, 0, stream);
}

extern "C" int fo_attn_fwd_dropout(const void* q, const void* k, const void* v, void* o, float* lse,
                                   int B, int H, int Sq, int Sk, int D,
                                   const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os,
                                   float softmax_scale, int causal, int dtype, float dropout_p, uint32_t seed, uint64_t rng_offset,
                                   void* stream) {
  return attn_fwd_impl(q, k, v, o, lse, B, H, Sq, Sk, D, qs, ks, vs, os, softmax_scale, causal, dtype, dropout_p, seed, rng_offset, nullptr, nullptr, 0, stream);
}

extern "C" int fo_attn_fwd_ex(const void* q, const void* k, const void* v, void* o, float* lse,
                              int B, int H, int Sq, int Sk, int D,
                              const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os,
                              float softmax_scale, int causal, int dtype, const fo_attn_extras* extras, void* stream) {
  if (!extras) return attn_fwd_impl(q, k, v, o, lse, B, H, Sq, Sk, D, qs, ks, vs, os, softmax_scale, causal, dtype, 0.0f, 0u, 0ull, nullptr, nullptr, 0, stream);
  return attn_fwd_impl(q, k, v, o, lse, B, H, Sq, Sk, D, qs, ks, vs, os, softmax_scale, causal, dtype, extras->dropout_p,
                       extras->dropout_seed, extras->dropout_offset, extras->bias, extras->bias_strides, extras->bias_dtype, stream);
}
#endif  // FO_ATTN_UNIT == 0
