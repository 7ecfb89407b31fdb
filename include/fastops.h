/* fastops.h - C ABI of libfastops_hip.so: FlashAttention forward and the fused Lion step for AMD MI355X (gfx950).
 *
 * This is the boundary that replaces the reference's two pybind11 torch extensions:
 *   fast_ops/flash_attention/flash_attention.cpp:12-14   forward(Q, K, V) -> O
 *   fast_ops/lion/lion.cpp:13-15                         lion_update(param, grad, exp_avg, lr, beta1, beta2, wd)
 *
 * Conventions
 *   - plain pointers and sizes only; every pointer is a device pointer unless its name ends in _host;
 *   - the library allocates nothing, frees nothing and keeps no pointer after a call returns;
 *   - every call is asynchronous on the hipStream_t passed as `stream` (NULL = the default stream), never
 *     synchronises, and may be issued from several host threads on different streams;
 *   - return value 0 (FO_OK) or a negative fo_status; nothing throws or aborts. All argument checks happen before
 *     any HIP call, so a rejected call has touched neither the device nor the stream.
 */
#ifndef FASTOPS_H_
#define FASTOPS_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum fo_status {
  FO_OK = 0,
  FO_ERR_NULL_POINTER = -1,   /* a required pointer is NULL */
  FO_ERR_BAD_DTYPE = -2,      /* dtype code is not FO_DTYPE_F16 / FO_DTYPE_BF16 (the reference dispatches half types only,
                                 flash_attention/common/launch_utils.h:8-21) */
  FO_ERR_BAD_HEAD_DIM = -3,   /* head_dim not supported: the reference's contract, a multiple of 8 up to 128
                                 (flash_attention.py:61-66), is what this library implements */
  FO_ERR_BAD_SHAPE = -4,      /* a size is <= 0, or too large for the kernel's indexing */
  FO_ERR_BAD_STRIDE = -5,     /* a stride breaks the layout contract (rows must be 16-byte aligned) */
  FO_ERR_MISALIGNED = -6,     /* a base pointer is not aligned as required */
  FO_ERR_LAUNCH = -7,         /* hipGetLastError() reported a failure after the launch (the reference's
                                 C10_CUDA_KERNEL_LAUNCH_CHECK, lion_update.cu:159) */
  FO_ERR_UNSUPPORTED = -8     /* valid request that this build does not implement */
} fo_status;

enum { FO_DTYPE_F16 = 0, FO_DTYPE_BF16 = 1, FO_DTYPE_F32 = 2 /* Lion entry points only */ };

/* Human-readable text for a status code; never NULL. */
const char* fo_strerror(int status);

/* Library ABI version: major*1000 + minor. 2000: the workspace of fo_attn_bwd holds two values per query row
 * ([2, B, H, Sq] fp32; 1000: one), and fo_attn_fwd_kernel / fo_attn_bwd_static_ws exist. */
int fo_version(void);

/* Tuning hook for benchmarks, profiling and tests: selects a kernel variant or a workgroup order by name
 * ("lion.variant", "attn.variant", "attn_bwd.variant", "attn.order", "attn.balance", "attn.keep_on", "attn.tail", "attn_bwd.order"). Every value it accepts selects
 * code that computes the same function as the default; value -1 restores the default (the measured best). Returns
 * FO_OK, or FO_ERR_UNSUPPORTED for an unknown key or a value that selects nothing. The settings are process-global
 * atomics: a call reads each one once, a call already issued is not affected. fo_tune_get additionally answers
 * "build.ablations" (1 if the library was built with the timing ablations of the attention forward, which produce
 * wrong results by design and which a default build does not contain; 0 otherwise). No reference counterpart. */
int fo_tune_set(const char* key, int value);
int fo_tune_get(const char* key);

/* ---------------------------------------------------------------------------------------------------------------
 * FlashAttention forward.
 * Replaces flash_attn_fwd / flash_attn_fwd_cuda (flash_attention.cpp:5-10, flash_attention_fwd.cu:154-181) and
 * implements what that unfinished kernel's comments describe (flash_attention_fwd.cu:37-47,120-151) with the numerics
 * of the reference's working Triton forward (flash_attention_triton.py:128-255): O = softmax(scale * Q K^T + mask) V
 * with fp32 scores and accumulators, and LSE = natural-log logsumexp of the scaled, masked scores.
 *
 *   q            [B, H, Sq, D]   element (b,h,s,d) at q + b*q_strides[0] + h*q_strides[1] + s*q_strides[2] + d
 *   k, v         [B, H, Sk, D]   same addressing with their own strides
 *   o            [B, H, Sq, D]   written for every (b,h,s,d); never read
 *   lse          [B, H, Sq] fp32, contiguous; may be NULL when the caller does not want it
 *   *_strides    three element strides (batch, head, sequence); the head_dim stride is 1. A [B,S,H,D] tensor (the
 *                layout of flash_attention_triton.py:734-737) is passed by swapping the head and sequence strides;
 *                a head stride of 0 expresses multi-query K/V.
 *   causal       non-zero: query i attends keys j <= i (top-left aligned, attention_ref.py:54-58)
 *   dtype        FO_DTYPE_F16 or FO_DTYPE_BF16, for q, k, v and o alike
 *
 * Requirements checked here: D a multiple of 8 from 8 to 128 (64 and 128 are the sizes the kernels are laid out for; any
 * other runs on the next of the two with the missing columns read as zeros and never stored - no copies, the same
 * results, the speed of the larger size); Sq, Sk >= 1; softmax_scale finite and > 0; base pointers and row strides
 * multiples of 16 bytes; sequence strides of k and v below 2^24 elements (FO_ERR_BAD_STRIDE otherwise: the kernels
 * address the rows of a key tile with 32-bit byte offsets).
 */
int fo_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
                int B, int H, int Sq, int Sk, int D,
                const int64_t* q_strides_host, const int64_t* k_strides_host,
                const int64_t* v_strides_host, const int64_t* o_strides_host,
                float softmax_scale, int causal, int dtype, void* stream);

/* Which kernel fo_attn_fwd (or _dropout / _ex, with has_dropout / has_bias non-zero) launches for a call of this shape
 * on the current device with the current "attn.variant": one of the FO_ATTN_KERNEL_* codes below, or a negative
 * fo_status where fo_attn_fwd would reject the shape. has_bias: 0 none, 1 a bias with a query stride, 2 a bias that is
 * the same for every query (query stride 0), which the pipelined kernels take as well. Launches nothing. The choice
 * depends on the number of compute units of the current device. No reference counterpart:
 * the reference has one kernel (flash_attention_fwd.cu:164-177); tests use this to assert which code they covered. */
enum {
  FO_ATTN_KERNEL_ROWS128 = 0,         /* 128 query rows per workgroup, reference maximum raised lazily */
  FO_ATTN_KERNEL_ROWS128_EXACT = 1,   /* the same with the exact running maximum of flash_attention_triton.py:200-213 */
  FO_ATTN_KERNEL_ROWS128_PIPE = 8,    /* 128 query rows per workgroup, four waves x 32 rows, in the 256-row kernel's pipeline */
  FO_ATTN_KERNEL_ROWS256_W8 = 16,     /* 256 query rows per workgroup, eight waves x 32 rows */
  FO_ATTN_KERNEL_ROWS256_W4 = 32      /* 256 query rows per workgroup, four waves x 64 rows */
};
int fo_attn_fwd_kernel(int B, int H, int Sq, int Sk, int D, const int64_t* k_strides_host, const int64_t* v_strides_host,
                       int causal, int has_bias, int has_dropout);

/* ---------------------------------------------------------------------------------------------------------------
 * FlashAttention backward: dQ, dK, dV.
 * Implements the backward that flash_attention.py:40-45 leaves unimplemented, with the arithmetic of the reference's
 * Triton backward (flash_attention_triton.py:273-315 delta pre-pass, :322-638 kernel, :832-958 host): with
 * P = exp(scale * Q K^T - LSE) (masked entries 0), delta_i = sum_d dO_id O_id,
 *     dV = P^T dO,   dS = P * (dO V^T - delta) * scale,   dQ = dS K,   dK = dS^T Q;
 * fp32 scores and accumulators, P and dS rounded to the operand type before the second products.
 *
 *   q, k, v, o, lse     as passed to / produced by fo_attn_fwd (lse is required here)
 *   d_o                 [B, H, Sq, D] gradient of the output
 *   delta_ws            [2, B, H, Sq] fp32, contiguous: workspace supplied by the caller, overwritten (per query row
 *                       -delta and -LSE / scale, written by the first launch for the second)
 *   dq / dk, dv         [B, H, Sq, D] / [B, H, Sk, D], written for every element; never read
 *   strides_host        eight pointers to three element strides each (batch, head, sequence; head_dim stride 1), in
 *                       the order q, k, v, o, d_o, dq, dk, dv. Only the inputs may repeat a batch or head (stride 0).
 * Same requirements as fo_attn_fwd (D a multiple of 8 up to 128, 16-byte aligned pointers and rows, scale finite and > 0).
 * Two launches on `stream`; no atomics, results are deterministic.
 */
int fo_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                float* delta_ws, void* dq, void* dk, void* dv, int B, int H, int Sq, int Sk, int D,
                const int64_t* const* strides_host, float softmax_scale, int causal, int dtype, void* stream);

/* fo_attn_bwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): no workspace argument, and the call itself allocates and frees nothing. The
 * [2, B, H, Sq] fp32 workspace lives in a device array of the library (2 * FO_ATTN_BWD_STATIC_ROWS floats = 8 MiB,
 * which each GPU the library runs on holds until the process ends). B*H*Sq above FO_ATTN_BWD_STATIC_ROWS is refused with
 * FO_ERR_BAD_SHAPE. Same results as fo_attn_bwd, bit for bit. All calls on one GPU share the array: calls that
 * overlap on one GPU (different streams or threads) race on it and must be serialised by the caller; calls in stream
 * order on one stream are safe. The first call on a device looks up the array's address there (hipGetSymbolAddress;
 * not while a capture is in progress). No counterpart in the reference. */
#define FO_ATTN_BWD_STATIC_ROWS (1 << 20)
int fo_attn_bwd_static_ws(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                          void* dq, void* dk, void* dv, int B, int H, int Sq, int Sk, int D,
                          const int64_t* const* strides_host, float softmax_scale, int causal, int dtype, void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * The same two with dropout of the attention probabilities, as the reference's Triton kernels define it
 * (flash_attention_triton.py:38-50 hash, :125,:216-219 forward, :421,:524-532,:551,:599 backward): element
 * (b*H + h, q, key) has the 32-bit index rng_offset + (b*H + h)*Sq*Sk + q*Sk + key (arithmetic modulo 2^32); the index
 * xor seed goes through the integer hash of :44-48; the probability is kept iff the hash exceeds
 * uint32(fp32(dropout_p) * 2^32) and is then multiplied by 1 / (1 - dropout_p). Row sums, and so LSE, use the undropped
 * probabilities. The caller supplies seed and offset (the reference takes them from torch's generator state,
 * :641-665) and must pass the same pair to the backward. dropout_p in [0, 1); 0 is exactly fo_attn_fwd / fo_attn_bwd.
 */
int fo_attn_fwd_dropout(const void* q, const void* k, const void* v, void* o, float* lse,
                        int B, int H, int Sq, int Sk, int D,
                        const int64_t* q_strides_host, const int64_t* k_strides_host,
                        const int64_t* v_strides_host, const int64_t* o_strides_host,
                        float softmax_scale, int causal, int dtype,
                        float dropout_p, uint32_t seed, uint64_t rng_offset, void* stream);
int fo_attn_bwd_dropout(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                        float* delta_ws, void* dq, void* dk, void* dv, int B, int H, int Sq, int Sk, int D,
                        const int64_t* const* strides_host, float softmax_scale, int causal, int dtype,
                        float dropout_p, uint32_t seed, uint64_t rng_offset, void* stream);

/* The dropout keep-mask as a tensor of its own, one byte per element of [B, H, Sq, Sk] flattened (1 = kept): what
 * fo_attn_fwd_dropout applies for the same (dropout_p, seed, rng_offset). Replaces triton_dropout_mask's kernel
 * (flash_attention_triton.py:669-717), which the reference's tests use to build the mask for attention_ref. */
int fo_dropout_mask(uint8_t* keep, int64_t n_elements, float dropout_p, uint32_t seed, uint64_t rng_offset, void* stream);

/* Additive bias on the scaled scores, optionally together with dropout: scores = scale * Q K^T + bias
 * (flash_attention_triton.py:176-198,752-770; attention_ref.py:50-51). The reference's "vector" bias [.,.,1,Sk] and
 * "matrix" bias [.,.,Sq,Sk], broadcast over batch and heads, are all expressed by strides: element (b, h, q, key) is
 * read at bias + b*bias_strides[0] + h*bias_strides[1] + q*bias_strides[2] + key, a stride of 0 broadcasting that
 * dimension. bias_dtype is FO_DTYPE_F32 or the dtype of q. No gradient is computed for the bias (nor does the reference).
 * extras == NULL, or bias == NULL and dropout_p == 0, is exactly fo_attn_fwd / fo_attn_bwd. */
typedef struct fo_attn_extras {
  const void* bias;          /* NULL = no bias */
  int64_t bias_strides[3];   /* element strides: batch, head, query */
  int bias_dtype;
  float dropout_p;           /* 0 = no dropout */
  uint32_t dropout_seed;
  uint64_t dropout_offset;
} fo_attn_extras;
int fo_attn_fwd_ex(const void* q, const void* k, const void* v, void* o, float* lse,
                   int B, int H, int Sq, int Sk, int D,
                   const int64_t* q_strides_host, const int64_t* k_strides_host,
                   const int64_t* v_strides_host, const int64_t* o_strides_host,
                   float softmax_scale, int causal, int dtype, const fo_attn_extras* extras_host, void* stream);
int fo_attn_bwd_ex(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                   float* delta_ws, void* dq, void* dk, void* dv, int B, int H, int Sq, int Sk, int D,
                   const int64_t* const* strides_host, float softmax_scale, int causal, int dtype,
                   const fo_attn_extras* extras_host, void* stream);

/* ---------------------------------------------------------------------------------------------------------------
 * Fused Lion step: fp32 parameters, fp32 gradients, bf16 momentum, one pass.
 * Per element, in this order and with these rounding points (lion_optimizer_ref.py:51,64,65,67):
 *     p1 = p * c_wd
 *     u  = f32(bf16(m * c_b1)) + g * c_1b1
 *     p  = p1 + c_nlr * sign(u)                 sign(+-0) = sign(NaN) = 0
 *     m  = bf16( fma(c_1b2, g, f32(bf16(m * c_b2))) )
 * bf16() is round-to-nearest-even; a NaN stays a quiet NaN whose payload bits are unspecified. The kernel fuses what lion_update_kernel fuses
 * (lion_update.cu:44-106) but keeps the fp32 rounding points of the Python formula instead of half arithmetic.
 */
typedef struct fo_lion_consts {
  float c_wd;   /* f32(1 - lr*weight_decay) */
  float c_b1;   /* f32(beta1)               */
  float c_1b1;  /* f32(1 - beta1)           */
  float c_nlr;  /* f32(-lr)                 */
  float c_b2;   /* f32(beta2)               */
  float c_1b2;  /* f32(1 - beta2)           */
} fo_lion_consts;

/* Computes the six constants in double precision and rounds each once to fp32, exactly as the Python expressions of
 * lion_optimizer_ref.py:51,64,65,67 do. Host-only; `out_host` is host memory. */
int fo_lion_make_consts(double lr, double beta1, double beta2, double weight_decay, fo_lion_consts* out_host);

/* One tensor, in place. Replaces lion_update (lion.cpp:4-15, lion_update.cu:121-161). Any numel >= 0 and any
 * alignment of 4 bytes (p, g) / 2 bytes (m) is accepted; 16-byte aligned p, g and 8-byte aligned m take the
 * vector path. */
int fo_lion_update(float* p, const float* g, uint16_t* m, int64_t numel, const fo_lion_consts* consts_host, void* stream);

/* Many tensors in one launch. Replaces the per-parameter loop of Lion.step (lion_optimizer.py:64-76).
 * The caller splits every tensor into chunks of at most FO_LION_CHUNK elements (all but a tensor's last chunk are
 * exactly FO_LION_CHUNK long) and passes, in device memory, one descriptor per chunk. */
#define FO_LION_CHUNK 8192

typedef struct fo_lion_chunk {
  float* p;          /* first parameter of the chunk                          */
  const float* g;    /* first gradient of the chunk                           */
  uint16_t* m;       /* first momentum element (bf16 bit pattern) of the chunk */
  int32_t n;         /* elements in this chunk, 1..FO_LION_CHUNK              */
  int32_t reserved;  /* must be 0                                             */
} fo_lion_chunk;

int fo_lion_step(const fo_lion_chunk* chunks_dev, int64_t n_chunks, const fo_lion_consts* consts_host, void* stream);

/* Host-only helper: fills `out_host[0 .. return value)` with the chunk descriptors of one tensor and returns how many
 * it wrote (ceil(numel / FO_LION_CHUNK)); with out_host == NULL it only counts. */
int64_t fo_lion_fill_chunks(float* p, const float* g, uint16_t* m, int64_t numel, fo_lion_chunk* out_host);

/* ---------------------------------------------------------------------------------------------------------------
 * Fused Lion step for any parameter/gradient dtype P and momentum dtype M out of FO_DTYPE_F32 / F16 / BF16.
 * Covers the reference kernel's own case, all three tensors in one half type (lion_update.cu:132-141; exercised by
 * tests/test_lion_optimizer.py:11-13), and momenta kept in fp32 or fp16. The arithmetic is the reference formula's
 * (lion_optimizer_ref.py:51,64,65,67) under PyTorch's type promotion: every tensor-valued intermediate is computed
 * in fp32 and rounded to the dtype the torch expression has (P for p*c and g*(1-beta1), M for m*beta1 and m*beta2,
 * P if P == M else fp32 for their sum), sign(0) = sign(NaN) = 0, the momentum's add_(grad, alpha) is one fused
 * multiply-add. P = F32 with M = BF16 is forwarded to fo_lion_update / fo_lion_step.
 *
 * fo_lion_make_consts_typed: as fo_lion_make_consts, and when P == M is a half type additionally rounds c_nlr and c_1b2
 * to that type, as torch does with the `alpha` of an add_ between two tensors of one half type.
 * fo_lion_fill_chunks_typed / fo_lion_step_typed / fo_lion_update_typed: as their fp32+bf16 counterparts; the pointers
 * in fo_lion_chunk are then reinterpreted as pointers to P (p, g) and M (m). Alignment: element size; 16-byte aligned
 * p, g and an m aligned to 16 bytes' worth of elements take the vector path.
 */
int fo_lion_make_consts_typed(double lr, double beta1, double beta2, double weight_decay, int p_dtype, int m_dtype,
                              fo_lion_consts* out_host);
int64_t fo_lion_fill_chunks_typed(void* p, const void* g, void* m, int64_t numel, int p_dtype, int m_dtype, fo_lion_chunk* out_host);
int fo_lion_step_typed(const fo_lion_chunk* chunks_dev, int64_t n_chunks, int p_dtype, int m_dtype,
                       const fo_lion_consts* consts_host, void* stream);
int fo_lion_update_typed(void* p, const void* g, void* m, int64_t numel, int p_dtype, int m_dtype,
                         const fo_lion_consts* consts_host, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FASTOPS_H_ */
