/* CPU oracle for the fused Lion step -- TEST INFRASTRUCTURE ONLY, never linked into the product library.
 *
 * Scalar restatement of fast_ops/lion/lion_optimizer_ref.py:51,64,65,67 for fp32 parameters and gradients with a
 * bf16 momentum, with every rounding point explicit (see oracle/lion_oracle.py for the derivation and for the tests
 * that pin it against the torch ops the reference calls). Build: `make -C oracle` (gcc -O2 -ffp-contract=off, so the
 * only fused multiply-add is the explicit fmaf of statement :67).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>
#include <pthread.h>

static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* fp32 -> bf16 bits, round to nearest even, NaN -> 0x7FC0 (what c10::BFloat16's constructor does) */
static inline uint16_t bf16_rne(float f) {
  if (f != f) return 0x7FC0;
  uint32_t u = f32_bits(f);
  uint32_t bias = ((u >> 16) & 1u) + 0x7FFFu;
  return (uint16_t)((u + bias) >> 16);
}
static inline float bf16_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }

void lion_oracle_step(float* p, const float* g, uint16_t* m, int64_t n,
                      float c_wd, float c_b1, float c_1b1, float c_nlr, float c_b2, float c_1b2) {
  for (int64_t i = 0; i < n; ++i) {
    const float mf = bf16_f32(m[i]);
    const float gi = g[i];
    const float p1 = p[i] * c_wd;                          /* :51 */
    const float t1 = bf16_f32(bf16_rne(mf * c_b1));        /* :64 exp_avg * beta1 -> bf16 tensor */
    const float t2 = gi * c_1b1;                           /* :64 */
    const float u = t1 + t2;                               /* :64 */
    const float s = (float)((u > 0.0f) - (u < 0.0f));      /* :65 torch.sign: 0 for zero and NaN */
    p[i] = p1 + c_nlr * s;                                 /* :65 product exact, one rounding */
    const float m1 = bf16_f32(bf16_rne(mf * c_b2));        /* :67 mul_ rounds to bf16 */
    m[i] = bf16_rne(fmaf(c_1b2, gi, m1));                  /* :67 add_(grad, alpha) is fused */
  }
}

typedef struct { float* p; const float* g; uint16_t* m; int64_t n; float c[6]; } job_t;
static void* worker(void* a) {
  job_t* j = (job_t*)a;
  lion_oracle_step(j->p, j->g, j->m, j->n, j->c[0], j->c[1], j->c[2], j->c[3], j->c[4], j->c[5]);
  return 0;
}

/* same step split over `threads` contiguous slices (elementwise, so the split cannot change a result) */
void lion_oracle_step_mt(float* p, const float* g, uint16_t* m, int64_t n,
                         float c_wd, float c_b1, float c_1b1, float c_nlr, float c_b2, float c_1b2, int threads) {
  if (threads < 1) threads = 1;
  if (threads > 256) threads = 256;
  pthread_t tid[256];
  job_t jobs[256];
  int64_t per = (n + threads - 1) / threads;
  int started = 0;
  for (int t = 0; t < threads; ++t) {
    int64_t lo = (int64_t)t * per, hi = lo + per > n ? n : lo + per;
    if (lo >= hi) break;
    jobs[t] = (job_t){p + lo, g + lo, m + lo, hi - lo, {c_wd, c_b1, c_1b1, c_nlr, c_b2, c_1b2}};
    pthread_create(&tid[t], 0, worker, &jobs[t]);
    started++;
  }
  for (int t = 0; t < started; ++t) pthread_join(tid[t], 0);
}
