/* C twin of oracle/mxopt_oracle.py -- TEST INFRASTRUCTURE ONLY.
 *
 * Two restatements of the reference's optimizer arithmetic on the CPU:
 *   *_unfused : the reference's own execution shape -- one full-array pass and one
 *               float32 temporary per MLX op, in the order the ops are issued at
 *               crates/mlx-core/src/optimizers/adamw.rs:84-116, adam.rs:79-108,
 *               sgd.rs:86-140, rmsprop.rs:69-93.  This is what the benchmark times
 *               as the CPU baseline.
 *   *_fused   : the same rounded operations in the same order, one pass.
 * Both give bit-identical results (every statement is one IEEE float32 op; build
 * with -ffp-contract=off and without -ffast-math).  Coefficients arrive already
 * cast to float32 by the caller, the way crates/mlx-sys/src/mlx.cpp:531-535 casts
 * every host scalar.  Tensors are float32, or bf16 bit patterns (dtype code 3,
 * crates/mlx-core/src/array/mod.rs:17-26) that are widened on load because MLX
 * promotes bf16 (op) float32-scalar to float32.
 *
 * Pinned by tests/test_oracle_c_twin.py: bit-exact agreement with the NumPy oracle,
 * which in turn is pinned by the reference's closed-form tests and torch.optim.
 * Nothing in the product links or loads this file.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define DT_F32 0
#define DT_BF16 3

static inline float bf16_to_f32(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static inline uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

static inline float ld(const void* a, int dt, size_t i) {
  return dt == DT_BF16 ? bf16_to_f32(((const uint16_t*)a)[i]) : ((const float*)a)[i];
}

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void oracle_f32_to_bf16(const float* x, uint16_t* out, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) out[i] = f32_to_bf16(x[i]);
}

void oracle_bf16_to_f32(const uint16_t* x, float* out, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) out[i] = bf16_to_f32(x[i]);
}

/* Host twin of the library's synthetic-data generator (defined at mxopt_fill_synthetic in include/mxopt.h). */
static inline uint64_t synth_hash(uint64_t seed, uint64_t idx) {
  uint64_t z = seed + (idx + 1ull) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

/* The quantile table of the Gaussian modes is the one the device code compiles. */
#include "mxopt_gauss_table.h"
static const float gauss_quantile[MXOPT_GAUSS_ROWS][MXOPT_GAUSS_COLS] = {MXOPT_GAUSS_TABLE};

static inline float synth_gauss_magnitude(uint32_t u) {
  if (u == 0u) u = 1u;
  const int k = __builtin_clz(u);
  const uint32_t v = u << k;
  const uint32_t j = (v >> 26) & 31u;
  const float f = (float)((v >> 10) & 0xffffu) * 0x1p-16f;
  const float t0 = gauss_quantile[k][j];
  const float d = gauss_quantile[k][j + 1] - t0;
  const float step = d * f;
  return t0 + step;
}

void oracle_fill_synthetic(void* out, int dtype, size_t n, uint64_t seed, uint64_t first_index, int dist, double a,
                           double b) {
  const int gauss = dist == 3 || dist == 4;
  const float fa = dist == 2 ? (float)((b - a) / 16777216.0)
                             : gauss ? (float)a : (float)(a / sqrt((65536.0 * 65536.0 - 1.0) / 3.0));
  const float fb = dist == 2 ? (float)a : (float)b;
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) {
    const uint64_t z = synth_hash(seed, first_index + i);
    float x;
    if (dist == 2) {
      x = (float)(uint32_t)(z >> 40) * fa;
      x = x + fb;
    } else if (gauss) {
      const float mag = synth_gauss_magnitude((uint32_t)(z >> 31));
      x = (z >> 63) ? -mag : mag;
      x = x * fa;
      if (dist == 4 && synth_hash(seed ^ 0xA5A5A5A5A5A5A5A5ull, first_index + i) % 100ull == 0ull) x = x * fb;
    } else {
      const int32_t sum = (int32_t)((z & 0xffffu) + ((z >> 16) & 0xffffu) + ((z >> 32) & 0xffffu) + (z >> 48)) - 131070;
      x = (float)sum * fa;
      if (dist == 1 && synth_hash(seed ^ 0xA5A5A5A5A5A5A5A5ull, first_index + i) % 100ull == 0ull) x = x * fb;
    }
    if (dtype == DT_BF16) ((uint16_t*)out)[i] = f32_to_bf16(x);
    else ((float*)out)[i] = x;
  }
}

/* Sum of squares in float64 (optimizers/mod.rs:43-55). */
double oracle_sumsq(const void* g, int dt, size_t n) {
  double s = 0.0;
#pragma omp parallel for schedule(static) reduction(+ : s)
  for (size_t i = 0; i < n; ++i) {
    double x = (double)ld(g, dt, i);
    s += x * x;
  }
  return s;
}

typedef struct {
  float lr, beta1, beta2, omb1, omb2, eps, decay, bc1, bc2;
  int decoupled_decay; /* 1: AdamW (adamw.rs:83-84), 0: Adam */
  int has_scale;       /* multiply g by `scale` first (clip_grad_norm, optimizers/mod.rs:98-102) */
  float scale;
  int bias_correction; /* unfused only: issue the two extra passes of adamw.rs:98-108 */
} oracle_adam_args;

/* One pass per MLX op, one temporary per op (13 for AdamW without bias correction). */
int oracle_adam_unfused(float* p_out, const void* p, int p_dt, const void* g, int g_dt, float* m,
                        float* v, size_t n, const oracle_adam_args* a) {
  float* t[8];
  for (int k = 0; k < 8; ++k) {
    t[k] = (float*)malloc(n * sizeof(float));
    if (!t[k]) {
      for (int j = 0; j < k; ++j) free(t[j]);
      return 1;
    }
  }
  float *gs = t[0], *pd = t[1], *b1m = t[2], *g1 = t[3], *gsq = t[4], *b2v = t[5], *g2 = t[6], *den = t[7];
  const oracle_adam_args c = *a;
#define PASS for (size_t i = 0; i < n; ++i)
#define G(i) (c.has_scale ? gs[i] : ld(g, g_dt, i))
  if (c.has_scale) {
#pragma omp parallel for schedule(static)
    PASS gs[i] = ld(g, g_dt, i) * c.scale;
  }
  if (c.decoupled_decay) {
#pragma omp parallel for schedule(static)
    PASS pd[i] = ld(p, p_dt, i) * c.decay;
  }
#pragma omp parallel for schedule(static)
  PASS b1m[i] = m[i] * c.beta1;
#pragma omp parallel for schedule(static)
  PASS g1[i] = G(i) * c.omb1;
#pragma omp parallel for schedule(static)
  PASS m[i] = b1m[i] + g1[i];
  /* mlx square keeps the operand's dtype (mlx.cpp:2016-2020): a bf16 gradient that was not scaled first
     gives a bf16 square (exact product, one rounding) */
  const int sq_bf16 = !c.has_scale && g_dt == DT_BF16;
#pragma omp parallel for schedule(static)
  PASS gsq[i] = sq_bf16 ? bf16_to_f32(f32_to_bf16(G(i) * G(i))) : G(i) * G(i);
#pragma omp parallel for schedule(static)
  PASS b2v[i] = v[i] * c.beta2;
#pragma omp parallel for schedule(static)
  PASS g2[i] = gsq[i] * c.omb2;
#pragma omp parallel for schedule(static)
  PASS v[i] = b2v[i] + g2[i];
  const float *mh = m, *vh = v;
  if (c.bias_correction) { /* two more passes (adamw.rs:98-108) */
#pragma omp parallel for schedule(static)
    PASS b1m[i] = m[i] * c.bc1;
#pragma omp parallel for schedule(static)
    PASS b2v[i] = v[i] * c.bc2;
    mh = b1m;
    vh = b2v;
  }
#pragma omp parallel for schedule(static)
  PASS gsq[i] = sqrtf(vh[i]);
#pragma omp parallel for schedule(static)
  PASS den[i] = gsq[i] + c.eps;
#pragma omp parallel for schedule(static)
  PASS g1[i] = mh[i] / den[i];
#pragma omp parallel for schedule(static)
  PASS g2[i] = g1[i] * c.lr;
#pragma omp parallel for schedule(static)
  PASS p_out[i] = (c.decoupled_decay ? pd[i] : ld(p, p_dt, i)) - g2[i];
#undef PASS
#undef G
  for (int k = 0; k < 8; ++k) free(t[k]);
  return 0;
}

void oracle_adam_fused(float* p_out, const void* p, int p_dt, const void* g, int g_dt, float* m,
                       float* v, size_t n, const oracle_adam_args* a) {
  const oracle_adam_args c = *a;
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) {
    float gi = ld(g, g_dt, i);
    if (c.has_scale) gi = gi * c.scale;
    float pi = ld(p, p_dt, i);
    float pd = c.decoupled_decay ? pi * c.decay : pi;
    float b1m = m[i] * c.beta1;
    float g1 = gi * c.omb1;
    float nm = b1m + g1;
    float gsq = gi * gi;
    if (!c.has_scale && g_dt == DT_BF16) gsq = bf16_to_f32(f32_to_bf16(gsq)); /* square of a bf16 tensor is bf16 */
    float b2v = v[i] * c.beta2;
    float g2 = gsq * c.omb2;
    float nv = b2v + g2;
    float mh = nm * c.bc1;
    float vh = nv * c.bc2;
    float den = sqrtf(vh) + c.eps;
    float u = mh / den;
    float lu = u * c.lr;
    m[i] = nm;
    v[i] = nv;
    p_out[i] = pd - lu;
  }
}

typedef struct {
  float lr, momentum, one_minus_damp, wd;
  int has_wd, has_momentum, nesterov, first; /* first: no velocity stored yet (sgd.rs:107-114) */
} oracle_sgd_args;

void oracle_sgd_fused(float* p_out, const float* p, const float* g, float* v, size_t n,
                      const oracle_sgd_args* a) {
  const oracle_sgd_args c = *a;
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) {
    float ge = g[i];
    if (c.has_wd) {
      float w = p[i] * c.wd;
      ge = g[i] + w;
    }
    float u = ge;
    if (c.has_momentum) {
      float nv;
      if (c.first) {
        nv = ge * 1.0f;
      } else {
        float mv = v[i] * c.momentum;
        float dg = ge * c.one_minus_damp;
        nv = mv + dg;
      }
      u = c.nesterov ? nv + ge : nv;
      v[i] = u;
    }
    float lu = u * c.lr;
    p_out[i] = p[i] - lu;
  }
}

/* sgd.rs:86-140 as issued: wd (2 passes), momentum (3 passes), lr*u, p-... */
int oracle_sgd_unfused(float* p_out, const float* p, const float* g, float* v, size_t n,
                       const oracle_sgd_args* a) {
  const oracle_sgd_args c = *a;
  float* t0 = (float*)malloc(n * sizeof(float));
  float* t1 = (float*)malloc(n * sizeof(float));
  float* t2 = (float*)malloc(n * sizeof(float));
  if (!t0 || !t1 || !t2) {
    free(t0); free(t1); free(t2);
    return 1;
  }
  const float* ge = g;
#define PASS for (size_t i = 0; i < n; ++i)
  if (c.has_wd) {
#pragma omp parallel for schedule(static)
    PASS t0[i] = p[i] * c.wd;
#pragma omp parallel for schedule(static)
    PASS t0[i] = g[i] + t0[i];
    ge = t0;
  }
  const float* u = ge;
  if (c.has_momentum) {
    if (c.first) {
#pragma omp parallel for schedule(static)
      PASS t1[i] = ge[i] * 1.0f;
    } else {
#pragma omp parallel for schedule(static)
      PASS t1[i] = v[i] * c.momentum;
#pragma omp parallel for schedule(static)
      PASS t2[i] = ge[i] * c.one_minus_damp;
#pragma omp parallel for schedule(static)
      PASS t1[i] = t1[i] + t2[i];
    }
    if (c.nesterov) {
#pragma omp parallel for schedule(static)
      PASS t1[i] = t1[i] + ge[i];
    }
#pragma omp parallel for schedule(static)
    PASS v[i] = t1[i];
    u = t1;
  }
#pragma omp parallel for schedule(static)
  PASS t2[i] = u[i] * c.lr;
#pragma omp parallel for schedule(static)
  PASS p_out[i] = p[i] - t2[i];
#undef PASS
  free(t0); free(t1); free(t2);
  return 0;
}

typedef struct {
  float lr, alpha, one_minus_alpha, eps, wd;
  int has_wd;
} oracle_rmsprop_args;

void oracle_rmsprop_fused(float* p_out, const float* p, const float* g, float* v, size_t n,
                          const oracle_rmsprop_args* a) {
  const oracle_rmsprop_args c = *a;
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) {
    float ge = g[i];
    if (c.has_wd) {
      float w = p[i] * c.wd;
      ge = g[i] + w;
    }
    float gsq = ge * ge;
    float av = v[i] * c.alpha;
    float g2 = gsq * c.one_minus_alpha;
    float nv = av + g2;
    float den = sqrtf(nv) + c.eps;
    float u = ge / den;
    float lu = u * c.lr;
    v[i] = nv;
    p_out[i] = p[i] - lu;
  }
}

int oracle_rmsprop_unfused(float* p_out, const float* p, const float* g, float* v, size_t n,
                           const oracle_rmsprop_args* a) {
  const oracle_rmsprop_args c = *a;
  float* t0 = (float*)malloc(n * sizeof(float));
  float* t1 = (float*)malloc(n * sizeof(float));
  float* t2 = (float*)malloc(n * sizeof(float));
  if (!t0 || !t1 || !t2) {
    free(t0); free(t1); free(t2);
    return 1;
  }
  const float* ge = g;
#define PASS for (size_t i = 0; i < n; ++i)
  if (c.has_wd) {
#pragma omp parallel for schedule(static)
    PASS t0[i] = p[i] * c.wd;
#pragma omp parallel for schedule(static)
    PASS t0[i] = g[i] + t0[i];
    ge = t0;
  }
#pragma omp parallel for schedule(static)
  PASS t1[i] = ge[i] * ge[i];
#pragma omp parallel for schedule(static)
  PASS t2[i] = v[i] * c.alpha;
#pragma omp parallel for schedule(static)
  PASS t1[i] = t1[i] * c.one_minus_alpha;
#pragma omp parallel for schedule(static)
  PASS v[i] = t2[i] + t1[i];
#pragma omp parallel for schedule(static)
  PASS t1[i] = sqrtf(v[i]);
#pragma omp parallel for schedule(static)
  PASS t1[i] = t1[i] + c.eps;
#pragma omp parallel for schedule(static)
  PASS t2[i] = ge[i] / t1[i];
#pragma omp parallel for schedule(static)
  PASS t2[i] = t2[i] * c.lr;
#pragma omp parallel for schedule(static)
  PASS p_out[i] = p[i] - t2[i];
#undef PASS
  free(t0); free(t1); free(t2);
  return 0;
}

/* acc(float32) += widen(g); first: acc = widen(g).  One float32 add per element. */
void oracle_accumulate_f32(float* acc, const void* g, int g_dt, size_t n, int first) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) {
    float gi = ld(g, g_dt, i);
    acc[i] = first ? gi : acc[i] + gi;
  }
}

/* In-place scale pass of clip_grad_norm (optimizers/mod.rs:98-102). */
void oracle_scale_f32(float* out, const void* g, int g_dt, size_t n, float scale) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) out[i] = ld(g, g_dt, i) * scale;
}
