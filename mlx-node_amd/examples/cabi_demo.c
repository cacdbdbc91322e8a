/* A plain-C host of libmxopt.so: what a cgo / Rust / N-API binding does, without any Python.
 *
 *   cabi_demo            known-answer checks through the optimizer objects (the reference's own
 *                        closed forms: __test__/core/optimizers.test.ts:151-203, 324-351) and the
 *                        engine entry points (with and without an accumulation buffer), then a timing of updateSingle-per-tensor against
 *                        one update_many call over the Qwen3-0.6B parameter list; before that the
 *                        region-interleaved pool (moments taken from it, the bare probes on its memory and on
 *                        plain memory), the global norm that allocates nothing, and the GRPO engine's call
 *                        that does not wait for the validity flag.
 * Prints "PASS" lines and one "TIMING" line; exits non-zero on the first mismatch.
 */
#define _POSIX_C_SOURCE 200809L
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "mxopt_engine.h"
#include "mxopt_diagnostics.h"   /* the bare probes */

#define CHECK_HIP(call)                                                                  \
  do {                                                                                   \
    hipError_t e_ = (call);                                                              \
    if (e_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_)); exit(2); } \
  } while (0)
#define CHECK_MX(call)                                                                   \
  do {                                                                                   \
    int rc_ = (call);                                                                    \
    if (rc_ != MXOPT_OK) { fprintf(stderr, "%s -> %d: %s\n", #call, rc_, mxopt_last_error(ctx)); exit(3); } \
  } while (0)

static mxopt_ctx* ctx;

static float* to_device(const float* host, size_t n) {
  float* d = NULL;
  CHECK_HIP(hipMalloc((void**)&d, (n ? n : 1) * sizeof(float)));
  if (n) CHECK_HIP(hipMemcpy(d, host, n * sizeof(float), hipMemcpyHostToDevice));
  return d;
}

static void expect_close(const char* what, const float* d, const double* want, size_t n, double tol) {
  float host[16];
  CHECK_MX(mxopt_synchronize(ctx));
  CHECK_HIP(hipMemcpy(host, d, n * sizeof(float), hipMemcpyDeviceToHost));
  for (size_t i = 0; i < n; ++i) {
    if (!(fabs((double)host[i] - want[i]) <= tol)) {
      fprintf(stderr, "FAIL %s[%zu]: got %.9g want %.9g\n", what, i, host[i], want[i]);
      exit(1);
    }
  }
  printf("PASS %s\n", what);
}

static double now_ms(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return ts.tv_sec * 1e3 + ts.tv_nsec * 1e-6;
}

static void known_answers(void) {
  /* SGD, lr 0.1: [1,2,3] - 0.1*[0.1,0.2,0.3]  (optimizers.test.ts:151-164) */
  const float p0[3] = {1.0f, 2.0f, 3.0f}, g0[3] = {0.1f, 0.2f, 0.3f};
  float *p = to_device(p0, 3), *g = to_device(g0, 3), *out = to_device(p0, 3);
  mxopt_optimizer* sgd = NULL;
  CHECK_MX(mxopt_sgd_new(ctx, 0.1, NULL, NULL, NULL, NULL, &sgd));
  mxopt_array ap = {p, 3, MXOPT_F32}, ag = {g, 3, MXOPT_F32}, ao = {out, 3, MXOPT_F32};
  CHECK_MX(mxopt_optimizer_update_single(sgd, "param", &ap, &ag, &ao));
  const double want_sgd[3] = {0.99, 1.98, 2.97};
  expect_close("SGD basic step", out, want_sgd, 3, 5e-6);
  mxopt_optimizer_free(sgd);

  /* Nesterov without momentum is refused with InvalidArg (optimizers.test.ts:205-214) */
  const int yes = 1;
  const double zero = 0.0;
  if (mxopt_sgd_new(ctx, 0.1, &zero, NULL, NULL, &yes, &sgd) != MXOPT_ERR_INVALID_ARG) {
    fprintf(stderr, "FAIL: invalid Nesterov configuration was accepted\n");
    exit(1);
  }
  printf("PASS SGD rejects Nesterov without momentum: %s\n", mxopt_last_error(ctx));

  /* clip_grad_norm: [3,4] has norm 5, max 2.5 halves it (optimizers.test.ts:324-351) */
  const float g1[2] = {3.0f, 4.0f};
  float *dg = to_device(g1, 2), *dc = to_device(g1, 2);
  mxopt_array cg = {dg, 2, MXOPT_F32}, co = {dc, 2, MXOPT_F32};
  double norm = 0.0;
  CHECK_MX(mxopt_clip_grad_norm(ctx, 1, &cg, 2.5, &co, &norm));
  const double want_clip[2] = {1.5, 2.0};
  expect_close("clip_grad_norm halves [3,4]", dc, want_clip, 2, 5e-6);
  if (fabs(norm - 5.0) > 1e-5) { fprintf(stderr, "FAIL norm %.9g\n", norm); exit(1); }

  /* GRPO engine, N = 4, lr 0.01, clips off: [10,20] - 0.0025*[10,14]
   * (__test__/trainers/grpo-gradient-accumulation.test.ts:134-171) */
  const float w0[2] = {10.0f, 20.0f};
  const float gs[4][2] = {{1, 2}, {2, 3}, {3, 4}, {4, 5}};
  float* w = to_device(w0, 2);
  mxopt_engine_config cfg;
  mxopt_engine_config_default(MXOPT_ENGINE_GRPO, &cfg);
  cfg.learning_rate = 0.01;
  cfg.gradient_accumulation_steps = 4;
  cfg.has_gradient_clip_norm = 0;
  cfg.gradient_clip_value = 100.0;
  const char* names[1] = {"w"};
  mxopt_array aw = {w, 2, MXOPT_F32};
  mxopt_engine* eng = NULL;
  CHECK_MX(mxopt_engine_new(ctx, &cfg, 1, names, &aw, &eng));
  mxopt_engine_metrics m;
  for (int k = 0; k < 4; ++k) {
    float* d = to_device(gs[k], 2);
    mxopt_array a = {d, 2, MXOPT_F32};
    CHECK_MX(mxopt_engine_micro_batch(eng, 1, names, &a, &m));
    if (m.gradients_applied != (k == 3) || m.step != k + 1) { fprintf(stderr, "FAIL engine bookkeeping at %d\n", k); exit(1); }
    CHECK_MX(mxopt_synchronize(ctx));
    CHECK_HIP(hipFree(d));
  }
  const double want_w[2] = {9.975, 19.965};
  expect_close("GRPO engine: 4 micro-batches, lr/N", w, want_w, 2, 5e-6);
  mxopt_engine_free(eng);

  /* The same known answer with no accumulation buffer: the engine only remembers where the four
   * micro-batches lie (the host keeps them alive) and the last call adds them in registers.  The
   * parameter and the gradients are allocated inside a placement window, as a host would at start-up. */
  mxopt_hbm_spread* window = NULL;
  CHECK_MX(mxopt_hbm_spread_begin(ctx, (size_t)512 << 20, 2, &window));
  float* w2 = to_device(w0, 2);
  float* held[4];
  for (int k = 0; k < 4; ++k) held[k] = to_device(gs[k], 2);
  CHECK_MX(mxopt_hbm_spread_end(window));
  cfg.defer_accumulation = 1;
  mxopt_array aw2 = {w2, 2, MXOPT_F32};
  CHECK_MX(mxopt_engine_new(ctx, &cfg, 1, names, &aw2, &eng));
  for (int k = 0; k < 4; ++k) {
    mxopt_array a = {held[k], 2, MXOPT_F32};
    CHECK_MX(mxopt_engine_micro_batch(eng, 1, names, &a, &m));
    if (m.gradients_applied != (k == 3) || m.step != k + 1) { fprintf(stderr, "FAIL deferred engine bookkeeping at %d\n", k); exit(1); }
  }
  expect_close("GRPO engine, deferred accumulation: same answer", w2, want_w, 2, 5e-6);
  mxopt_engine_free(eng);
  for (int k = 0; k < 4; ++k) CHECK_HIP(hipFree(held[k]));
}

/* Twelve micro-batches per step through the SFT engine (clip by global norm, decay), once with its
 * float32 accumulation buffer and once deferred -- more than the kernels have streams for, so the
 * oldest are added into a buffer as later ones arrive.  The parameters must come out bit-identical. */
static void long_cycle(void) {
  enum { N = 5003, MICRO = 12, CYCLES = 2 };
  static float host[N], a_out[N], b_out[N];
  for (int i = 0; i < N; ++i) host[i] = (float)((i * 37) % 201 - 100) * 1e-3f;
  float* w[2] = {to_device(host, N), to_device(host, N)};
  float* g[MICRO];
  mxopt_engine* eng[2] = {NULL, NULL};
  const char* names[1] = {"w"};
  for (int e = 0; e < 2; ++e) {
    mxopt_engine_config cfg;
    mxopt_engine_config_default(MXOPT_ENGINE_SFT, &cfg);
    cfg.learning_rate = 0.02;
    cfg.gradient_accumulation_steps = MICRO;
    cfg.has_gradient_clip_norm = 1;
    cfg.gradient_clip_norm = 0.5;
    cfg.weight_decay = 0.01;
    cfg.accumulate_in_f32 = 1;
    cfg.defer_accumulation = e;
    mxopt_array aw = {w[e], N, MXOPT_F32};
    CHECK_MX(mxopt_engine_new(ctx, &cfg, 1, names, &aw, &eng[e]));
  }
  for (int c = 0; c < CYCLES; ++c) {
    for (int k = 0; k < MICRO; ++k) {
      for (int i = 0; i < N; ++i)
        host[i] = (float)((int)(((unsigned)i * 2654435761u + (unsigned)(c * MICRO + k) * 40503u) % 2001u) - 1000) * 1e-4f;
      g[k] = to_device(host, N);
      for (int e = 0; e < 2; ++e) {
        mxopt_array a = {g[k], N, MXOPT_F32};
        mxopt_engine_metrics m;
        CHECK_MX(mxopt_engine_micro_batch(eng[e], 1, names, &a, &m));
        if (m.gradients_applied != (k == MICRO - 1)) { fprintf(stderr, "FAIL long cycle bookkeeping at %d\n", k); exit(1); }
      }
    }
    CHECK_MX(mxopt_synchronize(ctx));
    for (int k = 0; k < MICRO; ++k) CHECK_HIP(hipFree(g[k]));  /* the deferred engine needed them until here */
  }
  CHECK_HIP(hipMemcpy(a_out, w[0], sizeof a_out, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(b_out, w[1], sizeof b_out, hipMemcpyDeviceToHost));
  if (memcmp(a_out, b_out, sizeof a_out) != 0 || a_out[1] == (float)((37 % 201) - 100) * 1e-3f) {
    fprintf(stderr, "FAIL deferred and buffered SFT engines differ after %d micro-batches\n", MICRO);
    exit(1);
  }
  printf("PASS SFT engine, %d micro-batches per step: deferred accumulation bit-identical to the float32 buffer\n", MICRO);
  for (int e = 0; e < 2; ++e) {
    mxopt_engine_free(eng[e]);
    CHECK_HIP(hipFree(w[e]));
  }
}

/* The start-up utilities and the two entry points for hosts with constraints: a pool whose memory alternates
 * between the device's physical regions, optimizer state taken from it, the probes that show what that is
 * worth, mxopt_global_norm_static against mxopt_global_norm, and the asynchronous GRPO micro-batch call with a
 * NaN micro-batch in the middle of a cycle. */
static double probe_gbps(int kind, void* a, void* b, void* c, void* d, uint64_t n, double streams) {
  CHECK_MX(mxopt_probe_stream(ctx, kind, a, b, c, d, n));
  CHECK_MX(mxopt_synchronize(ctx));
  const double t0 = now_ms();
  for (int i = 0; i < 10; ++i) CHECK_MX(mxopt_probe_stream(ctx, kind, a, b, c, d, n));
  CHECK_MX(mxopt_synchronize(ctx));
  return streams * (double)n * 4.0 / 1e9 / ((now_ms() - t0) / 10.0 * 1e-3);
}

static void pool_and_friends(void) {
  const uint64_t n = (uint64_t)1 << 28;  /* 1 GiB per stream */
  void* plain[4];
  for (int i = 0; i < 4; ++i) CHECK_HIP(hipMalloc(&plain[i], n * 4));
  const double plain_mix = probe_gbps(MXOPT_PROBE_MIX43, plain[0], plain[1], plain[2], plain[3], n, 7.0);
  for (int i = 0; i < 4; ++i) CHECK_HIP(hipFree(plain[i]));

  mxopt_hbm_pool* pool = NULL;
  CHECK_MX(mxopt_hbm_pool_create(ctx, (size_t)6 << 30, 0, 2, &pool));
  mxopt_hbm_pool_info info;
  CHECK_MX(mxopt_hbm_pool_get_info(pool, &info));
  void* arena[4];
  for (int i = 0; i < 4; ++i) CHECK_MX(mxopt_hbm_pool_alloc(pool, n * 4, &arena[i]));
  const double arena_mix = probe_gbps(MXOPT_PROBE_MIX43, arena[0], arena[1], arena[2], arena[3], n, 7.0);
  printf("POOL regions=%d chunk_mib=%llu setup_s=%.2f (create %.2f, scan %.2f) probes=%d same_region_gbps=%.0f cross_region_gbps=%.0f "
         "mix43_plain_gbps=%.0f mix43_arena_gbps=%.0f\n", info.regions, (unsigned long long)(info.chunk_bytes >> 20),
         info.setup_seconds, info.create_seconds, info.scan_seconds, info.probes, info.probe_same_region_gbps, info.probe_cross_region_gbps, plain_mix, arena_mix);
  for (int i = 0; i < 4; ++i) {
    if (!mxopt_hbm_pool_owns(pool, arena[i])) { fprintf(stderr, "FAIL pool does not own its allocation\n"); exit(1); }
    CHECK_MX(mxopt_hbm_pool_free(pool, arena[i]));
  }

  /* moments from the pool: AdamW, lr 0.1, zero state, no decay -> first step moves every weight by lr * g / (|g| + eps) ... */
  CHECK_MX(mxopt_set_state_pool(ctx, pool));
  const float p0[3] = {1.0f, 2.0f, 3.0f}, g0[3] = {0.5f, -0.25f, 0.125f};
  float *dp = to_device(p0, 3), *dg = to_device(g0, 3), *m = NULL, *v = NULL;
  const mxopt_array ap = {dp, 3, MXOPT_F32}, ag = {dg, 3, MXOPT_F32};
  const double lr = 0.1, wd = 0.0, b1 = 0.9, b2 = 0.999, eps = 1e-8;
  const int bias = 1;
  mxopt_optimizer* opt = NULL;
  CHECK_MX(mxopt_adamw_new(ctx, &lr, &b1, &b2, &eps, &wd, &bias, &opt));
  CHECK_MX(mxopt_optimizer_update_single(opt, "w", &ap, &ag, &ap));
  uint64_t cnt = 0;
  int hv = 0;
  CHECK_MX(mxopt_optimizer_state(opt, "w", &m, &v, &cnt, &hv));
  if (!mxopt_hbm_pool_owns(pool, m) || !mxopt_hbm_pool_owns(pool, v)) { fprintf(stderr, "FAIL moments are not in the pool\n"); exit(1); }
  /* ... with bias correction m_hat = g, v_hat = g^2: p - lr * sign(g) up to eps */
  const double want[3] = {1.0 - 0.1, 2.0 + 0.1, 3.0 - 0.1};
  expect_close("AdamW with its moments in the region-interleaved pool", dp, want, 3, 1e-6);
  mxopt_optimizer_free(opt);
  CHECK_MX(mxopt_set_state_pool(ctx, NULL));

  /* the norm that allocates nothing against the one that sizes a buffer on first use: same bits */
  enum { NN = 100003 };
  float* hg = malloc(NN * sizeof *hg);
  for (int i = 0; i < NN; ++i) hg[i] = (float)((i * 2654435761u) % 2001u) * 1e-3f - 1.0f;
  float* dgn = to_device(hg, NN);
  mxopt_tensor row;
  memset(&row, 0, sizeof row);
  row.g = dgn; row.n = NN; row.g_dtype = MXOPT_F32; row.bc1 = row.bc2 = 1.0f;
  mxopt_table* t = NULL;
  CHECK_MX(mxopt_table_build(ctx, &row, 1, &t));
  mxopt_norm_result *d_res = NULL, a, b;
  CHECK_HIP(hipMalloc((void**)&d_res, 2 * sizeof *d_res));
  CHECK_MX(mxopt_global_norm_static(ctx, t, 0, NULL, 1.0, MXOPT_CLIP_ALWAYS_MULTIPLY, &d_res[0]));
  CHECK_MX(mxopt_global_norm(ctx, t, 0, NULL, 1.0, MXOPT_CLIP_ALWAYS_MULTIPLY, &d_res[1]));
  CHECK_MX(mxopt_read_norm_result(ctx, &d_res[0], &a));
  CHECK_MX(mxopt_read_norm_result(ctx, &d_res[1], &b));
  double exact = 0.0;
  for (int i = 0; i < NN; ++i) exact += (double)hg[i] * hg[i];
  if (memcmp(&a, &b, sizeof a) != 0 || fabs(a.sumsq - exact) > 1e-6 * exact) {
    fprintf(stderr, "FAIL static norm %.17g, allocating norm %.17g, exact %.17g\n", a.sumsq, b.sumsq, exact);
    exit(1);
  }
  printf("PASS mxopt_global_norm_static: bit-identical to mxopt_global_norm, sum of squares %.9g\n", a.sumsq);
  mxopt_table_destroy(t);
  CHECK_HIP(hipFree(d_res));
  CHECK_HIP(hipFree(dgn));
  free(hg);

  /* GRPO engine, two micro-batches per step, lr 0.5, no clamp or clip in reach: good, NaN (skipped), good
   * -> p = 1 - 0.5/2 * (0.25 + 0.25) after the third call, the NaN call counted, nothing waited for */
  mxopt_engine_config cfg;
  mxopt_engine_config_default(MXOPT_ENGINE_GRPO, &cfg);
  cfg.gradient_accumulation_steps = 2;
  cfg.learning_rate = 0.5;
  cfg.gradient_clip_norm = 1e9;
  const float one[4] = {1.0f, 1.0f, 1.0f, 1.0f}, good[4] = {0.25f, 0.25f, 0.25f, 0.25f};
  float bad[4] = {0.25f, 0.25f, 0.25f, 0.25f};
  bad[2] = NAN;
  float *w = to_device(one, 4), *dgood = to_device(good, 4), *dbad = to_device(bad, 4);
  const char* names[1] = {"w"};
  const mxopt_array aw = {w, 4, MXOPT_F32}, agood = {dgood, 4, MXOPT_F32}, abad = {dbad, 4, MXOPT_F32};
  mxopt_engine* eng = NULL;
  CHECK_MX(mxopt_engine_new(ctx, &cfg, 1, names, &aw, &eng));
  CHECK_MX(mxopt_engine_micro_batch_async(eng, 1, names, &agood));
  CHECK_MX(mxopt_engine_micro_batch_async(eng, 1, names, &abad));
  CHECK_MX(mxopt_engine_micro_batch_async(eng, 1, names, &agood));
  mxopt_engine_metrics em;
  CHECK_MX(mxopt_engine_settle(eng, &em));
  if (em.step != 3 || em.nan_gradient_count != 1 || em.micro_step != 0 || !em.gradients_applied) {
    fprintf(stderr, "FAIL async engine bookkeeping: step %lld nan %llu micro %d applied %d\n", (long long)em.step,
            (unsigned long long)em.nan_gradient_count, em.micro_step, em.gradients_applied);
    exit(1);
  }
  const double want_w[4] = {0.875, 0.875, 0.875, 0.875};
  expect_close("GRPO engine, asynchronous micro-batches with a NaN one in the middle of the cycle", w, want_w, 4, 0.0);
  mxopt_engine_free(eng);
  CHECK_HIP(hipFree(w)); CHECK_HIP(hipFree(dgood)); CHECK_HIP(hipFree(dbad));
  CHECK_HIP(hipFree(dp)); CHECK_HIP(hipFree(dg));
  CHECK_MX(mxopt_hbm_pool_destroy(pool));
}

/* Qwen3-0.6B: vocab 151936, hidden 1024, 28 layers, q 2048x1024, k/v 1024x1024, o 1024x2048,
 * gate/up 3072x1024, down 1024x3072, four norm vectors per layer, final norm, tied embedding. */
static size_t qwen3_06b(size_t* sizes) {
  size_t n = 0;
  sizes[n++] = (size_t)151936 * 1024;
  for (int l = 0; l < 28; ++l) {
    sizes[n++] = 2048 * 1024; sizes[n++] = 1024 * 1024; sizes[n++] = 1024 * 1024; sizes[n++] = 1024 * 2048;
    sizes[n++] = 3072 * 1024; sizes[n++] = 3072 * 1024; sizes[n++] = 1024 * 3072;
    sizes[n++] = 1024; sizes[n++] = 1024; sizes[n++] = 128; sizes[n++] = 128;
  }
  sizes[n++] = 1024;
  return n;
}

static void timing(void) {
  size_t sizes[512];
  const size_t nt = qwen3_06b(sizes);
  size_t total = 0;
  mxopt_array *p = calloc(nt, sizeof *p), *g = calloc(nt, sizeof *g);
  char (*names)[32] = calloc(nt, 32);
  const char** name_ptrs = calloc(nt, sizeof *name_ptrs);
  for (size_t i = 0; i < nt; ++i) {
    void *dp, *dg;
    CHECK_HIP(hipMalloc(&dp, sizes[i] * 4));
    CHECK_HIP(hipMalloc(&dg, sizes[i] * 4));
    CHECK_HIP(hipMemset(dp, 0, sizes[i] * 4));
    CHECK_HIP(hipMemset(dg, 0, sizes[i] * 4));
    p[i] = (mxopt_array){dp, sizes[i], MXOPT_F32};
    g[i] = (mxopt_array){dg, sizes[i], MXOPT_F32};
    snprintf(names[i], 32, "t%zu", i);
    name_ptrs[i] = names[i];
    total += sizes[i];
  }
  mxopt_optimizer* opt = NULL;
  CHECK_MX(mxopt_adamw_new(ctx, NULL, NULL, NULL, NULL, NULL, NULL, &opt));
  const int steps = 20;
  double wall[2], host[2];
  for (int mode = 0; mode < 2; ++mode) {
    double t0 = 0;
    for (int it = -3; it < steps; ++it) {
      if (it == 0) {
        CHECK_MX(mxopt_synchronize(ctx));
        t0 = now_ms();
      }
      if (mode == 0) {
        for (size_t i = 0; i < nt; ++i) CHECK_MX(mxopt_optimizer_update_single(opt, names[i], &p[i], &g[i], &p[i]));
      } else {
        CHECK_MX(mxopt_optimizer_update_many(opt, nt, name_ptrs, p, g, p, NULL));
      }
    }
    host[mode] = (now_ms() - t0) / steps;   /* time to enqueue */
    CHECK_MX(mxopt_synchronize(ctx));
    wall[mode] = (now_ms() - t0) / steps;   /* until the device has finished */
  }
  const double t_single = wall[0], t_many = wall[1], host_single = host[0] * steps, host_many = host[1] * steps;
  printf("TIMING tensors=%zu elements=%zu update_single_loop_ms=%.3f (host enqueue %.3f) update_many_ms=%.3f "
         "(host enqueue %.3f) bytes_per_step=%zu\n", nt, total, t_single, host_single / steps, t_many,
         host_many / steps, total * 28);
  mxopt_optimizer_free(opt);
}

int main(int argc, char** argv) {
  CHECK_MX(mxopt_create(0, NULL, &ctx));
  printf("%s\n", mxopt_version());
  known_answers();
  long_cycle();
  pool_and_friends();
  if (argc < 2 || strcmp(argv[1], "--no-timing") != 0) timing();
  mxopt_destroy(ctx);
  return 0;
}
