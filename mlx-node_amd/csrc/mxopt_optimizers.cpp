// Host layer of mxopt: the reference's optimizer objects and gradient utilities over raw
// device buffers.  Declarations, and the reference methods each entry point stands behind,
// are in include/mxopt_optimizers.h.  All arithmetic happens in the kernels (the *_kernels.hip files).
#include "mxopt_optimizers.h"

#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstring>
#include <new>
#include <string>
#include <unordered_map>
#include <vector>

#include "mxopt_checkpoint_internal.h"
#include "mxopt_internal.h"

namespace mxopt {

struct StateEntry {
  float* m = nullptr;  // first moment (Adam/AdamW)
  float* v = nullptr;  // second moment, or SGD velocity
  uint64_t n = 0;
  bool has_velocity = false;  // SGD: velocity written at least once (sgd.rs:98-114)
  float* sum = nullptr;       // update_many_accumulated with more micro-batches than streams: the oldest, added up
};

enum class Kind { Adam, AdamW, Sgd, Rmsprop };

mxopt_tensor blank_tensor() {
  mxopt_tensor t;
  std::memset(&t, 0, sizeof t);
  t.bc1 = t.bc2 = 1.0f;
  return t;
}

int check_array(mxopt_ctx* ctx, const mxopt_array* a, const char* what, bool allow_null_data) {
  if (!a) return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(what) + " is NULL");
  if (!float_dtype(a->dtype)) return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(what) + ": unsupported dtype code");
  if (!a->data && a->n && !allow_null_data)
    return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(what) + ": null handle");  // array/handle.rs:4-16
  return MXOPT_OK;
}

// Finds or builds the table for `rows` (compared bytewise, per-step scalars excluded).
int cached_table(mxopt_ctx* ctx, std::vector<mxopt_tensor>& rows, mxopt_table** out) {
  std::vector<mxopt_tensor> key = rows;
  for (auto& r : key) { r.bc1 = r.bc2 = 1.0f; r.flags = 0; }
  auto& cache = ctx->table_cache;
  for (size_t i = 0; i < cache.size(); ++i) {
    if (cache[i].key.size() == key.size() &&
        (key.empty() || std::memcmp(cache[i].key.data(), key.data(), key.size() * sizeof(mxopt_tensor)) == 0)) {
      mxopt_ctx::CachedTable hit = std::move(cache[i]);
      cache.erase(cache.begin() + i);
      cache.push_back(std::move(hit));
      *out = cache.back().table;
      return MXOPT_OK;
    }
  }
  // Same layout, other buffers (the caller's arrays moved): keep the chunk list, swap the pointers.
  // The least recently used candidate goes first so that alternating buffer sets each keep a table.
  for (size_t i = 0; i < cache.size(); ++i) {
    if (cache[i].key.size() != key.size() || key.empty()) continue;
    std::string why;  // a layout mismatch here is not the caller's error: try the next candidate
    if (const int rc = table_retarget_quiet(cache[i].table, rows.data(), rows.size(), &why)) {
      if (why.empty()) return rc;  // the descriptor upload failed and has said so
      continue;
    }
    mxopt_ctx::CachedTable hit = std::move(cache[i]);
    hit.key = std::move(key);
    cache.erase(cache.begin() + i);
    cache.push_back(std::move(hit));
    *out = cache.back().table;
    return MXOPT_OK;
  }
  mxopt_table* t = nullptr;
  int rc = mxopt_table_build(ctx, rows.data(), rows.size(), &t);
  if (rc) return rc;
  constexpr size_t kMaxCached = 16;  // two engines and the gradient utilities fit side by side
  if (cache.size() >= kMaxCached) {
    mxopt_table_destroy(cache.front().table);
    cache.erase(cache.begin());
  }
  cache.push_back({std::move(key), t});
  *out = t;
  return MXOPT_OK;
}

int norm_scratch(mxopt_ctx* ctx, mxopt_norm_result** out) {
  if (!ctx->d_norm_scratch) {
    DeviceGuard guard(ctx->device);
    HIP_TRY(ctx, hipMalloc((void**)&ctx->d_norm_scratch, sizeof(mxopt_norm_result)));
  }
  *out = ctx->d_norm_scratch;
  return MXOPT_OK;
}

}  // namespace mxopt

using namespace mxopt;

struct mxopt_optimizer {
  Kind kind;
  mxopt_ctx* ctx = nullptr;
  double lr = 0, beta1 = 0.9, beta2 = 0.999, eps = 1e-8, weight_decay = 0, momentum = 0, dampening = 0, alpha = 0.99;
  bool bias_correction = false, nesterov = false;
  int64_t step = 0;  // counts update_single CALLS (adam.rs:73, adamw.rs:77)
  std::unordered_map<std::string, StateEntry> state;
  // update_many keeps its table while the same buffers come back
  std::vector<mxopt_tensor> many_key;
  mxopt_table* many_table = nullptr;
};

void mxopt::optimizer_set_step_count(mxopt_optimizer* opt, int64_t calls) { opt->step = calls; }

namespace {

bool is_adam(const mxopt_optimizer* o) { return o->kind == Kind::Adam || o->kind == Kind::AdamW; }

void free_state(mxopt_optimizer* o) {
  if (o->state.empty() && !o->many_table) return;
  DeviceGuard guard(o->ctx->device);
  (void)hipStreamSynchronize(o->ctx->stream);  // kernels may still be using the buffers
  if (o->many_table) {
    mxopt_table_destroy(o->many_table);
    o->many_table = nullptr;
    o->many_key.clear();
  }
  for (auto& kv : o->state) {
    state_free(o->ctx, kv.second.m);
    state_free(o->ctx, kv.second.v);
    state_free(o->ctx, kv.second.sum);
  }
  o->state.clear();
}

// init_state (adam.rs:148-153, adamw.rs:152-157, rmsprop.rs:123-127): float32 zeros of the
// parameter's shape; SGD starts with no velocity (sgd.rs:80-83).
int get_state(mxopt_optimizer* o, const char* name, uint64_t n, StateEntry** out) {
  mxopt_ctx* ctx = o->ctx;
  auto it = o->state.find(name);
  if (it != o->state.end()) {
    if (it->second.n != n)
      return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string("state of '") + name + "' has " +
                  std::to_string(it->second.n) + " elements, parameter has " + std::to_string(n));
    *out = &it->second;
    return MXOPT_OK;
  }
  StateEntry e;
  e.n = n;
  DeviceGuard guard(ctx->device);
  const bool need_v = o->kind != Kind::Sgd || o->momentum != 0.0;
  if (n) {
    if (is_adam(o)) {
      HIP_TRY(ctx, state_alloc(ctx, (void**)&e.m, n * sizeof(float)));
      hipError_t err = hipMemsetAsync(e.m, 0, n * sizeof(float), ctx->stream);
      if (err != hipSuccess) { state_free(ctx, e.m); return hip_fail(ctx, err, "hipMemsetAsync(m)"); }
    }
    if (need_v) {
      hipError_t err = state_alloc(ctx, (void**)&e.v, n * sizeof(float));
      // SGD's velocity is written before it is ever read (first call: v = grad), no fill needed
      if (err == hipSuccess && o->kind != Kind::Sgd) err = hipMemsetAsync(e.v, 0, n * sizeof(float), ctx->stream);
      if (err != hipSuccess) {
        state_free(ctx, e.m);
        state_free(ctx, e.v);
        return hip_fail(ctx, err, "allocating optimizer state");
      }
    }
  }
  auto ins = o->state.emplace(name, e);
  *out = &ins.first->second;
  return MXOPT_OK;
}

int fill_row(mxopt_optimizer* o, const char* name, const mxopt_array* param, const mxopt_array* grad,
             const mxopt_array* out, mxopt_tensor* row, StateEntry** state_out) {
  mxopt_ctx* ctx = o->ctx;
  if (!name) return fail(ctx, MXOPT_ERR_INVALID_ARG, "param_name is NULL");
  int rc;
  if ((rc = check_array(ctx, param, "param"))) return rc;
  if ((rc = check_array(ctx, grad, "grad"))) return rc;
  if ((rc = check_array(ctx, out, "out"))) return rc;
  if (grad->n != param->n || out->n != param->n)
    return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string("'") + name + "': param, grad and out differ in size");
  if (out->dtype != MXOPT_F32 && out->dtype != param->dtype)
    return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string("'") + name + "': out must be float32 or the parameter's dtype");
  StateEntry* st = nullptr;
  if ((rc = get_state(o, name, param->n, &st))) return rc;
  *row = blank_tensor();
  row->p = param->data; row->p_out = out->data; row->g = grad->data;
  row->m = st->m; row->v = st->v;
  row->n = param->n;
  row->p_dtype = (uint8_t)param->dtype; row->p_out_dtype = (uint8_t)out->dtype; row->g_dtype = (uint8_t)grad->dtype;
  if (is_adam(o)) {
    o->step += 1;  // before the arithmetic, once per call (adam.rs:73, adamw.rs:77)
    if (o->bias_correction) mxopt_bias_correction(o->beta1, o->beta2, o->step, &row->bc1, &row->bc2);
  }
  if (o->kind == Kind::Sgd && o->momentum != 0.0 && !st->has_velocity) row->flags |= MXOPT_TF_FIRST;
  *state_out = st;
  return MXOPT_OK;
}

struct Hp {
  mxopt_adam_hp adam;
  mxopt_sgd_hp sgd;
  mxopt_rmsprop_hp rms;
};

int make_hp(mxopt_optimizer* o, Hp* hp) {
  switch (o->kind) {
    case Kind::Adam: mxopt_adam_hp_from_f64(o->lr, o->beta1, o->beta2, o->eps, 0.0, 0, &hp->adam); break;
    case Kind::AdamW: mxopt_adam_hp_from_f64(o->lr, o->beta1, o->beta2, o->eps, o->weight_decay, 1, &hp->adam); break;
    case Kind::Sgd:
      return mxopt_sgd_hp_from_f64(o->lr, o->momentum, o->weight_decay, o->dampening, o->nesterov, &hp->sgd);
    case Kind::Rmsprop: mxopt_rmsprop_hp_from_f64(o->lr, o->alpha, o->eps, o->weight_decay, &hp->rms); break;
  }
  return MXOPT_OK;
}

template <class T>
T opt_or(const T* p, T dflt) { return p ? *p : dflt; }

int new_optimizer(mxopt_ctx* ctx, Kind kind, mxopt_optimizer** out) {
  if (!ctx || !out) return fail(ctx, MXOPT_ERR_INVALID_ARG, "optimizer constructor: null argument");
  *out = new (std::nothrow) mxopt_optimizer();
  if (!*out) return fail(ctx, MXOPT_ERR_OOM, "out of host memory");
  (*out)->kind = kind;
  (*out)->ctx = ctx;
  return MXOPT_OK;
}

// One table row per array pair for the gradient utilities.
int grad_rows(mxopt_ctx* ctx, size_t n, const mxopt_array* grads, const mxopt_array* outs, const char* op,
              std::vector<mxopt_tensor>* rows) {
  if (n && !grads) return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(op) + ": gradients is NULL");
  rows->clear();
  rows->reserve(n);
  for (size_t i = 0; i < n; ++i) {
    int rc = check_array(ctx, &grads[i], op);
    if (rc) return rc;
    mxopt_tensor r = blank_tensor();
    r.g = grads[i].data; r.g_dtype = (uint8_t)grads[i].dtype; r.n = grads[i].n;
    if (outs) {
      if ((rc = check_array(ctx, &outs[i], op))) return rc;
      if (outs[i].n != grads[i].n) return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(op) + ": output size differs");
      r.g_out = outs[i].data; r.g_out_dtype = (uint8_t)outs[i].dtype;
    }
    rows->push_back(r);
  }
  return MXOPT_OK;
}

}  // namespace

extern "C" {

int mxopt_adam_new(mxopt_ctx* ctx, const double* learning_rate, const double* beta1, const double* beta2,
                   const double* eps, const int* bias_correction, mxopt_optimizer** out) {
  int rc = new_optimizer(ctx, Kind::Adam, out);
  if (rc) return rc;
  mxopt_optimizer* o = *out;
  o->lr = opt_or(learning_rate, 1e-3);
  o->beta1 = opt_or(beta1, 0.9);
  o->beta2 = opt_or(beta2, 0.999);
  o->eps = opt_or(eps, 1e-8);
  o->bias_correction = opt_or(bias_correction, 0) != 0;
  return MXOPT_OK;
}

int mxopt_adamw_new(mxopt_ctx* ctx, const double* learning_rate, const double* beta1, const double* beta2,
                    const double* eps, const double* weight_decay, const int* bias_correction,
                    mxopt_optimizer** out) {
  int rc = mxopt_adam_new(ctx, learning_rate, beta1, beta2, eps, bias_correction, out);
  if (rc) return rc;
  (*out)->kind = Kind::AdamW;
  (*out)->weight_decay = opt_or(weight_decay, 0.01);
  return MXOPT_OK;
}

int mxopt_sgd_new(mxopt_ctx* ctx, double learning_rate, const double* momentum, const double* weight_decay,
                  const double* dampening, const int* nesterov, mxopt_optimizer** out) {
  if (out) *out = nullptr;
  const double mu = opt_or(momentum, 0.0), damp = opt_or(dampening, 0.0);
  const bool nest = opt_or(nesterov, 0) != 0;
  if (nest && (mu <= 0.0 || damp != 0.0))  // sgd.rs:51-56
    return fail(ctx, MXOPT_ERR_INVALID_ARG, "Nesterov momentum requires momentum > 0 and dampening = 0");
  int rc = new_optimizer(ctx, Kind::Sgd, out);
  if (rc) return rc;
  mxopt_optimizer* o = *out;
  o->lr = learning_rate;
  o->momentum = mu;
  o->weight_decay = opt_or(weight_decay, 0.0);
  o->dampening = damp;
  o->nesterov = nest;
  return MXOPT_OK;
}

int mxopt_rmsprop_new(mxopt_ctx* ctx, const double* learning_rate, const double* alpha, const double* eps,
                      const double* weight_decay, mxopt_optimizer** out) {
  int rc = new_optimizer(ctx, Kind::Rmsprop, out);
  if (rc) return rc;
  mxopt_optimizer* o = *out;
  o->lr = opt_or(learning_rate, 1e-2);
  o->alpha = opt_or(alpha, 0.99);
  o->eps = opt_or(eps, 1e-8);
  o->weight_decay = opt_or(weight_decay, 0.0);
  return MXOPT_OK;
}

void mxopt_optimizer_free(mxopt_optimizer* opt) {
  if (!opt) return;
  free_state(opt);
  delete opt;
}

int mxopt_optimizer_update_single(mxopt_optimizer* opt, const char* param_name, const mxopt_array* param,
                                  const mxopt_array* grad, const mxopt_array* out) {
  if (!opt) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "update_single: optimizer is NULL");
  mxopt_ctx* ctx = opt->ctx;
  mxopt_tensor row;
  StateEntry* st = nullptr;
  int rc = fill_row(opt, param_name, param, grad, out, &row, &st);
  if (rc) return rc;
  Hp hp;
  if ((rc = make_hp(opt, &hp))) return rc;
  if (row.n == 0) return MXOPT_OK;
  DeviceGuard guard(ctx->device);
  const Launch L = make_single_launch(ctx, row, ctx->persistent != 0);
  const DevPrep prep = make_prep(nullptr);
  bool ok = false;
  switch (opt->kind) {
    case Kind::Adam:
    case Kind::AdamW: ok = launch_adam(row.p_dtype, row.g_dtype, row.p_out_dtype, -1, L, hp.adam, prep); break;
    case Kind::Sgd: ok = launch_sgd(row.p_dtype, row.g_dtype, row.p_out_dtype, L, hp.sgd, prep); break;
    case Kind::Rmsprop: ok = launch_rmsprop(row.p_dtype, row.g_dtype, row.p_out_dtype, L, hp.rms, prep); break;
  }
  if (!ok) return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string("update_single '") + param_name + "': unsupported dtypes");
  if ((rc = check_launch(ctx, "update_single"))) return rc;
  if (opt->kind == Kind::Sgd && opt->momentum != 0.0) st->has_velocity = true;
  return MXOPT_OK;
}

}  // extern "C"

// Rows, per-call step scalars and the cached table of one batched update; shared by update_many and
// update_many_accumulated.  On return opt->many_table describes `rows` and *hp holds the coefficients.
static int prepare_many(mxopt_optimizer* opt, size_t n, const char* const* param_names, const mxopt_array* params,
                        const mxopt_array* grads, const mxopt_array* outs, const mxopt_grad_prep* prep,
                        std::vector<StateEntry*>* states_out, Hp* hp_out) {
  mxopt_ctx* ctx = opt->ctx;
  std::vector<mxopt_tensor> rows(n);
  std::vector<StateEntry*>& states = *states_out;
  states.assign(n, nullptr);
  Hp& hp = *hp_out;
  const int64_t step_before = opt->step;
  for (size_t i = 0; i < n; ++i) {
    int rc = fill_row(opt, param_names[i], &params[i], &grads[i], &outs[i], &rows[i], &states[i]);
    if (rc) {
      opt->step = step_before;  // nothing was launched
      return rc;
    }
  }
  // A first momentum step writes the velocity that every later step reads.  Whether a conditional
  // update ran is known on the device only, so the host could not tell afterwards which kind of step
  // comes next.
  if (prep && prep->d_skip_if_nonzero)
    for (const mxopt_tensor& r : rows)
      if (r.flags & MXOPT_TF_FIRST)
        return fail(ctx, MXOPT_ERR_INVALID_ARG,
                    "SGD with momentum: the first update of a parameter cannot be conditional (prep->d_skip_if_nonzero)");
  int rc = make_hp(opt, &hp);
  if (rc) return rc;
  // Same buffers as last time?  Then only the per-step scalars change.
  std::vector<mxopt_tensor> key = rows;
  for (auto& r : key) { r.bc1 = r.bc2 = 1.0f; r.flags = 0; }
  const bool same = opt->many_table && key.size() == opt->many_key.size() &&
                    (key.empty() || std::memcmp(key.data(), opt->many_key.data(), key.size() * sizeof(mxopt_tensor)) == 0);
  if (!same) {
    // The same tensors in other buffers (a functional host hands back new arrays every step): keep the
    // chunk list and swap the pointers; anything else is a new table.
    bool moved = false;
    if (opt->many_table) {
      std::string why;
      moved = table_retarget_quiet(opt->many_table, rows.data(), rows.size(), &why) == MXOPT_OK;
      if (!moved) {
        mxopt_table_destroy(opt->many_table);
        opt->many_table = nullptr;
      }
    }
    if (!moved && (rc = mxopt_table_build(ctx, rows.data(), rows.size(), &opt->many_table))) return rc;
    opt->many_key = std::move(key);
  } else {
    bool scalars_differ = false;
    for (size_t i = 0; i < n && !scalars_differ; ++i) {
      const mxopt_tensor& h = opt->many_table->host[i];
      scalars_differ = h.bc1 != rows[i].bc1 || h.bc2 != rows[i].bc2 || h.flags != rows[i].flags;
    }
    if (scalars_differ) {
      std::vector<float> b1(n), b2(n);
      std::vector<uint32_t> fl(n);
      for (size_t i = 0; i < n; ++i) { b1[i] = rows[i].bc1; b2[i] = rows[i].bc2; fl[i] = rows[i].flags; }
      if ((rc = mxopt_table_set_step_scalars(opt->many_table, b1.data(), b2.data(), fl.data()))) return rc;
    }
  }
  return MXOPT_OK;
}

extern "C" {

int mxopt_optimizer_update_many(mxopt_optimizer* opt, size_t n, const char* const* param_names,
                                const mxopt_array* params, const mxopt_array* grads, const mxopt_array* outs,
                                const mxopt_grad_prep* prep) {
  if (!opt) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "update_many: optimizer is NULL");
  mxopt_ctx* ctx = opt->ctx;
  if (n && (!param_names || !params || !grads || !outs)) return fail(ctx, MXOPT_ERR_INVALID_ARG, "update_many: null argument");
  std::vector<StateEntry*> states;
  Hp hp;
  const int64_t step_before = opt->step;  // prepare_many counts the calls; a refused update must not
  int rc = prepare_many(opt, n, param_names, params, grads, outs, prep, &states, &hp);
  if (!rc) {
    switch (opt->kind) {
      case Kind::Adam:
      case Kind::AdamW: rc = mxopt_adam(ctx, opt->many_table, &hp.adam, prep); break;
      case Kind::Sgd: rc = mxopt_sgd(ctx, opt->many_table, &hp.sgd, prep); break;
      case Kind::Rmsprop: rc = mxopt_rmsprop(ctx, opt->many_table, &hp.rms, prep); break;
    }
  }
  if (rc) {
    opt->step = step_before;  // nothing was launched: later bias corrections see the count as it was
    return rc;
  }
  if (opt->kind == Kind::Sgd && opt->momentum != 0.0)
    for (StateEntry* st : states) st->has_velocity = true;
  return MXOPT_OK;
}

}  // extern "C"

// More micro-batches than the kernels have streams for: micro-batches 0 .. k - MXOPT_MAX_PENDING - 1 are
// added, in order, into a float32 buffer per parameter that the optimizer keeps with its state
// (accumulate_gradients' own additions, models/qwen3/model.rs:2217-2243); on return *folded holds those
// buffers followed by the last MXOPT_MAX_PENDING micro-batches.
static int fold_oldest(mxopt_optimizer* opt, size_t n, const char* const* param_names, const mxopt_array* params,
                       size_t k, const mxopt_array* grads, std::vector<mxopt_array>* folded) {
  mxopt_ctx* ctx = opt->ctx;
  const size_t spill = k - (size_t)MXOPT_MAX_PENDING;
  std::vector<float*> sums(n, nullptr);
  DeviceGuard guard(ctx->device);
  for (size_t i = 0; i < n; ++i) {
    if (!param_names[i]) return fail(ctx, MXOPT_ERR_INVALID_ARG, "param_name is NULL");
    int rc = check_array(ctx, &params[i], "param");
    if (rc) return rc;
    StateEntry* st = nullptr;
    if ((rc = get_state(opt, param_names[i], params[i].n, &st))) return rc;
    if (!st->sum && st->n) HIP_TRY(ctx, state_alloc(ctx, (void**)&st->sum, st->n * sizeof(float)));
    sums[i] = st->sum;
  }
  for (size_t j = 0; j < spill; ++j) {
    std::vector<mxopt_tensor> rows(n, blank_tensor());
    for (size_t i = 0; i < n; ++i) {
      const mxopt_array& g = grads[j * n + i];
      int rc = check_array(ctx, &g, "update_many_accumulated: gradient");
      if (rc) return rc;
      if (g.n != params[i].n)
        return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string("'") + param_names[i] + "': param and grad differ in size");
      rows[i].g = g.data; rows[i].g_dtype = (uint8_t)g.dtype;
      rows[i].g_out = sums[i]; rows[i].g_out_dtype = MXOPT_F32;
      rows[i].n = g.n;
    }
    mxopt_table* t = nullptr;
    int rc = cached_table(ctx, rows, &t);
    if (!rc) rc = mxopt_accumulate(ctx, t, j == 0, nullptr, -1.0, MXOPT_CLIP_ALWAYS_MULTIPLY, nullptr);
    if (rc) return rc;
  }
  folded->resize(((size_t)MXOPT_MAX_PENDING + 1) * n);
  for (size_t i = 0; i < n; ++i) (*folded)[i] = mxopt_array{sums[i], params[i].n, MXOPT_F32};
  for (size_t j = 0; j < (size_t)MXOPT_MAX_PENDING; ++j)
    for (size_t i = 0; i < n; ++i) (*folded)[(j + 1) * n + i] = grads[(spill + j) * n + i];
  return MXOPT_OK;
}

extern "C" {

int mxopt_optimizer_update_many_accumulated(mxopt_optimizer* opt, size_t n, const char* const* param_names,
                                            const mxopt_array* params, size_t k, const mxopt_array* grads,
                                            const mxopt_array* outs, const mxopt_grad_prep* prep, double max_norm,
                                            int clip_mode, mxopt_norm_result* d_norm) {
  const char* op = "update_many_accumulated";
  if (!opt) return fail(nullptr, MXOPT_ERR_INVALID_ARG, std::string(op) + ": optimizer is NULL");
  mxopt_ctx* ctx = opt->ctx;
  if (k < 1) return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(op) + ": at least one micro-batch");
  if (n && (!param_names || !params || !grads || !outs))
    return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(op) + ": null argument");
  if (n == 0) return MXOPT_OK;
  std::vector<mxopt_array> folded;
  if (k > (size_t)MXOPT_MAX_PENDING + 1) {
    int rc = fold_oldest(opt, n, param_names, params, k, grads, &folded);
    if (rc) return rc;
    grads = folded.data();
    k = (size_t)MXOPT_MAX_PENDING + 1;
  }
  if (prep && prep->d_scale && max_norm >= 0.0)
    return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(op) + ": prep->d_scale and max_norm exclude each other");
  // Every later micro-batch must look like the first: same sizes, one dtype.
  int xd = n && k > 1 ? grads[n].dtype : MXOPT_F32;
  for (size_t j = 1; j < k; ++j) {
    for (size_t i = 0; i < n; ++i) {
      const mxopt_array& g = grads[j * n + i];
      int rc = check_array(ctx, &g, "update_many_accumulated: gradient");
      if (rc) return rc;
      if (g.n != grads[i].n || g.dtype != xd)
        return fail(ctx, MXOPT_ERR_INVALID_ARG,
                    std::string(op) + ": micro-batch " + std::to_string(j) + " of '" + param_names[i] +
                        "' differs from the first in size, or from the other pending ones in dtype");
    }
  }
  const int64_t step_before = opt->step;
  std::vector<StateEntry*> states;
  Hp hp;
  int rc = prepare_many(opt, n, param_names, params, grads, outs, prep, &states, &hp);
  if (rc) {
    opt->step = step_before;
    return rc;
  }
  std::vector<const void*> streams((k - 1) * n);
  for (size_t j = 1; j < k; ++j)
    for (size_t i = 0; i < n; ++i) streams[(j - 1) * n + i] = grads[j * n + i].data;
  rc = mxopt_table_set_pending(opt->many_table, (int)(k - 1), streams.data(), xd);
  mxopt_grad_prep local;
  if (prep) local = *prep; else std::memset(&local, 0, sizeof local);
  if (!rc && max_norm >= 0.0) {
    mxopt_norm_result* slot = d_norm;
    if (!slot) rc = norm_scratch(ctx, &slot);
    if (!rc) rc = mxopt_norm_with_pending_list(ctx, opt->many_table, &local, max_norm, clip_mode, slot);
    local.d_scale = &slot->scale;
  }
  if (!rc) {
    switch (opt->kind) {
      case Kind::Adam:
      case Kind::AdamW: rc = mxopt_adam_with_pending_list(ctx, opt->many_table, &hp.adam, &local); break;
      case Kind::Sgd: rc = mxopt_sgd_with_pending_list(ctx, opt->many_table, &hp.sgd, &local); break;
      case Kind::Rmsprop: rc = mxopt_rmsprop_with_pending_list(ctx, opt->many_table, &hp.rms, &local); break;
    }
  }
  (void)mxopt_table_set_pending(opt->many_table, 0, nullptr, 0);
  if (rc) {
    opt->step = step_before;  // the update was not launched
    return rc;
  }
  if (opt->kind == Kind::Sgd && opt->momentum != 0.0)
    for (StateEntry* st : states) st->has_velocity = true;
  return MXOPT_OK;
}

int mxopt_optimizer_reset(mxopt_optimizer* opt) {
  if (!opt) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "reset: optimizer is NULL");
  free_state(opt);
  if (is_adam(opt)) opt->step = 0;  // adam.rs:143-146, adamw.rs:146-150
  return MXOPT_OK;
}

int64_t mxopt_optimizer_step_count(const mxopt_optimizer* opt) { return opt ? opt->step : 0; }

int mxopt_optimizer_state(mxopt_optimizer* opt, const char* param_name, float** m, float** v, uint64_t* n,
                          int* has_velocity) {
  if (!opt || !param_name) return fail(opt ? opt->ctx : nullptr, MXOPT_ERR_INVALID_ARG, "optimizer_state: null argument");
  auto it = opt->state.find(param_name);
  const bool found = it != opt->state.end();
  if (m) *m = found ? it->second.m : nullptr;
  if (v) *v = found ? it->second.v : nullptr;
  if (n) *n = found ? it->second.n : 0;
  if (has_velocity) *has_velocity = found && it->second.has_velocity;
  return MXOPT_OK;
}

int mxopt_optimizer_save_state(mxopt_optimizer* opt, const char* param_name, float* m_dst, float* v_dst) {
  if (!opt || !param_name) return fail(opt ? opt->ctx : nullptr, MXOPT_ERR_INVALID_ARG, "save_state: null argument");
  mxopt_ctx* ctx = opt->ctx;
  auto it = opt->state.find(param_name);
  if (it == opt->state.end())
    return fail(ctx, MXOPT_ERR_FAILURE, std::string("save_state: no state for '") + param_name + "'");
  const StateEntry& st = it->second;
  DeviceGuard guard(ctx->device);
  const size_t bytes = st.n * sizeof(float);
  if (m_dst && st.m && bytes) HIP_TRY(ctx, hipMemcpyAsync(m_dst, st.m, bytes, hipMemcpyDeviceToDevice, ctx->stream));
  if (v_dst && st.v && bytes) HIP_TRY(ctx, hipMemcpyAsync(v_dst, st.v, bytes, hipMemcpyDeviceToDevice, ctx->stream));
  return MXOPT_OK;
}

int mxopt_optimizer_load_state(mxopt_optimizer* opt, const char* param_name, const float* m, const float* v,
                               uint64_t n, int64_t step_count) {
  if (!opt || !param_name) return fail(opt ? opt->ctx : nullptr, MXOPT_ERR_INVALID_ARG, "load_state: null argument");
  mxopt_ctx* ctx = opt->ctx;
  StateEntry* st = nullptr;
  int rc = get_state(opt, param_name, n, &st);
  if (rc) return rc;
  DeviceGuard guard(ctx->device);
  if (st->m && m) HIP_TRY(ctx, hipMemcpyAsync(st->m, m, n * sizeof(float), hipMemcpyDeviceToDevice, ctx->stream));
  if (st->v && v) {
    HIP_TRY(ctx, hipMemcpyAsync(st->v, v, n * sizeof(float), hipMemcpyDeviceToDevice, ctx->stream));
    st->has_velocity = true;
  }
  if (is_adam(opt)) opt->step = step_count;
  return MXOPT_OK;
}

static const char* kind_name(Kind k) {
  switch (k) {
    case Kind::Adam: return "adam";
    case Kind::AdamW: return "adamw";
    case Kind::Sgd: return "sgd";
    default: return "rmsprop";
  }
}

int mxopt_optimizer_save_file(mxopt_optimizer* opt, const char* path) {
  if (!opt) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "optimizer_save_file: null optimizer");
  std::vector<CheckpointTensor> tensors;
  for (const auto& kv : opt->state) {
    const StateEntry& st = kv.second;
    if (st.m) tensors.push_back({kv.first + ".m", st.m, st.n});
    if (st.v && (opt->kind != Kind::Sgd || st.has_velocity)) tensors.push_back({kv.first + ".v", st.v, st.n});
  }
  return save_state_file(opt->ctx, path, kind_name(opt->kind), opt->step, tensors);
}

int mxopt_checkpoint_inspect(const char* path, char* optimizer, size_t optimizer_capacity, int64_t* step,
                             uint64_t* tensors, uint64_t* elements) {
  std::string kind;
  int rc = inspect_state_file(path, &kind, step, tensors, elements);
  if (rc) return rc;
  if (optimizer && optimizer_capacity) {
    std::strncpy(optimizer, kind.c_str(), optimizer_capacity - 1);
    optimizer[optimizer_capacity - 1] = '\0';
  }
  return MXOPT_OK;
}

int mxopt_optimizer_load_file(mxopt_optimizer* opt, const char* path) {
  if (!opt) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "optimizer_load_file: null optimizer");
  free_state(opt);  // a checkpoint replaces whatever state there was
  int64_t step = 0;
  int rc = load_state_file(opt->ctx, path, kind_name(opt->kind), &step,
                           [&](const std::string& key, uint64_t n, float** device) -> int {
    if (key.size() < 3 || key[key.size() - 2] != '.' || (key.back() != 'm' && key.back() != 'v'))
      return fail(opt->ctx, MXOPT_ERR_INVALID_ARG, "optimizer_load_file: unexpected tensor '" + key + "'");
    const std::string name = key.substr(0, key.size() - 2);
    StateEntry* st = nullptr;
    int r = get_state(opt, name.c_str(), n, &st);
    if (r) return r;
    if (key.back() == 'm') {
      *device = st->m;
    } else {
      *device = st->v;
      st->has_velocity = true;
    }
    if (!*device && n)
      return fail(opt->ctx, MXOPT_ERR_INVALID_ARG, "optimizer_load_file: this optimizer keeps no '" + key + "'");
    return MXOPT_OK;
  });
  if (rc) {
    free_state(opt);
    return rc;
  }
  if (is_adam(opt)) opt->step = step;
  return MXOPT_OK;
}

// ---- GradientUtils ------------------------------------------------------------------------

int mxopt_compute_gradient_norm(mxopt_ctx* ctx, size_t n, const mxopt_array* grads, double* norm_out) {
  if (!ctx || !norm_out) return fail(ctx, MXOPT_ERR_INVALID_ARG, "compute_gradient_norm: null argument");
  std::vector<mxopt_tensor> rows;
  int rc = grad_rows(ctx, n, grads, nullptr, "compute_gradient_norm", &rows);
  if (rc) return rc;
  mxopt_table* t = nullptr;
  mxopt_norm_result* d = nullptr;
  if ((rc = cached_table(ctx, rows, &t)) || (rc = norm_scratch(ctx, &d))) return rc;
  if ((rc = mxopt_global_norm(ctx, t, 0, nullptr, -1.0, MXOPT_CLIP_ALWAYS_MULTIPLY, d))) return rc;
  mxopt_norm_result h;
  if ((rc = mxopt_read_norm_result(ctx, d, &h))) return rc;
  *norm_out = h.norm;  // float64 accumulation, as optimizers/mod.rs:47-54
  return MXOPT_OK;
}

static int clip_by_norm(mxopt_ctx* ctx, size_t n, const mxopt_array* grads, const double* clip_value,
                        const double* max_norm, int clip_mode, const mxopt_array* outs, double* norm_out,
                        const char* op) {
  if (!ctx) return fail(nullptr, MXOPT_ERR_INVALID_ARG, std::string(op) + ": null context");
  if (n == 0) {  // empty map in, empty map out (optimizers/mod.rs:71-73, :120-122)
    if (norm_out) *norm_out = 0.0;
    return MXOPT_OK;
  }
  if (!outs) return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(op) + ": outs is NULL");
  std::vector<mxopt_tensor> rows;
  int rc = grad_rows(ctx, n, grads, outs, op, &rows);
  if (rc) return rc;
  mxopt_table* t = nullptr;
  mxopt_norm_result* d = nullptr;
  if ((rc = cached_table(ctx, rows, &t)) || (rc = norm_scratch(ctx, &d))) return rc;
  mxopt_grad_prep prep;
  std::memset(&prep, 0, sizeof prep);
  if (clip_value) {
    prep.has_clamp_pre = 1;
    prep.pre_lo = (float)(-*clip_value);
    prep.pre_hi = (float)(*clip_value);
  }
  if (max_norm) {
    if ((rc = mxopt_global_norm(ctx, t, 0, &prep, *max_norm, clip_mode, d))) return rc;
    prep.d_scale = &d->scale;
  }
  if ((rc = mxopt_grad_transform(ctx, t, &prep))) return rc;
  if (norm_out) {
    mxopt_norm_result h;
    if ((rc = mxopt_read_norm_result(ctx, d, &h))) return rc;
    *norm_out = (double)h.norm_f32;  // item_at_float32(0) as f64 (optimizers/mod.rs:138)
  }
  return MXOPT_OK;
}

int mxopt_clip_grad_norm(mxopt_ctx* ctx, size_t n, const mxopt_array* grads, double max_norm,
                         const mxopt_array* outs, double* norm_out) {
  return clip_by_norm(ctx, n, grads, nullptr, &max_norm, MXOPT_CLIP_ALWAYS_MULTIPLY, outs, norm_out, "clip_grad_norm");
}

int mxopt_clip_grad_value_and_norm(mxopt_ctx* ctx, size_t n, const mxopt_array* grads, double clip_value,
                                   const double* max_norm, const mxopt_array* outs) {
  return clip_by_norm(ctx, n, grads, &clip_value, max_norm, MXOPT_CLIP_ALWAYS_MULTIPLY, outs, nullptr,
                      "clip_grad_value_and_norm");
}

int mxopt_clip_gradients_by_global_norm(mxopt_ctx* ctx, size_t n, const mxopt_array* grads, double max_norm,
                                        const mxopt_array* outs) {
  return clip_by_norm(ctx, n, grads, nullptr, &max_norm, MXOPT_CLIP_IF_ABOVE, outs, nullptr,
                      "clip_gradients_by_global_norm");
}

static int clamp_arrays(mxopt_ctx* ctx, size_t n, const mxopt_array* grads, double lo, double hi,
                        const mxopt_array* outs, const char* op) {
  if (!ctx) return fail(nullptr, MXOPT_ERR_INVALID_ARG, std::string(op) + ": null context");
  if (n == 0) return MXOPT_OK;
  if (!outs) return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(op) + ": outs is NULL");
  mxopt_grad_prep prep;
  std::memset(&prep, 0, sizeof prep);
  prep.has_clamp_pre = 1;
  prep.pre_lo = (float)lo;  // static_cast<float> of the bound (mlx.cpp:474-478); non-finite = none
  prep.pre_hi = (float)hi;
  if (!std::isfinite(lo)) prep.pre_lo = -INFINITY;
  if (!std::isfinite(hi)) prep.pre_hi = INFINITY;
  std::vector<mxopt_tensor> rows;
  int rc = grad_rows(ctx, n, grads, outs, op, &rows);
  if (rc) return rc;
  if (n == 1) {  // one array: descriptor in the kernel arguments, no table
    if (rows[0].n == 0) return MXOPT_OK;
    DeviceGuard guard(ctx->device);
    const Launch L = make_single_launch(ctx, rows[0], ctx->persistent != 0);
    if (!launch_transform(rows[0].g_dtype, rows[0].g_out_dtype, L, make_prep(&prep), 0))
      return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(op) + ": unsupported dtypes");
    return check_launch(ctx, op);
  }
  mxopt_table* t = nullptr;
  if ((rc = cached_table(ctx, rows, &t))) return rc;
  return mxopt_grad_transform(ctx, t, &prep);
}

int mxopt_clip_grad_value(mxopt_ctx* ctx, const mxopt_array* grad, double min_val, double max_val,
                          const mxopt_array* out) {
  return clamp_arrays(ctx, 1, grad, min_val, max_val, out, "clip_grad_value");
}

int mxopt_clip_gradients_by_value(mxopt_ctx* ctx, size_t n, const mxopt_array* grads, double min_value,
                                  double max_value, const mxopt_array* outs) {
  return clamp_arrays(ctx, n, grads, min_value, max_value, outs, "clip_gradients_by_value");
}

// ---- accumulation / apply -----------------------------------------------------------------

int mxopt_accumulate_gradients(mxopt_ctx* ctx, size_t n, const mxopt_array* acc, const mxopt_array* new_grads,
                               const mxopt_array* outs) {
  if (!ctx) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "accumulate_gradients: null context");
  if (n == 0) return MXOPT_OK;
  if (!acc || !new_grads || !outs) return fail(ctx, MXOPT_ERR_INVALID_ARG, "accumulate_gradients: null argument");
  // widen_rows: a 16-bit running sum meets a gradient of another dtype.  `acc.add(new)` promotes such a
  // pair to float32 (models/qwen3/model.rs:2227): out = widen(acc), exact, then out += new.
  std::vector<mxopt_tensor> first_rows, add_rows, widen_rows;
  for (size_t i = 0; i < n; ++i) {
    int rc;
    if ((rc = check_array(ctx, &new_grads[i], "accumulate_gradients: new gradient"))) return rc;
    if ((rc = check_array(ctx, &outs[i], "accumulate_gradients: output"))) return rc;
    if ((rc = check_array(ctx, &acc[i], "accumulate_gradients: accumulated gradient", true))) return rc;
    if (outs[i].n != new_grads[i].n) return fail(ctx, MXOPT_ERR_INVALID_ARG, "accumulate_gradients: output size differs");
    mxopt_tensor r = blank_tensor();
    r.g = new_grads[i].data; r.g_dtype = (uint8_t)new_grads[i].dtype; r.n = new_grads[i].n;
    r.g_out = outs[i].data; r.g_out_dtype = (uint8_t)outs[i].dtype;
    if (acc[i].data == nullptr) {  // first time this name is seen: a copy (model.rs:2229-2232)
      first_rows.push_back(r);
      continue;
    }
    if (acc[i].n != new_grads[i].n) return fail(ctx, MXOPT_ERR_INVALID_ARG, "accumulate_gradients: shapes differ");
    const int promoted = acc[i].dtype == new_grads[i].dtype ? acc[i].dtype : MXOPT_F32;  // MLX promote_types
    if (outs[i].dtype != promoted)
      return fail(ctx, MXOPT_ERR_INVALID_ARG,
                  "accumulate_gradients: the output takes the promoted dtype of accumulator and gradient "
                  "(their own when equal, float32 otherwise)");
    if (acc[i].dtype != promoted) {  // 16-bit sum, other gradient dtype, float32 result
      if (acc[i].data == outs[i].data)
        return fail(ctx, MXOPT_ERR_INVALID_ARG, "accumulate_gradients: a 16-bit accumulator cannot hold the float32 sum in place");
      mxopt_tensor w = blank_tensor();
      w.g = acc[i].data; w.g_dtype = (uint8_t)acc[i].dtype; w.n = acc[i].n;
      w.g_out = outs[i].data; w.g_out_dtype = (uint8_t)outs[i].dtype;
      widen_rows.push_back(w);
    } else if (acc[i].data != outs[i].data) {  // out of place: read the running sum from a separate buffer
      r.p = acc[i].data;
      r.p_dtype = (uint8_t)acc[i].dtype;
    }
    add_rows.push_back(r);
  }
  for (int pass = 0; pass < 3; ++pass) {  // copies of new names, widened running sums, then the additions
    std::vector<mxopt_tensor>& rows = pass == 0 ? first_rows : pass == 1 ? widen_rows : add_rows;
    if (rows.empty()) continue;
    mxopt_table* t = nullptr;
    int rc = cached_table(ctx, rows, &t);
    if (rc) return rc;
    if ((rc = mxopt_accumulate(ctx, t, pass < 2, nullptr, -1.0, MXOPT_CLIP_ALWAYS_MULTIPLY, nullptr))) return rc;
  }
  return MXOPT_OK;
}

int mxopt_apply_gradients(mxopt_ctx* ctx, size_t n, const mxopt_array* params, const mxopt_array* grads,
                          double learning_rate, const mxopt_array* outs) {
  if (!ctx) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "apply_gradients: null context");
  if (n == 0) return MXOPT_OK;
  if (!params || !grads || !outs) return fail(ctx, MXOPT_ERR_INVALID_ARG, "apply_gradients: null argument");
  std::vector<mxopt_tensor> rows;
  rows.reserve(n);
  for (size_t i = 0; i < n; ++i) {
    int rc;
    if ((rc = check_array(ctx, &params[i], "apply_gradients: parameter"))) return rc;
    if ((rc = check_array(ctx, &grads[i], "apply_gradients: gradient"))) return rc;
    if ((rc = check_array(ctx, &outs[i], "apply_gradients: output"))) return rc;
    if (params[i].n != grads[i].n || params[i].n != outs[i].n)
      return fail(ctx, MXOPT_ERR_INVALID_ARG, "apply_gradients: sizes differ");
    if (outs[i].dtype != params[i].dtype)  // model.rs:2443-2448: the result keeps the parameter dtype
      return fail(ctx, MXOPT_ERR_INVALID_ARG, "apply_gradients: output dtype must equal the parameter's");
    mxopt_tensor r = blank_tensor();
    r.p = params[i].data; r.p_dtype = (uint8_t)params[i].dtype;
    r.p_out = outs[i].data; r.p_out_dtype = (uint8_t)outs[i].dtype;
    r.g = grads[i].data; r.g_dtype = (uint8_t)grads[i].dtype;
    r.n = params[i].n;
    rows.push_back(r);
  }
  mxopt_table* t = nullptr;
  int rc = cached_table(ctx, rows, &t);
  if (rc) return rc;
  return mxopt_sgd_plain(ctx, t, learning_rate, 0.0, nullptr);
}

// ---- LRScheduler (optimizers/mod.rs:239-292) ------------------------------------------------

double mxopt_lr_linear_decay(double initial_lr, double final_lr, int64_t current_step, int64_t total_steps) {
  if (current_step >= total_steps) return final_lr;
  const double progress = (double)current_step / (double)total_steps;
  return initial_lr + (final_lr - initial_lr) * progress;
}

double mxopt_lr_exponential_decay(double initial_lr, double decay_rate, int64_t current_step, int64_t decay_steps) {
  // the exponent is the INTEGER quotient of the step counters (optimizers/mod.rs:263)
  if (decay_steps == 0) return std::nan("");  // the reference panics on the division
  return initial_lr * std::pow(decay_rate, (double)(current_step / decay_steps));
}

double mxopt_lr_cosine_annealing(double initial_lr, double min_lr, int64_t current_step, int64_t total_steps) {
  if (current_step >= total_steps) return min_lr;
  const double progress = (double)current_step / (double)total_steps;
  const double cosine_val = std::cos(progress * 3.14159265358979323846);
  return min_lr + (initial_lr - min_lr) * 0.5 * (1.0 + cosine_val);
}

double mxopt_lr_step_decay(double initial_lr, double factor, int64_t current_step, int64_t step_size) {
  if (step_size == 0) return std::nan("");
  const int64_t num_decays = current_step / step_size;
  return initial_lr * std::pow(factor, (double)(int32_t)num_decays);  // powi(num_decays as i32)
}

}  // extern "C"
