// The optimizer side of the training engines: bookkeeping on the host, arithmetic in the kernels.
// Declarations, and the reference lines each entry point stands behind, are in
// include/mxopt_engine.h.
#include "mxopt_engine.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstring>
#include <new>
#include <string>
#include <unordered_map>
#include <vector>

#include "mxopt_internal.h"

using namespace mxopt;

namespace {

struct Slot {
  std::string name;
  mxopt_array param{};
  void* acc = nullptr;  // accumulation buffer, allocated on first use, reused by every cycle
  int acc_dtype = -1;
  bool in_acc = false;  // holds a value in the current accumulation cycle
};

int dtype_bytes(int dt) { return dt == MXOPT_F32 ? 4 : 2; }

}  // namespace

struct mxopt_engine {
  mxopt_ctx* ctx = nullptr;
  mxopt_engine_config cfg{};
  std::vector<Slot> slots;
  std::unordered_map<std::string, size_t> index;
  mxopt_optimizer* adamw = nullptr;       // APPLY_ADAMW: moments by parameter name
  mxopt_norm_result* d_result = nullptr;  // device slot of the norm pass
  // EngineState (grpo/engine.rs:227-271, sft/engine.rs:114-145), optimizer-side fields
  bool have_acc = false;
  int32_t micro_step = 0;
  int64_t step = 0;
  uint64_t nan_gradient_count = 0;
  uint32_t consecutive_nan_count = 0;
  bool needs_emergency_save = false;
  // defer_accumulation: where the accepted micro-batches of the current cycle lie.  Column c of every
  // entry belongs to slot held_slots[c] (the order of the cycle's first micro-batch).
  std::vector<size_t> held_slots;
  std::vector<std::vector<mxopt_array>> held;
  // More micro-batches than the kernels have streams for: the oldest ones have been added into the
  // slots' float32 buffers, which then stand in entry 0 (held_is_sum).  held_result[j]: which of the
  // device norm slots holds entry j's clip factor (GRPO), -1 for the sum.
  bool held_is_sum = false;
  std::vector<int> held_result;
  // mxopt_engine_micro_batch_async: the bookkeeping above has been advanced as if the last micro-batch
  // were valid; its kernels were told to do nothing otherwise, and its validity flag is on its way to
  // `h_pinned`.  `before` is the bookkeeping as it was, to go back to if the flag turns out set.
  struct Book {
    bool have_acc, needs_emergency_save, held_is_sum;
    int32_t micro_step;
    int64_t step;
    uint64_t nan_gradient_count;
    uint32_t consecutive_nan_count;
    int64_t adamw_calls;  // APPLY_ADAMW: the optimizer object's call counter
    std::vector<size_t> held_slots;
    std::vector<std::vector<mxopt_array>> held;
    std::vector<int> held_result;
    std::vector<char> in_acc;
  };
  bool async_mode = false;                            // inside an async call
  const uint64_t* async_skip = nullptr;            // ... the device flag its kernels obey
  bool async_enqueued = false;                        // ... a flag copy was enqueued
  Book* async_book = nullptr;                         // ... the bookkeeping to go back to (the caller's local)
  bool pending = false;
  int pending_applied = 0;
  Book before;
  mxopt_norm_result* h_pinned = nullptr;
  hipEvent_t copied = nullptr;
};

namespace {

mxopt_engine::Book take_book(const mxopt_engine* e) {
  mxopt_engine::Book b;
  b.have_acc = e->have_acc; b.needs_emergency_save = e->needs_emergency_save; b.held_is_sum = e->held_is_sum;
  b.micro_step = e->micro_step; b.step = e->step; b.nan_gradient_count = e->nan_gradient_count;
  b.consecutive_nan_count = e->consecutive_nan_count;
  b.adamw_calls = e->adamw ? mxopt_optimizer_step_count(e->adamw) : 0;
  b.held_slots = e->held_slots; b.held = e->held; b.held_result = e->held_result;
  b.in_acc.resize(e->slots.size());
  for (size_t i = 0; i < e->slots.size(); ++i) b.in_acc[i] = e->slots[i].in_acc ? 1 : 0;
  return b;
}

void put_book(mxopt_engine* e, const mxopt_engine::Book& b) {
  e->have_acc = b.have_acc; e->needs_emergency_save = b.needs_emergency_save; e->held_is_sum = b.held_is_sum;
  e->micro_step = b.micro_step; e->step = b.step; e->nan_gradient_count = b.nan_gradient_count;
  e->consecutive_nan_count = b.consecutive_nan_count;
  if (e->adamw) optimizer_set_step_count(e->adamw, b.adamw_calls);  // the update it counted did nothing on the device
  e->held_slots = b.held_slots; e->held = b.held; e->held_result = b.held_result;
  for (size_t i = 0; i < e->slots.size() && i < b.in_acc.size(); ++i) e->slots[i].in_acc = b.in_acc[i] != 0;
}

// A prep for a kernel that changes memory: inside an async call it also carries the micro-batch's
// validity flag, so that the kernel does nothing when the gradients held a NaN/Inf.
mxopt_grad_prep guarded(const mxopt_engine* e, mxopt_grad_prep prep) {
  if (e->async_skip) prep.d_skip_if_nonzero = e->async_skip;
  return prep;
}

int32_t acc_steps(const mxopt_engine* e) {
  return e->cfg.gradient_accumulation_steps < 1 ? 1 : e->cfg.gradient_accumulation_steps;
}
uint64_t max_nan(const mxopt_engine* e) {
  return e->cfg.max_nan_gradients < 1 ? 100u : (uint64_t)e->cfg.max_nan_gradients;
}
uint32_t emergency_threshold(const mxopt_engine* e) {
  return e->cfg.emergency_save_threshold < 1 ? 5u : (uint32_t)e->cfg.emergency_save_threshold;
}

void fill_metrics(const mxopt_engine* e, mxopt_engine_metrics* m, int applied, int skipped) {
  if (!m) return;
  std::memset(m, 0, sizeof *m);
  m->step = e->step;
  m->micro_step = e->micro_step;
  m->gradients_applied = applied;
  m->skipped = skipped;
  m->needs_emergency_save = e->needs_emergency_save ? 1 : 0;
  m->consecutive_nan_count = e->consecutive_nan_count;
  m->nan_gradient_count = e->nan_gradient_count;
  m->grad_sumsq = m->grad_norm = NAN;
  m->clip_scale = 1.0f;
}

void add_norm(mxopt_engine_metrics* m, const mxopt_norm_result& h) {
  if (!m) return;
  m->norm_measured = 1;
  m->grad_sumsq = h.sumsq;
  m->grad_norm = h.norm;
  m->clip_scale = h.scale;
}

int ensure_acc(mxopt_engine* e, Slot& s, int dtype) {
  if (s.acc && s.acc_dtype == dtype) return MXOPT_OK;
  DeviceGuard guard(e->ctx->device);
  if (s.acc) {
    HIP_TRY(e->ctx, hipStreamSynchronize(e->ctx->stream));
    state_free(e->ctx, s.acc);
    s.acc = nullptr;
  }
  if (s.param.n) HIP_TRY(e->ctx, state_alloc(e->ctx, &s.acc, s.param.n * (size_t)dtype_bytes(dtype)));
  s.acc_dtype = dtype;
  return MXOPT_OK;
}

// Checks names and sizes; on success idx[i] is the slot of gradient i.
int resolve(mxopt_engine* e, size_t n, const char* const* names, const mxopt_array* grads, std::vector<size_t>* idx) {
  mxopt_ctx* ctx = e->ctx;
  if (n && (!names || !grads)) return fail(ctx, MXOPT_ERR_INVALID_ARG, "engine: null names or gradients");
  idx->resize(n);
  for (size_t i = 0; i < n; ++i) {
    if (!names[i]) return fail(ctx, MXOPT_ERR_INVALID_ARG, "engine: null gradient name");
    auto it = e->index.find(names[i]);
    if (it == e->index.end())  // models/qwen3/model.rs:2427-2432
      return fail(ctx, MXOPT_ERR_FAILURE, std::string("Parameter '") + names[i] + "' not found in model");
    int rc = check_array(ctx, &grads[i], "engine: gradient");
    if (rc) return rc;
    if (grads[i].n != e->slots[it->second].param.n)
      return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string("engine: gradient '") + names[i] + "' has the wrong size");
    (*idx)[i] = it->second;
  }
  return MXOPT_OK;
}

mxopt_grad_prep no_prep() {
  mxopt_grad_prep p;
  std::memset(&p, 0, sizeof p);
  return p;
}

// The parameter update over every slot that holds an accumulated value.  `prep` turns the
// accumulated sum into the gradient that is applied.
int apply_accumulated(mxopt_engine* e, double lr, double weight_decay, const mxopt_grad_prep& prep) {
  mxopt_ctx* ctx = e->ctx;
  std::vector<mxopt_tensor> rows;
  std::vector<const char*> names;
  std::vector<mxopt_array> params, grads;
  for (Slot& s : e->slots) {
    if (!s.in_acc) continue;
    if (e->cfg.apply == MXOPT_ENGINE_APPLY_ADAMW) {
      names.push_back(s.name.c_str());
      params.push_back(s.param);
      grads.push_back(mxopt_array{s.acc, s.param.n, s.acc_dtype});
    } else {
      mxopt_tensor r = blank_tensor();
      r.p = s.param.data; r.p_out = s.param.data;
      r.p_dtype = r.p_out_dtype = (uint8_t)s.param.dtype;
      r.g = s.acc; r.g_dtype = (uint8_t)s.acc_dtype;
      r.n = s.param.n;
      rows.push_back(r);
    }
  }
  if (e->cfg.apply == MXOPT_ENGINE_APPLY_ADAMW) {
    if (names.empty()) return MXOPT_OK;
    return mxopt_optimizer_update_many(e->adamw, names.size(), names.data(), params.data(), grads.data(),
                                       params.data(), &prep);
  }
  if (rows.empty()) return MXOPT_OK;
  mxopt_table* t = nullptr;
  int rc = cached_table(ctx, rows, &t);
  if (rc) return rc;
  return mxopt_sgd_plain(ctx, t, lr, weight_decay, &prep);
}

void end_cycle(mxopt_engine* e) {
  // the reference's debug!("Applied gradients with lr ...") (grpo/engine.rs:684)
  MXOPT_DEBUG("%s engine: applied gradients with lr %g%s", e->cfg.kind == MXOPT_ENGINE_GRPO ? "GRPO" : "SFT",
              e->cfg.learning_rate, e->cfg.defer_accumulation ? " (deferred accumulation)" : "");
  for (Slot& s : e->slots) s.in_acc = false;
  e->have_acc = false;
  e->micro_step = 0;
  e->held.clear();
  e->held_slots.clear();
  e->held_result.clear();
  e->held_is_sum = false;
}

// ---- deferred accumulation ---------------------------------------------------------------

// Remembers where this micro-batch's gradients lie.  The first micro-batch of a cycle fixes the set of
// names (a name given twice keeps its first gradient, as the maps of the reference would); later ones
// must bring exactly that set.
int defer_record(mxopt_engine* e, const std::vector<size_t>& idx, const mxopt_array* grads) {
  mxopt_ctx* ctx = e->ctx;
  const size_t n = idx.size();
  if (e->held.empty()) {
    std::vector<char> seen(e->slots.size(), 0);
    e->held_slots.clear();
    std::vector<mxopt_array> first;
    for (size_t i = 0; i < n; ++i) {
      if (seen[idx[i]]) continue;
      seen[idx[i]] = 1;
      e->held_slots.push_back(idx[i]);
      first.push_back(grads[i]);
    }
    e->held.push_back(std::move(first));
    return MXOPT_OK;
  }
  std::vector<const mxopt_array*> by_slot(e->slots.size(), nullptr);
  size_t distinct = 0;
  for (size_t i = 0; i < n; ++i) {
    if (by_slot[idx[i]]) continue;
    by_slot[idx[i]] = &grads[i];
    ++distinct;
  }
  const char* same_names = "engine: deferred accumulation needs the same gradient names in every micro-batch of a cycle";
  if (distinct != e->held_slots.size()) return fail(ctx, MXOPT_ERR_INVALID_ARG, same_names);
  std::vector<mxopt_array> row;
  const int pending_dtype = e->held.size() > 1 && !e->held[1].empty() ? e->held[1][0].dtype : -1;
  for (size_t slot : e->held_slots) {
    if (!by_slot[slot]) return fail(ctx, MXOPT_ERR_INVALID_ARG, same_names);
    const mxopt_array& g = *by_slot[slot];
    const int want = pending_dtype >= 0 ? pending_dtype : (row.empty() ? g.dtype : row[0].dtype);
    const int first_dtype = e->held[0][row.size()].dtype;
    if (g.dtype != want || (first_dtype != g.dtype && first_dtype != MXOPT_F32))
      return fail(ctx, MXOPT_ERR_INVALID_ARG,
                  "engine: deferred accumulation needs one gradient dtype ('" + e->slots[slot].name + "' differs)");
    row.push_back(g);
  }
  e->held.push_back(std::move(row));
  return MXOPT_OK;
}

constexpr int kResultSlots = MXOPT_MAX_PENDING + 2;  // every held micro-batch and the one that arrives

// A device norm slot that no held micro-batch uses.
int free_result_slot(const mxopt_engine* e) {
  for (int slot = 0; slot < kResultSlots; ++slot)
    if (std::find(e->held_result.begin(), e->held_result.end(), slot) == e->held_result.end()) return slot;
  return kResultSlots - 1;  // not reached: at most MXOPT_MAX_PENDING + 1 entries are held
}

mxopt_grad_prep grpo_clamp(const mxopt_engine* e) {
  const double clip_value = e->cfg.has_gradient_clip_value ? e->cfg.gradient_clip_value : 1.0;  // grpo/engine.rs:636
  mxopt_grad_prep prep = no_prep();
  prep.has_clamp_pre = 1;
  prep.pre_lo = (float)(-clip_value);
  prep.pre_hi = (float)clip_value;
  return prep;
}

// Every stream is taken and one more micro-batch is about to be held: the two oldest entries become
// one.  Entry 0 is copied (GRPO: clamped and clipped by its own factor) into the slots' float32
// buffers unless it is such a sum already, entry 1 is added to it the same way -- the additions the
// buffered path makes, in the same order -- and the buffers take the place of entry 0.
int defer_spill(mxopt_engine* e) {
  mxopt_ctx* ctx = e->ctx;
  const size_t n = e->held_slots.size();
  const bool grpo = e->cfg.kind == MXOPT_ENGINE_GRPO;
  for (size_t c = 0; c < n; ++c) {
    int rc = ensure_acc(e, e->slots[e->held_slots[c]], MXOPT_F32);
    if (rc) return rc;
  }
  for (size_t j = e->held_is_sum ? 1 : 0; j < 2; ++j) {
    if (n == 0) break;
    std::vector<mxopt_tensor> rows(n, blank_tensor());
    for (size_t c = 0; c < n; ++c) {
      const Slot& s = e->slots[e->held_slots[c]];
      rows[c].g = e->held[j][c].data; rows[c].g_dtype = (uint8_t)e->held[j][c].dtype;
      rows[c].g_out = s.acc; rows[c].g_out_dtype = MXOPT_F32;
      rows[c].n = s.param.n;
    }
    mxopt_table* t = nullptr;
    int rc = cached_table(ctx, rows, &t);
    if (rc) return rc;
    if (grpo) {
      // Not guarded by the arriving micro-batch's validity flag: the two entries that move were accepted by
      // earlier calls, and their sum is the same whatever the new micro-batch turns out to hold.
      mxopt_grad_prep prep = grpo_clamp(e);
      if (e->cfg.has_gradient_clip_norm) prep.d_scale = &e->d_result[e->held_result[j]].scale;
      rc = mxopt_accumulate_transformed(ctx, t, j == 0, &prep);
    } else {
      rc = mxopt_accumulate(ctx, t, j == 0, nullptr, -1.0, MXOPT_CLIP_ALWAYS_MULTIPLY, nullptr);
    }
    if (rc) return rc;
  }
  MXOPT_DEBUG("%s engine: deferred accumulation spilled the oldest micro-batch into the float32 buffers",
              grpo ? "GRPO" : "SFT");
  for (size_t c = 0; c < n; ++c) {
    const Slot& s = e->slots[e->held_slots[c]];
    e->held[0][c] = mxopt_array{s.acc, s.param.n, MXOPT_F32};
  }
  e->held_is_sum = true;
  e->held_result[0] = -1;
  e->held.erase(e->held.begin() + 1);
  e->held_result.erase(e->held_result.begin() + 1);
  if (e->async_book) {  // the spill stays whatever the arriving micro-batch's flag says: the caller's buffers are free
    e->async_book->held = e->held;
    e->async_book->held_result = e->held_result;
    e->async_book->held_is_sum = true;
  }
  return MXOPT_OK;
}

// Table over the held columns: parameters updated in place, g = the first micro-batch, the later ones
// attached as pending streams.
int defer_table(mxopt_engine* e, mxopt_table** out) {
  mxopt_ctx* ctx = e->ctx;
  const size_t n = e->held_slots.size();
  std::vector<mxopt_tensor> rows(n, blank_tensor());
  for (size_t c = 0; c < n; ++c) {
    const Slot& s = e->slots[e->held_slots[c]];
    mxopt_tensor& r = rows[c];
    r.p = s.param.data; r.p_out = s.param.data;
    r.p_dtype = r.p_out_dtype = (uint8_t)s.param.dtype;
    r.g = e->held[0][c].data; r.g_dtype = (uint8_t)e->held[0][c].dtype;
    r.n = s.param.n;
  }
  int rc = cached_table(ctx, rows, out);
  if (rc) return rc;
  const size_t k = e->held.size() - 1;
  std::vector<const void*> streams(k * n);
  for (size_t j = 0; j < k; ++j)
    for (size_t c = 0; c < n; ++c) streams[j * n + c] = e->held[j + 1][c].data;
  return mxopt_table_set_pending(*out, (int)k, streams.data(), k && n ? e->held[1][0].dtype : MXOPT_F32);
}

// ---- GRPO: grpo/engine.rs:561-704 ------------------------------------------------------

// The bookkeeping of a micro-batch that held a NaN/Inf (engine.rs:571-633); nothing else is touched.
int grpo_skipped(mxopt_engine* e, mxopt_engine_metrics* out) {
  MXOPT_DEBUG("GRPO engine: NaN/Inf gradient, micro-batch skipped (%llu so far)",
              (unsigned long long)e->nan_gradient_count + 1);
  e->nan_gradient_count += 1;
  e->consecutive_nan_count += 1;
  if (e->nan_gradient_count >= max_nan(e)) {
    fill_metrics(e, out, 0, 1);
    return fail(e->ctx, MXOPT_ERR_FAILURE,
                "Training stopped: exceeded maximum NaN gradient count (" + std::to_string(e->nan_gradient_count) +
                    "/" + std::to_string(max_nan(e)) + ")");
  }
  if (e->consecutive_nan_count >= emergency_threshold(e)) e->needs_emergency_save = true;
  e->step += 1;
  fill_metrics(e, out, 0, 1);
  return MXOPT_OK;
}

// The result of the norm pass starts its way to pinned host memory; nobody waits for it here.
int enqueue_flag_copy(mxopt_engine* e, const mxopt_norm_result* d_result) {
  mxopt_ctx* ctx = e->ctx;
  DeviceGuard guard(ctx->device);
  launch_mirror_result(ctx->stream, d_result, e->h_pinned);
  int rc = check_launch(ctx, "mirror_result_kernel");
  if (rc) return rc;
  HIP_TRY(ctx, hipEventRecord(e->copied, ctx->stream));
  e->async_skip = &d_result->nonfinite;
  e->async_enqueued = true;
  return MXOPT_OK;
}

// Looks at the flag of the last async micro-batch (waiting for its copy if it is still under way) and
// puts the bookkeeping right: nothing to do when the gradients were valid; otherwise back to the state
// before that call, then the reference's skip.  `out` gets what the blocking call would have returned.
int settle(mxopt_engine* e, mxopt_engine_metrics* out) {
  if (!e->pending) {
    fill_metrics(e, out, 0, 0);
    return MXOPT_OK;
  }
  mxopt_ctx* ctx = e->ctx;
  {
    DeviceGuard guard(ctx->device);
    HIP_TRY(ctx, hipEventSynchronize(e->copied));
  }
  e->pending = false;
  const mxopt_norm_result h = *e->h_pinned;
  if (h.nonfinite & 1u) {  // bit 0: an invalid element; the kernels looked at the same bit
    put_book(e, e->before);
    return grpo_skipped(e, out);
  }
  fill_metrics(e, out, e->pending_applied, 0);
  add_norm(out, h);
  return MXOPT_OK;
}

int grpo_micro_batch(mxopt_engine* e, const std::vector<size_t>& idx, const mxopt_array* grads,
                     mxopt_engine_metrics* out) {
  mxopt_ctx* ctx = e->ctx;
  const size_t n = idx.size();
  mxopt_grad_prep prep = grpo_clamp(e);
  mxopt_norm_result h;
  std::memset(&h, 0, sizeof h);
  h.scale = 1.0f;
  // deferred: every accepted micro-batch of the cycle keeps its own clip factor on the device
  const int result_slot = e->cfg.defer_accumulation ? free_result_slot(e) : 0;
  mxopt_norm_result* d_result = e->d_result + result_slot;
  int rc;
  if (n) {
    // One read of the gradients: validity of the raw values and the norm of the clamped ones.
    std::vector<mxopt_tensor> rows(n, blank_tensor());
    for (size_t i = 0; i < n; ++i) {
      rows[i].g = grads[i].data; rows[i].g_dtype = (uint8_t)grads[i].dtype; rows[i].n = grads[i].n;
    }
    mxopt_table* t = nullptr;
    if ((rc = cached_table(ctx, rows, &t))) return rc;
    const double max_norm = e->cfg.has_gradient_clip_norm ? e->cfg.gradient_clip_norm : -1.0;
    if ((rc = mxopt_global_norm(ctx, t, 0, &prep, max_norm, MXOPT_CLIP_ALWAYS_MULTIPLY, d_result))) return rc;
    // async: the flag is not waited for; every kernel below obeys it on the device instead
    if ((rc = e->async_mode ? enqueue_flag_copy(e, d_result) : mxopt_read_norm_result(ctx, d_result, &h))) return rc;
  }
  if (h.nonfinite & 1u) return grpo_skipped(e, out);  // engine.rs:571-633: skip the whole micro-batch, touch nothing
  e->consecutive_nan_count = 0;  // engine.rs:660
  if (!e->have_acc)
    for (Slot& s : e->slots) s.in_acc = false;  // also after a call that failed half way
  if (e->cfg.has_gradient_clip_norm) prep.d_scale = &e->d_result->scale;
  const int32_t N = acc_steps(e);

  if (e->cfg.defer_accumulation) {
    // Nothing is accumulated: the micro-batch is only remembered.  At the end of the cycle one pass
    // over p and the held gradients forms sum_j clip_j(clamp(g_j)) in registers and applies lr/N.
    if (e->held.size() > (size_t)MXOPT_MAX_PENDING && (rc = defer_spill(e))) return rc;
    if ((rc = defer_record(e, idx, grads))) return rc;
    e->held_result.push_back(result_slot);
    e->have_acc = true;
    e->micro_step += 1;
    int applied = 0;
    if (e->micro_step >= N) {
      if (!e->held_slots.empty()) {
        mxopt_table* t = nullptr;
        if ((rc = defer_table(e, &t))) return rc;
        const float* scales[MXOPT_MAX_PENDING + 1] = {};
        if (e->cfg.has_gradient_clip_norm)
          for (size_t j = 0; j < e->held.size(); ++j)
            scales[j] = e->held_result[j] >= 0 ? &e->d_result[e->held_result[j]].scale : nullptr;
        prep.d_scale = nullptr;
        prep = guarded(e, prep);
        rc = mxopt_sgd_plain_with_pending_list_each(ctx, t, e->cfg.learning_rate / (double)N, 0.0, &prep, scales,
                                                    e->held_is_sum ? 1 : 0);
        (void)mxopt_table_set_pending(t, 0, nullptr, 0);
        if (rc) return rc;
      }
      end_cycle(e);
      applied = 1;
    }
    e->step += 1;
    fill_metrics(e, out, applied, 0);
    if (n) add_norm(out, h);
    return MXOPT_OK;
  }

  if (e->micro_step + 1 >= N && e->cfg.apply == MXOPT_ENGINE_APPLY_SGD) {
    // Last micro-batch of the cycle: p -= (lr/N) * (acc + clip(clamp(g))) in one pass over p, acc and
    // g; the sum is formed in registers exactly as the accumulation pass would have stored it.
    const double lr = e->cfg.learning_rate / (double)N;  // engine.rs:672
    std::vector<char> in_batch(e->slots.size(), 0);
    std::vector<mxopt_tensor> pending, direct, acc_only;
    for (size_t i = 0; i < n; ++i) {
      Slot& s = e->slots[idx[i]];
      if (in_batch[idx[i]]) continue;
      in_batch[idx[i]] = 1;
      mxopt_tensor r = blank_tensor();
      r.p = s.param.data; r.p_out = s.param.data;
      r.p_dtype = r.p_out_dtype = (uint8_t)s.param.dtype;
      r.n = s.param.n;
      if (s.in_acc) {
        r.g = s.acc; r.g_dtype = MXOPT_F32;
        r.g_out = grads[i].data; r.g_out_dtype = (uint8_t)grads[i].dtype;
        pending.push_back(r);
      } else {
        r.g = grads[i].data; r.g_dtype = (uint8_t)grads[i].dtype;
        direct.push_back(r);
      }
    }
    for (size_t k = 0; k < e->slots.size(); ++k) {
      Slot& s = e->slots[k];
      if (!s.in_acc || in_batch[k]) continue;
      mxopt_tensor r = blank_tensor();
      r.p = s.param.data; r.p_out = s.param.data;
      r.p_dtype = r.p_out_dtype = (uint8_t)s.param.dtype;
      r.g = s.acc; r.g_dtype = MXOPT_F32;
      r.n = s.param.n;
      acc_only.push_back(r);
    }
    mxopt_table* t = nullptr;
    prep = guarded(e, prep);
    const mxopt_grad_prep only_guard = guarded(e, no_prep());
    if (!pending.empty()) {
      if ((rc = cached_table(ctx, pending, &t)) || (rc = mxopt_sgd_plain_with_pending(ctx, t, lr, 0.0, &prep, 0))) return rc;
    }
    if (!direct.empty()) {
      if ((rc = cached_table(ctx, direct, &t)) || (rc = mxopt_sgd_plain(ctx, t, lr, 0.0, &prep))) return rc;
    }
    if (!acc_only.empty()) {
      if ((rc = cached_table(ctx, acc_only, &t)) ||
          (rc = mxopt_sgd_plain(ctx, t, lr, 0.0, e->async_skip ? &only_guard : nullptr)))
        return rc;
    }
    end_cycle(e);
    e->step += 1;
    fill_metrics(e, out, 1, 0);
    if (n) add_norm(out, h);
    return MXOPT_OK;
  }

  // acc (+)= clip_norm(clamp(g)) in float32 (engine.rs:636-661, :2632-2666)
  std::vector<mxopt_tensor> first_rows, add_rows;
  for (size_t i = 0; i < n; ++i) {
    Slot& s = e->slots[idx[i]];
    if ((rc = ensure_acc(e, s, MXOPT_F32))) return rc;
    mxopt_tensor r = blank_tensor();
    r.g = grads[i].data; r.g_dtype = (uint8_t)grads[i].dtype;
    r.g_out = s.acc; r.g_out_dtype = MXOPT_F32;
    r.n = grads[i].n;
    (s.in_acc ? add_rows : first_rows).push_back(r);
    s.in_acc = true;
  }
  for (int pass = 0; pass < 2; ++pass) {
    std::vector<mxopt_tensor>& rows = pass == 0 ? first_rows : add_rows;
    if (rows.empty()) continue;
    mxopt_table* t = nullptr;
    if ((rc = cached_table(ctx, rows, &t))) return rc;
    const mxopt_grad_prep gp = guarded(e, prep);
    if ((rc = mxopt_accumulate_transformed(ctx, t, pass == 0, &gp))) return rc;
  }
  e->have_acc = true;
  e->micro_step += 1;

  int applied = 0;
  if (e->micro_step >= N) {  // engine.rs:666-692, with AdamW on the averaged sum in place of apply_gradients
    mxopt_grad_prep ap = guarded(e, no_prep());
    ap.has_pre_mul = 1;
    ap.pre_mul = (float)(1.0 / (double)N);
    if ((rc = apply_accumulated(e, e->cfg.learning_rate, 0.0, ap))) return rc;
    end_cycle(e);
    applied = 1;
  }
  e->step += 1;  // engine.rs:690, :696
  fill_metrics(e, out, applied, 0);
  if (n) add_norm(out, h);
  return MXOPT_OK;
}

// ---- SFT: sft/engine.rs:268-371, :459-553 ------------------------------------------------

// Average by `count`, clip by norm, clamp, decay, update (sft/engine.rs:293-371).  `norm_ready`:
// *d_result already describes acc/count.
int sft_apply(mxopt_engine* e, int32_t count, bool norm_ready, mxopt_engine_metrics* out, mxopt_norm_result* h_out,
              bool* measured) {
  mxopt_ctx* ctx = e->ctx;
  mxopt_grad_prep prep = no_prep();
  prep.has_pre_mul = 1;
  prep.pre_mul = (float)(1.0 / (double)count);  // mul_scalar(scale): float64, then one cast
  int rc;
  *measured = false;
  if (e->cfg.has_gradient_clip_norm) {
    if (!norm_ready) {
      std::vector<mxopt_tensor> rows;
      for (Slot& s : e->slots) {
        if (!s.in_acc) continue;
        mxopt_tensor r = blank_tensor();
        r.g_out = s.acc; r.g_out_dtype = (uint8_t)s.acc_dtype; r.n = s.param.n;
        rows.push_back(r);
      }
      if (!rows.empty()) {
        mxopt_table* t = nullptr;
        if ((rc = cached_table(ctx, rows, &t))) return rc;
        if ((rc = mxopt_global_norm(ctx, t, 1, &prep, e->cfg.gradient_clip_norm, MXOPT_CLIP_ALWAYS_MULTIPLY,
                                    e->d_result)))
          return rc;
        norm_ready = true;
      }
    }
    if (norm_ready) {
      prep.d_scale = &e->d_result->scale;
      if (out) {  // only a caller that wants the figures pays for the read-back
        if ((rc = mxopt_read_norm_result(ctx, e->d_result, h_out))) return rc;
        *measured = true;
      }
    }
  }
  if (e->cfg.has_gradient_clip_value) {
    prep.has_clamp_post = 1;
    prep.post_lo = (float)(-e->cfg.gradient_clip_value);
    prep.post_hi = (float)e->cfg.gradient_clip_value;
  }
  if ((rc = apply_accumulated(e, e->cfg.learning_rate, e->cfg.weight_decay, prep))) return rc;
  end_cycle(e);
  e->step += 1;
  return MXOPT_OK;
}

// The boundary of sft_apply over held micro-batches: average by `count`, clip by the norm of the
// averaged sum, clamp, decay, update -- the sum itself is formed in registers by both passes.
int sft_apply_deferred(mxopt_engine* e, int32_t count, mxopt_engine_metrics* out, mxopt_norm_result* h_out,
                       bool* measured) {
  mxopt_ctx* ctx = e->ctx;
  *measured = false;
  int rc = MXOPT_OK;
  if (!e->held_slots.empty()) {
    mxopt_grad_prep prep = no_prep();
    prep.has_pre_mul = 1;
    prep.pre_mul = (float)(1.0 / (double)count);  // mul_scalar(scale): float64, then one cast
    if (e->cfg.has_gradient_clip_value) {
      prep.has_clamp_post = 1;
      prep.post_lo = (float)(-e->cfg.gradient_clip_value);
      prep.post_hi = (float)e->cfg.gradient_clip_value;
    }
    const bool clip = e->cfg.has_gradient_clip_norm != 0;
    if (e->cfg.apply == MXOPT_ENGINE_APPLY_ADAMW) {
      const size_t n = e->held_slots.size(), k = e->held.size();
      std::vector<const char*> names(n);
      std::vector<mxopt_array> params(n), grads(k * n);
      for (size_t c = 0; c < n; ++c) {
        const Slot& s = e->slots[e->held_slots[c]];
        names[c] = s.name.c_str();
        params[c] = s.param;
        for (size_t j = 0; j < k; ++j) grads[j * n + c] = e->held[j][c];
      }
      rc = mxopt_optimizer_update_many_accumulated(e->adamw, n, names.data(), params.data(), k, grads.data(),
                                                   params.data(), &prep, clip ? e->cfg.gradient_clip_norm : -1.0,
                                                   MXOPT_CLIP_ALWAYS_MULTIPLY, e->d_result);
    } else {
      mxopt_table* t = nullptr;
      if ((rc = defer_table(e, &t))) return rc;
      if (clip) {
        rc = mxopt_norm_with_pending_list(ctx, t, &prep, e->cfg.gradient_clip_norm, MXOPT_CLIP_ALWAYS_MULTIPLY,
                                          e->d_result);
        prep.d_scale = &e->d_result->scale;
      }
      if (!rc) rc = mxopt_sgd_plain_with_pending_list(ctx, t, e->cfg.learning_rate, e->cfg.weight_decay, &prep);
      (void)mxopt_table_set_pending(t, 0, nullptr, 0);
    }
    if (rc) return rc;
    if (clip && out) {
      if ((rc = mxopt_read_norm_result(ctx, e->d_result, h_out))) return rc;
      *measured = true;
    }
  }
  end_cycle(e);
  e->step += 1;
  return MXOPT_OK;
}

int sft_micro_batch(mxopt_engine* e, const std::vector<size_t>& idx, const mxopt_array* grads,
                    mxopt_engine_metrics* out) {
  mxopt_ctx* ctx = e->ctx;
  const size_t n = idx.size();
  e->consecutive_nan_count = 0;  // sft/engine.rs:261-267
  if (e->cfg.defer_accumulation) {
    int rc;
    if (e->held.size() > (size_t)MXOPT_MAX_PENDING && (rc = defer_spill(e))) return rc;
    if ((rc = defer_record(e, idx, grads))) return rc;
    e->held_result.push_back(-1);
    e->have_acc = true;
    e->micro_step += 1;
    int applied = 0;
    mxopt_norm_result h;
    bool measured = false;
    if (e->micro_step >= acc_steps(e)) {
      if ((rc = sft_apply_deferred(e, acc_steps(e), out, &h, &measured))) return rc;
      applied = 1;
    }
    fill_metrics(e, out, applied, 0);
    if (measured) add_norm(out, h);
    return MXOPT_OK;
  }
  const bool first_cycle_step = !e->have_acc;
  if (first_cycle_step)
    for (Slot& s : e->slots) s.in_acc = false;  // also after a call that failed half way
  const int32_t N = acc_steps(e);
  const bool boundary = e->micro_step + 1 >= N;
  const bool direct = boundary && first_cycle_step;  // N = 1: no accumulator is needed at all
  std::vector<mxopt_tensor> rows;
  int rc;
  size_t held = 0;
  for (const Slot& s : e->slots) held += s.in_acc ? 1 : 0;
  for (size_t i = 0; i < n; ++i) {
    Slot& s = e->slots[idx[i]];
    if (!first_cycle_step && !s.in_acc) continue;  // sft/engine.rs:283-287: silently dropped
    const int want = e->cfg.accumulate_in_f32 ? MXOPT_F32 : grads[i].dtype;
    if (first_cycle_step) {
      if (s.in_acc) continue;  // the same name twice in one call: the map keeps one
      if (!direct && (rc = ensure_acc(e, s, want))) return rc;
      s.in_acc = true;
    } else if (s.acc_dtype != want && !(s.acc_dtype == MXOPT_F32)) {
      return fail(ctx, MXOPT_ERR_INVALID_ARG,
                  "engine: gradient '" + s.name + "' changed dtype inside an accumulation cycle");
    }
    mxopt_tensor r = blank_tensor();
    r.g = grads[i].data; r.g_dtype = (uint8_t)grads[i].dtype;
    if (!direct) { r.g_out = s.acc; r.g_out_dtype = (uint8_t)s.acc_dtype; }
    r.n = grads[i].n;
    rows.push_back(r);
  }
  if (first_cycle_step) held = rows.size();

  // Last micro-batch of the cycle, every held tensor has a gradient in it: the sum acc + g is formed
  // in registers by the norm pass and again by the update, instead of being written back and read
  // twice.  With no accumulator yet (N = 1) the gradient is applied straight from where it lies.
  bool all_f32 = true;
  for (const mxopt_tensor& r : rows) all_f32 = all_f32 && r.g_out_dtype == MXOPT_F32;
  const bool pending = boundary && !first_cycle_step && e->cfg.apply == MXOPT_ENGINE_APPLY_SGD && all_f32 &&
                       rows.size() == held;
  if ((direct || pending) && !rows.empty()) {
    mxopt_grad_prep prep = no_prep();
    prep.has_pre_mul = 1;
    prep.pre_mul = (float)(1.0 / (double)N);  // mul_scalar(scale): float64, then one cast
    mxopt_table* t = nullptr;
    mxopt_norm_result h;
    bool measured = false;
    if (e->cfg.has_gradient_clip_norm) {
      if ((rc = cached_table(ctx, rows, &t))) return rc;
      rc = direct ? mxopt_global_norm(ctx, t, 0, &prep, e->cfg.gradient_clip_norm, MXOPT_CLIP_ALWAYS_MULTIPLY, e->d_result)
                  : mxopt_accumulate_norm_only(ctx, t, &prep, e->cfg.gradient_clip_norm, MXOPT_CLIP_ALWAYS_MULTIPLY,
                                               e->d_result);
      if (rc) return rc;
      prep.d_scale = &e->d_result->scale;
      if (out) {
        if ((rc = mxopt_read_norm_result(ctx, e->d_result, &h))) return rc;
        measured = true;
      }
    }
    if (e->cfg.has_gradient_clip_value) {
      prep.has_clamp_post = 1;
      prep.post_lo = (float)(-e->cfg.gradient_clip_value);
      prep.post_hi = (float)e->cfg.gradient_clip_value;
    }
    std::vector<mxopt_tensor> urows;
    std::vector<const char*> unames;
    std::vector<mxopt_array> uparams, ugrads;
    size_t k = 0;
    for (size_t i = 0; i < n && k < rows.size(); ++i) {
      Slot& s = e->slots[idx[i]];
      if (rows[k].g != grads[i].data || !s.in_acc) continue;  // rows follow the batch order, minus dropped names
      mxopt_tensor r = blank_tensor();
      r.p = s.param.data; r.p_out = s.param.data;
      r.p_dtype = r.p_out_dtype = (uint8_t)s.param.dtype;
      r.n = s.param.n;
      if (direct) {
        r.g = grads[i].data; r.g_dtype = (uint8_t)grads[i].dtype;
      } else {
        r.g = s.acc; r.g_dtype = MXOPT_F32;
        r.g_out = grads[i].data; r.g_out_dtype = (uint8_t)grads[i].dtype;
      }
      urows.push_back(r);
      unames.push_back(s.name.c_str());
      uparams.push_back(s.param);
      ugrads.push_back(grads[i]);
      ++k;
    }
    if (e->cfg.apply == MXOPT_ENGINE_APPLY_ADAMW) {  // direct only
      rc = mxopt_optimizer_update_many(e->adamw, unames.size(), unames.data(), uparams.data(), ugrads.data(),
                                       uparams.data(), &prep);
    } else {
      if ((rc = cached_table(ctx, urows, &t))) return rc;
      rc = direct ? mxopt_sgd_plain(ctx, t, e->cfg.learning_rate, e->cfg.weight_decay, &prep)
                  : mxopt_sgd_plain_with_pending(ctx, t, e->cfg.learning_rate, e->cfg.weight_decay, &prep, 1);
    }
    if (rc) return rc;
    end_cycle(e);
    e->step += 1;
    fill_metrics(e, out, 1, 0);
    if (measured) add_norm(out, h);
    return MXOPT_OK;
  }
  // The norm of acc/N rides on the last accumulation pass when that pass touches every held tensor.
  const bool fuse_norm = boundary && e->cfg.has_gradient_clip_norm && !rows.empty() && rows.size() == held;
  if (!rows.empty()) {
    mxopt_table* t = nullptr;
    if ((rc = cached_table(ctx, rows, &t))) return rc;
    mxopt_grad_prep prep = no_prep();
    prep.has_pre_mul = 1;
    prep.pre_mul = (float)(1.0 / (double)N);
    rc = mxopt_accumulate(ctx, t, first_cycle_step ? 1 : 0, fuse_norm ? &prep : nullptr,
                          fuse_norm ? e->cfg.gradient_clip_norm : -1.0, MXOPT_CLIP_ALWAYS_MULTIPLY,
                          fuse_norm ? e->d_result : nullptr);
    if (rc) return rc;
  }
  e->have_acc = true;  // Some(map), possibly empty
  e->micro_step += 1;
  int applied = 0;
  mxopt_norm_result h;
  bool measured = false;
  if (boundary) {
    if ((rc = sft_apply(e, N, fuse_norm, out, &h, &measured))) return rc;
    applied = 1;
  }
  fill_metrics(e, out, applied, 0);
  if (measured) add_norm(out, h);
  return MXOPT_OK;
}

}  // namespace

extern "C" {

void mxopt_engine_config_default(int32_t kind, mxopt_engine_config* c) {
  if (!c) return;
  std::memset(c, 0, sizeof *c);
  c->kind = kind;
  c->gradient_accumulation_steps = 1;
  c->has_gradient_clip_norm = 1;
  c->gradient_clip_norm = 1.0;
  c->max_nan_gradients = 100;
  c->emergency_save_threshold = 5;
  c->apply = MXOPT_ENGINE_APPLY_SGD;
  c->beta1 = 0.9; c->beta2 = 0.999; c->eps = 1e-8;
  if (kind == MXOPT_ENGINE_SFT) {  // sft/engine.rs:50-66
    c->learning_rate = 2e-5;
    c->weight_decay = 0.01;
  } else {                         // grpo/engine.rs:114-141
    c->learning_rate = 1e-6;
    c->has_gradient_clip_value = 1;
    c->gradient_clip_value = 1.0;
  }
}

int mxopt_engine_new(mxopt_ctx* ctx, const mxopt_engine_config* config, size_t n, const char* const* names,
                     const mxopt_array* params, mxopt_engine** out) {
  if (!ctx || !config || !out || (n && (!names || !params)))
    return fail(ctx, MXOPT_ERR_INVALID_ARG, "mxopt_engine_new: null argument");
  *out = nullptr;
  if (config->kind != MXOPT_ENGINE_GRPO && config->kind != MXOPT_ENGINE_SFT)
    return fail(ctx, MXOPT_ERR_INVALID_ARG, "mxopt_engine_new: unknown engine kind");
  if (config->apply != MXOPT_ENGINE_APPLY_SGD && config->apply != MXOPT_ENGINE_APPLY_ADAMW)
    return fail(ctx, MXOPT_ERR_INVALID_ARG, "mxopt_engine_new: unknown apply mode");
  if (config->defer_accumulation) {
    if (config->kind == MXOPT_ENGINE_SFT && !config->accumulate_in_f32)
      return fail(ctx, MXOPT_ERR_INVALID_ARG, "mxopt_engine_new: defer_accumulation adds in float32 (set accumulate_in_f32)");
    if (config->kind == MXOPT_ENGINE_GRPO && config->apply != MXOPT_ENGINE_APPLY_SGD)
      return fail(ctx, MXOPT_ERR_INVALID_ARG, "mxopt_engine_new: defer_accumulation in the GRPO engine applies plain SGD only");
  }
  mxopt_engine* e = new (std::nothrow) mxopt_engine();
  if (!e) return fail(ctx, MXOPT_ERR_OOM, "mxopt_engine_new: out of host memory");
  e->ctx = ctx;
  e->cfg = *config;
  e->slots.resize(n);
  for (size_t i = 0; i < n; ++i) {
    int rc = names[i] ? check_array(ctx, &params[i], "mxopt_engine_new: parameter")
                      : fail(ctx, MXOPT_ERR_INVALID_ARG, "mxopt_engine_new: null parameter name");
    if (!rc && !e->index.emplace(names[i], i).second)
      rc = fail(ctx, MXOPT_ERR_INVALID_ARG, std::string("mxopt_engine_new: duplicate parameter '") + names[i] + "'");
    if (rc) {
      delete e;
      return rc;
    }
    e->slots[i].name = names[i];
    e->slots[i].param = params[i];
  }
  int rc = MXOPT_OK;
  {
    DeviceGuard guard(ctx->device);
    // one slot per micro-batch a deferred cycle can hold and one for the arriving one; slot 0 serves everything else
    hipError_t err = hipMalloc((void**)&e->d_result, kResultSlots * sizeof(mxopt_norm_result));
    if (err != hipSuccess) rc = hip_fail(ctx, err, "mxopt_engine_new: hipMalloc");
  }
  if (!rc && config->apply == MXOPT_ENGINE_APPLY_ADAMW) {
    const int no_bias_correction = 0;  // the reference's default (adamw.rs:57)
    rc = mxopt_adamw_new(ctx, &config->learning_rate, &config->beta1, &config->beta2, &config->eps,
                         &config->weight_decay, &no_bias_correction, &e->adamw);
  }
  if (rc) {
    mxopt_engine_free(e);
    return rc;
  }
  *out = e;
  return MXOPT_OK;
}

void mxopt_engine_free(mxopt_engine* e) {
  if (!e) return;
  DeviceGuard guard(e->ctx->device);
  (void)hipStreamSynchronize(e->ctx->stream);
  for (Slot& s : e->slots)
    state_free(e->ctx, s.acc);
  if (e->d_result) (void)hipFree(e->d_result);
  if (e->h_pinned) (void)hipHostFree(e->h_pinned);
  if (e->copied) (void)hipEventDestroy(e->copied);
  if (e->adamw) mxopt_optimizer_free(e->adamw);
  delete e;
}

int mxopt_engine_micro_batch(mxopt_engine* e, size_t n, const char* const* names, const mxopt_array* grads,
                             mxopt_engine_metrics* out) {
  if (!e) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "mxopt_engine_micro_batch: null engine");
  int rc = settle(e, nullptr);
  if (rc) return rc;
  std::vector<size_t> idx;
  rc = resolve(e, n, names, grads, &idx);
  if (rc) return rc;
  return e->cfg.kind == MXOPT_ENGINE_GRPO ? grpo_micro_batch(e, idx, grads, out) : sft_micro_batch(e, idx, grads, out);
}

int mxopt_engine_micro_batch_async(mxopt_engine* e, size_t n, const char* const* names, const mxopt_array* grads) {
  const char* op = "mxopt_engine_micro_batch_async";
  if (!e) return fail(nullptr, MXOPT_ERR_INVALID_ARG, std::string(op) + ": null engine");
  mxopt_ctx* ctx = e->ctx;
  if (e->cfg.kind != MXOPT_ENGINE_GRPO)
    return fail(ctx, MXOPT_ERR_INVALID_ARG,
                std::string(op) + ": only the GRPO engine reads a flag back per micro-batch; the SFT engine does not "
                                  "block as it is");
  int rc = settle(e, nullptr);  // the previous micro-batch's flag has long arrived; a skip is booked now
  if (rc) return rc;
  std::vector<size_t> idx;
  if ((rc = resolve(e, n, names, grads, &idx))) return rc;
  if (!e->h_pinned) {
    DeviceGuard guard(ctx->device);
    HIP_TRY(ctx, hipHostMalloc((void**)&e->h_pinned, sizeof(mxopt_norm_result), hipHostMallocDefault));
    HIP_TRY(ctx, hipEventCreateWithFlags(&e->copied, hipEventDisableTiming));
  }
  mxopt_engine::Book before = take_book(e);
  e->async_mode = true;
  e->async_skip = nullptr;
  e->async_enqueued = false;
  e->async_book = &before;
  mxopt_engine_metrics m;
  rc = grpo_micro_batch(e, idx, grads, &m);
  const bool enqueued = e->async_enqueued;
  e->async_mode = false;
  e->async_skip = nullptr;
  e->async_enqueued = false;
  e->async_book = nullptr;
  if (rc) {
    // The call failed after its validity flag was asked for (a later check or a HIP error): the bookkeeping
    // goes back to where it was, and a micro-batch that held a NaN/Inf is still booked as the skip the
    // blocking call would have returned before it ever reached the failing step.
    if (enqueued) {
      const std::string why = ctx->err;
      put_book(e, before);
      bool bad = false;
      {
        DeviceGuard guard(ctx->device);
        bad = hipEventSynchronize(e->copied) == hipSuccess && (e->h_pinned->nonfinite & 1u) != 0;
      }
      if (bad) (void)grpo_skipped(e, nullptr);
      ctx->err = why;
    }
    return rc;
  }
  if (enqueued) {
    e->pending = true;
    e->pending_applied = m.gradients_applied;
    e->before = std::move(before);
  }
  return MXOPT_OK;
}

int mxopt_engine_settle(mxopt_engine* e, mxopt_engine_metrics* out) {
  if (!e) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "mxopt_engine_settle: null engine");
  return settle(e, out);
}

int mxopt_engine_flush_gradients(mxopt_engine* e, int* flushed, mxopt_engine_metrics* out) {
  if (!e) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "mxopt_engine_flush_gradients: null engine");
  if (e->cfg.kind != MXOPT_ENGINE_SFT)
    return fail(e->ctx, MXOPT_ERR_INVALID_ARG, "mxopt_engine_flush_gradients: only the SFT engine flushes");
  if (flushed) *flushed = 0;
  { int rc0 = settle(e, nullptr); if (rc0) return rc0; }
  if (e->micro_step == 0 || !e->have_acc) {  // sft/engine.rs:469-472
    fill_metrics(e, out, 0, 0);
    return MXOPT_OK;
  }
  mxopt_norm_result h;
  bool measured = false;
  int rc = e->cfg.defer_accumulation ? sft_apply_deferred(e, e->micro_step, out, &h, &measured)
                                     : sft_apply(e, e->micro_step, false, out, &h, &measured);
  if (rc) return rc;
  if (flushed) *flushed = 1;
  fill_metrics(e, out, 1, 0);
  if (measured) add_norm(out, h);
  return MXOPT_OK;
}

int mxopt_engine_report_nonfinite_loss(mxopt_engine* e, mxopt_engine_metrics* out) {
  if (!e) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "mxopt_engine_report_nonfinite_loss: null engine");
  { int rc0 = settle(e, nullptr); if (rc0) return rc0; }
  e->nan_gradient_count += 1;
  e->consecutive_nan_count += 1;
  if (e->consecutive_nan_count >= emergency_threshold(e)) e->needs_emergency_save = true;  // sft/engine.rs:228-235
  fill_metrics(e, out, 0, 1);
  if (e->nan_gradient_count >= max_nan(e))                                                  // sft/engine.rs:237-243
    return fail(e->ctx, MXOPT_ERR_FAILURE,
                "Training stopped: exceeded " + std::to_string(max_nan(e)) + " NaN gradient limit");
  return MXOPT_OK;
}

int mxopt_engine_get_metrics(const mxopt_engine* e, mxopt_engine_metrics* out) {
  if (!e || !out) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "mxopt_engine_get_metrics: null argument");
  if (e->pending) {  // the counters are only final once the last async micro-batch's flag has been seen
    int rc = settle(const_cast<mxopt_engine*>(e), nullptr);
    if (rc) return rc;
  }
  fill_metrics(e, out, 0, 0);
  return MXOPT_OK;
}

int mxopt_engine_clear_emergency_save_flag(mxopt_engine* e) {
  if (!e) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "mxopt_engine_clear_emergency_save_flag: null engine");
  { int rc0 = settle(e, nullptr); if (rc0) return rc0; }
  e->needs_emergency_save = false;
  return MXOPT_OK;
}

int mxopt_engine_reset(mxopt_engine* e) {
  if (!e) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "mxopt_engine_reset: null engine");
  if (e->pending) {  // whatever the flag says, everything is forgotten below
    DeviceGuard guard(e->ctx->device);
    (void)hipEventSynchronize(e->copied);
    e->pending = false;
  }
  for (Slot& s : e->slots) s.in_acc = false;
  e->have_acc = false;
  e->held.clear();
  e->held_slots.clear();
  e->held_result.clear();
  e->held_is_sum = false;
  e->micro_step = 0;
  e->step = 0;
  e->nan_gradient_count = 0;
  e->consecutive_nan_count = 0;
  e->needs_emergency_save = false;
  if (e->adamw) return mxopt_optimizer_reset(e->adamw);
  return MXOPT_OK;
}

int mxopt_engine_save_optimizer_state(mxopt_engine* e, const char* path) {
  if (!e) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "mxopt_engine_save_optimizer_state: null engine");
  if (!e->adamw) return fail(e->ctx, MXOPT_ERR_INVALID_ARG, "this engine applies plain SGD: there is no optimizer state");
  // An async micro-batch that is still unsettled has advanced the AdamW call counter as if it were valid:
  // the file must hold the counter of the updates the device really made.
  { int rc0 = settle(e, nullptr); if (rc0) return rc0; }
  return mxopt_optimizer_save_file(e->adamw, path);
}

int mxopt_engine_load_optimizer_state(mxopt_engine* e, const char* path) {
  if (!e) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "mxopt_engine_load_optimizer_state: null engine");
  if (!e->adamw) return fail(e->ctx, MXOPT_ERR_INVALID_ARG, "this engine applies plain SGD: there is no optimizer state");
  // Settled first: a later settle would otherwise write the counter of before the pending call over the loaded one.
  { int rc0 = settle(e, nullptr); if (rc0) return rc0; }
  return mxopt_optimizer_load_file(e->adamw, path);
}

}  // extern "C"
