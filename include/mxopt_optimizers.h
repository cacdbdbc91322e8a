/* mxopt host layer: the reference's optimizer objects and gradient utilities over raw device
 * buffers, C ABI.
 *
 * These entry points carry the *semantics* of the reference's Rust API (state keyed by
 * parameter name, per-call step counter, lazy state creation, reset, error cases) so that the
 * Rust methods shrink to "extract (ptr, n, dtype) from the MxArray handles, call, wrap the
 * output buffer".  Each one names the method it stands behind.  The arithmetic is done by the
 * kernels declared in mxopt.h.
 *
 * Arrays cross the boundary as mxopt_array = what the host extracts from an MxArray
 * (crates/mlx-core/src/array/mod.rs:28-82): a dense device buffer, an element count and the
 * reference's dtype code.  Outputs are allocated by the caller (the reference returns a fresh
 * array from every op, crates/mlx-sys/src/mlx.cpp:497-547); an output may alias its input for
 * an in-place update.  Optimizer state (m, v, velocity) is float32, owned by the optimizer
 * object, created zero-filled on the first update of a name (adamw.rs:152-157,
 * array/mod.rs:115-119) and released by reset / free.
 *
 * Optional arguments of the reference (Option<f64>, Option<bool>) are nullable pointers.
 * Nothing here synchronises with the host unless a result is returned by value
 * (a norm as double).  Work is enqueued on the context's stream ("lazy until eval").
 */
#ifndef MXOPT_OPTIMIZERS_H
#define MXOPT_OPTIMIZERS_H

#include "mxopt.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mxopt_array {
  void*    data;  /* device pointer; NULL only where an entry may be absent */
  uint64_t n;     /* elements */
  int32_t  dtype; /* MXOPT_F32 / MXOPT_F16 / MXOPT_BF16 */
} mxopt_array;

typedef struct mxopt_optimizer mxopt_optimizer;

/* ---- constructors ----------------------------------------------------------------- */
/* Adam::new (optimizers/adam.rs:41-57): defaults lr 1e-3, betas (0.9, 0.999), eps 1e-8,
 * bias_correction false. */
int mxopt_adam_new(mxopt_ctx* ctx, const double* learning_rate, const double* beta1, const double* beta2,
                   const double* eps, const int* bias_correction, mxopt_optimizer** out);
/* AdamW::new (optimizers/adamw.rs:43-61): as Adam plus weight_decay, default 0.01. */
int mxopt_adamw_new(mxopt_ctx* ctx, const double* learning_rate, const double* beta1, const double* beta2,
                    const double* eps, const double* weight_decay, const int* bias_correction,
                    mxopt_optimizer** out);
/* SGD::new (optimizers/sgd.rs:40-67): learning_rate required; momentum, weight_decay, dampening
 * default 0, nesterov false.  MXOPT_ERR_INVALID_ARG "Nesterov momentum requires momentum > 0 and
 * dampening = 0" (sgd.rs:51-56). */
int mxopt_sgd_new(mxopt_ctx* ctx, double learning_rate, const double* momentum, const double* weight_decay,
                  const double* dampening, const int* nesterov, mxopt_optimizer** out);
/* RMSprop::new (optimizers/rmsprop.rs:36-50): defaults lr 1e-2, alpha 0.99, eps 1e-8, wd 0. */
int mxopt_rmsprop_new(mxopt_ctx* ctx, const double* learning_rate, const double* alpha, const double* eps,
                      const double* weight_decay, mxopt_optimizer** out);
void mxopt_optimizer_free(mxopt_optimizer* opt);

/* ---- update_single / reset -------------------------------------------------------- */
/* {Adam,AdamW,SGD,RMSprop}::update_single(param_name, param, grad) -> new param
 * (adam.rs:61-140, adamw.rs:65-143, sgd.rs:70-153, rmsprop.rs:53-116).
 * `out` receives the new parameter: dtype MXOPT_F32 reproduces the reference (which never
 * casts back, so bf16 inputs yield float32), dtype == param->dtype gives one round-to-nearest-
 * even write-back; out->data may equal param->data.  Increments the optimizer's call counter
 * (Adam/AdamW) exactly like the reference: once per call, shared by all names.
 * One kernel launch, no allocation after the first call for a name, no host synchronisation. */
int mxopt_optimizer_update_single(mxopt_optimizer* opt, const char* param_name, const mxopt_array* param,
                                  const mxopt_array* grad, const mxopt_array* out);

/* The same as calling update_single for i = 0 .. n-1 in that order (so with bias correction
 * tensor i sees t = step + i + 1), but one launch per dtype group for the whole list.  The
 * table is cached while the same buffers are passed.  `prep` (nullable) applies fused gradient
 * pre-processing (clip scale etc.).  SGD with momentum refuses prep->d_skip_if_nonzero while a
 * parameter of the list has no velocity yet: the first step stores it, and the host cannot know
 * afterwards whether a conditional one ran.  No counterpart in the reference; it is what its
 * callers' `for (name, param) in params { opt.update_single(..) }` loops collapse into. */
int mxopt_optimizer_update_many(mxopt_optimizer* opt, size_t n, const char* const* param_names,
                                const mxopt_array* params, const mxopt_array* grads, const mxopt_array* outs,
                                const mxopt_grad_prep* prep);

/* update_many over k micro-batches that were never summed (deferred accumulation, see mxopt.h):
 * the gradient of parameter i is grads[i] + grads[n + i] + ... + grads[(k-1) n + i], added left to
 * right in float32 -- the sum k-1 calls of Qwen3Model::accumulate_gradients (model.rs:2217-2243)
 * would have left in a float32 buffer -- then `prep`, then, when max_norm >= 0, the clip factor of
 * GradientUtils::clip_grad_norm (optimizers/mod.rs:67-107; clip_mode as in mxopt_global_norm) of
 * that gradient's global norm, then the optimizer's own update (any of the four kinds) with
 * update_many's per-call step counting.  Two launches per dtype group, no accumulation buffer,
 * no host synchronisation.  k >= 1; with k = 1, no prep and no clip nothing is added or multiplied and
 * the call is update_many (the lone gradient reaches the optimizer in its own dtype, so a 16-bit
 * gradient's square is 16-bit there, mlx.cpp:2016-2020).  The kernels read MXOPT_MAX_PENDING + 1 streams: with a larger
 * k the oldest micro-batches are first added, in order, into a float32 buffer per parameter that
 * the optimizer keeps with its state (4 B/elem, freed by reset), and that buffer stands in for
 * them.  Of the streams the kernels read, the second to the last share one dtype and the first has
 * it or is float32; outs[i] has params[i]'s dtype (it may be params[i] itself).
 * d_norm (nullable, device memory) receives norm, clip factor and the non-finite flag; pass
 * prep->d_skip_if_nonzero = &d_norm->nonfinite to leave parameters and state untouched on a NaN/Inf
 * gradient.  The skip happens on the device: the host's call counter (Adam/AdamW bias correction)
 * advances all the same; a caller that must not count such a step reads d_norm and decides itself. */
int mxopt_optimizer_update_many_accumulated(mxopt_optimizer* opt, size_t n, const char* const* param_names,
                                            const mxopt_array* params, size_t k, const mxopt_array* grads,
                                            const mxopt_array* outs, const mxopt_grad_prep* prep, double max_norm,
                                            int clip_mode, mxopt_norm_result* d_norm);

/* reset(): drops all state; Adam/AdamW also zero the call counter (adam.rs:143-146,
 * adamw.rs:146-150, sgd.rs:157-159, rmsprop.rs:119-121). */
int mxopt_optimizer_reset(mxopt_optimizer* opt);
/* The call counter `step` (0 for SGD/RMSprop). */
int64_t mxopt_optimizer_step_count(const mxopt_optimizer* opt);
/* Device pointers to the state of `param_name` (for checkpointing and tests): m is NULL for
 * SGD/RMSprop; both NULL (and *n = 0) when the name has no state yet.  has_velocity tells
 * whether SGD's velocity has been written (false before the first momentum step). */
int mxopt_optimizer_state(mxopt_optimizer* opt, const char* param_name, float** m, float** v, uint64_t* n,
                          int* has_velocity);
/* Copies the state of `param_name` into caller-owned device buffers of *n floats each (either may
 * be NULL), on the context's stream: the "save" half of an optimizer-state checkpoint. */
int mxopt_optimizer_save_state(mxopt_optimizer* opt, const char* param_name, float* m_dst, float* v_dst);
/* Restores state saved with mxopt_optimizer_state / mxopt_optimizer_save_state (device-to-device copy into owned buffers). */
int mxopt_optimizer_load_state(mxopt_optimizer* opt, const char* param_name, const float* m, const float* v,
                               uint64_t n, int64_t step_count);

/* Optimizer-state checkpoint on disk, in the safetensors layout of the reference's own writer
 * (crates/mlx-core/src/utils/safetensors.rs:312-385): tensors "<param_name>.m" / "<param_name>.v",
 * float32, shape [elements], sorted by name; __metadata__ carries the optimizer kind and the call
 * counter `step`.  The reference saves no optimizer state at all (saveCheckpoint,
 * packages/trl/src/trainers/grpo-trainer.ts:1146-1206 writes the model only), so resuming there
 * restarts the moments from zero.  Both calls synchronise the context's stream; load replaces the
 * optimizer's current state and refuses a file written for another optimizer kind. */
int mxopt_optimizer_save_file(mxopt_optimizer* opt, const char* path);
int mxopt_optimizer_load_file(mxopt_optimizer* opt, const char* path);
/* Host-only look at a checkpoint (no device, no optimizer needed): which optimizer kind wrote it
 * ("adam", "adamw", "sgd", "rmsprop"), its call counter, how many tensors and float32 elements it
 * holds.  Fails like load_file on anything that is not a well-formed checkpoint.  Any out pointer
 * may be NULL. */
int mxopt_checkpoint_inspect(const char* path, char* optimizer, size_t optimizer_capacity, int64_t* step,
                             uint64_t* tensors, uint64_t* elements);

/* ---- GradientUtils (optimizers/mod.rs:33-227) -------------------------------------- */
/* compute_gradient_norm (:43-55): sqrt of the float64 sum of squares.  Synchronises. */
int mxopt_compute_gradient_norm(mxopt_ctx* ctx, size_t n, const mxopt_array* grads, double* norm_out);
/* clip_grad_norm (:67-107) and clip_grad_norm_with_norm (:116-158): outs[i] = grads[i] * scale with
 * scale = min(f32(max_norm) / (norm + f32(1e-6)), 1).  n == 0 is legal (norm 0).  If norm_out is
 * not NULL the float32 norm is returned as double and the call synchronises (the reference
 * evaluates and reads one scalar there, :137-138); with NULL nothing synchronises.
 * outs[i].dtype: MXOPT_F32 (MLX promotes bf16 * float32 scalar) or the gradient's dtype. */
int mxopt_clip_grad_norm(mxopt_ctx* ctx, size_t n, const mxopt_array* grads, double max_norm,
                         const mxopt_array* outs, double* norm_out);
/* clip_grad_value (:164-166): clamp to [f32(min_val), f32(max_val)]; a non-finite bound is no bound. */
int mxopt_clip_grad_value(mxopt_ctx* ctx, const mxopt_array* grad, double min_val, double max_val,
                          const mxopt_array* out);
/* clip_grad_value_and_norm (:174-226): clamp to +-clip_value, then (if max_norm != NULL) the
 * clip_grad_norm of the clamped values. */
int mxopt_clip_grad_value_and_norm(mxopt_ctx* ctx, size_t n, const mxopt_array* grads, double clip_value,
                                   const double* max_norm, const mxopt_array* outs);

/* ---- gradients/mod.rs Vec API -------------------------------------------------------- */
/* clip_gradients_by_global_norm (gradients/mod.rs:233-285): float64 norm; outs = unchanged copies
 * when norm <= max_norm, else grads * f32(max_norm / (norm + 1e-6)).  No synchronisation (the
 * comparison is made on the device). */
int mxopt_clip_gradients_by_global_norm(mxopt_ctx* ctx, size_t n, const mxopt_array* grads, double max_norm,
                                        const mxopt_array* outs);
/* clip_gradients_by_value (gradients/mod.rs:299-312). */
int mxopt_clip_gradients_by_value(mxopt_ctx* ctx, size_t n, const mxopt_array* grads, double min_value,
                                  double max_value, const mxopt_array* outs);

/* ---- accumulation and plain-SGD apply ------------------------------------------------ */
/* The element-wise part of Qwen3Model::accumulate_gradients (models/qwen3/model.rs:2217-2243),
 * the engines' accumulate_gradients (grpo/engine.rs:2632-2666) and the SFT engine's inline sum
 * (sft/engine.rs:282-290): outs[i] = acc[i] + new_grads[i] in the promoted dtype, or a copy of
 * new_grads[i] where acc[i].data is NULL (first micro-batch).  Which names exist on which side
 * is the host map's business.  outs[i] may alias acc[i]. */
int mxopt_accumulate_gradients(mxopt_ctx* ctx, size_t n, const mxopt_array* acc, const mxopt_array* new_grads,
                               const mxopt_array* outs);
/* Qwen3Model::apply_gradients (models/qwen3/model.rs:2409-2460), element-wise part: params[i] updated
 * to astype(p - astype(lr, dtype p) * g, dtype p); outs[i] may alias params[i].  The lookup of
 * names and the "Parameter '..' not found in model" error (:2427-2432) stay with the host map. */
int mxopt_apply_gradients(mxopt_ctx* ctx, size_t n, const mxopt_array* params, const mxopt_array* grads,
                          double learning_rate, const mxopt_array* outs);

/* ---- LRScheduler (optimizers/mod.rs:239-292): host float64 closed forms ---------------- */
double mxopt_lr_linear_decay(double initial_lr, double final_lr, int64_t current_step, int64_t total_steps);
double mxopt_lr_exponential_decay(double initial_lr, double decay_rate, int64_t current_step, int64_t decay_steps);
double mxopt_lr_cosine_annealing(double initial_lr, double min_lr, int64_t current_step, int64_t total_steps);
double mxopt_lr_step_decay(double initial_lr, double factor, int64_t current_step, int64_t step_size);

#ifdef __cplusplus
}
#endif
#endif /* MXOPT_OPTIMIZERS_H */
