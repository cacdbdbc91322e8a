/* mxopt_engine.h -- the optimizer side of mlx-node's training engines over raw device buffers.
 *
 * What GRPOTrainingEngine and SftTrainingEngine do between the backward pass of a micro-batch
 * and the next forward pass: gradient validity, value clamp, global-norm clip, accumulation
 * over micro-batches, the parameter update, and the NaN / step bookkeeping around them
 *   crates/mlx-core/src/grpo/engine.rs:561-704 (and its siblings :1691-1790),
 *   crates/mlx-core/src/grpo/engine.rs:2632-2666 (accumulate_gradients),
 *   crates/mlx-core/src/sft/engine.rs:215-371 (train_step), :459-553 (flush_gradients).
 * The engines keep their public surface (train_step*, getters); these entry points replace the
 * bodies cited at each function.  Gradients and parameters are handed over as
 * mxopt_array {device pointer, elements, dtype code}; parameters are updated IN PLACE, which
 * makes Qwen3Model::apply_gradients' per-name setters (models/qwen3/model.rs:2484-2528) a no-op.
 *
 * Per micro-batch the GRPO engine costs one read of the gradients (validity + norm of the
 * clamped values in one pass), one read-modify-write of the float32 accumulation buffer, and
 * one 32-byte read-back (none with mxopt_engine_micro_batch_async); nothing else leaves the device.
 */
#ifndef MXOPT_ENGINE_H
#define MXOPT_ENGINE_H

#include "mxopt_optimizers.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mxopt_engine mxopt_engine;

enum { MXOPT_ENGINE_GRPO = 0, MXOPT_ENGINE_SFT = 1 };
enum {
  MXOPT_ENGINE_APPLY_SGD = 0,  /* Qwen3Model::apply_gradients: what both engines run today */
  MXOPT_ENGINE_APPLY_ADAMW = 1 /* fused AdamW on the averaged, clipped gradient (no counterpart
                                  in the reference: the engines have no optimizer state) */
};

/* GRPOEngineConfig (grpo/engine.rs:59-141) / SftEngineConfig (sft/engine.rs:27-66), the fields
 * that reach the optimizer side.  A has_* flag of 0 is the reference's None. */
typedef struct mxopt_engine_config {
  int32_t kind;                        /* MXOPT_ENGINE_GRPO | MXOPT_ENGINE_SFT                  */
  int32_t gradient_accumulation_steps; /* < 1 is taken as 1                                      */
  double  learning_rate;
  int32_t has_gradient_clip_norm;
  double  gradient_clip_norm;
  int32_t has_gradient_clip_value;     /* GRPO: None means 1.0 (engine.rs:636); SFT: no clamp    */
  double  gradient_clip_value;
  double  weight_decay;                /* SFT + SGD: g += wd*p when > 0 (sft/engine.rs:345-365);
                                          ADAMW: decoupled decay; GRPO + SGD: unused              */
  int64_t max_nan_gradients;           /* < 1 is taken as 100                                     */
  int32_t emergency_save_threshold;    /* < 1 is taken as 5                                       */
  int32_t apply;                       /* MXOPT_ENGINE_APPLY_*                                    */
  double  beta1, beta2, eps;           /* ADAMW                                                   */
  int32_t accumulate_in_f32;           /* SFT: 0 = the reference's accumulator dtype (that of the
                                          gradients: bf16 + bf16 -> bf16), 1 = float32 buffer.
                                          GRPO accumulates clipped (float32) gradients either way */
  int32_t defer_accumulation;          /* 1 = no accumulation buffer: the engine only remembers where
                                          each micro-batch's gradients lie and the update adds them in
                                          registers (float32, arrival order: the numbers of the float32
                                          buffer, bit for bit).  The caller keeps every gradient buffer of
                                          a cycle alive and unchanged until the work that the applying call
                                          (or flush_gradients / reset) enqueued on the context's stream has
                                          completed -- the call returning is not enough: it only enqueues --
                                          or orders any reuse of the memory after it on that stream.  With more than
                                          MXOPT_MAX_PENDING + 1 micro-batches in a cycle the oldest ones
                                          are added into a float32 buffer as the later ones arrive (their
                                          buffers are free again after that call); the last
                                          MXOPT_MAX_PENDING stay deferred.  Needs the same gradient names
                                          in every micro-batch of a cycle, SFT: accumulate_in_f32 = 1,
                                          GRPO: apply = SGD.  No counterpart in the reference. */
} mxopt_engine_config;

/* The reference's defaults for `kind` (GRPOEngineConfig::default, SftEngineConfig::default). */
void mxopt_engine_config_default(int32_t kind, mxopt_engine_config* out);

/* EngineStepMetrics / SftStepMetrics fields that come from the optimizer side, plus the getters
 * step / micro_step / nan_gradient_count / needs_emergency_save (grpo/engine.rs:2460-2600). */
typedef struct mxopt_engine_metrics {
  int64_t  step;
  int32_t  micro_step;
  int32_t  gradients_applied;
  int32_t  skipped;               /* this micro-batch held a NaN/Inf and was dropped (GRPO)       */
  int32_t  needs_emergency_save;
  uint32_t consecutive_nan_count;
  uint64_t nan_gradient_count;
  int32_t  norm_measured;         /* 1 when the three fields below describe this call            */
  float    clip_scale;
  double   grad_sumsq;            /* GRPO: of the clamped micro-batch; SFT: of the averaged sum   */
  double   grad_norm;
} mxopt_engine_metrics;

/* `params`: the model's trainable parameters by name (Qwen3Model::get_parameters); the arrays
 * are borrowed for the engine's lifetime and updated in place. */
int mxopt_engine_new(mxopt_ctx* ctx, const mxopt_engine_config* config, size_t n, const char* const* names,
                     const mxopt_array* params, mxopt_engine** out);
void mxopt_engine_free(mxopt_engine* e);

/* One micro-batch of gradients.
 * GRPO (grpo/engine.rs:561-704): any NaN/Inf element => nothing is touched, the NaN counters
 *   advance, `step` advances, skipped = 1 (status MXOPT_ERR_FAILURE with the reference's
 *   "Training stopped" message once nan_gradient_count reaches max_nan_gradients); otherwise
 *   acc += clip_norm(clamp(g)), and every gradient_accumulation_steps-th accepted micro-batch
 *   p -= (lr/N) * acc.
 * SFT (sft/engine.rs:268-371): acc += g (names the accumulator does not hold are dropped);
 *   every N-th micro-batch p -= lr * (clamp(clip_norm(acc/N)) + wd*p).
 * A gradient whose name is not a parameter is refused before anything is touched with the
 * message of models/qwen3/model.rs:2427-2432 (the reference fails at apply time).
 * `out` may be NULL. */
int mxopt_engine_micro_batch(mxopt_engine* e, size_t n, const char* const* names, const mxopt_array* grads,
                             mxopt_engine_metrics* out);

/* mxopt_engine_micro_batch for the GRPO engine (either apply mode) without its one host synchronisation: the
 * blocking call reads the validity flag back (32 bytes) before it decides whether to accumulate, where
 * the reference reads every gradient back for the same test (grpo/engine.rs:563-569).  Here the flag
 * stays on the device: the norm pass writes it, every kernel of the call that would change memory
 * does nothing when it is set, and a copy of it is on its way to pinned host memory when the call
 * returns.  The host books the micro-batch as valid for the time being; the next engine call of any
 * kind (or mxopt_engine_settle) looks at the flag, which has long arrived by then, and if it was set
 * puts the bookkeeping back to what it was before that micro-batch and applies the reference's skip
 * (NaN counters, emergency flag, `step`).  Results -- parameters, buffers, counters -- are those of the
 * blocking calls.  Two differences in timing: metrics come from mxopt_engine_settle, and the
 * "Training stopped" failure of a micro-batch that reaches max_nan_gradients is returned by the call
 * that settles it.  With apply = ADAMW the optimizer's call counter goes back with the rest; moments
 * that a skipped first update allocated stay, zero-filled, which is what a later first update starts
 * from anyway.  With defer_accumulation the caller keeps a micro-batch's gradient buffers alive as for
 * the blocking call.  The SFT engine is refused: it reads nothing back unless the caller asks for
 * metrics. */
int mxopt_engine_micro_batch_async(mxopt_engine* e, size_t n, const char* const* names, const mxopt_array* grads);
/* Waits for the last async micro-batch's flag (a no-op after a blocking call) and returns the metrics the
 * blocking call would have returned for it.  `out` may be NULL. */
int mxopt_engine_settle(mxopt_engine* e, mxopt_engine_metrics* out);

/* SFT, sft/engine.rs:459-553: apply what has been accumulated, averaged over the micro-batches
 * actually seen.  *flushed = 0 when there was nothing to apply. */
int mxopt_engine_flush_gradients(mxopt_engine* e, int* flushed, mxopt_engine_metrics* out);

/* SFT, sft/engine.rs:221-258: the loss of this micro-batch was NaN/Inf; nothing is accumulated,
 * the NaN counters advance (status MXOPT_ERR_FAILURE once the limit is reached). */
int mxopt_engine_report_nonfinite_loss(mxopt_engine* e, mxopt_engine_metrics* out);

/* Getters, clear_emergency_save_flag (grpo/engine.rs:2591-2600) and reset (:2533-2546). */
int mxopt_engine_get_metrics(const mxopt_engine* e, mxopt_engine_metrics* out);
int mxopt_engine_clear_emergency_save_flag(mxopt_engine* e);
int mxopt_engine_reset(mxopt_engine* e);

/* MXOPT_ENGINE_APPLY_ADAMW only: the AdamW moments as a safetensors file
 * (mxopt_optimizer_save_file / mxopt_optimizer_load_file of the engine's optimizer). */
int mxopt_engine_save_optimizer_state(mxopt_engine* e, const char* path);
int mxopt_engine_load_optimizer_state(mxopt_engine* e, const char* path);

#ifdef __cplusplus
}
#endif
#endif /* MXOPT_ENGINE_H */
