/* mxopt -- MI355X (gfx950) kernels for the optimizer step of mlx-node, C ABI.
 *
 * This is the boundary a host (the reference's Rust crate `mlx-core`, or any other
 * caller) binds instead of building every optimizer out of ~13 lazy MLX element-wise
 * ops per tensor.  Every entry point takes plain pointers and sizes; device buffers
 * are owned by the caller and are never freed or retained beyond the lifetime of the
 * table that names them.  Nothing here allocates per call: a table (descriptors +
 * chunk list on the device) is built once for a parameter list and reused every step.
 *
 * All arithmetic is IEEE float32, one rounding per reference op, in the reference's
 * op order, so results are bit-identical to the reference's float32 op chain.
 * 16-bit tensors (bf16, f16) are widened on load and rounded to nearest-even once on
 * store.  Hyper-parameters cross the boundary ALREADY CAST to float32 the way the
 * reference casts them: evaluated in float64 on the host, then static_cast<float>
 * (crates/mlx-sys/src/mlx.cpp:335-338, 531-535); the *_hp_from_f64 helpers do that.
 *
 * Error convention: every call returns an int status (0 = ok), never throws or aborts
 * across the boundary, and leaves a message readable with mxopt_last_error()
 * (mirrors the reference's "null handle => Err(message)" idiom,
 * crates/mlx-core/src/array/handle.rs:4-16, and napi Status::{InvalidArg,GenericFailure}).
 *
 * Threading: calls on one context are serialised by the caller; different contexts
 * may be used from different threads.  Kernels are enqueued on the context's stream;
 * no call synchronises with the host except mxopt_synchronize / mxopt_read_*.
 *
 * Logging: the environment variable MXOPT_LOG (read once per process) = "error" prints every refused
 * call to stderr, "debug" also one line per launch group, table change and engine decision (the
 * counterpart of the reference's MLX_NODE_LOG filter, crates/mlx-core/src/tracing.rs:3-21).
 *
 * HIP graphs: the kernel entry points (mxopt_adam ... mxopt_norm_with_pending_list) only launch
 * kernels -- no allocation, copy or memset -- once the first reduction call on a context has
 * allocated its per-workgroup partials buffer, so a step may be recorded into a graph after
 * one eager warm-up call.  mxopt_table_build, mxopt_table_set_step_scalars, mxopt_table_retarget
 * and mxopt_table_set_pending copy from host memory and stay outside a capture.
 */
#ifndef MXOPT_H
#define MXOPT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dtype codes = the reference's DType enum (crates/mlx-core/src/array/mod.rs:17-26,
 * crates/mlx-sys/src/mlx.cpp:152-157).  Only the floating types are accepted. */
enum { MXOPT_F32 = 0, MXOPT_I32 = 1, MXOPT_F16 = 2, MXOPT_BF16 = 3, MXOPT_U32 = 4 };

enum {
  MXOPT_OK = 0,
  MXOPT_ERR_INVALID_ARG = 1, /* napi Status::InvalidArg (sgd.rs:51-56) */
  MXOPT_ERR_FAILURE = 2,     /* napi Status::GenericFailure (model.rs:2427-2432) */
  MXOPT_ERR_HIP = 3,         /* a HIP runtime call failed; message carries hipGetErrorString */
  MXOPT_ERR_OOM = 4
};

typedef struct mxopt_ctx mxopt_ctx;
typedef struct mxopt_table mxopt_table;

/* ---- context -------------------------------------------------------------------- */

/* One context per optimizer object / engine.  `hip_stream` is a hipStream_t (NULL = the
 * device's default stream).  Replaces nothing in the reference: MLX owns one implicit
 * device stream (crates/mlx-core/src/stream.rs). */
int mxopt_create(int device, void* hip_stream, mxopt_ctx** out);
void mxopt_destroy(mxopt_ctx* ctx);
/* Last error message of `ctx` (or of the calling thread when ctx is NULL). Never NULL. */
const char* mxopt_last_error(const mxopt_ctx* ctx);
/* Waits for everything enqueued on the context's stream (the reference's eval(),
 * crates/mlx-sys/src/mlx.cpp:189-209). */
int mxopt_synchronize(mxopt_ctx* ctx);
/* Tuning knobs, by name: "grid_blocks_per_cu" (persistent grid = CUs x this),
 * "persistent" (0: one workgroup per chunk for the update kernels), "persistent_accumulate" (1: the
 * persistent grid also for accumulation passes after the first that take no norm), "nontemporal" /
 * "nontemporal_reduce" (both 1 by default: streaming-hint memory instructions in the read-write / read-only
 * kernels -- on every load that fetches whole 32-byte sectors, and on stores to lines the kernel has read;
 * 0 = plain loads and stores; the list kernels of deferred accumulation always stream),
 * "pipelined_norm" (the plain norm of a 16-bit stream: 0 = the general reduction kernel always; 2 (default)
 * or 4 = a kernel that takes that many chunks per trip, for tables whose chunks are under 90 % full on
 * average, i.e. many small tensors; 1 = that kernel, two chunks per trip, for every table). */
int mxopt_set_option(mxopt_ctx* ctx, const char* name, int64_t value);
int mxopt_get_option(const mxopt_ctx* ctx, const char* name, int64_t* value);

/* ---- HBM placement (the older, luck-based way; see the region-interleaved pool below) -------------
 * Why placement matters at all is told at the pool: device memory consists of three physical regions and
 * a kernel that reads and writes wants its traffic in at least two of them.  This pair only raises the odds
 * of that for hosts that cannot route their allocations through a pool:
 *
 *   mxopt_hbm_spread_begin(ctx, 0, 0, &s);    all free device memory is taken in blocks, then two of
 *   ... allocate parameters, moments, ...      every three blocks are released: what is allocated now
 *   mxopt_hbm_spread_end(s);                   fills those gaps; end() releases the rest
 *
 * What is allocated in between lands in pieces all over the free memory instead of one compact run, which
 * usually -- not always, the driver decides -- means pieces of more than one region (measured over 17 fresh
 * processes on the Qwen3-8B list: 79.7 - 86.2 ms per step, against 84.6 - 85.8 ms without and 77.1 ms from
 * the pool).  block_bytes = 0: 64 MiB; keep_one_in = 0: every third block is kept (>= 2: every
 * keep_one_in-th).  Between the two calls about (1 - 1/keep_one_in) of the free memory can be allocated.
 * Both calls synchronise with the device and are meant for start-up, not for the training loop.  No
 * counterpart in the reference. */
typedef struct mxopt_hbm_spread mxopt_hbm_spread;
int mxopt_hbm_spread_begin(mxopt_ctx* ctx, size_t block_bytes, int keep_one_in, mxopt_hbm_spread** out);
int mxopt_hbm_spread_end(mxopt_hbm_spread* s);

/* ---- region-interleaved device memory ------------------------------------------------
 * Device memory on this part is made of three physical regions of 96 GiB.  A kernel that reads AND
 * writes (every update and accumulation kernel here) runs at about 5.3 TB/s when all it touches lies
 * in one region and at about 6.1 TB/s when its traffic is spread over two or three; read-only passes
 * do not care.  A process that allocates a few tens of GB from a fresh device gets one compact
 * physical run, i.e. one region.  Physical addresses cannot be asked for, so the pool finds the
 * regions by timing: it takes the free memory as physical chunks, runs a 4-read/3-write probe over
 * pairs of 1 GiB groups of them (slow = same region), maps an arena of `capacity_bytes` in which
 * consecutive chunks alternate between the regions found, and gives every chunk it does not need
 * back to the driver before it returns (about 1 - 3 s, once per process, at start-up; synchronises
 * with the device).  Whatever is allocated from the arena has its traffic spread over the regions,
 * whichever streams a kernel combines; this replaces the luck of mxopt_hbm_spread_begin/_end.
 * If all free memory lies in one region (regions == 1 in the info) the arena still works, without
 * the gain.  chunk_bytes = 0: 64 MiB (a power of two in [2 MiB, 1 GiB]; the free memory must make at
 * most 24 000 chunks, i.e. 16 MiB or more on an empty device).  max_regions = 0: alternate
 * between all regions found; 2: between the two with the most free memory (read-only passes lose about
 * 3 % on memory interleaved over two regions and 6 - 10 % over three, read-write passes gain 13 - 20 %
 * either way).  Allocations are 512-byte
 * aligned, first fit, thread-safe; contents are not cleared.  A pointer goes back to the pool it came
 * from whichever pool a context or the hooks point at by then.  Destroy the pool after everything that
 * allocated from it and before its context.
 * One pool per device at a time, made at start-up, and not within about ten seconds of a large release of
 * device memory.  The driver takes released memory back asynchronously: for a few seconds after tens of GB were
 * freed (a pool destroyed, this function's own hand-back of what the arena does not need, another process that
 * has just exited) every kernel on the device runs about 0.7 % slower, taking memory chunk by chunk is several
 * times slower, and a scan made in that time reads rates that belong to nothing: a second pool created right
 * after the first was destroyed found four groups and interleaved 138 of 200 GiB in 8.8 s, ten seconds later
 * three regions and 192 GiB in 1.8 s.  This function notices by the slow creation of its chunks, hands everything
 * back, waits four seconds and takes the memory again, at most twice (create_seconds then reads 10 - 15 s); a
 * host does better to wait by itself before creating a pool after such a release.  Allow about three seconds
 * after this function before timing anything: it hands back what the arena does not need.  A pool created while another pool or another
 * large allocation is alive only sees what is left, in pieces smaller than its 1 GiB groups: every pair of
 * groups answers at an in-between rate, it reports whatever grouping the rates suggest, and its arena is
 * interleaved by accident rather than by design.
 * No counterpart in the reference (MLX owns its allocator there). */
#define MXOPT_HBM_MAX_REGIONS 8
typedef struct mxopt_hbm_pool mxopt_hbm_pool;
typedef struct mxopt_hbm_pool_info {
  uint64_t capacity_bytes;
  uint64_t used_bytes;
  uint64_t chunk_bytes;
  int32_t regions;                                       /* regions found among the free memory */
  int32_t reserved_;
  uint64_t region_free_bytes[MXOPT_HBM_MAX_REGIONS];     /* free memory per region when the pool was made */
  uint64_t region_arena_bytes[MXOPT_HBM_MAX_REGIONS];    /* how much of the arena lies in each */
  double probe_same_region_gbps;                         /* the probe with all four streams in one region */
  double probe_cross_region_gbps;                        /* ... with two of them in another (0 if regions == 1) */
  double setup_seconds;                                  /* whole of mxopt_hbm_pool_create */
  double create_seconds;                                 /* ... of which taking the free memory as chunks (with the waits and retakes when the driver was busy) */
  double scan_seconds;                                   /* ... and timing probes to find the regions */
  int32_t probes;                                        /* probe measurements taken */
  int32_t reserved2_;
  uint64_t interleaved_bytes;  /* arena bytes [0, this) alternate between regions chunk by chunk; what lies behind
                                  comes from one region at a time (MXOPT_HBM_ONE_REGION allocations) */
  double arena_probe_gbps;     /* the 4-read/3-write probe over four pieces spread across the finished arena: what
                                  was built, measured (compare with the two probe levels above; 0 for an arena
                                  under 256 MiB) */
} mxopt_hbm_pool_info;
int mxopt_hbm_pool_create(mxopt_ctx* ctx, size_t capacity_bytes, size_t chunk_bytes, int max_regions,
                          mxopt_hbm_pool** out);
/* The same with every knob.  Zero-fill the struct first; a field left 0 takes its default.
 * While it scans, creation holds the device's free memory (all of it by default: memory far from what a small
 * allocation would get can only be reached by holding what lies in between) and times kernels on it, so the
 * process needs the GPU to itself for those seconds: another process's, or another thread's, allocation can
 * fail with out-of-memory meanwhile, and a co-tenant's traffic disturbs the timing.  max_take_bytes bounds what
 * is held (never less than the arena itself); with a bound below the free memory the scan sees less, possibly
 * one region only.  slab_bytes is the unit of classification (a power of two in [512 MiB, 4 GiB], default
 * 1 GiB): 512 MiB slabs follow fragmented free memory more closely for twice the probes at about the same scan
 * time; smaller ones would let the probe's working set sit in the last-level cache and hide the regions. */
typedef struct mxopt_hbm_pool_options {
  size_t capacity_bytes;
  size_t chunk_bytes;      /* 0: 64 MiB */
  int    max_regions;      /* 0: all regions found */
  int    reserved_;
  size_t max_take_bytes;   /* 0: all free memory but 1 GiB */
  size_t slab_bytes;       /* 0: 1 GiB */
} mxopt_hbm_pool_options;
int mxopt_hbm_pool_create_ex(mxopt_ctx* ctx, const mxopt_hbm_pool_options* options, mxopt_hbm_pool** out);
/* Refused (MXOPT_ERR_INVALID_ARG, nothing happens) while allocations from the pool are live: their memory would
 * be unmapped under whoever still uses it. */
int mxopt_hbm_pool_destroy(mxopt_hbm_pool* pool);
int mxopt_hbm_pool_alloc(mxopt_hbm_pool* pool, size_t bytes, void** out);
/* Where in the arena: MXOPT_HBM_INTERLEAVED (what mxopt_hbm_pool_alloc gives) for buffers a kernel writes or
 * reads together with ones it writes; MXOPT_HBM_ONE_REGION for buffers that are only ever read (gradients):
 * the part of the arena behind the alternation, when the arena is large enough to have one (info.capacity_bytes
 * > info.interleaved_bytes), else anywhere.  Read-only passes are 3 % (two regions) to 10 % (three) faster on
 * memory of one region. */
enum { MXOPT_HBM_INTERLEAVED = 0, MXOPT_HBM_ONE_REGION = 1 };
int mxopt_hbm_pool_alloc_kind(mxopt_hbm_pool* pool, size_t bytes, int kind, void** out);
/* Gives the range back.  Like every pool free (the hook's and the library's own included) this does NOT
 * synchronise with the device the way hipFree does: a caller that frees memory which kernels on another stream
 * may still use, or reuses it from another stream, orders that itself. */
int mxopt_hbm_pool_free(mxopt_hbm_pool* pool, void* ptr);
int mxopt_hbm_pool_owns(const mxopt_hbm_pool* pool, const void* ptr);   /* 1 if ptr lies inside the arena */
int mxopt_hbm_pool_get_info(mxopt_hbm_pool* pool, mxopt_hbm_pool_info* out);
/* The memory the library itself owns on behalf of the reference's objects -- the optimizers' moments
 * (init_state: adam.rs:148-153, adamw.rs:152-157, rmsprop.rs:123-127), the engines' accumulation buffers
 * (grpo/engine.rs:2632-2666, sft/engine.rs:282-306) -- is taken from `pool` while it has room (NULL: from
 * the driver again).  Objects created before the call keep what they have. */
int mxopt_set_state_pool(mxopt_ctx* ctx, mxopt_hbm_pool* pool);
/* For hosts whose allocator takes plug-in functions (torch's CUDAPluggableAllocator has exactly these
 * signatures): allocations on the target pool's device come from its arena while it has room and from
 * hipMalloc otherwise; frees find their way back by address. */
int mxopt_hbm_pool_set_hook_target(mxopt_hbm_pool* pool);
int mxopt_hbm_pool_set_hook_kind(int kind);   /* kind of the hook's allocations from now on (process-wide) */
void* mxopt_hbm_pool_hook_alloc(ptrdiff_t size, int device, void* stream);
void mxopt_hbm_pool_hook_free(void* ptr, ptrdiff_t size, int device, void* stream);

/* ---- tensor table ------------------------------------------------------------------
 * One descriptor per tensor.  Which fields a kernel reads is listed at that kernel;
 * unused pointers may be NULL.  All buffers are dense, `n` elements long.
 * Buffers need only their natural alignment.  A tensor whose used pointers all become
 * 16-byte aligned after the same number (0..7) of leading elements takes the 128-bit
 * path (those leading elements are handled one by one); others an element-wise path. */
typedef struct mxopt_tensor {
  const void* p;     /* parameter, read                                             */
  void*       p_out; /* parameter, written; may equal p (in place)                  */
  const void* g;     /* gradient, read                                              */
  void*       g_out; /* transformed gradient (mxopt_grad_transform), or the
                        accumulation buffer (mxopt_accumulate: read+written)        */
  float*      m;     /* first moment, float32, in place (Adam/AdamW)                */
  float*      v;     /* second moment (Adam/AdamW/RMSprop) or velocity (SGD),
                        float32, in place                                           */
  uint64_t    n;     /* elements; 0 is legal and skipped                            */
  uint8_t     p_dtype, p_out_dtype, g_dtype, g_out_dtype; /* MXOPT_F32/F16/BF16     */
  uint32_t    flags; /* MXOPT_TF_*                                                  */
  float       bc1;   /* f32(1/(1-beta1^t)) for THIS tensor, 1.0f when bias          */
  float       bc2;   /* correction is off (t counts update_single calls:
                        adam.rs:73, adamw.rs:77, so it differs per tensor)          */
} mxopt_tensor;

#define MXOPT_TF_FIRST 0x1u /* SGD: no velocity stored yet -> v' = ge (sgd.rs:107-114); v is not read */

int mxopt_table_build(mxopt_ctx* ctx, const mxopt_tensor* tensors, size_t n, mxopt_table** out);
/* Per-step scalars, `n` entries each; a NULL array leaves that field unchanged. */
int mxopt_table_set_step_scalars(mxopt_table* t, const float* bc1, const float* bc2, const uint32_t* flags);
/* Same tensors (sizes, dtypes, which pointers are set, alignment class), new buffers: swaps the
 * pointers of an existing table without rebuilding its chunk list (hosts whose arrays move every
 * step, as MLX's do).  Stream-ordered like a kernel.  Returns MXOPT_ERR_INVALID_ARG and changes
 * nothing when the layout differs; build a new table then. */
int mxopt_table_retarget(mxopt_table* t, const mxopt_tensor* tensors, size_t n);
void mxopt_table_destroy(mxopt_table* t);
uint64_t mxopt_table_total_elems(const mxopt_table* t);
uint64_t mxopt_table_num_chunks(const mxopt_table* t);
uint64_t mxopt_table_num_tensors(const mxopt_table* t);
/* Host-only query (no device needed, pointers are not dereferenced): how the table builder
 * lays out one tensor.  *head = leading elements handled one by one (0..7), *vector_path = 1
 * when the rest takes the 128-bit path, *num_chunks = table entries (workgroups of work).
 * Any out pointer may be NULL.  No counterpart in the reference (MLX picks its own kernels). */
int mxopt_tensor_layout(const mxopt_tensor* t, uint32_t* head, int* vector_path, uint64_t* num_chunks);
#define MXOPT_CHUNK_ELEMS 4096 /* elements one workgroup handles per table entry */

/* ---- device-resident result of the global-norm reduction ------------------------ */
typedef struct mxopt_norm_result {
  double   sumsq;     /* sum of squares, accumulated in float64                     */
  double   norm;      /* sqrt(sumsq)                                                */
  float    norm_f32;  /* (float)norm: what clip_grad_norm_with_norm returns          */
  float    scale;     /* clip factor, see mxopt_clip_mode                           */
  uint64_t nonfinite; /* 0: every element finite.  1: some element is a NaN or an infinity -- the
                         engines' per-element validity check (grpo/engine.rs:563-569), also under
                         prep's clamp_pre, which would have hidden a raw +-Inf; sumsq, norm and
                         scale are NaN then.  2: every element is finite but their squares left
                         float32 range: sumsq and norm are +Inf and scale 0, which is what the
                         reference's own float32 chain makes of such gradients
                         (optimizers/mod.rs:78-96); kernels told to skip on this flag look at
                         bit 0 only and still run                                           */
} mxopt_norm_result;

/* How `scale` is derived from the norm. */
enum {
  /* GradientUtils::clip_grad_norm (optimizers/mod.rs:87-96):
   * scale = min(f32(max) / (norm_f32 + f32(1e-6)), 1.0f), applied also when it is 1. */
  MXOPT_CLIP_ALWAYS_MULTIPLY = 0,
  /* clip_gradients_by_global_norm (gradients/mod.rs:255-270): norm <= max -> 1.0f
   * exactly (gradients unchanged), else f32(max / (norm + 1e-6)) evaluated in float64. */
  MXOPT_CLIP_IF_ABOVE = 1
};

/* ---- gradient pre-processing done in registers ----------------------------------
 * g_eff = clamp_post( d_scale * clamp_pre( pre_mul * g ) ), each stage optional, each one
 * float32 op per reference op.  Covers the engines' orders:
 *  GRPO: clamp(+-v) -> clip-norm                 (grpo/engine.rs:636-653)
 *  SFT : x(1/N) -> clip-norm -> clamp(+-v)       (sft/engine.rs:299-329)
 * The global norm is always taken after pre_mul and clamp_pre.  NaN passes through
 * the clamps unchanged. */
typedef struct mxopt_grad_prep {
  int          has_pre_mul;    float pre_mul;           /* f32(1/N) (sft/engine.rs:299-306) */
  int          has_clamp_pre;  float pre_lo, pre_hi;    /* mlx clip, mlx.cpp:469-481        */
  const float* d_scale;        /* device scalar (e.g. &norm_result->scale); NULL = none    */
  int          has_clamp_post; float post_lo, post_hi;
  /* Device flag word (e.g. &norm_result->nonfinite); when its bit 0 is set -- some gradient element was a
   * NaN or an infinity -- the update / transform kernel changes nothing: the engines' "any NaN/Inf
   * gradient => skip the whole step" policy (grpo/engine.rs:561-607, sft/engine.rs:221-258) without a
   * host round trip.  NULL = never skip. */
  const uint64_t* d_skip_if_nonzero;
} mxopt_grad_prep;

/* ---- hyper-parameters: float32 coefficients exactly as the reference hands them to MLX */
typedef struct mxopt_adam_hp {
  float lr, beta1, beta2, one_minus_beta1, one_minus_beta2, eps;
  float decay;           /* f32(1 - lr*wd) (adamw.rs:83); used when decoupled_decay      */
  int   decoupled_decay; /* 1 = AdamW (adamw.rs:84), 0 = Adam (adam.rs:108)              */
} mxopt_adam_hp;
void mxopt_adam_hp_from_f64(double lr, double beta1, double beta2, double eps, double weight_decay,
                            int decoupled_decay, mxopt_adam_hp* out);
/* bc = f32(1/(1-beta^t)) in float64 then cast (adamw.rs:99-104). */
void mxopt_bias_correction(double beta1, double beta2, int64_t t, float* bc1, float* bc2);

typedef struct mxopt_sgd_hp {
  float lr, momentum, one_minus_dampening, weight_decay;
  int   has_weight_decay; /* wd != 0 (sgd.rs:86) */
  int   has_momentum;     /* momentum != 0 (sgd.rs:96) */
  int   nesterov;         /* stores v'+ge as the new state (sgd.rs:117-130) */
} mxopt_sgd_hp;
/* Returns MXOPT_ERR_INVALID_ARG for nesterov with momentum <= 0 or dampening != 0 (sgd.rs:51-56). */
int mxopt_sgd_hp_from_f64(double lr, double momentum, double weight_decay, double dampening, int nesterov,
                          mxopt_sgd_hp* out);

typedef struct mxopt_rmsprop_hp {
  float lr, alpha, one_minus_alpha, eps, weight_decay;
  int   has_weight_decay;
} mxopt_rmsprop_hp;
void mxopt_rmsprop_hp_from_f64(double lr, double alpha, double eps, double weight_decay, mxopt_rmsprop_hp* out);

/* ---- update kernels: one launch per dtype group for the whole table -------------- */

/* Adam / AdamW step.  Reads p, g, m, v; writes p_out, m, v.
 * Replaces the 12/13-op chains of Adam::update_single (optimizers/adam.rs:77-108) and
 * AdamW::update_single (optimizers/adamw.rs:81-116) for every tensor of the table.
 * `prep` may be NULL. */
int mxopt_adam(mxopt_ctx* ctx, const mxopt_table* t, const mxopt_adam_hp* hp, const mxopt_grad_prep* prep);

/* mxopt_adam with the last micro-batch still pending: the gradient is tensor.g (the float32
 * accumulation buffer) + tensor.g_out (the micro-batch that mxopt_accumulate_norm_only measured
 * but did not store), one float32 add, i.e. exactly the value mxopt_accumulate would have
 * written.  Saves the accumulation buffer's last write (4 B/elem) at the price of re-reading the
 * micro-batch (2 B/elem for bf16).  The accumulation buffer is left WITHOUT the last micro-batch.
 * No counterpart in the reference (it has no fused accumulate/update at all). */
int mxopt_adam_with_pending(mxopt_ctx* ctx, const mxopt_table* t, const mxopt_adam_hp* hp,
                            const mxopt_grad_prep* prep);

/* SGD with momentum / dampening / Nesterov / coupled L2.  Reads p, g, v (unless
 * MXOPT_TF_FIRST); writes p_out, v.  Replaces SGD::update_single (optimizers/sgd.rs:84-150). */
int mxopt_sgd(mxopt_ctx* ctx, const mxopt_table* t, const mxopt_sgd_hp* hp, const mxopt_grad_prep* prep);

/* RMSprop.  Reads p, g, v; writes p_out, v.  Replaces RMSprop::update_single
 * (optimizers/rmsprop.rs:67-112). */
int mxopt_rmsprop(mxopt_ctx* ctx, const mxopt_table* t, const mxopt_rmsprop_hp* hp, const mxopt_grad_prep* prep);

/* Plain SGD in the parameter's dtype: p_out = astype(p - astype(lr, dtype(p)) * g, dtype(p)),
 * with the intermediate product rounded to the 16-bit dtype when p and g share it.
 * Optional coupled decay g + f32(wd)*p first (sft/engine.rs:345-365).
 * Replaces Qwen3Model::apply_gradients (models/qwen3/model.rs:2434-2451). */
int mxopt_sgd_plain(mxopt_ctx* ctx, const mxopt_table* t, double learning_rate, double weight_decay,
                    const mxopt_grad_prep* prep);

/* mxopt_sgd_plain with the last micro-batch still pending: g is the float32 accumulation buffer,
 * g_out the micro-batch that was NOT added to it.  The sum is formed in registers (one float32
 * add, the value an accumulation pass would have stored) instead of being written back and read
 * again: r(p, acc, g) + w(p) replaces an accumulation pass plus an apply pass.  The buffer is
 * left without the last micro-batch.
 *   prep_covers_sum = 0: gradient = g + prep(g_out)   the buffer holds already clipped
 *                        micro-batches, the pending one is clamped / scaled here
 *                        (grpo/engine.rs:636-692: clip, accumulate, apply_gradients);
 *   prep_covers_sum = 1: gradient = prep(g + g_out)   average, clip and clamp act on the sum
 *                        (sft/engine.rs:293-371), pair with mxopt_accumulate_norm_only.
 * weight_decay as in mxopt_sgd_plain. */
int mxopt_sgd_plain_with_pending(mxopt_ctx* ctx, const mxopt_table* t, double learning_rate, double weight_decay,
                                 const mxopt_grad_prep* prep, int prep_covers_sum);

/* ---- deferred accumulation ---------------------------------------------------------
 * With HBM to spare the accumulation buffer need not exist.  The micro-batch gradients of one
 * optimizer step stay where the backward passes left them; the norm pass and the update kernel add
 * them in registers, left to right in float32:  ((g + x0) + x1) + x2.  These are the additions
 * Qwen3Model::accumulate_gradients (models/qwen3/model.rs:2217-2243) / the engines
 * (grpo/engine.rs:2632-2666, sft/engine.rs:282-290) would have made into a float32 buffer, in the
 * same order, so parameters and moments come out bit-identical while the buffer is never written
 * or read back: four bf16 micro-batches + AdamW move 36 B/elem instead of 58.  Up to
 * MXOPT_MAX_PENDING + 1 = 8 micro-batches can be held (with more than four the kernels walk a chunk
 * in smaller pieces and reach somewhat less bandwidth: ten or more concurrent streams).
 *
 * tensor.g is the first addend: the first micro-batch, or a float32 buffer that already holds
 * earlier ones (more micro-batches than MXOPT_MAX_PENDING + 1).  The pending streams x0.. all have
 * one dtype; tensor.g has that dtype or float32.  The caller keeps every stream alive and unchanged
 * until the update has RUN, i.e. until the work the call enqueued on the context's stream has
 * completed (the call returning only means it is enqueued), or orders any reuse of that memory after
 * it on the same stream.  No counterpart in the reference (it materialises every sum). */
#define MXOPT_MAX_PENDING 7

/* Attach k (0..MXOPT_MAX_PENDING; 0 detaches) pending streams to every row of the table:
 * streams[j * num_tensors + i] is pending stream j of row i, `dtype` their element type.  A
 * stream of a row with n > 0 must not be NULL and must share the 16-byte phase of the row's other
 * buffers (see mxopt_tensor_layout).  Stream-ordered like mxopt_table_retarget; call it again when
 * the buffers of the next step differ. */
int mxopt_table_set_pending(mxopt_table* t, int k, const void* const* streams, int dtype);

/* Norm (and clip factor) of prep_pre(g + x0 + ...) over the whole table; nothing is stored.
 * Arguments as mxopt_global_norm. */
int mxopt_norm_with_pending_list(mxopt_ctx* ctx, const mxopt_table* t, const mxopt_grad_prep* prep, double max_norm,
                                 int clip_mode, mxopt_norm_result* d_result);

/* mxopt_adam on the gradient prep(g + x0 + ...).  p_out must have p's dtype (in place or not). */
int mxopt_adam_with_pending_list(mxopt_ctx* ctx, const mxopt_table* t, const mxopt_adam_hp* hp,
                                 const mxopt_grad_prep* prep);

/* mxopt_sgd and mxopt_rmsprop on the gradient prep(g + x0 + ...); p_out must have p's dtype. */
int mxopt_sgd_with_pending_list(mxopt_ctx* ctx, const mxopt_table* t, const mxopt_sgd_hp* hp,
                                const mxopt_grad_prep* prep);
int mxopt_rmsprop_with_pending_list(mxopt_ctx* ctx, const mxopt_table* t, const mxopt_rmsprop_hp* hp,
                                    const mxopt_grad_prep* prep);

/* mxopt_sgd_plain on the gradient prep(g + x0 + ...), which is float32 (the sum promotes);
 * the SFT engine's boundary (sft/engine.rs:293-371) without its accumulation buffer. */
int mxopt_sgd_plain_with_pending_list(mxopt_ctx* ctx, const mxopt_table* t, double learning_rate,
                                      double weight_decay, const mxopt_grad_prep* prep);

/* The same update with every micro-batch pre-processed on its own before it is added:
 * gradient = prep_0(g) + prep_1(x0) + ..., where prep_j is `prep` (d_scale ignored) with the clip factor
 * read from d_scales[j] (k + 1 device pointers, or all NULL for no factor) -- the GRPO engine's
 * "clamp, clip by this micro-batch's own norm, accumulate" (grpo/engine.rs:636-661) followed by its
 * apply_gradients (:666-692), without the accumulation buffer.  first_is_sum != 0: tensor.g is a
 * float32 buffer into which earlier micro-batches were added after their own pre-processing (more
 * micro-batches than streams); it is added as it is and d_scales[0] must be NULL. */
int mxopt_sgd_plain_with_pending_list_each(mxopt_ctx* ctx, const mxopt_table* t, double learning_rate,
                                           double weight_decay, const mxopt_grad_prep* prep,
                                           const float* const* d_scales, int first_is_sum);

/* ---- global norm ------------------------------------------------------------------ */

/* Sum of squares of the gradients (after prep's pre_mul / clamp_pre) over the whole
 * table: wavefront shuffle -> LDS -> one float64 partial per workgroup -> one
 * single-workgroup second pass; no atomics, run-to-run deterministic; the same pass yields the gradient-validity flag.  `which` = 0 reads
 * tensor.g, 1 reads tensor.g_out (the accumulation buffer).  If max_norm >= 0 the second
 * pass also derives `scale` per `clip_mode`; otherwise scale = 1.  Writes *d_result
 * (device memory).  Replaces the square/sum/add chain of GradientUtils::clip_grad_norm
 * (optimizers/mod.rs:76-96), compute_gradient_norm (:43-55) and the per-tensor reductions
 * of clip_gradients_by_global_norm (gradients/mod.rs:246-256). */
int mxopt_global_norm(mxopt_ctx* ctx, const mxopt_table* t, int which, const mxopt_grad_prep* prep,
                      double max_norm, int clip_mode, mxopt_norm_result* d_result);

/* mxopt_global_norm for callers that cannot allocate device memory (a step being captured into a HIP
 * graph, a serving loop that forbids hipMalloc, a harness that counts allocations).  It has no
 * counterpart in the reference.  Same arguments, same kernels and bit-identical *d_result; the one
 * difference is where the per-workgroup partial sums live: in a fixed array of
 * MXOPT_STATIC_NORM_WORKGROUPS float64 values (128 KiB) inside the library's code object, of which
 * every GPU the library runs on holds one copy until the process ends, instead of a buffer the
 * context allocates on first use and grows on demand.  The call allocates and frees nothing on the
 * device and records no memset.  A table whose reduction takes more workgroups than the array has
 * slots (sum over dtype groups of min(chunks, CUs x grid_blocks_per_cu); 4096 per group by default)
 * is refused with MXOPT_ERR_INVALID_ARG.  All contexts on one GPU share that GPU's array: every slot
 * a call reads was written by the same call, so nothing has to be cleared, but two such calls that
 * overlap in time on one GPU (different streams) race and must be ordered by the caller. */
#define MXOPT_STATIC_NORM_WORKGROUPS 16384
int mxopt_global_norm_static(mxopt_ctx* ctx, const mxopt_table* t, int which, const mxopt_grad_prep* prep,
                             double max_norm, int clip_mode, mxopt_norm_result* d_result);

/* g_out = prep(g) element-wise (scale and/or clamps): the scale pass of clip_grad_norm
 * (optimizers/mod.rs:98-102), clip_grad_value (:164-166), clip_gradients_by_value
 * (gradients/mod.rs:299-312).  Only needed when the clipped gradients themselves must be
 * handed back; the update kernels apply `prep` in registers instead. */
int mxopt_grad_transform(mxopt_ctx* ctx, const mxopt_table* t, const mxopt_grad_prep* prep);

/* ---- accumulation -------------------------------------------------------------------
 * g_out = first ? astype(g) : g_out + g, in promote(dtype(g_out), dtype(g)) then stored as
 * dtype(g_out).  With a float32 g_out and bf16 g this is the mixed-precision accumulation
 * buffer; with equal dtypes it is the reference's `acc.add(&grad)`
 * (models/qwen3/model.rs:2227, grpo/engine.rs:2643, sft/engine.rs:285).  If d_result is not
 * NULL the sum of squares of the NEW buffer contents (after prep's pre_mul/clamp_pre) is
 * reduced in the same pass and finished exactly like mxopt_global_norm. */
int mxopt_accumulate(mxopt_ctx* ctx, const mxopt_table* t, int first, const mxopt_grad_prep* prep,
                     double max_norm, int clip_mode, mxopt_norm_result* d_result);

/* The global norm the accumulation buffer would have after adding g, without writing it:
 * *d_result describes g_out + g (read only, 6 B/elem for a float32 buffer and bf16 gradients).
 * Pair with mxopt_adam_with_pending. */
int mxopt_accumulate_norm_only(mxopt_ctx* ctx, const mxopt_table* t, const mxopt_grad_prep* prep, double max_norm,
                               int clip_mode, mxopt_norm_result* d_result);

/* g_out = first ? prep(g) : g_out + prep(g): the engines' per-micro-batch "clamp, clip by norm,
 * then accumulate" (grpo/engine.rs:636-661, :1737-1754) without materialising the clipped
 * gradient.  prep(g) is float32 (clip and the scale multiply promote); the sum is one float32
 * add, rounded once to dtype(g_out).  Honours prep->d_skip_if_nonzero: a micro-batch flagged
 * non-finite by mxopt_global_norm leaves the buffer untouched (grpo/engine.rs:561-562). */
int mxopt_accumulate_transformed(mxopt_ctx* ctx, const mxopt_table* t, int first, const mxopt_grad_prep* prep);

/* ---- small host<->device helpers (each synchronises the context's stream) --------- */
int mxopt_read_norm_result(mxopt_ctx* ctx, const mxopt_norm_result* d_result, mxopt_norm_result* host_out);

const char* mxopt_version(void);

#ifdef __cplusplus
}
#endif
#endif /* MXOPT_H */
