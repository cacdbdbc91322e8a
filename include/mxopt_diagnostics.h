/* mxopt_diagnostics.h -- entry points of libmxopt.so that no reference call site binds.
 *
 * What the reference's optimizer path needs is in mxopt.h, mxopt_optimizers.h and mxopt_engine.h.  This
 * header holds what this repository's benchmark and tests use besides: bare streaming probes (the measured
 * ceilings the kernels are compared with), the counter-based data generator whose host twin lets a checker
 * regenerate any slice of any input, and the region scan of the memory pool as pure functions so that it
 * can be driven with synthetic rate maps on a machine without a GPU.  None of them has a counterpart in the
 * reference.
 */
#ifndef MXOPT_DIAGNOSTICS_H
#define MXOPT_DIAGNOSTICS_H

#include "mxopt.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- bare streaming probes ------------------------------------------------------------
 * The measured ceilings the update kernels are compared with: float32 buffers of n_elems elements
 * (a positive multiple of 4096, 16-byte aligned), no table, no tails, no arithmetic to speak of.
 *   MXOPT_PROBE_READ   reads a                       MXOPT_PROBE_WRITE  writes a
 *   MXOPT_PROBE_COPY   reads a, writes b             MXOPT_PROBE_MIX43  reads a, b, c, d and writes a, c, d
 * (MIX43 is float32 AdamW's byte mix, 28 B/elem.)  One launch on the context's stream.
 * kind | MXOPT_PROBE_STREAMING: the same streams with streaming-hint loads and stores, which is how the update
 * kernels access memory by default (READ always streams; the pool's own region scan uses plain MIX43). */
enum { MXOPT_PROBE_READ = 0, MXOPT_PROBE_WRITE = 1, MXOPT_PROBE_COPY = 2, MXOPT_PROBE_MIX43 = 3 };
#define MXOPT_PROBE_STREAMING 0x100
int mxopt_probe_stream(mxopt_ctx* ctx, int kind, void* a, void* b, void* c, void* d, uint64_t n_elems);
/* The byte mix of the update over k un-summed 16-bit micro-batches (mxopt_adam_with_pending_list) without its
 * arithmetic: g[0..k) and p are 2-byte streams of n_elems elements, m and v 4-byte ones; p, m and v are
 * rewritten in place (2k + 20 B/elem).  k in [1, 8], n_elems a positive multiple of 4096.
 * k | MXOPT_PROBE_STREAMING: the 2-byte streams with streaming-hint loads and stores (the list kernels' way). */
int mxopt_probe_list(mxopt_ctx* ctx, void* p, void* m, void* v, const void* const* g, int k, uint64_t n_elems);

/* ---- synthetic data for benchmarks and parity tests ----------------------------------
 * out[i] = f(hash(seed, first_index + i)), hash = splitmix64 finaliser of seed + (index+1)*golden:
 *   MXOPT_SYNTH_NORMAL          (sum of four 16-bit fields of the hash - 131070) * f32(a / sqrt((65536^2-1)/3)):
 *                               mean 0, standard deviation a, bell shaped, |x| <= 3.46 a
 *   MXOPT_SYNTH_NORMAL_OUTLIERS the same, and on average every 100th element (second hash % 100 == 0) times f32(b)
 *   MXOPT_SYNTH_UNIFORM         f32(top 24 bits) * f32((b - a) / 2^24) + f32(a): uniform on [a, b)
 *   MXOPT_SYNTH_GAUSSIAN        normal with standard deviation a and true tails: bit 63 of the hash is the sign,
 *                               bits 31..62 a uniform u that stands for the two-sided tail probability
 *                               (u + 0.5) / 2^32 of |x|; u is split like a floating-point number (leading zeros:
 *                               octave, next 5 bits: sub-interval, 16 more bits: linear interpolation) into a
 *                               committed 32 x 33 table of float32 quantiles, so |x| reaches 6.3 a with the same
 *                               relative resolution everywhere; then * f32(a)
 *   MXOPT_SYNTH_GAUSSIAN_OUTLIERS  the same, and on average every 100th element times f32(b)
 * then rounded once to out's dtype.  Only integer arithmetic, exact conversions and at most two rounded
 * float32 operations (three and a table look-up for the Gaussian modes): a host program regenerates any slice bit for bit (as the CPU checker in this
 * repository does), so inputs never have to be copied or read back to compare results at full size.
 * No counterpart in the reference (its tests build inputs on the host). */
enum { MXOPT_SYNTH_NORMAL = 0, MXOPT_SYNTH_NORMAL_OUTLIERS = 1, MXOPT_SYNTH_UNIFORM = 2, MXOPT_SYNTH_GAUSSIAN = 3,
       MXOPT_SYNTH_GAUSSIAN_OUTLIERS = 4 };
int mxopt_fill_synthetic(mxopt_ctx* ctx, void* out, uint64_t n, int dtype, uint64_t seed, uint64_t first_index,
                         int distribution, double a, double b);
/* The stream key used by this repository's benchmark and tests:
 * splitmix64(seed ^ config ^ step << 32 ^ micro_batch << 48 ^ tensor_index).  Host only. */
uint64_t mxopt_synthetic_key(uint64_t seed, uint64_t config, uint64_t step, uint64_t micro_batch, uint64_t tensor_index);

/* ---- the pool's region scan, without a device ------------------------------------------
 * mxopt_hbm_pool_create decides which 1 GiB groups of physical chunks ("slabs") share a memory region from
 * probe rates alone; these two run the very same decisions on rates the caller supplies.
 * probe(user, ref_slab, slab, &gbps): rate of the 4-read/3-write probe with two streams in `ref_slab` and two
 * in `slab` (slow = same region); non-zero return = error, handed back.  slab_region[i] = region of slab i. */
typedef int (*mxopt_slab_probe_fn)(void* user, int ref_slab, int slab, double* gbps);
typedef struct mxopt_hbm_scan_report {
  int32_t regions;            /* groups found (leftover groups of a few slabs included) */
  int32_t probes;             /* probe calls made */
  double  same_region_gbps;   /* levels of the two classes in the scan that first showed both */
  double  cross_region_gbps;
} mxopt_hbm_scan_report;
int mxopt_hbm_classify_regions(int n_slabs, mxopt_slab_probe_fn probe, void* user, int* slab_region,
                               mxopt_hbm_scan_report* report);
/* The arena's chunk order for a classification: order[i] = physical chunk of arena chunk i.  Consecutive
 * arena chunks alternate between the `max_regions` (0 = all) largest regions that hold at least a tenth of the
 * chunks, then the rest follows region by region. */
typedef struct mxopt_hbm_arena_report {
  int32_t real_regions;        /* regions holding at least a tenth of all chunks */
  int32_t active_regions;      /* regions in the alternation */
  int32_t interleaved_chunks;  /* arena chunks [0, this) alternate */
  int32_t reserved_;
} mxopt_hbm_arena_report;
int mxopt_hbm_plan_arena(int n_slabs, const int* slab_region, int regions, int chunks_per_slab, int total_chunks,
                         int want_chunks, int max_regions, int* order, mxopt_hbm_arena_report* report);

#ifdef __cplusplus
}
#endif
#endif /* MXOPT_DIAGNOSTICS_H */
