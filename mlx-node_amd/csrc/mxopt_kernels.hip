// mxopt kernels for gfx950, part 1: the multi-tensor optimizer updates and the gradient transform.
// Every kernel walks a device-side chunk table so that thousands of tensors share one launch; each is
// a pure streaming pass whose roof is HBM bandwidth.  Build with -ffp-contract=off: one IEEE float32
// rounding per reference op.
#include "mxopt_kernels_common.h"

namespace mxopt {

// ------------------------------------------------------------------------------------
// Update kernel.  G2 >= 0: a second gradient stream of that dtype in tensor.g_out is added to g
// first (one float32 add: the last micro-batch folded into the update instead of being written
// back to the accumulation buffer).
// ------------------------------------------------------------------------------------

template <int PD, int GD, int OD, int G2, class Math, bool NT>
__global__ __launch_bounds__(kThreads) void update_kernel(const DevTensor* __restrict__ T,
                                                          const DevChunk* __restrict__ C, DevTensor one,
                                                          uint32_t nchunks, Math math, DevPrep prep) {
  constexpr bool kHasG2 = G2 >= 0;
  constexpr int G2D = kHasG2 ? G2 : MXOPT_F32;
  // Elements per lane and group.  With a 16-bit stream in the mix, 8 (one 16-byte access of the 16-bit stream,
  // two of every float32 stream) when a second gradient stream is folded in, 4 (8-byte accesses of the 16-bit
  // streams, one 16-byte access of the float32 ones) without: then every access covers whole sectors and can
  // stream (see load_group).  Measured for bf16 AdamW: no difference on a large list (6.05 against 6.07 ms on
  // Qwen3-1.7B), 11 % less time on a list that a few passes of the memory-side cache cover (10,000 small tensors,
  // 2 GB of traffic per step: 0.316 against 0.353 ms) -- accesses that all stream leave a part of the list
  // resident from one step to the next, plain ones push it out.  With the second stream the wider group wins
  // (fewer, larger requests for three 16-bit streams): 8 there.
  constexpr bool kMixed = PD != MXOPT_F32 || GD != MXOPT_F32 || OD != MXOPT_F32 || (kHasG2 && G2D != MXOPT_F32);
  constexpr int E = (kMixed && kHasG2) ? 8 : 4;
  constexpr int U = kElemsPerLane / E;
  if (skip_requested(prep)) return;
  const PrepRegs pr = load_prep(prep);
  const uint32_t tid = threadIdx.x;
  // The gradient the update sees: prep(g), prep(g + g2) (an accumulation buffer plus the micro-batch
  // that was not written back to it), or g + prep(g2) (the buffer holds already-clipped gradients and
  // the pending micro-batch still has to be clipped: grpo/engine.rs:636-661).
  const bool pending_only = kHasG2 && (pr.flags & kPrepPendingOnly);
  auto combine = [&](float g, float g2) {
    if (!kHasG2) return prep_all(pr, g);
    return pending_only ? g + prep_all(pr, g2) : prep_all(pr, g + g2);
  };

  for (uint32_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
    const ChunkView cv = locate(T, C, one, c);
    const uint64_t start = cv.start;
    const uint32_t len = cv.len, flags = cv.t.flags;
    const float bc1 = cv.t.bc1, bc2 = cv.t.bc2;
    const void* P = cv.t.p;
    void* PO = cv.t.p_out;
    const void* G = cv.t.g;
    const void* G2P = cv.t.g_out;
    float* M = cv.t.m;
    float* V = cv.t.v;
    const bool use_v = math.uses_v(flags), read_v = math.reads_v(flags);
    auto one_element = [&](uint64_t off) {
      float p = Elem<PD>::load(P, off);
      const float ge = combine(Elem<GD>::load(G, off), kHasG2 ? Elem<G2D>::load(G2P, off) : 0.0f);
      float m = Math::kM ? Elem<MXOPT_F32>::load(M, off) : 0.0f;
      float v = read_v ? Elem<MXOPT_F32>::load(V, off) : 0.0f;
      math(p, ge, m, v, bc1, bc2, flags);
      Elem<OD>::store(PO, off, p);
      if (Math::kM) Elem<MXOPT_F32>::store(M, off, m);
      if (use_v) Elem<MXOPT_F32>::store(V, off, v);
    };

    if (cv.fast) {
      // Full chunk: issue every load of the chunk before the first use.
      float p[U][E], g[U][E], g2[U][E], m[U][E], v[U][E];
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const uint64_t off = start + (uint64_t)(j * kThreads + tid) * E;
        load_group<PD, E, NT>(P, off, p[j]);
        load_group<GD, E, NT>(G, off, g[j]);
        if (kHasG2) load_group<G2D, E, NT>(G2P, off, g2[j]);
        if (Math::kM) load_group<MXOPT_F32, E, NT>(M, off, m[j]);
        if (read_v) load_group<MXOPT_F32, E, NT>(V, off, v[j]);
      }
#pragma unroll
      for (int j = 0; j < U; ++j) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
          math(p[j][e], combine(g[j][e], g2[j][e]), m[j][e], v[j][e], bc1, bc2, flags);
        }
      }
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const uint64_t off = start + (uint64_t)(j * kThreads + tid) * E;
        if (PO == P) store_group<OD, E, NT>(PO, off, p[j]);  // streaming only where the line was read
        else store_group<OD, E, false>(PO, off, p[j]);
        if (Math::kM) store_group<MXOPT_F32, E, NT>(M, off, m[j]);
        if (use_v) store_group<MXOPT_F32, E, NT>(V, off, v[j]);
      }
    } else {
      // Last chunk of a tensor, or a tensor whose buffers are not 16-byte aligned.
      const uint32_t ngroups = (flags & kTfUnaligned) ? 0u : len / E;
      for (uint32_t q = tid; q < ngroups; q += kThreads) {
        const uint64_t off = start + (uint64_t)q * E;
        float p[E], g[E], g2[E], m[E], v[E];
        load_group<PD, E, false>(P, off, p);
        load_group<GD, E, false>(G, off, g);
        if (kHasG2) load_group<G2D, E, false>(G2P, off, g2);
        if (Math::kM) load_group<MXOPT_F32, E, false>(M, off, m);
        if (read_v) load_group<MXOPT_F32, E, false>(V, off, v);
#pragma unroll
        for (int e = 0; e < E; ++e) {
          math(p[e], combine(g[e], g2[e]), m[e], v[e], bc1, bc2, flags);
        }
        store_group<OD, E, false>(PO, off, p);
        if (Math::kM) store_group<MXOPT_F32, E, false>(M, off, m);
        if (use_v) store_group<MXOPT_F32, E, false>(V, off, v);
      }
      for (uint32_t i = ngroups * E + tid; i < len; i += kThreads) one_element(start + i);
    }
    if (tid < cv.head) one_element(tid);  // elements in front of the first aligned group
  }
}

// ------------------------------------------------------------------------------------
// Gradient transform: g_out = prep(g)
// ------------------------------------------------------------------------------------

// add != 0: g_out = g_out + prep(g) (one float32 add, rounded to g_out's dtype by the store): the
// engines' "clamp, clip-norm, then accumulate" (grpo/engine.rs:636-661) without materialising the
// clipped gradient.
template <int GD, int OD, bool NT, bool ADD>
__global__ __launch_bounds__(kThreads) void transform_kernel(const DevTensor* __restrict__ T,
                                                             const DevChunk* __restrict__ C, DevTensor one,
                                                             uint32_t nchunks, DevPrep prep) {
  constexpr bool add = ADD;
  // Elements per lane and group: 4 when the kernel adds into g_out (every access then covers whole sectors and
  // streams: the GRPO engine's accumulate of clamp * scale, bf16 into float32, 13.0 against 13.4 ms on the
  // Qwen3-8B list), 8 when a 16-bit stream is only converted (the first micro-batch: 8 was not slower there).
  constexpr int E = ((GD != MXOPT_F32 || OD != MXOPT_F32) && !ADD) ? 8 : 4;
  constexpr int U = kElemsPerLane / E;
  if (skip_requested(prep)) return;
  const PrepRegs pr = load_prep(prep);
  const uint32_t tid = threadIdx.x;
  for (uint32_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
    const ChunkView cv = locate(T, C, one, c);
    const uint64_t start = cv.start;
    const void* G = cv.t.g;
    void* GO = cv.t.g_out;
    auto one_element = [&](uint64_t off) {
      float t = prep_all(pr, Elem<GD>::load(G, off));
      if (add) t = Elem<OD>::load(GO, off) + t;
      Elem<OD>::store(GO, off, t);
    };
    if (cv.fast) {
      float g[U][E], a[U][E];
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const uint64_t off = start + (uint64_t)(j * kThreads + tid) * E;
        load_group<GD, E, NT>(G, off, g[j]);
        if (add) load_group<OD, E, NT>(GO, off, a[j]);
      }
      // The GRPO engine's order -- clamp, then the clip factor -- with its stage flags tested once per
      // chunk: tested per element they cost the 16-bit first pass (6 B/elem) more instruction issue than
      // it has to spare.
      const bool clamp_then_scale =
          (pr.flags & (kPrepPreMul | kPrepClampPre | kPrepClampPost)) == kPrepClampPre && pr.has_scale;
#pragma unroll
      for (int j = 0; j < U; ++j) {
        if (clamp_then_scale) {
#pragma unroll
          for (int e = 0; e < E; ++e) {
            g[j][e] = clamp_median_keep_nan(g[j][e], pr.pre_lo, pr.pre_hi) * pr.scale;
            if (add) g[j][e] = a[j][e] + g[j][e];
          }
        } else {
#pragma unroll
          for (int e = 0; e < E; ++e) {
            g[j][e] = prep_all(pr, g[j][e]);
            if (add) g[j][e] = a[j][e] + g[j][e];
          }
        }
        store_group<OD, E, NT && ADD>(GO, start + (uint64_t)(j * kThreads + tid) * E, g[j]);  // streaming only where the line was read
      }
    } else {
      const uint32_t ngroups = (cv.t.flags & kTfUnaligned) ? 0u : cv.len / E;
      for (uint32_t q = tid; q < ngroups; q += kThreads) {
        float g[E], a[E];
        load_group<GD, E, false>(G, start + (uint64_t)q * E, g);
        if (add) load_group<OD, E, false>(GO, start + (uint64_t)q * E, a);
#pragma unroll
        for (int e = 0; e < E; ++e) {
          g[e] = prep_all(pr, g[e]);
          if (add) g[e] = a[e] + g[e];
        }
        store_group<OD, E, false>(GO, start + (uint64_t)q * E, g);
      }
      for (uint32_t i = ngroups * E + tid; i < cv.len; i += kThreads) one_element(start + i);
    }
    if (tid < cv.head) one_element(tid);
  }
}

// ------------------------------------------------------------------------------------
// Launchers (dtype dispatch)
// ------------------------------------------------------------------------------------

template <int PD, int GD, int OD, int G2, class Math>
static void launch_update_t(const Launch& L, const Math& math, const DevPrep& prep) {
  if (L.nontemporal)
    MXOPT_LAUNCH((update_kernel<PD, GD, OD, G2, Math, true>), L, math, prep);
  else
    MXOPT_LAUNCH((update_kernel<PD, GD, OD, G2, Math, false>), L, math, prep);
}

template <int PD, int GD, class Math>
static bool dispatch_od(int od, const Launch& L, const Math& math, const DevPrep& prep) {
  // The output is either float32 (what the reference returns) or the parameter's own dtype.
  if (od == MXOPT_F32) { launch_update_t<PD, GD, MXOPT_F32, -1>(L, math, prep); return true; }
  if (od == PD) { launch_update_t<PD, GD, PD, -1>(L, math, prep); return true; }
  return false;
}

template <int PD, class Math>
static bool dispatch_gd(int gd, int od, const Launch& L, const Math& math, const DevPrep& prep) {
  switch (gd) {
    case MXOPT_F32: return dispatch_od<PD, MXOPT_F32>(od, L, math, prep);
    case MXOPT_BF16: return dispatch_od<PD, MXOPT_BF16>(od, L, math, prep);
    case MXOPT_F16: return dispatch_od<PD, MXOPT_F16>(od, L, math, prep);
  }
  return false;
}

template <class Math>
static bool dispatch_update(int pd, int gd, int od, const Launch& L, const Math& math, const DevPrep& prep) {
  switch (pd) {
    case MXOPT_F32: return dispatch_gd<MXOPT_F32>(gd, od, L, math, prep);
    case MXOPT_BF16: return dispatch_gd<MXOPT_BF16>(gd, od, L, math, prep);
    case MXOPT_F16: return dispatch_gd<MXOPT_F16>(gd, od, L, math, prep);
  }
  return false;
}

// Adam with the last micro-batch folded in: g is the float32 accumulation buffer, g2 any dtype.
template <int PD>
static bool adam_g2_for_pd(int od, int g2d, const Launch& L, const AdamMath& math, const DevPrep& prep) {
  if (od != PD && od != MXOPT_F32) return false;
  const bool same = od == PD;
  switch (g2d) {
    case MXOPT_F32:
      if (same) launch_update_t<PD, MXOPT_F32, PD, MXOPT_F32>(L, math, prep);
      else launch_update_t<PD, MXOPT_F32, MXOPT_F32, MXOPT_F32>(L, math, prep);
      return true;
    case MXOPT_BF16:
      if (same) launch_update_t<PD, MXOPT_F32, PD, MXOPT_BF16>(L, math, prep);
      else launch_update_t<PD, MXOPT_F32, MXOPT_F32, MXOPT_BF16>(L, math, prep);
      return true;
    case MXOPT_F16:
      if (same) launch_update_t<PD, MXOPT_F32, PD, MXOPT_F16>(L, math, prep);
      else launch_update_t<PD, MXOPT_F32, MXOPT_F32, MXOPT_F16>(L, math, prep);
      return true;
  }
  return false;
}

bool launch_adam(int pd, int gd, int od, int g2d, const Launch& L, const mxopt_adam_hp& hp, const DevPrep& prep) {
  if (g2d < 0) return dispatch_update(pd, gd, od, L, AdamMath{hp, prep_promotes(prep) ? MXOPT_F32 : gd}, prep);
  if (gd != MXOPT_F32) return false;
  switch (pd) {
    case MXOPT_F32: return adam_g2_for_pd<MXOPT_F32>(od, g2d, L, AdamMath{hp}, prep);
    case MXOPT_BF16: return adam_g2_for_pd<MXOPT_BF16>(od, g2d, L, AdamMath{hp}, prep);
    case MXOPT_F16: return adam_g2_for_pd<MXOPT_F16>(od, g2d, L, AdamMath{hp}, prep);
  }
  return false;
}
bool launch_sgd(int pd, int gd, int od, const Launch& L, const mxopt_sgd_hp& hp, const DevPrep& prep) {
  return dispatch_update(pd, gd, od, L, SgdMath{hp}, prep);
}
bool launch_rmsprop(int pd, int gd, int od, const Launch& L, const mxopt_rmsprop_hp& hp, const DevPrep& prep) {
  // with coupled decay the square is taken of g + wd * p, already float32 (rmsprop.rs:69-80)
  const int gsq_dtype = (prep_promotes(prep) || hp.has_weight_decay) ? MXOPT_F32 : gd;
  return dispatch_update(pd, gd, od, L, RmspropMath{hp, gsq_dtype}, prep);
}

template <int PD>
static bool plain_for_pd(int gd, int od, const Launch& L, float lr_p, float wd, int has_wd, bool g_promoted,
                         const DevPrep& prep) {
  if (od != PD) return false;  // apply_gradients always hands back the parameter's dtype
  const bool round_product = (PD != MXOPT_F32) && gd == PD && !g_promoted;
  if (round_product) {
    PlainSgdMath<PD, true> m{lr_p, wd, has_wd};
    return dispatch_gd<PD>(gd, od, L, m, prep);
  }
  PlainSgdMath<PD, false> m{lr_p, wd, has_wd};
  return dispatch_gd<PD>(gd, od, L, m, prep);
}

// Plain SGD on (float32 accumulation buffer + prep(pending gradient)); output in the parameter's dtype.
template <int PD>
static bool plain_pending_for_pd(int g2d, const Launch& L, float lr_p, float wd, int has_wd, const DevPrep& prep) {
  PlainSgdMath<PD, false> m{lr_p, wd, has_wd};
  switch (g2d) {
    case MXOPT_F32: launch_update_t<PD, MXOPT_F32, PD, MXOPT_F32>(L, m, prep); return true;
    case MXOPT_BF16: launch_update_t<PD, MXOPT_F32, PD, MXOPT_BF16>(L, m, prep); return true;
    case MXOPT_F16: launch_update_t<PD, MXOPT_F32, PD, MXOPT_F16>(L, m, prep); return true;
  }
  return false;
}

bool launch_sgd_plain_pending(int pd, int gd, int od, int g2d, const Launch& L, float lr_p, float wd, int has_wd,
                              const DevPrep& prep) {
  if (gd != MXOPT_F32 || od != pd) return false;
  switch (pd) {
    case MXOPT_F32: return plain_pending_for_pd<MXOPT_F32>(g2d, L, lr_p, wd, has_wd, prep);
    case MXOPT_BF16: return plain_pending_for_pd<MXOPT_BF16>(g2d, L, lr_p, wd, has_wd, prep);
    case MXOPT_F16: return plain_pending_for_pd<MXOPT_F16>(g2d, L, lr_p, wd, has_wd, prep);
  }
  return false;
}

bool launch_sgd_plain(int pd, int gd, int od, const Launch& L, float lr_p, float wd, int has_wd, bool g_promoted,
                      const DevPrep& prep) {
  switch (pd) {
    case MXOPT_F32: return plain_for_pd<MXOPT_F32>(gd, od, L, lr_p, wd, has_wd, g_promoted, prep);
    case MXOPT_BF16: return plain_for_pd<MXOPT_BF16>(gd, od, L, lr_p, wd, has_wd, g_promoted, prep);
    case MXOPT_F16: return plain_for_pd<MXOPT_F16>(gd, od, L, lr_p, wd, has_wd, g_promoted, prep);
  }
  return false;
}

template <int GD, int OD>
static void launch_transform_t(const Launch& L, const DevPrep& prep, int add) {
  if (L.nontemporal) {
    if (add) MXOPT_LAUNCH((transform_kernel<GD, OD, true, true>), L, prep);
    else MXOPT_LAUNCH((transform_kernel<GD, OD, true, false>), L, prep);
  } else {
    if (add) MXOPT_LAUNCH((transform_kernel<GD, OD, false, true>), L, prep);
    else MXOPT_LAUNCH((transform_kernel<GD, OD, false, false>), L, prep);
  }
}

template <int GD>
static bool transform_for_gd(int od, const Launch& L, const DevPrep& prep, int add) {
  if (od == MXOPT_F32) { launch_transform_t<GD, MXOPT_F32>(L, prep, add); return true; }
  if (od == GD) { launch_transform_t<GD, GD>(L, prep, add); return true; }
  return false;
}

bool launch_transform(int gd, int od, const Launch& L, const DevPrep& prep, int add) {
  switch (gd) {
    case MXOPT_F32: return transform_for_gd<MXOPT_F32>(od, L, prep, add);
    case MXOPT_BF16: return transform_for_gd<MXOPT_BF16>(od, L, prep, add);
    case MXOPT_F16: return transform_for_gd<MXOPT_F16>(od, L, prep, add);
  }
  return false;
}

}  // namespace mxopt
