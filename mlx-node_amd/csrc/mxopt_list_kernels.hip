// mxopt kernels for gfx950, part 3: deferred accumulation -- the norm over gradient streams that were never
// summed into a buffer, and the Adam/AdamW and plain-SGD updates over them.
#include "mxopt_list_kernels.h"

namespace mxopt {

// Sum of squares of prep_pre(g + x_0 + ...), nothing stored: the norm the update kernel will clip by.
template <int GD, int XD, int KMAX, bool NT>
__global__ __launch_bounds__(kThreads) void sumsq_list_kernel(const DevTensor* __restrict__ T,
                                                              const DevChunk* __restrict__ C, DevTensor one,
                                                              uint32_t nchunks, uint32_t ntensors,
                                                              const void* const* __restrict__ X, int kx, DevPrep prep,
                                                              double* __restrict__ partial_sum) {
  constexpr int E = (GD != MXOPT_F32 || XD != MXOPT_F32) ? 8 : 4;
  constexpr int U = kElemsPerLane / E;
  const PrepRegs pr = load_prep(prep);
  const bool clamped = (pr.flags & kPrepClampPre) != 0;
  const uint32_t tid = threadIdx.x;
  double acc_sum = 0.0;

  for (uint32_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
    const ChunkView cv = locate(T, C, one, c);
    const PendingStreams<KMAX> ps = pending_of<KMAX>(X, ntensors, cv.tensor, kx);
    const void* G = cv.t.g;
    float s32 = 0.0f, poison = 0.0f;
    bool bad = false;
    // Full chunks: validity of the sum costs one multiply-add per element (s * 0 is NaN exactly for a NaN or an
    // infinity); under a clamp the lane's partial is poisoned afterwards, so the clamp need not care about NaN.
    auto fast_value = [&](float s) {
      poison = fmaf(s, 0.0f, poison);
      if (pr.flags & kPrepPreMul) s = s * pr.pre_mul;
      return clamped ? __builtin_amdgcn_fmed3f(s, pr.pre_lo, pr.pre_hi) : s;
    };
    auto one_element = [&](uint64_t off) {
      const float y = norm_value(pr, pending_sum_element<GD, XD, KMAX>(G, ps, kx, off), clamped, bad);
      s32 = fmaf(y, y, s32);
    };
    if (cv.fast && KMAX > 3) {
#pragma unroll 1
      for (int j = 0; j < U; ++j) {
        const uint64_t off = cv.start + (uint64_t)(j * kThreads + tid) * E;
        float g[E], x[KMAX][E];
        load_group<GD, E, NT>(G, off, g);
#pragma unroll
        for (int k = 0; k < KMAX; ++k)
          if (k < kx) load_group<XD, E, NT>(ps.x[k], off, x[k]);
#pragma unroll
        for (int e = 0; e < E; ++e) {
          float s = g[e];
#pragma unroll
          for (int k = 0; k < KMAX; ++k)
            if (k < kx) s = s + x[k][e];
          const float y = fast_value(s);
          s32 = fmaf(y, y, s32);
        }
      }
    } else if (cv.fast) {
      float g[U][E], x[KMAX][U][E];
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const uint64_t off = cv.start + (uint64_t)(j * kThreads + tid) * E;
        load_group<GD, E, NT>(G, off, g[j]);
#pragma unroll
        for (int k = 0; k < KMAX; ++k)
          if (k < kx) load_group<XD, E, NT>(ps.x[k], off, x[k][j]);
      }
#pragma unroll
      for (int j = 0; j < U; ++j) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
          float s = g[j][e];
#pragma unroll
          for (int k = 0; k < KMAX; ++k)
            if (k < kx) s = s + x[k][j][e];
          const float y = fast_value(s);
          s32 = fmaf(y, y, s32);
        }
      }
    } else {
      const uint32_t ngroups = (cv.t.flags & kTfUnaligned) ? 0u : cv.len / E;
      for (uint32_t q = tid; q < ngroups; q += kThreads) {
        const uint64_t off = cv.start + (uint64_t)q * E;
        float g[E], x[E];
        load_group<GD, E, false>(G, off, g);
#pragma unroll
        for (int k = 0; k < KMAX; ++k) {
          if (k < kx) {
            load_group<XD, E, false>(ps.x[k], off, x);
#pragma unroll
            for (int e = 0; e < E; ++e) g[e] = g[e] + x[e];
          }
        }
#pragma unroll
        for (int e = 0; e < E; ++e) {
          const float y = norm_value(pr, g[e], clamped, bad);
          s32 = fmaf(y, y, s32);
        }
      }
      for (uint32_t i = ngroups * E + tid; i < cv.len; i += kThreads) one_element(cv.start + i);
    }
    if (tid < cv.head) one_element(tid);
    // As in sumsq_kernel: float32 inside a chunk, float64 across chunks; a hidden NaN/Inf poisons the partial.
    acc_sum += (double)((bad || poison != poison) ? __builtin_nanf("") : s32);
  }

  unsigned long long unused = 0;
  block_sum(acc_sum, unused);
  if (tid == 0) partial_sum[blockIdx.x] = acc_sum;
}

bool launch_adam_list(int pd, int gd, int od, int xd, const Launch& L, const mxopt_adam_hp& hp, const DevPrep& prep) {
  if (od != pd) return false;
  // With no pending stream and no stage in front, the gradient reaches the square as it came: a 16-bit
  // tensor whose square is 16-bit too (as in launch_adam); any add or stage makes it float32 first.
  const AdamMath math{hp, (L.npending == 0 && !prep_promotes(prep)) ? gd : MXOPT_F32};
  switch (pd) {
    case MXOPT_F32: return update_list_for_pd<MXOPT_F32>(gd, xd, L, math, prep);
    case MXOPT_BF16: return update_list_for_pd<MXOPT_BF16>(gd, xd, L, math, prep);
    case MXOPT_F16: return update_list_for_pd<MXOPT_F16>(gd, xd, L, math, prep);
  }
  return false;
}

bool launch_sgd_plain_list(int pd, int gd, int od, int xd, const Launch& L, float lr_p, float wd, int has_wd,
                           const DevPrep& prep) {
  if (od != pd) return false;
  switch (pd) {
    case MXOPT_F32: return update_list_for_pd<MXOPT_F32>(gd, xd, L, PlainSgdMath<MXOPT_F32, false>{lr_p, wd, has_wd}, prep);
    case MXOPT_BF16: return update_list_for_pd<MXOPT_BF16>(gd, xd, L, PlainSgdMath<MXOPT_BF16, false>{lr_p, wd, has_wd}, prep);
    case MXOPT_F16: return update_list_for_pd<MXOPT_F16>(gd, xd, L, PlainSgdMath<MXOPT_F16, false>{lr_p, wd, has_wd}, prep);
  }
  return false;
}

template <int GD, int XD>
static void launch_sumsq_list_t(const Launch& L, const DevPrep& prep, double* ps) {
  if (L.npending <= kFewPending) {
    if (L.nontemporal) MXOPT_LAUNCH_LIST((sumsq_list_kernel<GD, XD, kFewPending, true>), L, prep, ps);
    else MXOPT_LAUNCH_LIST((sumsq_list_kernel<GD, XD, kFewPending, false>), L, prep, ps);
  } else {
    if (L.nontemporal) MXOPT_LAUNCH_LIST((sumsq_list_kernel<GD, XD, MXOPT_MAX_PENDING, true>), L, prep, ps);
    else MXOPT_LAUNCH_LIST((sumsq_list_kernel<GD, XD, MXOPT_MAX_PENDING, false>), L, prep, ps);
  }
}

bool launch_sumsq_list(int gd, int xd, const Launch& L, const DevPrep& prep, double* partial_sum) {
  if (gd != xd && gd != MXOPT_F32) return false;
  const bool same = gd == xd;
  switch (xd) {
    case MXOPT_F32: launch_sumsq_list_t<MXOPT_F32, MXOPT_F32>(L, prep, partial_sum); return true;
    case MXOPT_BF16:
      if (same) launch_sumsq_list_t<MXOPT_BF16, MXOPT_BF16>(L, prep, partial_sum);
      else launch_sumsq_list_t<MXOPT_F32, MXOPT_BF16>(L, prep, partial_sum);
      return true;
    case MXOPT_F16:
      if (same) launch_sumsq_list_t<MXOPT_F16, MXOPT_F16>(L, prep, partial_sum);
      else launch_sumsq_list_t<MXOPT_F32, MXOPT_F16>(L, prep, partial_sum);
      return true;
  }
  return false;
}

}  // namespace mxopt
