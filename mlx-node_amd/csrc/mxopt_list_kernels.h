// Deferred accumulation, shared by the translation units that instantiate it: the update kernel over
// gradient streams that were never summed into a buffer, and its launch helpers.
#pragma once
#include "mxopt_kernels_common.h"

namespace mxopt {

// ------------------------------------------------------------------------------------
// Deferred accumulation.  The gradient is g + x_0 + ... + x_{kx-1}, added left to right in float32:
// the additions Qwen3Model::accumulate_gradients (models/qwen3/model.rs:2217-2243) would have made
// into a float32 buffer, made in registers instead, so that the buffer is never written or re-read.
// X[j * ntensors + row] is stream j of table row `row` (dtype XD); g is either the first micro-batch
// or a float32 buffer that already holds earlier ones.
// ------------------------------------------------------------------------------------

// KMAX: how many pending streams the instance has registers for (3 for up to four micro-batches, else 7).

template <int KMAX>
struct PendingStreams {
  const void* x[KMAX];
};

template <int KMAX>
__device__ __forceinline__ PendingStreams<KMAX> pending_of(const void* const* __restrict__ X, uint32_t ntensors, uint32_t row,
                                                     int kx) {
  PendingStreams<KMAX> ps;
#pragma unroll
  for (int j = 0; j < KMAX; ++j) ps.x[j] = j < kx ? (const void*)load_constant<uint64_t>(X, (size_t)j * ntensors + row) : nullptr;
  return ps;
}

template <int GD, int XD, int KMAX>
__device__ __forceinline__ float pending_sum_element(const void* G, const PendingStreams<KMAX>& ps, int kx, uint64_t off) {
  float s = Elem<GD>::load(G, off);
#pragma unroll
  for (int j = 0; j < KMAX; ++j)
    if (j < kx) s = s + Elem<XD>::load(ps.x[j], off);
  return s;
}

// Full chunks use streaming loads and stores (the rules of load_group / store_group apply: every line written
// here was read first).  Measured on the Qwen3-8B list against plain accesses: four-stream bf16 AdamW 37.0 ms
// instead of 37.5 - 38.4, the GRPO engine's four-stream update 18.9 instead of 19.4.  Not an option of the
// context: a second instance of every list kernel is not worth a knob nobody would turn.
constexpr bool kListNT = true;

template <int PD, int GD, int XD, int KMAX, class Math>
__global__ __launch_bounds__(kThreads) void update_list_kernel(const DevTensor* __restrict__ T,
                                                               const DevChunk* __restrict__ C, DevTensor one,
                                                               uint32_t nchunks, uint32_t ntensors,
                                                               const void* const* __restrict__ X, int kx,
                                                               StreamScales scales, Math math, DevPrep prep) {
  constexpr int E = (PD != MXOPT_F32 || GD != MXOPT_F32 || XD != MXOPT_F32) ? 8 : 4;
  constexpr int U = kElemsPerLane / E;
  if (skip_requested(prep)) return;
  const PrepRegs pr = load_prep(prep);
  const uint32_t tid = threadIdx.x;
  // Either prep(g + x0 + ...) or, with kPrepEachStream, prep_0(g) + prep_1(x0) + ...: every micro-batch
  // clamped and scaled by its own clip factor before it is added (grpo/engine.rs:636-661).
  const bool each = (pr.flags & kPrepEachStream) != 0;
  PrepRegs ps_regs[KMAX + 1];
#pragma unroll
  for (int j = 0; j <= KMAX; ++j) {
    ps_regs[j] = pr;
    const bool has = each && j <= kx && scales.s[j] != nullptr;
    ps_regs[j].has_scale = has;
    ps_regs[j].scale = has ? *constant_ptr<float>(scales.s[j]) : 1.0f;
  }
  if (pr.flags & kPrepFirstIsSum) {  // a buffer of earlier micro-batches, each prepared before it was added
    ps_regs[0].flags = 0;
    ps_regs[0].has_scale = false;
  }
  // The GRPO engine's case, every stream clamped and multiplied by its own factor (1 when it has none,
  // which changes no value), without a branch per stage and stream.
  const bool each_clamp_scale = each && (pr.flags & (kPrepPreMul | kPrepClampPre | kPrepClampPost)) == kPrepClampPre;
  const bool first_raw = (pr.flags & kPrepFirstIsSum) != 0;
  auto gradient = [&](float g, const float (&x)[KMAX]) {
    if (each_clamp_scale) {
      float s = first_raw ? g : clamp_keep_nan(g, pr.pre_lo, pr.pre_hi) * ps_regs[0].scale;
#pragma unroll
      for (int k = 0; k < KMAX; ++k)
        if (k < kx) s = s + clamp_keep_nan(x[k], pr.pre_lo, pr.pre_hi) * ps_regs[k + 1].scale;
      return s;
    }
    if (!each) {
      float s = g;
#pragma unroll
      for (int k = 0; k < KMAX; ++k)
        if (k < kx) s = s + x[k];
      return prep_all(pr, s);
    }
    float s = prep_all(ps_regs[0], g);
#pragma unroll
    for (int k = 0; k < KMAX; ++k)
      if (k < kx) s = s + prep_all(ps_regs[k + 1], x[k]);
    return s;
  };

  for (uint32_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
    const ChunkView cv = locate(T, C, one, c);
    const PendingStreams<KMAX> ps = pending_of<KMAX>(X, ntensors, cv.tensor, kx);
    const uint64_t start = cv.start;
    const uint32_t len = cv.len, flags = cv.t.flags;
    const float bc1 = cv.t.bc1, bc2 = cv.t.bc2;
    const void* P = cv.t.p;
    void* PO = cv.t.p_out;
    const void* G = cv.t.g;
    float* M = cv.t.m;
    float* V = cv.t.v;
    const bool use_v = math.uses_v(flags), read_v = math.reads_v(flags);
    auto one_element = [&](uint64_t off) {
      float p = Elem<PD>::load(P, off);
      float xs[KMAX];
#pragma unroll
      for (int k = 0; k < KMAX; ++k) xs[k] = k < kx ? Elem<XD>::load(ps.x[k], off) : 0.0f;
      const float ge = gradient(Elem<GD>::load(G, off), xs);
      float m = Math::kM ? Elem<MXOPT_F32>::load(M, off) : 0.0f;
      float v = read_v ? Elem<MXOPT_F32>::load(V, off) : 0.0f;
      math(p, ge, m, v, bc1, bc2, flags);
      Elem<PD>::store(PO, off, p);
      if (Math::kM) Elem<MXOPT_F32>::store(M, off, m);
      if (use_v) Elem<MXOPT_F32>::store(V, off, v);
    };

    if (cv.fast && KMAX > 3) {
      // Many streams: one group per lane at a time (the same bytes in flight as four streams with the
      // whole chunk loaded up front, and half the registers).
#pragma unroll 1
      for (int j = 0; j < U; ++j) {
        const uint64_t off = start + (uint64_t)(j * kThreads + tid) * E;
        float p[E], g[E], x[KMAX][E], m[E], v[E];
        load_group<GD, E, kListNT>(G, off, g);
#pragma unroll
        for (int k = 0; k < KMAX; ++k)
          if (k < kx) load_group<XD, E, kListNT>(ps.x[k], off, x[k]);
        load_group<PD, E, kListNT>(P, off, p);
        if (Math::kM) load_group<MXOPT_F32, E, kListNT>(M, off, m);
        if (read_v) load_group<MXOPT_F32, E, kListNT>(V, off, v);
#pragma unroll
        for (int e = 0; e < E; ++e) {
          float xs[KMAX];
#pragma unroll
          for (int k = 0; k < KMAX; ++k) xs[k] = k < kx ? x[k][e] : 0.0f;
          math(p[e], gradient(g[e], xs), m[e], v[e], bc1, bc2, flags);
        }
        store_group<PD, E, kListNT>(PO, off, p);
        if (Math::kM) store_group<MXOPT_F32, E, kListNT>(M, off, m);
        if (use_v) store_group<MXOPT_F32, E, kListNT>(V, off, v);
      }
    } else if (cv.fast) {
      float p[U][E], g[U][E], x[KMAX][U][E], m[U][E], v[U][E];
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const uint64_t off = start + (uint64_t)(j * kThreads + tid) * E;
        load_group<GD, E, kListNT>(G, off, g[j]);
#pragma unroll
        for (int k = 0; k < KMAX; ++k)
          if (k < kx) load_group<XD, E, kListNT>(ps.x[k], off, x[k][j]);
        load_group<PD, E, kListNT>(P, off, p[j]);
        if (Math::kM) load_group<MXOPT_F32, E, kListNT>(M, off, m[j]);
        if (read_v) load_group<MXOPT_F32, E, kListNT>(V, off, v[j]);
      }
      // One group at a time: its results are stored before the next group's values are unpacked, so that
      // only the loaded words of the later groups stay live (fewer registers, one more wave per SIMD).
#pragma unroll
      for (int j = 0; j < U; ++j) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
          float xs[KMAX];
#pragma unroll
          for (int k = 0; k < KMAX; ++k) xs[k] = k < kx ? x[k][j][e] : 0.0f;
          math(p[j][e], gradient(g[j][e], xs), m[j][e], v[j][e], bc1, bc2, flags);
        }
        const uint64_t off = start + (uint64_t)(j * kThreads + tid) * E;
        store_group<PD, E, kListNT>(PO, off, p[j]);
        if (Math::kM) store_group<MXOPT_F32, E, kListNT>(M, off, m[j]);
        if (use_v) store_group<MXOPT_F32, E, kListNT>(V, off, v[j]);
      }
    } else {
      const uint32_t ngroups = (flags & kTfUnaligned) ? 0u : len / E;
      for (uint32_t q = tid; q < ngroups; q += kThreads) {
        const uint64_t off = start + (uint64_t)q * E;
        float p[E], g[E], x[KMAX][E], m[E], v[E];
        load_group<PD, E, false>(P, off, p);
        load_group<GD, E, false>(G, off, g);
#pragma unroll
        for (int k = 0; k < KMAX; ++k)
          if (k < kx) load_group<XD, E, false>(ps.x[k], off, x[k]);
        if (Math::kM) load_group<MXOPT_F32, E, false>(M, off, m);
        if (read_v) load_group<MXOPT_F32, E, false>(V, off, v);
#pragma unroll
        for (int e = 0; e < E; ++e) {
          float xs[KMAX];
#pragma unroll
          for (int k = 0; k < KMAX; ++k) xs[k] = k < kx ? x[k][e] : 0.0f;
          math(p[e], gradient(g[e], xs), m[e], v[e], bc1, bc2, flags);
        }
        store_group<PD, E, false>(PO, off, p);
        if (Math::kM) store_group<MXOPT_F32, E, false>(M, off, m);
        if (use_v) store_group<MXOPT_F32, E, false>(V, off, v);
      }
      for (uint32_t i = ngroups * E + tid; i < len; i += kThreads) one_element(start + i);
    }
    if (tid < cv.head) one_element(tid);
  }
}

#define MXOPT_LAUNCH_LIST(kernel, L, ...)                                                                     \
  hipLaunchKernelGGL(kernel, dim3((L).grid), dim3(kThreads), 0, (L).stream, (L).tensors, (L).chunks, (L).one, \
                     (L).nchunks, (L).ntensors, (L).pending, (L).npending, __VA_ARGS__)
#define MXOPT_LAUNCH_UPDATE_LIST(kernel, L, ...) MXOPT_LAUNCH_LIST(kernel, L, (L).scales, __VA_ARGS__)

constexpr int kFewPending = 3;  // up to four micro-batches take the instance with fewer registers

template <int PD, int GD, int XD, class Math>
static void launch_update_list_t(const Launch& L, const Math& math, const DevPrep& prep) {
  if (L.npending <= kFewPending)
    MXOPT_LAUNCH_UPDATE_LIST((update_list_kernel<PD, GD, XD, kFewPending, Math>), L, math, prep);
  else
    MXOPT_LAUNCH_UPDATE_LIST((update_list_kernel<PD, GD, XD, MXOPT_MAX_PENDING, Math>), L, math, prep);
}

// g is either of the pending streams' dtype (the first micro-batch) or float32 (a buffer of earlier ones).
template <int PD, class Math>
static bool update_list_for_pd(int gd, int xd, const Launch& L, const Math& math, const DevPrep& prep) {
  if (gd != xd && gd != MXOPT_F32) return false;
  const bool same = gd == xd;
  switch (xd) {
    case MXOPT_F32:
      launch_update_list_t<PD, MXOPT_F32, MXOPT_F32>(L, math, prep);
      return true;
    case MXOPT_BF16:
      if (same) launch_update_list_t<PD, MXOPT_BF16, MXOPT_BF16>(L, math, prep);
      else launch_update_list_t<PD, MXOPT_F32, MXOPT_BF16>(L, math, prep);
      return true;
    case MXOPT_F16:
      if (same) launch_update_list_t<PD, MXOPT_F16, MXOPT_F16>(L, math, prep);
      else launch_update_list_t<PD, MXOPT_F32, MXOPT_F16>(L, math, prep);
      return true;
  }
  return false;
}

}  // namespace mxopt
