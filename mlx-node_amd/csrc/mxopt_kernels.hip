// mxopt kernels for gfx950: multi-tensor optimizer updates, global-norm reduction,
// gradient transform and accumulation.  Every kernel walks a device-side chunk table so
// that thousands of tensors share one launch; each is a pure streaming pass whose roof is
// HBM bandwidth.  Build with -ffp-contract=off: one IEEE float32 rounding per reference op.
#include "mxopt_device.h"
#include "mxopt_launch.h"

namespace mxopt {

// ------------------------------------------------------------------------------------
// Math functors: the reference's op chains, one rounded float32 operation per line.
// ------------------------------------------------------------------------------------

// Adam::update_single (optimizers/adam.rs:77-108) / AdamW::update_single (adamw.rs:81-116).
struct AdamMath {
  mxopt_adam_hp hp;
  static constexpr bool kM = true;
  __device__ __forceinline__ bool uses_v(uint32_t) const { return true; }
  __device__ __forceinline__ bool reads_v(uint32_t) const { return true; }
  __device__ __forceinline__ void operator()(float& p, float g, float& m, float& v, float bc1, float bc2,
                                             uint32_t) const {
    float pd = hp.decoupled_decay ? p * hp.decay : p;
    float b1m = m * hp.beta1;
    float g1 = g * hp.one_minus_beta1;
    float nm = b1m + g1;
    float gsq = g * g;
    float b2v = v * hp.beta2;
    float g2 = gsq * hp.one_minus_beta2;
    float nv = b2v + g2;
    float mh = nm * bc1;  // bc == 1.0f reproduces "bias correction off" exactly
    float vh = nv * bc2;
    float den = sqrtf(vh) + hp.eps;
    float u = mh / den;
    float lu = u * hp.lr;
    p = pd - lu;
    m = nm;
    v = nv;
  }
};

// SGD::update_single (optimizers/sgd.rs:84-150).
struct SgdMath {
  mxopt_sgd_hp hp;
  static constexpr bool kM = false;
  __device__ __forceinline__ bool uses_v(uint32_t) const { return hp.has_momentum != 0; }
  __device__ __forceinline__ bool reads_v(uint32_t flags) const { return hp.has_momentum && !(flags & kTfFirst); }
  __device__ __forceinline__ void operator()(float& p, float g, float&, float& v, float, float,
                                             uint32_t flags) const {
    float ge = g;
    if (hp.has_weight_decay) {
      float w = p * hp.weight_decay;
      ge = g + w;
    }
    float u = ge;
    if (hp.has_momentum) {
      float nv;
      if (flags & kTfFirst) {
        nv = ge * 1.0f;
      } else {
        float mv = v * hp.momentum;
        float dg = ge * hp.one_minus_dampening;
        nv = mv + dg;
      }
      u = hp.nesterov ? nv + ge : nv;
      v = u;
    }
    float lu = u * hp.lr;
    p = p - lu;
  }
};

// RMSprop::update_single (optimizers/rmsprop.rs:67-112).
struct RmspropMath {
  mxopt_rmsprop_hp hp;
  static constexpr bool kM = false;
  __device__ __forceinline__ bool uses_v(uint32_t) const { return true; }
  __device__ __forceinline__ bool reads_v(uint32_t) const { return true; }
  __device__ __forceinline__ void operator()(float& p, float g, float&, float& v, float, float, uint32_t) const {
    float ge = g;
    if (hp.has_weight_decay) {
      float w = p * hp.weight_decay;
      ge = g + w;
    }
    float gsq = ge * ge;
    float av = v * hp.alpha;
    float g2 = gsq * hp.one_minus_alpha;
    float nv = av + g2;
    float den = sqrtf(nv) + hp.eps;
    float u = ge / den;
    float lu = u * hp.lr;
    p = p - lu;
    v = nv;
  }
};

// Qwen3Model::apply_gradients (models/qwen3/model.rs:2434-2451): lr already rounded to the
// parameter dtype on the host; ROUND_PRODUCT when p and g share a 16-bit dtype (the product
// is then itself a tensor of that dtype).
template <int PD, bool ROUND_PRODUCT>
struct PlainSgdMath {
  float lr_p, weight_decay;
  int has_weight_decay;
  static constexpr bool kM = false;
  __device__ __forceinline__ bool uses_v(uint32_t) const { return false; }
  __device__ __forceinline__ bool reads_v(uint32_t) const { return false; }
  __device__ __forceinline__ void operator()(float& p, float g, float&, float&, float, float, uint32_t) const {
    float ge = g;
    if (has_weight_decay) {  // sft/engine.rs:345-365: g + f32(wd)*p, promoted to float32
      float w = p * weight_decay;
      ge = g + w;
    }
    float s = lr_p * ge;
    if (ROUND_PRODUCT) s = Elem<PD>::round(s);
    p = p - s;
  }
};

// ------------------------------------------------------------------------------------
// Chunk lookup shared by all kernels
// ------------------------------------------------------------------------------------

struct ChunkView {
  DevTensor t;
  uint64_t start;  // first element of the chunk inside the tensor
  uint32_t len;    // elements in this chunk (kChunk except for the last one)
  uint32_t head;   // chunk 0 of a shifted tensor: elements [0, head) are this workgroup's too
  uint32_t tensor; // row of the table (0 for a single tensor passed by value)
  bool fast;       // full chunk of a 16-byte aligned (after the head) tensor: 128-bit path, fully unrolled
};

__device__ __forceinline__ ChunkView locate(const DevTensor* __restrict__ T, const DevChunk* __restrict__ C,
                                            const DevTensor& one, uint32_t c) {
  ChunkView cv;
  uint32_t index;
  if (C != nullptr) {  // table walk
    const DevChunk ch = C[c];
    cv.t = T[ch.tensor];
    cv.tensor = ch.tensor;
    index = ch.index;
  } else {             // a single tensor described in the kernel arguments: chunk c of `one`
    cv.t = one;
    cv.tensor = 0;
    index = c;
  }
  cv.start = (uint64_t)cv.t.head + (uint64_t)index * kChunk;
  const uint64_t left = cv.t.n > cv.start ? cv.t.n - cv.start : 0;
  cv.len = left < (uint64_t)kChunk ? (uint32_t)left : (uint32_t)kChunk;
  cv.head = index == 0 ? (cv.t.n < (uint64_t)cv.t.head ? (uint32_t)cv.t.n : cv.t.head) : 0u;
  cv.fast = !(cv.t.flags & kTfUnaligned) && cv.len == (uint32_t)kChunk;
  return cv;
}

// The engines skip the whole step when any gradient element is NaN/Inf (grpo/engine.rs:561-607):
// with a counter from the norm pass the update kernels honour that without a host round trip.
__device__ __forceinline__ bool skip_requested(const DevPrep& prep) {
  return prep.d_skip_if_nonzero != nullptr && *prep.d_skip_if_nonzero != 0ull;
}

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
  constexpr int E =
      (PD != MXOPT_F32 || GD != MXOPT_F32 || OD != MXOPT_F32 || (kHasG2 && G2D != MXOPT_F32)) ? 8 : 4;
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
      float m = Math::kM ? M[off] : 0.0f;
      float v = read_v ? V[off] : 0.0f;
      math(p, ge, m, v, bc1, bc2, flags);
      Elem<OD>::store(PO, off, p);
      if (Math::kM) M[off] = m;
      if (use_v) V[off] = v;
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
        store_group<OD, E, NT>(PO, off, p[j]);
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
template <int GD, int OD, bool NT>
__global__ __launch_bounds__(kThreads) void transform_kernel(const DevTensor* __restrict__ T,
                                                             const DevChunk* __restrict__ C, DevTensor one,
                                                             uint32_t nchunks, DevPrep prep, int add) {
  constexpr int E = (GD != MXOPT_F32 || OD != MXOPT_F32) ? 8 : 4;
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
#pragma unroll
      for (int j = 0; j < U; ++j) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
          g[j][e] = prep_all(pr, g[j][e]);
          if (add) g[j][e] = a[j][e] + g[j][e];
        }
        store_group<OD, E, NT>(GO, start + (uint64_t)(j * kThreads + tid) * E, g[j]);
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
// Sum of squares, pass 1 (one float64 partial per workgroup), optionally fused with the
// accumulation  acc = first ? g : acc + g.
//   MODE 0: square tensor.g                 MODE 1: square tensor.g_out
//   MODE 2: g_out = first ? g : acc + g, square the new contents (partials optional); acc is
//           tensor.p when set (out of place), else g_out itself
//   MODE 3: square (g_out + g) without storing it (the update kernel adds g again itself)
// AD: dtype of the stream that is squared / accumulated into; GD: dtype of g (MODE 2, 3).
// ------------------------------------------------------------------------------------

// A value clamp would turn +-Inf into a finite bound and hide it from the sum-based validity
// check; the engines test the raw values (grpo/engine.rs:563-569), so such a lane poisons its partial.

// The value whose square enters the norm.  Under a clamp the lane only has to remember that it met
// a NaN or an infinity (its partial is poisoned afterwards), so the clamp itself can be a single
// median-of-three that does not care about NaN.
__device__ __forceinline__ float norm_value(const PrepRegs& pr, float x, bool clamped, bool& bad) {
  if (!clamped) return prep_pre(pr, x);
  bad |= !__builtin_isfinite(x);
  if (pr.flags & kPrepPreMul) x = x * pr.pre_mul;
  return __builtin_amdgcn_fmed3f(x, pr.pre_lo, pr.pre_hi);
}

template <int AD, int GD>
__device__ __forceinline__ float accumulate_op(float acc, float g, bool first) {
  float s = first ? g : acc + g;
  // bf16 + bf16 -> bf16 and friends: the store rounds.  Squares are taken of the stored value.
  return Elem<AD>::round(s);
}

template <int MODE, int AD, int GD, bool NT>
struct SumsqChunk {
  static constexpr bool kTwoStreams = MODE >= 2;
  static constexpr int E = (AD != MXOPT_F32 || (kTwoStreams && GD != MXOPT_F32)) ? 8 : 4;
  static constexpr int U = kElemsPerLane / E;
  float x[U][E], g[U][E];

  static __device__ __forceinline__ const void* squared_stream(const ChunkView& cv) {
    if (MODE == 0) return cv.t.g;
    if (MODE == 2 && cv.t.p != nullptr) return cv.t.p;
    return cv.t.g_out;
  }

  __device__ __forceinline__ void load(const ChunkView& cv, uint32_t tid, bool first) {
    const void* X = squared_stream(cv);
#pragma unroll
    for (int j = 0; j < U; ++j) {
      const uint64_t off = cv.start + (uint64_t)(j * kThreads + tid) * E;
      if (MODE != 2 || !first) {
        load_group<AD, E, NT>(X, off, x[j]);
      } else {
#pragma unroll
        for (int e = 0; e < E; ++e) x[j][e] = 0.0f;
      }
      if (kTwoStreams) load_group<GD, E, NT>(cv.t.g, off, g[j]);
    }
  }

  // Returns this lane's float32 sum of squares over the chunk; stores the new sum in MODE 2.
  __device__ __forceinline__ float finish(const ChunkView& cv, const PrepRegs& pr, uint32_t tid, bool first) {
    float s32 = 0.0f;
    const bool clamped = (pr.flags & kPrepClampPre) != 0;
    bool hidden_inf = false;
#pragma unroll
    for (int j = 0; j < U; ++j) {
#pragma unroll
      for (int e = 0; e < E; ++e) {
        if (MODE == 2) x[j][e] = accumulate_op<AD, GD>(x[j][e], g[j][e], first);
        if (MODE == 3) x[j][e] = accumulate_op<AD, GD>(x[j][e], g[j][e], false);
        const float y = norm_value(pr, x[j][e], clamped, hidden_inf);
        s32 = fmaf(y, y, s32);
      }
      if (MODE == 2) store_group<AD, E, NT>(cv.t.g_out, cv.start + (uint64_t)(j * kThreads + tid) * E, x[j]);
    }
    return hidden_inf ? __builtin_nanf("") : s32;
  }

  // Partial or unaligned chunk.
  static __device__ __forceinline__ float slow(const ChunkView& cv, const PrepRegs& pr, uint32_t tid, bool first) {
    const void* X = squared_stream(cv);
    const void* G = cv.t.g;
    void* A = cv.t.g_out;
    float s32 = 0.0f;
    const bool clamped = (pr.flags & kPrepClampPre) != 0;
    const uint32_t ngroups = (cv.t.flags & kTfUnaligned) ? 0u : cv.len / E;
    for (uint32_t q = tid; q < ngroups; q += kThreads) {
      const uint64_t off = cv.start + (uint64_t)q * E;
      float x[E], g[E];
      if (MODE != 2 || !first) {
        load_group<AD, E, false>(X, off, x);
      } else {
#pragma unroll
        for (int e = 0; e < E; ++e) x[e] = 0.0f;
      }
      if (kTwoStreams) load_group<GD, E, false>(G, off, g);
#pragma unroll
      for (int e = 0; e < E; ++e) {
        if (MODE == 2) x[e] = accumulate_op<AD, GD>(x[e], g[e], first);
        if (MODE == 3) x[e] = accumulate_op<AD, GD>(x[e], g[e], false);
        bool bad = false;
        const float y = norm_value(pr, x[e], clamped, bad);
        s32 = bad ? __builtin_nanf("") : fmaf(y, y, s32);
      }
      if (MODE == 2) store_group<AD, E, false>(A, off, x);
    }
    for (uint32_t i = ngroups * E + tid; i < cv.len; i += kThreads) s32 = one_element(cv, pr, cv.start + i, first, s32);
    return s32;
  }

  // Element `off` of the tensor on its own: s32 + its square.
  static __device__ __forceinline__ float one_element(const ChunkView& cv, const PrepRegs& pr, uint64_t off,
                                                      bool first, float s32) {
    const void* X = squared_stream(cv);
    float x = (MODE != 2 || !first) ? Elem<AD>::load(X, off) : 0.0f;
    if (MODE == 2) {
      x = accumulate_op<AD, GD>(x, Elem<GD>::load(cv.t.g, off), first);
      Elem<AD>::store(cv.t.g_out, off, x);
    }
    if (MODE == 3) x = accumulate_op<AD, GD>(x, Elem<GD>::load(cv.t.g, off), false);
    bool bad = false;
    const float y = norm_value(pr, x, (pr.flags & kPrepClampPre) != 0, bad);
    return bad ? __builtin_nanf("") : fmaf(y, y, s32);
  }
};

template <int MODE, int AD, int GD, bool NT>
__global__ __launch_bounds__(kThreads) void sumsq_kernel(const DevTensor* __restrict__ T,
                                                         const DevChunk* __restrict__ C, DevTensor one,
                                                         uint32_t nchunks, DevPrep prep, int first_i,
                                                         double* __restrict__ partial_sum) {
  using Chunk = SumsqChunk<MODE, AD, GD, NT>;
  const PrepRegs pr = load_prep(prep);
  const uint32_t tid = threadIdx.x;
  const bool first = first_i != 0;
  double acc_sum = 0.0;

  uint32_t c = blockIdx.x;
  for (; c < nchunks; c += gridDim.x) {
    const ChunkView cv = locate(T, C, one, c);
    float s;
    if (cv.fast) {
      Chunk k;
      k.load(cv, tid, first);
      s = k.finish(cv, pr, tid, first);
    } else {
      s = Chunk::slow(cv, pr, tid, first);
    }
    if (tid < cv.head) s = Chunk::one_element(cv, pr, tid, first, s);
    // A lane's float32 partial covers <= 16 squares of one chunk; chunks are combined in float64.
    // A NaN/Inf element (or squares that overflow float32) makes the partial, and so the total,
    // non-finite: that is the validity check (the reference's sum-based one, grpo/engine.rs:1692-1698).
    acc_sum += (double)s;
  }

  if (partial_sum != nullptr) {
    unsigned long long unused = 0;
    block_sum(acc_sum, unused);
    if (tid == 0) partial_sum[blockIdx.x] = acc_sum;
  }
}

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
  for (int j = 0; j < KMAX; ++j) ps.x[j] = j < kx ? X[(size_t)j * ntensors + row] : nullptr;
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
    ps_regs[j].scale = has ? *scales.s[j] : 1.0f;
  }
  auto gradient = [&](float g, const float (&x)[KMAX]) {
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
      float m = Math::kM ? M[off] : 0.0f;
      float v = read_v ? V[off] : 0.0f;
      math(p, ge, m, v, bc1, bc2, flags);
      Elem<PD>::store(PO, off, p);
      if (Math::kM) M[off] = m;
      if (use_v) V[off] = v;
    };

    if (cv.fast && KMAX > 3) {
      // Many streams: one group per lane at a time (the same bytes in flight as four streams with the
      // whole chunk loaded up front, and half the registers).
#pragma unroll 1
      for (int j = 0; j < U; ++j) {
        const uint64_t off = start + (uint64_t)(j * kThreads + tid) * E;
        float p[E], g[E], x[KMAX][E], m[E], v[E];
        load_group<GD, E, false>(G, off, g);
#pragma unroll
        for (int k = 0; k < KMAX; ++k)
          if (k < kx) load_group<XD, E, false>(ps.x[k], off, x[k]);
        load_group<PD, E, false>(P, off, p);
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
    } else if (cv.fast) {
      float p[U][E], g[U][E], x[KMAX][U][E], m[U][E], v[U][E];
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const uint64_t off = start + (uint64_t)(j * kThreads + tid) * E;
        load_group<GD, E, false>(G, off, g[j]);
#pragma unroll
        for (int k = 0; k < KMAX; ++k)
          if (k < kx) load_group<XD, E, false>(ps.x[k], off, x[k][j]);
        load_group<PD, E, false>(P, off, p[j]);
        if (Math::kM) load_group<MXOPT_F32, E, false>(M, off, m[j]);
        if (read_v) load_group<MXOPT_F32, E, false>(V, off, v[j]);
      }
#pragma unroll
      for (int j = 0; j < U; ++j) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
          float xs[KMAX];
#pragma unroll
          for (int k = 0; k < KMAX; ++k) xs[k] = k < kx ? x[k][j][e] : 0.0f;
          math(p[j][e], gradient(g[j][e], xs), m[j][e], v[j][e], bc1, bc2, flags);
        }
      }
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const uint64_t off = start + (uint64_t)(j * kThreads + tid) * E;
        store_group<PD, E, false>(PO, off, p[j]);
        if (Math::kM) store_group<MXOPT_F32, E, false>(M, off, m[j]);
        if (use_v) store_group<MXOPT_F32, E, false>(V, off, v[j]);
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

// Sum of squares of prep_pre(g + x_0 + ...), nothing stored: the norm the update above will clip by.
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
    float s32 = 0.0f;
    bool bad = false;
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
          const float y = norm_value(pr, s, clamped, bad);
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
          const float y = norm_value(pr, s, clamped, bad);
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
    acc_sum += (double)(bad ? __builtin_nanf("") : s32);
  }

  unsigned long long unused = 0;
  block_sum(acc_sum, unused);
  if (tid == 0) partial_sum[blockIdx.x] = acc_sum;
}

// Pass 2: one workgroup folds the partials in a fixed order and derives norm and scale.
__global__ __launch_bounds__(kThreads) void norm_finish_kernel(const double* __restrict__ partial_sum,
                                                               uint32_t npartials, double max_norm, int has_max,
                                                               int clip_mode, mxopt_norm_result* __restrict__ out) {
  double s = 0.0;
  unsigned long long unused = 0;
  for (uint32_t i = threadIdx.x; i < npartials; i += kThreads) s += partial_sum[i];
  block_sum(s, unused);
  if (threadIdx.x == 0) {
    const double sumsq = s;
    const double norm = sqrt(sumsq);
    const float norm32 = (float)norm;
    float scale = 1.0f;
    if (has_max) {
      if (clip_mode == MXOPT_CLIP_ALWAYS_MULTIPLY) {
        // optimizers/mod.rs:87-96: all float32 scalars
        float d = norm32 + (float)1e-6;
        float q = (float)max_norm / d;
        scale = (q != q) ? q : fminf(q, 1.0f);  // a NaN norm gives a NaN scale
      } else {
        // gradients/mod.rs:255-270: float64 on the host, gradients unchanged when norm <= max
        if (!(norm <= max_norm)) scale = (float)(max_norm / (norm + 1e-6));
      }
    }
    out->sumsq = sumsq;
    out->norm = norm;
    out->norm_f32 = norm32;
    out->scale = scale;
    out->nonfinite = (sumsq - sumsq == 0.0) ? 0ull : 1ull;  // x - x is 0 exactly for finite x only
  }
}

// ------------------------------------------------------------------------------------
// Launchers (dtype dispatch)
// ------------------------------------------------------------------------------------

#define MXOPT_LAUNCH(kernel, L, ...)                                                                          \
  hipLaunchKernelGGL(kernel, dim3((L).grid), dim3(kThreads), 0, (L).stream, (L).tensors, (L).chunks, (L).one, \
                     (L).nchunks, __VA_ARGS__)

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
  if (g2d < 0) return dispatch_update(pd, gd, od, L, AdamMath{hp}, prep);
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
  return dispatch_update(pd, gd, od, L, RmspropMath{hp}, prep);
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

template <int GD>
static bool transform_for_gd(int od, const Launch& L, const DevPrep& prep, int add) {
  if (od == MXOPT_F32) {
    if (L.nontemporal) MXOPT_LAUNCH((transform_kernel<GD, MXOPT_F32, true>), L, prep, add);
    else MXOPT_LAUNCH((transform_kernel<GD, MXOPT_F32, false>), L, prep, add);
    return true;
  }
  if (od == GD) {
    if (L.nontemporal) MXOPT_LAUNCH((transform_kernel<GD, GD, true>), L, prep, add);
    else MXOPT_LAUNCH((transform_kernel<GD, GD, false>), L, prep, add);
    return true;
  }
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

template <int MODE, int AD, int GD>
static void launch_sumsq_t(const Launch& L, const DevPrep& prep, int first, double* ps) {
  if (L.nontemporal) MXOPT_LAUNCH((sumsq_kernel<MODE, AD, GD, true>), L, prep, first, ps);
  else MXOPT_LAUNCH((sumsq_kernel<MODE, AD, GD, false>), L, prep, first, ps);
}

template <int MODE, int AD>
static bool sumsq_for_ad(int gd, const Launch& L, const DevPrep& prep, int first, double* ps) {
  if (MODE < 2) { launch_sumsq_t<MODE, AD, MXOPT_F32>(L, prep, first, ps); return true; }
  switch (gd) {
    case MXOPT_F32: launch_sumsq_t<MODE, AD, MXOPT_F32>(L, prep, first, ps); return true;
    case MXOPT_BF16: launch_sumsq_t<MODE, AD, MXOPT_BF16>(L, prep, first, ps); return true;
    case MXOPT_F16: launch_sumsq_t<MODE, AD, MXOPT_F16>(L, prep, first, ps); return true;
  }
  return false;
}

template <int MODE>
static bool sumsq_for_mode(int ad, int gd, const Launch& L, const DevPrep& prep, int first, double* ps) {
  switch (ad) {
    case MXOPT_F32: return sumsq_for_ad<MODE, MXOPT_F32>(gd, L, prep, first, ps);
    case MXOPT_BF16: return sumsq_for_ad<MODE, MXOPT_BF16>(gd, L, prep, first, ps);
    case MXOPT_F16: return sumsq_for_ad<MODE, MXOPT_F16>(gd, L, prep, first, ps);
  }
  return false;
}

bool launch_sumsq(int mode, int ad, int gd, const Launch& L, const DevPrep& prep, int first, double* partial_sum) {
  switch (mode) {
    case 0: return sumsq_for_mode<0>(ad, gd, L, prep, first, partial_sum);
    case 1: return sumsq_for_mode<1>(ad, gd, L, prep, first, partial_sum);
    case 2: return sumsq_for_mode<2>(ad, gd, L, prep, first, partial_sum);
    case 3: return sumsq_for_mode<3>(ad, gd, L, prep, first, partial_sum);
  }
  return false;
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

bool launch_adam_list(int pd, int gd, int od, int xd, const Launch& L, const mxopt_adam_hp& hp, const DevPrep& prep) {
  if (od != pd) return false;
  switch (pd) {
    case MXOPT_F32: return update_list_for_pd<MXOPT_F32>(gd, xd, L, AdamMath{hp}, prep);
    case MXOPT_BF16: return update_list_for_pd<MXOPT_BF16>(gd, xd, L, AdamMath{hp}, prep);
    case MXOPT_F16: return update_list_for_pd<MXOPT_F16>(gd, xd, L, AdamMath{hp}, prep);
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

// ------------------------------------------------------------------------------------
// Synthetic data.  Element i = f(hash(seed, first_index + i)): integer hashing and exact integer
// -> float conversions followed by one or two rounded float32 operations, so that a host
// restatement produces the same bits for any slice of any buffer without materialising it.
// ------------------------------------------------------------------------------------

__device__ __forceinline__ uint64_t synth_hash(uint64_t seed, uint64_t idx) {
  uint64_t z = seed + (idx + 1ull) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

template <int OD>
__global__ __launch_bounds__(kThreads) void synth_kernel(void* __restrict__ out, uint64_t n, uint64_t seed,
                                                         uint64_t first_index, int dist, float a, float b) {
  for (uint64_t i = (uint64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (uint64_t)gridDim.x * kThreads) {
    const uint64_t z = synth_hash(seed, first_index + i);
    float x;
    if (dist == MXOPT_SYNTH_UNIFORM) {
      x = (float)(uint32_t)(z >> 40) * a;   // a = (hi - lo) / 2^24, b = lo
      x = x + b;
    } else {
      // sum of four 16-bit uniforms, centred: a bell shape on [-131070, 131070] with an exactly known variance
      const int32_t sum = (int32_t)((z & 0xffffu) + ((z >> 16) & 0xffffu) + ((z >> 32) & 0xffffu) + (z >> 48)) - 131070;
      x = (float)sum * a;                    // a = sigma / sqrt((65536^2 - 1) / 3)
      if (dist == MXOPT_SYNTH_NORMAL_OUTLIERS && synth_hash(seed ^ 0xA5A5A5A5A5A5A5A5ull, first_index + i) % 100ull == 0ull)
        x = x * b;                           // b = outlier multiplier
    }
    Elem<OD>::store(out, i, x);
  }
}

bool launch_synth(int od, void* out, uint64_t n, uint64_t seed, uint64_t first_index, int dist, float a, float b,
                  uint32_t grid, hipStream_t stream) {
  switch (od) {
    case MXOPT_F32: hipLaunchKernelGGL(synth_kernel<MXOPT_F32>, dim3(grid), dim3(kThreads), 0, stream, out, n, seed, first_index, dist, a, b); return true;
    case MXOPT_BF16: hipLaunchKernelGGL(synth_kernel<MXOPT_BF16>, dim3(grid), dim3(kThreads), 0, stream, out, n, seed, first_index, dist, a, b); return true;
    case MXOPT_F16: hipLaunchKernelGGL(synth_kernel<MXOPT_F16>, dim3(grid), dim3(kThreads), 0, stream, out, n, seed, first_index, dist, a, b); return true;
  }
  return false;
}

void launch_norm_finish(hipStream_t stream, const double* partial_sum, uint32_t npartials, double max_norm,
                        int has_max, int clip_mode, mxopt_norm_result* d_out) {
  hipLaunchKernelGGL(norm_finish_kernel, dim3(1), dim3(kThreads), 0, stream, partial_sum, npartials, max_norm,
                     has_max, clip_mode, d_out);
}

}  // namespace mxopt
