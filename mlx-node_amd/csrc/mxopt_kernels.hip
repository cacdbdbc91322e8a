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
// Update kernel
// ------------------------------------------------------------------------------------

template <int PD, int GD, int OD, class Math, int NT>
__global__ __launch_bounds__(kThreads) void update_kernel(const DevTensor* __restrict__ T,
                                                          const DevChunk* __restrict__ C, DevTensor one, uint32_t nchunks,
                                                          Math math, DevPrep prep) {
  constexpr int E = (PD != MXOPT_F32 || GD != MXOPT_F32 || OD != MXOPT_F32) ? 8 : 4;
  constexpr int U = kElemsPerLane / E;
  const PrepRegs pr = load_prep(prep);
  const uint32_t tid = threadIdx.x;

  for (uint32_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
    DevTensor tv;
    uint32_t index;
    if (C != nullptr) {  // table walk
      const DevChunk ch = C[c];
      tv = T[ch.tensor];
      index = ch.index;
    } else {             // a single tensor described in the kernel arguments: chunk c of `one`
      tv = one;
      index = c;
    }
    const DevTensor* t = &tv;
    const uint64_t start = (uint64_t)index * kChunk;
    const uint64_t left = t->n - start;
    const uint32_t len = left < (uint64_t)kChunk ? (uint32_t)left : (uint32_t)kChunk;
    const uint32_t flags = t->flags;
    const float bc1 = t->bc1, bc2 = t->bc2;
    const void* P = t->p;
    void* PO = t->p_out;
    const void* G = t->g;
    float* M = t->m;
    float* V = t->v;
    const bool use_v = math.uses_v(flags), read_v = math.reads_v(flags);

    if (!(flags & kTfUnaligned) && len == (uint32_t)kChunk) {
      // Full chunk: issue every load of the chunk before the first use.
      float p[U][E], g[U][E], m[U][E], v[U][E];
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const uint64_t off = start + (uint64_t)(j * kThreads + tid) * E;
        load_group<PD, E, (NT & 1) != 0>(P, off, p[j]);
        load_group<GD, E, (NT & 1) != 0>(G, off, g[j]);
        if (Math::kM) load_group<MXOPT_F32, E, (NT & 1) != 0>(M, off, m[j]);
        if (read_v) load_group<MXOPT_F32, E, (NT & 1) != 0>(V, off, v[j]);
      }
#pragma unroll
      for (int j = 0; j < U; ++j) {
#pragma unroll
        for (int e = 0; e < E; ++e) math(p[j][e], prep_all(pr, g[j][e]), m[j][e], v[j][e], bc1, bc2, flags);
      }
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const uint64_t off = start + (uint64_t)(j * kThreads + tid) * E;
        store_group<OD, E, (NT & 2) != 0>(PO, off, p[j]);
        if (Math::kM) store_group<MXOPT_F32, E, (NT & 2) != 0>(M, off, m[j]);
        if (use_v) store_group<MXOPT_F32, E, (NT & 2) != 0>(V, off, v[j]);
      }
    } else {
      // Last chunk of a tensor, or a tensor whose buffers are not 16-byte aligned.
      const uint32_t ngroups = (flags & kTfUnaligned) ? 0u : len / E;
      for (uint32_t q = tid; q < ngroups; q += kThreads) {
        const uint64_t off = start + (uint64_t)q * E;
        float p[E], g[E], m[E], v[E];
        load_group<PD, E, false>(P, off, p);
        load_group<GD, E, false>(G, off, g);
        if (Math::kM) load_group<MXOPT_F32, E, false>(M, off, m);
        if (read_v) load_group<MXOPT_F32, E, false>(V, off, v);
#pragma unroll
        for (int e = 0; e < E; ++e) math(p[e], prep_all(pr, g[e]), m[e], v[e], bc1, bc2, flags);
        store_group<OD, E, false>(PO, off, p);
        if (Math::kM) store_group<MXOPT_F32, E, false>(M, off, m);
        if (use_v) store_group<MXOPT_F32, E, false>(V, off, v);
      }
      for (uint32_t i = ngroups * E + tid; i < len; i += kThreads) {
        const uint64_t off = start + i;
        float p = Elem<PD>::load(P, off);
        float g = prep_all(pr, Elem<GD>::load(G, off));
        float m = Math::kM ? M[off] : 0.0f;
        float v = read_v ? V[off] : 0.0f;
        math(p, g, m, v, bc1, bc2, flags);
        Elem<OD>::store(PO, off, p);
        if (Math::kM) M[off] = m;
        if (use_v) V[off] = v;
      }
    }
  }
}

// ------------------------------------------------------------------------------------
// Gradient transform: g_out = prep(g)
// ------------------------------------------------------------------------------------

template <int GD, int OD, int NT>
__global__ __launch_bounds__(kThreads) void transform_kernel(const DevTensor* __restrict__ T,
                                                             const DevChunk* __restrict__ C, DevTensor one, uint32_t nchunks,
                                                             DevPrep prep) {
  constexpr int E = (GD != MXOPT_F32 || OD != MXOPT_F32) ? 8 : 4;
  constexpr int U = kElemsPerLane / E;
  const PrepRegs pr = load_prep(prep);
  const uint32_t tid = threadIdx.x;
  for (uint32_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
    DevTensor tv;
    uint32_t index;
    if (C != nullptr) {  // table walk
      const DevChunk ch = C[c];
      tv = T[ch.tensor];
      index = ch.index;
    } else {             // a single tensor described in the kernel arguments: chunk c of `one`
      tv = one;
      index = c;
    }
    const DevTensor* t = &tv;
    const uint64_t start = (uint64_t)index * kChunk;
    const uint64_t left = t->n - start;
    const uint32_t len = left < (uint64_t)kChunk ? (uint32_t)left : (uint32_t)kChunk;
    const uint32_t flags = t->flags;
    const void* G = t->g;
    void* GO = t->g_out;
    if (!(flags & kTfUnaligned) && len == (uint32_t)kChunk) {
      float g[U][E];
#pragma unroll
      for (int j = 0; j < U; ++j) load_group<GD, E, (NT & 1) != 0>(G, start + (uint64_t)(j * kThreads + tid) * E, g[j]);
#pragma unroll
      for (int j = 0; j < U; ++j) {
#pragma unroll
        for (int e = 0; e < E; ++e) g[j][e] = prep_all(pr, g[j][e]);
        store_group<OD, E, (NT & 2) != 0>(GO, start + (uint64_t)(j * kThreads + tid) * E, g[j]);
      }
    } else {
      const uint32_t ngroups = (flags & kTfUnaligned) ? 0u : len / E;
      for (uint32_t q = tid; q < ngroups; q += kThreads) {
        float g[E];
        load_group<GD, E, false>(G, start + (uint64_t)q * E, g);
#pragma unroll
        for (int e = 0; e < E; ++e) g[e] = prep_all(pr, g[e]);
        store_group<OD, E, false>(GO, start + (uint64_t)q * E, g);
      }
      for (uint32_t i = ngroups * E + tid; i < len; i += kThreads)
        Elem<OD>::store(GO, start + i, prep_all(pr, Elem<GD>::load(G, start + i)));
    }
  }
}

// ------------------------------------------------------------------------------------
// Sum of squares, pass 1 (one float64 partial per workgroup), optionally fused with the
// accumulation  acc = first ? g : acc + g.
//   MODE 0: read tensor.g          MODE 1: read tensor.g_out
//   MODE 2: accumulate into g_out and square the new contents (partials optional)
// ------------------------------------------------------------------------------------

template <int AD, int GD>
__device__ __forceinline__ float accumulate_op(float acc, float g, bool first) {
  float s = first ? g : acc + g;
  // bf16 + bf16 -> bf16 and friends: the store rounds.  Squares are taken of the stored value.
  return Elem<AD>::round(s);
}

template <int MODE, int AD, int GD, int NT>
__global__ __launch_bounds__(kThreads) void sumsq_kernel(const DevTensor* __restrict__ T,
                                                         const DevChunk* __restrict__ C, DevTensor one, uint32_t nchunks,
                                                         DevPrep prep, int first, double* __restrict__ partial_sum,
                                                         unsigned long long* __restrict__ partial_cnt) {
  // AD: dtype of the stream that is squared (g for MODE 0, g_out for MODE 1/2); GD: dtype of g (MODE 2).
  constexpr int E = (AD != MXOPT_F32 || (MODE == 2 && GD != MXOPT_F32)) ? 8 : 4;
  constexpr int U = kElemsPerLane / E;
  const PrepRegs pr = load_prep(prep);
  const uint32_t tid = threadIdx.x;
  double acc_sum = 0.0;
  unsigned long long acc_cnt = 0;

  for (uint32_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
    DevTensor tv;
    uint32_t index;
    if (C != nullptr) {  // table walk
      const DevChunk ch = C[c];
      tv = T[ch.tensor];
      index = ch.index;
    } else {             // a single tensor described in the kernel arguments: chunk c of `one`
      tv = one;
      index = c;
    }
    const DevTensor* t = &tv;
    const uint64_t start = (uint64_t)index * kChunk;
    const uint64_t left = t->n - start;
    const uint32_t len = left < (uint64_t)kChunk ? (uint32_t)left : (uint32_t)kChunk;
    const uint32_t flags = t->flags;
    const void* G = t->g;
    void* A = t->g_out;
    // MODE 2 reads the running sum from tensor.p when that is set (out-of-place accumulate:
    // g_out = p + g) and from g_out itself otherwise (in place).
    const void* X = (MODE == 0) ? G : ((MODE == 2 && t->p != nullptr) ? t->p : (const void*)A);
    float s32 = 0.0f;  // float32 partial of this lane's <=16 squares, widened once per chunk

    if (!(flags & kTfUnaligned) && len == (uint32_t)kChunk) {
      float x[U][E], g[U][E];
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const uint64_t off = start + (uint64_t)(j * kThreads + tid) * E;
        if (MODE != 2 || !first) load_group<AD, E, (NT & 1) != 0>(X, off, x[j]);
        else {
#pragma unroll
          for (int e = 0; e < E; ++e) x[j][e] = 0.0f;
        }
        if (MODE == 2) load_group<GD, E, (NT & 1) != 0>(G, off, g[j]);
      }
#pragma unroll
      for (int j = 0; j < U; ++j) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
          if (MODE == 2) x[j][e] = accumulate_op<AD, GD>(x[j][e], g[j][e], first);
          float y = prep_pre(pr, x[j][e]);
          acc_cnt += is_nonfinite(y);
          s32 = s32 + y * y;
        }
        if (MODE == 2) store_group<AD, E, (NT & 2) != 0>(A, start + (uint64_t)(j * kThreads + tid) * E, x[j]);
      }
    } else {
      const uint32_t ngroups = (flags & kTfUnaligned) ? 0u : len / E;
      for (uint32_t q = tid; q < ngroups; q += kThreads) {
        const uint64_t off = start + (uint64_t)q * E;
        float x[E], g[E];
        if (MODE != 2 || !first) load_group<AD, E, false>(X, off, x);
        else {
#pragma unroll
          for (int e = 0; e < E; ++e) x[e] = 0.0f;
        }
        if (MODE == 2) load_group<GD, E, false>(G, off, g);
#pragma unroll
        for (int e = 0; e < E; ++e) {
          if (MODE == 2) x[e] = accumulate_op<AD, GD>(x[e], g[e], first);
          float y = prep_pre(pr, x[e]);
          acc_cnt += is_nonfinite(y);
          s32 = s32 + y * y;
        }
        if (MODE == 2) store_group<AD, E, false>(A, off, x);
      }
      for (uint32_t i = ngroups * E + tid; i < len; i += kThreads) {
        const uint64_t off = start + i;
        float x = (MODE != 2 || !first) ? Elem<AD>::load(X, off) : 0.0f;
        if (MODE == 2) {
          x = accumulate_op<AD, GD>(x, Elem<GD>::load(G, off), first);
          Elem<AD>::store(A, off, x);
        }
        float y = prep_pre(pr, x);
        acc_cnt += is_nonfinite(y);
        s32 = s32 + y * y;
      }
    }
    acc_sum += (double)s32;
  }

  if (partial_sum != nullptr) {
    block_sum(acc_sum, acc_cnt);
    if (tid == 0) {
      partial_sum[blockIdx.x] = acc_sum;
      partial_cnt[blockIdx.x] = acc_cnt;
    }
  }
}

// Pass 2: one workgroup folds the partials in a fixed order and derives norm and scale.
__global__ __launch_bounds__(kThreads) void norm_finish_kernel(const double* __restrict__ partial_sum,
                                                               const unsigned long long* __restrict__ partial_cnt,
                                                               uint32_t npartials, double max_norm, int has_max,
                                                               int clip_mode, mxopt_norm_result* __restrict__ out) {
  double s = 0.0;
  unsigned long long c = 0;
  for (uint32_t i = threadIdx.x; i < npartials; i += kThreads) {
    s += partial_sum[i];
    c += partial_cnt[i];
  }
  block_sum(s, c);
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
    out->nonfinite = c;
  }
}

// ------------------------------------------------------------------------------------
// Launchers (dtype dispatch)
// ------------------------------------------------------------------------------------

#define MXOPT_LAUNCH(kernel, L, ...) \
  hipLaunchKernelGGL(kernel, dim3((L).grid), dim3(kThreads), 0, (L).stream, (L).tensors, (L).chunks, (L).one, (L).nchunks, __VA_ARGS__)

template <int PD, int GD, int OD, class Math>
static void launch_update_t(const Launch& L, const Math& math, const DevPrep& prep) {
  switch (L.nontemporal & 3) {
    case 0: MXOPT_LAUNCH((update_kernel<PD, GD, OD, Math, 0>), L, math, prep); break;
    case 1: MXOPT_LAUNCH((update_kernel<PD, GD, OD, Math, 1>), L, math, prep); break;
    case 2: MXOPT_LAUNCH((update_kernel<PD, GD, OD, Math, 2>), L, math, prep); break;
    case 3: MXOPT_LAUNCH((update_kernel<PD, GD, OD, Math, 3>), L, math, prep); break;
  }
}

template <int PD, int GD, class Math>
static bool dispatch_od(int od, const Launch& L, const Math& math, const DevPrep& prep) {
  // The output is either float32 (what the reference returns) or the parameter's own dtype.
  if (od == MXOPT_F32) { launch_update_t<PD, GD, MXOPT_F32>(L, math, prep); return true; }
  if (od == PD) { launch_update_t<PD, GD, PD>(L, math, prep); return true; }
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

bool launch_adam(int pd, int gd, int od, const Launch& L, const mxopt_adam_hp& hp, const DevPrep& prep) {
  return dispatch_update(pd, gd, od, L, AdamMath{hp}, prep);
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
static bool transform_for_gd(int od, const Launch& L, const DevPrep& prep) {
  if (od == MXOPT_F32) {
    if (L.nontemporal & 2) MXOPT_LAUNCH((transform_kernel<GD, MXOPT_F32, 2>), L, prep);
    else MXOPT_LAUNCH((transform_kernel<GD, MXOPT_F32, 0>), L, prep);
    return true;
  }
  if (od == GD) {
    if (L.nontemporal & 2) MXOPT_LAUNCH((transform_kernel<GD, GD, 2>), L, prep);
    else MXOPT_LAUNCH((transform_kernel<GD, GD, 0>), L, prep);
    return true;
  }
  return false;
}

bool launch_transform(int gd, int od, const Launch& L, const DevPrep& prep) {
  switch (gd) {
    case MXOPT_F32: return transform_for_gd<MXOPT_F32>(od, L, prep);
    case MXOPT_BF16: return transform_for_gd<MXOPT_BF16>(od, L, prep);
    case MXOPT_F16: return transform_for_gd<MXOPT_F16>(od, L, prep);
  }
  return false;
}

template <int MODE, int AD, int GD>
static void launch_sumsq_t(const Launch& L, const DevPrep& prep, int first, double* ps, unsigned long long* pc) {
  switch (L.nontemporal & 3) {
    case 0: MXOPT_LAUNCH((sumsq_kernel<MODE, AD, GD, 0>), L, prep, first, ps, pc); break;
    case 1: MXOPT_LAUNCH((sumsq_kernel<MODE, AD, GD, 1>), L, prep, first, ps, pc); break;
    case 2: MXOPT_LAUNCH((sumsq_kernel<MODE, AD, GD, 2>), L, prep, first, ps, pc); break;
    case 3: MXOPT_LAUNCH((sumsq_kernel<MODE, AD, GD, 3>), L, prep, first, ps, pc); break;
  }
}

template <int MODE, int AD>
static bool sumsq_for_ad(int gd, const Launch& L, const DevPrep& prep, int first, double* ps, unsigned long long* pc) {
  if (MODE != 2) { launch_sumsq_t<MODE, AD, MXOPT_F32>(L, prep, first, ps, pc); return true; }
  switch (gd) {
    case MXOPT_F32: launch_sumsq_t<MODE, AD, MXOPT_F32>(L, prep, first, ps, pc); return true;
    case MXOPT_BF16: launch_sumsq_t<MODE, AD, MXOPT_BF16>(L, prep, first, ps, pc); return true;
    case MXOPT_F16: launch_sumsq_t<MODE, AD, MXOPT_F16>(L, prep, first, ps, pc); return true;
  }
  return false;
}

template <int MODE>
static bool sumsq_for_mode(int ad, int gd, const Launch& L, const DevPrep& prep, int first, double* ps,
                           unsigned long long* pc) {
  switch (ad) {
    case MXOPT_F32: return sumsq_for_ad<MODE, MXOPT_F32>(gd, L, prep, first, ps, pc);
    case MXOPT_BF16: return sumsq_for_ad<MODE, MXOPT_BF16>(gd, L, prep, first, ps, pc);
    case MXOPT_F16: return sumsq_for_ad<MODE, MXOPT_F16>(gd, L, prep, first, ps, pc);
  }
  return false;
}

bool launch_sumsq(int mode, int ad, int gd, const Launch& L, const DevPrep& prep, int first, double* partial_sum,
                  unsigned long long* partial_cnt) {
  switch (mode) {
    case 0: return sumsq_for_mode<0>(ad, gd, L, prep, first, partial_sum, partial_cnt);
    case 1: return sumsq_for_mode<1>(ad, gd, L, prep, first, partial_sum, partial_cnt);
    case 2: return sumsq_for_mode<2>(ad, gd, L, prep, first, partial_sum, partial_cnt);
  }
  return false;
}

void launch_norm_finish(hipStream_t stream, const double* partial_sum, const unsigned long long* partial_cnt,
                        uint32_t npartials, double max_norm, int has_max, int clip_mode,
                        mxopt_norm_result* d_out) {
  hipLaunchKernelGGL(norm_finish_kernel, dim3(1), dim3(kThreads), 0, stream, partial_sum, partial_cnt, npartials,
                     max_norm, has_max, clip_mode, d_out);
}

}  // namespace mxopt
