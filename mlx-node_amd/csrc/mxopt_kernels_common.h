// Device code shared by the kernel translation units: the reference's op chains as math functors,
// the chunk lookup, the norm's per-element value and the launch macro.
#pragma once

#include "mxopt_device.h"
#include "mxopt_launch.h"

namespace mxopt {

// ------------------------------------------------------------------------------------
// Math functors: the reference's op chains, one rounded float32 operation per line.
// ------------------------------------------------------------------------------------

// mlx square is a unary op and keeps its operand's dtype (mlx.cpp:2016-2020): the square of a 16-bit
// gradient that reaches it as it came (no prep stage, no pending sum, no coupled decay in front of it)
// is a 16-bit tensor, and only the multiply by the float32 scalar that follows promotes it.  g * g is
// exact in float32 for 16-bit inputs, so rounding it once is that tensor.
__device__ __forceinline__ float round_square_to(int dtype, float sq) {
  if (dtype == MXOPT_BF16) return Elem<MXOPT_BF16>::round(sq);
  if (dtype == MXOPT_F16) return Elem<MXOPT_F16>::round(sq);
  return sq;
}

// Adam::update_single (optimizers/adam.rs:77-108) / AdamW::update_single (adamw.rs:81-116).
struct AdamMath {
  mxopt_adam_hp hp;
  int gsq_dtype = MXOPT_F32;  // dtype the square of the gradient is rounded to (adamw.rs:92, adam.rs:88)
  static constexpr bool kM = true;
  __device__ __forceinline__ bool uses_v(uint32_t) const { return true; }
  __device__ __forceinline__ bool reads_v(uint32_t) const { return true; }
  __device__ __forceinline__ void operator()(float& p, float g, float& m, float& v, float bc1, float bc2,
                                             uint32_t) const {
    float pd = hp.decoupled_decay ? p * hp.decay : p;
    float b1m = m * hp.beta1;
    float g1 = g * hp.one_minus_beta1;
    float nm = b1m + g1;
    float gsq = round_square_to(gsq_dtype, g * g);
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
  int gsq_dtype = MXOPT_F32;  // as in AdamMath (rmsprop.rs:80)
  static constexpr bool kM = false;
  __device__ __forceinline__ bool uses_v(uint32_t) const { return true; }
  __device__ __forceinline__ bool reads_v(uint32_t) const { return true; }
  __device__ __forceinline__ void operator()(float& p, float g, float&, float& v, float, float, uint32_t) const {
    float ge = g;
    if (hp.has_weight_decay) {
      float w = p * hp.weight_decay;
      ge = g + w;
    }
    float gsq = round_square_to(gsq_dtype, ge * ge);
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
  if (C != nullptr) {  // table walk: two dependent scalar loads
    const DevChunk ch = load_constant<DevChunk>(C, c);
    cv.t = load_constant<DevTensor>(T, ch.tensor);
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
// Bit 0 of mxopt_norm_result.nonfinite is "some element was a NaN or an infinity"; bit 1 (finite elements
// whose squares overflowed) does not stop a step: the reference clips such gradients to zero and goes on.
__device__ __forceinline__ bool skip_requested(const DevPrep& prep) {
  return prep.d_skip_if_nonzero != nullptr && (*constant_ptr<unsigned long long>(prep.d_skip_if_nonzero) & 1ull) != 0ull;
}

// A value clamp would turn +-Inf into a finite bound and hide it from the sum-based validity
// check; the engines test the raw values (grpo/engine.rs:563-569), so such a lane poisons its partial.

// The value whose square enters the norm.  Under a clamp the lane only has to remember that it met
// a NaN or an infinity (its partial is poisoned afterwards), so the clamp itself can be a single
// median-of-three that does not care about NaN.
__device__ __forceinline__ float norm_value(const PrepRegs& pr, float x, bool clamped, bool& bad) {
  bad |= !__builtin_isfinite(x);
  if (!clamped) return prep_pre(pr, x);
  if (pr.flags & kPrepPreMul) x = x * pr.pre_mul;
  return __builtin_amdgcn_fmed3f(x, pr.pre_lo, pr.pre_hi);
}

#define MXOPT_LAUNCH(kernel, L, ...)                                                                          \
  hipLaunchKernelGGL(kernel, dim3((L).grid), dim3(kThreads), 0, (L).stream, (L).tensors, (L).chunks, (L).one, \
                     (L).nchunks, __VA_ARGS__)

}  // namespace mxopt
