// mxopt kernels for gfx950, part 2: global-norm reduction (optionally fused with gradient accumulation)
// and the synthetic-data generator.
#include <mutex>
#include <type_traits>

#include "mxopt_kernels_common.h"
#include "mxopt_gauss_table.h"

namespace mxopt {

// ------------------------------------------------------------------------------------
// Sum of squares, pass 1 (one float64 partial per workgroup), optionally fused with the
// accumulation  acc = first ? g : acc + g.
//   MODE 0: square tensor.g                 MODE 1: square tensor.g_out
//   MODE 2: g_out = first ? g : acc + g, square the new contents (partials optional); acc is
//           tensor.p when set (out of place), else g_out itself
//   MODE 3: square (g_out + g) without storing it (the update kernel adds g again itself)
// AD: dtype of the stream that is squared / accumulated into; GD: dtype of g (MODE 2, 3).
// ------------------------------------------------------------------------------------


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

  // The new sum of group j.  A streaming store pays off where the pass has just read the line it writes; the
  // first pass of a cycle writes lines nobody read (acc = widen(g)), and there streaming stores cost 60 % more
  // time (measured on the bf16 -> float32 pass, whose float32 stores come in sector-sharing pairs that
  // store_group no longer streams anyway; single-piece stores were not measured on their own).
  static __device__ __forceinline__ void store_sum(const ChunkView& cv, uint32_t tid, int j, bool first,
                                                   const float (&v)[E]) {
    const uint64_t off = cv.start + (uint64_t)(j * kThreads + tid) * E;
    if (first) store_group<AD, E, false>(cv.t.g_out, off, v);
    else store_group<AD, E, NT>(cv.t.g_out, off, v);
  }

  // Returns this lane's float32 sum of squares over the chunk; stores the new sum in MODE 2.
  __device__ __forceinline__ float finish(const ChunkView& cv, const PrepRegs& pr, uint32_t tid, bool first) {
    float s32 = 0.0f;
    if ((pr.flags & (kPrepClampPre | kPrepPreMul)) == kPrepClampPre) {
      // A clamp and nothing else before the norm (the GRPO engine's validity + norm pass).  The flags are
      // tested once per chunk, not per element, and the raw values' validity costs one multiply-add each:
      // x * 0 is NaN exactly when x is a NaN or an infinity, which the clamp would have hidden.
      float poison = 0.0f;
#pragma unroll
      for (int j = 0; j < U; ++j) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
          if (MODE == 2) x[j][e] = accumulate_op<AD, GD>(x[j][e], g[j][e], first);
          if (MODE == 3) x[j][e] = accumulate_op<AD, GD>(x[j][e], g[j][e], false);
          poison = fmaf(x[j][e], 0.0f, poison);
          const float y = __builtin_amdgcn_fmed3f(x[j][e], pr.pre_lo, pr.pre_hi);
          s32 = fmaf(y, y, s32);
        }
        if (MODE == 2) store_sum(cv, tid, j, first, x[j]);
      }
      return poison != poison ? __builtin_nanf("") : s32;
    }
    // No clamp: x * 0 is NaN exactly for a NaN or an infinity, so one multiply-add per element tells an
    // invalid element (the partial becomes NaN) from squares of finite elements that overflow float32 (+Inf).
    if (!(pr.flags & kPrepClampPre)) {
      float poison = 0.0f;
      auto body = [&](auto with_mul) {  // the stage flag is tested once per chunk, not per element
#pragma unroll
        for (int j = 0; j < U; ++j) {
#pragma unroll
          for (int e = 0; e < E; ++e) {
            if (MODE == 2) x[j][e] = accumulate_op<AD, GD>(x[j][e], g[j][e], first);
            if (MODE == 3) x[j][e] = accumulate_op<AD, GD>(x[j][e], g[j][e], false);
            poison = fmaf(x[j][e], 0.0f, poison);
            const float y = decltype(with_mul)::value ? x[j][e] * pr.pre_mul : x[j][e];
            s32 = fmaf(y, y, s32);
          }
          if (MODE == 2) store_sum(cv, tid, j, first, x[j]);
        }
      };
      if (pr.flags & kPrepPreMul) body(std::true_type{}); else body(std::false_type{});
      return poison != poison ? __builtin_nanf("") : s32;
    }
    bool hidden_inf = false;
#pragma unroll
    for (int j = 0; j < U; ++j) {
#pragma unroll
      for (int e = 0; e < E; ++e) {
        if (MODE == 2) x[j][e] = accumulate_op<AD, GD>(x[j][e], g[j][e], first);
        if (MODE == 3) x[j][e] = accumulate_op<AD, GD>(x[j][e], g[j][e], false);
        const float y = norm_value(pr, x[j][e], true, hidden_inf);
        s32 = fmaf(y, y, s32);
      }
      if (MODE == 2) store_sum(cv, tid, j, first, x[j]);
    }
    return hidden_inf ? __builtin_nanf("") : s32;
  }

  // MODE 2 when nobody asked for the norm: the new sum is stored and nothing is squared.  With 16-bit
  // gradients the squares (widen, transform, multiply-add per element) cost more instruction issue than
  // the pass has to spare beside its memory traffic.
  __device__ __forceinline__ void finish_store_only(const ChunkView& cv, uint32_t tid, bool first) {
#pragma unroll
    for (int j = 0; j < U; ++j) {
#pragma unroll
      for (int e = 0; e < E; ++e) x[j][e] = accumulate_op<AD, GD>(x[j][e], g[j][e], first);
      store_sum(cv, tid, j, first, x[j]);
    }
  }

  // Partial or unaligned chunk.
  static __device__ __forceinline__ float slow(const ChunkView& cv, const PrepRegs& pr, uint32_t tid, bool first) {
    const void* X = squared_stream(cv);
    const void* G = cv.t.g;
    void* A = cv.t.g_out;
    float s32 = 0.0f;
    const bool clamped = (pr.flags & kPrepClampPre) != 0;
    bool bad = false;
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
        const float y = norm_value(pr, x[e], clamped, bad);
        s32 = fmaf(y, y, s32);
      }
      if (MODE == 2) store_group<AD, E, false>(A, off, x);
    }
    if (bad) s32 = __builtin_nanf("");
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
  if (MODE == 2 && partial_sum == nullptr) {  // accumulation only
    for (; c < nchunks; c += gridDim.x) {
      const ChunkView cv = locate(T, C, one, c);
      if (cv.fast) {
        Chunk k;
        k.load(cv, tid, first);
        k.finish_store_only(cv, tid, first);
      } else {
        (void)Chunk::slow(cv, pr, tid, first);
      }
      if (tid < cv.head) (void)Chunk::one_element(cv, pr, tid, first, 0.0f);
    }
    return;
  }
  for (; c < nchunks; c += gridDim.x) {
    const ChunkView cv = locate(T, C, one, c);
    float s;
    if (MODE < 2 && AD != MXOPT_F32 && cv.fast && pr.flags == 0) {
      // 16-bit values squared as they are: one packed dot product per pair (v_dot2_f32_bf16 / v_dot2_f32_f16)
      // instead of two widenings and two multiply-adds; with twice the elements per byte the widening path
      // is bound by instruction issue (6.3 against 6.8 TB/s).  The norm is held to 1e-5, not bitwise; NaN
      // and Inf propagate into the partial sum as before.
      const MXOPT_GLOBAL u32x4* q =
          global_ptr<u32x4>((const void*)((const uint16_t*)Chunk::squared_stream(cv) + cv.start)) + tid;
      u32x4 r[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) r[j] = NT ? __builtin_nontemporal_load(q + j * kThreads) : q[j * kThreads];
      s = 0.0f;
      // validity: a pair times (0, 0) is NaN exactly when one of the two is a NaN or an infinity
      float poison = 0.0f;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const uint32_t w[4] = {r[j].x, r[j].y, r[j].z, r[j].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (AD == MXOPT_BF16) {
            const bf16x2_t v = __builtin_bit_cast(bf16x2_t, w[e]);
            s = __builtin_amdgcn_fdot2_f32_bf16(v, v, s, false);
            poison = __builtin_amdgcn_fdot2_f32_bf16(v, __builtin_bit_cast(bf16x2_t, 0u), poison, false);
          } else {
            const f16x2_t v = __builtin_bit_cast(f16x2_t, w[e]);
            s = __builtin_amdgcn_fdot2(v, v, s, false);
            poison = __builtin_amdgcn_fdot2(v, __builtin_bit_cast(f16x2_t, 0u), poison, false);
          }
        }
      }
      if (poison != poison) s = __builtin_nanf("");
    } else if (cv.fast) {
      Chunk k;
      k.load(cv, tid, first);
      s = k.finish(cv, pr, tid, first);
    } else {
      s = Chunk::slow(cv, pr, tid, first);
    }
    if (tid < cv.head) s = Chunk::one_element(cv, pr, tid, first, s);
    // A lane's float32 partial covers <= 16 squares of one chunk; chunks are combined in float64.
    // A NaN/Inf element makes the partial, and so the total, NaN: the engines' validity check
    // (grpo/engine.rs:563-569).  Squares of finite elements that overflow float32 make it +Inf instead.
    acc_sum += (double)s;
  }

  if (partial_sum != nullptr) {
    unsigned long long unused = 0;
    block_sum(acc_sum, unused);
    if (tid == 0) partial_sum[blockIdx.x] = acc_sum;
  }
}


// ------------------------------------------------------------------------------------
// The plain norm of a 16-bit stream (no stage in front of the squares), several chunks per trip.  A trip of
// the general kernel waits for its table entry, then its descriptor, then its data; with 2 bytes per element
// that data is 8 KB per workgroup (half of it for the last chunk of a small tensor), too little to cover the
// three round trips, and a list of ten thousand small tensors ran at 4.3 TB/s where one flat tensor reached
// 6.2.  Here a workgroup takes NCH chunks per trip: their descriptors are fetched together (scalar loads),
// then all their data loads are issued before the first square is taken, and the descriptors of the next trip
// are on their way meanwhile.  Nothing in a trip is conditional on a lane's data being there: lanes without
// work load 16 bytes of the table itself and discard them, so the code is one straight line the compiler can
// count outstanding loads in.  (A loop that keeps loads in flight across its back edge was tried first: the
// compiler waits for all of them at the top of every trip.)
//   per lane and chunk: two 16-byte pieces of the chunk's full 8-element groups and one single element (lanes
//   0-6: the up to 7 elements behind the last full group; lanes 8-14: the up to 7 elements in front of a
//   shifted tensor's first chunk).  A table with a tensor whose streams disagree about alignment (element-wise
//   path) is not launched here.
// WHICH: 0 squares tensor.g, 1 tensor.g_out.
// ------------------------------------------------------------------------------------
template <int AD, int WHICH, bool NT, int NCH>
__global__ __launch_bounds__(kThreads) void sumsq16_multi_kernel(const DevTensor* __restrict__ T,
                                                                 const DevChunk* __restrict__ C, DevTensor one,
                                                                 uint32_t nchunks, DevPrep prep, int,
                                                                 double* __restrict__ partial_sum) {
  static_assert(AD != MXOPT_F32, "16-bit streams only");
  using Chunk = SumsqChunk<WHICH, AD, MXOPT_F32, NT>;
  (void)prep;  // no stage (the launcher's condition)
  const uint32_t tid = threadIdx.x;
  // at least 16 readable bytes in either case: a table has one 80-byte descriptor or more, a single tensor's
  // launch no table but the partial sums
  const void* safe = T != nullptr ? (const void*)T : (const void*)partial_sum;
  double acc_sum = 0.0;

  struct InFlight {
    u32x4 r[2];
    uint32_t single;  // one 16-bit element, or 0
  };
  // Starts the loads of one chunk.  `live` false: every lane reads the safe address.
  auto issue = [&](const ChunkView& cv, bool live) {
    InFlight f;
    const uint32_t ng = live ? cv.len / 8u : 0u;
    const uint32_t rem = live ? cv.len - ng * 8u : 0u;
    const uint32_t head = live ? cv.head : 0u;
    const uint16_t* X = (const uint16_t*)Chunk::squared_stream(cv);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint32_t q = tid + (uint32_t)j * kThreads;
      const void* a = q < ng ? (const void*)(X + cv.start + (uint64_t)q * 8u) : safe;
      const MXOPT_GLOBAL u32x4* gp = global_ptr<u32x4>(a);
      f.r[j] = NT ? __builtin_nontemporal_load(gp) : *gp;
    }
    const bool tail_lane = tid < rem, head_lane = tid >= 8u && tid - 8u < head;
    const void* a1 = tail_lane ? (const void*)(X + cv.start + (uint64_t)ng * 8u + tid)
                               : head_lane ? (const void*)(X + (tid - 8u)) : safe;
    f.single = *global_ptr<uint16_t>(a1);
    return f;
  };
  // This lane's float32 sum of squares over what `issue` loaded for it (NaN when it met a NaN or an infinity).
  auto consume = [&](const ChunkView& cv, bool live, const InFlight& f) {
    const uint32_t ng = live ? cv.len / 8u : 0u;
    const uint32_t rem = live ? cv.len - ng * 8u : 0u;
    const uint32_t head = live ? cv.head : 0u;
    float s = 0.0f, poison = 0.0f;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const bool ok = tid + (uint32_t)j * kThreads < ng;
      const uint32_t w[4] = {ok ? f.r[j].x : 0u, ok ? f.r[j].y : 0u, ok ? f.r[j].z : 0u, ok ? f.r[j].w : 0u};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (AD == MXOPT_BF16) {
          const bf16x2_t v = __builtin_bit_cast(bf16x2_t, w[e]);
          s = __builtin_amdgcn_fdot2_f32_bf16(v, v, s, false);
          poison = __builtin_amdgcn_fdot2_f32_bf16(v, __builtin_bit_cast(bf16x2_t, 0u), poison, false);
        } else {
          const f16x2_t v = __builtin_bit_cast(f16x2_t, w[e]);
          s = __builtin_amdgcn_fdot2(v, v, s, false);
          poison = __builtin_amdgcn_fdot2(v, __builtin_bit_cast(f16x2_t, 0u), poison, false);
        }
      }
    }
    const bool has_single = tid < rem || (tid >= 8u && tid - 8u < head);
    const float x = has_single ? Elem<AD>::unpack(f.single) : 0.0f;
    s = fmaf(x, x, s);
    poison = fmaf(x, 0.0f, poison);
    return poison != poison ? __builtin_nanf("") : s;
  };

  const uint32_t stride = gridDim.x;
  ChunkView cv[NCH], ahead[NCH];
  bool live[NCH], live_ahead[NCH];
  auto fetch = [&](uint32_t c0, ChunkView (&v)[NCH], bool (&l)[NCH]) {
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
      const uint64_t ck = (uint64_t)c0 + (uint64_t)k * stride;
      l[k] = ck < nchunks;
      v[k] = locate(T, C, one, l[k] ? (uint32_t)ck : blockIdx.x);  // a dead slot re-reads the first descriptor
    }
  };
  uint32_t c = blockIdx.x;
  if (c < nchunks) fetch(c, ahead, live_ahead);
  while (c < nchunks) {
#pragma unroll
    for (int k = 0; k < NCH; ++k) { cv[k] = ahead[k]; live[k] = live_ahead[k]; }
    InFlight f[NCH];
#pragma unroll
    for (int k = 0; k < NCH; ++k) f[k] = issue(cv[k], live[k]);
    const uint64_t next = (uint64_t)c + (uint64_t)NCH * stride;
    if (next < nchunks) fetch((uint32_t)next, ahead, live_ahead);  // scalar loads: they do not wait for the data
#pragma unroll
    for (int k = 0; k < NCH; ++k) acc_sum += (double)consume(cv[k], live[k], f[k]);
    if (next >= nchunks) break;
    c = (uint32_t)next;
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
    // NaN: some element was a NaN or an infinity (1).  +Inf: every element was finite and their squares left
    // float32 range (2): the reference goes on with a clip factor of 0 there, and so does `scale` above.
    out->nonfinite = (sumsq != sumsq) ? 1ull : (sumsq - sumsq == 0.0) ? 0ull : 2ull;
  }
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

template <int AD, int NCH>
static void launch_sumsq16_multi(int which, const Launch& L, const DevPrep& prep, double* ps) {
  if (which == 0) {
    if (L.nontemporal) MXOPT_LAUNCH((sumsq16_multi_kernel<AD, 0, true, NCH>), L, prep, 0, ps);
    else MXOPT_LAUNCH((sumsq16_multi_kernel<AD, 0, false, NCH>), L, prep, 0, ps);
  } else {
    if (L.nontemporal) MXOPT_LAUNCH((sumsq16_multi_kernel<AD, 1, true, NCH>), L, prep, 0, ps);
    else MXOPT_LAUNCH((sumsq16_multi_kernel<AD, 1, false, NCH>), L, prep, 0, ps);
  }
}

bool launch_sumsq(int mode, int ad, int gd, const Launch& L, const DevPrep& prep, int first, double* partial_sum) {
  // The plain norm of a 16-bit stream over many small tensors has a kernel of its own (option pipelined_norm:
  // 0 never, 1 always, 2 / 4 = that many chunks per trip where the chunks are partly empty).  Measured on
  // 10,000 tensors of 64 ... 65,536 elements: 45.9 against 53.1 us; on the Qwen3-1.7B list, whose chunks are
  // full, the general kernel is the leaner one (0.581 against 0.593 ms).
  const bool wanted = L.pipelined_norm == 1 || (L.pipelined_norm > 1 && L.partial_chunks);
  if (mode < 2 && partial_sum != nullptr && prep.flags == 0 && wanted && !L.any_unaligned) {
    if (ad == MXOPT_BF16) {
      if (L.pipelined_norm >= 4) launch_sumsq16_multi<MXOPT_BF16, 4>(mode, L, prep, partial_sum);
      else launch_sumsq16_multi<MXOPT_BF16, 2>(mode, L, prep, partial_sum);
      return true;
    }
    if (ad == MXOPT_F16) {
      if (L.pipelined_norm >= 4) launch_sumsq16_multi<MXOPT_F16, 4>(mode, L, prep, partial_sum);
      else launch_sumsq16_multi<MXOPT_F16, 2>(mode, L, prep, partial_sum);
      return true;
    }
  }
  switch (mode) {
    case 0: return sumsq_for_mode<0>(ad, gd, L, prep, first, partial_sum);
    case 1: return sumsq_for_mode<1>(ad, gd, L, prep, first, partial_sum);
    case 2: return sumsq_for_mode<2>(ad, gd, L, prep, first, partial_sum);
    case 3: return sumsq_for_mode<3>(ad, gd, L, prep, first, partial_sum);
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

// |x| of a standard normal by its two-sided tail probability, a 32-bit uniform split like a floating-point
// number: leading zeros pick the octave (row), the next 5 bits the sub-interval, 16 more bits interpolate.
static __device__ const float kGaussQuantile[MXOPT_GAUSS_ROWS][MXOPT_GAUSS_COLS] = {MXOPT_GAUSS_TABLE};

__device__ __forceinline__ float synth_gauss_magnitude(uint32_t u) {
  if (u == 0u) u = 1u;
  const int k = __clz((int)u);
  const uint32_t v = u << k;
  const uint32_t j = (v >> 26) & 31u;
  const float f = (float)((v >> 10) & 0xffffu) * 0x1p-16f;  // exact
  const float t0 = kGaussQuantile[k][j];
  const float d = kGaussQuantile[k][j + 1] - t0;
  const float step = d * f;
  return t0 + step;
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
    } else if (dist == MXOPT_SYNTH_GAUSSIAN || dist == MXOPT_SYNTH_GAUSSIAN_OUTLIERS) {
      const float mag = synth_gauss_magnitude((uint32_t)(z >> 31));
      x = (z >> 63) ? -mag : mag;
      x = x * a;                             // a = sigma
      if (dist == MXOPT_SYNTH_GAUSSIAN_OUTLIERS && synth_hash(seed ^ 0xA5A5A5A5A5A5A5A5ull, first_index + i) % 100ull == 0ull)
        x = x * b;
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

// One result of the second pass copied into pinned host memory by a kernel (a 40-byte store over the
// bus instead of a copy command): the engines' asynchronous micro-batch call looks at it later.
__global__ void mirror_result_kernel(const mxopt_norm_result* __restrict__ src, mxopt_norm_result* __restrict__ dst) {
  *dst = *src;
  __threadfence_system();
}

void launch_mirror_result(hipStream_t stream, const mxopt_norm_result* d_src, mxopt_norm_result* host_mapped_dst) {
  hipLaunchKernelGGL(mirror_result_kernel, dim3(1), dim3(1), 0, stream, d_src, host_mapped_dst);
}

// ------------------------------------------------------------------------------------
// Partial sums that need no allocation: a fixed array in the code object's own device memory, one
// copy per GPU, for callers that may not allocate (mxopt_global_norm_static).  On the host the
// array's name is only a handle for hipGetSymbolAddress: kernels are given the address that call
// returned for the device they run on, never the name.
// ------------------------------------------------------------------------------------

static __device__ __align__(256) double scratch[kStaticPartials];

// Looked up once per device, with that device current (mxopt_create calls this), and kept.
hipError_t static_partials_address(int device, double** out) {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static double* known[kMaxDevices];
  *out = nullptr;
  if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(mu);
  if (known[device] == nullptr) {
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    known[device] = (double*)ptr;
  }
  *out = known[device];
  return hipSuccess;
}

}  // namespace mxopt
