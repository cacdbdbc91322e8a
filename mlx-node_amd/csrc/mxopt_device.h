// Device-side building blocks of the mxopt kernels (gfx950 only).
//
// Layout in HBM: every tensor is a dense buffer owned by the caller.  The table holds one
// DevTensor per tensor and one DevChunk per kChunk-element slice of a tensor; a workgroup
// of 256 lanes (4 wavefronts of 64) takes one chunk at a time.  Inside a chunk, lane L of
// pass j owns the E contiguous elements starting at (j*256 + L)*E, so one wavefront-wide
// load instruction covers 64 consecutive 16-byte pieces of a stream.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mxopt.h"
#include "mxopt_host_types.h"

namespace mxopt {

constexpr int kThreads = 256;
constexpr int kChunk = kChunkElems;
constexpr int kElemsPerLane = kChunk / kThreads;  // 16

// Every buffer of a table is device memory, but the kernels only see its address as a number read from
// the table, so the compiler would fall back to FLAT memory instructions (which probe the LDS and scratch
// apertures as well); naming the global address space gives global_load / global_store.
#define MXOPT_GLOBAL __attribute__((address_space(1)))
template <class T>
__device__ __forceinline__ const MXOPT_GLOBAL T* global_ptr(const void* p) {
  return (const MXOPT_GLOBAL T*)(uintptr_t)p;
}
template <class T>
__device__ __forceinline__ MXOPT_GLOBAL T* global_ptr(void* p) {
  return (MXOPT_GLOBAL T*)(uintptr_t)p;
}

// Tables (descriptors, chunk lists, pending-stream pointers) and the device scalars a kernel is handed are
// written before the launch and never during it.  Read through the constant address space, a load whose
// address is the same for the whole wavefront becomes a scalar load: it lands in scalar registers, goes
// through the scalar cache, and is counted apart from the vector loads, so that waiting for a descriptor
// never means waiting for the data loads already in flight.
#define MXOPT_CONSTANT __attribute__((address_space(4)))
template <class T>
__device__ __forceinline__ const MXOPT_CONSTANT T* constant_ptr(const void* p) {
  return (const MXOPT_CONSTANT T*)(uintptr_t)p;
}

// Element `index` of an array of plain structs, read word by word through the constant address space (the
// compiler merges the words into s_load_dwordx2 ... x16).
template <class S>
__device__ __forceinline__ S load_constant(const void* array, size_t index) {
  static_assert(sizeof(S) % 4 == 0 && alignof(S) >= 4, "whole 32-bit words");
  struct Words { uint32_t w[sizeof(S) / 4]; };
  const MXOPT_CONSTANT uint32_t* src = constant_ptr<uint32_t>(array) + index * (sizeof(S) / 4);
  Words tmp;
#pragma unroll
  for (size_t i = 0; i < sizeof(S) / 4; ++i) tmp.w[i] = src[i];
  return __builtin_bit_cast(S, tmp);
}

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// ---- element conversions ----------------------------------------------------------

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// float32 -> bf16, round-to-nearest-even, NaN stays a quiet NaN: gfx950's v_cvt_pk_bf16_f32
// (two elements per instruction), reached through the compiler's native bf16 vector type.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_bits(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) { return f32x2_to_bf16x2_bits(f, 0.0f) & 0xffffu; }

__device__ __forceinline__ float f16_bits_to_f32(uint32_t b) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)b);
}
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);  // v_cvt_f16_f32: RNE
}

template <int DT>
struct Elem;
template <>
struct Elem<MXOPT_F32> {
  using T = float;
  static constexpr int kBytes = 4;
  static __device__ __forceinline__ float load(const void* base, uint64_t i) { return global_ptr<float>(base)[i]; }
  static __device__ __forceinline__ void store(void* base, uint64_t i, float x) { global_ptr<float>(base)[i] = x; }
  static __device__ __forceinline__ float round(float x) { return x; }
};
template <>
struct Elem<MXOPT_BF16> {
  using T = uint16_t;
  static constexpr int kBytes = 2;
  static __device__ __forceinline__ float unpack(uint32_t b) { return bf16_bits_to_f32(b); }
  static __device__ __forceinline__ uint32_t pack(float x) { return f32_to_bf16_bits(x); }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return f32x2_to_bf16x2_bits(lo, hi); }
  static __device__ __forceinline__ float load(const void* base, uint64_t i) {
    return unpack(global_ptr<uint16_t>(base)[i]);
  }
  static __device__ __forceinline__ void store(void* base, uint64_t i, float x) {
    global_ptr<uint16_t>(base)[i] = (uint16_t)pack(x);
  }
  static __device__ __forceinline__ float round(float x) { return unpack(pack(x)); }
};
template <>
struct Elem<MXOPT_F16> {
  using T = uint16_t;
  static constexpr int kBytes = 2;
  static __device__ __forceinline__ float unpack(uint32_t b) { return f16_bits_to_f32(b); }
  static __device__ __forceinline__ uint32_t pack(float x) { return f32_to_f16_bits(x); }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack(lo) | (pack(hi) << 16); }
  static __device__ __forceinline__ float load(const void* base, uint64_t i) {
    return unpack(global_ptr<uint16_t>(base)[i]);
  }
  static __device__ __forceinline__ void store(void* base, uint64_t i, float x) {
    global_ptr<uint16_t>(base)[i] = (uint16_t)pack(x);
  }
  static __device__ __forceinline__ float round(float x) { return unpack(pack(x)); }
};

// ---- E-element group loads / stores (E = 4 or 8), 128-bit where the type allows -----
// `off` is an element offset whose byte offset is 16-byte aligned (8-byte for E=4 x 16-bit).

template <int DT, int E, bool NT>
__device__ __forceinline__ void load_group(const void* base, uint64_t off, float (&x)[E]) {
  if constexpr (DT == MXOPT_F32) {
    const MXOPT_GLOBAL f32x4* q = global_ptr<f32x4>((const void*)((const float*)base + off));
    // Eight float32 values are two 16-byte loads that share every 32-byte sector they touch.  As streaming
    // loads the second of the pair finds its sector gone again about one time in thirteen and fetches it from
    // memory twice (the norm-only pass over a float32 buffer and a bf16 gradient fetched 5 % more than it used
    // and ran 3 % slower); as plain loads it never does.  So only an unsplit load streams.
    constexpr bool kStream = NT && E == 4;
#pragma unroll
    for (int k = 0; k < E / 4; ++k) {
      f32x4 t = kStream ? __builtin_nontemporal_load(q + k) : q[k];
      x[4 * k + 0] = t.x; x[4 * k + 1] = t.y; x[4 * k + 2] = t.z; x[4 * k + 3] = t.w;
    }
  } else if constexpr (E == 8) {
    const MXOPT_GLOBAL u32x4* q = global_ptr<u32x4>((const void*)((const uint16_t*)base + off));
    u32x4 t = NT ? __builtin_nontemporal_load(q) : *q;
    uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      x[2 * k + 0] = Elem<DT>::unpack(w[k] & 0xffffu);
      x[2 * k + 1] = Elem<DT>::unpack(w[k] >> 16);
    }
  } else {
    const MXOPT_GLOBAL u32x2* q = global_ptr<u32x2>((const void*)((const uint16_t*)base + off));
    u32x2 t = NT ? __builtin_nontemporal_load(q) : *q;
    x[0] = Elem<DT>::unpack(t.x & 0xffffu); x[1] = Elem<DT>::unpack(t.x >> 16);
    x[2] = Elem<DT>::unpack(t.y & 0xffffu); x[3] = Elem<DT>::unpack(t.y >> 16);
  }
}

template <int DT, int E, bool NT>
__device__ __forceinline__ void store_group(void* base, uint64_t off, const float (&x)[E]) {
  if constexpr (DT == MXOPT_F32) {
    MXOPT_GLOBAL f32x4* q = global_ptr<f32x4>((void*)((float*)base + off));
    constexpr bool kStream = NT && E == 4;  // as for loads: a pair of stores that share their sectors does not stream
#pragma unroll
    for (int k = 0; k < E / 4; ++k) {
      f32x4 t = {x[4 * k + 0], x[4 * k + 1], x[4 * k + 2], x[4 * k + 3]};
      if (kStream) __builtin_nontemporal_store(t, q + k); else q[k] = t;
    }
  } else if constexpr (E == 8) {
    u32x4 t;
    t.x = Elem<DT>::pack2(x[0], x[1]);
    t.y = Elem<DT>::pack2(x[2], x[3]);
    t.z = Elem<DT>::pack2(x[4], x[5]);
    t.w = Elem<DT>::pack2(x[6], x[7]);
    MXOPT_GLOBAL u32x4* q = global_ptr<u32x4>((void*)((uint16_t*)base + off));
    if (NT) __builtin_nontemporal_store(t, q); else *q = t;
  } else {
    u32x2 t;
    t.x = Elem<DT>::pack2(x[0], x[1]);
    t.y = Elem<DT>::pack2(x[2], x[3]);
    MXOPT_GLOBAL u32x2* q = global_ptr<u32x2>((void*)((uint16_t*)base + off));
    if (NT) __builtin_nontemporal_store(t, q); else *q = t;
  }
}

// ---- gradient pre-processing (one float32 op per reference op) ----------------------

__device__ __forceinline__ float clamp_keep_nan(float g, float lo, float hi) {
  float c = fminf(fmaxf(g, lo), hi);
  return (g != g) ? g : c;
}

// The same clamp as one median-of-three (v_med3_f32 takes no care of NaN) and a select that puts a NaN back.
// For lo <= hi and any non-NaN g, including the infinities and both zeros, the median is min(max(g, lo), hi).
__device__ __forceinline__ float clamp_median_keep_nan(float g, float lo, float hi) {
  const float c = __builtin_amdgcn_fmed3f(g, lo, hi);
  return (g != g) ? g : c;
}

struct PrepRegs {  // block-uniform copy of DevPrep with the device scalar already loaded
  float pre_mul, pre_lo, pre_hi, scale, post_lo, post_hi;
  uint32_t flags;
  bool has_scale;
};

__device__ __forceinline__ PrepRegs load_prep(const DevPrep& p) {
  PrepRegs r;
  r.pre_mul = p.pre_mul; r.pre_lo = p.pre_lo; r.pre_hi = p.pre_hi;
  r.post_lo = p.post_lo; r.post_hi = p.post_hi; r.flags = p.flags;
  r.has_scale = p.d_scale != nullptr;
  // A scalar load: every workgroup of the launch reads this one word, and as a vector load that is one request
  // per wavefront to a single L2 channel (millions of them beside that channel's share of the streams).
  r.scale = r.has_scale ? *constant_ptr<float>(p.d_scale) : 1.0f;
  return r;
}

// Stages before the norm is taken.
__device__ __forceinline__ float prep_pre(const PrepRegs& r, float g) {
  if (r.flags & kPrepPreMul) g = g * r.pre_mul;
  if (r.flags & kPrepClampPre) g = clamp_keep_nan(g, r.pre_lo, r.pre_hi);
  return g;
}
__device__ __forceinline__ float prep_all(const PrepRegs& r, float g) {
  g = prep_pre(r, g);
  if (r.has_scale) g = g * r.scale;
  if (r.flags & kPrepClampPost) g = clamp_keep_nan(g, r.post_lo, r.post_hi);
  return g;
}

// ---- block reduction: wavefront shuffle -> LDS -> lane 0 ---------------------------

__device__ __forceinline__ double wave_sum(double x) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) x += __shfl_down(x, off, 64);
  return x;
}
__device__ __forceinline__ unsigned long long wave_sum(unsigned long long x) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) x += __shfl_down(x, off, 64);
  return x;
}

// Valid on thread 0 only.  Fixed order => deterministic.
__device__ __forceinline__ void block_sum(double& s, unsigned long long& c) {
  __shared__ double sh_s[kThreads / 64];
  __shared__ unsigned long long sh_c[kThreads / 64];
  s = wave_sum(s);
  c = wave_sum(c);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) { sh_s[wave] = s; sh_c[wave] = c; }
  __syncthreads();
  if (threadIdx.x == 0) {
    s = sh_s[0]; c = sh_c[0];
#pragma unroll
    for (int w = 1; w < kThreads / 64; ++w) { s += sh_s[w]; c += sh_c[w]; }
  }
  __syncthreads();
}

__device__ __forceinline__ bool is_nonfinite(float x) {
  return (__float_as_uint(x) & 0x7f800000u) == 0x7f800000u;
}

}  // namespace mxopt
