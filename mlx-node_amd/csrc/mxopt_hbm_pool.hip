// Bare streaming probes (the measured ceilings the update kernels are compared with) and the
// region-interleaved device-memory pool.
//
// What the pool is for.  Device memory on this part consists of three physical regions of 96 GiB.
// A kernel that reads and writes several streams runs at about 5.3 TB/s when everything it touches
// lies in one region and at about 6.1 TB/s when its traffic is spread over two or three of them
// (read-only streams do not care).  A fresh process that allocates a few tens of GB gets one compact
// physical run, i.e. one region.  The pool takes the free memory as physical chunks (64 MiB), finds
// out by timing which chunks share a region, and maps an arena in which consecutive chunks alternate
// between the regions; everything allocated from the arena then has its traffic spread evenly
// whatever streams a kernel combines.  The physical memory it does not need goes back to the driver
// before mxopt_hbm_pool_create returns.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <new>
#include <thread>
#include <unordered_map>
#include <vector>

#include "mxopt_internal.h"
#include "mxopt_region_scan.h"

namespace mxopt {

typedef uint32_t pu32x4 __attribute__((ext_vector_type(4)));
constexpr int kProbeThreads = 256;
constexpr int kProbeVecs = 4;                                    // 16-byte pieces per lane per stream
constexpr uint64_t kProbeTileElems = kProbeThreads * kProbeVecs * 4;  // float32 elements per workgroup trip

// One read stream.
__global__ __launch_bounds__(kProbeThreads) void probe_read_kernel(const pu32x4* __restrict__ a, uint32_t ntiles,
                                                                  uint32_t* __restrict__ sink) {
  uint32_t s = 0;
  for (uint32_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const size_t b = (size_t)t * (kProbeThreads * kProbeVecs) + threadIdx.x;
    pu32x4 r[kProbeVecs];
#pragma unroll
    for (int j = 0; j < kProbeVecs; ++j) r[j] = __builtin_nontemporal_load(a + b + j * kProbeThreads);
#pragma unroll
    for (int j = 0; j < kProbeVecs; ++j) s ^= r[j].x ^ r[j].y ^ r[j].z ^ r[j].w;
  }
  if (s == 0x9E3779B9u && sink != nullptr) *sink = s;  // keeps the loads alive
}

// NT (the MXOPT_PROBE_STREAMING bit of the kind): streaming-hint stores, and loads where the plain form has plain
// loads; what the update kernels do by default.
template <bool NT, class T>
__device__ __forceinline__ T probe_ld(const T* q) { return NT ? __builtin_nontemporal_load(q) : *q; }
template <bool NT, class T>
__device__ __forceinline__ void probe_st(T* q, T v) { if (NT) __builtin_nontemporal_store(v, q); else *q = v; }

// One write stream.
template <bool NT>
__global__ __launch_bounds__(kProbeThreads) void probe_write_kernel(pu32x4* __restrict__ a, uint32_t ntiles) {
  for (uint32_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const size_t b = (size_t)t * (kProbeThreads * kProbeVecs) + threadIdx.x;
    const pu32x4 r = {t, t, t, t};
#pragma unroll
    for (int j = 0; j < kProbeVecs; ++j) probe_st<NT>(a + b + j * kProbeThreads, r);
  }
}

// One read and one write stream.
template <bool NT>
__global__ __launch_bounds__(kProbeThreads) void probe_copy_kernel(const pu32x4* __restrict__ a, pu32x4* __restrict__ o,
                                                                  uint32_t ntiles) {
  for (uint32_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const size_t b = (size_t)t * (kProbeThreads * kProbeVecs) + threadIdx.x;
    pu32x4 r[kProbeVecs];
#pragma unroll
    for (int j = 0; j < kProbeVecs; ++j) r[j] = probe_ld<NT>(a + b + j * kProbeThreads);
#pragma unroll
    for (int j = 0; j < kProbeVecs; ++j) probe_st<NT>(o + b + j * kProbeThreads, r[j]);
  }
}

// AdamW's float32 byte mix without its arithmetic: reads a, b, c, d; writes a, c, d in place.
template <bool NT>
__global__ __launch_bounds__(kProbeThreads) void probe_mix43_kernel(pu32x4* __restrict__ a, const pu32x4* __restrict__ g,
                                                                   pu32x4* __restrict__ c, pu32x4* __restrict__ d,
                                                                   uint32_t ntiles) {
  for (uint32_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const size_t b = (size_t)t * (kProbeThreads * kProbeVecs) + threadIdx.x;
    pu32x4 ra[kProbeVecs], rg[kProbeVecs], rc[kProbeVecs], rd[kProbeVecs];
#pragma unroll
    for (int j = 0; j < kProbeVecs; ++j) {
      ra[j] = probe_ld<NT>(a + b + j * kProbeThreads); rg[j] = probe_ld<NT>(g + b + j * kProbeThreads);
      rc[j] = probe_ld<NT>(c + b + j * kProbeThreads); rd[j] = probe_ld<NT>(d + b + j * kProbeThreads);
    }
#pragma unroll
    for (int j = 0; j < kProbeVecs; ++j) {
      probe_st<NT>(a + b + j * kProbeThreads, ra[j] ^ rg[j]);
      probe_st<NT>(c + b + j * kProbeThreads, rc[j] + rg[j]);
      probe_st<NT>(d + b + j * kProbeThreads, rd[j] ^ (rg[j] >> 1));
    }
  }
}

// The byte mix of the update over un-summed 16-bit micro-batches (deferred accumulation) without its
// arithmetic: per element K + 1 two-byte reads (the gradient streams and the parameter), two four-byte
// reads (the moments); the parameter and the moments are written back in place.  One workgroup per
// 4096-element tile, every load of the tile issued before the first store, as in the update kernels.  NT: the
// 2-byte streams use streaming loads and stores; the 4-byte ones, whose two 16-byte pieces per lane share their
// sectors, stay plain (the list kernels' rule).
template <int K, bool NT>
__global__ __launch_bounds__(kProbeThreads) void probe_list_kernel(pu32x4* __restrict__ p, pu32x4* __restrict__ m,
                                                                  pu32x4* __restrict__ v,
                                                                  const pu32x4* __restrict__ g0, const pu32x4* __restrict__ g1,
                                                                  const pu32x4* __restrict__ g2, const pu32x4* __restrict__ g3,
                                                                  const pu32x4* __restrict__ g4, const pu32x4* __restrict__ g5,
                                                                  const pu32x4* __restrict__ g6, const pu32x4* __restrict__ g7,
                                                                  uint32_t ntiles) {
  constexpr int U = 2;  // groups of 8 elements per lane: 2 x 256 x 8 = 4096 elements per tile
  const pu32x4* gs[8] = {g0, g1, g2, g3, g4, g5, g6, g7};
  for (uint32_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const size_t b16 = (size_t)t * (kProbeThreads * U) + threadIdx.x;      // 16-byte pieces of a 2-byte stream
    const size_t b32 = (size_t)t * (kProbeThreads * U * 2) + threadIdx.x;  // ... of a 4-byte stream
    pu32x4 rg[K][U], rp[U], rm[U][2], rv[U][2];
#pragma unroll
    for (int j = 0; j < U; ++j) {
#pragma unroll
      for (int k = 0; k < K; ++k) rg[k][j] = probe_ld<NT>(gs[k] + b16 + j * kProbeThreads);
      rp[j] = probe_ld<NT>(p + b16 + j * kProbeThreads);
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        rm[j][h] = m[b32 + (2 * j + h) * kProbeThreads];
        rv[j][h] = v[b32 + (2 * j + h) * kProbeThreads];
      }
    }
#pragma unroll
    for (int j = 0; j < U; ++j) {
      pu32x4 s = rg[0][j];
#pragma unroll
      for (int k = 1; k < K; ++k) s += rg[k][j];
      probe_st<NT>(p + b16 + j * kProbeThreads, rp[j] ^ s);
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        m[b32 + (2 * j + h) * kProbeThreads] = rm[j][h] + s;
        v[b32 + (2 * j + h) * kProbeThreads] = rv[j][h] ^ (s >> 1);
      }
    }
  }
}

template <int K, bool NT>
static void launch_probe_list_k(mxopt_ctx* ctx, void* p, void* m, void* v, const void* const* g, uint32_t ntiles) {
  const pu32x4* q[8];
  for (int k = 0; k < 8; ++k) q[k] = (const pu32x4*)g[k < K ? k : 0];
  hipLaunchKernelGGL((probe_list_kernel<K, NT>), dim3(ntiles), dim3(kProbeThreads), 0, ctx->stream, (pu32x4*)p, (pu32x4*)m,
                     (pu32x4*)v, q[0], q[1], q[2], q[3], q[4], q[5], q[6], q[7], ntiles);
}

static int launch_probe(mxopt_ctx* ctx, int kind_and_flags, void* a, void* b, void* c, void* d, uint64_t n) {
  const bool nt = (kind_and_flags & MXOPT_PROBE_STREAMING) != 0;
  const int kind = kind_and_flags & ~MXOPT_PROBE_STREAMING;
  const uint32_t ntiles = (uint32_t)(n / kProbeTileElems);
  const uint32_t bounded = (uint32_t)std::min<uint64_t>(ntiles, (uint64_t)ctx->num_cus * 16u);
  switch (kind) {
    case MXOPT_PROBE_READ:
      hipLaunchKernelGGL(probe_read_kernel, dim3(bounded), dim3(kProbeThreads), 0, ctx->stream, (const pu32x4*)a, ntiles,
                         (uint32_t*)nullptr);
      break;
    case MXOPT_PROBE_WRITE:
      if (nt) hipLaunchKernelGGL(probe_write_kernel<true>, dim3(ntiles), dim3(kProbeThreads), 0, ctx->stream, (pu32x4*)a, ntiles);
      else hipLaunchKernelGGL(probe_write_kernel<false>, dim3(ntiles), dim3(kProbeThreads), 0, ctx->stream, (pu32x4*)a, ntiles);
      break;
    case MXOPT_PROBE_COPY:
      if (nt) hipLaunchKernelGGL(probe_copy_kernel<true>, dim3(ntiles), dim3(kProbeThreads), 0, ctx->stream, (const pu32x4*)a,
                                 (pu32x4*)b, ntiles);
      else hipLaunchKernelGGL(probe_copy_kernel<false>, dim3(ntiles), dim3(kProbeThreads), 0, ctx->stream, (const pu32x4*)a,
                              (pu32x4*)b, ntiles);
      break;
    case MXOPT_PROBE_MIX43:
      if (nt) hipLaunchKernelGGL(probe_mix43_kernel<true>, dim3(ntiles), dim3(kProbeThreads), 0, ctx->stream, (pu32x4*)a,
                                 (const pu32x4*)b, (pu32x4*)c, (pu32x4*)d, ntiles);
      else hipLaunchKernelGGL(probe_mix43_kernel<false>, dim3(ntiles), dim3(kProbeThreads), 0, ctx->stream, (pu32x4*)a,
                              (const pu32x4*)b, (pu32x4*)c, (pu32x4*)d, ntiles);
      break;
    default:
      return fail(ctx, MXOPT_ERR_INVALID_ARG, "mxopt_probe_stream: unknown kind");
  }
  return check_launch(ctx, "mxopt_probe_stream");
}

}  // namespace mxopt

using namespace mxopt;

// ---------------------------------------------------------------------------------------
// The pool
// ---------------------------------------------------------------------------------------

struct mxopt_hbm_pool {
  mxopt_ctx* ctx = nullptr;
  size_t chunk = 0;
  std::vector<hipMemGenericAllocationHandle_t> handles;  // the arena's chunks, in address order
  char* base = nullptr;
  size_t capacity = 0;
  std::map<size_t, size_t> free_list;                    // offset -> bytes, coalesced
  size_t one_region_begin = 0;                           // arena bytes from here on lie in one region at a time
  std::unordered_map<size_t, size_t> live;               // offset -> bytes
  std::mutex mu;
  mxopt_hbm_pool_info info{};
};

namespace {

constexpr size_t kAlign = 512;
constexpr size_t kSlabChunksBytes = (size_t)1 << 30;  // chunks are classified in groups of this many bytes by default
// The driver limits the live allocations of a process (about 60 000 were seen to succeed) and maps fewer still.
constexpr size_t kMaxChunks = 24000;

// Taking the free memory as chunks, measured on 286 GiB: 0.08 - 0.13 s as 4,566 chunks of 64 MiB and 0.56 - 2.06 s as
// 18,266 of 16 MiB on a quiet device (under 0.5 ms per GiB plus 0.03 - 0.11 ms per chunk), 3.9 s as 64 MiB chunks
// (13.6 ms per GiB) while the driver is still taking back memory released a moment ago.  Slower than this bound the
// call hands everything back, waits and starts over.  (With 16 MiB chunks the sign is weaker -- 2.2 - 4.6 s busy
// against 0.6 - 2.1 s quiet -- and the bound only catches the worse cases; 64 MiB is the default for more than one
// reason.)
constexpr double kBusyCreateSecondsPerGiB = 0.004;
constexpr double kBusyCreateSecondsPerChunk = 0.00015;
constexpr int kMaxTakeAttempts = 3;
constexpr int kBusyWaitMs = 4000;

struct Builder {  // everything pool creation holds until it either succeeds or fails
  mxopt_ctx* ctx;
  std::vector<hipMemGenericAllocationHandle_t> all;
  std::vector<char> released;
  void* probe_va = nullptr;
  size_t probe_bytes = 0;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  ~Builder() {
    if (probe_va) {
      // after an error some of it may still be mapped; on the normal path these two fail harmlessly
      (void)hipMemUnmap(probe_va, probe_bytes / 2);
      (void)hipMemUnmap((char*)probe_va + probe_bytes / 2, probe_bytes / 2);
      (void)hipGetLastError();
      (void)hipMemAddressFree(probe_va, probe_bytes);
    }
    for (size_t i = 0; i < all.size(); ++i)
      if (!released[i]) (void)hipMemRelease(all[i]);
    if (ev0) (void)hipEventDestroy(ev0);
    if (ev1) (void)hipEventDestroy(ev1);
  }
};

hipMemAllocationProp device_prop(int device) {
  hipMemAllocationProp prop = {};
  prop.type = hipMemAllocationTypePinned;
  prop.location.type = hipMemLocationTypeDevice;
  prop.location.id = device;
  return prop;
}

hipMemAccessDesc rw_access(int device) {
  hipMemAccessDesc acc = {};
  acc.location.type = hipMemLocationTypeDevice;
  acc.location.id = device;
  acc.flags = hipMemAccessFlagsProtReadWrite;
  return acc;
}

// Every live pool of the process: a pointer is given back to the pool it came from, whichever pool a
// context or the allocator hooks point at by then.
std::mutex g_pools_mu;
std::vector<mxopt_hbm_pool*> g_pools;
std::mutex g_hook_mu;
mxopt_hbm_pool* g_hook_pool = nullptr;
int g_hook_kind = MXOPT_HBM_INTERLEAVED;

mxopt_hbm_pool* pool_of(const void* ptr) {
  std::lock_guard<std::mutex> all(g_pools_mu);
  for (mxopt_hbm_pool* p : g_pools)
    if (ptr && (const char*)ptr >= p->base && (const char*)ptr < p->base + p->capacity) return p;
  return nullptr;
}

}  // namespace

extern "C" {

int mxopt_probe_stream(mxopt_ctx* ctx, int kind, void* a, void* b, void* c, void* d, uint64_t n_elems) {
  if (!ctx) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "mxopt_probe_stream: null context");
  if (n_elems == 0 || n_elems % kProbeTileElems != 0 || n_elems / kProbeTileElems > 0xffffffffull)
    return fail(ctx, MXOPT_ERR_INVALID_ARG, "mxopt_probe_stream: n_elems must be a positive multiple of 4096");
  const int base_kind = kind & ~MXOPT_PROBE_STREAMING;
  const int need = base_kind == MXOPT_PROBE_MIX43 ? 4 : base_kind == MXOPT_PROBE_COPY ? 2 : 1;
  void* ptrs[4] = {a, b, c, d};
  for (int i = 0; i < need; ++i)
    if (!ptrs[i] || (reinterpret_cast<uintptr_t>(ptrs[i]) & 15u))
      return fail(ctx, MXOPT_ERR_INVALID_ARG, "mxopt_probe_stream: buffers must be non-NULL and 16-byte aligned");
  DeviceGuard guard(ctx->device);
  return launch_probe(ctx, kind, a, b, c, d, n_elems);
}

int mxopt_probe_list(mxopt_ctx* ctx, void* p, void* m, void* v, const void* const* g, int k_and_flags,
                     uint64_t n_elems) {
  const char* op = "mxopt_probe_list";
  const bool nt = (k_and_flags & MXOPT_PROBE_STREAMING) != 0;
  const int k = k_and_flags & ~MXOPT_PROBE_STREAMING;
  if (!ctx) return fail(nullptr, MXOPT_ERR_INVALID_ARG, std::string(op) + ": null context");
  if (n_elems == 0 || n_elems % 4096 != 0 || n_elems / 4096 > 0xffffffffull)
    return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(op) + ": n_elems must be a positive multiple of 4096");
  if (k < 1 || k > 8 || !g) return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(op) + ": 1 to 8 gradient streams");
  const void* ptrs[11] = {p, m, v};
  for (int i = 0; i < k; ++i) ptrs[3 + i] = g[i];
  for (int i = 0; i < 3 + k; ++i)
    if (!ptrs[i] || (reinterpret_cast<uintptr_t>(ptrs[i]) & 15u))
      return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(op) + ": buffers must be non-NULL and 16-byte aligned");
  DeviceGuard guard(ctx->device);
  const uint32_t ntiles = (uint32_t)(n_elems / 4096);
  switch (k) {
    case 1: nt ? launch_probe_list_k<1, true>(ctx, p, m, v, g, ntiles) : launch_probe_list_k<1, false>(ctx, p, m, v, g, ntiles); break;
    case 2: nt ? launch_probe_list_k<2, true>(ctx, p, m, v, g, ntiles) : launch_probe_list_k<2, false>(ctx, p, m, v, g, ntiles); break;
    case 3: nt ? launch_probe_list_k<3, true>(ctx, p, m, v, g, ntiles) : launch_probe_list_k<3, false>(ctx, p, m, v, g, ntiles); break;
    case 4: nt ? launch_probe_list_k<4, true>(ctx, p, m, v, g, ntiles) : launch_probe_list_k<4, false>(ctx, p, m, v, g, ntiles); break;
    case 5: nt ? launch_probe_list_k<5, true>(ctx, p, m, v, g, ntiles) : launch_probe_list_k<5, false>(ctx, p, m, v, g, ntiles); break;
    case 6: nt ? launch_probe_list_k<6, true>(ctx, p, m, v, g, ntiles) : launch_probe_list_k<6, false>(ctx, p, m, v, g, ntiles); break;
    case 7: nt ? launch_probe_list_k<7, true>(ctx, p, m, v, g, ntiles) : launch_probe_list_k<7, false>(ctx, p, m, v, g, ntiles); break;
    default: nt ? launch_probe_list_k<8, true>(ctx, p, m, v, g, ntiles) : launch_probe_list_k<8, false>(ctx, p, m, v, g, ntiles); break;
  }
  return check_launch(ctx, op);
}

int mxopt_hbm_pool_create(mxopt_ctx* ctx, size_t capacity_bytes, size_t chunk_bytes, int max_regions,
                          mxopt_hbm_pool** out) {
  mxopt_hbm_pool_options o;
  std::memset(&o, 0, sizeof o);
  o.capacity_bytes = capacity_bytes;
  o.chunk_bytes = chunk_bytes;
  o.max_regions = max_regions;
  return mxopt_hbm_pool_create_ex(ctx, &o, out);
}

int mxopt_hbm_pool_create_ex(mxopt_ctx* ctx, const mxopt_hbm_pool_options* options, mxopt_hbm_pool** out) {
  const char* op = "mxopt_hbm_pool_create";
  if (!ctx || !out || !options) return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(op) + ": null argument");
  *out = nullptr;
  const size_t capacity_bytes = options->capacity_bytes;
  size_t chunk_bytes = options->chunk_bytes;
  const int max_regions = options->max_regions;
  size_t slab_bytes = options->slab_bytes ? options->slab_bytes : kSlabChunksBytes;
  if (chunk_bytes == 0) chunk_bytes = (size_t)64 << 20;
  if (chunk_bytes < ((size_t)2 << 20) || (chunk_bytes & (chunk_bytes - 1)) || chunk_bytes > kSlabChunksBytes)
    return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(op) + ": chunk_bytes must be a power of two in [2 MiB, 1 GiB]");
  // Two slabs are a probe's working set; at 256 MiB per slab most of it stays in the 256 MB last-level cache
  // between the probe's launches and every pair looks alike (measured: one "region" of 285 GiB).
  if ((slab_bytes & (slab_bytes - 1)) || slab_bytes < ((size_t)512 << 20) || slab_bytes > ((size_t)4 << 30))
    return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(op) + ": slab_bytes must be a power of two in [512 MiB, 4 GiB]");
  if (slab_bytes < chunk_bytes) slab_bytes = chunk_bytes;
  if (capacity_bytes == 0) return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(op) + ": capacity_bytes is 0");
  if (max_regions < 0) return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(op) + ": max_regions is negative");
  const auto t_begin = std::chrono::steady_clock::now();
  DeviceGuard guard(ctx->device);
  HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
  size_t free_b = 0, total_b = 0;
  HIP_TRY(ctx, hipMemGetInfo(&free_b, &total_b));
  const size_t margin = (size_t)1 << 30;  // left to the runtime
  const size_t want_chunks = (capacity_bytes + chunk_bytes - 1) / chunk_bytes;
  size_t avail_chunks = free_b > margin ? (free_b - margin) / chunk_bytes : 0;
  if (want_chunks > avail_chunks)
    return fail(ctx, MXOPT_ERR_OOM, std::string(op) + ": " + std::to_string(capacity_bytes >> 20) + " MiB wanted, " +
                                        std::to_string(free_b >> 20) + " MiB free");
  // A caller that shares the device bounds what creation may hold while it scans (never less than the arena).
  if (options->max_take_bytes)
    avail_chunks = std::min(avail_chunks, std::max(want_chunks, options->max_take_bytes / chunk_bytes));
  if (avail_chunks > kMaxChunks)  // the driver limits the number of live allocations of a process, and maps fewer still
    return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string(op) + ": chunk_bytes too small for this much free memory");

  // 1. The free memory as physical chunks: memory far from what a small allocation would get can only be
  //    reached by holding what lies in between.
  //    The driver takes released memory back asynchronously: within seconds of a large release (a pool that was
  //    just destroyed, a process that has just exited) chunk creation is thirty times slower than on a quiet
  //    device, and a scan made then reads rates that mean nothing (measured: four groups, 138 of
  //    200 GiB interleaved, against three regions and 192 GiB ten seconds later).  Creation that slow is taken as
  //    the sign: everything goes back, the call waits and takes the memory again, at most twice.
  Builder b{ctx};
  const hipMemAllocationProp prop = device_prop(ctx->device);
  b.all.reserve(avail_chunks);
  int take_attempts = 0;
  for (;;) {
    ++take_attempts;
    const auto t_take = std::chrono::steady_clock::now();
    for (size_t i = 0; i < avail_chunks; ++i) {
      hipMemGenericAllocationHandle_t h;
      if (hipMemCreate(&h, chunk_bytes, &prop, 0) != hipSuccess) {
        (void)hipGetLastError();
        break;
      }
      b.all.push_back(h);
    }
    const double took = std::chrono::duration<double>(std::chrono::steady_clock::now() - t_take).count();
    const double gib = (double)b.all.size() * (double)chunk_bytes / (double)((size_t)1 << 30);
    const bool busy = gib >= 16.0 && took > kBusyCreateSecondsPerGiB * gib + kBusyCreateSecondsPerChunk * (double)b.all.size();
    MXOPT_DEBUG("hbm pool: %zu chunks taken in %.2f s (%.1f ms per GiB)%s", b.all.size(), took,
                gib > 0 ? took * 1e3 / gib : 0.0, busy ? ": the driver is busy taking memory back" : "");
    if (!busy || take_attempts >= kMaxTakeAttempts) break;
    for (hipMemGenericAllocationHandle_t h : b.all) (void)hipMemRelease(h);
    b.all.clear();
    std::this_thread::sleep_for(std::chrono::milliseconds(kBusyWaitMs));
  }
  b.released.assign(b.all.size(), 0);
  const auto t_created = std::chrono::steady_clock::now();
  if (b.all.size() < want_chunks)
    return fail(ctx, MXOPT_ERR_OOM, std::string(op) + ": the driver handed out fewer chunks than the capacity needs");

  // 2. Which chunks share a region?  Chunks are judged in creation-order groups ("slabs"): the 4-read/3-write
  //    probe runs with two of its streams in a reference slab and two in the slab under test; it is slow when
  //    both lie in one region.  The decisions are classify_slabs' (mxopt_region_scan.cpp), this function only
  //    measures.
  const size_t per_slab = slab_bytes / chunk_bytes;
  const size_t nslab = b.all.size() / per_slab;
  ScanResult scan;
  scan.slab_region.assign(nslab, 0);
  const ScanLimits limits;
  if (nslab >= limits.min_region_slabs) {
    const hipMemAccessDesc acc = rw_access(ctx->device);
    b.probe_bytes = 2 * slab_bytes;
    HIP_TRY(ctx, hipMemAddressReserve(&b.probe_va, b.probe_bytes, 0, nullptr, 0));
    HIP_TRY(ctx, hipEventCreate(&b.ev0));
    HIP_TRY(ctx, hipEventCreate(&b.ev1));
    char* va_ref = (char*)b.probe_va;
    char* va_x = va_ref + slab_bytes;
    const uint64_t stream_elems = slab_bytes / 2 / 4;  // two streams per slab
    auto map_slab = [&](char* va, size_t slab) -> hipError_t {
      for (size_t k = 0; k < per_slab; ++k) {
        hipError_t e = hipMemMap(va + k * chunk_bytes, chunk_bytes, 0, b.all[slab * per_slab + k], 0);
        if (e != hipSuccess) return e;
      }
      return hipMemSetAccess(va, slab_bytes, &acc, 1);
    };
    int mapped_ref = -1;
    // Rate of the probe with streams p, g in the reference slab and m, v in slab x.
    const SlabProbe probe = [&](int ref, int x, double* out_gbps) -> int {
      if (mapped_ref != ref) {
        if (mapped_ref >= 0) HIP_TRY(ctx, hipMemUnmap(va_ref, slab_bytes));
        mapped_ref = -1;
        hipError_t me = map_slab(va_ref, (size_t)ref);
        if (me != hipSuccess) return hip_fail(ctx, me, "mxopt_hbm_pool_create: mapping a slab");
        mapped_ref = ref;
      }
      hipError_t e = map_slab(va_x, (size_t)x);
      if (e != hipSuccess) return hip_fail(ctx, e, "mxopt_hbm_pool_create: mapping a slab");
      void* p = va_ref;
      void* g = va_ref + slab_bytes / 2;
      void* m = va_x;
      void* v = va_x + slab_bytes / 2;
      int rc = launch_probe(ctx, MXOPT_PROBE_MIX43, p, g, m, v, stream_elems);
      if (rc) return rc;
      HIP_TRY(ctx, hipEventRecord(b.ev0, ctx->stream));
      for (int rep = 0; rep < 2 && !rc; ++rep) rc = launch_probe(ctx, MXOPT_PROBE_MIX43, p, g, m, v, stream_elems);
      if (rc) return rc;
      HIP_TRY(ctx, hipEventRecord(b.ev1, ctx->stream));
      HIP_TRY(ctx, hipEventSynchronize(b.ev1));
      float ms = 0.f;
      HIP_TRY(ctx, hipEventElapsedTime(&ms, b.ev0, b.ev1));
      *out_gbps = 2.0 * 7.0 * (double)(slab_bytes / 2) / 1e9 / ((double)ms * 1e-3);
      HIP_TRY(ctx, hipMemUnmap(va_x, slab_bytes));
      return MXOPT_OK;
    };
    const int rc = classify_slabs(nslab, probe, limits, &scan);
    if (mapped_ref >= 0) (void)hipMemUnmap(va_ref, slab_bytes);
    if (rc) return rc;
    if (log_level() >= 2) std::fprintf(stderr, "mxopt: hbm pool %s", scan.trace.c_str());  // longer than log_line's buffer
  }
  const int nregions = scan.regions;
  const double same_gbps = scan.same_region_gbps, cross_gbps = scan.cross_region_gbps;
  const int probes = scan.probes;
  const auto t_scanned = std::chrono::steady_clock::now();

  // 3. The arena: consecutive chunks alternate between the regions for as long as each has chunks.
  const ArenaPlan plan = plan_arena(scan.slab_region, nregions, per_slab, b.all.size(), want_chunks, max_regions);
  const std::vector<size_t>& order = plan.order;
  const int real_regions = plan.real_regions;
  if (order.size() < want_chunks) return fail(ctx, MXOPT_ERR_OOM, std::string(op) + ": ran out of chunks");

  mxopt_hbm_pool* pool = new (std::nothrow) mxopt_hbm_pool();
  if (!pool) return fail(ctx, MXOPT_ERR_OOM, std::string(op) + ": out of host memory");
  pool->ctx = ctx;
  pool->chunk = chunk_bytes;
  pool->capacity = want_chunks * chunk_bytes;
  void* base = nullptr;
  hipError_t e = hipMemAddressReserve(&base, pool->capacity, 0, nullptr, 0);
  if (e != hipSuccess) { delete pool; return hip_fail(ctx, e, "mxopt_hbm_pool_create: hipMemAddressReserve"); }
  pool->base = (char*)base;
  size_t mapped = 0;
  for (; mapped < order.size(); ++mapped) {
    e = hipMemMap(pool->base + mapped * chunk_bytes, chunk_bytes, 0, b.all[order[mapped]], 0);
    if (e != hipSuccess) break;
  }
  if (e == hipSuccess) {
    const hipMemAccessDesc acc = rw_access(ctx->device);
    e = hipMemSetAccess(pool->base, pool->capacity, &acc, 1);
  }
  if (e != hipSuccess) {
    if (mapped) (void)hipMemUnmap(pool->base, mapped * chunk_bytes);
    (void)hipMemAddressFree(pool->base, pool->capacity);
    delete pool;
    return hip_fail(ctx, e, "mxopt_hbm_pool_create: mapping the arena");
  }
  for (size_t k = 0; k < order.size(); ++k) {
    pool->handles.push_back(b.all[order[k]]);
    b.released[order[k]] = 1;  // now owned by the pool; everything else goes back to the driver with `b`
  }
  pool->free_list[0] = pool->capacity;
  // With one region in the alternation nothing is interleaved: the whole arena is "one region at a time".
  pool->one_region_begin = plan.active > 1 ? plan.interleaved_chunks * chunk_bytes : 0;
  mxopt_hbm_pool_info& info = pool->info;
  info.capacity_bytes = pool->capacity;
  info.chunk_bytes = chunk_bytes;
  info.regions = real_regions;
  info.interleaved_bytes = pool->one_region_begin;
  for (int k = 0; k < nregions && k < MXOPT_HBM_MAX_REGIONS; ++k) {  // largest first; entries past `regions` are leftovers
    info.region_free_bytes[k] = plan.region_chunks[(size_t)k] * chunk_bytes;
    info.region_arena_bytes[k] = plan.region_used[(size_t)k] * chunk_bytes;
  }
  info.probe_same_region_gbps = same_gbps;
  info.probe_cross_region_gbps = cross_gbps;
  // What was built, measured: the 4-read/3-write probe over four pieces spread across the arena.  Whatever
  // the scan concluded -- and when the free memory came in no physical order its grouping means little --
  // this is the rate a kernel will see on memory from here.
  info.arena_probe_gbps = 0.0;
  if (pool->capacity >= 4 * ((size_t)64 << 20) && b.ev0 == nullptr) {
    (void)hipEventCreate(&b.ev0);
    (void)hipEventCreate(&b.ev1);
  }
  if (pool->capacity >= 4 * ((size_t)64 << 20) && b.ev0 && b.ev1) {
    const size_t quarter = pool->capacity / 4 / kAlign * kAlign;
    const size_t piece = std::min<size_t>(quarter, (size_t)1 << 30) / (kProbeTileElems * 4) * (kProbeTileElems * 4);
    void* q[4];
    for (int k = 0; k < 4; ++k) q[k] = pool->base + (size_t)k * quarter;
    const uint64_t elems = piece / 4;
    int rc = launch_probe(ctx, MXOPT_PROBE_MIX43, q[0], q[1], q[2], q[3], elems);
    if (!rc && hipEventRecord(b.ev0, ctx->stream) == hipSuccess) {
      for (int rep = 0; rep < 2 && !rc; ++rep) rc = launch_probe(ctx, MXOPT_PROBE_MIX43, q[0], q[1], q[2], q[3], elems);
      float ms = 0.f;
      if (!rc && hipEventRecord(b.ev1, ctx->stream) == hipSuccess && hipEventSynchronize(b.ev1) == hipSuccess &&
          hipEventElapsedTime(&ms, b.ev0, b.ev1) == hipSuccess && ms > 0.f)
        info.arena_probe_gbps = 2.0 * 7.0 * (double)piece / 1e9 / ((double)ms * 1e-3);
    }
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipGetLastError();
  }
  for (size_t i = 0; i < b.all.size(); ++i)   // what the arena does not use goes back to the driver now
    if (!b.released[i]) { (void)hipMemRelease(b.all[i]); b.released[i] = 1; }
  const auto t_end = std::chrono::steady_clock::now();
  info.setup_seconds = std::chrono::duration<double>(t_end - t_begin).count();
  info.create_seconds = std::chrono::duration<double>(t_created - t_begin).count();
  info.scan_seconds = std::chrono::duration<double>(t_scanned - t_created).count();
  info.probes = probes;
  MXOPT_DEBUG("hbm pool: %zu MiB arena of %zu MiB chunks over %d region(s); probe %.0f GB/s inside one region, %.0f across, "
              "%.0f on the arena; %.2f s",
              pool->capacity >> 20, chunk_bytes >> 20, nregions, same_gbps, cross_gbps, info.arena_probe_gbps,
              info.setup_seconds);
  {
    std::lock_guard<std::mutex> all(g_pools_mu);
    g_pools.push_back(pool);
  }
  *out = pool;
  return MXOPT_OK;
}

int mxopt_hbm_pool_destroy(mxopt_hbm_pool* pool) {
  if (!pool) return MXOPT_OK;
  {
    // Unmapping memory that someone still uses would make their next kernel fault: refuse instead.
    std::lock_guard<std::mutex> all(g_pools_mu);
    size_t live = 0, bytes = 0;
    {
      std::lock_guard<std::mutex> lock(pool->mu);
      live = pool->live.size();
      for (auto& kv : pool->live) bytes += kv.second;
    }
    if (live)
      return fail(pool->ctx, MXOPT_ERR_INVALID_ARG,
                  "mxopt_hbm_pool_destroy: " + std::to_string(live) + " allocation(s), " + std::to_string(bytes >> 20) +
                      " MiB, are still live; free them (optimizer and engine objects, the host allocator's segments) first");
    g_pools.erase(std::remove(g_pools.begin(), g_pools.end(), pool), g_pools.end());
  }
  {
    std::lock_guard<std::mutex> lock(g_hook_mu);
    if (g_hook_pool == pool) g_hook_pool = nullptr;
  }
  {
    DeviceGuard guard(pool->ctx->device);
    (void)hipStreamSynchronize(pool->ctx->stream);
    if (pool->base) {
      (void)hipMemUnmap(pool->base, pool->capacity);
      (void)hipMemAddressFree(pool->base, pool->capacity);
    }
    for (auto h : pool->handles) (void)hipMemRelease(h);
    if (pool->ctx->state_pool == pool) pool->ctx->state_pool = nullptr;
  }
  delete pool;
  return MXOPT_OK;
}

// First fit; NULL when no free range is large enough.  MXOPT_HBM_ONE_REGION looks at the part of the arena that
// lies behind the alternation first (consecutive chunks of one region), then anywhere.
static void* pool_try_alloc(mxopt_hbm_pool* pool, size_t bytes, int kind = MXOPT_HBM_INTERLEAVED) {
  const size_t need = std::max<size_t>((bytes + kAlign - 1) / kAlign * kAlign, kAlign);
  std::lock_guard<std::mutex> lock(pool->mu);
  const size_t zone = kind == MXOPT_HBM_ONE_REGION ? pool->one_region_begin : 0;
  for (int pass = zone ? 0 : 1; pass < 2; ++pass) {
    const size_t from = pass == 0 ? zone : 0;
    for (auto it = pool->free_list.begin(); it != pool->free_list.end(); ++it) {
      const size_t off = it->first, len = it->second;
      const size_t begin = std::max(off, from);
      if (begin >= off + len || off + len - begin < need) continue;
      pool->free_list.erase(it);
      if (begin > off) pool->free_list[off] = begin - off;
      if (off + len > begin + need) pool->free_list[begin + need] = off + len - begin - need;
      pool->live[begin] = need;
      return pool->base + begin;
    }
  }
  return nullptr;
}

int mxopt_hbm_pool_alloc(mxopt_hbm_pool* pool, size_t bytes, void** out) {
  return mxopt_hbm_pool_alloc_kind(pool, bytes, MXOPT_HBM_INTERLEAVED, out);
}

int mxopt_hbm_pool_alloc_kind(mxopt_hbm_pool* pool, size_t bytes, int kind, void** out) {
  if (!pool || !out) return fail(pool ? pool->ctx : nullptr, MXOPT_ERR_INVALID_ARG, "mxopt_hbm_pool_alloc: null argument");
  if (kind != MXOPT_HBM_INTERLEAVED && kind != MXOPT_HBM_ONE_REGION)
    return fail(pool->ctx, MXOPT_ERR_INVALID_ARG, "mxopt_hbm_pool_alloc: unknown kind");
  *out = pool_try_alloc(pool, bytes, kind);
  if (*out) return MXOPT_OK;
  return fail(pool->ctx, MXOPT_ERR_OOM, "mxopt_hbm_pool_alloc: the arena has no free range of " + std::to_string(bytes) + " bytes");
}

int mxopt_hbm_pool_free(mxopt_hbm_pool* pool, void* ptr) {
  if (!pool) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "mxopt_hbm_pool_free: null pool");
  if (!ptr) return MXOPT_OK;
  std::lock_guard<std::mutex> lock(pool->mu);
  const size_t off = (size_t)((char*)ptr - pool->base);
  auto it = pool->live.find(off);
  if ((char*)ptr < pool->base || it == pool->live.end())
    return fail(pool->ctx, MXOPT_ERR_INVALID_ARG, "mxopt_hbm_pool_free: not a live allocation of this pool");
  size_t begin = off, size = it->second;
  pool->live.erase(it);
  auto nextf = pool->free_list.lower_bound(begin);
  if (nextf != pool->free_list.end() && nextf->first == begin + size) {
    size += nextf->second;
    nextf = pool->free_list.erase(nextf);
  }
  if (nextf != pool->free_list.begin()) {
    auto prev = std::prev(nextf);
    if (prev->first + prev->second == begin) {
      begin = prev->first;
      size += prev->second;
      pool->free_list.erase(prev);
    }
  }
  pool->free_list[begin] = size;
  return MXOPT_OK;
}

int mxopt_hbm_pool_owns(const mxopt_hbm_pool* pool, const void* ptr) {
  return pool && ptr && (const char*)ptr >= pool->base && (const char*)ptr < pool->base + pool->capacity;
}

int mxopt_hbm_pool_get_info(mxopt_hbm_pool* pool, mxopt_hbm_pool_info* out) {
  if (!pool || !out) return fail(pool ? pool->ctx : nullptr, MXOPT_ERR_INVALID_ARG, "mxopt_hbm_pool_get_info: null argument");
  std::lock_guard<std::mutex> lock(pool->mu);
  *out = pool->info;
  size_t used = 0;
  for (auto& kv : pool->live) used += kv.second;
  out->used_bytes = used;
  return MXOPT_OK;
}

int mxopt_hbm_classify_regions(int n_slabs, mxopt_slab_probe_fn probe, void* user, int* slab_region,
                               mxopt_hbm_scan_report* report) {
  if (n_slabs < 0 || !probe || (n_slabs && !slab_region))
    return fail(nullptr, MXOPT_ERR_INVALID_ARG, "mxopt_hbm_classify_regions: null argument");
  ScanResult r;
  const SlabProbe fn = [&](int ref, int x, double* gbps) { return probe(user, ref, x, gbps); };
  const int rc = classify_slabs((size_t)n_slabs, fn, ScanLimits{}, &r);
  if (rc) return rc;
  for (int i = 0; i < n_slabs; ++i) slab_region[i] = r.slab_region[(size_t)i];
  if (report) {
    report->regions = r.regions;
    report->probes = r.probes;
    report->same_region_gbps = r.same_region_gbps;
    report->cross_region_gbps = r.cross_region_gbps;
  }
  return MXOPT_OK;
}

int mxopt_hbm_plan_arena(int n_slabs, const int* slab_region, int regions, int chunks_per_slab, int total_chunks,
                         int want_chunks, int max_regions, int* order, mxopt_hbm_arena_report* report) {
  if (n_slabs < 0 || chunks_per_slab < 1 || total_chunks < 0 || want_chunks < 0 || (n_slabs && !slab_region) ||
      (want_chunks && !order))
    return fail(nullptr, MXOPT_ERR_INVALID_ARG, "mxopt_hbm_plan_arena: bad argument");
  const std::vector<int> sr(slab_region, slab_region + n_slabs);
  const ArenaPlan plan = plan_arena(sr, regions, (size_t)chunks_per_slab, (size_t)total_chunks, (size_t)want_chunks, max_regions);
  if (plan.order.size() < (size_t)want_chunks)
    return fail(nullptr, MXOPT_ERR_OOM, "mxopt_hbm_plan_arena: fewer chunks than wanted");
  for (int i = 0; i < want_chunks; ++i) order[i] = (int)plan.order[(size_t)i];
  if (report) {
    report->real_regions = plan.real_regions;
    report->active_regions = plan.active;
    report->interleaved_chunks = (int)plan.interleaved_chunks;
  }
  return MXOPT_OK;
}

int mxopt_set_state_pool(mxopt_ctx* ctx, mxopt_hbm_pool* pool) {
  if (!ctx) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "mxopt_set_state_pool: null context");
  if (pool && pool->ctx->device != ctx->device)
    return fail(ctx, MXOPT_ERR_INVALID_ARG, "mxopt_set_state_pool: the pool lives on another device");
  ctx->state_pool = pool;
  return MXOPT_OK;
}

// ---- hooks with the signature host allocators plug in (torch's CUDAPluggableAllocator) ------------

int mxopt_hbm_pool_set_hook_target(mxopt_hbm_pool* pool) {
  std::lock_guard<std::mutex> lock(g_hook_mu);
  g_hook_pool = pool;
  return MXOPT_OK;
}

int mxopt_hbm_pool_set_hook_kind(int kind) {
  if (kind != MXOPT_HBM_INTERLEAVED && kind != MXOPT_HBM_ONE_REGION)
    return fail(nullptr, MXOPT_ERR_INVALID_ARG, "mxopt_hbm_pool_set_hook_kind: unknown kind");
  std::lock_guard<std::mutex> lock(g_hook_mu);
  g_hook_kind = kind;
  return MXOPT_OK;
}

void* mxopt_hbm_pool_hook_alloc(ptrdiff_t size, int device, void* stream) {
  (void)stream;
  mxopt_hbm_pool* pool;
  int kind;
  {
    std::lock_guard<std::mutex> lock(g_hook_mu);
    pool = g_hook_pool;
    kind = g_hook_kind;
  }
  void* p = nullptr;
  if (pool && pool->ctx->device == device && (p = pool_try_alloc(pool, (size_t)size, kind)) != nullptr) return p;
  int prev = -1;                              // arena full, or no pool: plain device memory
  (void)hipGetDevice(&prev);
  if (prev != device) (void)hipSetDevice(device);
  if (hipMalloc(&p, (size_t)size) != hipSuccess) { (void)hipGetLastError(); p = nullptr; }
  if (prev >= 0 && prev != device) (void)hipSetDevice(prev);
  return p;
}

void mxopt_hbm_pool_hook_free(void* ptr, ptrdiff_t size, int device, void* stream) {
  (void)size; (void)device; (void)stream;
  if (mxopt_hbm_pool* pool = pool_of(ptr)) { (void)mxopt_hbm_pool_free(pool, ptr); return; }
  (void)hipFree(ptr);
}

}  // extern "C"

namespace mxopt {

// Device memory the host layer owns (moments, accumulation buffers): from the context's pool when one
// is attached and has room, else from the driver.
hipError_t state_alloc(mxopt_ctx* ctx, void** out, size_t bytes) {
  *out = nullptr;
  if (ctx->state_pool && (*out = pool_try_alloc(ctx->state_pool, bytes)) != nullptr) return hipSuccess;
  return hipMalloc(out, bytes);
}

void state_free(mxopt_ctx* ctx, void* ptr) {
  (void)ctx;
  if (!ptr) return;
  if (mxopt_hbm_pool* pool = pool_of(ptr)) { (void)mxopt_hbm_pool_free(pool, ptr); return; }
  (void)hipFree(ptr);
}

}  // namespace mxopt
