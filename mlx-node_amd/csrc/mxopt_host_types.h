// Plain structs shared by the host API and the kernels: the device-side table layout and
// the opaque handle types behind the C ABI.
#pragma once

#include <hip/hip_runtime_api.h>
#include <stdint.h>

#include <string>
#include <vector>

#include "mxopt.h"
#include "mxopt_diagnostics.h"

namespace mxopt {

constexpr int kChunkElems = MXOPT_CHUNK_ELEMS;
constexpr uint32_t kTfFirst = MXOPT_TF_FIRST;
constexpr uint32_t kTfUnaligned = 0x80000000u;  // set by the table builder: element-wise path
constexpr uint32_t kMaxHead = 7;                // a shifted tensor peels at most this many elements

// One per tensor, in device memory.
struct DevTensor {
  const void* p;
  void* p_out;
  const void* g;
  void* g_out;
  float* m;
  float* v;
  uint64_t n;
  float bc1, bc2;
  uint32_t flags;
  // Elements in front of the first chunk.  When every stream of the tensor becomes 16-byte aligned
  // after the same small number of elements (views into packed slabs), chunk c covers
  // [head + c*kChunkElems, ...) on the 128-bit path and the workgroup of chunk 0 also handles
  // elements [0, head) one by one.
  uint32_t head;
};

// One per kChunkElems-element slice of a tensor, in device memory.
struct DevChunk {
  uint32_t tensor;  // index into the DevTensor array
  uint32_t index;   // chunk number inside that tensor; first element = head + index * kChunkElems
};

constexpr uint32_t kPrepPreMul = 1u, kPrepClampPre = 2u, kPrepClampPost = 4u;
constexpr uint32_t kPrepPendingOnly = 8u;  // update kernels with a pending gradient: g + prep(g2), not prep(g + g2)
constexpr uint32_t kPrepEachStream = 16u;  // list kernels: prep every stream (own clip factor), then add
// with kPrepEachStream: tensor.g holds already prepared micro-batches and is added as it is
constexpr uint32_t kPrepFirstIsSum = 32u;
struct DevPrep {  // kernel argument
  const float* d_scale;
  const unsigned long long* d_skip_if_nonzero;
  float pre_mul, pre_lo, pre_hi, post_lo, post_hi;
  uint32_t flags;
};

// True when a gradient stage runs before the optimizer's own ops: its result is float32 whatever g's dtype.
inline bool prep_promotes(const DevPrep& prep) {
  return (prep.flags & (kPrepPreMul | kPrepClampPre | kPrepClampPost)) != 0 || prep.d_scale != nullptr;
}

// Deferred accumulation with kPrepEachStream: the clip factor of tensor.g and of each pending stream
// (device scalars; all NULL = no factor).
struct StreamScales {
  const float* s[MXOPT_MAX_PENDING + 1];
};

// Tensors of one dtype combination: a contiguous run of chunk entries, one launch.
struct Group {
  int pd, gd, pod, god;
  uint32_t chunk_begin, nchunks;
  bool any_unaligned = false;  // some tensor of the group takes the element-wise path
  uint64_t elems = 0;          // elements of the group's tensors (chunks * kChunkElems when every chunk is full)
};

}  // namespace mxopt

struct mxopt_table;
struct mxopt_hbm_pool;

struct mxopt_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  int num_cus = 0;
  int grid_blocks_per_cu = 16;  // bounded grids (reductions, accumulation): workgroups per CU
  int persistent = 0;           // update kernels: 0 = one workgroup per chunk, 1 = bounded grid
  int nontemporal = 1;          // streaming-hint loads/stores in update, transform, accumulate kernels
  int nontemporal_reduce = 1;   // streaming-hint loads in the read-only reduction kernels
  int persistent_accumulate = 0;  // bounded grid also for accumulation passes that take no norm
  int pipelined_norm = 2;         // plain 16-bit norms: the software-pipelined kernel
  double* d_partial_sum = nullptr;            // one float64 partial per workgroup of a reduction
  size_t partial_cap = 0;
  double* d_static_partials = nullptr;        // this device's copy of the library's fixed partial-sum array
  mxopt_norm_result* d_norm_scratch = nullptr;  // result slot of the gradient utilities
  mxopt_hbm_pool* state_pool = nullptr;         // where the host layer takes moments and accumulation buffers from
  struct CachedTable {                          // tables built by the host layer, most recent last
    std::vector<mxopt_tensor> key;
    mxopt_table* table;
  };
  std::vector<CachedTable> table_cache;
  std::string err;
};

struct mxopt_table {
  mxopt_ctx* ctx = nullptr;
  std::vector<mxopt_tensor> host;             // caller's descriptors (kept for per-step scalar updates)
  std::vector<mxopt::DevTensor> dev;          // staging copy of the device descriptors
  std::vector<mxopt::Group> groups;
  mxopt::DevTensor* d_tensors = nullptr;
  mxopt::DevChunk* d_chunks = nullptr;
  uint64_t total_elems = 0;
  uint64_t num_chunks = 0;
  uint32_t have_mask = 0;                     // which pointers are non-NULL in every non-empty tensor
  mxopt::DevTensor* pinned[2] = {nullptr, nullptr};  // staging for per-step scalar updates
  hipEvent_t copied[2] = {nullptr, nullptr};
  int turn = 0;
  // Deferred accumulation: pending gradient streams, pending_k x tensors pointers (stream-major).
  int pending_k = 0;
  int pending_dtype = 0;
  const void** d_pending = nullptr;                  // MXOPT_MAX_PENDING x tensors slots
  const void** pinned_pending[2] = {nullptr, nullptr};
  hipEvent_t copied_pending[2] = {nullptr, nullptr};
  int turn_pending = 0;
};
