// Host-side launch interface between the C ABI (mxopt_api.cpp) and the kernels.
#pragma once

#include <hip/hip_runtime_api.h>
#include <stdint.h>

#include "mxopt.h"
#include "mxopt_host_types.h"

namespace mxopt {

// One launch = one dtype group of a table (a contiguous run of chunk entries), or -- when
// `chunks` is NULL -- the single tensor `one`, whose descriptor travels in the kernel
// arguments so that nothing has to be staged in device memory.
struct Launch {
  const DevTensor* tensors = nullptr;
  const DevChunk* chunks = nullptr;  // first chunk of the group
  DevTensor one{};
  uint32_t nchunks = 0;
  uint32_t grid = 0;                 // workgroups (<= nchunks)
  hipStream_t stream = nullptr;
  int nontemporal = 1;               // non-zero: streaming-hint loads and stores
  int pipelined_norm = 2;            // plain 16-bit norms take the software-pipelined kernel
  bool any_unaligned = false;        // some tensor of the launch takes the element-wise path
  bool partial_chunks = false;       // the chunks are under 90 % full on average (many small tensors)
  // Deferred accumulation (the *_list launchers): stream j of table row r is pending[j * ntensors + r].
  const void* const* pending = nullptr;
  uint32_t ntensors = 0;
  int npending = 0;
  StreamScales scales{};             // used when the prep carries kPrepEachStream
};

// Each returns false when the dtype combination has no kernel.
// g2d >= 0: tensor.g_out holds a second gradient of that dtype which is added to g (float32) first.
bool launch_adam(int pd, int gd, int od, int g2d, const Launch& L, const mxopt_adam_hp& hp, const DevPrep& prep);
bool launch_sgd(int pd, int gd, int od, const Launch& L, const mxopt_sgd_hp& hp, const DevPrep& prep);
bool launch_rmsprop(int pd, int gd, int od, const Launch& L, const mxopt_rmsprop_hp& hp, const DevPrep& prep);
// g_promoted: the gradient reaches the multiply as float32 (decay or a prep stage ran first).
bool launch_sgd_plain(int pd, int gd, int od, const Launch& L, float lr_p, float wd, int has_wd, bool g_promoted,
                      const DevPrep& prep);
// add != 0: g_out = g_out + prep(g) instead of g_out = prep(g).
// g: float32 accumulation buffer, tensor.g_out: pending gradient of dtype g2d; prep's kPrepPendingOnly
// flag says whether prep covers the pending gradient alone or the sum.
bool launch_sgd_plain_pending(int pd, int gd, int od, int g2d, const Launch& L, float lr_p, float wd, int has_wd,
                              const DevPrep& prep);
bool launch_transform(int gd, int od, const Launch& L, const DevPrep& prep, int add);
// mode 0: square g; 1: square g_out; 2: g_out = first ? g : g_out + g, square the result;
// 3: square g_out + g without storing it.
// partial_sum (one entry per workgroup) may be NULL in mode 2.
bool launch_sumsq(int mode, int ad, int gd, const Launch& L, const DevPrep& prep, int first, double* partial_sum);
// Deferred accumulation: the gradient is g + pending_0 + ... (float32 adds, left to right); xd is the
// pending streams' dtype, gd either xd or float32.  Parameters are updated in their own dtype.
bool launch_adam_list(int pd, int gd, int od, int xd, const Launch& L, const mxopt_adam_hp& hp, const DevPrep& prep);
bool launch_sgd_plain_list(int pd, int gd, int od, int xd, const Launch& L, float lr_p, float wd, int has_wd,
                           const DevPrep& prep);
bool launch_sgd_list(int pd, int gd, int od, int xd, const Launch& L, const mxopt_sgd_hp& hp, const DevPrep& prep);
bool launch_rmsprop_list(int pd, int gd, int od, int xd, const Launch& L, const mxopt_rmsprop_hp& hp,
                         const DevPrep& prep);
bool launch_sumsq_list(int gd, int xd, const Launch& L, const DevPrep& prep, double* partial_sum);
bool launch_synth(int od, void* out, uint64_t n, uint64_t seed, uint64_t first_index, int dist, float a, float b,
                  uint32_t grid, hipStream_t stream);
// *host_mapped_dst = *d_src by a one-lane kernel (dst: pinned host memory, visible to the device).
void launch_mirror_result(hipStream_t stream, const mxopt_norm_result* d_src, mxopt_norm_result* host_mapped_dst);
// Address, on `device` (which must be the current device), of the library's fixed array of
// kStaticPartials float64 partial sums: every GPU holds its own copy at its own address.
constexpr uint32_t kStaticPartials = MXOPT_STATIC_NORM_WORKGROUPS;
hipError_t static_partials_address(int device, double** out);
void launch_norm_finish(hipStream_t stream, const double* partial_sum, uint32_t npartials, double max_norm,
                        int has_max, int clip_mode, mxopt_norm_result* d_out);

}  // namespace mxopt
