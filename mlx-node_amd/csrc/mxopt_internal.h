// Helpers shared by the two host translation units (mxopt_api.cpp, mxopt_optimizers.cpp).
#pragma once

#include <hip/hip_runtime_api.h>

#include <string>
#include <vector>

#include "mxopt.h"
#include "mxopt_optimizers.h"
#include "mxopt_host_types.h"
#include "mxopt_launch.h"

namespace mxopt {

int fail(mxopt_ctx* ctx, int code, const std::string& msg);
// mxopt_table_retarget without the error report: a refusal because the layout differs sets *why and
// leaves the table as it was; *why stays empty when the descriptor upload itself failed.
int table_retarget_quiet(mxopt_table* t, const mxopt_tensor* tensors, size_t n, std::string* why);
int hip_fail(mxopt_ctx* ctx, hipError_t e, const char* what);

// Logging to stderr, filtered by the environment variable MXOPT_LOG (read once): unset or "off" = nothing,
// "error" = refused calls, "debug" = also one line per launch group, table change and engine decision.
// The counterpart of the reference's tracing subscriber filtered by MLX_NODE_LOG
// (crates/mlx-core/src/tracing.rs:3-21) and of its debug!("Applied gradients ...") (grpo/engine.rs:684).
int log_level();  // 0 off, 1 error, 2 debug
void log_line(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
#define MXOPT_DEBUG(...)                                      \
  do {                                                        \
    if (::mxopt::log_level() >= 2) ::mxopt::log_line(__VA_ARGS__); \
  } while (0)

#define HIP_TRY(ctx, call)                                            \
  do {                                                                \
    hipError_t e_ = (call);                                           \
    if (e_ != hipSuccess) return ::mxopt::hip_fail((ctx), e_, #call); \
  } while (0)

// Makes `dev` current for the calling thread and restores the previous device on exit.
struct DeviceGuard {
  int prev = -1;
  explicit DeviceGuard(int dev) {
    if (hipGetDevice(&prev) != hipSuccess) prev = -1;
    if (prev != dev) (void)hipSetDevice(dev);
  }
  ~DeviceGuard() {
    int cur = -1;
    if (prev >= 0 && hipGetDevice(&cur) == hipSuccess && cur != prev) (void)hipSetDevice(prev);
  }
};

bool float_dtype(int dt);
float round_to_dtype(float x, int dt);
DevPrep make_prep(const mxopt_grad_prep* p);
bool prep_active(const mxopt_grad_prep* p);
uint32_t persistent_grid(const mxopt_ctx* ctx, uint32_t nchunks);
int ensure_partials(mxopt_ctx* ctx, size_t need);
int check_launch(mxopt_ctx* ctx, const char* what);
// partials == NULL: the context's own buffer.
int finish_norm(mxopt_ctx* ctx, uint32_t npartials, double max_norm, int clip_mode, mxopt_norm_result* d_result,
                const double* partials = nullptr);
void fill_dev_tensor(const mxopt_tensor& s, DevTensor& d);
uint64_t chunks_of(const DevTensor& d);  // chunk-table entries (= workgroups of work) of one tensor
// A launch over the single tensor `t` (descriptor passed in the kernel arguments).
Launch make_single_launch(const mxopt_ctx* ctx, const mxopt_tensor& t, bool persistent);


// Device memory the host layer owns (moments, accumulation buffers): from the context's pool
// (mxopt_set_state_pool) while it has room, else from the driver.
hipError_t state_alloc(mxopt_ctx* ctx, void** out, size_t bytes);
void state_free(mxopt_ctx* ctx, void* ptr);

// Shared by the host-layer translation units (mxopt_optimizers.cpp, mxopt_engine.cpp).
mxopt_tensor blank_tensor();  // all pointers NULL, bc1 = bc2 = 1
int check_array(mxopt_ctx* ctx, const mxopt_array* a, const char* what, bool allow_null_data = false);
// Finds or builds the table for `rows` (compared bytewise, per-step scalars excluded); the context
// keeps the most recently used few.
int cached_table(mxopt_ctx* ctx, std::vector<mxopt_tensor>& rows, mxopt_table** out);
int norm_scratch(mxopt_ctx* ctx, mxopt_norm_result** out);
// Puts an optimizer's call counter (mxopt_optimizer_step_count) back: for a caller whose conditional
// update turned out to have been skipped on the device.
void optimizer_set_step_count(mxopt_optimizer* opt, int64_t calls);

}  // namespace mxopt
