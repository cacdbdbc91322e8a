// Safetensors reading/writing of float32 device buffers, shared by the optimizer objects.
#pragma once

#include <functional>
#include <string>
#include <vector>

#include "mxopt_internal.h"

namespace mxopt {

struct CheckpointTensor {
  std::string key;        // tensor name in the file
  const float* device;    // n floats in device memory
  uint64_t n;
};

// Writes `tensors` (sorted by key) with __metadata__ {format, optimizer, step} to `path`
// (through path + ".tmp" and a rename).  Synchronises the context's stream.
int save_state_file(mxopt_ctx* ctx, const char* path, const char* optimizer, int64_t step,
                    const std::vector<CheckpointTensor>& tensors);

// Reads a file written by save_state_file (or any safetensors file with the same metadata).  For each
// tensor `place(key, n, &device)` says where its n floats go (NULL = skip it); a non-zero return aborts.
int load_state_file(mxopt_ctx* ctx, const char* path, const char* optimizer, int64_t* step,
                    const std::function<int(const std::string& key, uint64_t n, float** device)>& place);

// Header of a checkpoint without touching a device: optimizer kind, call counter, tensor and element counts.
int inspect_state_file(const char* path, std::string* optimizer, int64_t* step, uint64_t* tensors, uint64_t* elements);

}  // namespace mxopt
