// Shared between the translation units of the host layer (not part of the C ABI).
#pragma once
#include <hip/hip_runtime.h>

#include "gemmkernels_hip.h"
#include "kernels/common.hpp"
#include "kernels/registry.hpp"

namespace gk_internal {

// Records the thread-local error message and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

struct Launch {
  gk::InstanceKey key;
  gk::InstanceInfo info;
  gk::GemmArgs args;
  int gx, gy;
  bool ragged;      // an aligned kernel runs bounds-checked layouts and has to take the last K tile out of its pipeline
};

int prepare_launch(const gk_config* conf, const void* a, const void* b, const void* c, void* d, const gk_transforms* transforms,
                   const gk_epilogue* epilogue, int32_t kernel, const gk::InstanceInfo* custom, Launch* out);

// The K-split launch on a workspace of `workspace_bytes` bytes at `workspace` ([arrival counters | partial tiles]);
// `whose` names the workspace in the message that refuses a launch it cannot hold.
int launch_split_k(const gk_config* conf, const void* a, const void* b, const void* c, void* d, const gk_transforms* transforms,
                   const gk_epilogue* epilogue, void* workspace, size_t workspace_bytes, const char* whose, void* stream);

}  // namespace gk_internal
