// The K-split launch for callers that cannot allocate device memory (code under HIP graph capture, serving
// loops, harnesses that forbid it): the workspace in which the K slices of an output tile meet is a
// file-scope device array of this translation unit instead of a buffer the caller brings.
#include "gemmkernels_hip.h"

#include <hip/hip_runtime.h>

#include <mutex>

#include "gk_internal.hpp"

namespace {

using gk_internal::fail;

// [arrival counters | partial tiles] of one K-split launch.  Every GPU the library runs on holds its own
// copy, at its own address, until the process ends; the loader hands it out zeroed and every launch leaves
// the counters at zero again.
constexpr size_t kScratchBytes = (size_t)32 << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::once_flag g_once[kMaxDevices];
void* g_scratch_ptr[kMaxDevices];
hipError_t g_scratch_err[kMaxDevices];

// Device address of `scratch` on the current device.  In host code the array's name is only a handle for
// the symbol, not an address a kernel could use: the address is asked of the runtime once per device.
int scratch_address(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(GK_ERR_HIP, "hipGetDevice failed: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(GK_ERR_UNSUPPORTED, "device ordinal %d is beyond the %d the static workspace table holds", dev, kMaxDevices);
  std::call_once(g_once[dev], [dev]() {
    void* p = nullptr;
    g_scratch_err[dev] = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    g_scratch_ptr[dev] = g_scratch_err[dev] == hipSuccess ? p : nullptr;
  });
  if (g_scratch_err[dev] != hipSuccess || !g_scratch_ptr[dev])
    return fail(GK_ERR_HIP, "hipGetSymbolAddress of the static K-split workspace failed on device %d: %s", dev, hipGetErrorString(g_scratch_err[dev]));
  *out = g_scratch_ptr[dev];
  return GK_OK;
}

}  // namespace

extern "C" {

size_t gk_split_k_noalloc_capacity(void) { return kScratchBytes; }

int gk_matmul_split_k_noalloc(const gk_config* conf, const void* a, const void* b, const void* c, void* d, const gk_transforms* transforms,
                              const gk_epilogue* epilogue, void* stream) {
  void* ws = nullptr;
  int rc = scratch_address(&ws);
  if (rc != GK_OK) return rc;
  return gk_internal::launch_split_k(conf, a, b, c, d, transforms, epilogue, ws, kScratchBytes,
                                     "the library's static workspace (gk_matmul_split_k_noalloc)", stream);
}

}  // extern "C"
