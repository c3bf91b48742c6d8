// Kernel-instance registry: every translation unit that instantiates kernels exposes one
// "family" function which, given the run-time key of a launch, either launches (or just
// describes) the matching compiled instance or reports that it has none.
#pragma once
#include <atomic>
#include "common.hpp"

namespace gk {

struct InstanceKey {
  int family;        // FAMILY_*
  int BM, BN, BK;
  int waves_m, waves_n;
  int a_kmajor, b_kmajor;   // 1: the K index is contiguous in the operand's memory
  int dtype;         // element type of A and B
  int acc_dtype;     // element type of C / D and of the accumulators (vector-ALU kernels)
  int fused;         // 1: transforms / bias present
  int variant;       // family specific
};

enum : int { FAMILY_MFMA = 0, FAMILY_MFMA_CHECKED = 1, FAMILY_FPU = 2, FAMILY_COMPLEX = 3, FAMILY_DIAGONAL = 4, FAMILY_GETT = 5 };

struct InstanceInfo {
  const char* name;
  int lds_bytes;
  int threads;
};

// mode 0: describe only (fills info), mode 1: describe and launch.
// returns 1 when an instance matched, 0 otherwise; *err receives the launch status.
typedef int (*FamilyFn)(const InstanceKey& key, const GemmArgs& args, dim3 grid, hipStream_t stream, int mode,
                        InstanceInfo* info, hipError_t* err);

// (TAG tells the kernels of one configuration apart: the record of raised LDS limits below is per instantiation)
template <class Cfg, int TAG = 0, class Kernel>
inline int run_instance(Kernel kernel, const char* name, const GemmArgs& args, dim3 grid, hipStream_t stream, int mode,
                        InstanceInfo* info, hipError_t* err, int lds_bytes, int threads) {
  info->name = name;
  info->lds_bytes = lds_bytes;
  info->threads = threads;
  if (mode == 1) {
    hipError_t e = hipSuccess;
    if (lds_bytes > 64 * 1024) {
      // the dynamic LDS limit of a kernel is raised once per device: the call costs tens of
      // microseconds, which a small problem would pay on every launch
      static std::atomic<unsigned long long> raised{0};       // one bit per device, one mask per kernel instance
      int dev = 0;
      e = hipGetDevice(&dev);
      const unsigned long long bit = 1ull << (dev & 63);
      if (e == hipSuccess && !(raised.load(std::memory_order_acquire) & bit)) {
        e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (e == hipSuccess) raised.fetch_or(bit, std::memory_order_release);
      }
    }
    if (e == hipSuccess) {
      hipLaunchKernelGGL(kernel, grid, dim3(threads), lds_bytes, stream, args);
      e = hipGetLastError();
    }
    *err = e;
  }
  return 1;
}

int family_mfma_tn(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);
int family_mfma_nn(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);
int family_mfma_nt(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);
int family_mfma_tt(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);
int family_mfma_wide_tn(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);
int family_mfma_wide_tn_192x256(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);
int family_mfma_wide_nn(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);
int family_mfma_wide_nt(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);
int family_mfma_wide_tt(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);
// (the instances that stream C in: called by the family functions above with the path they chose)
int family_mfma_stream_tn(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*, int path);
int family_mfma_stream_nn(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*, int path);
int family_mfma_stream_nt(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*, int path);
int family_mfma_stream_tt(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*, int path);
int family_fpu(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);
int family_fpu_types(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);
int family_fpu_lanes(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);
int family_fpu_more(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);
int family_mfma_splitk(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);
int family_complex(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);
int family_complex_pair(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);
int family_complex_planar(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);
int family_diagonal(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);
int family_mfma_checked(const InstanceKey&, const GemmArgs&, dim3, hipStream_t, int, InstanceInfo*, hipError_t*);

}  // namespace gk
