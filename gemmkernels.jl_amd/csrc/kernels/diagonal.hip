// Instances of the diagonal-A GEMM (Layout.Diagonal).
#include "diagonal.hpp"
#include "registry.hpp"

namespace gk {

int family_diagonal(const InstanceKey& key, const GemmArgs& args, dim3 grid, hipStream_t stream, int mode, InstanceInfo* info,
                    hipError_t* err) {
  if (key.BM % 64 != 0 || key.BN % 64 != 0) return 0;
  const int threads = key.waves_m * key.waves_n * kWaveSize;
  if (threads <= 0 || threads > 1024) return 0;
  const bool row = key.b_kmajor == 0;       // B stored N x K
  const int lds = row ? 64 * 72 * 2 : 0;
  info->lds_bytes = lds;
  info->threads = threads;
  hipError_t e = hipSuccess;
#define GK_DIAG(ROW, TYPE, DT, NAME)                                                                      \
  if (row == ROW && key.dtype == DT) {                                                                    \
    info->name = NAME;                                                                                    \
    if (mode == 1) {                                                                                      \
      hipLaunchKernelGGL((diagonal_gemm_kernel<ROW, TYPE>), grid, dim3(threads), lds, stream, args, key.BM, key.BN); \
      e = hipGetLastError();                                                                              \
      *err = e;                                                                                           \
    }                                                                                                     \
    return 1;                                                                                             \
  }
  GK_DIAG(false, _Float16, DT_F16, "diagonal_gemm_n_f16")
  GK_DIAG(true, _Float16, DT_F16, "diagonal_gemm_t_f16")
  GK_DIAG(false, __bf16, DT_BF16, "diagonal_gemm_n_bf16")
  GK_DIAG(true, __bf16, DT_BF16, "diagonal_gemm_t_bf16")
#undef GK_DIAG
  return 0;
}

}  // namespace gk
