// Instances of the bounds-checked MFMA GEMM.
#include "mfma_checked.hpp"
#include "registry.hpp"

namespace gk {

int family_mfma_checked(const InstanceKey& key, const GemmArgs& args, dim3 grid, hipStream_t stream, int mode,
                        InstanceInfo* info, hipError_t* err) {
#define GK_CHK(bm_, bn_, bk_, wm_, wn_, TYPE, DT, akm_, bkm_, NAME)                                                        \
  if (key.BM == bm_ && key.BN == bn_ && key.BK == bk_ && key.waves_m == wm_ && key.waves_n == wn_ && key.dtype == DT &&   \
      key.a_kmajor == akm_ && key.b_kmajor == bkm_) {                                                                     \
    typedef MfmaCheckedConfig<bm_, bn_, bk_, wm_, wn_, (akm_ != 0), (bkm_ != 0), TYPE> Cfg;                                \
    return run_instance<Cfg>(mfma_gemm_checked_kernel<Cfg>, NAME, args, grid, stream, mode, info, err, Cfg::LDS_BYTES,    \
                             Cfg::THREADS);                                                                               \
  }
#define GK_CHK_T(bm_, bn_, bk_, wm_, wn_, TYPE, DT, TAG)                         \
  GK_CHK(bm_, bn_, bk_, wm_, wn_, TYPE, DT, 0, 1, "mfma_gemm_checked_nn_" TAG)   \
  GK_CHK(bm_, bn_, bk_, wm_, wn_, TYPE, DT, 0, 0, "mfma_gemm_checked_nt_" TAG)   \
  GK_CHK(bm_, bn_, bk_, wm_, wn_, TYPE, DT, 1, 1, "mfma_gemm_checked_tn_" TAG)   \
  GK_CHK(bm_, bn_, bk_, wm_, wn_, TYPE, DT, 1, 0, "mfma_gemm_checked_tt_" TAG)
  GK_CHK_T(64, 64, 32, 2, 2, _Float16, DT_F16, "64x64x32_w2x2_f16")
  GK_CHK_T(64, 64, 32, 2, 2, __bf16, DT_BF16, "64x64x32_w2x2_bf16")
#undef GK_CHK_T
#undef GK_CHK
  (void)args; (void)grid; (void)stream; (void)mode; (void)info; (void)err;
  return 0;
}

}  // namespace gk
