// Instances of the vector-ALU GEMM (FPUOp / TropicalFPUOp) and of the bounds-checked MFMA GEMM.
#include "fpu_gemm.hpp"
#include "mfma_checked.hpp"
#include "registry.hpp"

namespace gk {

int family_fpu(const InstanceKey& key, const GemmArgs& args, dim3 grid, hipStream_t stream, int mode, InstanceInfo* info,
               hipError_t* err) {
  // key.variant: bit 0 tropical, bit 1 bounds-checked
#define GK_FPU(bm_, bn_, bk_, wm_, wn_, TYPE, akm_, bkm_, chk_, trop_, NAME)                                               \
  if (key.BM == bm_ && key.BN == bn_ && key.BK == bk_ && key.waves_m == wm_ && key.waves_n == wn_ &&                      \
      key.dtype == DtypeOf<TYPE>::DT && key.acc_dtype == DT_F32 && key.a_kmajor == akm_ && key.b_kmajor == bkm_ && key.variant == (trop_ + 2 * chk_)) { \
    typedef FpuGemmConfig<bm_, bn_, bk_, wm_, wn_, TYPE, (akm_ != 0), (bkm_ != 0), (chk_ != 0), (trop_ != 0)> Cfg;          \
    return run_instance<Cfg>(fpu_gemm_kernel<Cfg>, NAME, args, grid, stream, mode, info, err, Cfg::LDS_BYTES, Cfg::THREADS); \
  }
#define GK_FPU_T(bm_, bn_, bk_, wm_, wn_, TYPE, chk_, trop_, TAG)                         \
  GK_FPU(bm_, bn_, bk_, wm_, wn_, TYPE, 0, 1, chk_, trop_, "fpu_gemm_nn_" TAG)             \
  GK_FPU(bm_, bn_, bk_, wm_, wn_, TYPE, 0, 0, chk_, trop_, "fpu_gemm_nt_" TAG)             \
  GK_FPU(bm_, bn_, bk_, wm_, wn_, TYPE, 1, 1, chk_, trop_, "fpu_gemm_tn_" TAG)             \
  GK_FPU(bm_, bn_, bk_, wm_, wn_, TYPE, 1, 0, chk_, trop_, "fpu_gemm_tt_" TAG)
  GK_FPU_T(64, 64, 32, 2, 2, float, 0, 0, "64x64x32_w2x2_f32")
  GK_FPU_T(64, 64, 32, 2, 2, float, 1, 0, "64x64x32_w2x2_f32_checked")
  GK_FPU_T(128, 128, 16, 2, 2, float, 0, 0, "128x128x16_w2x2_f32")
  GK_FPU_T(64, 64, 32, 2, 2, _Float16, 0, 0, "64x64x32_w2x2_f16")
  GK_FPU_T(64, 64, 32, 2, 2, _Float16, 1, 0, "64x64x32_w2x2_f16_checked")
  GK_FPU_T(64, 64, 32, 2, 2, float, 0, 1, "64x64x32_w2x2_f32_tropical")
  GK_FPU_T(64, 64, 32, 2, 2, float, 1, 1, "64x64x32_w2x2_f32_tropical_checked")
#undef GK_FPU_T
#undef GK_FPU
  // the other element types of FPUOp
  return family_fpu_types(key, args, grid, stream, mode, info, err);
}

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
