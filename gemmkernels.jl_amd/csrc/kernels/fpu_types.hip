// Instances of the vector-ALU GEMM for the element types of FPUOp beyond fp32 accumulation
// (reference configs/configs.jl:489-497): Float32 -> Float64, Float64, Int16, Int32, Int64.
#include "fpu_gemm.hpp"
#include "registry.hpp"

namespace gk {

int family_fpu_types(const InstanceKey& key, const GemmArgs& args, dim3 grid, hipStream_t stream, int mode, InstanceInfo* info,
                     hipError_t* err) {
  // key.variant: bit 0 tropical (fp32 only, not here), bit 1 bounds-checked
#define GK_FPU(TIN, TACC, akm_, bkm_, chk_, NAME)                                                                          \
  if (key.BM == 64 && key.BN == 64 && key.BK == 32 && key.waves_m == 2 && key.waves_n == 2 &&                             \
      key.dtype == DtypeOf<TIN>::DT && key.acc_dtype == DtypeOf<TACC>::DT && key.a_kmajor == akm_ && key.b_kmajor == bkm_ && \
      key.variant == 2 * chk_) {                                                                                          \
    typedef FpuGemmConfig<64, 64, 32, 2, 2, TIN, (akm_ != 0), (bkm_ != 0), (chk_ != 0), false, TACC> Cfg;                   \
    return run_instance<Cfg>(fpu_gemm_kernel<Cfg>, NAME, args, grid, stream, mode, info, err, Cfg::LDS_BYTES, Cfg::THREADS); \
  }
#define GK_FPU_T(TIN, TACC, TAG)                                            \
  GK_FPU(TIN, TACC, 0, 1, 0, "fpu_gemm_nn_64x64x32_w2x2_" TAG)               \
  GK_FPU(TIN, TACC, 0, 0, 0, "fpu_gemm_nt_64x64x32_w2x2_" TAG)               \
  GK_FPU(TIN, TACC, 1, 1, 0, "fpu_gemm_tn_64x64x32_w2x2_" TAG)               \
  GK_FPU(TIN, TACC, 1, 0, 0, "fpu_gemm_tt_64x64x32_w2x2_" TAG)               \
  GK_FPU(TIN, TACC, 0, 1, 1, "fpu_gemm_nn_64x64x32_w2x2_" TAG "_checked")    \
  GK_FPU(TIN, TACC, 0, 0, 1, "fpu_gemm_nt_64x64x32_w2x2_" TAG "_checked")    \
  GK_FPU(TIN, TACC, 1, 1, 1, "fpu_gemm_tn_64x64x32_w2x2_" TAG "_checked")    \
  GK_FPU(TIN, TACC, 1, 0, 1, "fpu_gemm_tt_64x64x32_w2x2_" TAG "_checked")
  GK_FPU_T(float, double, "f32_f64")
  GK_FPU_T(double, double, "f64")
  GK_FPU_T(short, short, "i16")
  GK_FPU_T(int, int, "i32")
  GK_FPU_T(long long, long long, "i64")
#undef GK_FPU_T
#undef GK_FPU
  (void)args; (void)grid; (void)stream; (void)mode; (void)info; (void)err;
  return 0;
}

}  // namespace gk
