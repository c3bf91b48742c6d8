// Complex GEMM on planar (split re / im) global matrices in one launch (the global-memory
// counterpart of the reference's SplitColMajor / SplitRowMajor layouts, src/layout.jl:340-411, with
// the sign pattern of WMMAComplexOp.mma, src/operator.jl:307-311).
//
// With D = [D_re; D_im] stacked along M, the product is the real GEMM
//     [D_re]   [C_re]   [-A_im]          [A_re]
//     [D_im] = [C_im] + [ A_re] B_im  +  [A_im] B_re
// so it runs on the real MFMA kernel with a real tile of 2*BM rows and two passes over K; only the
// tile addressing and one sign flip of the upper accumulators differ (FIX_PLANAR).  Every element
// of A and B is staged through LDS exactly as in the real kernel; nothing is expanded in registers.
// Every instance carries the hooks of C and D and the bias (they cost nothing when absent).
// Tile shapes below are in complex elements.
#include "mfma_gemm.hpp"
#include "registry.hpp"

namespace gk {

int family_complex_planar(const InstanceKey& key, const GemmArgs& args, dim3 grid, hipStream_t stream, int mode, InstanceInfo* info,
                          hipError_t* err) {
  if (key.dtype != DT_F16 || (key.fused != 0 && key.fused != 3) || key.variant != 2) return 0;
#define GK_PLANAR(bm_, bn_, bk_, wm_, wn_, st_, akm_, bkm_, NAME)                                                          \
  if (key.BM == bm_ && key.BN == bn_ && key.BK == bk_ && key.waves_m == wm_ && key.waves_n == wn_ &&                      \
      key.a_kmajor == akm_ && key.b_kmajor == bkm_) {                                                                     \
    typedef MfmaGemmConfig<2 * bm_, bn_, bk_, wm_, wn_, st_, (akm_ ? OPK_KMAJOR : OPK_MMAJOR),                             \
                           (bkm_ ? OPK_KMAJOR : OPK_MMAJOR), _Float16, 3, false, FIX_PLANAR, false, 16> Cfg;                          \
    return run_instance<Cfg>(mfma_gemm_kernel<Cfg>, NAME, args, grid, stream, mode, info, err, Cfg::LDS_BYTES, Cfg::THREADS); \
  }
#define GK_PLANAR_T(bm_, bn_, bk_, wm_, wn_, st_)                                                               \
  GK_PLANAR(bm_, bn_, bk_, wm_, wn_, st_, 0, 1, "mfma_complex_planar_nn_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_)  \
  GK_PLANAR(bm_, bn_, bk_, wm_, wn_, st_, 0, 0, "mfma_complex_planar_nt_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_)  \
  GK_PLANAR(bm_, bn_, bk_, wm_, wn_, st_, 1, 1, "mfma_complex_planar_tn_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_)  \
  GK_PLANAR(bm_, bn_, bk_, wm_, wn_, st_, 1, 0, "mfma_complex_planar_tt_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_)
  GK_PLANAR_T(128, 256, 64, 2, 4, 2)
  GK_PLANAR_T(128, 128, 64, 2, 2, 2)
  GK_PLANAR_T(64, 128, 64, 2, 2, 2)
  GK_PLANAR_T(64, 128, 32, 2, 2, 4)
  GK_PLANAR_T(64, 64, 32, 2, 2, 2)
#undef GK_PLANAR_T
#undef GK_PLANAR
  (void)args; (void)grid; (void)stream; (void)mode; (void)info; (void)err;
  return 0;
}

}  // namespace gk
