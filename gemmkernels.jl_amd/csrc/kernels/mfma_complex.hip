// Complex and dual-number GEMM on the matrix cores (WMMAComplexOp / WMMADualOp of the reference,
// src/operator.jl:251-372, with the Interleaved* global layouts of src/layout.jl:276-334).
//
// An interleaved complex product D = A * B is the real product of the expanded matrix
// [re(A) -im(A); im(A) re(A)] (rows and columns interleaved) with B read as a real matrix of twice
// the K extent; D comes out interleaved.  So the complex GEMM runs on the real MFMA kernel with
// M and K doubled: B and D are used as they are, and the A fragments are expanded in registers
// (expand_fixup).  Tile shapes below are in complex elements.
#include "mfma_gemm.hpp"
#include "registry.hpp"

#ifndef GK_CPLX_MI
// MFMA block of the complex / dual instances with A contiguous along m (16: v_mfma_f32_16x16x32).  With a
// K-major A (one complex row feeds two MFMA rows) a 16-row fragment spans 8 tile rows, which the row swizzle
// of the tile does not leave invariant under the immediate offsets of the reads: those stay with 32.
#define GK_CPLX_MI 16
#endif

namespace gk {

int family_complex(const InstanceKey& key, const GemmArgs& args, dim3 grid, hipStream_t stream, int mode, InstanceInfo* info,
                   hipError_t* err) {
  if (key.dtype != DT_F16 || key.fused != 0) return 0;
  if (key.variant == 2) return family_complex_planar(key, args, grid, stream, mode, info, err);   // planar global matrices
#define GK_CPLX(bm_, bn_, bk_, wm_, wn_, st_, akm_, bkm_, dual_, NAME)                                                     \
  if (key.BM == bm_ && key.BN == bn_ && key.BK == bk_ && key.waves_m == wm_ && key.waves_n == wn_ &&                      \
      key.a_kmajor == akm_ && key.b_kmajor == bkm_ && key.variant == dual_) {                                             \
    typedef MfmaGemmConfig<2 * bm_, bn_, 2 * bk_, wm_, wn_, st_, (akm_ ? OPK_KMAJOR : OPK_CROWK),                          \
                           (bkm_ ? OPK_KMAJOR : OPK_CROWK), _Float16, 0, false, (dual_ ? FIX_DUAL : FIX_COMPLEX), false, (akm_ ? 32 : GK_CPLX_MI)> Cfg; \
    return run_instance<Cfg>(mfma_gemm_kernel<Cfg>, NAME, args, grid, stream, mode, info, err, Cfg::LDS_BYTES, Cfg::THREADS); \
  }
#define GK_CPLX_T(bm_, bn_, bk_, wm_, wn_, st_, dual_, TAG)                                     \
  GK_CPLX(bm_, bn_, bk_, wm_, wn_, st_, 0, 1, dual_, "mfma_" TAG "_nn_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_)  \
  GK_CPLX(bm_, bn_, bk_, wm_, wn_, st_, 0, 0, dual_, "mfma_" TAG "_nt_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_)  \
  GK_CPLX(bm_, bn_, bk_, wm_, wn_, st_, 1, 1, dual_, "mfma_" TAG "_tn_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_)  \
  GK_CPLX(bm_, bn_, bk_, wm_, wn_, st_, 1, 0, dual_, "mfma_" TAG "_tt_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_)
  GK_CPLX_T(128, 256, 32, 2, 4, 3, 0, "complex")
  GK_CPLX_T(128, 128, 32, 2, 2, 4, 0, "complex")
  GK_CPLX_T(64, 128, 32, 2, 2, 3, 0, "complex")
  GK_CPLX_T(64, 64, 32, 4, 2, 2, 0, "complex")
  GK_CPLX_T(32, 64, 32, 2, 2, 2, 0, "complex")
  GK_CPLX_T(64, 128, 32, 2, 2, 3, 1, "dual")
  GK_CPLX_T(64, 64, 32, 4, 2, 2, 1, "dual")
#undef GK_CPLX_T
#undef GK_CPLX
  (void)args; (void)grid; (void)stream; (void)mode; (void)info; (void)err;
  return 0;
}

}  // namespace gk
