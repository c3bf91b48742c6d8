// Complex and dual-number GEMM on the matrix cores (WMMAComplexOp / WMMADualOp of the reference,
// src/operator.jl:251-372, with the Interleaved* global layouts of src/layout.jl:276-334).
//
// family_complex() hands a product to one of three sets of instances:
//   * planar global matrices (mfma_complex_planar.hip);
//   * interleaved matrices of which at least one is contiguous along m or n: one real product of the real views
//     (mfma_complex_pair.hip);
//   * interleaved A and B that are both contiguous along k ('T','N'): the instances below.  An interleaved
//     complex product D = A * B is the real product of the expanded matrix [re(A) -im(A); im(A) re(A)] (rows
//     and columns interleaved) with B read as a real matrix of twice the K extent; D comes out interleaved.  So
//     the product runs on the real MFMA kernel with M and K doubled: B and D are used as they are, and the A
//     fragments are expanded in registers (expand_fixup).  Both operands are read with one 16-byte LDS read per
//     fragment, where the real view would need two.
// Tile shapes are in complex elements.  Every instance carries the hooks of C and D and the bias.
#include "mfma_gemm.hpp"
#include "registry.hpp"

namespace gk {

int family_complex(const InstanceKey& key, const GemmArgs& args, dim3 grid, hipStream_t stream, int mode, InstanceInfo* info,
                   hipError_t* err) {
  if (key.dtype != DT_F16 || (key.fused != 0 && key.fused != 3)) return 0;
  if (key.variant == 2) return family_complex_planar(key, args, grid, stream, mode, info, err);   // planar global matrices
  if (!(key.a_kmajor && key.b_kmajor)) return family_complex_pair(key, args, grid, stream, mode, info, err);
  // (32-row blocks: with one complex row feeding two MFMA rows, a 16-row fragment would span 8 tile rows, which the
  // row swizzle of the tile does not leave invariant under the immediate offsets of the reads)
#define GK_CPLX(bm_, bn_, bk_, wm_, wn_, st_, dual_, NAME)                                                                 \
  if (key.BM == bm_ && key.BN == bn_ && key.BK == bk_ && key.waves_m == wm_ && key.waves_n == wn_ && key.variant == dual_) { \
    typedef MfmaGemmConfig<2 * bm_, bn_, 2 * bk_, wm_, wn_, st_, OPK_KMAJOR, OPK_KMAJOR, _Float16, 3, false,               \
                           (dual_ ? FIX_DUAL : FIX_COMPLEX), false, 32> Cfg;                                               \
    return run_instance<Cfg>(mfma_gemm_kernel<Cfg>, NAME, args, grid, stream, mode, info, err, Cfg::LDS_BYTES, Cfg::THREADS); \
  }
  GK_CPLX(64, 128, 32, 2, 2, 3, 0, "mfma_complex_tn_64x128x32_w2x2")
  GK_CPLX(128, 128, 32, 2, 2, 4, 0, "mfma_complex_tn_128x128x32_w2x2")
  GK_CPLX(64, 64, 32, 4, 2, 2, 0, "mfma_complex_tn_64x64x32_w4x2")
  GK_CPLX(32, 64, 32, 2, 2, 2, 0, "mfma_complex_tn_32x64x32_w2x2")
  GK_CPLX(64, 128, 32, 2, 2, 3, 1, "mfma_dual_tn_64x128x32_w2x2")
  GK_CPLX(64, 64, 32, 4, 2, 2, 1, "mfma_dual_tn_64x64x32_w4x2")
  GK_CPLX(32, 64, 32, 2, 2, 2, 1, "mfma_dual_tn_32x64x32_w2x2")
#undef GK_CPLX
  (void)args; (void)grid; (void)stream; (void)mode; (void)info; (void)err;
  return 0;
}

}  // namespace gk
