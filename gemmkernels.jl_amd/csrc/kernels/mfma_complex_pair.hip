// Complex and dual-number GEMM on interleaved global matrices as ONE real product of the matrices seen as real
// ones (WMMAComplexOp / WMMADualOp of the reference, src/operator.jl:251-372, with the Interleaved* global
// layouts of src/layout.jl:276-334).
//
// An interleaved Complex{Float16} matrix that is contiguous along m (A of an 'N' product, B of a 'T' one) IS a
// real FP16 matrix with twice the rows, row 2m the real and row 2m+1 the imaginary parts: the real kernel
// stages and reads it like any other matrix.  One that is contiguous along k is staged as it lies (OPK_KSPLIT) and
// a lane makes a fragment of real parts and a fragment of imaginary parts out of the 32 bytes it reads.  Either way
// the 2M x 2N real product of the two views holds re*re, re*im, im*re and im*im of every element of D, and they are
// combined once, before the epilogue (FIX_PAIR in mfma_gemm.hpp): nothing else happens on the way to the matrix
// cores, and the K loop is the one of the real kernel on a 256 x 256 x 64 real tile.
// Tile shapes below are in complex elements; the real tile has twice the rows and columns.
#include "mfma_gemm.hpp"
#include "registry.hpp"

namespace gk {

int family_complex_pair(const InstanceKey& key, const GemmArgs& args, dim3 grid, hipStream_t stream, int mode, InstanceInfo* info,
                        hipError_t* err) {
  if (key.dtype != DT_F16 || (key.fused != 0 && key.fused != 3) || key.variant > 1) return 0;
  // every instance carries the hooks of C and D and the bias (FUSE level 3: they cost nothing when absent)
#define GK_PAIR(bm_, bn_, bk_, wm_, wn_, st_, akm_, bkm_, dual_, NAME)                                                     \
  if (key.BM == bm_ && key.BN == bn_ && key.BK == bk_ && key.waves_m == wm_ && key.waves_n == wn_ &&                      \
      key.a_kmajor == akm_ && key.b_kmajor == bkm_ && key.variant == dual_) {                                             \
    typedef MfmaGemmConfig<2 * bm_, 2 * bn_, bk_, wm_, wn_, st_, (akm_ ? OPK_KSPLIT : OPK_MMAJOR),                         \
                           (bkm_ ? OPK_KSPLIT : OPK_MMAJOR), _Float16, 3, false, (dual_ ? FIX_PAIR_DUAL : FIX_PAIR), false, 16> Cfg; \
    return run_instance<Cfg>(mfma_gemm_kernel<Cfg>, NAME, args, grid, stream, mode, info, err, Cfg::LDS_BYTES, Cfg::THREADS); \
  }
#define GK_PAIR_T(bm_, bn_, bk_, wm_, wn_, st_, dual_, TAG)                                                         \
  GK_PAIR(bm_, bn_, bk_, wm_, wn_, st_, 0, 1, dual_, "mfma_" TAG "_nn_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_)  \
  GK_PAIR(bm_, bn_, bk_, wm_, wn_, st_, 0, 0, dual_, "mfma_" TAG "_nt_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_)  \
  GK_PAIR(bm_, bn_, bk_, wm_, wn_, st_, 1, 1, dual_, "mfma_" TAG "_tn_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_)  \
  GK_PAIR(bm_, bn_, bk_, wm_, wn_, st_, 1, 0, dual_, "mfma_" TAG "_tt_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_)
  // 'N','N' on four waves, one per SIMD (MfmaGemmConfig::SOLO; launches without hooks): one kernel per way of moving C and D
#define GK_PAIR_SOLO(dual_, NAME)                                                                                         \
  if (key.BM == 128 && key.BN == 128 && key.BK == 64 && key.waves_m == 2 && key.waves_n == 2 && key.a_kmajor == 0 &&     \
      key.b_kmajor == 1 && key.variant == dual_ && key.fused == 0) {                                                      \
    typedef MfmaGemmConfig<256, 256, 64, 2, 2, 2, OPK_MMAJOR, OPK_KSPLIT, _Float16, 0, false, (dual_ ? FIX_PAIR_DUAL : FIX_PAIR), false, 16> Cfg; \
    static_assert(Cfg::SOLO, "the four-wave arrangement");                                                               \
    const int path = mode == 1 ? solo_cd_path(args) : 0;                                                                 \
    if (path == 1) return run_instance<Cfg, 1>(mfma_gemm_kernel<Cfg, 1>, NAME, args, grid, stream, mode, info, err, Cfg::LDS_BYTES, Cfg::THREADS); \
    if (path == 2) return run_instance<Cfg, 2>(mfma_gemm_kernel<Cfg, 2>, NAME, args, grid, stream, mode, info, err, Cfg::LDS_BYTES, Cfg::THREADS); \
    return run_instance<Cfg, 0>(mfma_gemm_kernel<Cfg, 0>, NAME, args, grid, stream, mode, info, err, Cfg::LDS_BYTES, Cfg::THREADS); \
  }
  GK_PAIR_SOLO(0, "mfma_complex_pair_nn_128x128x64_w2x2")
  GK_PAIR_SOLO(1, "mfma_dual_pair_nn_128x128x64_w2x2")
#undef GK_PAIR_SOLO
  GK_PAIR_T(128, 128, 64, 2, 4, 2, 0, "complex_pair")
  GK_PAIR_T(64, 64, 64, 2, 2, 2, 0, "complex_pair")
  GK_PAIR_T(64, 64, 32, 2, 2, 4, 0, "complex_pair")
  GK_PAIR_T(32, 32, 32, 2, 2, 4, 0, "complex_pair")
  GK_PAIR_T(128, 128, 64, 2, 4, 2, 1, "dual_pair")
  GK_PAIR_T(64, 64, 64, 2, 2, 2, 1, "dual_pair")
  GK_PAIR_T(64, 64, 32, 2, 2, 4, 1, "dual_pair")
  GK_PAIR_T(32, 32, 32, 2, 2, 4, 1, "dual_pair")
#undef GK_PAIR_T
#undef GK_PAIR
  (void)args; (void)grid; (void)stream; (void)mode; (void)info; (void)err;
  return 0;
}

}  // namespace gk
