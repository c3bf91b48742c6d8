// Complex GEMM on planar (split re / im) global matrices in one launch (the global-memory
// counterpart of the reference's SplitColMajor / SplitRowMajor layouts, src/layout.jl:340-411, with
// the products of WMMAComplexOp.mma, src/operator.jl:307-311).
//
// The planes of a planar matrix are plain real matrices, so the product is ONE real product of the real views
// [A_re; A_im] (2M x K) and [B_re, B_im] (K x 2N), like the interleaved form (mfma_complex_pair.hip), on the K loop
// of the real kernel.  Only the tile addressing differs: the rows and columns of a tile are dealt out so that every
// wave holds both parts of its complex rows and columns, and the four real products of an element of D are combined
// inside a lane before the epilogue (FIX_PLANAR in mfma_gemm.hpp).  All four transposes read their operands the way
// the real kernel does: nothing is expanded or read twice.
// Every instance carries the hooks of C and D and the bias (they cost nothing when absent).
// Tile shapes below are in complex elements; the real tile has twice the rows and columns.
#include "mfma_gemm.hpp"
#include "registry.hpp"

namespace gk {

int family_complex_planar(const InstanceKey& key, const GemmArgs& args, dim3 grid, hipStream_t stream, int mode, InstanceInfo* info,
                          hipError_t* err) {
  if (key.dtype != DT_F16 || (key.fused != 0 && key.fused != 3) || key.variant != 2) return 0;
#define GK_PLANAR(bm_, bn_, bk_, wm_, wn_, st_, akm_, bkm_, NAME)                                                          \
  if (key.BM == bm_ && key.BN == bn_ && key.BK == bk_ && key.waves_m == wm_ && key.waves_n == wn_ &&                      \
      key.a_kmajor == akm_ && key.b_kmajor == bkm_) {                                                                     \
    typedef MfmaGemmConfig<2 * bm_, 2 * bn_, bk_, wm_, wn_, st_, (akm_ ? OPK_KMAJOR : OPK_MMAJOR),                             \
                           (bkm_ ? OPK_KMAJOR : OPK_MMAJOR), _Float16, 3, false, FIX_PLANAR, false, 16> Cfg;                          \
    return run_instance<Cfg>(mfma_gemm_kernel<Cfg>, NAME, args, grid, stream, mode, info, err, Cfg::LDS_BYTES, Cfg::THREADS); \
  }
#define GK_PLANAR_T(bm_, bn_, bk_, wm_, wn_, st_)                                                               \
  GK_PLANAR(bm_, bn_, bk_, wm_, wn_, st_, 0, 1, "mfma_complex_planar_nn_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_)  \
  GK_PLANAR(bm_, bn_, bk_, wm_, wn_, st_, 0, 0, "mfma_complex_planar_nt_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_)  \
  GK_PLANAR(bm_, bn_, bk_, wm_, wn_, st_, 1, 1, "mfma_complex_planar_tn_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_)  \
  GK_PLANAR(bm_, bn_, bk_, wm_, wn_, st_, 1, 0, "mfma_complex_planar_tt_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_)
  // four waves, one per SIMD (MfmaGemmConfig::SOLO; launches without hooks): one kernel per way of moving C and D
#define GK_PLANAR_SOLO(akm_, bkm_, NAME)                                                                                  \
  if (key.BM == 128 && key.BN == 128 && key.BK == 64 && key.waves_m == 2 && key.waves_n == 2 && key.a_kmajor == akm_ &&  \
      key.b_kmajor == bkm_ && key.fused == 0) {                                                                           \
    typedef MfmaGemmConfig<256, 256, 64, 2, 2, 2, (akm_ ? OPK_KMAJOR : OPK_MMAJOR), (bkm_ ? OPK_KMAJOR : OPK_MMAJOR), _Float16, 0, false, FIX_PLANAR, false, 16> Cfg; \
    static_assert(Cfg::SOLO, "the four-wave arrangement");                                                               \
    const int path = mode == 1 ? solo_cd_path(args) : 0;                                                                 \
    if (path == 1) return run_instance<Cfg, 1>(mfma_gemm_kernel<Cfg, 1>, NAME, args, grid, stream, mode, info, err, Cfg::LDS_BYTES, Cfg::THREADS); \
    if (path == 2) return run_instance<Cfg, 2>(mfma_gemm_kernel<Cfg, 2>, NAME, args, grid, stream, mode, info, err, Cfg::LDS_BYTES, Cfg::THREADS); \
    return run_instance<Cfg, 0>(mfma_gemm_kernel<Cfg, 0>, NAME, args, grid, stream, mode, info, err, Cfg::LDS_BYTES, Cfg::THREADS); \
  }
  GK_PLANAR_SOLO(0, 1, "mfma_complex_planar_nn_128x128x64_w2x2")
  GK_PLANAR_SOLO(0, 0, "mfma_complex_planar_nt_128x128x64_w2x2")
  GK_PLANAR_SOLO(1, 1, "mfma_complex_planar_tn_128x128x64_w2x2")
  GK_PLANAR_SOLO(1, 0, "mfma_complex_planar_tt_128x128x64_w2x2")
#undef GK_PLANAR_SOLO
  GK_PLANAR_T(128, 128, 64, 2, 4, 2)
  GK_PLANAR_T(64, 64, 64, 2, 2, 2)
  GK_PLANAR_T(64, 64, 32, 2, 2, 4)
  GK_PLANAR_T(32, 32, 32, 2, 2, 4)
#undef GK_PLANAR_T
#undef GK_PLANAR
  (void)args; (void)grid; (void)stream; (void)mode; (void)info; (void)err;
  return 0;
}

}  // namespace gk
