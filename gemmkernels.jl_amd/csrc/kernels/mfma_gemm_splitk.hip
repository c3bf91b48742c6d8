// K-split instances of the MFMA GEMM (kernel kind GK_KERNEL_SPLIT_K): the small tiles that skinny
// products run, all four transposes, FP16 with no hooks, with C / D hooks and bias, or with those and one exact
// FP16 scale on A and B (what the BLAS-style entry points produce), BF16 with no hooks or C / D hooks and bias.
#include "mfma_gemm.hpp"
#include "registry.hpp"

namespace gk {

int family_mfma_splitk(const InstanceKey& key, const GemmArgs& args, dim3 grid, hipStream_t stream, int mode, InstanceInfo* info,
                       hipError_t* err) {
#define GK_SK(bm_, bn_, bk_, wm_, wn_, st_, akm_, bkm_, TYPE, DT, FUSED, NAME)                                              \
  if (key.BM == bm_ && key.BN == bn_ && key.BK == bk_ && key.waves_m == wm_ && key.waves_n == wn_ && key.dtype == DT &&   \
      key.fused == FUSED && key.a_kmajor == akm_ && key.b_kmajor == bkm_) {                                               \
    typedef MfmaGemmConfig<bm_, bn_, bk_, wm_, wn_, st_, (akm_ ? OPK_KMAJOR : OPK_MMAJOR), (bkm_ ? OPK_KMAJOR : OPK_MMAJOR), \
                           TYPE, FUSED, false, FIX_NONE, true, 16> Cfg;                                                        \
    return run_instance<Cfg>(mfma_gemm_kernel<Cfg>, NAME, args, grid, stream, mode, info, err, Cfg::LDS_BYTES, Cfg::THREADS); \
  }
#define GK_SK_T(bm_, bn_, bk_, wm_, wn_, st_, TYPE, DT, FUSED, TAG)                                                                  \
  GK_SK(bm_, bn_, bk_, wm_, wn_, st_, 0, 1, TYPE, DT, FUSED, "mfma_gemm_splitk_nn_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_ TAG)  \
  GK_SK(bm_, bn_, bk_, wm_, wn_, st_, 0, 0, TYPE, DT, FUSED, "mfma_gemm_splitk_nt_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_ TAG)  \
  GK_SK(bm_, bn_, bk_, wm_, wn_, st_, 1, 1, TYPE, DT, FUSED, "mfma_gemm_splitk_tn_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_ TAG)  \
  GK_SK(bm_, bn_, bk_, wm_, wn_, st_, 1, 0, TYPE, DT, FUSED, "mfma_gemm_splitk_tt_" #bm_ "x" #bn_ "x" #bk_ "_w" #wm_ "x" #wn_ TAG)
#define GK_SK_TILE(bm_, bn_, bk_, wm_, wn_, st_)                            \
  GK_SK_T(bm_, bn_, bk_, wm_, wn_, st_, _Float16, DT_F16, 0, "_f16")        \
  GK_SK_T(bm_, bn_, bk_, wm_, wn_, st_, _Float16, DT_F16, 1, "_f16_fused")  \
  GK_SK_T(bm_, bn_, bk_, wm_, wn_, st_, _Float16, DT_F16, 3, "_f16_fused_cd")  \
  GK_SK_T(bm_, bn_, bk_, wm_, wn_, st_, __bf16, DT_BF16, 0, "_bf16")  \
  GK_SK_T(bm_, bn_, bk_, wm_, wn_, st_, __bf16, DT_BF16, 3, "_bf16_fused_cd")
  GK_SK_TILE(128, 128, 64, 2, 2, 2)
  GK_SK_TILE(64, 64, 64, 2, 2, 4)
  GK_SK_TILE(64, 64, 32, 1, 1, 2)
#undef GK_SK_TILE
#undef GK_SK_T
#undef GK_SK
  (void)args; (void)grid; (void)stream; (void)mode; (void)info; (void)err;
  return 0;
}

}  // namespace gk
