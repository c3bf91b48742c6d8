// Vector-ALU GEMM instances (FPUOp) on the lane grids other than 8 x 8: Float32 operands, aligned layouts, the
// 128 x 128 x 16 tile (64 x 64 wave tiles divide by every one of them).  Reference: the base shapes
// OPERATOR_M_BASE x OPERATOR_N_BASE swept at configs/configs.jl:545-550, doubled for 64 lanes.
#include "fpu_instances.inc"

int family_fpu_lanes(const InstanceKey& key, const GemmArgs& args, dim3 grid, hipStream_t stream, int mode, InstanceInfo* info,
                     hipError_t* err) {
  GK_FPU_GRID_T(128, 128, 16, 2, 2, float, 1, 1, "128x128x16_w2x2_f32_lanes1x64")
  GK_FPU_GRID_T(128, 128, 16, 2, 2, float, 2, 2, "128x128x16_w2x2_f32_lanes2x32")
  GK_FPU_GRID_T(128, 128, 16, 2, 2, float, 4, 3, "128x128x16_w2x2_f32_lanes4x16")
  GK_FPU_GRID_T(128, 128, 16, 2, 2, float, 16, 5, "128x128x16_w2x2_f32_lanes16x4")
  GK_FPU_GRID_T(128, 128, 16, 2, 2, float, 32, 6, "128x128x16_w2x2_f32_lanes32x2")
  GK_FPU_GRID_T(128, 128, 16, 2, 2, float, 64, 7, "128x128x16_w2x2_f32_lanes64x1")
  (void)args; (void)grid; (void)stream; (void)mode; (void)info; (void)err;
  return 0;
}

}  // namespace gk
