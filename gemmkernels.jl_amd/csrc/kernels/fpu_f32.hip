// Vector-ALU GEMM instances (FPUOp): Float32 operands, aligned layouts.
#include "fpu_instances.inc"

int family_fpu(const InstanceKey& key, const GemmArgs& args, dim3 grid, hipStream_t stream, int mode, InstanceInfo* info,
               hipError_t* err) {
  GK_FPU_T(64, 64, 32, 2, 2, float, 0, 0, true, "64x64x32_w2x2_f32")
  GK_FPU_T(32, 32, 32, 1, 1, float, 0, 0, true, "32x32x32_w1x1_f32")     // small problems: four times the workgroups of 64 x 64
  GK_FPU_T(32, 32, 32, 2, 2, float, 0, 0, true, "32x32x32_w2x2_f32")     // ... on four waves: 2 x 2 outputs per lane, a quarter of the fma chain per lane
  GK_FPU_T(128, 128, 16, 2, 2, float, 0, 0, false, "128x128x16_w2x2_f32")
  // the other lane grids of a wave
  if ((key.variant >> 4) != 0) return family_fpu_lanes(key, args, grid, stream, mode, info, err);
  // bounds-checked layouts, Float16 operands, the max-plus product
  return family_fpu_more(key, args, grid, stream, mode, info, err);
}

}  // namespace gk
