// Vector-ALU GEMM instances (FPUOp / TropicalFPUOp): bounds-checked Float32, Float16 operands, max-plus.
#include "fpu_instances.inc"

int family_fpu_more(const InstanceKey& key, const GemmArgs& args, dim3 grid, hipStream_t stream, int mode, InstanceInfo* info,
                    hipError_t* err) {
  GK_FPU_T(64, 64, 32, 2, 2, float, 1, 0, false, "64x64x32_w2x2_f32_checked")
  GK_FPU_T(64, 64, 32, 2, 2, _Float16, 0, 0, false, "64x64x32_w2x2_f16")
  GK_FPU_T(64, 64, 32, 2, 2, _Float16, 1, 0, false, "64x64x32_w2x2_f16_checked")
  GK_FPU_T(64, 64, 32, 2, 2, float, 0, 1, false, "64x64x32_w2x2_f32_tropical")
  GK_FPU_T(64, 64, 32, 2, 2, float, 1, 1, false, "64x64x32_w2x2_f32_tropical_checked")
  // the other element types of FPUOp
  return family_fpu_types(key, args, grid, stream, mode, info, err);
}

}  // namespace gk
