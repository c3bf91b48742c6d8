// Complex and dual-number GEMM on the matrix cores (WMMAComplexOp / WMMADualOp of the reference,
// src/operator.jl:251-372, with the Interleaved* global layouts of src/layout.jl:276-334).
//
// family_complex() hands a product to one of two sets of instances, both of which run it as ONE real product of the
// real views of A and B on the K loop of the real kernel and combine the four real products of every element of D
// before the epilogue (mfma_gemm.hpp, FIX_PAIR / FIX_PLANAR):
//   * planar global matrices (mfma_complex_planar.hip);
//   * interleaved global matrices, the reference's form (mfma_complex_pair.hip).
#include "mfma_gemm.hpp"
#include "registry.hpp"

namespace gk {

int family_complex(const InstanceKey& key, const GemmArgs& args, dim3 grid, hipStream_t stream, int mode, InstanceInfo* info,
                   hipError_t* err) {
  if (key.variant == 2) return family_complex_planar(key, args, grid, stream, mode, info, err);
  return family_complex_pair(key, args, grid, stream, mode, info, err);
}

}  // namespace gk
