"""GemmKernels for the MI355X: the host API of GemmKernels.jl (Config, Layouts, Transforms,
Operators, Epilogues, CTA swizzles, ``matmul`` / ``matmatmul_`` / ``mul_``) over hand-written
gfx950 HIP kernels in libgemmkernels_hip.so.

Mirrors reference src/GemmKernels.jl:1-23 module by module.
"""
from . import tiling as Tiling
from . import layout as Layout
from . import operator as Operator
from . import transform as Transform
from . import epilogue as Epilogue
from . import kernel as Kernel
from . import cta_swizzle as CTASwizzle
from .config import Config, get_config, heuristic_block_shape, adjacent_elements, default_block_shape, check_config
from .dtypes import Float16, BFloat16, Float32, Float64, Int16, Int32, Int64, ComplexF16, ComplexF32, DType
from .errors import ConfigError, DimensionMismatch
from .matmul import matmul, plan, Plan, specialize, SpecializedKernel, matmatmul_plan, matmatmul_, mul_, create_config, Transpose, Adjoint, kernel_name
from .arrays import colmajor, colmajor_empty, to_numpy, bf16_bits, bf16_values
from .tiling import NT
from . import contraction
from .contraction import contract

__all__ = ["Tiling", "Layout", "Operator", "Transform", "Epilogue", "Kernel", "CTASwizzle", "Config", "get_config",
           "heuristic_block_shape", "adjacent_elements", "default_block_shape", "check_config", "ConfigError",
           "DimensionMismatch", "matmul", "plan", "Plan", "specialize", "SpecializedKernel", "matmatmul_plan", "matmatmul_", "mul_", "create_config", "Transpose", "Adjoint", "kernel_name",
           "colmajor", "colmajor_empty", "to_numpy", "bf16_bits", "bf16_values", "NT", "Float16", "BFloat16", "Float32", "Float64", "Int16", "Int32", "Int64", "ComplexF16",
           "ComplexF32", "DType", "contraction", "contract"]
