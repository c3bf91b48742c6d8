"""Operators: the inner-product engine of a warp tile (reference src/operator.jl)."""
from __future__ import annotations

from dataclasses import dataclass

from .dtypes import DType
from .tiling import NT

# gk_operator_kind
MFMA, FPU, FPU_TROPICAL, MFMA_COMPLEX, MFMA_DUAL = range(5)


@dataclass(frozen=True)
class OperatorType:
    kind: int
    M: int
    N: int
    K: int
    CT: DType
    AT: DType
    mb: int = 0
    nb: int = 0
    kb: int = 0
    name: str = ""

    def __repr__(self):
        if self.kind in (FPU, FPU_TROPICAL):
            return f"Operator.{self.name}{{{self.M}, {self.N}, {self.K}, {self.mb}, {self.nb}, {self.kb}, {self.CT}, {self.AT}}}"
        return f"Operator.{self.name}{{{self.M}, {self.N}, {self.K}, {self.CT}, {self.AT}}}"


class _MatrixCoreOp:
    def __init__(self, kind, name):
        self.kind, self.name = kind, name

    def __getitem__(self, args) -> OperatorType:
        M, N, K, CT, AT = args
        return OperatorType(self.kind, M, N, K, CT, AT, name=self.name)


class _FPUOp:
    def __init__(self, kind, name):
        self.kind, self.name = kind, name

    def __getitem__(self, args) -> OperatorType:
        M, N, K, mb, nb, kb, CT, AT = args
        return OperatorType(self.kind, M, N, K, CT, AT, mb, nb, kb, name=self.name)


# The matrix-core operator.  MFMAOp[32, 32, 16, CT, AT] is v_mfma_f32_32x32x16_{f16,bf16}.
# WMMAOp keeps the reference's name and shapes ((16,16,16), (8,32,16), (32,8,16), reference
# src/operator.jl:163-245, src/config.jl:159-169); such a config runs on the same MFMA
# instruction as long as its warp tile is made of 32x32 blocks.
MFMAOp = _MatrixCoreOp(MFMA, "MFMAOp")
WMMAOp = _MatrixCoreOp(MFMA, "WMMAOp")
MFMAComplexOp = _MatrixCoreOp(MFMA_COMPLEX, "MFMAComplexOp")      # src/operator.jl:251-314
WMMAComplexOp = _MatrixCoreOp(MFMA_COMPLEX, "WMMAComplexOp")
MFMADualOp = _MatrixCoreOp(MFMA_DUAL, "MFMADualOp")               # src/operator.jl:320-372
WMMADualOp = _MatrixCoreOp(MFMA_DUAL, "WMMADualOp")
FPUOp = _FPUOp(FPU, "FPUOp")                                      # src/operator.jl:35-153
TropicalFPUOp = _FPUOp(FPU_TROPICAL, "TropicalFPUOp")             # src/operator.jl:134-137


def shape(op: OperatorType) -> NT:
    """reference src/operator.jl:41, :165, :253, :322."""
    return NT(M=op.M, N=op.N, K=op.K)


def base_shape(op: OperatorType) -> NT:
    """reference src/operator.jl:42."""
    return NT(M=op.M, N=op.N, K=op.K, mb=op.mb, nb=op.nb, kb=op.kb)
