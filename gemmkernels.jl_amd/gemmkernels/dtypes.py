"""Element types, named as in the reference's Julia code."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class DType:
    name: str
    code: int        # gk_dtype of the C ABI
    size: int        # bytes
    is_complex: bool = False

    def __repr__(self):
        return self.name


Float16 = DType("Float16", 0, 2)
BFloat16 = DType("BFloat16", 1, 2)
Float32 = DType("Float32", 2, 4)
Float64 = DType("Float64", 3, 8)
Int16 = DType("Int16", 4, 2)
Int32 = DType("Int32", 5, 4)
Int64 = DType("Int64", 6, 8)
ComplexF16 = DType("Complex{Float16}", 0, 4, True)
ComplexF32 = DType("Complex{Float32}", 2, 8, True)

_RANK = {"Float16": 1, "BFloat16": 1, "Float32": 2, "Float64": 3}
_INT_RANK = {"Int16": 1, "Int32": 2, "Int64": 3}


def is_integer(t: DType) -> bool:
    return t.name in _INT_RANK


def promote_type(a: DType, b: DType) -> DType:
    """Julia's promote_type restricted to the types used here: the wider of two integers or of two
    floats, the float of a float and an integer."""
    if a == b:
        return a
    if {a.name, b.name} == {"Float16", "BFloat16"}:
        return Float32
    if is_integer(a) and is_integer(b):
        return a if _INT_RANK[a.name] >= _INT_RANK[b.name] else b
    if is_integer(a):
        return b
    if is_integer(b):
        return a
    return a if _RANK[a.name] >= _RANK[b.name] else b


def real_type(t: DType) -> DType:
    if t == ComplexF16:
        return Float16
    if t == ComplexF32:
        return Float32
    return t


def from_torch(dtype) -> DType:
    import torch
    table = {torch.float16: Float16, torch.bfloat16: BFloat16, torch.float32: Float32, torch.float64: Float64,
             torch.int16: Int16, torch.int32: Int32, torch.int64: Int64, torch.complex64: ComplexF32}
    if hasattr(torch, "complex32"):
        table[torch.complex32] = ComplexF16
    return table[dtype]


def to_torch(t: DType):
    import torch
    return {"Float16": torch.float16, "BFloat16": torch.bfloat16, "Float32": torch.float32, "Float64": torch.float64,
            "Int16": torch.int16, "Int32": torch.int32, "Int64": torch.int64,
            "Complex{Float32}": torch.complex64, "Complex{Float16}": torch.complex32}[t.name]
