"""CPU oracle for the tiled GEMM hot path -- TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the cpu_baseline leg of the benchmark may import this module;
the product package never does.  It binds ``libgk_oracle.so`` (the C restatement in
``gk_oracle.c``, which cites the reference lines it follows) and adds float64 numpy
references used to pin that restatement and to compute error norms.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libgk_oracle.so")

F16, BF16, F32, F64, I16, I32, I64 = 0, 1, 2, 3, 4, 5, 6
L_ZERO, L_COL, L_ROW, L_DIAG, L_ICOL, L_IROW, L_GETT = range(7)
OP_FMA, OP_TROPICAL, OP_COMPLEX, OP_DUAL = range(4)
T_IDENTITY, T_SCALE, T_ADD, T_RELU, T_NEG, T_ABS, T_CLAMP, T_SQUARE = range(8)
EPI_DEFAULT, EPI_BIAS_COL, EPI_BIAS_ROW = range(3)

# hook order of the reference launcher (src/matmul.jl:8-15)
HOOKS = ("global_to_shared_a", "global_to_shared_b", "global_to_shared_c", "shared_to_global_d",
         "shared_to_regs_a", "shared_to_regs_b", "shared_to_regs_c", "regs_to_shared_d")

_NP_OF = {F16: np.float16, BF16: np.uint16, F32: np.float32, F64: np.float64}


class _Op(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("p0", ctypes.c_float), ("p1", ctypes.c_float)]


class _Transform(ctypes.Structure):
    _fields_ = [("n", ctypes.c_int32), ("ops", _Op * 4)]


class _Layout(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("dtype", ctypes.c_int32), ("ld", ctypes.c_int64),
                ("nmodes", ctypes.c_int32 * 2), ("extent", (ctypes.c_int64 * 4) * 2),
                ("stride", (ctypes.c_int64 * 4) * 2)]


class _Problem(ctypes.Structure):
    _fields_ = [("M", ctypes.c_int64), ("N", ctypes.c_int64), ("K", ctypes.c_int64),
                ("a", _Layout), ("b", _Layout), ("c", _Layout), ("d", _Layout),
                ("shared_a_dtype", ctypes.c_int32), ("shared_b_dtype", ctypes.c_int32),
                ("shared_c_dtype", ctypes.c_int32), ("shared_d_dtype", ctypes.c_int32),
                ("compute_dtype", ctypes.c_int32), ("accum_dtype", ctypes.c_int32),
                ("op_kind", ctypes.c_int32), ("wide_accum", ctypes.c_int32),
                ("t", _Transform * 8), ("epilogue", ctypes.c_int32), ("bias", ctypes.c_void_p)]


def build(force: bool = False) -> str:
    """Compile the C restatement with the Makefile beside it (gcc, a second or two)."""
    src = os.path.join(_HERE, "gk_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libgk_oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.gko_matmul.argtypes = [ctypes.POINTER(_Problem), ctypes.c_void_p, ctypes.c_void_p,
                                    ctypes.c_void_p, ctypes.c_void_p]
        _lib.gko_matmul.restype = ctypes.c_int
        _lib.gko_double_to_half.argtypes = [ctypes.c_double]
        _lib.gko_double_to_half.restype = ctypes.c_uint16
        _lib.gko_half_to_float.argtypes = [ctypes.c_uint16]
        _lib.gko_half_to_float.restype = ctypes.c_float
        assert _lib.gko_struct_sizes(0) == ctypes.sizeof(_Problem)
        assert _lib.gko_struct_sizes(1) == ctypes.sizeof(_Layout)
        assert _lib.gko_struct_sizes(2) == ctypes.sizeof(_Transform)
    return _lib


def num_threads() -> int:
    return int(lib().gko_num_threads())


@dataclass
class Layout:
    """Where logical element (row, col) of an operand lives in memory."""
    kind: int
    dtype: int
    ld: int = 0
    row_modes: Sequence[Tuple[int, int]] = ()   # GETT: (extent, stride), fastest digit first
    col_modes: Sequence[Tuple[int, int]] = ()

    def to_c(self) -> _Layout:
        L = _Layout()
        L.kind, L.dtype, L.ld = self.kind, self.dtype, self.ld
        for which, modes in enumerate((self.row_modes, self.col_modes)):
            L.nmodes[which] = len(modes)
            for i, (e, s) in enumerate(modes):
                L.extent[which][i] = e
                L.stride[which][i] = s
        return L


@dataclass
class Problem:
    M: int
    N: int
    K: int
    a: Layout
    b: Layout
    c: Layout
    d: Layout
    compute_dtype: int = F16
    accum_dtype: int = F32
    shared_a_dtype: Optional[int] = None
    shared_b_dtype: Optional[int] = None
    shared_c_dtype: Optional[int] = None
    shared_d_dtype: Optional[int] = None
    op_kind: int = OP_FMA
    transforms: dict = field(default_factory=dict)   # hook name -> [(kind, p0, p1), ...]
    epilogue: int = EPI_DEFAULT
    bias: Optional[np.ndarray] = None


def _as_buffer(x: Optional[np.ndarray]):
    if x is None:
        return None
    assert x.flags.c_contiguous or x.flags.f_contiguous
    return x.ctypes.data_as(ctypes.c_void_p)


def matmul(p: Problem, a: Optional[np.ndarray], b: Optional[np.ndarray], c: Optional[np.ndarray],
           d: np.ndarray, wide_accum: bool = False) -> np.ndarray:
    """Run the C restatement; ``d`` is written in place (it may be the same array as ``c``)."""
    P = _Problem()
    P.M, P.N, P.K = p.M, p.N, p.K
    P.a, P.b, P.c, P.d = p.a.to_c(), p.b.to_c(), p.c.to_c(), p.d.to_c()
    P.shared_a_dtype = p.compute_dtype if p.shared_a_dtype is None else p.shared_a_dtype
    P.shared_b_dtype = p.compute_dtype if p.shared_b_dtype is None else p.shared_b_dtype
    P.shared_c_dtype = p.accum_dtype if p.shared_c_dtype is None else p.shared_c_dtype
    P.shared_d_dtype = p.accum_dtype if p.shared_d_dtype is None else p.shared_d_dtype
    P.compute_dtype, P.accum_dtype = p.compute_dtype, p.accum_dtype
    P.op_kind, P.wide_accum = p.op_kind, int(wide_accum)
    for i, hook in enumerate(HOOKS):
        ops = list(p.transforms.get(hook, ()))
        assert len(ops) <= 4
        P.t[i].n = len(ops)
        for j, op in enumerate(ops):
            kind, p0, p1 = (tuple(op) + (0.0, 0.0))[:3]
            P.t[i].ops[j].kind, P.t[i].ops[j].p0, P.t[i].ops[j].p1 = int(kind), float(p0), float(p1)
    P.epilogue = p.epilogue
    bias = None
    if p.bias is not None:
        bias = np.ascontiguousarray(p.bias, dtype=np.float32)
        P.bias = bias.ctypes.data
    rc = lib().gko_matmul(ctypes.byref(P), _as_buffer(a), _as_buffer(b), _as_buffer(c), _as_buffer(d))
    if rc != 0:
        raise RuntimeError(f"gko_matmul failed with status {rc}")
    return d


# ----------------------------------------------------------------------------------------
# float64 numpy references (used to pin the restatement and as the error-norm baseline)
# ----------------------------------------------------------------------------------------

def to_f64(x: np.ndarray, dtype: int) -> np.ndarray:
    if dtype == BF16:
        return (x.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    return x.astype(np.float64)


def gemm_f64(a: np.ndarray, b: np.ndarray, c: Optional[np.ndarray], alpha: float = 1.0,
             beta: float = 0.0, trans_a: bool = False, trans_b: bool = False) -> np.ndarray:
    """alpha * op(A) * op(B) + beta * C in float64 (the textbook GEMM that the reference's own
    tests compare against, configs/configs.jl:87-93)."""
    A = a.astype(np.float64)
    B = b.astype(np.float64)
    A = A.T if trans_a else A
    B = B.T if trans_b else B
    out = alpha * (A @ B)
    if c is not None and beta != 0.0:
        out = out + beta * c.astype(np.float64)
    return out


def gemm_blas_f32(a: np.ndarray, b: np.ndarray, c: Optional[np.ndarray], alpha: float = 1.0,
                  beta: float = 0.0, trans_a: bool = False, trans_b: bool = False) -> np.ndarray:
    """The reference CPU path: LinearAlgebra.mul! on Float32 host arrays is OpenBLAS sgemm, which
    is what numpy.matmul calls on float32 operands."""
    A = np.asarray(a, dtype=np.float32)
    B = np.asarray(b, dtype=np.float32)
    A = A.T if trans_a else A
    B = B.T if trans_b else B
    out = A @ B
    if alpha != 1.0:
        out *= np.float32(alpha)
    if c is not None and beta != 0.0:
        out += np.float32(beta) * c.astype(np.float32)
    return out


def rel_frobenius(x: np.ndarray, ref: np.ndarray) -> float:
    x = np.asarray(x, dtype=np.float64 if not np.iscomplexobj(x) else np.complex128)
    ref = np.asarray(ref, dtype=x.dtype)
    den = np.linalg.norm(ref.ravel())
    num = np.linalg.norm((x - ref).ravel())
    return float(num / den) if den > 0 else float(num)
