"""Complex GEMM on planar (split re / im) global arrays.

The reference keeps complex matrices interleaved in global memory and planar only in shared memory
(``Layout.SplitColMajor``, src/layout.jl:340-411; configs/configs.jl:393-401).  When the *global*
arrays are planar already -- a real array of logical shape (rows, cols, 2), column-major, plane 0 the
real part -- a complex product is four real products on whole planes,

    D_re = A_re B_re - A_im B_im + C_re          D_im = A_re B_im + A_im B_re + C_im

(the sign pattern of WMMAComplexOp.mma, src/operator.jl:307-311).  When the two planes of every
operand are adjacent in memory (the array is contiguous in its third dimension) the library runs the
whole product as ONE launch of a kernel that walks K twice (``gemmkernels.matmul`` goes there
directly).  This module is the path for operands whose planes lie apart: each of the four products is
an ordinary aligned FP16 x FP16 -> FP32 GEMM, the minus sign rides on the A-side transform hook as an
exact FP16 scale by -1, and with 'N' B the two products that share an A plane run as one GEMM of
width 2N when B, C and D happen to have adjacent planes, so a product is three or four launches.
"""
from __future__ import annotations

from . import kernel as Kernel
from . import layout as Layout
from . import operator as Operator
from . import transform as Transform
from .config import get_config
from .dtypes import Float16, Float32
from .errors import ConfigError
from .tiling import NT

_NEGATE = Transform.Elementwise(ops=[(Transform.SCALE, -1.0, 0.0)])


def is_planar(conf) -> bool:
    return conf.global_a_layout.kind in (Layout.SPLIT_COL_MAJOR, Layout.SPLIT_ROW_MAJOR)


def planes_adjacent(*operands) -> bool:
    """True when every operand is a (rows, cols, 2) tensor whose imaginary plane starts where the real
    plane ends: what the single-launch kernel of the library addresses."""
    for x in operands:
        if x is None:
            continue
        if x.dim() != 3 or x.size(2) != 2 or x.stride(2) != x.stride(1) * x.size(1):
            return False
    return True


def _plane(x, i):
    """Plane i of a planar tensor of logical shape (rows, cols, 2): a column-major matrix view."""
    if x is None:
        return None
    if x.dim() != 3 or x.size(2) != 2 or (x.size(0) > 1 and x.stride(0) != 1):
        raise ConfigError("planar complex operands must have shape (rows, cols, 2) in column-major order")
    return x[:, :, i]


def _real_config(M, N, K, ta, tb, zero_c, ab=Float16, cd=Float32, **kw):
    col, row = Layout.UnsafeAlignedColMajor, Layout.UnsafeAlignedRowMajor
    return get_config(gemm_shape=NT(M=M, N=N, K=K), operator=Operator.MFMAOp[32, 32, 16, ab, Float32],
                      global_a_layout=(row if ta else col)[ab], global_b_layout=(row if tb else col)[ab],
                      global_c_layout=Layout.Zero[cd] if zero_c else col[cd], global_d_layout=col[cd],
                      is_a_col_major=not ta, is_b_col_major=not tb, **kw)


class PlanarComplexPlan:
    """The launches of one complex product on planar operands; calling it enqueues them in order on
    the current stream.  ``d`` may be ``c`` (every plane of C is read by the launch that first writes
    the same plane of D)."""

    def __init__(self, conf, a, b, c, d):
        from .matmul import Plan, _DEFAULT_EPILOGUE, _IDENTITY
        if conf.operator.kind != Operator.MFMA_COMPLEX:
            raise ConfigError("planar global layouts are offered for the complex operator")
        M, N, K = conf.matmul_shape.M, conf.matmul_shape.N, conf.matmul_shape.K
        ta = conf.global_a_layout.kind == Layout.SPLIT_ROW_MAJOR
        tb = conf.global_b_layout.kind == Layout.SPLIT_ROW_MAJOR
        zero_c = conf.global_c_layout.kind == Layout.ZERO or c is None
        a_re, a_im, b_re, b_im = _plane(a, 0), _plane(a, 1), _plane(b, 0), _plane(b, 1)
        c_re, c_im, d_re, d_im = _plane(c, 0), _plane(c, 1), _plane(d, 0), _plane(d, 1)
        pipelined = Kernel.matmul_pipelined
        ident = {}
        neg = {"transform_shared_to_regs_a": _NEGATE}

        def launch(cfg, A, B, C, D, hooks):
            full = {k: hooks.get(k, _IDENTITY) for k in ("transform_global_to_shared_a", "transform_global_to_shared_b",
                                                         "transform_global_to_shared_c", "transform_shared_to_global_d",
                                                         "transform_shared_to_regs_a", "transform_shared_to_regs_b",
                                                         "transform_shared_to_regs_c", "transform_regs_to_shared_d")}
            return Plan(cfg, A, B, C, D, full, _DEFAULT_EPILOGUE, pipelined)

        self.steps = []

        def side_by_side(x):
            """[plane 0 | plane 1] as one column-major matrix of twice the width, when the planes are adjacent."""
            import torch
            if x is None or x.stride(2) != x.stride(1) * x.size(1):
                return None
            return torch.as_strided(x, (x.size(0), 2 * x.size(1)), (1, x.stride(1)), x.storage_offset())

        b_wide = None if tb else side_by_side(b)
        d_wide = side_by_side(d)
        c_wide = None if zero_c else (d_wide if c is d else side_by_side(c))
        if b_wide is not None and d_wide is not None and (zero_c or c_wide is not None):
            # 'N' B: planar B is the (K, 2N) matrix [B_re | B_im], planar C / D are (M, 2N)
            cfg2 = _real_config(M, 2 * N, K, ta, False, zero_c)
            acc = _real_config(M, N, K, ta, False, False)
            self.steps.append(launch(cfg2, a_re, b_wide, c_wide, d_wide, ident))        # [D_re | D_im] = A_re [B_re | B_im] + C
            self.steps.append(launch(acc, a_im, b_im, d_re, d_re, neg))                 # D_re -= A_im B_im
            self.steps.append(launch(acc, a_im, b_re, d_im, d_im, ident))               # D_im += A_im B_re
        else:
            first = _real_config(M, N, K, ta, tb, zero_c)
            acc = _real_config(M, N, K, ta, tb, False)
            self.steps.append(launch(first, a_re, b_re, c_re, d_re, ident))
            self.steps.append(launch(acc, a_im, b_im, d_re, d_re, neg))
            self.steps.append(launch(first, a_re, b_im, c_im, d_im, ident))
            self.steps.append(launch(acc, a_im, b_re, d_im, d_im, ident))
        self._keep = (a, b, c, d)
        self.d = d

    def __call__(self, stream=None):
        for step in self.steps:
            step(stream)
        return self.d
