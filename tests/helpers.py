"""Glue between the product API and the CPU oracle, used by the parity tests."""
from __future__ import annotations

import numpy as np

import gemmkernels as gk
from gemmkernels import Layout, Operator, Epilogue, Transform
from oracle import oracle

_DT = {"Float16": oracle.F16, "BFloat16": oracle.BF16, "Float32": oracle.F32, "Float64": oracle.F64,
       "Int16": oracle.I16, "Int32": oracle.I32, "Int64": oracle.I64}
HOOK_KW = {"transform_global_to_shared_a": "global_to_shared_a", "transform_global_to_shared_b": "global_to_shared_b",
           "transform_global_to_shared_c": "global_to_shared_c", "transform_shared_to_global_d": "shared_to_global_d",
           "transform_shared_to_regs_a": "shared_to_regs_a", "transform_shared_to_regs_b": "shared_to_regs_b",
           "transform_shared_to_regs_c": "shared_to_regs_c", "transform_regs_to_shared_d": "regs_to_shared_d"}


def _olayout(l, ld, role, gett=None):
    dt = _DT[l.T.name]
    k = l.kind
    if k == Layout.ZERO:
        return oracle.Layout(oracle.L_ZERO, dt)
    if k in (Layout.COL_MAJOR, Layout.ALIGNED_COL_MAJOR):
        return oracle.Layout(oracle.L_COL, dt, ld)
    if k in (Layout.ROW_MAJOR, Layout.ALIGNED_ROW_MAJOR):
        return oracle.Layout(oracle.L_ROW, dt, ld)
    if k == Layout.DIAGONAL:
        return oracle.Layout(oracle.L_DIAG, dt)
    if k == Layout.INTERLEAVED_COL_MAJOR:
        return oracle.Layout(oracle.L_ICOL, dt, ld)
    if k == Layout.INTERLEAVED_ROW_MAJOR:
        return oracle.Layout(oracle.L_IROW, dt, ld)
    if k == Layout.GETT_KIND:
        g = l.gett
        if role == "a":
            return oracle.Layout(oracle.L_GETT, dt, 0, [(e, s0) for e, s0, _ in g.m], [(e, s0) for e, s0, _ in g.k])
        if role == "b":
            return oracle.Layout(oracle.L_GETT, dt, 0, [(e, s1) for e, _, s1 in g.k], [(e, s0) for e, s0, _ in g.n])
        return oracle.Layout(oracle.L_GETT, dt, 0, [(e, s1) for e, _, s1 in g.m], [(e, s1) for e, _, s1 in g.n])
    raise ValueError(k)


def oracle_problem(conf, lds, transforms=None, epilogue=None, bias=None):
    """Translate a product Config (+ leading dimensions lda, ldb, ldc, ldd) into an oracle Problem."""
    lda, ldb, ldc, ldd = lds
    op = conf.operator
    kind = {Operator.MFMA: oracle.OP_FMA, Operator.FPU: oracle.OP_FMA, Operator.FPU_TROPICAL: oracle.OP_TROPICAL,
            Operator.MFMA_COMPLEX: oracle.OP_COMPLEX, Operator.MFMA_DUAL: oracle.OP_DUAL}[op.kind]
    p = oracle.Problem(
        M=conf.matmul_shape.M, N=conf.matmul_shape.N, K=conf.matmul_shape.K,
        a=_olayout(conf.global_a_layout, lda, "a"), b=_olayout(conf.global_b_layout, ldb, "b"),
        c=_olayout(conf.global_c_layout, ldc, "c"), d=_olayout(conf.global_d_layout, ldd, "d"),
        compute_dtype=_DT[op.CT.name], accum_dtype=_DT[op.AT.name], op_kind=kind)
    p.shared_a_dtype = _DT[conf.shared_a_layout.T.name]
    p.shared_b_dtype = _DT[conf.shared_b_layout.T.name]
    if transforms:
        p.transforms = {HOOK_KW[k]: list(v.ops) for k, v in transforms.items() if v is not None}
    if epilogue is not None and epilogue.kind != Epilogue.DEFAULT:
        p.epilogue = oracle.EPI_BIAS_COL if epilogue.kind == Epilogue.BIAS else oracle.EPI_BIAS_ROW
        p.bias = bias
    return p


def fortran(x: np.ndarray) -> np.ndarray:
    return np.asfortranarray(x)


def run_oracle(conf, a, b, c, d_shape, d_dtype=np.float32, transforms=None, epilogue=None, bias=None, wide=False):
    """a, b, c: Fortran-ordered numpy arrays (or None).  Returns D as a Fortran-ordered array."""
    def ld(x):
        return 0 if x is None or x.ndim != 2 else x.shape[0]
    d = np.zeros(d_shape, dtype=d_dtype, order="F")
    p = oracle_problem(conf, (ld(a), ld(b), ld(c), d.shape[0]), transforms, epilogue, bias)
    oracle.matmul(p, a, b, c, d, wide_accum=wide)
    return d


def run_gpu(conf, a, b, c, d_shape, d_dtype=None, transforms=None, epilogue_cls=None, bias=None, kernel=None,
            alias_cd=False):
    """Same inputs through the product: gemmkernels.matmul -> C ABI -> HIP kernel."""
    import torch
    from gemmkernels import Kernel
    def up(x, layout):     # uint16 arrays are bfloat16 bit patterns
        if x is None:
            return None
        return gk.colmajor(x, torch.bfloat16 if (x.dtype == np.uint16 and layout.T.name == "BFloat16") else None)
    ta, tb, tc = up(a, conf.global_a_layout), up(b, conf.global_b_layout), up(c, conf.global_c_layout)
    td = tc if alias_cd else gk.colmajor_empty(d_shape, d_dtype or torch.float32)
    if not alias_cd:
        td.fill_(float("nan") if td.is_floating_point() else -12345)    # poison: every element must be written
    epi = None
    keep = None
    if epilogue_cls is not None:
        keep = torch.from_numpy(np.ascontiguousarray(bias, dtype=np.float32)).cuda()
        epi = epilogue_cls(keep)
    gk.matmul(conf, ta, tb, tc, td, epilogue=epi, kernel=kernel or Kernel.matmul_singlestage, **(transforms or {}))
    torch.cuda.synchronize()
    return gk.to_numpy(td)
