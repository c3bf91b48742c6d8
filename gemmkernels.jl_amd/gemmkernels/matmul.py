"""The launcher ``matmul`` and the BLAS-like ``matmatmul_`` / ``mul_`` (reference src/matmul.jl;
Julia's ``matmatmul!`` / ``mul!`` lose their ``!`` in Python).

Device arrays are torch CUDA tensors in COLUMN-MAJOR order like Julia's CuArrays: a logical
(rows, cols) matrix is a tensor with ``stride(0) == 1`` (see ``gemmkernels.colmajor``).  torch is
only the owner of the memory and of the stream; every flop runs in libgemmkernels_hip.so.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import numpy as np

from . import _lib
from . import cta_swizzle as CTASwizzle
from . import epilogue as Epilogue
from . import kernel as Kernel
from . import layout as Layout
from . import operator as Operator
from . import transform as Transform
from .config import Config, default_block_shape, get_config as _get_config
from .dtypes import BFloat16, DType, Float16, Float32, Float64, from_torch, promote_type
from .errors import ConfigError, DimensionMismatch
from .tiling import NT

_HOOKS = ("transform_global_to_shared_a", "transform_global_to_shared_b", "transform_global_to_shared_c",
          "transform_shared_to_global_d", "transform_shared_to_regs_a", "transform_shared_to_regs_b",
          "transform_shared_to_regs_c", "transform_regs_to_shared_d")


def _ptr(x) -> Optional[int]:
    if x is None:
        return None
    if isinstance(x, int):
        return x
    return int(x.data_ptr())


_NO_LD = (Layout.ZERO, Layout.DIAGONAL, Layout.GETT_KIND)
_INTERLEAVED = (Layout.INTERLEAVED_COL_MAJOR, Layout.INTERLEAVED_ROW_MAJOR)


_SPLIT = (Layout.SPLIT_COL_MAJOR, Layout.SPLIT_ROW_MAJOR)


def _leading_dim(x, layout) -> int:
    """Leading dimension, in elements, of a column-major device matrix."""
    kind = layout.kind
    if x is None or kind in _NO_LD or isinstance(x, int):
        return 0
    shape, stride = x.shape, x.stride()
    if kind in _INTERLEAVED:
        # interleaved complex data: a real tensor of logical shape (2, rows, cols), column-major,
        # or a complex tensor of shape (rows, cols); the leading dimension counts complex elements
        if x.is_complex():
            if len(shape) != 2 or (shape[0] > 1 and stride[0] != 1):
                raise ConfigError("complex operands must be column-major matrices")
            return int(stride[1]) if shape[1] > 1 else max(int(shape[0]), 1)
        if len(shape) != 3 or shape[0] != 2 or stride[0] != 1 or (shape[1] > 1 and stride[1] != 2):
            raise ConfigError("interleaved complex operands must have shape (2, rows, cols) in column-major order")
        return int(stride[2]) // 2 if shape[2] > 1 else max(int(shape[1]), 1)
    if kind in _SPLIT:
        # planar complex data: a real tensor of logical shape (rows, cols, 2), column-major, the
        # imaginary plane right behind the real one
        if len(shape) != 3 or shape[2] != 2 or (shape[0] > 1 and stride[0] != 1) or stride[2] != stride[1] * shape[1]:
            raise ConfigError("planar complex operands must have shape (rows, cols, 2) in column-major order")
        return int(stride[1])
    if len(shape) != 2:
        raise ConfigError("matrix operands must be 2-dimensional")
    if shape[0] > 1 and stride[0] != 1:
        raise ConfigError("matrix operands must be column-major (stride(0) == 1); see gemmkernels.colmajor")
    return int(stride[1]) if shape[1] > 1 else max(int(shape[0]), 1)


def _current_stream() -> int:
    """Raw handle of torch's current HIP stream."""
    import torch
    try:
        return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device())
    except AttributeError:
        return torch.cuda.current_stream().cuda_stream


_workspaces = {}


def split_k_workspace(conf_c, stream: int):
    """Device workspace for a K-split launch of ``conf_c`` on ``stream``: (pointer, bytes).  The slices of an
    output tile leave their partial tiles there and the last one to arrive adds them up in slice order
    (``gk_matmul_split_k``).  One zero-initialised buffer per device and stream, grown when a launch needs
    more: launches on one stream are ordered, so they can share it, and every launch leaves the arrival
    counters at its head at zero.  (0, 0) when the product runs unsplit."""
    import torch
    need = ctypes.c_size_t()
    rc = _lib.lib().gk_split_k_workspace_size(ctypes.byref(conf_c), ctypes.byref(need))
    if rc != _lib.GK_OK:
        _raise(rc)
    if need.value == 0:
        return 0, 0
    key = (torch.cuda.current_device(), int(stream))
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < need.value:
        size = max(need.value, 1 << 20)
        buf = _workspaces[key] = torch.zeros(size, dtype=torch.uint8, device="cuda")
    return int(buf.data_ptr()), int(buf.numel())


_IDENTITY = Transform.Elementwise()
_DEFAULT_EPILOGUE = Epilogue.Default()
_lowered = {}


def lower_transforms(transforms: dict) -> Optional[_lib.gk_transforms]:
    if all(t.is_identity for t in transforms.values()):
        return None
    if any(t.expr is not None for t in transforms.values()):
        raise ConfigError("expression transforms need a specialised kernel (gemmkernels.specialize)")
    key = tuple(transforms[name].ops for name in _HOOKS)
    hit = _lowered.get(key)
    if hit is not None:
        return hit
    out = _lowered[key] = _lib.gk_transforms()
    for i, name in enumerate(_HOOKS):
        ops = transforms[name].ops
        out.hook[i].n_ops = len(ops)
        for j, (kind, p0, p1) in enumerate(ops):
            out.hook[i].ops[j].kind, out.hook[i].ops[j].p0, out.hook[i].ops[j].p1 = kind, p0, p1
    return out


def _raise(rc: int):
    msg = _lib.last_error()
    if rc == _lib.GK_ERR_DIMENSION_MISMATCH:
        raise DimensionMismatch(msg)
    raise ConfigError(msg, rc)


class SpecializedKernel:
    """A kernel compiled at run time (hipRTC) for one configuration with its transform hooks inlined:
    arbitrary C expressions in x, and block shapes outside the table compiled into the library.  The
    counterpart of the reference's one-JIT-compiled-kernel-per-Config with inlined functors
    (src/matmul.jl:38, src/transform.jl:26-30).  The first construction for a given configuration and
    set of expressions compiles (seconds); later ones are served from the library's cache."""

    def __init__(self, conf: Config, transforms: dict):
        self.conf = conf
        exprs = (ctypes.c_char_p * 8)()
        self.expressions = []
        for i, name in enumerate(_HOOKS):
            t = transforms.get(name) or _IDENTITY
            e = t.c_expression()
            self.expressions.append(e)
            exprs[i] = e.encode() if e is not None else None
        handle = ctypes.c_void_p()
        cconf = conf.to_c()
        rc = _lib.lib().gk_rtc_compile(ctypes.byref(cconf), exprs, Kernel.matmul_pipelined.code, ctypes.byref(handle))
        if rc != _lib.GK_OK:
            _raise(rc)
        self._handle = handle
        buf = ctypes.create_string_buffer(200)
        _lib.lib().gk_rtc_kernel_name(handle, buf, len(buf))
        self.name = buf.value.decode()

    def plan(self, a, b, c, d, epilogue=None) -> "Plan":
        return Plan(self.conf, a, b, c, d, {}, _DEFAULT_EPILOGUE if epilogue is None else epilogue, Kernel.matmul_pipelined,
                    specialized=self)

    def __call__(self, a, b, c, d, epilogue=None, stream=None):
        return self.plan(a, b, c, d, epilogue)(stream)


def specialize(conf: Config, *,
               transform_global_to_shared_a=None, transform_global_to_shared_b=None,
               transform_global_to_shared_c=None, transform_shared_to_global_d=None,
               transform_shared_to_regs_a=None, transform_shared_to_regs_b=None,
               transform_shared_to_regs_c=None, transform_regs_to_shared_d=None) -> SpecializedKernel:
    """Compile (or fetch from the cache) the kernel of ``conf`` with these hooks inlined.  A hook is a
    ``Transform.Elementwise`` (op list or ``expr="..."``) or directly a C expression string in x."""
    given = dict(transform_global_to_shared_a=transform_global_to_shared_a, transform_global_to_shared_b=transform_global_to_shared_b,
                 transform_global_to_shared_c=transform_global_to_shared_c, transform_shared_to_global_d=transform_shared_to_global_d,
                 transform_shared_to_regs_a=transform_shared_to_regs_a, transform_shared_to_regs_b=transform_shared_to_regs_b,
                 transform_shared_to_regs_c=transform_shared_to_regs_c, transform_regs_to_shared_d=transform_regs_to_shared_d)
    return SpecializedKernel(conf, {k: (Transform.Elementwise(expr=v) if isinstance(v, str) else v) for k, v in given.items()})


class Plan:
    """One launch with everything but the stream lowered ahead of time: the descriptors of the
    configuration, the transforms and the epilogue, and the operand addresses.  Calling the plan is
    one call into the library (which still runs every launch-time check of reference
    src/matmul.jl:28-41).  The plan keeps its operands alive; they must not be resized or freed by
    other means while it is in use.  For loops that launch the same GEMM many times, where the
    microseconds a general ``matmul`` call spends on lowering would rival the kernel itself."""

    __slots__ = ("_fn", "_conf", "_trans", "_epi", "_args", "_keep", "_split_k", "d", "kernel_names")

    def __init__(self, conf: Config, a, b, c, d, transforms: dict, epilogue, kernel, specialized=None):
        if specialized is None and any(t.expr is not None for t in transforms.values()):
            specialized = SpecializedKernel(conf, transforms)       # expression hooks: a run-time compiled kernel
        cconf = conf.to_c(_leading_dim(a, conf.global_a_layout), _leading_dim(b, conf.global_b_layout),
                          _leading_dim(c, conf.global_c_layout), _leading_dim(d, conf.global_d_layout))
        self._conf = _lib.gk_config.from_buffer_copy(cconf)        # to_c hands out a cached, shared descriptor
        self._trans = None if specialized is not None else lower_transforms(transforms)
        self._epi = None
        self._split_k = False
        if epilogue.kind != Epilogue.DEFAULT:
            self._epi = _lib.gk_epilogue()
            self._epi.kind = epilogue.kind
            self._epi.bias = _ptr(epilogue.bias)
        epi_ref = ctypes.byref(self._epi) if self._epi is not None else None
        if specialized is not None:
            self._fn = _lib.lib().gk_rtc_matmul
            self._args = (specialized._handle, ctypes.byref(self._conf), _ptr(a), _ptr(b), _ptr(c), _ptr(d), epi_ref)
        elif kernel is Kernel.matmul_split_k:
            self._fn = _lib.lib().gk_matmul_split_k
            self._args = (ctypes.byref(self._conf), _ptr(a), _ptr(b), _ptr(c), _ptr(d),
                          ctypes.byref(self._trans) if self._trans is not None else None, epi_ref)
            self._split_k = True
        else:
            self._fn = _lib.lib().gk_matmul
            self._args = (ctypes.byref(self._conf), _ptr(a), _ptr(b), _ptr(c), _ptr(d),
                          ctypes.byref(self._trans) if self._trans is not None else None, epi_ref, kernel.code)
        self._keep = (a, b, c, d, epilogue, specialized)
        self.d = d
        self.kernel_names = ()      # filled in by the BLAS-level front end

    def __call__(self, stream=None):
        stream = _current_stream() if stream is None else int(stream)
        if self._split_k:
            rc = self._fn(*self._args, *split_k_workspace(self._conf, stream), stream)
            if rc != _lib.GK_OK:
                _raise(rc)
            return self.d
        rc = self._fn(*self._args, stream)
        if rc != _lib.GK_OK:
            _raise(rc)
        return self.d


def _collect(given: dict) -> dict:
    return {k: (_IDENTITY if v is None else v) for k, v in given.items()}


def plan(conf: Config, a, b, c, d, *,
         transform_global_to_shared_a=None, transform_global_to_shared_b=None,
         transform_global_to_shared_c=None, transform_shared_to_global_d=None,
         transform_shared_to_regs_a=None, transform_shared_to_regs_b=None,
         transform_shared_to_regs_c=None, transform_regs_to_shared_d=None,
         epilogue=None, kernel=Kernel.matmul_singlestage) -> Plan:
    """Same arguments as ``matmul``; returns a ``Plan`` whose call launches on the current stream."""
    from . import complex_planar
    if complex_planar.is_planar(conf) and not complex_planar.planes_adjacent(a, b, c, d):
        return complex_planar.PlanarComplexPlan(conf, a, b, c, d)
    transforms = _collect(dict(transform_global_to_shared_a=transform_global_to_shared_a,
                               transform_global_to_shared_b=transform_global_to_shared_b,
                               transform_global_to_shared_c=transform_global_to_shared_c,
                               transform_shared_to_global_d=transform_shared_to_global_d,
                               transform_shared_to_regs_a=transform_shared_to_regs_a,
                               transform_shared_to_regs_b=transform_shared_to_regs_b,
                               transform_shared_to_regs_c=transform_shared_to_regs_c,
                               transform_regs_to_shared_d=transform_regs_to_shared_d))
    return Plan(conf, a, b, c, d, transforms, _DEFAULT_EPILOGUE if epilogue is None else epilogue, kernel)


def matmul(conf: Config, a, b, c, d, *,
           transform_global_to_shared_a=None, transform_global_to_shared_b=None,
           transform_global_to_shared_c=None, transform_shared_to_global_d=None,
           transform_shared_to_regs_a=None, transform_shared_to_regs_b=None,
           transform_shared_to_regs_c=None, transform_regs_to_shared_d=None,
           epilogue=None, kernel=Kernel.matmul_singlestage, stream=None):
    """reference src/matmul.jl:7-44: launch geometry, checks (ConfigError) and the asynchronous
    launch on the current stream.  Same positional and keyword arguments as the reference."""
    from . import complex_planar
    if complex_planar.is_planar(conf) and not complex_planar.planes_adjacent(a, b, c, d):
        return complex_planar.PlanarComplexPlan(conf, a, b, c, d)(stream)
    ctrans = None
    if not (transform_global_to_shared_a is None and transform_global_to_shared_b is None and
            transform_global_to_shared_c is None and transform_shared_to_global_d is None and
            transform_shared_to_regs_a is None and transform_shared_to_regs_b is None and
            transform_shared_to_regs_c is None and transform_regs_to_shared_d is None):
        collected = _collect(dict(
            transform_global_to_shared_a=transform_global_to_shared_a, transform_global_to_shared_b=transform_global_to_shared_b,
            transform_global_to_shared_c=transform_global_to_shared_c, transform_shared_to_global_d=transform_shared_to_global_d,
            transform_shared_to_regs_a=transform_shared_to_regs_a, transform_shared_to_regs_b=transform_shared_to_regs_b,
            transform_shared_to_regs_c=transform_shared_to_regs_c, transform_regs_to_shared_d=transform_regs_to_shared_d))
        if any(t.expr is not None for t in collected.values()):
            return Plan(conf, a, b, c, d, collected, _DEFAULT_EPILOGUE if epilogue is None else epilogue, kernel)(stream)
        ctrans = lower_transforms(collected)

    cconf = conf.to_c(_leading_dim(a, conf.global_a_layout), _leading_dim(b, conf.global_b_layout),
                      _leading_dim(c, conf.global_c_layout), _leading_dim(d, conf.global_d_layout))
    cepi = None
    if epilogue is not None and epilogue.kind != Epilogue.DEFAULT:
        cepi = _lib.gk_epilogue()
        cepi.kind = epilogue.kind
        cepi.bias = _ptr(epilogue.bias)
    stream = _current_stream() if stream is None else int(stream)
    if kernel is Kernel.matmul_split_k:
        rc = _lib.lib().gk_matmul_split_k(ctypes.byref(cconf), _ptr(a), _ptr(b), _ptr(c), _ptr(d),
                                          ctypes.byref(ctrans) if ctrans is not None else None,
                                          ctypes.byref(cepi) if cepi is not None else None,
                                          *split_k_workspace(cconf, stream), stream)
    else:
        rc = _lib.lib().gk_matmul(ctypes.byref(cconf), _ptr(a), _ptr(b), _ptr(c), _ptr(d),
                                  ctypes.byref(ctrans) if ctrans is not None else None,
                                  ctypes.byref(cepi) if cepi is not None else None, kernel.code, stream)
    if rc != _lib.GK_OK:
        _raise(rc)
    return d


def kernel_name(conf: Config, kernel=Kernel.matmul_singlestage, transforms=None, epilogue=None) -> str:
    """Name of the compiled kernel instance a launch of ``conf`` runs (for logs and profiles)."""
    cconf = conf.to_c()
    buf = ctypes.create_string_buffer(256)
    ctrans = None
    if transforms:
        full = {k: transforms.get(k, Transform.Elementwise()) for k in _HOOKS}
        ctrans = lower_transforms(full)
    cepi = None
    if epilogue is not None and epilogue.kind != Epilogue.DEFAULT:
        cepi = _lib.gk_epilogue()
        cepi.kind = epilogue.kind
    rc = _lib.lib().gk_kernel_name(ctypes.byref(cconf), ctypes.byref(ctrans) if ctrans is not None else None,
                                   ctypes.byref(cepi) if cepi is not None else None, kernel.code, buf, len(buf))
    if rc != _lib.GK_OK:
        raise ConfigError(_lib.last_error(), rc)
    return buf.value.decode()


# ------------------------------------------------------------------------------------------------
# BLAS-like
# ------------------------------------------------------------------------------------------------

def _select_kernel(layout_a, layout_b):
    """reference src/matmul.jl:52-56: the pipelined kernel when both operands are aligned."""
    if layout_a.is_aligned and layout_b.is_aligned:
        return Kernel.matmul_pipelined
    return Kernel.matmul_singlestage


_configs = {}


def get_config(*args):
    """Memoised create_config (reference src/matmul.jl:58-65)."""
    val = _configs.get(args)
    if val is None:
        val = _configs[args] = create_config(*args)
    return val


def create_config(A: DType, sizeA, stridesA, transA: bool, B: DType, sizeB, stridesB, transB: bool,
                  C: DType, sizeC, stridesC, alpha: type, zeroAlpha: bool, beta: type, zeroBeta: bool, wmma=None):
    """reference src/matmul.jl:66-183, with the MI355X operator and block-shape choices."""
    m = sizeA[1 if transA else 0]
    k = sizeA[0 if transA else 1]
    n = sizeB[0 if transB else 1]
    if m != sizeC[0] or n != sizeC[1] or k != sizeB[1 if transB else 0]:
        raise DimensionMismatch("Dimensions do not match")

    a_layout_base = Layout.RowMajor if transA else Layout.ColMajor
    b_layout_base = Layout.RowMajor if transB else Layout.ColMajor
    a_aligned_layout_base = Layout.UnsafeAlignedRowMajor if transA else Layout.UnsafeAlignedColMajor
    b_aligned_layout_base = Layout.UnsafeAlignedRowMajor if transB else Layout.UnsafeAlignedColMajor

    # operator: the matrix cores for 16-bit inputs with fp32 accumulation (src/matmul.jl:85-91)
    mfma_types = [(Float16, Float16, Float32), (BFloat16, BFloat16, Float32), (Float16, Float16, Float16)]
    compute_type = promote_type(A, B)
    use_mfma = ((compute_type, compute_type, C) in mfma_types) if wmma is None else bool(wmma)

    shared_a_layout = Layout.Padded[a_aligned_layout_base[compute_type if use_mfma else A], 8]
    shared_b_layout = Layout.Padded[b_aligned_layout_base[compute_type if use_mfma else B], 8]
    shared_c_layout = Layout.Zero[C] if zeroBeta else Layout.UnsafeAlignedColMajor[C]
    shared_d_layout = Layout.UnsafeAlignedColMajor[C]

    if use_mfma:
        operator = Operator.MFMAOp[32, 32, 16, compute_type, Float32 if C == Float16 else C]
    else:
        operator = Operator.FPUOp[8, 8, 1, 8, 8, 1, compute_type, C]
    a_aligned = (stridesA[1] * A.size) % 16 == 0
    b_aligned = (stridesB[1] * B.size) % 16 == 0
    c_aligned = (stridesC[1] * C.size) % 16 == 0

    def layouts_for(block_shape):
        # src/matmul.jl:121-156: vector loads and stores need 16-byte aligned columns and whole tiles
        if zeroAlpha:
            ga, gb = Layout.Zero[A], Layout.Zero[B]
        else:
            ga = (a_aligned_layout_base[A] if a_aligned and m % block_shape.M == 0 and k % block_shape.K == 0
                  else a_layout_base[A])
            gb = (b_aligned_layout_base[B] if b_aligned and k % block_shape.K == 0 and n % block_shape.N == 0
                  else b_layout_base[B])
        cd_aligned = c_aligned and m % block_shape.M == 0 and n % block_shape.N == 0
        gc = Layout.Zero[C] if zeroBeta else (Layout.UnsafeAlignedColMajor[C] if cd_aligned else Layout.ColMajor[C])
        gd = Layout.UnsafeAlignedColMajor[C] if cd_aligned else Layout.ColMajor[C]
        return ga, gb, gc, gd

    # The library runs a product on bounds-checked layouts on the aligned kernels all the same (tiles over the
    # edge clamp their loads and mask their stores, a partial last K tile is zeroed beyond K) when the columns
    # of A and B are 16-byte aligned, K is a multiple of 8 and M (N) is a multiple of 8 where it is the
    # contiguous index of A (B).  Then the tile is chosen among all tiles, not only those that divide the
    # sizes (4096 x 4096 x 4000: the 64-deep tile with a partial last step instead of the 32-deep one), and
    # the operands it does not divide get the bounds-checked layouts, as the reference's rule says.
    edge_ok = (use_mfma and a_aligned and b_aligned and k % 8 == 0 and (transA or m % 8 == 0) and (not transB or n % 8 == 0)
               and not zeroAlpha)
    block_shape = default_block_shape(operator, NT(M=m, N=n, K=k), tile_sized=not edge_ok, a_kmajor=transA, b_kmajor=not transB)
    global_a_layout, global_b_layout, global_c_layout, global_d_layout = layouts_for(block_shape)
    if not edge_ok and any(l.kind in (Layout.COL_MAJOR, Layout.ROW_MAJOR) for l in (global_a_layout, global_b_layout, global_c_layout, global_d_layout)):
        # some operand needs bounds checks: the bounds-checked kernels have one tile shape
        block_shape = NT(M=64, N=64, K=32)
        global_a_layout, global_b_layout, global_c_layout, global_d_layout = layouts_for(block_shape)

    conf = _get_config(gemm_shape=NT(M=m, N=n, K=k), block_shape=block_shape, operator=operator,
                       global_a_layout=global_a_layout, global_b_layout=global_b_layout,
                       global_c_layout=global_c_layout, global_d_layout=global_d_layout,
                       shared_a_layout=shared_a_layout, shared_b_layout=shared_b_layout,
                       shared_c_layout=shared_c_layout, shared_d_layout=shared_d_layout,
                       is_a_col_major=not transA, is_b_col_major=not transB)
    return conf, compute_type, _select_kernel(global_a_layout, global_b_layout)


def _round_to(dtype: DType, x: float) -> float:
    if dtype == Float16:
        return float(np.float16(x))
    if dtype == BFloat16:
        import torch
        return float(torch.tensor(x, dtype=torch.bfloat16))
    if dtype == Float32:
        return float(np.float32(x))
    return float(x)


def _single_plan(C, tA: bool, tB: bool, A, B, alpha, beta, wmma=None) -> Plan:
    """One launch for C = alpha * op(A) * op(B) + beta * C: the configuration ``create_config`` picks."""
    conf, compute_type, kernel = get_config(
        from_torch(A.dtype), tuple(A.shape), tuple(A.stride()), tA,
        from_torch(B.dtype), tuple(B.shape), tuple(B.stride()), tB,
        from_torch(C.dtype), tuple(C.shape), tuple(C.stride()),
        type(alpha), alpha == 0, type(beta), beta == 0, wmma)
    alpha_c = _round_to(compute_type, float(alpha))          # convert(compute_type, alpha), :196
    beta_c = _round_to(from_torch(C.dtype), float(beta))     # convert(eltype(C), beta), :197
    for name, value in (("alpha", alpha_c), ("beta", beta_c)):
        if float(np.float32(value)) != value:
            # transform parameters travel as binary32; Float64 (or large integer) factors that do not
            # fit would silently change the result
            raise ConfigError(f"{name} = {value!r} is not representable in binary32, the parameter type of the transform hooks")
    # beta = 0 has already turned C into a Zero layout: nothing is loaded, nothing to scale
    ta = Transform.Elementwise(ops=[] if alpha_c == 1.0 else [(Transform.SCALE, alpha_c, 0.0)])
    tc = Transform.Elementwise(ops=[] if beta_c == 1.0 or beta == 0 else [(Transform.SCALE, beta_c, 0.0)])
    if conf.operator.kind == Operator.MFMA and from_torch(C.dtype) == Float32:
        # few output tiles and a long K loop (skinny products, the rims of a cut-up product): cut K into
        # slices so that every CU gets work
        bs, ms = conf.block_shape, conf.matmul_shape
        tiles = -(-ms.M // bs.M) * -(-ms.N // bs.N)
        if kernel is Kernel.matmul_pipelined and tiles <= 128 and ms.K // bs.K >= 4:
            kernel = Kernel.matmul_split_k
        elif kernel is Kernel.matmul_singlestage and tiles <= 128 and ms.K // bs.K >= 16:
            kernel = Kernel.matmul_split_k          # the bounds-checked kernel: slices of at least eight K tiles
    p = plan(conf, A, B, C, C, transform_shared_to_regs_a=ta, transform_shared_to_regs_c=tc, kernel=kernel)
    p.kernel_names = (kernel_name(conf, kernel, dict(transform_shared_to_regs_a=ta, transform_shared_to_regs_c=tc)),)
    return p


class PlanSequence:
    """Several launches on one stream that together compute one product (``matmatmul_plan`` for sizes
    that are not whole tiles).  Called like a ``Plan``."""

    def __init__(self, plans, d):
        self.plans = list(plans)
        self.d = d
        self.kernel_names = tuple(n for p in self.plans for n in p.kernel_names)

    def __call__(self, stream=None):
        for p in self.plans:
            p(stream)
        return self.d


_REGION_TILES = (256, 128, 64)


def overlapping_regions(M: int, N: int):
    """For a product that does not read C (beta = 0): whole tiles only.  The part of the output whose
    sizes are multiples of 64 is cut like ``output_regions``; the ragged right and bottom edges are covered
    by 64-wide windows that end at the edge and reach back over cells another launch has already written
    (which then get the same value, up to the order of the sums, a second time).  M, N >= 64."""
    M64, N64 = M // 64 * 64, N // 64 * 64
    out = output_regions(M64, N64)
    if N > N64:
        out.append((0, M64, N - 64, 64, True))
    if M > M64:
        out.append((M - 64, 64, 0, N64, True))
    if N > N64 and M > M64:
        out.append((M - 64, 64, N - 64, 64, True))
    return out


def output_regions(M: int, N: int):
    """Cuts an M x N output into disjoint rectangles ``(m0, m, n0, n, whole_tiles)``.  The first is the
    largest top-left block made of 256 x 256 tiles; the strip to its right (all rows) and the strip below
    it are cut the same way with 128 and then 64; what is left over, or narrower than 64, is marked
    ``whole_tiles = False`` and goes to the bounds-checked kernel.  Offsets of rectangles with whole tiles
    are multiples of 64 elements, so 16-byte aligned columns stay 16-byte aligned."""
    out = []

    def cut(m0, m, n0, n, level):
        if m <= 0 or n <= 0:
            return
        while level < len(_REGION_TILES) and (m < _REGION_TILES[level] or n < _REGION_TILES[level]):
            level += 1
        if level == len(_REGION_TILES):
            out.append((m0, m, n0, n, False))
            return
        t = _REGION_TILES[level]
        mi, ni = m // t * t, n // t * t
        out.append((m0, mi, n0, ni, True))
        cut(m0, m, n0 + ni, n - ni, level + 1)       # right of the block: every row
        cut(m0 + mi, m - mi, n0, ni, level + 1)      # below the block
    cut(0, M, 0, N, 0)
    return out


def _estimate_us(operator, M: int, N: int, K: int, whole_tiles: bool) -> float:
    """Rough duration of one launch, from two measured rates: a CU multiplies a 256 x 256 x 64 tile over
    K = 4096 in 108 us (other tiles by ``config._MFMA_TILE_RATE``), and the bounds-checked kernel spends
    0.53 us per CU on a 64 x 64 x 32 step; a launch costs a few microseconds whatever it does, a K-split
    rim two launches and the atomic adds."""
    from .config import _MFMA_TILE_RATE, NUM_CUS, default_block_shape
    if whole_tiles:
        bs = default_block_shape(operator, NT(M=M, N=N, K=K))
        tiles = -(-M // bs.M) * -(-N // bs.N)
        rate = _MFMA_TILE_RATE.get((bs.M, bs.N, bs.K), 0.5)
        rate = rate[0 if tiles <= NUM_CUS else 1] if isinstance(rate, tuple) else rate
        per_cu = -(-tiles // NUM_CUS) * bs.M * bs.N / rate
        return per_cu * K / (65536.0 * 4096.0) * 108.0 + 6.0
    steps = -(-M // 64) * -(-N // 64) * -(-K // 32)
    return max(-(-steps // NUM_CUS), 8) * 0.53 + 25.0


def matmatmul_plan(C, transA: str, transB: str, A, B, alpha, beta, *, wmma=None, regions=None):
    """The launches ``matmatmul_`` would make, as a ``Plan`` (or a ``PlanSequence``) to call any number of
    times.

    Sizes that are whole tiles, and everything the matrix cores do not run, take one launch of the
    configuration ``create_config`` picks (reference src/matmul.jl:185-204).  A large 16-bit product whose
    sizes are *not* whole tiles would run entirely on the bounds-checked kernel, at a tenth of the speed
    (the reference has the same cliff, src/matmul.jl:121-156 and src/layout.jl:117-184).  When the columns
    of A, B and C are 16-byte aligned it is cut up instead: ``output_regions`` of whole tiles run on the
    fast kernels over the first K - K % 32 values of k, the ragged rims on the bounds-checked kernel (in
    slices of K: a rim has few tiles), and one more bounds-checked launch adds the last K % 32 values of k
    to all of C.  With beta = 0 and M, N multiples of 8 there are no rims: ``overlapping_regions`` covers the
    edges with whole tiles that reach back over finished cells.

    Since the aligned kernels handle tiles that stick out over M, N or K themselves (K a multiple of 8, and
    M, or N, where it is the contiguous index of A, or B), such products take one launch and the cutting
    above is what remains for the others: aligned leading dimensions around an M or N that is not a multiple
    of 8, as sub-matrices have them.  Every element of C is
    still computed as alpha * op(A) * op(B) + beta * C with alpha applied to A in the compute type; only
    the order of the fp32 additions along k differs from the single launch.  ``regions`` forces the
    cutting on (True) or off (False); by default it is used when a rough estimate (``_estimate_us``) puts
    the launches together clearly below the single one (from about 3000^3 on)."""
    tA, tB = transA == 'T', transB == 'T'
    single = _single_plan(C, tA, tB, A, B, alpha, beta, wmma)
    conf = get_config(from_torch(A.dtype), tuple(A.shape), tuple(A.stride()), tA,
                      from_torch(B.dtype), tuple(B.shape), tuple(B.stride()), tB,
                      from_torch(C.dtype), tuple(C.shape), tuple(C.stride()),
                      type(alpha), alpha == 0, type(beta), beta == 0, wmma)[0]
    ms = conf.matmul_shape
    M, N, K = ms.M, ms.N, ms.K
    checked = any(l.kind in (Layout.COL_MAJOR, Layout.ROW_MAJOR)
                  for l in (conf.global_a_layout, conf.global_b_layout, conf.global_c_layout, conf.global_d_layout))
    aligned_columns = all((int(x.stride()[1]) * x.element_size()) % 16 == 0 and x.data_ptr() % 16 == 0 for x in (A, B, C))
    Kw = K // 32 * 32        # every tile table has tiles 32 deep
    if (regions is None and checked and conf.operator.kind == Operator.MFMA and aligned_columns and alpha != 0
            and K % 8 == 0 and (tA or M % 8 == 0) and (not tB or N % 8 == 0)):
        # the aligned kernels take ragged M, N and K themselves (create_config has picked their tile)
        return single
    if (regions is False or conf.operator.kind != Operator.MFMA or not aligned_columns or alpha == 0
            or Kw == 0 or min(M, N) < _REGION_TILES[-1]):
        return single
    # windows that overlap need rows M - 64 and columns N - 64 to start on 16-byte boundaries in A, B and C
    if beta == 0 and M % 8 == 0 and N % 8 == 0:
        cut = overlapping_regions(M, N)
    else:
        cut = output_regions(M, N)
    if len(cut) == 1 and Kw == K:
        return single           # whole tiles already
    if regions is None:
        # worth it when the launches together are clearly shorter than the one launch
        together = sum(_estimate_us(conf.operator, m, n, Kw, whole) for _, m, _, n, whole in cut)
        together += _estimate_us(conf.operator, M, N, K - Kw, False) if Kw < K else 0.0
        if together > 0.8 * _estimate_us(conf.operator, M, N, K, not checked):
            return single

    def sub(X, trans, r0, r, c0, c):          # rows r0.., columns c0.. of op(X)
        return X[c0:c0 + c, r0:r0 + r] if trans else X[r0:r0 + r, c0:c0 + c]
    plans = []
    for m0, m, n0, n, _ in cut:
        plans.append(_single_plan(C[m0:m0 + m, n0:n0 + n], tA, tB, sub(A, tA, m0, m, 0, Kw), sub(B, tB, 0, Kw, n0, n),
                                  alpha, beta, wmma))
    if Kw < K:
        plans.append(_single_plan(C, tA, tB, sub(A, tA, 0, M, Kw, K - Kw), sub(B, tB, Kw, K - Kw, 0, N), alpha, 1.0, wmma))
    return PlanSequence(plans, C)


def matmatmul_(C, transA: str, transB: str, A, B, alpha, beta, *, wmma=None):
    """``matmatmul!`` (reference src/matmul.jl:185-204): C = alpha * op(A) * op(B) + beta * C."""
    matmatmul_plan(C, transA, transB, A, B, alpha, beta, wmma=wmma)()
    return C


class Transpose:
    """Lazy transpose wrapper, Julia's ``transpose(A)`` / ``A'`` (no conjugation, src/matmul.jl:211-213)."""

    def __init__(self, parent):
        self.parent = parent


Adjoint = Transpose


def mul_(C, A, B, alpha=True, beta=False):
    """``mul!`` (reference src/matmul.jl:207-215): unwraps Transpose/Adjoint and forwards."""
    tA, tB = isinstance(A, Transpose), isinstance(B, Transpose)
    return matmatmul_(C, 'T' if tA else 'N', 'T' if tB else 'N', A.parent if tA else A, B.parent if tB else B,
                      float(alpha), float(beta))
