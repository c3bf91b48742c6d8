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
                  C: DType, sizeC, stridesC, alpha: type, zeroAlpha: bool, beta: type, zeroBeta: bool, wmma=None,
                  aligned_pointers=(True, True, True)):
    """reference src/matmul.jl:66-183, with the MI355X operator and block-shape choices.  ``aligned_pointers``
    says whether A, B and C start on 16-byte boundaries: the reference decides on the aligned layouts from the
    strides alone (a misaligned view then traps on the device, src/layout.jl:22-25); here such an operand gets
    the bounds-checked layout, which takes any address."""
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
    a_aligned = (stridesA[1] * A.size) % 16 == 0 and aligned_pointers[0]
    b_aligned = (stridesB[1] * B.size) % 16 == 0 and aligned_pointers[1]
    c_aligned = (stridesC[1] * C.size) % 16 == 0 and aligned_pointers[2]

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

    # The library runs a 16-bit product on bounds-checked layouts on the aligned kernels all the same (any address
    # and leading dimension; tiles over the edge clamp their loads and mask their stores; the last K tile is
    # repaired in LDS when a 16-byte chunk reaches over the end of an operand) as long as A and B hold one whole
    # chunk of 8 elements along their contiguous index.  Then the tile is chosen among all tiles, not only those
    # that divide the sizes (4096 x 4096 x 4000: the 64-deep tile with a partial last step instead of the 32-deep
    # one), and the operands it does not divide get the bounds-checked layouts, as the reference's rule says.
    edge_ok = use_mfma and not zeroAlpha and (k if transA else m) >= 8 and (n if transB else k) >= 8
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
        type(alpha), alpha == 0, type(beta), beta == 0, wmma, tuple(x.data_ptr() % 16 == 0 for x in (A, B, C)))
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
    if conf.operator.kind == Operator.MFMA:
        # few output tiles and a long K loop (skinny products, the rims of a cut-up product): the K-split kind
        # cuts K into slices so that every CU gets work (the library decides how many, and runs the product
        # unsplit when slices would be shorter than 1024 or the tile has no K-split instance).  Its sum is
        # ordered, so the result is the same on every run, like the reference's mul!.
        bs, ms = conf.block_shape, conf.matmul_shape
        tiles = -(-ms.M // bs.M) * -(-ms.N // bs.N)
        if tiles <= 256 and ms.K >= 2048:
            kernel = Kernel.matmul_split_k
    p = plan(conf, A, B, C, C, transform_shared_to_regs_a=ta, transform_shared_to_regs_c=tc, kernel=kernel)
    p.kernel_names = (kernel_name(conf, kernel, dict(transform_shared_to_regs_a=ta, transform_shared_to_regs_c=tc)),)
    return p


def matmatmul_plan(C, transA: str, transB: str, A, B, alpha, beta, *, wmma=None):
    """The launch ``matmatmul_`` would make, as a ``Plan`` to call any number of times: one launch of the
    configuration ``create_config`` picks (reference src/matmul.jl:185-204), whatever the sizes.  A 16-bit
    product whose sizes are not whole tiles, whose leading dimensions are odd or whose operands start off a
    16-byte boundary still runs on the aligned kernels (``create_config``); the bounds-checked kernel is left
    with operands that have fewer than 8 elements along their contiguous index."""
    return _single_plan(C, transA == 'T', transB == 'T', A, B, alpha, beta, wmma)


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
