"""The configurations used by tests and benchmarks (the role of reference configs/configs.jl:
``Configuration`` :31-47, ``generate_inputs`` :77-96, ``run_gemm`` :99-110 and the ``@get_*_config``
macros :161-490), plus the five benchmark workloads with their seeded synthetic inputs.

Seeds: workload n uses 1000n + {1: A, 2: B, 3: C, 4: bias / diagonal}.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Optional

import numpy as np

from . import cta_swizzle as CTASwizzle
from . import epilogue as Epilogue
from . import kernel as Kernel
from . import layout as Layout
from . import operator as Operator
from . import rng
from . import transform as Transform
from .arrays import colmajor, colmajor_empty
from .config import get_config
from .dtypes import Float16, Float32
from .matmul import kernel_name, matmul, plan
from .tiling import NT


@dataclass
class Workload:
    name: str
    description: str
    flops: int
    bytes: int
    bound: str                      # "mfma", "hbm" or "latency"
    make_host: Callable[[], dict]   # seeded numpy inputs
    make_launch: Callable[[dict], Callable[[], None]]
    kernel_name: str = ""
    _host: Optional[dict] = field(default=None, repr=False)

    def host(self) -> dict:
        if self._host is None:
            self._host = self.make_host()
        return self._host

    def host_inputs(self):
        h = self.host()
        return h.get("a"), h.get("b"), h.get("c")

    def prepare(self):
        """Upload the inputs and return a zero-argument function that enqueues one launch (a prepared
        ``Plan``: descriptors are lowered once, every call still passes the library's launch checks).
        The device tensors are reachable as attributes of the returned function (``.d`` is the output)."""
        return self.make_launch(self.host())


def _aligned(T, transposed):
    return Layout.UnsafeAlignedRowMajor[T] if transposed else Layout.UnsafeAlignedColMajor[T]


def mfma_config(M, N, K, ta=False, tb=False, zero_c=False, block_shape=None, **kw):
    """An MFMA configuration with aligned layouts in the spirit of @get_wmma_config
    (reference configs/configs.jl:246-289)."""
    params = dict(gemm_shape=NT(M=M, N=N, K=K), operator=Operator.MFMAOp[32, 32, 16, Float16, Float32],
                  global_a_layout=_aligned(Float16, ta), global_b_layout=_aligned(Float16, tb),
                  global_c_layout=Layout.Zero[Float32] if zero_c else Layout.UnsafeAlignedColMajor[Float32],
                  global_d_layout=Layout.UnsafeAlignedColMajor[Float32],
                  is_a_col_major=not ta, is_b_col_major=not tb)
    if block_shape is not None:
        params["block_shape"] = NT(M=block_shape[0], N=block_shape[1], K=block_shape[2])
    params.update(kw)
    return get_config(**params)


def _attach(fn, **tensors):
    for k, v in tensors.items():
        setattr(fn, k, v)
    return fn


def _config2(variant: str) -> Workload:
    ta, tb = variant[0] == "T", variant[1] == "T"
    M = N = K = 4096
    conf = mfma_config(M, N, K, ta, tb)

    def host():
        return dict(a=rng.matrix("upm1_f16", 2001, (K, M) if ta else (M, K)),
                    b=rng.matrix("upm1_f16", 2002, (N, K) if tb else (K, N)),
                    c=rng.matrix("upm1_f32", 2003, (M, N)))

    def launch(h):
        import torch
        a, b, c = colmajor(h["a"]), colmajor(h["b"]), colmajor(h["c"])
        d = colmajor_empty((M, N), torch.float32)

        launch_plan = plan(conf, a, b, c, d, kernel=Kernel.matmul_pipelined)

        def run():
            launch_plan()
        return _attach(run, a=a, b=b, c=c, d=d, conf=conf)

    return Workload(
        name=f"config 2 {variant}",
        description=f"config 2: C = A*B + C, FP16 A/B ~ U[-1,1), FP32 C ~ U[-1,1) read and accumulated, M=N=K=4096, "
                    f"column-major '{variant[0]}','{variant[1]}', alpha=beta=1",
        flops=2 * M * N * K, bytes=M * K * 2 + K * N * 2 + 2 * M * N * 4, bound="mfma",
        make_host=host, make_launch=launch, kernel_name=kernel_name(conf, Kernel.matmul_pipelined))


def _config3() -> Workload:
    M, N, K = 4096, 4096, 2048
    conf = mfma_config(M, N, K, zero_c=True)
    transforms = dict(transform_global_to_shared_a=Transform.Elementwise(lambda x: x * 0.5),
                      transform_shared_to_global_d=Transform.Elementwise(Transform.relu))

    def host():
        return dict(a=rng.matrix("upm1_f16", 3001, (M, K)), b=rng.matrix("upm1_f16", 3002, (K, N)),
                    bias=rng.normal_f32(3004, N))

    def launch(h):
        import torch
        a, b = colmajor(h["a"]), colmajor(h["b"])
        bias = torch.from_numpy(h["bias"]).cuda()
        d = colmajor_empty((M, N), torch.float32)
        epi = Epilogue.Bias(bias)

        launch_plan = plan(conf, a, b, None, d, epilogue=epi, kernel=Kernel.matmul_pipelined, **transforms)

        def run():
            launch_plan()
        return _attach(run, a=a, b=b, bias=bias, d=d, conf=conf)

    return Workload(
        name="config 3",
        description="config 3: D = relu((0.5*A)*B + bias[j]), FP16 A/B ~ U[-1,1), FP32 D, M=N=4096, K=2048, bias ~ N(0,1) per "
                    "column (Epilogue.Bias), scale on the global->shared load of A, ReLU on the shared->global store of D",
        flops=2 * M * N * K, bytes=M * K * 2 + K * N * 2 + N * 4 + M * N * 4, bound="mfma",
        make_host=host, make_launch=launch,
        kernel_name=kernel_name(conf, Kernel.matmul_pipelined, transforms, Epilogue.Bias(0)))


def _config1() -> Workload:
    M = N = K = 256
    from .matmul import create_config
    from .dtypes import Float32 as F32

    def host():
        return dict(a=rng.matrix("u01_f32", 1001, (M, K)), b=rng.matrix("u01_f32", 1002, (K, N)), c=None)

    conf, _, kern = create_config(F32, (M, K), (1, M), False, F32, (K, N), (1, K), False, F32, (M, N), (1, M),
                                  bool, False, bool, True, None)

    def launch(h):
        import torch
        from .matmul import matmatmul_plan
        a, b = colmajor(h["a"]), colmajor(h["b"])
        d = colmajor_empty((M, N), torch.float32)
        d.zero_()

        launch_plan = matmatmul_plan(d, "N", "N", a, b, True, False)     # mul!(C, A, B): alpha = 1, beta = 0  =>  FPUOp, C as Layout.Zero

        def run():
            launch_plan()
        return _attach(run, a=a, b=b, d=d, conf=conf)

    return Workload(
        name="config 1",
        description="config 1: C = A*B through mul!, FP32, M=N=K=256, column-major NN, A,B ~ U[0,1), beta = 0 (FPUOp on the vector ALUs)",
        flops=2 * M * N * K, bytes=3 * M * N * 4, bound="latency", make_host=host, make_launch=launch,
        kernel_name=kernel_name(conf, kern))


def gett_config(a_modes, b_modes, d_modes, extents, block_shape=None, zero_c=True, **kw):
    """A tensor-contraction configuration: the index arithmetic of the contraction lives in the
    Layout loaders (the pattern of reference benchmarks/tensor-contractions/run.jl:22-85)."""
    gmap = Layout.gett_map(a_modes, b_modes, d_modes, extents)
    M, N, K = gmap.extent("m"), gmap.extent("n"), gmap.extent("k")
    params = dict(gemm_shape=NT(M=M, N=N, K=K), operator=Operator.MFMAOp[32, 32, 16, Float16, Float32],
                  global_a_layout=Layout.GETT[Float16, gmap], global_b_layout=Layout.GETT[Float16, gmap],
                  global_c_layout=Layout.Zero[Float32] if zero_c else Layout.GETT[Float32, gmap],
                  global_d_layout=Layout.GETT[Float32, gmap],
                  shared_a_layout=Layout.UnsafeAlignedColMajor[Float16], shared_b_layout=Layout.UnsafeAlignedColMajor[Float16],
                  shared_c_layout=Layout.Zero[Float32] if zero_c else Layout.UnsafeAlignedColMajor[Float32],
                  shared_d_layout=Layout.UnsafeAlignedColMajor[Float32])
    if block_shape is not None:
        params["block_shape"] = NT(M=block_shape[0], N=block_shape[1], K=block_shape[2])
    params.update(kw)
    return get_config(**params), gmap


def diagonal_config(M, N, tb=False, zero_c=False, **kw):
    """@get_wmma_diagonal_config of the reference (configs/configs.jl:331-383): A is given by its
    diagonal, the kernel is matmul_singlestage."""
    params = dict(gemm_shape=NT(M=M, N=N, K=M), operator=Operator.MFMAOp[32, 32, 16, Float16, Float32],
                  global_a_layout=Layout.Diagonal[Float16], global_b_layout=_aligned(Float16, tb),
                  global_c_layout=Layout.Zero[Float32] if zero_c else Layout.UnsafeAlignedColMajor[Float32],
                  global_d_layout=Layout.UnsafeAlignedColMajor[Float32],
                  shared_a_layout=Layout.Padded[Layout.UnsafeAlignedColMajor[Float16], 8],
                  is_a_col_major=True, is_b_col_major=not tb)
    params.update(kw)
    return get_config(**params)


def _config4b() -> Workload:
    M = N = 4096
    conf = diagonal_config(M, N, zero_c=True)

    def host():
        return dict(a=rng.uniform_pm1_f16(4004, M), b=rng.matrix("upm1_f16", 4002, (M, N)), c=None)

    def launch(h):
        import torch
        a = torch.from_numpy(h["a"]).cuda()
        b = colmajor(h["b"])
        d = colmajor_empty((M, N), torch.float32)

        launch_plan = plan(conf, a, b, None, d, kernel=Kernel.matmul_singlestage)

        def run():
            launch_plan()
        return _attach(run, a=a, b=b, d=d, conf=conf)

    return Workload(
        name="config 4b",
        description="config 4b: D = diag(a) * B, a 4096 FP16 ~ U[-1,1), B 4096x4096 FP16 ~ U[-1,1), D FP32, no C "
                    "(Layout.Diagonal, single-stage kernel); bandwidth bound",
        flops=M * N, bytes=M * 2 + M * N * 2 + M * N * 4, bound="hbm", make_host=host, make_launch=launch,
        kernel_name=kernel_name(conf, Kernel.matmul_singlestage))


def complex_config(M, N, K, ta=False, tb=False, zero_c=True, dual=False, cd_type=Float32, **kw):
    """@get_wmma_complex_config / @get_wmma_dual_config of the reference (configs/configs.jl:385-490):
    interleaved Complex{Float16} in global memory, planar in shared memory, Complex{Float32} out
    (``cd_type``: the real type of the complex elements of C and D)."""
    il = lambda t: Layout.InterleavedRowMajor[Float16] if t else Layout.InterleavedColMajor[Float16]
    sp = lambda t: Layout.Padded[Layout.SplitRowMajor[Float16], 8] if t else Layout.Padded[Layout.SplitColMajor[Float16], 8]
    op = (Operator.MFMADualOp if dual else Operator.MFMAComplexOp)[16, 16, 16, Float16, Float32]
    params = dict(gemm_shape=NT(M=M, N=N, K=K), operator=op,
                  global_a_layout=il(ta), global_b_layout=il(tb),
                  global_c_layout=Layout.Zero[cd_type] if zero_c else Layout.InterleavedColMajor[cd_type],
                  global_d_layout=Layout.InterleavedColMajor[cd_type],
                  shared_a_layout=sp(ta), shared_b_layout=sp(tb),
                  shared_c_layout=Layout.Zero[Float32] if zero_c else Layout.SplitColMajor[Float32],
                  shared_d_layout=Layout.SplitColMajor[Float32],
                  is_a_col_major=not ta, is_b_col_major=not tb)
    params.update(kw)
    return get_config(**params)


def complex_planar_config(M, N, K, ta=False, tb=False, zero_c=True, **kw):
    """Complex GEMM on planar (split re / im) global arrays of logical shape (rows, cols, 2): the
    reference's LDS layouts Layout.SplitColMajor / SplitRowMajor (src/layout.jl:340-411) used as global
    layouts.  One launch when the planes of every operand are adjacent in memory, real GEMMs on the
    planes otherwise (gemmkernels.complex_planar)."""
    sp = lambda t, T: Layout.SplitRowMajor[T] if t else Layout.SplitColMajor[T]
    params = dict(gemm_shape=NT(M=M, N=N, K=K), operator=Operator.MFMAComplexOp[16, 16, 16, Float16, Float32],
                  global_a_layout=sp(ta, Float16), global_b_layout=sp(tb, Float16),
                  global_c_layout=Layout.Zero[Float32] if zero_c else Layout.SplitColMajor[Float32],
                  global_d_layout=Layout.SplitColMajor[Float32],
                  is_a_col_major=not ta, is_b_col_major=not tb)
    params.update(kw)
    return get_config(**params)


def complex_matrix(seed, rows, cols):
    """Interleaved Complex{Float16} matrix as a real array of shape (2, rows, cols), column-major:
    re and im ~ U[-1,1) from one stream in storage order."""
    return rng.matrix("upm1_f16", seed, (2, rows, cols))


def _config4a() -> Workload:
    M = N = K = 2048
    conf = complex_config(M, N, K)

    def host():
        return dict(a=complex_matrix(4001, M, K), b=complex_matrix(4002, K, N), c=None)

    def launch(h):
        import torch
        a, b = colmajor(h["a"]), colmajor(h["b"])
        d = colmajor_empty((2, M, N), torch.float32)

        launch_plan = plan(conf, a, b, None, d, kernel=Kernel.matmul_pipelined)

        def run():
            launch_plan()
        return _attach(run, a=a, b=b, d=d, conf=conf)

    return Workload(
        name="config 4a",
        description="config 4a: complex D = A*B, Complex{Float16} in (interleaved, re/im ~ U[-1,1)), Complex{Float32} out, "
                    "M=N=K=2048, column-major NN; 8*N^3 real flop",
        flops=8 * M * N * K, bytes=M * K * 4 + K * N * 4 + M * N * 8, bound="mfma", make_host=host, make_launch=launch,
        kernel_name=kernel_name(conf, Kernel.matmul_pipelined))


def _config5() -> Workload:
    ext = dict(a=64, b=64, c=64, d=64, e=64, f=64)
    conf, gmap = gett_config("aebf", "dfce", "abcd", ext)
    M = N = K = 4096

    def host():
        return dict(a=rng.matrix("upm1_f16", 5001, (64, 64, 64, 64)), b=rng.matrix("upm1_f16", 5002, (64, 64, 64, 64)), c=None)

    def launch(h):
        import torch
        a, b = colmajor(h["a"]), colmajor(h["b"])
        d = colmajor_empty((64, 64, 64, 64), torch.float32)

        launch_plan = plan(conf, a, b, None, d, kernel=Kernel.matmul_pipelined)

        def run():
            launch_plan()
        return _attach(run, a=a, b=b, d=d, conf=conf)

    return Workload(
        name="config 5",
        description="config 5: GETT D[a,b,c,d] = sum_{e,f} A[a,e,b,f] * B[d,f,c,e], all extents 64 (M=N=K=4096), FP16 in ~ U[-1,1), "
                    "FP32 out, dense column-major tensors, contraction index map in the Layout loader",
        flops=2 * M * N * K, bytes=M * K * 2 + K * N * 2 + M * N * 4, bound="mfma", make_host=host, make_launch=launch,
        kernel_name=kernel_name(conf, Kernel.matmul_pipelined))


def _config4a_planar() -> Workload:
    """Config 4a on planar (split re / im) global arrays: one launch that walks K twice."""
    M = N = K = 2048
    conf = complex_planar_config(M, N, K)

    def planar(seed, rows, cols):
        return rng.matrix("upm1_f16", seed, (rows * cols, 2)).reshape((rows, cols, 2), order="F")

    def host():
        return dict(a=planar(4001, M, K), b=planar(4002, K, N), c=None)

    def launch(h):
        import torch
        a, b = colmajor(h["a"]), colmajor(h["b"])
        d = colmajor_empty((M, N, 2), torch.float32)
        launch_plan = plan(conf, a, b, None, d, kernel=Kernel.matmul_pipelined)

        def run():
            launch_plan()
        return _attach(run, a=a, b=b, d=d, conf=conf)

    return Workload(
        name="config 4a planar",
        description="config 4a on planar global arrays (rows, cols, 2): Complex{Float16} A, B 2048x2048, Complex{Float32} D, no C; "
                    "one launch, two passes over K",
        flops=8 * M * N * K, bytes=(M * K + K * N) * 4 + M * N * 8, bound="mfma", make_host=host, make_launch=launch,
        kernel_name=kernel_name(conf, Kernel.matmul_pipelined))


def _skinny() -> Workload:
    """Not one of the five benchmark configurations: a skinny product (few output tiles, long K) that
    is bound by memory and latency, timed with the K-split kernel kind."""
    M, N, K = 4096, 64, 4096
    conf = mfma_config(M, N, K, block_shape=(64, 64, 64))

    def host():
        return dict(a=rng.matrix("upm1_f16", 6001, (M, K)), b=rng.matrix("upm1_f16", 6002, (K, N)), c=rng.matrix("upm1_f32", 6003, (M, N)))

    def launch(h):
        import torch
        a, b, c = colmajor(h["a"]), colmajor(h["b"]), colmajor(h["c"])
        d = colmajor_empty((M, N), torch.float32)
        launch_plan = plan(conf, a, b, c, d, kernel=Kernel.matmul_split_k)

        def run():
            launch_plan()
        return _attach(run, a=a, b=b, c=c, d=d, conf=conf)

    return Workload(
        name="skinny",
        description="skinny product C = A*B + C, M=4096, N=64, K=4096, FP16 A/B, FP32 C/D, 'N','N', K-split kernel (64 tiles x 4 K slices, ordered reduction)",
        flops=2 * M * N * K, bytes=M * K * 2 + K * N * 2 + 2 * M * N * 4, bound="hbm", make_host=host, make_launch=launch,
        kernel_name="mfma_gemm_splitk_nn_64x64x64_w2x2_f16")


def _mul4000() -> Workload:
    """Not one of the five benchmark configurations: mul!(C, A, B) at a size that is not a whole number of
    tiles, through the BLAS-level front end (bounds-checked layouts with 16-byte aligned columns, which the
    library runs on the aligned kernel with masked edge tiles: four waves, one per SIMD, as M and N are multiples of 8)."""
    M = N = K = 4000

    def host():
        return dict(a=rng.matrix("upm1_f16", 9001, (M, K)), b=rng.matrix("upm1_f16", 9002, (K, N)))

    def launch(h):
        import torch
        from .matmul import matmatmul_plan
        a, b = colmajor(h["a"]), colmajor(h["b"])
        c = colmajor_empty((M, N), torch.float32)
        launch_plan = matmatmul_plan(c, "N", "N", a, b, 1.0, 0.0)

        def run():
            launch_plan()
        return _attach(run, a=a, b=b, c=c, d=c, conf=None)

    return Workload(
        name="mul4000",
        description="mul!(C, A, B), M=N=K=4000 (not whole tiles), FP16 A/B, FP32 C, 'N','N', C not read",
        flops=2 * M * N * K, bytes=M * K * 2 + K * N * 2 + M * N * 4, bound="mfma", make_host=host, make_launch=launch,
        kernel_name="mfma_gemm_nn_256x256x64_w2x2_s2__Float16_edges")


def benchmark_config(n, variant: Optional[str] = None) -> Workload:
    """The benchmark workloads 1, 2 (variant NN/NT/TN/TT), 3, "4a", "4b", 5, "skinny" and "mul4000"."""
    if n == 2:
        return _config2(variant or "NN")
    if n == 3:
        return _config3()
    builders = _LATE_BUILDERS
    if n in builders:
        return builders[n]()
    raise NotImplementedError(f"benchmark config {n}")


_LATE_BUILDERS = {1: _config1, "4a": _config4a, "4a-planar": _config4a_planar, "4b": _config4b, 5: _config5, "skinny": _skinny, "mul4000": _mul4000}
