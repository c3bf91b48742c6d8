"""GPU parity of the complex and dual-number GEMM (benchmark config 4a; reference
configs/configs.jl:385-490, test sweep :656-695) against numpy complex128 and the CPU oracle.
Tolerance: relative Frobenius error <= 1e-3 (FP16 in, FP32 accumulate)."""
import numpy as np
import pytest
import torch

import gemmkernels as gk
from gemmkernels import Kernel, NT, configs, rng
import helpers
from oracle import oracle

pytestmark = pytest.mark.gpu
TOL = 1e-3


def to_c128(x):            # (2, rows, cols) -> complex (rows, cols)
    return x[0].astype(np.float64) + 1j * x[1].astype(np.float64)


def run(conf, a, b, c, M, N):
    ta, tb = gk.colmajor(a), gk.colmajor(b)
    tc = None if c is None else gk.colmajor(c)
    td = gk.colmajor_empty((2, M, N), torch.float32)
    td.fill_(float("nan"))
    gk.matmul(conf, ta, tb, tc, td, kernel=Kernel.matmul_pipelined)
    torch.cuda.synchronize()
    return gk.to_numpy(td)


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("dims,block", [((128, 128, 64), (32, 64, 32)), ((128, 128, 128), (64, 64, 32)), ((128, 256, 96), (64, 128, 32)),
                                        ((256, 256, 160), (128, 128, 32)),
                                        ((256, 512, 64), (128, 256, 32))])
def test_complex_all_transposes(gpu, dims, block, ta, tb):
    M, N, K = dims
    conf = configs.complex_config(M, N, K, ta, tb, block_shape=gk.NT(M=block[0], N=block[1], K=block[2]))
    a = configs.complex_matrix(61, K if ta else M, M if ta else K)
    b = configs.complex_matrix(62, N if tb else K, K if tb else N)
    print("case", dims, block, ta, tb, gk.kernel_name(conf, Kernel.matmul_pipelined), flush=True)
    d = run(conf, a, b, None, M, N)
    A = to_c128(a).T if ta else to_c128(a)          # 'T' is a plain transpose, no conjugation (src/matmul.jl:211-213)
    B = to_c128(b).T if tb else to_c128(b)
    assert oracle.rel_frobenius(to_c128(d), A @ B) <= TOL
    # the CPU oracle restates WMMAComplexOp.mma (src/operator.jl:307-311)
    ref = np.zeros((2, M, N), np.float32, order="F")
    p = helpers.oracle_problem(conf, (a.shape[1], b.shape[1], M, M))
    oracle.matmul(p, a, b, None, ref)
    assert oracle.rel_frobenius(to_c128(d), to_c128(ref)) <= TOL


def test_complex_identities_and_c(gpu):
    M = N = K = 128
    conf = configs.complex_config(M, N, K, block_shape=gk.NT(M=64, N=64, K=32))
    a = configs.complex_matrix(71, M, K)
    b = configs.complex_matrix(72, K, N)
    a_real, b_real = a.copy(order="F"), b.copy(order="F")
    a_real[1] = 0
    b_real[1] = 0
    d = run(conf, a_real, b_real, None, M, N)
    assert np.all(d[1] == 0)                                   # real inputs => imaginary part exactly zero
    bi = np.zeros((2, K, N), np.float16, order="F")
    bi[1, np.arange(K), np.arange(K)] = 1                      # B = i * I  =>  A * B = (-im A, re A)
    d = run(conf, a, bi, None, M, N)
    assert np.array_equal(d[0], -a[1].astype(np.float32)) and np.array_equal(d[1], a[0].astype(np.float32))
    conf_c = configs.complex_config(M, N, K, zero_c=False, block_shape=gk.NT(M=64, N=64, K=32))
    c = rng.matrix("upm1_f32", 73, (2, M, N))
    d = run(conf_c, a, b, c, M, N)
    assert oracle.rel_frobenius(to_c128(d), to_c128(a) @ to_c128(b) + to_c128(c)) <= TOL


@pytest.mark.parametrize("block", [(64, 64, 32), (64, 128, 32)])
def test_dual_numbers(gpu, block):
    """(re, du): re = a_re b_re, du = a_re b_du + a_du b_re (reference src/operator.jl:366-369)."""
    M, N, K = 128, 256, 64
    conf = configs.complex_config(M, N, K, dual=True, block_shape=gk.NT(M=block[0], N=block[1], K=block[2]))
    a = configs.complex_matrix(81, M, K)
    b = configs.complex_matrix(82, K, N)
    d = run(conf, a, b, None, M, N)
    a0, a1, b0, b1 = (x.astype(np.float64) for x in (a[0], a[1], b[0], b[1]))
    assert oracle.rel_frobenius(d[0], a0 @ b0) <= TOL
    assert oracle.rel_frobenius(d[1], a0 @ b1 + a1 @ b0) <= TOL
    # and against the oracle's dual-number product (itself pinned against these float64 forms on the CPU)
    ref = np.zeros((2, M, N), np.float32, order="F")
    p = helpers.oracle_problem(conf, (M, K, M, M))
    assert p.op_kind == oracle.OP_DUAL
    oracle.matmul(p, a, b, None, ref)
    assert oracle.rel_frobenius(d[0], ref[0]) <= TOL and oracle.rel_frobenius(d[1], ref[1]) <= TOL


def test_config4a_full_size(gpu):
    w = configs.benchmark_config("4a")
    r = w.prepare()
    r()
    torch.cuda.synchronize()
    h = w.host()
    d = to_c128(gk.to_numpy(r.d))
    ref = (to_c128(h["a"]).astype(np.complex64) @ to_c128(h["b"]).astype(np.complex64))
    assert oracle.rel_frobenius(d, ref) <= TOL


def planar(seed, rows, cols, dtype=np.float16):
    """Planar complex matrix as a real array of logical shape (rows, cols, 2), column-major."""
    kind = "upm1_f16" if dtype == np.float16 else "upm1_f32"
    return rng.matrix(kind, seed, (rows * cols, 2)).reshape((rows, cols, 2), order="F")


def planar_to_c128(x):
    return x[:, :, 0].astype(np.float64) + 1j * x[:, :, 1].astype(np.float64)


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("zero_c", [True, False])
def test_planar_global_layouts(gpu, ta, tb, zero_c):
    """Complex GEMM on split re / im global arrays (Layout.SplitColMajor / SplitRowMajor as global
    layouts): real GEMMs on the planes with the sign pattern of WMMAComplexOp.mma (src/operator.jl:307-311)."""
    M, N, K = 256, 384, 192
    conf = configs.complex_planar_config(M, N, K, ta, tb, zero_c=zero_c)
    a = planar(81, K if ta else M, M if ta else K)
    b = planar(82, N if tb else K, K if tb else N)
    c = None if zero_c else planar(83, M, N, np.float32)
    ta_, tb_ = gk.colmajor(a), gk.colmajor(b)
    tc = None if zero_c else gk.colmajor(c)
    td = gk.colmajor_empty((M, N, 2), torch.float32)
    td.fill_(float("nan"))
    gk.matmul(conf, ta_, tb_, tc, td, kernel=Kernel.matmul_pipelined)
    torch.cuda.synchronize()
    A = planar_to_c128(a).T if ta else planar_to_c128(a)
    B = planar_to_c128(b).T if tb else planar_to_c128(b)
    ref = A @ B + (0 if zero_c else planar_to_c128(c))
    d = planar_to_c128(gk.to_numpy(td))
    assert np.isfinite(d).all()
    assert oracle.rel_frobenius(d, ref) <= TOL
    if not zero_c:      # in place, mul! style: d is c
        gk.matmul(conf, ta_, tb_, tc, tc, kernel=Kernel.matmul_pipelined)
        torch.cuda.synchronize()
        assert oracle.rel_frobenius(planar_to_c128(gk.to_numpy(tc)), ref) <= TOL


def _run_planar(M, N, K, ta, tb, zero_c, block=None, seed=90):
    kw = {} if block is None else dict(block_shape=NT(M=block[0], N=block[1], K=block[2]))
    conf = configs.complex_planar_config(M, N, K, ta, tb, zero_c=zero_c, **kw)
    a = planar(seed + 1, K if ta else M, M if ta else K)
    b = planar(seed + 2, N if tb else K, K if tb else N)
    c = None if zero_c else planar(seed + 3, M, N, np.float32)
    ta_, tb_ = gk.colmajor(a), gk.colmajor(b)
    tc = None if zero_c else gk.colmajor(c)
    td = gk.colmajor_empty((M, N, 2), torch.float32)
    td.fill_(float("nan"))
    gk.matmul(conf, ta_, tb_, tc, td, kernel=Kernel.matmul_pipelined)
    torch.cuda.synchronize()
    A = planar_to_c128(a).T if ta else planar_to_c128(a)
    B = planar_to_c128(b).T if tb else planar_to_c128(b)
    ref = A @ B + (0 if zero_c else planar_to_c128(c))
    d = planar_to_c128(gk.to_numpy(td))
    assert np.isfinite(d).all()
    return conf, oracle.rel_frobenius(d, ref), oracle.rel_frobenius(d.real, ref.real), oracle.rel_frobenius(d.imag, ref.imag)


@pytest.mark.parametrize("block", [(128, 256, 64), (128, 128, 64), (64, 128, 32), (64, 128, 64), (64, 64, 32)])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_planar_kernel_every_tile(gpu, block, ta, tb):
    """The single-launch kernel for planar matrices, every compiled tile and transpose, C read: each
    plane of D is checked on its own (a wrong sign or a swapped plane leaves the other one intact)."""
    M, N, K = 2 * block[0], 3 * block[1], 5 * block[2]
    conf, err, err_re, err_im = _run_planar(M, N, K, ta, tb, False, block)
    assert "planar" in gk.kernel_name(conf, Kernel.matmul_pipelined)
    assert err <= TOL and err_re <= TOL and err_im <= TOL


@pytest.mark.parametrize("ktiles", [1, 2, 3])
def test_planar_kernel_short_k(gpu, ktiles):
    """K of one to three tiles: the switch from the first pass over K to the second falls into the
    prologue of the pipeline."""
    for block in [(128, 256, 64), (64, 128, 32)]:
        _, err, err_re, err_im = _run_planar(block[0], block[1], ktiles * block[2], False, False, True, block, seed=95)
        assert err <= TOL and err_re <= TOL and err_im <= TOL


def test_planar_operands_with_separate_planes_fall_back_to_real_gemms(gpu):
    """Planes that do not follow each other in memory (a view into a wider array) run as real GEMMs on
    the planes; same result."""
    M, N, K = 128, 256, 96
    conf = configs.complex_planar_config(M, N, K, False, False, zero_c=True)
    a, b = planar(101, M, K), planar(102, K, N)
    wide_a = gk.colmajor_empty((M, K + 8, 2), torch.float16)
    wide_a.zero_()
    wide_a[:, :K, :] = gk.colmajor(a)
    ta_ = wide_a[:, :K, :]
    assert ta_.stride(2) != ta_.stride(1) * ta_.size(1)
    td = gk.colmajor_empty((M, N, 2), torch.float32)
    gk.matmul(conf, ta_, gk.colmajor(b), None, td, kernel=Kernel.matmul_pipelined)
    torch.cuda.synchronize()
    ref = planar_to_c128(a) @ planar_to_c128(b)
    assert oracle.rel_frobenius(planar_to_c128(gk.to_numpy(td)), ref) <= TOL


def test_config4a_planar_full_size(gpu):
    """Benchmark config 4a on planar arrays at its full size (2048^3), one launch; both planes checked
    against a complex64 product of the same inputs."""
    w = configs.benchmark_config("4a-planar")
    assert "planar" in w.kernel_name
    r = w.prepare()
    r()
    torch.cuda.synchronize()
    h = w.host()
    d = planar_to_c128(gk.to_numpy(r.d))
    ref = planar_to_c128(h["a"]).astype(np.complex64) @ planar_to_c128(h["b"]).astype(np.complex64)
    assert oracle.rel_frobenius(d.real, ref.real) <= TOL
    assert oracle.rel_frobenius(d.imag, ref.imag) <= TOL
