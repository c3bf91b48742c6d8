"""GPU parity of the MFMA GEMM (config 2 of the benchmark: FP16 x FP16 -> FP32, all four transposes)
against the CPU oracle.  Tolerance: relative Frobenius error <= 1e-3 (FP16 in / FP32 accumulate)."""
import numpy as np
import pytest

import gemmkernels as gk
from gemmkernels import Layout, Operator, Kernel, CTASwizzle, NT, Float16, Float32, rng
import helpers
from oracle import oracle

pytestmark = pytest.mark.gpu

TOL = 1e-3

TILES = [  # block shape, (waves_m, waves_n)
    ((256, 256, 64), (2, 4)),
    ((256, 256, 64), (2, 2)),
    ((256, 256, 32), (2, 4)),
    ((256, 256, 32), (2, 2)),
    ((256, 256, 32), (4, 2)),
    ((256, 128, 64), (2, 2)),
    ((128, 256, 64), (2, 2)),
    ((128, 128, 64), (2, 2)),
    ((128, 128, 64), (4, 2)),
    ((128, 128, 32), (2, 2)),
    ((64, 64, 64), (2, 2)),
    ((64, 64, 32), (1, 1)),
]


def make_config(M, N, K, ta, tb, block, waves, zero_c=False, swizzle=None, op=None):
    BM, BN, BK = block
    la = Layout.UnsafeAlignedRowMajor[Float16] if ta else Layout.UnsafeAlignedColMajor[Float16]
    lb = Layout.UnsafeAlignedRowMajor[Float16] if tb else Layout.UnsafeAlignedColMajor[Float16]
    kw = {}
    if swizzle is not None:
        kw["cta_swizzle"] = swizzle
    return gk.get_config(
        gemm_shape=NT(M=M, N=N, K=K), block_shape=NT(M=BM, N=BN, K=BK),
        warps_per_block=waves[0] * waves[1], compute_warp=NT(M=BM // waves[0], N=BN // waves[1], K=16),
        operator=op or Operator.MFMAOp[32, 32, 16, Float16, Float32],
        global_a_layout=la, global_b_layout=lb,
        global_c_layout=Layout.Zero[Float32] if zero_c else Layout.UnsafeAlignedColMajor[Float32],
        global_d_layout=Layout.UnsafeAlignedColMajor[Float32],
        is_a_col_major=not ta, is_b_col_major=not tb, **kw)


def inputs(M, N, K, ta, tb, seed):
    a = rng.matrix("upm1_f16", seed + 1, (K, M) if ta else (M, K))
    b = rng.matrix("upm1_f16", seed + 2, (N, K) if tb else (K, N))
    c = rng.matrix("upm1_f32", seed + 3, (M, N))
    return a, b, c


@pytest.mark.parametrize("block,waves", TILES)
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_tiles_all_transposes(gpu, block, waves, ta, tb):
    BM, BN, BK = block
    M, N, K = 2 * BM, 2 * BN, 5 * BK
    conf = make_config(M, N, K, ta, tb, block, waves)
    a, b, c = inputs(M, N, K, ta, tb, 2000)
    print("case", block, waves, ta, tb, gk.kernel_name(conf, Kernel.matmul_pipelined), flush=True)
    d = helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    ref = helpers.run_oracle(conf, a, b, c, (M, N))
    assert np.isfinite(d).all()
    err = oracle.rel_frobenius(d, ref)
    assert err <= TOL, err
    # the C restatement itself agrees with float64 GEMM
    ref64 = oracle.gemm_f64(a, b, c, 1.0, 1.0, ta, tb)
    assert oracle.rel_frobenius(d, ref64) <= TOL


@pytest.mark.parametrize("ta,tb", [(False, False), (True, True)])
def test_zero_c_and_alias(gpu, ta, tb):
    M, N, K = 512, 256, 192
    a, b, c = inputs(M, N, K, ta, tb, 2100)
    conf = make_config(M, N, K, ta, tb, (128, 128, 64), (2, 2), zero_c=True)
    d = helpers.run_gpu(conf, a, b, None, (M, N), kernel=Kernel.matmul_pipelined)
    assert oracle.rel_frobenius(d, oracle.gemm_f64(a, b, None, 1.0, 0.0, ta, tb)) <= TOL
    # d aliases c (reference src/matmul.jl:198)
    conf = make_config(M, N, K, ta, tb, (128, 128, 64), (2, 2))
    d = helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_pipelined, alias_cd=True)
    assert oracle.rel_frobenius(d, oracle.gemm_f64(a, b, c, 1.0, 1.0, ta, tb)) <= TOL


def test_identity_and_ones_closed_forms(gpu):
    M = N = K = 256
    conf = make_config(M, N, K, False, False, (128, 128, 64), (2, 2))
    b = rng.matrix("upm1_f16", 7, (K, N))
    c = rng.matrix("upm1_f32", 8, (M, N))
    eye = np.asfortranarray(np.eye(M, dtype=np.float16))
    d = helpers.run_gpu(conf, eye, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d, b.astype(np.float32) + c)           # A = I  =>  D = B + C exactly
    ones_a = np.asfortranarray(np.ones((M, K), dtype=np.float16))
    ones_b = np.asfortranarray(np.ones((K, N), dtype=np.float16))
    conf0 = make_config(M, N, K, False, False, (128, 128, 64), (2, 2), zero_c=True)
    d = helpers.run_gpu(conf0, ones_a, ones_b, None, (M, N), kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d, np.full((M, N), float(K), dtype=np.float32))


def test_distinct_index_probe(gpu):
    """A single non-zero in A and in B: exactly one product lands in exactly one place, for every
    transpose -- catches any swapped index or wrong tile origin."""
    M, N, K = 256, 384, 128
    for ta, tb in [(False, False), (False, True), (True, False), (True, True)]:
        conf = make_config(M, N, K, ta, tb, (128, 128, 64), (2, 2), zero_c=True)
        for (i, k, j) in [(0, 0, 0), (255, 127, 383), (130, 65, 257), (31, 100, 200)]:
            a = np.zeros((K, M) if ta else (M, K), dtype=np.float16, order="F")
            b = np.zeros((N, K) if tb else (K, N), dtype=np.float16, order="F")
            if ta: a[k, i] = 3.0
            else: a[i, k] = 3.0
            if tb: b[j, k] = 0.5
            else: b[k, j] = 0.5
            d = helpers.run_gpu(conf, a, b, None, (M, N), kernel=Kernel.matmul_pipelined)
            expect = np.zeros((M, N), dtype=np.float32)
            expect[i, j] = 1.5
            assert np.array_equal(d, expect), (ta, tb, i, k, j)


@pytest.mark.parametrize("swz", [CTASwizzle.Identity, CTASwizzle.HorizontallyTiled[2], CTASwizzle.VerticallyTiled[2],
                                 CTASwizzle.LebesgueCurve, CTASwizzle.XCDAware[4], CTASwizzle.XCDAware[3]])
def test_cta_swizzles(gpu, swz):
    M, N, K = 512, 512, 128
    conf = make_config(M, N, K, False, True, (128, 128, 64), (2, 2), swizzle=swz)
    a, b, c = inputs(M, N, K, False, True, 2200)
    d = helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    assert oracle.rel_frobenius(d, oracle.gemm_f64(a, b, c, 1.0, 1.0, False, True)) <= TOL


def test_wmma_compat_operator(gpu):
    """A reference-style config (WMMAOp 16x16x16, block 128x128x64, 8 warps as 4 x 2) runs as is."""
    M = N = K = 256
    conf = make_config(M, N, K, False, False, (128, 128, 64), (4, 2), op=Operator.WMMAOp[16, 16, 16, Float16, Float32])
    a, b, c = inputs(M, N, K, False, False, 2300)
    d = helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    assert oracle.rel_frobenius(d, oracle.gemm_f64(a, b, c, 1.0, 1.0)) <= TOL


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_full_size_4096(gpu, ta, tb):
    """Benchmark config 2 at full size, checked against the CPU BLAS path (OpenBLAS sgemm on the
    exactly converted inputs) and through linearity: D(C) - D(0) == C."""
    M = N = K = 4096
    a, b, c = inputs(M, N, K, ta, tb, 2000)
    conf = make_config(M, N, K, ta, tb, (256, 256, 64), (2, 4))
    d = helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    ref = oracle.gemm_blas_f32(a, b, c, 1.0, 1.0, ta, tb)
    assert oracle.rel_frobenius(d, ref) <= TOL
    conf0 = make_config(M, N, K, ta, tb, (256, 256, 64), (2, 4), zero_c=True)
    d0 = helpers.run_gpu(conf0, a, b, None, (M, N), kernel=Kernel.matmul_pipelined)
    assert oracle.rel_frobenius(d - d0, c) <= 1e-4
