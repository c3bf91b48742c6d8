"""GPU parity of the MFMA GEMM (config 2 of the benchmark: FP16 x FP16 -> FP32, all four transposes)
against the CPU oracle.  Tolerance: relative Frobenius error <= 1e-3 (FP16 in / FP32 accumulate)."""
import numpy as np
import pytest

import gemmkernels as gk
from gemmkernels import Layout, Operator, Kernel, CTASwizzle, NT, Float16, Float32, configs, rng
import helpers
from oracle import oracle

pytestmark = pytest.mark.gpu

TOL = 1e-3

TILES = [  # block shape, (waves_m, waves_n)
    ((256, 256, 64), (2, 4)),
    ((256, 256, 64), (2, 2)),     # one wave per SIMD
    ((256, 256, 32), (2, 4)),
    ((256, 256, 32), (4, 2)),
    ((256, 128, 64), (2, 2)),
    ((128, 256, 64), (2, 2)),
    ((128, 128, 64), (2, 2)),
    ((128, 128, 64), (4, 2)),
    ((128, 128, 32), (2, 2)),
    ((64, 64, 64), (2, 2)),
    ((64, 64, 32), (1, 1)),
    ((64, 64, 32), (2, 2)),
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


@pytest.mark.parametrize("waves", [(2, 4), "default"])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_full_size_4096(gpu, ta, tb, waves):
    """Benchmark config 2 at full size, checked against the CPU BLAS path (OpenBLAS sgemm on the
    exactly converted inputs) and through linearity: D(C) - D(0) == C.  `default` is the configuration of the
    benchmark itself (configs.benchmark_config(2, variant): the tile, wave arrangement and tile walk that bench.py times),
    (2, 4) the eight-wave arrangement of the same tile.  Comparison as in reference test/matmul.jl:12-20."""
    M = N = K = 4096
    a, b, c = inputs(M, N, K, ta, tb, 2000)
    if waves == "default":
        variant = ("T" if ta else "N") + ("T" if tb else "N")
        wl = configs.benchmark_config(2, variant=variant)
        conf = configs.mfma_config(M, N, K, ta, tb)
        assert gk.kernel_name(conf, Kernel.matmul_pipelined) == wl.kernel_name        # the kernel that the benchmark times
        assert "w2x2" in wl.kernel_name
        conf0 = configs.mfma_config(M, N, K, ta, tb, zero_c=True)
    else:
        conf = make_config(M, N, K, ta, tb, (256, 256, 64), waves)
        conf0 = make_config(M, N, K, ta, tb, (256, 256, 64), waves, zero_c=True)
    d = helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    ref = oracle.gemm_blas_f32(a, b, c, 1.0, 1.0, ta, tb)
    assert oracle.rel_frobenius(d, ref) <= TOL
    d0 = helpers.run_gpu(conf0, a, b, None, (M, N), kernel=Kernel.matmul_pipelined)
    assert oracle.rel_frobenius(d - d0, c) <= 1e-4
    if waves == "default":
        # the benchmark's own inputs and prepared launch: what bench.py times is what is checked here
        run = wl.prepare()
        run()
        import torch
        torch.cuda.synchronize()
        ha, hb, hc = wl.host_inputs()
        assert oracle.rel_frobenius(gk.to_numpy(run.d), oracle.gemm_blas_f32(ha, hb, hc, 1.0, 1.0, ta, tb)) <= TOL


@pytest.mark.parametrize("block,waves", [((256, 256, 64), (2, 4)), ((128, 128, 64), (2, 2)), ((64, 64, 32), (1, 1))])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, True)])
def test_f16_c_and_d(gpu, block, waves, ta, tb):
    """FP16 C and D with FP32 accumulation (the reference's F16 -> F16 WMMA configuration,
    configs/configs.jl:574, accumulates in FP16; one rounding at the store is at least as accurate)."""
    import torch
    BM, BN, BK = block
    M, N, K = 2 * BM, BN, 4 * BK
    la = Layout.UnsafeAlignedRowMajor[Float16] if ta else Layout.UnsafeAlignedColMajor[Float16]
    lb = Layout.UnsafeAlignedRowMajor[Float16] if tb else Layout.UnsafeAlignedColMajor[Float16]
    conf = gk.get_config(
        gemm_shape=NT(M=M, N=N, K=K), block_shape=NT(M=BM, N=BN, K=BK), warps_per_block=waves[0] * waves[1],
        compute_warp=NT(M=BM // waves[0], N=BN // waves[1], K=16), operator=Operator.MFMAOp[32, 32, 16, Float16, Float32],
        global_a_layout=la, global_b_layout=lb, global_c_layout=Layout.UnsafeAlignedColMajor[Float16],
        global_d_layout=Layout.UnsafeAlignedColMajor[Float16], is_a_col_major=not ta, is_b_col_major=not tb)
    a, b, _ = inputs(M, N, K, ta, tb, 2300)
    c = rng.matrix("upm1_f16", 2304, (M, N))
    d = helpers.run_gpu(conf, a, b, c, (M, N), d_dtype=torch.float16, kernel=Kernel.matmul_pipelined)
    assert d.dtype == np.float16
    ref = helpers.run_oracle(conf, a, b, c, (M, N), d_dtype=np.float16)
    assert oracle.rel_frobenius(d, ref) <= TOL
    # a different summation order moves a result across an FP16 rounding boundary only rarely, and then by one ulp
    differ = d != ref
    assert differ.mean() < 0.02
    assert np.all(np.abs(d.astype(np.float64) - ref.astype(np.float64))[differ] <= np.spacing(np.abs(ref).astype(np.float16))[differ])
    assert oracle.rel_frobenius(d, oracle.gemm_f64(a, b, c, 1.0, 1.0, ta, tb)) <= TOL


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("d16", [False, True])
def test_bf16(gpu, ta, tb, d16):
    """BFloat16 multiplicands (v_mfma_f32_32x32x16_bf16), FP32 or BFloat16 C / D."""
    import torch
    from gemmkernels import BFloat16
    M, N, K = 256, 384, 320
    block, waves = (128, 128, 64), (2, 2)
    a = gk.bf16_bits(rng.matrix("upm1_f32", 2401, (K, M) if ta else (M, K)))
    b = gk.bf16_bits(rng.matrix("upm1_f32", 2402, (N, K) if tb else (K, N)))
    c32 = rng.matrix("upm1_f32", 2403, (M, N))
    c = gk.bf16_bits(c32) if d16 else c32
    CD = BFloat16 if d16 else Float32
    la = Layout.UnsafeAlignedRowMajor[BFloat16] if ta else Layout.UnsafeAlignedColMajor[BFloat16]
    lb = Layout.UnsafeAlignedRowMajor[BFloat16] if tb else Layout.UnsafeAlignedColMajor[BFloat16]
    conf = gk.get_config(
        gemm_shape=NT(M=M, N=N, K=K), block_shape=NT(M=block[0], N=block[1], K=block[2]), warps_per_block=4,
        compute_warp=NT(M=64, N=64, K=16), operator=Operator.MFMAOp[32, 32, 16, BFloat16, Float32],
        global_a_layout=la, global_b_layout=lb, global_c_layout=Layout.UnsafeAlignedColMajor[CD],
        global_d_layout=Layout.UnsafeAlignedColMajor[CD], is_a_col_major=not ta, is_b_col_major=not tb)
    d = helpers.run_gpu(conf, a, b, c, (M, N), d_dtype=torch.bfloat16 if d16 else torch.float32, kernel=Kernel.matmul_pipelined)
    ref = helpers.run_oracle(conf, a, b, c, (M, N), d_dtype=np.uint16 if d16 else np.float32)
    if d16:
        # same rounding (to nearest even, once, at the store) as the oracle: the bit patterns differ only where the
        # two fp32 sums (different orders) straddle a rounding boundary or nearly cancel -- a few elements in a
        # hundred thousand.  Truncation or round-half-up would differ in about half of the elements.
        got_bits = gk.bf16_bits(d.astype(np.float32))
        assert (got_bits != ref).mean() < 1e-3, (got_bits != ref).mean()
        ref = gk.bf16_values(ref)
    tol = 4e-3 if d16 else TOL        # against float64, a BFloat16 result carries 2^-9 relative rounding per element
    assert oracle.rel_frobenius(d, ref) <= (1e-3 if d16 else tol)
    A, B = gk.bf16_values(a), gk.bf16_values(b)
    C = gk.bf16_values(c) if d16 else c
    assert oracle.rel_frobenius(d, oracle.gemm_f64(A, B, C, 1.0, 1.0, ta, tb)) <= tol


def test_concurrent_launches_from_two_host_threads_on_two_streams(gpu):
    """The launcher is re-entrant: two host threads enqueue different GEMMs on their own streams."""
    import threading
    import torch
    results, errors = {}, []

    def worker(tag, M, N, K, ta, tb, seed):
        try:
            conf = make_config(M, N, K, ta, tb, (128, 128, 64), (2, 2))
            a, b, c = inputs(M, N, K, ta, tb, seed)
            A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
            D = gk.colmajor_empty((M, N), torch.float32)
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(20):
                    gk.matmul(conf, A, B, C, D, kernel=Kernel.matmul_pipelined)
            stream.synchronize()
            results[tag] = (gk.to_numpy(D), oracle.gemm_f64(a, b, c, 1.0, 1.0, ta, tb))
        except Exception as e:      # surfaced by the assertion below
            errors.append((tag, repr(e)))

    threads = [threading.Thread(target=worker, args=("x", 512, 256, 320, False, False, 3100)),
               threading.Thread(target=worker, args=("y", 256, 384, 192, True, True, 3200))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for tag, (d, ref) in results.items():
        assert oracle.rel_frobenius(d, ref) <= TOL, tag
