"""GPU parity of the BLAS-like entry points (matmatmul_ / mul_), in the manner of the reference's
test/blas.jl:11-68: sizes that are not multiples of any tile (10, 1000) next to 128 / 256, all four
transposes, random alpha and beta, the matrix cores for FP16 inputs and the vector ALUs for FP32."""
import numpy as np
import pytest
import torch

import gemmkernels as gk
from gemmkernels import Transpose, configs, rng
from gemmkernels.matmul import create_config
from gemmkernels.dtypes import Float16, Float32
import helpers
from oracle import oracle

pytestmark = pytest.mark.gpu


def operands(M, N, K, ta, tb, dtype, seed):
    kind = "upm1_f16" if dtype == np.float16 else "upm1_f32"
    a = rng.matrix(kind, seed + 1, (K, M) if ta else (M, K)).astype(dtype)
    b = rng.matrix(kind, seed + 2, (N, K) if tb else (K, N)).astype(dtype)
    c = rng.matrix("upm1_f32", seed + 3, (M, N))
    return a, b, c


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("N", "T"), ("T", "N"), ("T", "T")])
@pytest.mark.parametrize("dims", [(10, 10, 10), (128, 128, 128), (256, 256, 256), (1000, 1000, 1000), (10, 1000, 256), (130, 70, 33)])
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_matmatmul(gpu, dims, ta, tb, dtype):
    M, N, K = dims
    a, b, c = operands(M, N, K, ta == "T", tb == "T", dtype, 100)
    rs = np.random.RandomState(M + N)
    alpha, beta = float(np.float16(rs.rand())), float(np.float32(rs.rand()))      # reference test/blas.jl:22-23
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    print("case", dims, ta, tb, dtype.__name__, flush=True)
    gk.matmatmul_(C, ta, tb, A, B, alpha, beta)
    torch.cuda.synchronize()
    ref = oracle.gemm_f64(a, b, c, alpha, beta, ta == "T", tb == "T")
    err = oracle.rel_frobenius(gk.to_numpy(C), ref)
    # FP16: alpha is applied to A in FP16 like the reference does (src/matmul.jl:196-199), which
    # rounds every scaled element: 2^-11 relative per element, averaged down by the sum
    assert err <= (1e-3 if dtype == np.float16 else 1e-5), err


# (A / B type, C type, min_dimension, tolerance) -- the three type rows of reference test/blas.jl:15 and :43; the
# reference's own tolerance is the norm-wise sqrt(eps(AB_type)) (0.031 for Float16, 3.5e-4 for Float32)
_CUBE_ROWS = {"f16_f16": (np.float16, np.float16, 256, 2e-3), "f16_f32": (np.float16, np.float32, 128, 1e-3),
              "f32_f32": (np.float32, np.float32, 128, 1e-5)}


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("N", "T"), ("T", "N"), ("T", "T")])
@pytest.mark.parametrize("row", sorted(_CUBE_ROWS))
def test_the_reference_cube_of_sizes(gpu, row, ta, tb):
    """reference test/blas.jl:11-67 in full: M, N, K each from {10, min_dimension, 1000} (27 shapes) for every
    transpose pair and type row, A and B ~ U[0,1) / sqrt(K), random alpha (in the A / B type) and beta (in the C
    type), through matmatmul_ with wmma = true for the Float16 rows and false for the Float32 row."""
    ab_t, c_t, min_dim, tol = _CUBE_ROWS[row]
    rs = np.random.RandomState(hash((row, ta, tb)) % (2 ** 31))
    worst = 0.0
    for M in (10, min_dim, 1000):
        for N in (10, min_dim, 1000):
            for K in (10, min_dim, 1000):
                a = np.asfortranarray((rs.rand(*((K, M) if ta == "T" else (M, K))) / np.sqrt(K)).astype(ab_t))
                b = np.asfortranarray((rs.rand(*((N, K) if tb == "T" else (K, N))) / np.sqrt(K)).astype(ab_t))
                c = np.asfortranarray(rs.rand(M, N).astype(c_t))
                alpha, beta = float(ab_t(rs.rand())), float(c_t(rs.rand()))
                C = gk.colmajor(c)
                gk.matmatmul_(C, ta, tb, gk.colmajor(a), gk.colmajor(b), alpha, beta, wmma=(ab_t == np.float16))
                torch.cuda.synchronize()
                err = oracle.rel_frobenius(gk.to_numpy(C), oracle.gemm_f64(a, b, c, alpha, beta, ta == "T", tb == "T"))
                worst = max(worst, err)
                assert err <= tol, (row, ta, tb, (M, N, K), err)
    print("cube", row, ta, tb, "worst relative error", worst, flush=True)


@pytest.mark.parametrize("dims", [(256, 256, 256), (1000, 200, 72)])
def test_matmatmul_f16_output(gpu, dims):
    """FP16 A, B and C (reference test/blas.jl:15, the (Float16, Float16, Float16) row): FP32
    accumulation on the matrix cores, beta in FP16, one rounding at the store."""
    M, N, K = dims
    a, b, c = operands(M, N, K, False, True, np.float16, 300)
    c = c.astype(np.float16)
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    gk.matmatmul_(C, "N", "T", A, B, 0.5, 0.25)
    torch.cuda.synchronize()
    out = gk.to_numpy(C)
    assert out.dtype == np.float16
    assert oracle.rel_frobenius(out, oracle.gemm_f64(a, b, c, 0.5, 0.25, False, True)) <= 1e-3


def test_fp32_is_bit_exact_against_the_sequential_fma_chain(gpu):
    """FPUOp semantics: one fp32 fma per k in ascending order (reference src/operator.jl:139-153);
    the oracle's C restatement is that loop, so the results must be identical."""
    for (M, N, K, ta, tb) in [(256, 256, 256, False, False), (64, 192, 96, True, False), (100, 36, 50, False, True), (77, 65, 129, True, True)]:
        a, b, c = operands(M, N, K, ta, tb, np.float32, 7)
        sa, sb = a.shape, b.shape
        conf, _, kern = create_config(Float32, sa, (1, sa[0]), ta, Float32, sb, (1, sb[0]), tb, Float32, (M, N), (1, M),
                                      float, False, float, False, None)
        d = helpers.run_gpu(conf, a, b, c, (M, N), kernel=kern)
        ref = helpers.run_oracle(conf, a, b, c, (M, N))
        assert np.array_equal(d, ref), (M, N, K, ta, tb)


def test_mul_wrappers_and_zero_alpha(gpu):
    M, N, K = 128, 64, 96
    a, b, c = operands(M, N, K, True, False, np.float16, 9)
    A, B = gk.colmajor(a), gk.colmajor(b)
    C = gk.colmajor(np.asfortranarray(np.full((M, N), np.nan, np.float32)))
    gk.mul_(C, Transpose(A), B)                           # alpha = true, beta = false: C is never read
    torch.cuda.synchronize()
    assert oracle.rel_frobenius(gk.to_numpy(C), oracle.gemm_f64(a, b, None, 1.0, 0.0, True, False)) <= 1e-3
    C = gk.colmajor(c)
    gk.matmatmul_(C, "T", "N", A, B, 0.0, 2.0)            # alpha = 0: A and B are Layout.Zero, C = 2 C exactly
    torch.cuda.synchronize()
    assert np.array_equal(gk.to_numpy(C), 2.0 * c)
    with pytest.raises(gk.DimensionMismatch):
        gk.matmatmul_(C, "N", "N", A, B, 1.0, 0.0)


def test_tropical(gpu):
    """max-plus product on the vector ALUs (reference src/operator.jl:134-137, configs/configs.jl:209-244)."""
    from gemmkernels import Layout, Operator, Kernel, NT
    M, N, K = 128, 128, 64
    a, b, c = operands(M, N, K, False, False, np.float32, 11)
    conf = gk.get_config(gemm_shape=NT(M=M, N=N, K=K), block_shape=NT(M=64, N=64, K=32),
                         operator=Operator.TropicalFPUOp[8, 8, 1, 8, 8, 1, Float32, Float32],
                         global_a_layout=Layout.UnsafeAlignedColMajor[Float32], global_c_layout=Layout.UnsafeAlignedColMajor[Float32])
    d = helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    want = np.maximum(c, (a[:, :, None] + b[None, :, :]).max(axis=1))
    assert np.array_equal(d, want)


def test_config1_benchmark_workload(gpu):
    w = configs.benchmark_config(1)
    run = w.prepare()
    run()
    torch.cuda.synchronize()
    h = w.host()
    d = gk.to_numpy(run.d)
    assert oracle.rel_frobenius(d, oracle.gemm_f64(h["a"], h["b"], None)) <= 1e-5
    conf = run.conf
    assert np.array_equal(d, helpers.run_oracle(conf, h["a"], h["b"], None, (256, 256)))


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("N", "T"), ("T", "N"), ("T", "T")])
@pytest.mark.parametrize("dims", [(1000, 1000, 1000), (1001, 1001, 1001), (841, 329, 203), (327, 1097, 139), (265, 263, 65), (9, 8, 8)])
def test_any_size_is_one_launch_of_an_aligned_kernel(gpu, dims, ta, tb):
    """Sizes that are not whole tiles, not multiples of 8, with odd leading dimensions: still one launch of the
    aligned kernels (the reference would run them on its bounds-checked layouts, src/matmul.jl:121-156)."""
    from gemmkernels.matmul import matmatmul_plan
    M, N, K = dims
    a, b, c = operands(M, N, K, ta == "T", tb == "T", np.float16, 500)
    alpha, beta = 0.75, -1.5
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    p = matmatmul_plan(C, ta, tb, A, B, alpha, beta)
    assert len(p.kernel_names) == 1 and "checked" not in p.kernel_names[0], p.kernel_names
    print("case", dims, ta, tb, p.kernel_names, flush=True)
    p()
    torch.cuda.synchronize()
    ref = oracle.gemm_f64(a, b, c, alpha, beta, ta == "T", tb == "T")
    assert oracle.rel_frobenius(gk.to_numpy(C), ref) <= 1e-3


def test_operands_with_less_than_a_chunk_along_their_contiguous_index_run_bounds_checked(gpu):
    from gemmkernels.matmul import matmatmul_plan
    for M, N, K, ta, tb in ((5, 40, 64, "N", "N"), (40, 40, 4, "N", "N"), (40, 3, 64, "N", "T")):
        a, b, c = operands(M, N, K, ta == "T", tb == "T", np.float16, 600)
        C = gk.colmajor(c)
        p = matmatmul_plan(C, ta, tb, gk.colmajor(a), gk.colmajor(b), 1.0, 1.0)
        assert "checked" in p.kernel_names[0], p.kernel_names
        p()
        torch.cuda.synchronize()
        assert oracle.rel_frobenius(gk.to_numpy(C), oracle.gemm_f64(a, b, c, 1.0, 1.0, ta == "T", tb == "T")) <= 1e-3


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "T")])
def test_views_that_start_off_a_16_byte_boundary(gpu, ta, tb):
    """A[1:M+1, :] of a larger array has aligned strides and a misaligned first element: the operand gets the
    bounds-checked layout and the product still runs on the aligned kernel (1000^3 and a small one)."""
    from gemmkernels.matmul import matmatmul_plan
    for M, N, K in ((1000, 1000, 1000), (200, 136, 96)):
        a, b, c = operands(M, N, K, ta == "T", tb == "T", np.float16, 650)
        big_a = np.zeros((a.shape[0] + 8, a.shape[1]), np.float16, order="F"); big_a[1:a.shape[0] + 1, :] = a
        big_b = np.zeros((b.shape[0] + 8, b.shape[1]), np.float16, order="F"); big_b[1:b.shape[0] + 1, :] = b
        A = gk.colmajor(big_a)[1:a.shape[0] + 1, :]
        B = gk.colmajor(big_b)[1:b.shape[0] + 1, :]
        assert A.data_ptr() % 16 == 2 and B.data_ptr() % 16 == 2
        C = gk.colmajor(c)
        p = matmatmul_plan(C, ta, tb, A, B, 1.0, 0.5)
        assert "checked" not in p.kernel_names[0], p.kernel_names
        p()
        torch.cuda.synchronize()
        assert oracle.rel_frobenius(gk.to_numpy(C), oracle.gemm_f64(a, b, c, 1.0, 0.5, ta == "T", tb == "T")) <= 1e-3


@pytest.mark.parametrize("beta", [0.0, 0.25])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_odd_sizes_with_16_bit_c(gpu, beta, dtype):
    """FP16 A, B and C, and BF16 A, B with Float32 C, on sizes that are not multiples of 8."""
    from gemmkernels.matmul import matmatmul_plan
    M, N, K = 1001, 203, 107
    a, b, c = operands(M, N, K, False, True, np.float16, 800)
    if dtype == "f16":
        A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c.astype(np.float16))
        c_in = c.astype(np.float16).astype(np.float64)
    else:
        A, B = gk.colmajor(a, dtype=torch.bfloat16), gk.colmajor(b, dtype=torch.bfloat16)
        C = gk.colmajor(c)                                                        # BF16 inputs pair with a Float32 C
        a, b = A.float().cpu().numpy(), B.float().cpu().numpy()                  # the values after rounding to BF16
        c_in = c.astype(np.float64)
    p = matmatmul_plan(C, "N", "T", A, B, 0.5, beta)
    assert "checked" not in p.kernel_names[0], p.kernel_names
    p()
    torch.cuda.synchronize()
    out = C.float().cpu().numpy()
    ref = 0.5 * a.astype(np.float64) @ b.astype(np.float64).T + beta * c_in
    assert oracle.rel_frobenius(out, ref) <= 2e-3       # FP16 C: one rounding of D to 11 bits; BF16: alpha on A in BF16


@pytest.mark.parametrize("ta,tb", [(False, False), (True, True)])
def test_fpu_operator_shapes(gpu, ta, tb):
    """The operator-shape sweep of the reference (configs/configs.jl:521-551) on 64-lane waves: operator shapes that
    are multiples of the 8 x 8 lane grid run and give, bit for bit, the sequential fma chain (the shape only says
    which lane owns which output); the other lane grids run on the tile they are compiled for, see below."""
    from gemmkernels import Kernel, Layout, NT, Operator
    M = N = K = 128
    a, b, c = operands(M, N, K, ta, tb, np.float32, 900)
    la = Layout.UnsafeAlignedRowMajor[Float32] if ta else Layout.UnsafeAlignedColMajor[Float32]
    lb = Layout.UnsafeAlignedRowMajor[Float32] if tb else Layout.UnsafeAlignedColMajor[Float32]
    def conf_for(shape, block):
        return gk.get_config(gemm_shape=NT(M=M, N=N, K=K), block_shape=NT(M=block[0], N=block[1], K=block[2]),
                             operator=Operator.FPUOp[(*shape, Float32, Float32)], global_a_layout=la, global_b_layout=lb,
                             global_c_layout=Layout.UnsafeAlignedColMajor[Float32], global_d_layout=Layout.UnsafeAlignedColMajor[Float32],
                             is_a_col_major=not ta, is_b_col_major=not tb)
    ref = None
    for shape in [(8, 8, 1, 8, 8, 1), (16, 8, 1, 8, 8, 1), (8, 16, 1, 8, 8, 1), (8, 8, 2, 8, 8, 1), (16, 16, 2, 8, 8, 1)]:
        for block in ((64, 64, 32), (32, 32, 32)):
            conf = conf_for(shape, block)
            d = helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
            if ref is None:
                ref = helpers.run_oracle(conf, a, b, c, (M, N))
            assert np.array_equal(d, ref), (shape, block)
    # The other lane grids of the reference's sweep (base shapes 1 x 32 ... 32 x 1 there, 1 x 64 ... 64 x 1 on 64 lanes) run on the
    # 128 x 128 x 16 tile, whose 64 x 64 wave tiles every grid divides: which lane owns which output changes, the fma chain of
    # an output does not -- same bits as the oracle.  On other tiles they are refused with the operator-shape error, not replaced.
    grids = [(4, 64, 1, 1, 64, 1), (4, 32, 1, 2, 32, 1), (16, 16, 1, 4, 16, 1), (16, 16, 1, 16, 4, 1), (32, 4, 1, 32, 2, 1), (64, 4, 1, 64, 1, 1)]
    for shape in grids:
        conf = gk.get_config(gemm_shape=NT(M=M, N=N, K=K), block_shape=NT(M=128, N=128, K=16), warps_per_block=4,
                             compute_warp=NT(M=64, N=64, K=shape[2]),
                             operator=Operator.FPUOp[(*shape, Float32, Float32)], global_a_layout=la, global_b_layout=lb,
                             global_c_layout=Layout.UnsafeAlignedColMajor[Float32], global_d_layout=Layout.UnsafeAlignedColMajor[Float32],
                             is_a_col_major=not ta, is_b_col_major=not tb)
        name = gk.kernel_name(conf, Kernel.matmul_pipelined)
        print("lane grid", shape[3], "x", shape[4], name, flush=True)
        assert f"lanes{shape[3]}x{shape[4]}" in name
        d = helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
        assert np.array_equal(d, ref), shape
        # ... with hooks: scale on A, bias per column, ReLU on D
        from gemmkernels import Epilogue, Transform
        hooks = dict(transform_shared_to_regs_a=Transform.Elementwise(lambda x: x * 0.75), transform_shared_to_global_d=Transform.Elementwise(Transform.relu))
        bias = rng.matrix("upm1_f32", 905, (N, 1))[:, 0] * 30
        dh = helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_pipelined, transforms=hooks, epilogue_cls=Epilogue.Bias, bias=bias)
        assert np.array_equal(dh, helpers.run_oracle(conf, a, b, c, (M, N), transforms=hooks, epilogue=Epilogue.Bias(0), bias=bias)), shape
    for shape in grids:
        with pytest.raises(gk.ConfigError) as ei:
            conf = conf_for(shape, (128, 128, 32))
            helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
        assert ei.value.status == _lib_status_op_shape(), shape


def _lib_status_op_shape():
    from gemmkernels import _lib
    return _lib.GK_ERR_OP_SHAPE
