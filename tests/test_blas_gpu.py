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
@pytest.mark.parametrize("dims", [(1000, 1000, 1000), (840, 328, 200), (328, 1096, 136), (264, 264, 64)])
def test_products_cut_into_regions_of_whole_tiles(gpu, dims, ta, tb):
    """Sizes that are not whole tiles with 16-byte aligned columns: blocks of whole tiles on the fast
    kernels, rims and the tail of K on the bounds-checked kernel (matmatmul_plan).  Same tolerance as
    the single launch, and the same kernels must not be all bounds-checked ones."""
    from gemmkernels.matmul import matmatmul_plan, PlanSequence, output_regions
    M, N, K = dims
    a, b, c = operands(M, N, K, ta == "T", tb == "T", np.float16, 500)
    alpha, beta = 0.75, -1.5
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    p = matmatmul_plan(C, ta, tb, A, B, alpha, beta, regions=True)
    assert isinstance(p, PlanSequence)
    assert len(p.plans) == len(output_regions(M, N)) + (1 if K % 32 else 0)
    assert any("checked" not in n for n in p.kernel_names), p.kernel_names
    print("case", dims, ta, tb, p.kernel_names, flush=True)
    p()
    torch.cuda.synchronize()
    ref = oracle.gemm_f64(a, b, c, alpha, beta, ta == "T", tb == "T")
    assert oracle.rel_frobenius(gk.to_numpy(C), ref) <= 1e-3
    # the single bounds-checked launch gives the same values up to the order of the fp32 sums
    C1 = gk.colmajor(c)
    matmatmul_plan(C1, ta, tb, A, B, alpha, beta, regions=False)()
    torch.cuda.synchronize()
    assert oracle.rel_frobenius(gk.to_numpy(C), gk.to_numpy(C1).astype(np.float64)) <= 1e-5


def test_region_cutting_is_left_alone_where_it_cannot_help(gpu):
    from gemmkernels.matmul import matmatmul_plan, PlanSequence
    # whole tiles: one fast launch; columns that are not 16-byte aligned: one bounds-checked launch; FP32: vector ALUs
    for dims, dtype in (((1024, 1024, 1024), np.float16), ((1001, 1001, 1001), np.float16), ((1000, 1000, 1000), np.float32)):
        M, N, K = dims
        a, b, c = operands(M, N, K, False, False, dtype, 600)
        p = matmatmul_plan(gk.colmajor(c), "N", "N", gk.colmajor(a), gk.colmajor(b), 1.0, 1.0, regions=True)
        assert not isinstance(p, PlanSequence), dims


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("N", "T"), ("T", "N"), ("T", "T")])
@pytest.mark.parametrize("dims", [(1000, 1000, 1000), (840, 328, 192), (264, 72, 136)])
def test_products_that_do_not_read_c_need_no_rims(gpu, dims, ta, tb):
    """beta = 0 and M, N multiples of 8: the ragged edges are covered by whole tiles that reach back over
    finished cells; nothing runs on the bounds-checked kernel."""
    from gemmkernels.matmul import matmatmul_plan, PlanSequence
    M, N, K = dims
    a, b, c = operands(M, N, K, ta == "T", tb == "T", np.float16, 700)
    A, B = gk.colmajor(a), gk.colmajor(b)
    C = gk.colmajor(np.asfortranarray(np.full((M, N), np.nan, np.float32)))       # never read
    p = matmatmul_plan(C, ta, tb, A, B, 1.25, 0.0, regions=True)
    assert isinstance(p, PlanSequence)
    assert not any("checked" in n for n in p.kernel_names), p.kernel_names     # the tail of K is a partial tile of the aligned kernel
    p()
    torch.cuda.synchronize()
    ref = oracle.gemm_f64(a, b, None, 1.25, 0.0, ta == "T", tb == "T")
    assert oracle.rel_frobenius(gk.to_numpy(C), ref) <= 1e-3


@pytest.mark.parametrize("beta", [0.0, 0.25])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_cut_up_products_with_16_bit_c(gpu, beta, dtype):
    """FP16 A, B and C, and BF16 A, B with Float32 C, through the region cutting: rims (beta != 0) and
    overlapping windows (beta = 0)."""
    from gemmkernels.matmul import matmatmul_plan, PlanSequence
    M, N, K = 1000, 200, 104
    a, b, c = operands(M, N, K, False, True, np.float16, 800)
    if dtype == "f16":
        A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c.astype(np.float16))
        c_in = c.astype(np.float16).astype(np.float64)
    else:
        A, B = gk.colmajor(a, dtype=torch.bfloat16), gk.colmajor(b, dtype=torch.bfloat16)
        C = gk.colmajor(c)                                                        # BF16 inputs pair with a Float32 C
        a, b = A.float().cpu().numpy(), B.float().cpu().numpy()                  # the values after rounding to BF16
        c_in = c.astype(np.float64)
    p = matmatmul_plan(C, "N", "T", A, B, 0.5, beta, regions=True)
    assert isinstance(p, PlanSequence), type(p)
    p()
    torch.cuda.synchronize()
    out = C.float().cpu().numpy()
    ref = 0.5 * a.astype(np.float64) @ b.astype(np.float64).T + beta * c_in
    assert oracle.rel_frobenius(out, ref) <= 2e-3       # FP16 C: one rounding of D to 11 bits; BF16: alpha on A in BF16
