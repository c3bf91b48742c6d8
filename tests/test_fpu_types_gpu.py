"""GPU parity of the vector-ALU operator for every element-type triple the reference runs FPUOp with
(configs/configs.jl:489-497: Float16/Float32 -> Float32, Float32 -> Float64, Float64, Int16, Int32,
Int64), alpha = 2 and beta = 3 as there (configs/configs.jl:193-194).  One sequential fma chain per
output in ascending k (src/operator.jl:139-153), so the results are bit-identical to the oracle's."""
import numpy as np
import pytest
import torch

import gemmkernels as gk
from gemmkernels import Layout, Operator, Kernel, NT, Transform, rng
from gemmkernels import Float16, Float32, Float64, Int16, Int32, Int64
import helpers
from oracle import oracle

pytestmark = pytest.mark.gpu

TRIPLES = [  # (A and B, C and D, numpy in, numpy out)
    (Float16, Float32, np.float16, np.float32),
    (Float32, Float32, np.float32, np.float32),
    (Float32, Float64, np.float32, np.float64),
    (Float64, Float64, np.float64, np.float64),
    (Int16, Int16, np.int16, np.int16),
    (Int32, Int32, np.int32, np.int32),
    (Int64, Int64, np.int64, np.int64),
]
IDS = [f"{t[0]}-{t[1]}" for t in TRIPLES]
TORCH = {np.float16: torch.float16, np.float32: torch.float32, np.float64: torch.float64,
         np.int16: torch.int16, np.int32: torch.int32, np.int64: torch.int64}


def operand(shape, np_t, seed):
    if np.issubdtype(np_t, np.integer):
        hi = {2: 300, 4: 70000, 8: 2 ** 40}[np.dtype(np_t).itemsize]        # large enough to wrap Int16 / Int32
        return np.asfortranarray(np.random.RandomState(seed).randint(-hi, hi, size=shape).astype(np_t))
    kind = "upm1_f16" if np_t == np.float16 else "upm1_f32"
    x = rng.matrix(kind, seed, shape)
    if np_t == np.float64:       # full 53-bit mantissas
        x = np.asfortranarray(x.astype(np.float64) + np.random.RandomState(seed).standard_normal(shape) * 1e-9)
    return np.asfortranarray(x.astype(np_t))


def config(M, N, K, ta, tb, AB, CD, aligned=True):
    col = Layout.UnsafeAlignedColMajor if aligned else Layout.ColMajor
    row = Layout.UnsafeAlignedRowMajor if aligned else Layout.RowMajor
    return gk.get_config(gemm_shape=NT(M=M, N=N, K=K), block_shape=NT(M=64, N=64, K=32),
                         operator=Operator.FPUOp[8, 8, 1, 8, 8, 1, AB, CD],
                         global_a_layout=(row if ta else col)[AB], global_b_layout=(row if tb else col)[AB],
                         global_c_layout=col[CD], global_d_layout=col[CD], is_a_col_major=not ta, is_b_col_major=not tb)


ALPHA_BETA = dict(transform_shared_to_regs_a=Transform.Elementwise(lambda x: x * 2),
                  transform_shared_to_regs_c=Transform.Elementwise(lambda x: x * 3))


@pytest.mark.parametrize("AB,CD,np_in,np_out", TRIPLES, ids=IDS)
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_type_triples_all_transposes(gpu, AB, CD, np_in, np_out, ta, tb):
    M, N, K = 128, 192, 96
    conf = config(M, N, K, ta, tb, AB, CD)
    a = operand((K, M) if ta else (M, K), np_in, 11)
    b = operand((N, K) if tb else (K, N), np_in, 12)
    c = operand((M, N), np_out, 13)
    print("case", AB, CD, ta, tb, gk.kernel_name(conf, Kernel.matmul_pipelined), flush=True)
    d = helpers.run_gpu(conf, a, b, c, (M, N), d_dtype=TORCH[np_out], transforms=ALPHA_BETA, kernel=Kernel.matmul_pipelined)
    ref = helpers.run_oracle(conf, a, b, c, (M, N), d_dtype=np_out, transforms=ALPHA_BETA)
    assert d.dtype == np_out
    assert np.array_equal(d, ref)
    if np.issubdtype(np_out, np.integer):
        # exact arithmetic modulo 2^bits (int64 matmul wraps the same way for every narrower type)
        A, B = (a.T if ta else a).astype(np.int64), (b.T if tb else b).astype(np.int64)
        with np.errstate(over="ignore"):
            exact = (2 * A) @ B + 3 * c.astype(np.int64)
        assert np.array_equal(d, exact.astype(np_out))
    else:
        ref64 = oracle.gemm_f64(a, b, c, 2.0, 3.0, ta, tb)
        assert oracle.rel_frobenius(d, ref64) <= (1e-5 if np_out == np.float32 and np_in == np.float32 else 1e-3 if np_in == np.float16 else 1e-12)


@pytest.mark.parametrize("AB,CD,np_in,np_out", [TRIPLES[2], TRIPLES[3], TRIPLES[5]], ids=[IDS[2], IDS[3], IDS[5]])
def test_bounds_checked_sizes(gpu, AB, CD, np_in, np_out):
    """Sizes that are multiples of no tile go through Layout.ColMajor / RowMajor (src/layout.jl:117-184)."""
    M, N, K = 100, 36, 50
    conf = config(M, N, K, True, False, AB, CD, aligned=False)
    a, b, c = operand((K, M), np_in, 21), operand((K, N), np_in, 22), operand((M, N), np_out, 23)
    d = helpers.run_gpu(conf, a, b, c, (M, N), d_dtype=TORCH[np_out], transforms=ALPHA_BETA, kernel=Kernel.matmul_singlestage)
    ref = helpers.run_oracle(conf, a, b, c, (M, N), d_dtype=np_out, transforms=ALPHA_BETA)
    assert np.array_equal(d, ref)


@pytest.mark.parametrize("np_t", [np.float64, np.int32, np.int64])
def test_blas_entry_points(gpu, np_t):
    """mul! / matmatmul! on Float64 and integer CuArrays (reference src/matmul.jl:85-119 picks FPUOp)."""
    M, N, K = 256, 128, 64
    a, b, c = operand((M, K), np_t, 31), operand((N, K), np_t, 32), operand((M, N), np_t, 33)
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    gk.matmatmul_(C, "N", "T", A, B, 2, 3)
    torch.cuda.synchronize()
    out = gk.to_numpy(C)
    if np.issubdtype(np_t, np.integer):
        with np.errstate(over="ignore"):
            exact = (2 * a.astype(np.int64)) @ b.T.astype(np.int64) + 3 * c.astype(np.int64)
        assert np.array_equal(out, exact.astype(np_t))
    else:
        assert oracle.rel_frobenius(out, 2.0 * (a @ b.T) + 3.0 * c) <= 1e-13
