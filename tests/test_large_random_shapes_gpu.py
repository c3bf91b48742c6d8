"""mul!(C, A, B, alpha, beta) at random extents around 4000, where the default plan picks the large tiles: whole 256 x 256
tiles with K long enough for C to arrive during the first K tiles, multiples of 8 and any extents (tiles over the edges, a
partial last K tile), and multiples of 192 (the tiles with a side of 192), every transpose, alpha in {1, 0.5} and beta in
{0, 1} (alpha = 0.5 folds into the accumulators where there is no C and runs the kernels with hooks next to one).  Each
result is compared with the float64 product of the CPU oracle on a slab of 384 columns (relative Frobenius error <= 1e-3,
the tolerance of FP16 multiplicands with FP32 accumulation) and checked for values that were never written; the sizes
follow reference test/blas.jl:12-20 (every transpose, sizes that are not whole tiles) at the scale of the benchmark."""
import numpy as np
import pytest

import gemmkernels as gk
from gemmkernels import rng
from gemmkernels.matmul import matmatmul_plan
from oracle import oracle

pytestmark = pytest.mark.gpu


def extents(kind, rs):
    if kind == "whole tiles":
        return 256 * int(rs.randint(14, 19)), 256 * int(rs.randint(14, 19)), 64 * int(rs.randint(11, 60))
    if kind == "multiples of 8":
        return 8 * int(rs.randint(480, 560)), 8 * int(rs.randint(480, 560)), 8 * int(rs.randint(90, 500))
    if kind == "any extents":
        return int(rs.randint(3900, 4500)), int(rs.randint(3900, 4500)), int(rs.randint(700, 3000))
    return 192 * int(rs.randint(14, 24)), 192 * int(rs.randint(14, 24)), 64 * int(rs.randint(11, 50))


@pytest.mark.parametrize("kind", ["whole tiles", "multiples of 8", "any extents", "multiples of 192"])
@pytest.mark.parametrize("seed", [1, 2, 3])
def test_mul_at_random_large_extents(gpu, kind, seed):
    import torch
    rs = np.random.RandomState(1000 * seed + len(kind))
    M, N, K = extents(kind, rs)
    ta, tb = bool(rs.randint(2)), bool(rs.randint(2))
    alpha, beta = float(rs.choice([1.0, 1.0, 0.5])), float(rs.choice([0.0, 1.0, 1.0]))
    a = rng.matrix("upm1_f16", 9100 + seed, (K, M) if ta else (M, K))
    b = rng.matrix("upm1_f16", 9200 + seed, (N, K) if tb else (K, N))
    c = rng.matrix("upm1_f32", 9300 + seed, (M, N))
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    plan = matmatmul_plan(C, "T" if ta else "N", "T" if tb else "N", A, B, alpha, beta)
    print("case", kind, (M, N, K), ta, tb, alpha, beta, plan.kernel_names, flush=True)
    plan()
    torch.cuda.synchronize()
    d = gk.to_numpy(C)
    assert not np.isnan(d).any()
    j0 = int(rs.randint(0, N - 384))
    bs = np.asfortranarray(b[j0:j0 + 384, :] if tb else b[:, j0:j0 + 384])
    ref = oracle.gemm_f64(a, bs, np.asfortranarray(c[:, j0:j0 + 384]), alpha, beta, ta, tb)
    assert oracle.rel_frobenius(d[:, j0:j0 + 384], ref) <= 1e-3
