"""The K-split kernel kind: few output tiles, long K.  Partial sums of the K slices are added into D
with fp32 atomics, so the comparison is by norm (and the last bits may differ between runs)."""
import numpy as np
import pytest
import torch

import gemmkernels as gk
from gemmkernels import Epilogue, Kernel, Transform, configs, rng, _lib
from oracle import oracle

pytestmark = pytest.mark.gpu
TOL = 1e-3


def operands(M, N, K, ta, tb, seed):
    a = rng.matrix("upm1_f16", seed + 1, (K, M) if ta else (M, K))
    b = rng.matrix("upm1_f16", seed + 2, (N, K) if tb else (K, N))
    c = rng.matrix("upm1_f32", seed + 3, (M, N))
    return a, b, c


@pytest.mark.parametrize("dims,block", [((4096, 64, 4096), (64, 64, 64)), ((64, 4096, 2048), (64, 64, 64)), ((256, 256, 8192), (128, 128, 64)),
                                        ((128, 128, 1088), (64, 64, 64))])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, True)])
def test_skinny_products(gpu, dims, block, ta, tb):
    M, N, K = dims
    conf = configs.mfma_config(M, N, K, ta, tb, block_shape=block)
    a, b, c = operands(M, N, K, ta, tb, 4000)
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    D = gk.colmajor_empty((M, N), torch.float32)
    D.fill_(float("nan"))
    gk.matmul(conf, A, B, C, D, kernel=Kernel.matmul_split_k)
    torch.cuda.synchronize()
    ref = oracle.gemm_f64(a, b, c, 1.0, 1.0, ta, tb)
    assert oracle.rel_frobenius(gk.to_numpy(D), ref) <= TOL
    # d aliases c (mul! style), with hooks on A and C: C is read by the first slice only
    gk.matmul(conf, A, B, C, C, kernel=Kernel.matmul_split_k, transform_shared_to_regs_a=Transform.Elementwise(lambda x: x * 0.5),
              transform_shared_to_regs_c=Transform.Elementwise(lambda x: x * 3.0))
    torch.cuda.synchronize()
    ref2 = oracle.gemm_f64(a, b, c, 0.5, 3.0, ta, tb)
    assert oracle.rel_frobenius(gk.to_numpy(C), ref2) <= TOL


@pytest.mark.parametrize("dims,block", [((4096, 64, 4096), (64, 64, 64)), ((256, 256, 8192), (128, 128, 64))])
def test_in_place_with_an_untouched_c_is_one_launch_of_atomic_adds(gpu, dims, block):
    """C = A*B + C in place (mul!(C, A, B, 1, 1)): D already holds C, every K slice adds into it."""
    M, N, K = dims
    conf = configs.mfma_config(M, N, K, block_shape=block)
    a, b, c = operands(M, N, K, False, False, 4300)
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    gk.matmul(conf, A, B, C, C, kernel=Kernel.matmul_split_k)
    torch.cuda.synchronize()
    assert oracle.rel_frobenius(gk.to_numpy(C), oracle.gemm_f64(a, b, c, 1.0, 1.0, False, False)) <= TOL
    # a second product on top, with a scale on A (the hook applies in every slice)
    gk.matmul(conf, A, B, C, C, kernel=Kernel.matmul_split_k, transform_shared_to_regs_a=Transform.Elementwise(lambda x: x * -2.0))
    torch.cuda.synchronize()
    ref = oracle.gemm_f64(a, b, c, 1.0, 1.0, False, False) + oracle.gemm_f64(a, b, None, -2.0, 0.0, False, False)
    assert oracle.rel_frobenius(gk.to_numpy(C), ref) <= TOL


def test_what_the_k_split_kernel_refuses(gpu):
    M, N, K = 128, 128, 2048
    conf = configs.mfma_config(M, N, K, block_shape=(64, 64, 64))
    a, b, c = operands(M, N, K, False, False, 4100)
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    D = gk.colmajor_empty((M, N), torch.float32)
    with pytest.raises(gk.ConfigError) as ei:          # a transform on D would see partial sums
        gk.matmul(conf, A, B, C, D, kernel=Kernel.matmul_split_k, transform_shared_to_global_d=Transform.Elementwise(Transform.relu))
    assert ei.value.status == _lib.GK_ERR_UNSUPPORTED
    bias = torch.zeros(N, device="cuda")
    with pytest.raises(gk.ConfigError):
        gk.matmul(conf, A, B, C, D, kernel=Kernel.matmul_split_k, epilogue=Epilogue.Bias(bias))


def test_blas_entry_picks_the_k_split_kernel_for_skinny_products(gpu):
    M, N, K = 2048, 64, 4096
    a, b, c = operands(M, N, K, False, False, 4200)
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    gk.matmatmul_(C, "N", "N", A, B, 0.5, 2.0)
    torch.cuda.synchronize()
    assert oracle.rel_frobenius(gk.to_numpy(C), oracle.gemm_f64(a, b, c, 0.5, 2.0)) <= TOL


@pytest.mark.parametrize("beta", [1.0, 0.5, 0.0])
def test_skinny_products_with_tiles_over_the_edge_are_split_too(gpu, beta):
    """N = 100 columns of a K x N B (contiguous along k, so any N is fine), M a multiple of 8 that is not a
    whole number of tiles, K whole tiles: the K-split instances mask the tiles over the edge; in place with
    beta = 1 it is one launch of atomic adds."""
    import torch
    from gemmkernels import rng
    from gemmkernels.matmul import matmatmul_plan
    from oracle import oracle
    M, N, K = 1000, 100, 4096
    a = rng.matrix("upm1_f16", 8101, (M, K)); b = rng.matrix("upm1_f16", 8102, (K, N)); c = rng.matrix("upm1_f32", 8103, (M, N))
    ld, cols = M + 8, N + 3
    full = gk.colmajor(np.asfortranarray(np.full((ld, cols), 555.0, np.float32)))
    C = full[:M, :N]
    C.copy_(gk.colmajor(c))
    p = matmatmul_plan(C, "N", "N", gk.colmajor(a), gk.colmajor(b), 1.0, beta)
    assert "checked" not in p.kernel_names[0], p.kernel_names
    p()
    torch.cuda.synchronize()
    out = full.cpu().numpy()
    assert (out[M:, :] == 555.0).all() and (out[:, N:] == 555.0).all()
    assert oracle.rel_frobenius(out[:M, :N], oracle.gemm_f64(a, b, c, 1.0, beta, False, False)) <= 1e-3
