"""GPU parity of the diagonal-A GEMM (benchmark config 4b, reference configs/configs.jl:331-383):
bit-exact against the closed form D[i,j] = fp32(a[i]) * fp32(B[i,j]) (+ C[i,j]) and against the oracle."""
import numpy as np
import pytest
import torch

import gemmkernels as gk
from gemmkernels import ConfigError, Epilogue, Kernel, Transform, configs, rng
import helpers
from oracle import oracle

pytestmark = pytest.mark.gpu
E = Transform.Elementwise


def run_diag(conf, a, b, c, d_shape, **kw):
    ta = torch.from_numpy(a).cuda()
    tb = gk.colmajor(b)
    tc = None if c is None else gk.colmajor(c)
    td = gk.colmajor_empty(d_shape, torch.float32)
    td.fill_(float("nan"))
    gk.matmul(conf, ta, tb, tc, td, kernel=Kernel.matmul_singlestage, **kw)
    torch.cuda.synchronize()
    return gk.to_numpy(td)


@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("zero_c", [True, False])
@pytest.mark.parametrize("M,N", [(256, 256), (512, 1024)])
def test_closed_form_bit_exact(gpu, M, N, tb, zero_c):
    conf = configs.diagonal_config(M, N, tb=tb, zero_c=zero_c)
    a = rng.uniform_pm1_f16(41, M)
    b = rng.matrix("upm1_f16", 42, (N, M) if tb else (M, N))
    c = None if zero_c else rng.matrix("upm1_f32", 43, (M, N))
    d = run_diag(conf, a, b, c, (M, N))
    B = b.T if tb else b
    prod = a.astype(np.float32)[:, None] * B.astype(np.float32)              # exact in fp32
    want = prod if zero_c else (prod.astype(np.float64) + c.astype(np.float64)).astype(np.float32)   # one rounding = fma
    assert np.array_equal(d, want)
    # the oracle runs the full sum over k with the Diagonal layout (reference src/layout.jl:225-236)
    ref = helpers.run_oracle(conf, a, np.asfortranarray(b), c, (M, N))
    assert np.array_equal(d, ref)
    # the reference's own check: mul!(Ch, Diagonal(Ah[1:M, 1]), Bh, true, true) (configs/configs.jl:358-365)
    dense = np.diag(a.astype(np.float64)) @ B.astype(np.float64) + (0 if zero_c else c.astype(np.float64))
    assert oracle.rel_frobenius(d, dense) <= 1e-6


def test_hooks_and_bias(gpu):
    M, N = 256, 384
    conf = configs.diagonal_config(M, N, zero_c=False)
    a, b, c = rng.uniform_pm1_f16(51, M), rng.matrix("upm1_f16", 52, (M, N)), rng.matrix("upm1_f32", 53, (M, N))
    bias = rng.normal_f32(54, N)
    tr = dict(transform_global_to_shared_a=E(lambda x: x * 0.5), transform_shared_to_regs_b=E(lambda x: -x),
              transform_shared_to_regs_c=E(lambda x: x * 3.0), transform_shared_to_global_d=E(Transform.relu))
    keep = torch.from_numpy(bias).cuda()
    d = run_diag(conf, a, b, c, (M, N), epilogue=Epilogue.Bias(keep), **tr)
    ref = helpers.run_oracle(conf, a, b, c, (M, N), transforms=tr, epilogue=Epilogue.Bias(0), bias=bias)
    assert np.array_equal(d, ref)
    with pytest.raises(ConfigError):      # x + 1 would turn the off-diagonal zeros into ones
        run_diag(conf, a, b, c, (M, N), transform_global_to_shared_a=E(lambda x: x + 1))


def test_config4b_full_size(gpu):
    w = configs.benchmark_config("4b")
    run = w.prepare()
    run()
    torch.cuda.synchronize()
    h = w.host()
    assert np.array_equal(gk.to_numpy(run.d), h["a"].astype(np.float32)[:, None] * h["b"].astype(np.float32))
