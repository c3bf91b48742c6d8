"""GPU parity of the fused transforms and epilogues (benchmark config 3 and the eight hooks of the
launcher) against the CPU oracle, which restates the reference's order of operations."""
import numpy as np
import pytest

import gemmkernels as gk
from gemmkernels import Epilogue, Kernel, Transform, configs, rng
import helpers
from oracle import oracle

pytestmark = pytest.mark.gpu
TOL = 1e-3
E = Transform.Elementwise


def small_inputs(M, N, K, seed):
    return (rng.matrix("upm1_f16", seed + 1, (M, K)), rng.matrix("upm1_f16", seed + 2, (K, N)),
            rng.matrix("upm1_f32", seed + 3, (M, N)))


def test_config3_reduced(gpu):
    M, N, K = 256, 384, 128
    conf = configs.mfma_config(M, N, K, zero_c=True, block_shape=(128, 128, 64))
    a, b, _ = small_inputs(M, N, K, 3000)
    bias = rng.normal_f32(3004, N)
    tr = dict(transform_global_to_shared_a=E(lambda x: x * 0.5), transform_shared_to_global_d=E(Transform.relu))
    d = helpers.run_gpu(conf, a, b, None, (M, N), transforms=tr, epilogue_cls=Epilogue.Bias, bias=bias, kernel=Kernel.matmul_pipelined)
    ref = helpers.run_oracle(conf, a, b, None, (M, N), transforms=tr, epilogue=Epilogue.Bias(0), bias=bias)
    assert oracle.rel_frobenius(d, ref) <= TOL
    # textbook form in float64
    ref64 = np.maximum(0.5 * a.astype(np.float64) @ b.astype(np.float64) + bias[None, :].astype(np.float64), 0.0)
    assert oracle.rel_frobenius(d, ref64) <= TOL
    assert (d >= 0).all()


def test_bias_only_closed_form(gpu):
    """A = 0  =>  D[i, j] = relu(bias[j]) exactly (per-column bias, reference src/epilogue.jl:44-52)."""
    M, N, K = 256, 256, 64
    conf = configs.mfma_config(M, N, K, zero_c=True, block_shape=(128, 128, 64))
    a = np.zeros((M, K), dtype=np.float16, order="F")
    b = rng.matrix("upm1_f16", 5, (K, N))
    bias = rng.normal_f32(6, N)
    tr = dict(transform_shared_to_global_d=E(Transform.relu))
    d = helpers.run_gpu(conf, a, b, None, (M, N), transforms=tr, epilogue_cls=Epilogue.Bias, bias=bias, kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d, np.broadcast_to(np.maximum(bias, 0)[None, :], (M, N)))
    # per-row variant
    bias_m = rng.normal_f32(7, M)
    d = helpers.run_gpu(conf, a, b, None, (M, N), transforms=tr, epilogue_cls=Epilogue.BiasRow, bias=bias_m, kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d, np.broadcast_to(np.maximum(bias_m, 0)[:, None], (M, N)))


def test_exact_scaling_and_relu_idempotence(gpu):
    M, N, K = 256, 256, 128
    a, b, _ = small_inputs(M, N, K, 40)
    conf = configs.mfma_config(M, N, K, zero_c=True, block_shape=(128, 128, 64))
    d1 = helpers.run_gpu(conf, a, b, None, (M, N), kernel=Kernel.matmul_pipelined)
    d2 = helpers.run_gpu(conf, a, b, None, (M, N), transforms=dict(transform_global_to_shared_a=E(lambda x: x * 0.5)), kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d2, 0.5 * d1)           # a power-of-two scale commutes with every rounding
    r1 = helpers.run_gpu(conf, a, b, None, (M, N), transforms=dict(transform_shared_to_global_d=E(Transform.relu)), kernel=Kernel.matmul_pipelined)
    r2 = helpers.run_gpu(conf, a, b, None, (M, N), transforms=dict(transform_regs_to_shared_d=E(Transform.relu), transform_shared_to_global_d=E(Transform.relu)), kernel=Kernel.matmul_pipelined)
    assert np.array_equal(r1, np.maximum(d1, 0)) and np.array_equal(r1, r2)


@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("block", [(256, 256, 64), (128, 128, 64), (64, 64, 32)])
def test_fp16_scales_on_a_and_b_equal_prescaled_operands_bit_for_bit(gpu, block, ta, tb):
    """A factor that is exact in FP16, on either operand or on both, is applied inside the K loop with one
    rounding to FP16 per element: the result equals, bit for bit, what the same tile computes from operands
    scaled (and rounded to FP16) beforehand.  Factors 1.5 and -0.375 are not powers of two, so the rounding
    of the scaled operand is visible."""
    BM, BN, BK = block
    M, N, K = 2 * BM, BN, 4 * BK
    conf = configs.mfma_config(M, N, K, ta, tb, block_shape=block)
    a = rng.matrix("upm1_f16", 71, (K, M) if ta else (M, K))
    b = rng.matrix("upm1_f16", 72, (N, K) if tb else (K, N))
    c = rng.matrix("upm1_f32", 73, (M, N))
    sa, sb = np.float16(1.5), np.float16(-0.375)
    a_s = np.asfortranarray((a.astype(np.float32) * np.float32(sa)).astype(np.float16))
    b_s = np.asfortranarray((b.astype(np.float32) * np.float32(sb)).astype(np.float16))
    cases = [(dict(transform_shared_to_regs_b=E(lambda x: x * -0.375)), a, b_s),
             (dict(transform_global_to_shared_a=E(lambda x: x * 1.5), transform_global_to_shared_b=E(lambda x: x * -0.375)), a_s, b_s),
             (dict(transform_shared_to_regs_a=E(lambda x: x * 1.5)), a_s, b)]
    for tr, a_ref, b_ref in cases:
        name = gk.kernel_name(conf, Kernel.matmul_pipelined, tr)
        assert name.endswith("_fused"), name        # the kernels with the packed FP16 multiply, not the per-element interpreter
        d = helpers.run_gpu(conf, a, b, c, (M, N), transforms=tr, kernel=Kernel.matmul_pipelined)
        want = helpers.run_gpu(conf, a_ref, b_ref, c, (M, N), kernel=Kernel.matmul_pipelined)
        assert np.array_equal(d, want), sorted(tr)


@pytest.mark.parametrize("ta,tb", [(False, False), (True, True)])
@pytest.mark.parametrize("block", [(256, 256, 64), (64, 64, 32)])
def test_power_of_two_scales_leave_the_k_loop_and_keep_every_bit(gpu, block, ta, tb):
    """A factor +-2^e on A or B commutes with every rounding, so the library runs the K loop of the plain kernel
    (instances `_fused_cd`), starts the accumulators from C / s and multiplies them by s at the end.  The result
    equals, bit for bit, the plain kernel on operands scaled beforehand (exact in FP16 for this data), with C."""
    BM, BN, BK = block
    M, N, K = 2 * BM, BN, 4 * BK
    conf = configs.mfma_config(M, N, K, ta, tb, block_shape=block)
    a = rng.matrix("upm1_f16", 74, (K, M) if ta else (M, K))
    b = rng.matrix("upm1_f16", 75, (N, K) if tb else (K, N))
    c = rng.matrix("upm1_f32", 76, (M, N))
    a_s = np.asfortranarray(a * np.float16(2.0))
    b_s = np.asfortranarray(b * np.float16(-0.25))
    cases = [(dict(transform_shared_to_regs_a=E(lambda x: x * 2.0)), a_s, b),
             (dict(transform_global_to_shared_b=E(lambda x: x * -0.25)), a, b_s),
             (dict(transform_global_to_shared_a=E(lambda x: x * 2.0), transform_shared_to_regs_b=E(lambda x: x * -0.25)), a_s, b_s)]
    for tr, a_ref, b_ref in cases:
        name = gk.kernel_name(conf, Kernel.matmul_pipelined, tr)
        assert name.endswith("_fused_cd"), name
        d = helpers.run_gpu(conf, a, b, c, (M, N), transforms=tr, kernel=Kernel.matmul_pipelined)
        want = helpers.run_gpu(conf, a_ref, b_ref, c, (M, N), kernel=Kernel.matmul_pipelined)
        assert np.array_equal(d, want), sorted(tr)
        ref = helpers.run_oracle(conf, a, b, c, (M, N), transforms=tr)
        assert oracle.rel_frobenius(d, ref) <= TOL


@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_all_eight_hooks(gpu, ta, tb):
    """Every hook carries a different op list; the oracle applies them at the same points with the
    same rounding (alpha on A in FP16, beta on C in FP32 as matmatmul! does, src/matmul.jl:196-201)."""
    M, N, K = 256, 256, 192
    conf = configs.mfma_config(M, N, K, ta, tb, block_shape=(128, 128, 64))
    a = rng.matrix("upm1_f16", 51, (K, M) if ta else (M, K))
    b = rng.matrix("upm1_f16", 52, (N, K) if tb else (K, N))
    c = rng.matrix("upm1_f32", 53, (M, N))
    bias = rng.normal_f32(54, N)
    tr = dict(transform_global_to_shared_a=E(lambda x: x * 0.75),
              transform_global_to_shared_b=E(lambda x: abs(x)),
              transform_global_to_shared_c=E(lambda x: x + 0.125),
              transform_shared_to_regs_a=E(lambda x: x * 2.0 - 0.25),
              transform_shared_to_regs_b=E(lambda x: -x),
              transform_shared_to_regs_c=E(lambda x: x * 3.0),
              transform_regs_to_shared_d=E(lambda x: Transform.clamp(x, -20.0, 25.0)),
              transform_shared_to_global_d=E(lambda x: Transform.square(x) * 0.01))
    d = helpers.run_gpu(conf, a, b, c, (M, N), transforms=tr, epilogue_cls=Epilogue.Bias, bias=bias, kernel=Kernel.matmul_pipelined)
    ref = helpers.run_oracle(conf, a, b, c, (M, N), transforms=tr, epilogue=Epilogue.Bias(0), bias=bias)
    assert oracle.rel_frobenius(d, ref) <= TOL


ALL_TILES = [((256, 256, 64), (2, 4)), ((256, 256, 32), (2, 4)), ((256, 256, 32), (4, 2)),
             ((256, 128, 64), (2, 2)), ((128, 256, 64), (2, 2)), ((128, 128, 64), (2, 2)), ((128, 128, 64), (4, 2)), ((128, 128, 32), (2, 2)),
             ((64, 64, 64), (2, 2)), ((64, 64, 32), (1, 1)), ((64, 64, 32), (2, 2))]


@pytest.mark.parametrize("block,waves", ALL_TILES)
@pytest.mark.parametrize("level", [1, 2, 3])
def test_every_tile_at_every_fuse_level(gpu, block, waves, level):
    """Level 1: C / D hooks, bias and one exact FP16 scale on A (0.75: not a power of two); level 2: arbitrary op
    lists on A and B evaluated per element inside the K loop (the large-code kernels); level 3: C / D hooks and
    bias, with a power-of-two scale of A folded into the accumulators.  'T','N' puts both operands on the
    direct-read path, 'N','T' on the transposing reads."""
    from gemmkernels import NT
    BM, BN, BK = block
    M, N, K = 2 * BM, BN, 3 * BK
    for ta, tb in ((True, False), (False, True)):
        conf = configs.mfma_config(M, N, K, ta, tb, block_shape=block, warps_per_block=waves[0] * waves[1],
                                   compute_warp=NT(M=BM // waves[0], N=BN // waves[1], K=16))
        a = rng.matrix("upm1_f16", 61, (K, M) if ta else (M, K))
        b = rng.matrix("upm1_f16", 62, (N, K) if tb else (K, N))
        c = rng.matrix("upm1_f32", 63, (M, N))
        bias = rng.normal_f32(64, N)
        tr = dict(transform_global_to_shared_a=E((lambda x: x * 0.5) if level == 3 else (lambda x: x * 0.75)),
                  transform_shared_to_global_d=E(Transform.relu), transform_shared_to_regs_c=E(lambda x: x * 3.0))
        if level == 2:
            tr["transform_shared_to_regs_a"] = E(lambda x: Transform.square(x) - 0.25)
            tr["transform_global_to_shared_b"] = E(lambda x: abs(x) * 1.5)
        name = gk.kernel_name(conf, Kernel.matmul_pipelined, tr, Epilogue.Bias(0))
        print("case", block, waves, level, ta, tb, name, flush=True)
        assert name.endswith({1: "_fused", 2: "_fused_ab", 3: "_fused_cd"}[level]), name
        d = helpers.run_gpu(conf, a, b, c, (M, N), transforms=tr, epilogue_cls=Epilogue.Bias, bias=bias, kernel=Kernel.matmul_pipelined)
        ref = helpers.run_oracle(conf, a, b, c, (M, N), transforms=tr, epilogue=Epilogue.Bias(0), bias=bias)
        assert oracle.rel_frobenius(d, ref) <= TOL, (ta, tb)


def test_config3_full_size(gpu):
    w = configs.benchmark_config(3)
    run = w.prepare()
    run()
    import torch
    torch.cuda.synchronize()
    d = gk.to_numpy(run.d)
    h = w.host()
    ref = np.maximum(0.5 * oracle.gemm_blas_f32(h["a"], h["b"], None) + h["bias"][None, :], 0.0)
    assert oracle.rel_frobenius(d, ref) <= TOL
    assert (d >= 0).all()


def test_power_of_two_scales_beyond_the_folded_range_run_in_the_k_loop(gpu):
    """A scale of A by 2^e leaves the K loop only for |e| <= 4.  2^-20 takes U[-1,1) FP16 values into the subnormal range
    of FP16, where the reference's hook (and the oracle, and the in-loop scale) rounds s * a to FP16 and loses bits that
    a fold into the accumulators would keep: the result must be the oracle's, not the exact product."""
    import torch
    from gemmkernels import Kernel, Transform, configs, rng
    M, N, K = 256, 256, 256
    conf = configs.mfma_config(M, N, K, block_shape=(128, 128, 64), zero_c=True)
    a, b = rng.matrix("upm1_f16", 9401, (M, K)), rng.matrix("upm1_f16", 9402, (K, N))
    small = dict(transform_global_to_shared_a=Transform.Elementwise(lambda x: x * 2.0 ** -20))
    assert "fused_cd" not in gk.kernel_name(conf, Kernel.matmul_pipelined, transforms=small)          # (the level that runs folded scales)
    d = helpers.run_gpu(conf, a, b, None, (M, N), kernel=Kernel.matmul_pipelined, transforms=small)
    ref = helpers.run_oracle(conf, a, b, None, (M, N), transforms=small)
    exact = 2.0 ** -20 * oracle.gemm_f64(a, b, None, 1.0, 0.0)
    assert oracle.rel_frobenius(d, ref) <= 1e-5
    assert oracle.rel_frobenius(ref, exact) > 1e-3           # the rounding of s * a to FP16 shows: a fold would not have it
    # at the edge of the range, 2^-4, the scale is folded: the plain product times 2^-4, bit for bit
    edge = dict(transform_global_to_shared_a=Transform.Elementwise(lambda x: x * 2.0 ** -4))
    assert "fused_cd" in gk.kernel_name(conf, Kernel.matmul_pipelined, transforms=edge)
    d4 = helpers.run_gpu(conf, a, b, None, (M, N), kernel=Kernel.matmul_pipelined, transforms=edge)
    plain = helpers.run_gpu(conf, a, b, None, (M, N), kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d4, plain * np.float32(2.0 ** -4))
