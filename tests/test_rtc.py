"""Kernels specialised at run time (hipRTC): arbitrary elementwise expressions at the transform hooks
and block shapes outside the compiled table, the flexibility the reference gets from its JIT
(src/matmul.jl:38, src/transform.jl:26-30).  Compilation needs no GPU; the launches are GPU tests."""
import numpy as np
import pytest

import gemmkernels as gk
from gemmkernels import configs, Epilogue, Kernel, Layout, NT, Operator, Transform, Float16, Float32, rng
from gemmkernels import _lib

LEAKY = "x > 0.0f ? x : 0.01f * x"


def test_compile_and_cache_without_a_gpu():
    conf = configs.mfma_config(512, 512, 256, block_shape=(128, 128, 64))
    k = gk.specialize(conf, transform_shared_to_global_d=LEAKY, transform_global_to_shared_a=Transform.Elementwise(lambda x: x * 0.5))
    assert k.name == "mfma_gemm_rtc_nn_128x128x64_w2x2_s4_f16"
    assert k.expressions[0] == "(x * 0x1.0000000000000p-1f)" and k.expressions[3] == LEAKY
    again = gk.specialize(conf, transform_shared_to_global_d=LEAKY, transform_global_to_shared_a=Transform.Elementwise(lambda x: x * 0.5))
    assert again._handle.value == k._handle.value                       # served from the cache


def test_errors_come_back_as_config_errors():
    conf = configs.mfma_config(512, 512, 256, block_shape=(128, 128, 64))
    with pytest.raises(gk.ConfigError) as ei:
        gk.specialize(conf, transform_shared_to_global_d="x +")
    assert ei.value.status == _lib.GK_ERR_UNSUPPORTED and "error" in ei.value.message
    with pytest.raises(gk.ConfigError):
        Transform.Elementwise(expr="1.0f")                                # does not depend on x
    # a tile the kernel template cannot form: wave tile not made of 32x32 blocks
    bad = gk.get_config(gemm_shape=NT(M=480, N=512, K=256), operator=Operator.MFMAOp[32, 32, 16, Float16, Float32],
                        global_a_layout=Layout.UnsafeAlignedColMajor[Float16], global_c_layout=Layout.UnsafeAlignedColMajor[Float32],
                        block_shape=NT(M=96, N=128, K=64), warps_per_block=4, compute_warp=NT(M=48, N=64, K=16), specialize=True)
    with pytest.raises(gk.ConfigError) as ei:
        gk.specialize(bad)
    assert ei.value.status == _lib.GK_ERR_BLOCK_SHAPE
    # expression transforms cannot travel as op lists
    with pytest.raises(gk.ConfigError):
        gk.matmul.__globals__["lower_transforms"]({"transform_global_to_shared_a": Transform.Elementwise(expr="x * x")})


def reference(a, b, c, bias, leaky=True, scale_a=1.0):
    acc = (a.astype(np.float64) * scale_a) @ b.astype(np.float64)
    if c is not None:
        acc = acc + c
    if bias is not None:
        acc = acc + bias[None, :]
    return np.where(acc > 0, acc, 0.01 * acc) if leaky else acc


@pytest.mark.gpu
def test_leaky_relu_epilogue_with_bias(gpu):
    import torch
    M, N, K = 512, 384, 256
    conf = configs.mfma_config(M, N, K, block_shape=(128, 128, 64))
    a, b, c = rng.matrix("upm1_f16", 1, (M, K)), rng.matrix("upm1_f16", 2, (K, N)), rng.matrix("upm1_f32", 3, (M, N))
    bias = rng.normal_f32(4, N)
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    D = gk.colmajor_empty((M, N), torch.float32)
    D.fill_(float("nan"))
    tb = torch.from_numpy(bias).cuda()
    gk.matmul(conf, A, B, C, D, transform_shared_to_global_d=Transform.Elementwise(expr=LEAKY), epilogue=Epilogue.Bias(tb),
              kernel=Kernel.matmul_pipelined)
    torch.cuda.synchronize()
    d = gk.to_numpy(D)
    ref = reference(a, b, c, bias)
    assert np.linalg.norm(d - ref) / np.linalg.norm(ref) <= 1e-3
    assert (d < 0).any() and (d > 0).any()


@pytest.mark.gpu
@pytest.mark.parametrize("ta,tb", [(False, False), (True, True)])
def test_closed_vocabulary_hooks_give_the_same_bits_as_the_compiled_kernels(gpu, ta, tb):
    """The op lists spelled as expressions and inlined must reproduce the library's interpreted hooks."""
    import torch
    M, N, K = 256, 256, 192
    conf = configs.mfma_config(M, N, K, ta, tb, block_shape=(128, 128, 64))
    a = rng.matrix("upm1_f16", 11, (K, M) if ta else (M, K))
    b = rng.matrix("upm1_f16", 12, (N, K) if tb else (K, N))
    c = rng.matrix("upm1_f32", 13, (M, N))
    hooks = dict(transform_global_to_shared_a=Transform.Elementwise(lambda x: x * 0.5),
                 transform_shared_to_regs_b=Transform.Elementwise(lambda x: Transform.clamp(x, -0.75, 0.5)),
                 transform_global_to_shared_c=Transform.Elementwise(lambda x: x * 3.0 + 1.0),
                 transform_shared_to_global_d=Transform.Elementwise(Transform.relu))
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    D1, D2 = gk.colmajor_empty((M, N), torch.float32), gk.colmajor_empty((M, N), torch.float32)
    gk.matmul(conf, A, B, C, D1, kernel=Kernel.matmul_pipelined, **hooks)
    gk.specialize(conf, **hooks)(A, B, C, D2)
    torch.cuda.synchronize()
    assert np.array_equal(gk.to_numpy(D1), gk.to_numpy(D2))


@pytest.mark.gpu
@pytest.mark.parametrize("block,waves", [((64, 128, 64), (1, 2)), ((128, 64, 32), (2, 1)), ((64, 256, 64), (2, 2)), ((256, 64, 64), (2, 2)), ((128, 128, 128), (2, 2))])
def test_block_shapes_outside_the_compiled_table(gpu, block, waves):
    """The reference's parameter sweep (configs/configs.jl:594-611) runs rectangular tiles such as
    64x128 and 256x64; here they are compiled on demand."""
    import torch
    from oracle import oracle
    BM, BN, BK = block
    M, N, K = 2 * BM, 2 * BN, 3 * BK
    conf = gk.get_config(gemm_shape=NT(M=M, N=N, K=K), operator=Operator.MFMAOp[32, 32, 16, Float16, Float32],
                         global_a_layout=Layout.UnsafeAlignedColMajor[Float16], global_b_layout=Layout.UnsafeAlignedRowMajor[Float16],
                         global_c_layout=Layout.UnsafeAlignedColMajor[Float32], global_d_layout=Layout.UnsafeAlignedColMajor[Float32],
                         is_b_col_major=False, block_shape=NT(M=BM, N=BN, K=BK), warps_per_block=waves[0] * waves[1],
                         compute_warp=NT(M=BM // waves[0], N=BN // waves[1], K=16), specialize=True)
    a, b, c = rng.matrix("upm1_f16", 21, (M, K)), rng.matrix("upm1_f16", 22, (N, K)), rng.matrix("upm1_f32", 23, (M, N))
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    D = gk.colmajor_empty((M, N), torch.float32)
    D.fill_(float("nan"))
    k = gk.specialize(conf, transform_global_to_shared_a="x * x")
    print("case", block, waves, k.name, flush=True)
    k(A, B, C, D)
    torch.cuda.synchronize()
    ref = oracle.gemm_f64((a.astype(np.float32) ** 2).astype(np.float16), b, c, 1.0, 1.0, False, True)
    assert oracle.rel_frobenius(gk.to_numpy(D), ref) <= 1e-3


@pytest.mark.gpu
def test_wave_tile_of_sixteen_blocks_runs_with_synchronous_fragment_reads(gpu):
    """A 256x256 tile on 2x2 waves keeps 256 accumulator registers per lane and spills; kernels like
    that read their fragments synchronously (a spill between an asynchronous read and its wait would
    save stale values).  Only a hook on D here, so the K loop is the plain one."""
    import torch
    from oracle import oracle
    M, N, K = 512, 512, 192
    conf = gk.get_config(gemm_shape=NT(M=M, N=N, K=K), operator=Operator.MFMAOp[32, 32, 16, Float16, Float32],
                         global_a_layout=Layout.UnsafeAlignedColMajor[Float16], global_c_layout=Layout.UnsafeAlignedColMajor[Float32],
                         block_shape=NT(M=256, N=256, K=32), warps_per_block=4, compute_warp=NT(M=128, N=128, K=16), specialize=True)
    a, b, c = rng.matrix("upm1_f16", 31, (M, K)), rng.matrix("upm1_f16", 32, (K, N)), rng.matrix("upm1_f32", 33, (M, N))
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    D = gk.colmajor_empty((M, N), torch.float32)
    D.fill_(float("nan"))
    gk.specialize(conf, transform_shared_to_global_d="2.0f * x")(A, B, C, D)
    torch.cuda.synchronize()
    assert oracle.rel_frobenius(gk.to_numpy(D), 2.0 * oracle.gemm_f64(a, b, c, 1.0, 1.0, False, False)) <= 1e-3


@pytest.mark.gpu
def test_a_specialised_kernel_refuses_bounds_checked_layouts_at_launch(gpu):
    """Compiled for aligned layouts; a launch configuration of the same tile on bounds-checked layouts (which
    admit sizes the specialised kernel cannot mask) is turned down before anything runs."""
    import torch
    from gemmkernels.matmul import Plan, _DEFAULT_EPILOGUE
    M, N, K = 256, 256, 128
    common = dict(operator=Operator.MFMAOp[32, 32, 16, Float16, Float32], block_shape=NT(M=128, N=128, K=64), warps_per_block=4,
                  compute_warp=NT(M=64, N=64, K=16))
    conf = gk.get_config(gemm_shape=NT(M=M, N=N, K=K), global_a_layout=Layout.UnsafeAlignedColMajor[Float16],
                         global_b_layout=Layout.UnsafeAlignedColMajor[Float16], global_c_layout=Layout.Zero[Float32],
                         global_d_layout=Layout.UnsafeAlignedColMajor[Float32], specialize=True, **common)
    k = gk.specialize(conf, transform_shared_to_global_d="x + 1.0f")
    loose = gk.get_config(gemm_shape=NT(M=M - 8, N=N, K=K), global_a_layout=Layout.ColMajor[Float16],
                          global_b_layout=Layout.ColMajor[Float16], global_c_layout=Layout.Zero[Float32],
                          global_d_layout=Layout.ColMajor[Float32], **common)
    A = gk.colmajor(rng.matrix("upm1_f16", 31, (M, K))); B = gk.colmajor(rng.matrix("upm1_f16", 32, (K, N)))
    D = gk.colmajor_empty((M, N), torch.float32)
    with pytest.raises(gk.ConfigError):
        Plan(loose, A[:M - 8, :], B, None, D[:M - 8, :], {}, _DEFAULT_EPILOGUE, Kernel.matmul_pipelined, specialized=k)()
    k(A, B, None, D)                                  # the configuration it was compiled for still runs
    torch.cuda.synchronize()


# The reference's parameter sweep of the tensor-core GEMM (configs/configs.jl:597-612): M = N = K = 256, block shapes of at
# most 128 x 128 outputs out of {64, 128, 256}^2, BLOCK_K in {16, 32, 64}, 1 / 2 / 4 warps along M and N with at least four in
# all.  Every tile that the kernel template can be built for is compiled on demand and checked against the oracle; the
# others are refused with a configuration error before anything is compiled, which the reference's test counts as
# skipped (test/matmul.jl:21-27).  'N','N' for every tile, 'T','T' as well for BLOCK_K = 16 (which runs on the 32 x 32 x 16
# instruction: the k-step of v_mfma_f32_16x16x32 is 32).
SWEEP_BLOCKS = [(bm, bn, bk) for bm in (64, 128, 256) for bn in (64, 128, 256) if bm * bn <= 128 * 128 for bk in (16, 32, 64)]
SWEEP_WAVES = [(wm, wn) for wm in (1, 2, 4) for wn in (1, 2, 4) if wm * wn >= 4]


@pytest.mark.gpu
@pytest.mark.parametrize("block", SWEEP_BLOCKS)
def test_the_reference_sweep_of_block_shapes_and_warp_arrangements(gpu, block):
    import torch
    from gemmkernels import ConfigError
    from oracle import oracle
    BM, BN, BK = block
    M = N = K = 256
    ran = refused = 0
    for ta, tb in ([(False, False), (True, True)] if BK == 16 else [(False, False)]):
        a = rng.matrix("upm1_f16", 41, (K, M) if ta else (M, K))
        b = rng.matrix("upm1_f16", 42, (N, K) if tb else (K, N))
        c = rng.matrix("upm1_f32", 43, (M, N))
        A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
        ref = oracle.gemm_f64(a, b, c, 1.0, 1.0, ta, tb)
        for wm, wn in SWEEP_WAVES:
            try:
                conf = gk.get_config(gemm_shape=NT(M=M, N=N, K=K), operator=Operator.MFMAOp[32, 32, 16, Float16, Float32],
                                     global_a_layout=(Layout.UnsafeAlignedRowMajor if ta else Layout.UnsafeAlignedColMajor)[Float16],
                                     global_b_layout=(Layout.UnsafeAlignedRowMajor if tb else Layout.UnsafeAlignedColMajor)[Float16],
                                     global_c_layout=Layout.UnsafeAlignedColMajor[Float32], global_d_layout=Layout.UnsafeAlignedColMajor[Float32],
                                     is_a_col_major=not ta, is_b_col_major=not tb, block_shape=NT(M=BM, N=BN, K=BK), warps_per_block=wm * wn,
                                     compute_warp=NT(M=BM // wm, N=BN // wn, K=16), specialize=True)
                k = gk.specialize(conf)
            except ConfigError as e:
                refused += 1
                print("refused", block, (wm, wn), "TT" if ta else "NN", e.message[:90], flush=True)
                continue
            print("runs   ", block, (wm, wn), "TT" if ta else "NN", k.name, flush=True)
            D = gk.colmajor_empty((M, N), torch.float32)
            D.fill_(float("nan"))
            k(A, B, C, D)
            torch.cuda.synchronize()
            assert oracle.rel_frobenius(gk.to_numpy(D), ref) <= 1e-3, (block, wm, wn, ta, tb)
            ran += 1
    print(f"block {block}: {ran} ran, {refused} refused", flush=True)
    # what runs is exactly what the kernel template can be built for: wave tiles made of 32 x 32 blocks (at most sixteen),
    # and an A tile and a B tile whose 1 KiB pieces divide evenly over the waves (64 x 64 x 16 has two pieces per operand
    # and no arrangement of four or more waves: the whole block shape counts as skipped, like a ConfigError of the reference)
    def buildable(wm, wn):
        wtm, wtn = BM // wm, BN // wn
        pieces_a, pieces_b = BM * BK * 2 // 1024, BN * BK * 2 // 1024
        return (wtm % 32 == 0 and wtn % 32 == 0 and (wtm // 32) * (wtn // 32) <= 16 and pieces_a % (wm * wn) == 0 and pieces_b % (wm * wn) == 0)
    expected = sum(buildable(wm, wn) for wm, wn in SWEEP_WAVES) * (2 if BK == 16 else 1)
    assert ran == expected, (block, ran, expected)
