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
