"""The K-split kernel kind: few output tiles, long K.  The K slices of a tile run as workgroups of one launch,
leave their partial tiles in a workspace and the last one to arrive adds them in slice order: results are
compared by norm against float64, bit for bit between runs, and exactly on data whose sums are exact."""
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
def test_in_place_twice(gpu, dims, block):
    """C = A*B + C in place (mul!(C, A, B, 1, 1)), then a second product on top with a scale on A (the hook
    applies in every slice; C is read by the first slice only and written by the last to arrive)."""
    M, N, K = dims
    conf = configs.mfma_config(M, N, K, block_shape=block)
    a, b, c = operands(M, N, K, False, False, 4300)
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    gk.matmul(conf, A, B, C, C, kernel=Kernel.matmul_split_k)
    torch.cuda.synchronize()
    assert oracle.rel_frobenius(gk.to_numpy(C), oracle.gemm_f64(a, b, c, 1.0, 1.0, False, False)) <= TOL
    gk.matmul(conf, A, B, C, C, kernel=Kernel.matmul_split_k, transform_shared_to_regs_a=Transform.Elementwise(lambda x: x * -2.0))
    torch.cuda.synchronize()
    ref = oracle.gemm_f64(a, b, c, 1.0, 1.0, False, False) + oracle.gemm_f64(a, b, None, -2.0, 0.0, False, False)
    assert oracle.rel_frobenius(gk.to_numpy(C), ref) <= TOL


@pytest.mark.parametrize("dims,block", [((4096, 64, 4096), (64, 64, 64)), ((192, 320, 8192), (64, 64, 64)), ((256, 256, 8192), (128, 128, 64))])
def test_same_bits_on_every_run_and_exact_on_exact_data(gpu, dims, block):
    """The slices are added in slice order whatever the order in which they arrive: ten launches give the same
    bits.  On small-integer data every partial sum is exact in fp32, so the result equals the float64 product
    exactly, whatever the association of the sum."""
    M, N, K = dims
    conf = configs.mfma_config(M, N, K, block_shape=block)
    a, b, c = operands(M, N, K, False, False, 4400)
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    D = gk.colmajor_empty((M, N), torch.float32)
    first = None
    for _ in range(10):
        D.fill_(float("nan"))
        gk.matmul(conf, A, B, C, D, kernel=Kernel.matmul_split_k)
        torch.cuda.synchronize()
        got = gk.to_numpy(D).copy()
        if first is None:
            first = got
        assert np.array_equal(got.view(np.uint32), first.view(np.uint32))
    rs = np.random.RandomState(5)
    ai = np.asfortranarray(rs.randint(-4, 5, size=(M, K)).astype(np.float16))
    bi = np.asfortranarray(rs.randint(-4, 5, size=(K, N)).astype(np.float16))
    ci = np.asfortranarray(rs.randint(-64, 65, size=(M, N)).astype(np.float32))
    gk.matmul(conf, gk.colmajor(ai), gk.colmajor(bi), gk.colmajor(ci), D, kernel=Kernel.matmul_split_k)
    torch.cuda.synchronize()
    assert np.array_equal(gk.to_numpy(D).astype(np.float64), ai.astype(np.float64) @ bi.astype(np.float64) + ci)


def test_hooks_on_d_bias_and_a_16_bit_d(gpu):
    """The last slice to arrive holds the whole sum, so the D hooks, the bias and the rounding to the element
    type of D apply to it like in the unsplit kernel (with atomic partial sums they could not)."""
    M, N, K = 128, 192, 4096
    conf = configs.mfma_config(M, N, K, block_shape=(64, 64, 64))
    a, b, c = operands(M, N, K, False, False, 4100)
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    D = gk.colmajor_empty((M, N), torch.float32)
    bias_h = rng.matrix("upm1_f32", 4104, (N, 1))[:, 0] * 50
    bias = torch.from_numpy(np.ascontiguousarray(bias_h)).cuda()
    gk.matmul(conf, A, B, C, D, kernel=Kernel.matmul_split_k, epilogue=Epilogue.Bias(bias),
              transform_regs_to_shared_d=Transform.Elementwise(lambda x: x * 0.25),
              transform_shared_to_global_d=Transform.Elementwise(Transform.relu))
    torch.cuda.synchronize()
    ref = np.maximum(0.25 * oracle.gemm_f64(a, b, c, 1.0, 1.0) + bias_h[None, :].astype(np.float64), 0.0)
    assert oracle.rel_frobenius(gk.to_numpy(D), ref) <= TOL
    assert (gk.to_numpy(D) == 0).any() and (gk.to_numpy(D) > 0).any()
    # the same product on the unsplit kernel: same hooks, same order of operations after the sum
    D2 = gk.colmajor_empty((M, N), torch.float32)
    gk.matmul(conf, A, B, C, D2, kernel=Kernel.matmul_pipelined, epilogue=Epilogue.Bias(bias),
              transform_regs_to_shared_d=Transform.Elementwise(lambda x: x * 0.25),
              transform_shared_to_global_d=Transform.Elementwise(Transform.relu))
    torch.cuda.synchronize()
    assert oracle.rel_frobenius(gk.to_numpy(D), gk.to_numpy(D2).astype(np.float64)) <= 1e-5
    # Float16 C and D
    from gemmkernels import Float16, Layout
    acm = Layout.UnsafeAlignedColMajor
    conf_h = configs.mfma_config(M, N, K, block_shape=(64, 64, 64), global_c_layout=acm[Float16], global_d_layout=acm[Float16])
    c16 = (c * 8).astype(np.float16)
    Dh = gk.colmajor_empty((M, N), torch.float16)
    gk.matmul(conf_h, A, B, gk.colmajor(c16), Dh, kernel=Kernel.matmul_split_k)
    torch.cuda.synchronize()
    assert oracle.rel_frobenius(gk.to_numpy(Dh), oracle.gemm_f64(a, b, c16, 1.0, 1.0)) <= TOL


def test_the_launcher_without_a_workspace_refuses_the_k_split_kind(gpu):
    M, N, K = 128, 128, 2048
    conf = configs.mfma_config(M, N, K, block_shape=(64, 64, 64))
    a, b, c = operands(M, N, K, False, False, 4100)
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    D = gk.colmajor_empty((M, N), torch.float32)
    import ctypes
    cconf = conf.to_c(M, K, M, M)
    rc = _lib.lib().gk_matmul(ctypes.byref(cconf), A.data_ptr(), B.data_ptr(), C.data_ptr(), D.data_ptr(), None, None,
                              Kernel.matmul_split_k.code, None)
    assert rc == _lib.GK_ERR_INVALID_ARGUMENT and "gk_matmul_split_k" in _lib.last_error()
    need = ctypes.c_size_t()
    assert _lib.lib().gk_split_k_workspace_size(ctypes.byref(cconf), ctypes.byref(need)) == 0 and need.value > 0
    small = torch.zeros(1024, dtype=torch.uint8, device="cuda")       # a workspace that is too small is refused, nothing runs
    rc = _lib.lib().gk_matmul_split_k(ctypes.byref(cconf), A.data_ptr(), B.data_ptr(), C.data_ptr(), D.data_ptr(), None, None,
                                      small.data_ptr(), small.numel(), None)
    assert rc == _lib.GK_ERR_INVALID_ARGUMENT and "workspace" in _lib.last_error()


def test_blas_entry_picks_the_k_split_kernel_for_skinny_products(gpu):
    M, N, K = 2048, 64, 4096
    a, b, c = operands(M, N, K, False, False, 4200)
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    gk.matmatmul_(C, "N", "N", A, B, 0.5, 2.0)
    torch.cuda.synchronize()
    first = gk.to_numpy(C).copy()
    assert oracle.rel_frobenius(first, oracle.gemm_f64(a, b, c, 0.5, 2.0)) <= TOL
    # mul! is deterministic in the reference (src/matmul.jl:185-204) and here: same inputs, same bits
    for _ in range(5):
        C2 = gk.colmajor(c)
        gk.matmatmul_(C2, "N", "N", A, B, 0.5, 2.0)
        torch.cuda.synchronize()
        assert np.array_equal(gk.to_numpy(C2).view(np.uint32), first.view(np.uint32))


@pytest.mark.parametrize("beta", [1.0, 0.5, 0.0])
def test_skinny_products_with_tiles_over_the_edge_are_split_too(gpu, beta):
    """N = 100 columns of a K x N B (contiguous along k, so any N is fine), M a multiple of 8 that is not a
    whole number of tiles, K whole tiles: the K-split instances mask the tiles over the edge."""
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


def _split_on(ws, M, N, K, block, seed, swizzle=None):
    """One K-split launch of small-integer data on the workspace `ws`, through the C ABI; returns (D, exact reference)."""
    import ctypes
    kw = {} if swizzle is None else {"cta_swizzle": swizzle}
    conf = configs.mfma_config(M, N, K, block_shape=block, **kw)
    rs = np.random.RandomState(seed)
    ai = np.asfortranarray(rs.randint(-4, 5, size=(M, K)).astype(np.float16))
    bi = np.asfortranarray(rs.randint(-4, 5, size=(K, N)).astype(np.float16))
    ci = np.asfortranarray(rs.randint(-64, 65, size=(M, N)).astype(np.float32))
    A, B, C = gk.colmajor(ai), gk.colmajor(bi), gk.colmajor(ci)
    D = gk.colmajor_empty((M, N), torch.float32)
    D.fill_(float("nan"))
    cconf = conf.to_c(M, K, M, M)
    need = ctypes.c_size_t()
    assert _lib.lib().gk_split_k_workspace_size(ctypes.byref(cconf), ctypes.byref(need)) == 0 and 0 < need.value <= ws.numel()
    rc = _lib.lib().gk_matmul_split_k(ctypes.byref(cconf), A.data_ptr(), B.data_ptr(), C.data_ptr(), D.data_ptr(), None, None,
                                      ws.data_ptr(), ws.numel(), None)
    assert rc == _lib.GK_OK, _lib.last_error()
    torch.cuda.synchronize()
    return gk.to_numpy(D).astype(np.float64), ai.astype(np.float64) @ bi.astype(np.float64) + ci


def test_one_workspace_serves_products_with_different_tile_counts(gpu):
    """The arrival counters sit in a region of fixed size at the head of the workspace.  (With a region as large as the
    tile count asked for, a product of 128 tiles found the partial sums of an earlier product of 64 tiles where its
    counters 64 .. 127 are: no workgroup of those tiles ever saw itself arrive last and D stayed unwritten.)  Small-integer
    data: every sum is exact, so D must equal the float64 product whatever is left in the workspace."""
    ws = torch.zeros(16 << 20, dtype=torch.uint8, device="cuda")
    seq = [((4096, 64, 8192), (64, 64, 64)),      # 64 tiles x 8 slices
           ((1024, 512, 2048), (64, 64, 64)),     # 128 tiles x 2 slices
           ((4096, 64, 4096), (64, 64, 64)),      # 64 tiles again
           ((1024, 1024, 2048), (64, 64, 64)),    # 256 tiles x 2 slices
           ((256, 256, 8192), (128, 128, 64)),    # 4 tiles
           ((1024, 512, 2048), (64, 64, 64))]
    for i, (dims, block) in enumerate(seq):
        print("K-split on a shared workspace:", dims, block, flush=True)
        got, ref = _split_on(ws, *dims, block, 9000 + i)
        assert np.array_equal(got, ref), (dims, block)
    # ... and every counter is back at zero
    assert int(ws[:2048].to(torch.int32).abs().sum()) == 0


def test_many_launches_on_one_workspace_with_other_data_and_other_tile_walks(gpu):
    """The partial tiles cross from one XCD's L2 to another's through memory (device-scope stores and loads).  A line of
    the workspace that a launch reads was written by the launch before as well: forty launches on one workspace, each
    with data of its own and every other one with another tile-to-XCD mapping, must each give the exact product -- a
    stale line from an earlier launch would show."""
    from gemmkernels import CTASwizzle
    ws = torch.zeros(8 << 20, dtype=torch.uint8, device="cuda")
    walks = [None, CTASwizzle.Identity, CTASwizzle.XCDAware[2], CTASwizzle.HorizontallyTiled[2]]
    for i in range(40):
        got, ref = _split_on(ws, 512, 256, 4096, (64, 64, 64), 9100 + i, walks[i % 4])
        assert np.array_equal(got, ref), i


def test_blas_entry_after_a_product_with_fewer_tiles(gpu):
    """mul! on 4096 x 64 x 8192 (64 tiles) and then on 1024 x 512 x 2048 (128 tiles): both take the K-split kernel and
    share the workspace the host layer keeps per stream."""
    for (M, N, K), seed in (((4096, 64, 8192), 9300), ((1024, 512, 2048), 9301), ((4096, 64, 8192), 9302)):
        rs = np.random.RandomState(seed)
        ai = np.asfortranarray(rs.randint(-4, 5, size=(M, K)).astype(np.float16))
        bi = np.asfortranarray(rs.randint(-4, 5, size=(K, N)).astype(np.float16))
        ci = np.asfortranarray(rs.randint(-64, 65, size=(M, N)).astype(np.float32))
        C = gk.colmajor(ci)
        gk.matmatmul_(C, "N", "N", gk.colmajor(ai), gk.colmajor(bi), 1.0, 1.0)
        torch.cuda.synchronize()
        assert np.array_equal(gk.to_numpy(C).astype(np.float64), ai.astype(np.float64) @ bi.astype(np.float64) + ci), (M, N, K)
