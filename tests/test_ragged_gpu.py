"""Products on the bounds-checked layouts (Layout.ColMajor / RowMajor, reference src/layout.jl:117-184) run on
the aligned kernels: tiles that stick out over M or N clamp their loads and mask their C loads and D stores, the
last K tile is repaired in LDS when it is partial or a 16-byte chunk reaches over the end of an operand.  Parity
against the oracle, bit-for-bit equality with the same tile on zero-padded operands, no write outside D, odd
sizes, odd leading dimensions and misaligned pointers."""
import numpy as np
import pytest
import torch

import gemmkernels as gk
from gemmkernels import Epilogue, Kernel, Layout, NT, Operator, Transform, rng
from gemmkernels.dtypes import Float16, Float32
import helpers
from oracle import oracle

pytestmark = pytest.mark.gpu
E = Transform.Elementwise
TILES = [((256, 256, 64), (2, 4)), ((256, 256, 32), (2, 4)), ((256, 128, 64), (2, 2)), ((128, 256, 64), (2, 2)),
         ((128, 128, 32), (2, 2)), ((128, 128, 64), (2, 2)), ((128, 128, 64), (4, 2)), ((64, 64, 64), (2, 2)), ((64, 64, 32), (2, 2))]


def checked_config(M, N, K, ta, tb, block, waves, zero_c=False, cd=Float32):
    BM, BN, BK = block
    return gk.get_config(
        gemm_shape=NT(M=M, N=N, K=K), block_shape=NT(M=BM, N=BN, K=BK),
        warps_per_block=waves[0] * waves[1], compute_warp=NT(M=BM // waves[0], N=BN // waves[1], K=16),
        operator=Operator.MFMAOp[32, 32, 16, Float16, Float32],
        global_a_layout=Layout.RowMajor[Float16] if ta else Layout.ColMajor[Float16],
        global_b_layout=Layout.RowMajor[Float16] if tb else Layout.ColMajor[Float16],
        global_c_layout=Layout.Zero[cd] if zero_c else Layout.ColMajor[cd], global_d_layout=Layout.ColMajor[cd],
        is_a_col_major=not ta, is_b_col_major=not tb)


def operands(M, N, K, ta, tb, seed):
    a = rng.matrix("upm1_f16", seed + 1, (K, M) if ta else (M, K))
    b = rng.matrix("upm1_f16", seed + 2, (N, K) if tb else (K, N))
    c = rng.matrix("upm1_f32", seed + 3, (M, N))
    return a, b, c


@pytest.mark.parametrize("block,waves", TILES)
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_tiles_over_the_edge_against_the_oracle_and_against_padded_operands(gpu, block, waves, ta, tb):
    BM, BN, BK = block
    for K in (3 * BK, 2 * BK + 24, 8):              # whole tiles; a partial last tile; less than one tile
        _one_shape(block, waves, ta, tb, BM + 72, 2 * BN - 56, K)    # M, N: multiples of 8, not of any tile


@pytest.mark.parametrize("block,waves", TILES)
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_sizes_that_are_not_multiples_of_8(gpu, block, waves, ta, tb):
    """M, N and K odd: 16-byte chunks straddle the last row of A / column of B / value of k, and every column
    starts at a different offset from a 16-byte boundary.  Same bits as the tile on zero-padded operands."""
    BM, BN, BK = block
    for K in (3 * BK, 2 * BK + 27, 2 * BK + 1, 13):     # whole tiles (the last one leaves the pipeline at the edges); partial tiles; less than a tile
        _one_shape(block, waves, ta, tb, BM + 73, 2 * BN - 59, K)
    _one_shape(block, waves, ta, tb, 2 * BM, BN, 2 * BK + 3)             # only K is odd
    _one_shape(block, waves, ta, tb, 9, 11, 8)                           # a corner of one tile


def _one_shape(block, waves, ta, tb, M, N, K):
    BM, BN, BK = block
    conf = checked_config(M, N, K, ta, tb, block, waves)
    name = gk.kernel_name(conf, Kernel.matmul_singlestage)
    assert "checked" not in name, name
    a, b, c = operands(M, N, K, ta, tb, 4000)
    print("case", block, waves, ta, tb, (M, N, K), name, flush=True)
    d = helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_singlestage)
    ref = helpers.run_oracle(conf, a, b, c, (M, N))
    assert oracle.rel_frobenius(d, ref) <= 1e-3
    # the same tile on operands padded with zeros to whole tiles: identical sums, identical bits
    Mp, Np, Kp = -(-M // BM) * BM, -(-N // BN) * BN, -(-K // BK) * BK
    ap = np.zeros((Kp, Mp) if ta else (Mp, Kp), np.float16, order="F")
    bp = np.zeros((Np, Kp) if tb else (Kp, Np), np.float16, order="F")
    cp = np.zeros((Mp, Np), np.float32, order="F")
    if ta: ap[:K, :M] = a
    else: ap[:M, :K] = a
    if tb: bp[:N, :K] = b
    else: bp[:K, :N] = b
    cp[:M, :N] = c
    import test_mfma_gemm_gpu as T
    dp = helpers.run_gpu(T.make_config(Mp, Np, Kp, ta, tb, block, waves), ap, bp, cp, (Mp, Np), kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d, dp[:M, :N])


@pytest.mark.parametrize("ta,tb", [(False, False), (True, True)])
def test_nothing_is_written_outside_d_and_hooks_bias_and_fp16_d_work_over_the_edge(gpu, ta, tb):
    M, N, K = 328, 264, 152                      # K: two whole tiles and 24 more
    block, waves = (256, 256, 64), (2, 4)
    a, b, c = operands(M, N, K, ta, tb, 4100)
    bias = rng.normal_f32(4104, N)
    tr = dict(transform_global_to_shared_a=E(lambda x: x * 0.5), transform_shared_to_regs_c=E(lambda x: x * 3.0),
              transform_shared_to_global_d=E(Transform.relu))
    for cd, tdtype, tol in ((Float32, torch.float32, 1e-3), (Float16, torch.float16, 2e-3)):
        conf = checked_config(M, N, K, ta, tb, block, waves, cd=cd)
        A, B = gk.colmajor(a), gk.colmajor(b)
        c_h = c if cd is Float32 else c.astype(np.float16)
        C = gk.colmajor(c_h)
        ld, cols = M + 24, N + 5
        full = gk.colmajor(np.asfortranarray(np.full((ld, cols), 777.0, np.float32 if cd is Float32 else np.float16)))
        D = full[:M, :N]                           # a window of a larger array: rows and columns around it must stay
        gk.matmul(conf, A, B, C, D, epilogue=Epilogue.Bias(torch.from_numpy(bias).cuda()), kernel=Kernel.matmul_singlestage, **tr)
        torch.cuda.synchronize()
        out = full.float().cpu().numpy()
        assert (out[M:, :] == 777.0).all() and (out[:, N:] == 777.0).all()
        ref = helpers.run_oracle(conf, a, b, c_h, (M, N), d_dtype=np.float32 if cd is Float32 else np.float16, transforms=tr,
                                 epilogue=Epilogue.Bias(0), bias=bias)
        assert oracle.rel_frobenius(out[:M, :N], ref.astype(np.float32)) <= tol, cd


def test_misaligned_pointers_and_odd_leading_dimensions(gpu):
    """Operands that start two bytes off a 16-byte boundary inside arrays with odd leading dimensions: the same
    aligned kernel, the same bits as with aligned copies of the operands."""
    M, N, K = 200, 136, 96
    for ta, tb in ((False, False), (True, True), (False, True), (True, False)):
        conf = checked_config(M, N, K, ta, tb, (64, 64, 32), (2, 2))
        assert "checked" not in gk.kernel_name(conf, Kernel.matmul_singlestage)
        a, b, c = operands(M, N, K, ta, tb, 4200)
        a_big = np.zeros((a.shape[0] + 9, a.shape[1]), np.float16, order="F"); a_big[1:a.shape[0] + 1, :] = a
        b_big = np.zeros((b.shape[0] + 11, b.shape[1]), np.float16, order="F"); b_big[1:b.shape[0] + 1, :] = b
        A, B, C = gk.colmajor(a_big)[1:a.shape[0] + 1, :], gk.colmajor(b_big)[1:b.shape[0] + 1, :], gk.colmajor(c)
        assert A.data_ptr() % 16 == 2 and B.data_ptr() % 16 == 2 and A.stride(1) % 2 == 1 and B.stride(1) % 2 == 1
        D = gk.colmajor_empty((M, N), torch.float32)
        gk.matmul(conf, A, B, C, D, kernel=Kernel.matmul_singlestage)
        torch.cuda.synchronize()
        ref = helpers.run_oracle(conf, a, b, c, (M, N))
        assert oracle.rel_frobenius(gk.to_numpy(D), ref) <= 1e-3
        D2 = gk.colmajor_empty((M, N), torch.float32)
        gk.matmul(conf, gk.colmajor(a), gk.colmajor(b), C, D2, kernel=Kernel.matmul_singlestage)
        torch.cuda.synchronize()
        assert np.array_equal(gk.to_numpy(D2), gk.to_numpy(D)), (ta, tb)


def test_the_last_element_of_an_operand_may_be_the_last_of_its_allocation(gpu):
    """The chunk that straddles the last row of A in the last k must not be read past the end of A: here A and B
    end exactly where their device allocations end (the library's own allocator, sizes rounded to nothing)."""
    import ctypes
    from gemmkernels import _lib
    lib = _lib.lib()
    M, N, K = 2 * 256 - 3, 256 + 5, 64 + 7
    for ta, tb in ((False, False), (True, True)):
        conf = checked_config(M, N, K, ta, tb, (256, 256, 64), (2, 4), zero_c=True)
        a, b, _ = operands(M, N, K, ta, tb, 4250)
        # place the operands at the very end of 2 MiB allocations
        size = 2 << 20
        pa, pb = ctypes.c_void_p(), ctypes.c_void_p()
        assert lib.gk_dev_alloc(size, ctypes.byref(pa)) == 0 and lib.gk_dev_alloc(size, ctypes.byref(pb)) == 0
        try:
            a_addr = pa.value + size - a.nbytes
            b_addr = pb.value + size - b.nbytes
            assert lib.gk_copy_to_device(a_addr, a.ctypes.data, a.nbytes) == 0
            assert lib.gk_copy_to_device(b_addr, b.ctypes.data, b.nbytes) == 0
            D = gk.colmajor_empty((M, N), torch.float32)
            cconf = conf.to_c(a.shape[0], b.shape[0], M, M)
            print("case end of allocation", ta, tb, hex(a_addr), hex(b_addr), flush=True)
            rc = lib.gk_matmul(ctypes.byref(cconf), a_addr, b_addr, None, D.data_ptr(), None, None, Kernel.matmul_singlestage.code, None)
            assert rc == 0, _lib.last_error()
            torch.cuda.synchronize()
            ref = helpers.run_oracle(conf, a, b, None, (M, N))
            assert oracle.rel_frobenius(gk.to_numpy(D), ref) <= 1e-3
        finally:
            lib.gk_dev_free(pa)
            lib.gk_dev_free(pb)


def test_full_size_4000(gpu):
    """mul!(C, A, B) at 4000^3: one launch of the 256 x 256 tile, checked through linearity and a few exact rows."""
    from gemmkernels.matmul import matmatmul_plan
    n = 4000
    a = rng.matrix("upm1_f16", 4301, (n, n)); b = rng.matrix("upm1_f16", 4302, (n, n))
    A, B = gk.colmajor(a), gk.colmajor(b)
    C = gk.colmajor_empty((n, n), torch.float32)
    p = matmatmul_plan(C, "N", "N", A, B, 1.0, 0.0)
    assert "checked" not in p.kernel_names[0], p.kernel_names
    p()
    torch.cuda.synchronize()
    out = gk.to_numpy(C)
    rows = [0, 1, 255, 256, 3839, 3840, 3967, 3999]
    ref = a[rows, :].astype(np.float64) @ b.astype(np.float64)
    assert oracle.rel_frobenius(out[rows, :], ref) <= 1e-3
    colsel = [0, 3840, 3999]
    refc = a.astype(np.float64) @ b[:, colsel].astype(np.float64)
    assert oracle.rel_frobenius(out[:, colsel], refc) <= 1e-3


# tiles with a side of 192 are compiled per transpose
TILES_192 = [((256, 192, 64), (4, 2), [(False, False), (True, False), (False, True)]), ((192, 256, 64), (2, 4), [(True, False), (True, True)])]


@pytest.mark.parametrize("block,waves,transposes", TILES_192)
def test_tiles_with_a_side_of_192(gpu, block, waves, transposes):
    """Whole tiles (aligned layouts, C read, hooks and bias) and tiles over the edge (bounds-checked layouts,
    partial last K tile), against the oracle; the ragged case bit for bit against zero-padded operands."""
    import test_mfma_gemm_gpu as T
    BM, BN, BK = block
    for ta, tb in transposes:
        M, N, K = 2 * BM, 3 * BN, 3 * BK
        conf = T.make_config(M, N, K, ta, tb, block, waves)
        a, b, c = operands(M, N, K, ta, tb, 4400)
        name = gk.kernel_name(conf, Kernel.matmul_pipelined)
        print("case", block, waves, ta, tb, name, flush=True)
        d = helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
        assert oracle.rel_frobenius(d, helpers.run_oracle(conf, a, b, c, (M, N))) <= 1e-3
        bias = rng.normal_f32(4404, N)
        for tr in (dict(transform_global_to_shared_a=E(lambda x: x * 0.5), transform_shared_to_global_d=E(Transform.relu)),
                   dict(transform_shared_to_regs_a=E(lambda x: Transform.square(x) - 0.25), transform_global_to_shared_b=E(lambda x: abs(x) * 1.5))):
            d = helpers.run_gpu(conf, a, b, c, (M, N), transforms=tr, epilogue_cls=Epilogue.Bias, bias=bias, kernel=Kernel.matmul_pipelined)
            ref = helpers.run_oracle(conf, a, b, c, (M, N), transforms=tr, epilogue=Epilogue.Bias(0), bias=bias)
            assert oracle.rel_frobenius(d, ref) <= 1e-3, sorted(tr)
        _one_shape(block, waves, ta, tb, BM + 72, 2 * BN - 56, 2 * BK + 24)
    # the default picks them where they fill the chip and only where the kernel has them
    from gemmkernels import default_block_shape
    op = Operator.MFMAOp[32, 32, 16, Float16, Float32]
    big = NT(M=3072, N=3072, K=3072)
    assert default_block_shape(op, big) == NT(M=256, N=192, K=64)                                        # 'N','N'
    assert default_block_shape(op, big, a_kmajor=False, b_kmajor=False) == NT(M=256, N=192, K=64)        # 'N','T'
    assert default_block_shape(op, big, a_kmajor=True, b_kmajor=False) == NT(M=192, N=256, K=64)         # 'T','T'
    assert default_block_shape(op, big, a_kmajor=True, b_kmajor=True) in (NT(M=256, N=192, K=64), NT(M=192, N=256, K=64))


def test_random_shapes_through_the_blas_level_front_end(gpu):
    """Sixty seeded shapes (multiples of 8, some with an odd M, which only a K-major A lets onto the aligned
    kernels), random transposes, alpha and beta, against the float64 product."""
    from gemmkernels.matmul import matmatmul_plan
    rs = np.random.RandomState(7)
    aligned_kernel_runs = 0
    for it in range(60):
        M, N, K = (int(rs.randint(1, 90)) * 8 for _ in range(3))
        if it % 5 == 0:
            M = int(rs.randint(1, 700))
        if it % 7 == 0:
            K = int(rs.randint(1, 40)) * 8
        ta, tb = bool(rs.randint(2)), bool(rs.randint(2))
        alpha, beta = float(np.float16(rs.rand())), float(rs.choice([0.0, 1.0, -0.5]))
        a, b, c = operands(M, N, K, ta, tb, 5000 + 10 * it)
        C = gk.colmajor(c)
        p = matmatmul_plan(C, "T" if ta else "N", "T" if tb else "N", gk.colmajor(a), gk.colmajor(b), alpha, beta)
        print("case", it, (M, N, K), ta, tb, alpha, beta, p.kernel_names, flush=True)
        p()
        torch.cuda.synchronize()
        aligned_kernel_runs += "checked" not in p.kernel_names[0]
        assert oracle.rel_frobenius(gk.to_numpy(C), oracle.gemm_f64(a, b, c, alpha, beta, ta, tb)) <= 1e-3, (it, M, N, K, ta, tb)
    assert aligned_kernel_runs >= 50
