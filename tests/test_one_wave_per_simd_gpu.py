"""The tiles that run on four waves (one per SIMD: 256 x 256 x 64 with 128 x 128 wave tiles, the tiles with a side of 192
with 128 x 96 / 96 x 128) against the CPU oracle and the float64 product, which are the gate (relative Frobenius error
<= 1e-3 like the other MFMA tests; <= 1e-6 against float64 where the test says so).

Comparisons with the eight-wave arrangement of the same tile come on top of that and say two different things.  Where the
summation order is the same by construction -- C loaded before the K loop or absent, tiles over the edges, the fused,
complex and contraction kernels: the k-steps and the products inside them run in the same order however a tile is dealt
out to waves -- the two must agree bit for bit, which catches a wrong register, lane or address that a norm would let
pass.  Where C is added during the first K tiles (plain products of at least eleven K tiles with FP32 or FP16 C / D) the place of
that one addition differs, so the two agree to rounding only; there the tests pin what the order cannot change: linearity
in C, D(C) - D(0) = C, and sums of small integers, which are exact in any order.

Launches the four waves are not compiled for (hooks on A, B or C, more than one op in a hook of D, extents the edge
instances do not take) run the eight-wave arrangement of the same configuration."""
import numpy as np
import pytest

import gemmkernels as gk
from gemmkernels import Layout, Operator, Kernel, Transform, Epilogue, NT, Float16, Float32, BFloat16, rng
import helpers
from oracle import oracle

pytestmark = pytest.mark.gpu
TOL = 1e-3
BLOCK = (256, 256, 64)


def config(M, N, K, ta, tb, waves, ab=Float16, c=Float32, d=Float32, zero_c=False, checked=False, block=BLOCK):
    col = Layout.ColMajor if checked else Layout.UnsafeAlignedColMajor
    row = Layout.RowMajor if checked else Layout.UnsafeAlignedRowMajor
    return gk.get_config(
        gemm_shape=NT(M=M, N=N, K=K), block_shape=NT(M=block[0], N=block[1], K=block[2]),
        warps_per_block=waves[0] * waves[1], compute_warp=NT(M=block[0] // waves[0], N=block[1] // waves[1], K=16),
        operator=Operator.MFMAOp[32, 32, 16, ab, Float32],
        global_a_layout=(row if ta else col)[ab], global_b_layout=(row if tb else col)[ab],
        global_c_layout=Layout.Zero[c] if zero_c else col[c], global_d_layout=col[d],
        is_a_col_major=not ta, is_b_col_major=not tb)


def operands(M, N, K, ta, tb, seed):
    a = rng.matrix("upm1_f16", seed + 1, (K, M) if ta else (M, K))
    b = rng.matrix("upm1_f16", seed + 2, (N, K) if tb else (K, N))
    c = rng.matrix("upm1_f32", seed + 3, (M, N))
    return a, b, c


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("K", [64, 128, 192, 448])
def test_same_bits_as_eight_waves(gpu, ta, tb, K):
    """One, two, three and seven K tiles: the pipeline start, the superfluous read-ahead of the last tile."""
    M, N = 512, 768
    a, b, c = operands(M, N, K, ta, tb, 7000 + K)
    four, eight = config(M, N, K, ta, tb, (2, 2)), config(M, N, K, ta, tb, (2, 4))
    name = gk.kernel_name(four, Kernel.matmul_pipelined)
    print("case", ta, tb, K, name, flush=True)
    assert "_w2x2_" in name and "_w2x4_" in gk.kernel_name(eight, Kernel.matmul_pipelined)
    d4 = helpers.run_gpu(four, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    d8 = helpers.run_gpu(eight, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d4, d8)
    assert oracle.rel_frobenius(d4, helpers.run_oracle(four, a, b, c, (M, N))) <= TOL
    assert oracle.rel_frobenius(d4, oracle.gemm_f64(a, b, c, 1.0, 1.0, ta, tb)) <= TOL


def test_zero_c_and_d_in_place(gpu):
    M, N, K = 256, 512, 320
    a, b, c = operands(M, N, K, False, False, 7100)
    conf = config(M, N, K, False, False, (2, 2), zero_c=True)
    d = helpers.run_gpu(conf, a, b, None, (M, N), kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d, helpers.run_gpu(config(M, N, K, False, False, (2, 4), zero_c=True), a, b, None, (M, N), kernel=Kernel.matmul_pipelined))
    assert oracle.rel_frobenius(d, oracle.gemm_f64(a, b, None, 1.0, 0.0, False, False)) <= TOL
    # d aliases c (reference src/matmul.jl:198)
    conf = config(M, N, K, False, False, (2, 2))
    d_alias = helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_pipelined, alias_cd=True)
    assert np.array_equal(d_alias, helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_pipelined))


@pytest.mark.parametrize("c16,d16", [(True, True), (False, True), (True, False)])
def test_16_bit_c_and_d(gpu, c16, d16):
    """C / D that are not FP32 go element by element (the 16-byte accesses are those of FP32 columns)."""
    import torch
    M, N, K = 512, 256, 256
    a, b, c32 = operands(M, N, K, True, False, 7200)
    c = rng.matrix("upm1_f16", 7204, (M, N)) if c16 else c32
    kw = dict(c=Float16 if c16 else Float32, d=Float16 if d16 else Float32)
    dt = torch.float16 if d16 else torch.float32
    d4 = helpers.run_gpu(config(M, N, K, True, False, (2, 2), **kw), a, b, c, (M, N), d_dtype=dt, kernel=Kernel.matmul_pipelined)
    d8 = helpers.run_gpu(config(M, N, K, True, False, (2, 4), **kw), a, b, c, (M, N), d_dtype=dt, kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d4, d8)
    assert oracle.rel_frobenius(d4, oracle.gemm_f64(a, b, c, 1.0, 1.0, True, False)) <= TOL


def test_bf16_operands(gpu):
    import torch
    M, N, K = 256, 256, 192
    a = gk.bf16_bits(rng.matrix("upm1_f32", 7301, (M, K)))      # uint16 arrays are bfloat16 bit patterns
    b = gk.bf16_bits(rng.matrix("upm1_f32", 7302, (K, N)))
    c = rng.matrix("upm1_f32", 7303, (M, N))
    four, eight = config(M, N, K, False, False, (2, 2), ab=BFloat16), config(M, N, K, False, False, (2, 4), ab=BFloat16)
    assert "_w2x2_" in gk.kernel_name(four, Kernel.matmul_pipelined)
    d4 = helpers.run_gpu(four, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d4, helpers.run_gpu(eight, a, b, c, (M, N), kernel=Kernel.matmul_pipelined))
    assert oracle.rel_frobenius(d4, helpers.run_oracle(four, a, b, c, (M, N))) <= TOL


def test_c_and_d_off_a_16_byte_boundary(gpu):
    """Bounds-checked layouts take any pointer: C and D that start 4 bytes into a 16-byte line go element by element."""
    import torch
    M, N, K = 256, 256, 128
    a, b, c = operands(M, N, K, False, False, 7400)
    conf = config(M, N, K, False, False, (2, 2), checked=True)
    assert "_w2x2_" in gk.kernel_name(conf, Kernel.matmul_pipelined)
    A, B = gk.colmajor(a), gk.colmajor(b)
    cbuf = torch.zeros(M * N + 1, dtype=torch.float32, device="cuda")
    dbuf = torch.full((M * N + 1,), float("nan"), dtype=torch.float32, device="cuda")
    C = cbuf[1:].view(N, M).t()
    D = dbuf[1:].view(N, M).t()
    C.copy_(torch.from_numpy(c).cuda())
    assert C.data_ptr() % 16 == 4 and D.data_ptr() % 16 == 4
    gk.matmul(conf, A, B, C, D, kernel=Kernel.matmul_pipelined)
    torch.cuda.synchronize()
    d = D.cpu().numpy()
    assert np.array_equal(d, helpers.run_gpu(config(M, N, K, False, False, (2, 4)), a, b, c, (M, N), kernel=Kernel.matmul_pipelined))


@pytest.mark.parametrize("epilogue_cls", [Epilogue.Bias, Epilogue.BiasRow])
@pytest.mark.parametrize("with_c", [False, True])
def test_hooks_of_d_in_closed_form_and_a_bias_run_on_four_waves(gpu, epilogue_cls, with_c):
    """At most one op in each hook of D, a bias, and (where there is no C) a power-of-two scale of A folded into the
    accumulators: the shape of benchmark config 3.  The four waves apply them without walking op lists."""
    M, N, K = 512, 256, 192
    a, b, c = operands(M, N, K, False, True, 7500)
    E = Transform.Elementwise
    hooks = dict(transform_regs_to_shared_d=E(Transform.relu), transform_shared_to_global_d=E(lambda x: x * 3.0))
    if not with_c:
        hooks["transform_global_to_shared_a"] = E(lambda x: x * 0.5)
    bias = rng.normal_f32(7504, N if epilogue_cls is Epilogue.Bias else M)
    four, eight = config(M, N, K, False, True, (2, 2), zero_c=not with_c), config(M, N, K, False, True, (2, 4), zero_c=not with_c)
    name = gk.kernel_name(four, Kernel.matmul_pipelined, transforms=hooks, epilogue=epilogue_cls(None))
    print("with hooks:", name, flush=True)
    assert "_w2x2_" in name and name.endswith("_fused_d")
    assert "_w2x4_" in gk.kernel_name(eight, Kernel.matmul_pipelined, transforms=hooks, epilogue=epilogue_cls(None))
    cc = c if with_c else None
    d4 = helpers.run_gpu(four, a, b, cc, (M, N), transforms=hooks, epilogue_cls=epilogue_cls, bias=bias, kernel=Kernel.matmul_pipelined)
    d8 = helpers.run_gpu(eight, a, b, cc, (M, N), transforms=hooks, epilogue_cls=epilogue_cls, bias=bias, kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d4, d8)
    ref = helpers.run_oracle(four, a, b, cc, (M, N), transforms=hooks, epilogue=epilogue_cls(0), bias=bias)
    assert oracle.rel_frobenius(d4, ref) <= TOL
    bias2d = bias[None, :] if epilogue_cls is Epilogue.Bias else bias[:, None]
    acc = (1.0 if with_c else 0.5) * (a.astype(np.float64) @ b.astype(np.float64).T) + (c.astype(np.float64) if with_c else 0.0)
    assert oracle.rel_frobenius(d4, 3.0 * (np.maximum(acc, 0.0) + bias2d)) <= TOL
    # a bias alone, and one op alone
    assert gk.kernel_name(four, Kernel.matmul_pipelined, epilogue=epilogue_cls(None)).endswith("_fused_d")
    only = dict(transform_shared_to_global_d=E(lambda x: Transform.clamp(x, -1.0, 2.0)))
    d4 = helpers.run_gpu(four, a, b, cc, (M, N), transforms=only, kernel=Kernel.matmul_pipelined)
    d8 = helpers.run_gpu(eight, a, b, cc, (M, N), transforms=only, kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d4, d8)


@pytest.mark.parametrize("case", ["no C", "C before the loop", "bias per column", "bias per row"])
def test_d_as_a_window_on_the_paths_that_store_from_a_scalar_base(gpu, case):
    """D (and C) as windows of larger matrices, leading dimension beyond M, on the four-wave paths that take the block
    column's origin from scalar registers: no C, C loaded before a short K loop, hooks of D in closed form with either bias.
    Same bits as in a matrix of its own; nothing written outside the window."""
    import torch
    M, N, K = 512, 256, 192
    a, b, c = operands(M, N, K, False, False, 7550)
    E = Transform.Elementwise
    with_c = case == "C before the loop"
    hooks, epi_cls, bias = None, None, None
    if case.startswith("bias"):
        hooks = dict(transform_shared_to_global_d=E(Transform.relu))
        epi_cls = Epilogue.Bias if case == "bias per column" else Epilogue.BiasRow
        bias = rng.normal_f32(7554, N if epi_cls is Epilogue.Bias else M)
    conf = config(M, N, K, False, False, (2, 2), zero_c=not with_c)
    plain = helpers.run_gpu(conf, a, b, c if with_c else None, (M, N), transforms=hooks, epilogue_cls=epi_cls, bias=bias, kernel=Kernel.matmul_pipelined)
    ref = helpers.run_oracle(conf, a, b, c if with_c else None, (M, N), transforms=hooks, epilogue=epi_cls(0) if epi_cls else None, bias=bias)
    assert oracle.rel_frobenius(plain, ref) <= TOL
    ld = M + 64
    dbig = torch.full((N, ld), float("nan"), dtype=torch.float32, device="cuda")
    D = dbig.t()[:M, :]
    C = None
    if with_c:
        cbig = torch.full((N, ld), 7.0, dtype=torch.float32, device="cuda")
        C = cbig.t()[:M, :]
        C.copy_(torch.from_numpy(c).cuda())
    keep = torch.from_numpy(np.ascontiguousarray(bias, dtype=np.float32)).cuda() if bias is not None else None
    gk.matmul(conf, gk.colmajor(a), gk.colmajor(b), C, D, epilogue=epi_cls(keep) if epi_cls else None, kernel=Kernel.matmul_pipelined, **(hooks or {}))
    torch.cuda.synchronize()
    assert np.array_equal(D.cpu().numpy(), plain)
    assert bool(torch.isnan(dbig.t()[M:, :]).all())


def test_other_hooks_run_on_eight_waves(gpu):
    """Hooks on C, two ops in one hook of D, a scale folded next to a C, hooks on A that stay in the K loop."""
    M, N, K = 512, 256, 128
    a, b, c = operands(M, N, K, False, False, 7550)
    conf = config(M, N, K, False, False, (2, 2))
    E = Transform.Elementwise
    cases = [dict(transform_global_to_shared_c=E(lambda x: x * 0.25)),
             dict(transform_shared_to_global_d=E(lambda x: Transform.relu(x) * 2.0)),
             dict(transform_global_to_shared_a=E(lambda x: x * 0.5)),                # folded, but C would have to be scaled the other way
             dict(transform_global_to_shared_a=E(lambda x: x * 0.75))]               # not a power of two: runs in the K loop
    for hooks in cases:
        name = gk.kernel_name(conf, Kernel.matmul_pipelined, transforms=hooks)
        print("hooks", list(hooks), name, flush=True)
        assert "_w2x4_" in name and "fused" in name
        d = helpers.run_gpu(conf, a, b, c, (M, N), transforms=hooks, kernel=Kernel.matmul_pipelined)
        ref = helpers.run_gpu(config(M, N, K, False, False, (2, 4)), a, b, c, (M, N), transforms=hooks, kernel=Kernel.matmul_pipelined)
        assert np.array_equal(d, ref)
        assert oracle.rel_frobenius(d, helpers.run_oracle(conf, a, b, c, (M, N), transforms=hooks)) <= TOL


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("M,N,K", [(264, 520, 136), (512, 776, 104), (1000, 8, 197), (256, 256, 100), (8, 1032, 64)])
def test_tiles_over_the_edges_same_bits_as_eight_waves(gpu, ta, tb, M, N, K):
    """M and N multiples of 8: edge tiles leave out what lies outside D, the partial last K tile runs behind the loop
    (one whole tile in front of it, several, none after it; a K that is odd)."""
    a, b, c = operands(M, N, K, ta, tb, 7700 + M + K)
    four, eight = config(M, N, K, ta, tb, (2, 2), checked=True), config(M, N, K, ta, tb, (2, 4), checked=True)
    name = gk.kernel_name(four, Kernel.matmul_pipelined)
    print("case", ta, tb, M, N, K, name, flush=True)
    assert "_w2x2_" in name and name.endswith("_edges") and "_w2x4_" in gk.kernel_name(eight, Kernel.matmul_pipelined)
    d4 = helpers.run_gpu(four, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    d8 = helpers.run_gpu(eight, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d4, d8)
    assert oracle.rel_frobenius(d4, helpers.run_oracle(four, a, b, c, (M, N))) <= TOL
    assert oracle.rel_frobenius(d4, oracle.gemm_f64(a, b, c, 1.0, 1.0, ta, tb)) <= TOL


def test_tiles_over_the_edges_without_c_in_place_and_off_a_16_byte_boundary(gpu):
    import torch
    M, N, K = 520, 264, 232
    a, b, c = operands(M, N, K, False, False, 7800)
    four, eight = config(M, N, K, False, False, (2, 2), checked=True), config(M, N, K, False, False, (2, 4), checked=True)
    zero4, zero8 = (config(M, N, K, False, False, w, zero_c=True, checked=True) for w in ((2, 2), (2, 4)))
    assert "_w2x2_" in gk.kernel_name(zero4, Kernel.matmul_pipelined)
    d = helpers.run_gpu(zero4, a, b, None, (M, N), kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d, helpers.run_gpu(zero8, a, b, None, (M, N), kernel=Kernel.matmul_pipelined))
    assert oracle.rel_frobenius(d, oracle.gemm_f64(a, b, None, 1.0, 0.0, False, False)) <= TOL
    # d aliases c (reference src/matmul.jl:198)
    ref = helpers.run_gpu(eight, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    assert np.array_equal(helpers.run_gpu(four, a, b, c, (M, N), kernel=Kernel.matmul_pipelined, alias_cd=True), ref)
    # C and D that start 4 bytes into a 16-byte line; nothing outside D is written
    A, B = gk.colmajor(a), gk.colmajor(b)
    cbuf = torch.zeros(M * N + 1, dtype=torch.float32, device="cuda")
    dbuf = torch.full((M * N + 9,), float("nan"), dtype=torch.float32, device="cuda")
    C = cbuf[1:].view(N, M).t()
    D = dbuf[1:1 + M * N].view(N, M).t()
    C.copy_(torch.from_numpy(c).cuda())
    gk.matmul(four, A, B, C, D, kernel=Kernel.matmul_pipelined)
    torch.cuda.synchronize()
    assert np.array_equal(D.cpu().numpy(), ref)
    assert bool(torch.isnan(dbuf[0])) and bool(torch.isnan(dbuf[1 + M * N:]).all())


@pytest.mark.parametrize("M,LD", [(264, 272), (261, 272), (263, 272), (264, 273), (262, 275)])
def test_nothing_is_written_outside_d(gpu, M, LD):
    """D as a window of a larger matrix (leading dimension beyond M, columns on and off 16-byte boundaries) whose other
    elements keep their values."""
    import torch
    N, K = 136, 128
    a, b, c = operands(M, N, K, False, True, 7850)
    col = Layout.ColMajor
    conf = gk.get_config(
        gemm_shape=NT(M=M, N=N, K=K), block_shape=NT(M=256, N=256, K=64), warps_per_block=4, compute_warp=NT(M=128, N=128, K=16),
        operator=Operator.MFMAOp[32, 32, 16, Float16, Float32],
        global_a_layout=col[Float16], global_b_layout=Layout.RowMajor[Float16], global_c_layout=col[Float32], global_d_layout=col[Float32],
        is_a_col_major=True, is_b_col_major=False)
    assert "_w2x2_" in gk.kernel_name(conf, Kernel.matmul_pipelined)
    big = torch.full((N + 3, LD), float("nan"), dtype=torch.float32, device="cuda")
    Dw = big[1:1 + N, :M].t()                     # M x N, column-major with leading dimension LD
    Cw = torch.zeros((N, LD), dtype=torch.float32, device="cuda")[:, :M].t()
    Cw.copy_(torch.from_numpy(c).cuda())
    gk.matmul(conf, gk.colmajor(a), gk.colmajor(b), Cw, Dw, kernel=Kernel.matmul_pipelined)      # ('T' B: stored N x K)
    torch.cuda.synchronize()
    assert oracle.rel_frobenius(Dw.cpu().numpy(), oracle.gemm_f64(a, b, c, 1.0, 1.0, False, True)) <= TOL
    outside = big.clone()
    outside[1:1 + N, :M] = float("nan")
    assert bool(torch.isnan(outside).all()) and not bool(torch.isnan(big[1:1 + N, :M]).any())


@pytest.mark.parametrize("ta,tb,M,N,K", [
    (False, False, 264, 515, 100),     # an odd N
    (True, False, 260, 515, 136),
    (True, True, 260, 517, 197),
    # operands whose 16-byte chunks run along M or N and reach over the edge: the last K tile runs behind the loop
    (False, False, 260, 515, 128), (False, False, 260, 515, 100), (False, False, 260, 515, 64),
    (True, True, 260, 517, 192), (False, True, 516, 262, 320),
    # M not in fours: the group of four rows that reaches over the last row of C / D goes element by element, and the
    # columns of C / D are not 16-byte aligned
    (False, False, 257, 512, 128), (False, False, 258, 300, 64), (False, False, 259, 513, 197), (False, False, 261, 512, 128),
    (True, False, 258, 512, 128), (False, True, 511, 258, 100), (True, True, 1001, 33, 203), (False, False, 1001, 1003, 1005)])
def test_any_extents(gpu, ta, tb, M, N, K):
    """Tiles over the edges at any M, N and K (M of at least 8, K of at least 64): same bits as eight waves."""
    a, b, c = operands(M, N, K, ta, tb, 7900 + M + N)
    four, eight = config(M, N, K, ta, tb, (2, 2), checked=True), config(M, N, K, ta, tb, (2, 4), checked=True)
    name = gk.kernel_name(four, Kernel.matmul_pipelined)
    print("case", ta, tb, M, N, K, name, flush=True)
    assert "_w2x2_" in name and name.endswith("_edges")
    d4 = helpers.run_gpu(four, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d4, helpers.run_gpu(eight, a, b, c, (M, N), kernel=Kernel.matmul_pipelined))
    assert oracle.rel_frobenius(d4, oracle.gemm_f64(a, b, c, 1.0, 1.0, ta, tb)) <= TOL
    # ... without C, and with D in the place of C
    zero4, zero8 = (config(M, N, K, ta, tb, w, zero_c=True, checked=True) for w in ((2, 2), (2, 4)))
    assert np.array_equal(helpers.run_gpu(zero4, a, b, None, (M, N), kernel=Kernel.matmul_pipelined),
                          helpers.run_gpu(zero8, a, b, None, (M, N), kernel=Kernel.matmul_pipelined))
    assert np.array_equal(helpers.run_gpu(four, a, b, c, (M, N), kernel=Kernel.matmul_pipelined, alias_cd=True), d4)


def test_16_bit_d_and_short_products_with_tiles_over_the_edges_run_on_eight_waves(gpu):
    import torch
    M2, N2, K2 = 302, 520, 136
    a2, b2, c2 = operands(M2, N2, K2, False, False, 7510)
    ragged = config(M2, N2, K2, False, False, (2, 2), d=Float16, checked=True)
    assert "_w2x4_" in gk.kernel_name(ragged, Kernel.matmul_pipelined)
    d2 = helpers.run_gpu(ragged, a2, b2, c2, (M2, N2), d_dtype=torch.float16, kernel=Kernel.matmul_pipelined)
    assert oracle.rel_frobenius(d2, oracle.gemm_f64(a2, b2, c2, 1.0, 1.0, False, False)) <= TOL
    short = config(M2, N2, 40, False, False, (2, 2), checked=True)
    assert "_w2x4_" in gk.kernel_name(short, Kernel.matmul_pipelined)


def test_default_configuration_of_a_large_product(gpu):
    """get_config picks the four-wave arrangement for plain products made of whole 256 x 256 x 64 tiles."""
    M = N = K = 1024
    col = Layout.UnsafeAlignedColMajor
    conf = gk.get_config(gemm_shape=NT(M=M, N=N, K=K), operator=Operator.MFMAOp[32, 32, 16, Float16, Float32],
                         global_a_layout=col[Float16], global_c_layout=col[Float32], block_shape=NT(M=256, N=256, K=64))
    assert conf.warps_per_block == 4 and (conf.compute_warp.M, conf.compute_warp.N) == (128, 128)
    a, b, c = operands(M, N, K, False, False, 7600)
    d = helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    assert oracle.rel_frobenius(d, helpers.run_oracle(conf, a, b, c, (M, N))) <= TOL


# --- C on its way during the first K tiles (products of at least eleven K tiles, FP32 C and D with 16-byte accesses) -------------
# The sum runs (products of the first K tiles) + C + (the rest) there, where the eight-wave arrangement starts from C: results
# are compared with the oracle and with float64 by norm, and exactly on data whose partial sums are all exact in FP32.

@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("K", [704, 768, 1344, 2240, 2304, 2880])
def test_c_streamed_during_the_first_k_tiles(gpu, ta, tb, K):
    """Eleven K tiles (the fewest that take this route: nine that bring C in, none in between, the two last), twelve, twenty-one;
    from thirty-five K tiles on C comes in two blocks per K tile (thirty-three tiles that bring it in, the two last): the fewest,
    one more, forty-five."""
    M, N = 512, 768
    a, b, c = operands(M, N, K, ta, tb, 7600 + K)
    conf = config(M, N, K, ta, tb, (2, 2))
    print("case", ta, tb, K, gk.kernel_name(conf, Kernel.matmul_pipelined), flush=True)
    d = helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    assert oracle.rel_frobenius(d, helpers.run_oracle(conf, a, b, c, (M, N))) <= TOL
    assert oracle.rel_frobenius(d, oracle.gemm_f64(a, b, c, 1.0, 1.0, ta, tb)) <= 1e-6
    # linearity in C, which pins that every element of C went into its own accumulator exactly once: D(C) - D(0) = C
    d0 = helpers.run_gpu(config(M, N, K, ta, tb, (2, 2), zero_c=True), a, b, None, (M, N), kernel=Kernel.matmul_pipelined)
    assert np.abs((d.astype(np.float64) - d0) - c).max() <= 1e-4
    # small integers: every partial sum is exact, whatever the place of C in the sum
    rs = np.random.RandomState(K)
    ai = np.asfortranarray(rs.randint(-4, 5, size=a.shape).astype(np.float16))
    bi = np.asfortranarray(rs.randint(-4, 5, size=b.shape).astype(np.float16))
    ci = np.asfortranarray(rs.randint(-999, 1000, size=(M, N)).astype(np.float32))
    di = helpers.run_gpu(conf, ai, bi, ci, (M, N), kernel=Kernel.matmul_pipelined)
    assert np.array_equal(di.astype(np.float64), oracle.gemm_f64(ai, bi, ci, 1.0, 1.0, ta, tb))
    # the eight-wave arrangement adds the same products in the same order but for the place of C: same values to rounding
    d8 = helpers.run_gpu(config(M, N, K, ta, tb, (2, 4)), a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    assert oracle.rel_frobenius(d, d8.astype(np.float64)) <= 1e-6


def test_c_streamed_d_in_place_and_as_a_window(gpu):
    """d aliases c (reference src/matmul.jl:198): every workgroup has read its C tile before it writes the same tile of D.
    C and D as windows of larger matrices (leading dimension beyond M)."""
    import torch
    M, N, K = 256, 512, 960
    a, b, c = operands(M, N, K, False, False, 7700)
    conf = config(M, N, K, False, False, (2, 2))
    ref = oracle.gemm_f64(a, b, c, 1.0, 1.0, False, False)
    d_alias = helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_pipelined, alias_cd=True)
    assert np.array_equal(d_alias, helpers.run_gpu(conf, a, b, c, (M, N), kernel=Kernel.matmul_pipelined))
    assert oracle.rel_frobenius(d_alias, ref) <= 1e-6
    ld = M + 64
    cbig = torch.full((N, ld), 7.0, dtype=torch.float32, device="cuda")
    dbig = torch.full((N, ld), float("nan"), dtype=torch.float32, device="cuda")
    C, D = cbig.t()[:M, :], dbig.t()[:M, :]
    C.copy_(torch.from_numpy(c).cuda())
    gk.matmul(conf, gk.colmajor(a), gk.colmajor(b), C, D, kernel=Kernel.matmul_pipelined)
    torch.cuda.synchronize()
    assert np.array_equal(D.cpu().numpy(), d_alias)
    assert bool(torch.isnan(dbig.t()[M:, :]).all())            # nothing written outside the window


def test_c_streamed_bf16_operands(gpu):
    M, N, K = 256, 256, 832
    a = gk.bf16_bits(rng.matrix("upm1_f32", 7801, (M, K)))
    b = gk.bf16_bits(rng.matrix("upm1_f32", 7802, (K, N)))
    c = rng.matrix("upm1_f32", 7803, (M, N))
    four = config(M, N, K, False, False, (2, 2), ab=BFloat16)
    d4 = helpers.run_gpu(four, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    assert oracle.rel_frobenius(d4, helpers.run_oracle(four, a, b, c, (M, N))) <= TOL
    d8 = helpers.run_gpu(config(M, N, K, False, False, (2, 4), ab=BFloat16), a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
    assert oracle.rel_frobenius(d4, d8.astype(np.float64)) <= 1e-6


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("K", [704, 1344])
def test_c_streamed_fp16_c_and_d(gpu, ta, tb, K):
    """An FP16 C and an FP16 D that take 8-byte accesses come in and go out the same way (C one block column per K tile,
    widened where it is added; D rounded once, to nearest even, where it is stored)."""
    import torch
    M, N = 512, 768
    a, b, _ = operands(M, N, K, ta, tb, 7900 + K)
    c = rng.matrix("upm1_f16", 7904 + K, (M, N))
    kw = dict(c=Float16, d=Float16)
    conf = config(M, N, K, ta, tb, (2, 2), **kw)
    d = helpers.run_gpu(conf, a, b, c, (M, N), d_dtype=torch.float16, kernel=Kernel.matmul_pipelined)
    assert oracle.rel_frobenius(d, helpers.run_oracle(conf, a, b, c, (M, N), d_dtype=np.float16)) <= TOL
    ref = oracle.gemm_f64(a, b, c, 1.0, 1.0, ta, tb)
    # one rounding to FP16: half a unit in the last place of every element (2^-11 relative)
    assert np.all(np.abs(d.astype(np.float64) - ref) <= np.abs(ref) * 2.0 ** -11 + 1e-4)
    # sums of small integers that FP16 represents: exact wherever C enters the sum
    rs = np.random.RandomState(K)
    ai = np.asfortranarray(rs.randint(-1, 2, size=a.shape).astype(np.float16))
    bi = np.asfortranarray(rs.randint(-1, 2, size=b.shape).astype(np.float16))
    ci = np.asfortranarray(rs.randint(-500, 501, size=(M, N)).astype(np.float16))
    di = helpers.run_gpu(conf, ai, bi, ci, (M, N), d_dtype=torch.float16, kernel=Kernel.matmul_pipelined)
    assert np.array_equal(di.astype(np.float64), oracle.gemm_f64(ai, bi, ci, 1.0, 1.0, ta, tb))
    # the eight waves start from C and round the same way: the same values but for the last place of a few
    d8 = helpers.run_gpu(config(M, N, K, ta, tb, (2, 4), **kw), a, b, c, (M, N), d_dtype=torch.float16, kernel=Kernel.matmul_pipelined)
    assert np.mean(d != d8) <= 1e-3
    assert oracle.rel_frobenius(d, d8.astype(np.float64)) <= 1e-4


def test_c_streamed_fp16_c_and_d_in_place_and_as_a_window(gpu):
    """d aliases c; C and D as windows of larger FP16 matrices: nothing is written outside."""
    import torch
    M, N, K = 256, 512, 960
    a, b, _ = operands(M, N, K, False, False, 7950)
    c = rng.matrix("upm1_f16", 7953, (M, N))
    conf = config(M, N, K, False, False, (2, 2), c=Float16, d=Float16)
    ref = oracle.gemm_f64(a, b, c, 1.0, 1.0, False, False)
    plain = helpers.run_gpu(conf, a, b, c, (M, N), d_dtype=torch.float16, kernel=Kernel.matmul_pipelined)
    d_alias = helpers.run_gpu(conf, a, b, c, (M, N), d_dtype=torch.float16, kernel=Kernel.matmul_pipelined, alias_cd=True)
    assert np.array_equal(d_alias, plain)
    assert oracle.rel_frobenius(plain, ref) <= TOL
    ld = M + 8
    cbig = torch.full((N, ld), 7.0, dtype=torch.float16, device="cuda")
    dbig = torch.full((N, ld), float("nan"), dtype=torch.float16, device="cuda")
    C, D = cbig.t()[:M, :], dbig.t()[:M, :]
    C.copy_(torch.from_numpy(c).cuda())
    gk.matmul(conf, gk.colmajor(a), gk.colmajor(b), C, D, kernel=Kernel.matmul_pipelined)
    torch.cuda.synchronize()
    assert np.array_equal(D.cpu().numpy(), plain)
    assert bool(torch.isnan(dbig.t()[M:, :]).all())            # nothing written outside the window


# The tiles with a side of 192 on four waves (wave tiles of 128 x 96 and 96 x 128: 48 accumulator blocks per wave),
# compiled per transpose like their eight-wave arrangements (4 x 2 and 2 x 4 waves).
WIDE = [((256, 192, 64), (4, 2), [(False, False), (True, False), (False, True)]), ((192, 256, 64), (2, 4), [(True, False), (True, True)])]


@pytest.mark.parametrize("block,eight,transposes", WIDE)
def test_tiles_with_a_side_of_192_on_four_waves(gpu, block, eight, transposes):
    """C added at the end (fewer than eleven K tiles) and no C: the same bits as the eight waves.  C on its way during
    the first K tiles (from eleven K tiles on: 704 is the fewest, 1344 has generic tiles in between; from 27 on, 1728, in
    thinner slices): the oracle, linearity in C, exact sums of small integers."""
    BM, BN, _ = block
    M, N = 2 * BM, 3 * BN
    for ta, tb in transposes:
        for K in (64, 192, 448, 704, 768, 1344, 1728, 1792, 2368):       # (from 27 K tiles on: C two blocks per K tile)
            a, b, c = operands(M, N, K, ta, tb, 7900 + K)
            four, eight8 = config(M, N, K, ta, tb, (2, 2), block=block), config(M, N, K, ta, tb, eight, block=block)
            name = gk.kernel_name(four, Kernel.matmul_pipelined)
            print("case", block, ta, tb, K, name, flush=True)
            assert "_w2x2_" in name and "_w%dx%d_" % eight in gk.kernel_name(eight8, Kernel.matmul_pipelined)
            d4 = helpers.run_gpu(four, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
            d8 = helpers.run_gpu(eight8, a, b, c, (M, N), kernel=Kernel.matmul_pipelined)
            assert oracle.rel_frobenius(d4, helpers.run_oracle(four, a, b, c, (M, N))) <= TOL
            assert oracle.rel_frobenius(d4, oracle.gemm_f64(a, b, c, 1.0, 1.0, ta, tb)) <= 1e-6
            z4 = helpers.run_gpu(config(M, N, K, ta, tb, (2, 2), zero_c=True, block=block), a, b, None, (M, N), kernel=Kernel.matmul_pipelined)
            z8 = helpers.run_gpu(config(M, N, K, ta, tb, eight, zero_c=True, block=block), a, b, None, (M, N), kernel=Kernel.matmul_pipelined)
            assert np.array_equal(z4, z8)
            if K < 704:
                assert np.array_equal(d4, d8)
                continue
            assert oracle.rel_frobenius(d4, d8.astype(np.float64)) <= 1e-6
            # every element of C went into its own accumulator exactly once
            assert np.abs((d4.astype(np.float64) - z4) - c).max() <= 1e-4
            rs = np.random.RandomState(K)
            ai = np.asfortranarray(rs.randint(-4, 5, size=a.shape).astype(np.float16))
            bi = np.asfortranarray(rs.randint(-4, 5, size=b.shape).astype(np.float16))
            ci = np.asfortranarray(rs.randint(-999, 1000, size=(M, N)).astype(np.float32))
            di = helpers.run_gpu(four, ai, bi, ci, (M, N), kernel=Kernel.matmul_pipelined)
            assert np.array_equal(di.astype(np.float64), oracle.gemm_f64(ai, bi, ci, 1.0, 1.0, ta, tb))


@pytest.mark.parametrize("block,eight,transposes", WIDE)
def test_what_the_four_waves_of_a_192_tile_leave_to_the_eight(gpu, block, eight, transposes):
    """A hook, a bias, a 16-bit D, tiles over the edges and BF16 operands on a configuration of 2 x 2 waves: the first four
    run the eight-wave arrangement of the same tile with the same bits, BF16 runs on the four waves."""
    import torch
    BM, BN, _ = block
    ta, tb = transposes[0]
    M, N, K = BM, 2 * BN, 832
    a, b, c = operands(M, N, K, ta, tb, 8100)
    four, eight8 = config(M, N, K, ta, tb, (2, 2), block=block), config(M, N, K, ta, tb, eight, block=block)
    E = Transform.Elementwise
    tr = dict(transform_shared_to_global_d=E(Transform.relu))
    assert "_w%dx%d_" % eight in gk.kernel_name(four, Kernel.matmul_pipelined, transforms=tr)
    d4 = helpers.run_gpu(four, a, b, c, (M, N), transforms=tr, kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d4, helpers.run_gpu(eight8, a, b, c, (M, N), transforms=tr, kernel=Kernel.matmul_pipelined))
    assert oracle.rel_frobenius(d4, helpers.run_oracle(four, a, b, c, (M, N), transforms=tr)) <= TOL
    bias = rng.normal_f32(8104, N)
    d4 = helpers.run_gpu(four, a, b, c, (M, N), epilogue_cls=Epilogue.Bias, bias=bias, kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d4, helpers.run_gpu(eight8, a, b, c, (M, N), epilogue_cls=Epilogue.Bias, bias=bias, kernel=Kernel.matmul_pipelined))
    assert oracle.rel_frobenius(d4, helpers.run_oracle(four, a, b, c, (M, N), epilogue=Epilogue.Bias(0), bias=bias)) <= TOL
    # a 16-bit D is found out at the launch (the kernel's name still tells the configured arrangement)
    kw = dict(d=Float16, block=block)
    d4 = helpers.run_gpu(config(M, N, K, ta, tb, (2, 2), **kw), a, b, c, (M, N), d_dtype=torch.float16, kernel=Kernel.matmul_pipelined)
    d8 = helpers.run_gpu(config(M, N, K, ta, tb, eight, **kw), a, b, c, (M, N), d_dtype=torch.float16, kernel=Kernel.matmul_pipelined)
    assert np.array_equal(d4, d8)
    assert oracle.rel_frobenius(d4, oracle.gemm_f64(a, b, c, 1.0, 1.0, ta, tb)) <= TOL
    # tiles over the edges (bounds-checked layouts)
    Mr, Nr, Kr = BM + 40, BN + 72, 840
    ar, br, cr = operands(Mr, Nr, Kr, ta, tb, 8200)
    ragged = config(Mr, Nr, Kr, ta, tb, (2, 2), checked=True, block=block)
    assert "_w%dx%d_" % eight in gk.kernel_name(ragged, Kernel.matmul_pipelined)
    dr = helpers.run_gpu(ragged, ar, br, cr, (Mr, Nr), kernel=Kernel.matmul_pipelined)
    assert oracle.rel_frobenius(dr, oracle.gemm_f64(ar, br, cr, 1.0, 1.0, ta, tb)) <= 1e-6
    # BF16 operands
    ab = gk.bf16_bits(rng.matrix("upm1_f32", 8301, a.shape))
    bb = gk.bf16_bits(rng.matrix("upm1_f32", 8302, b.shape))
    fourb = config(M, N, K, ta, tb, (2, 2), ab=BFloat16, block=block)
    assert "_w2x2_" in gk.kernel_name(fourb, Kernel.matmul_pipelined)
    db = helpers.run_gpu(fourb, ab, bb, c, (M, N), kernel=Kernel.matmul_pipelined)
    assert oracle.rel_frobenius(db, helpers.run_oracle(fourb, ab, bb, c, (M, N))) <= TOL
    d8b = helpers.run_gpu(config(M, N, K, ta, tb, eight, ab=BFloat16, block=block), ab, bb, c, (M, N), kernel=Kernel.matmul_pipelined)
    assert oracle.rel_frobenius(db, d8b.astype(np.float64)) <= 1e-6
