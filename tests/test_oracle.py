"""Pins the CPU oracle (the C restatement in oracle/gk_oracle.c) before it is trusted as the
checker: conversions against numpy, GEMM against float64 matmul and pure-Python brute force,
closed forms, layouts with index-distinct values, transform and epilogue order."""
import itertools

import numpy as np
import pytest

from oracle import oracle
from oracle.oracle import F16, BF16, F32, F64, Layout, Problem


def test_half_conversions_match_numpy_exhaustively():
    lib = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    got = np.array([lib.gko_half_to_float(int(b)) for b in bits], dtype=np.float32)
    finite = np.isfinite(ref)
    assert np.array_equal(got[finite], ref[finite]) and np.isnan(got[~finite & np.isnan(ref)]).all()
    rs = np.random.RandomState(0)
    xs = np.concatenate([rs.standard_normal(20000), rs.standard_normal(5000) * 1e-6, rs.standard_normal(5000) * 7e4,
                         np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 2.0 ** -24, 2.0 ** -25, 3 * 2.0 ** -25, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11])])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    have = np.array([lib.gko_double_to_half(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(have, want)


def plain(M, N, K, ta=False, tb=False, dt=F16, cd=F32, zero_c=False, **kw):
    a = Layout(oracle.L_ROW if ta else oracle.L_COL, dt, K if ta else M)
    b = Layout(oracle.L_ROW if tb else oracle.L_COL, dt, N if tb else K)
    c = Layout(oracle.L_ZERO, cd) if zero_c else Layout(oracle.L_COL, cd, M)
    return Problem(M, N, K, a, b, c, Layout(oracle.L_COL, cd, M), compute_dtype=dt, accum_dtype=cd, **kw)


def rand(shape, dtype, seed):
    rs = np.random.RandomState(seed)
    return np.asfortranarray((rs.randint(-1024, 1024, size=shape) / 1024.0).astype(dtype))


@pytest.mark.parametrize("ta,tb", list(itertools.product([False, True], repeat=2)))
def test_gemm_against_float64_and_brute_force(ta, tb):
    M, N, K = 7, 5, 9
    a = rand((K, M) if ta else (M, K), np.float16, 1)
    b = rand((N, K) if tb else (K, N), np.float16, 2)
    c = rand((M, N), np.float32, 3)
    d = np.zeros((M, N), np.float32, order="F")
    oracle.matmul(plain(M, N, K, ta, tb), a, b, c, d)
    # pure-Python triple loop, float64 (products and partial sums of these dyadic inputs are exact)
    A = a.T if ta else a
    B = b.T if tb else b
    want = np.zeros((M, N))
    for i in range(M):
        for j in range(N):
            s = float(c[i, j])
            for k in range(K):
                s += float(A[i, k]) * float(B[k, j])
            want[i, j] = s
    assert np.array_equal(d.astype(np.float64), want)          # exact: sums of multiples of 2^-20 below 2^24
    assert np.array_equal(want, oracle.gemm_f64(a, b, c, 1.0, 1.0, ta, tb))


def test_gemm_medium_against_float64_both_accumulators():
    M, N, K = 96, 80, 200
    a, b, c = rand((M, K), np.float16, 4), rand((K, N), np.float16, 5), rand((M, N), np.float32, 6)
    d = np.zeros((M, N), np.float32, order="F")
    oracle.matmul(plain(M, N, K), a, b, c, d)
    ref = oracle.gemm_f64(a, b, c, 1.0, 1.0)
    assert oracle.rel_frobenius(d, ref) < 1e-6
    oracle.matmul(plain(M, N, K), a, b, c, d, wide_accum=True)
    assert np.array_equal(d, ref.astype(np.float32))


def test_closed_forms():
    n = 16
    eye = np.asfortranarray(np.eye(n, dtype=np.float16))
    b, c = rand((n, n), np.float16, 7), rand((n, n), np.float32, 8)
    d = np.zeros((n, n), np.float32, order="F")
    oracle.matmul(plain(n, n, n), eye, b, c, d)
    assert np.array_equal(d, b.astype(np.float32) + c)                       # A = I
    ones = np.asfortranarray(np.ones((n, n), np.float16))
    oracle.matmul(plain(n, n, n, zero_c=True), ones, ones, None, d)
    assert np.array_equal(d, np.full((n, n), float(n), np.float32))          # all ones => K
    a1 = np.zeros((n, n), np.float16, order="F"); a1[3, 5] = 2.0
    b1 = np.zeros((n, n), np.float16, order="F"); b1[5, 11] = 0.25
    oracle.matmul(plain(n, n, n, zero_c=True), a1, b1, None, d)
    want = np.zeros((n, n), np.float32); want[3, 11] = 0.5
    assert np.array_equal(d, want)                                           # single non-zero


def test_layout_index_maps_with_distinct_values():
    """Each element carries a distinct value, so a swapped index or a wrong leading dimension moves
    a known number to a wrong place."""
    M, K = 3, 4
    vals = np.arange(1, 1 + 5 * 6, dtype=np.float32)
    buf = np.asfortranarray(vals.reshape((5, 6), order="F"))                 # ld = 5 > M
    one = np.asfortranarray(np.eye(K, dtype=np.float32))
    d = np.zeros((M, K), np.float32, order="F")
    p = Problem(M, K, K, Layout(oracle.L_COL, F32, 5), Layout(oracle.L_COL, F32, K), Layout(oracle.L_ZERO, F32),
                Layout(oracle.L_COL, F32, M), compute_dtype=F32, accum_dtype=F32)
    oracle.matmul(p, buf, one, None, d)
    assert np.array_equal(d, buf[:M, :K])                                    # (r, c) at p[r + c*ld]
    p.a = Layout(oracle.L_ROW, F32, 5)
    oracle.matmul(p, buf, one, None, d)
    assert np.array_equal(d, buf[:K, :M].T)                                  # (r, c) at p[c + r*ld]
    diag = np.array([2, 3, 5, 7], np.float32)
    p2 = Problem(K, K, K, Layout(oracle.L_DIAG, F32), Layout(oracle.L_COL, F32, K), Layout(oracle.L_ZERO, F32),
                 Layout(oracle.L_COL, F32, K), compute_dtype=F32, accum_dtype=F32)
    bb = np.asfortranarray(np.arange(1, 17, dtype=np.float32).reshape((4, 4), order="F"))
    d2 = np.zeros((K, K), np.float32, order="F")
    oracle.matmul(p2, diag, bb, None, d2)
    assert np.array_equal(d2, np.diag(diag) @ bb)                            # reference src/layout.jl:225-236


def test_gett_index_map_against_einsum_with_primes():
    """D[a,b,c,d] = sum_{e,f} A[a,e,b,f] * B[d,f,c,e] with distinct extents and prime values."""
    ea, eb, ec, ed, ee, ef = 2, 3, 2, 2, 3, 2
    rs = np.random.RandomState(9)
    primes = np.array([2, 3, 5, 7, 11, 13, 17, 19, 23, 29, 31], np.float32)
    A = np.asfortranarray(rs.choice(primes, size=(ea, ee, eb, ef)).astype(np.float32))
    B = np.asfortranarray(rs.choice(primes, size=(ed, ef, ec, ee)).astype(np.float32))
    sA, sB = [s // 4 for s in A.strides], [s // 4 for s in B.strides]
    M, N, K = ea * eb, ec * ed, ee * ef
    D = np.zeros((ea, eb, ec, ed), np.float32, order="F")
    sD = [s // 4 for s in D.strides]
    la = Layout(oracle.L_GETT, F32, 0, [(ea, sA[0]), (eb, sA[2])], [(ee, sA[1]), (ef, sA[3])])     # rows m=(a,b), cols k=(e,f)
    lb = Layout(oracle.L_GETT, F32, 0, [(ee, sB[3]), (ef, sB[1])], [(ec, sB[2]), (ed, sB[0])])     # rows k=(e,f), cols n=(c,d)
    ld = Layout(oracle.L_GETT, F32, 0, [(ea, sD[0]), (eb, sD[1])], [(ec, sD[2]), (ed, sD[3])])
    p = Problem(M, N, K, la, lb, Layout(oracle.L_ZERO, F32), ld, compute_dtype=F32, accum_dtype=F32)
    oracle.matmul(p, A, B, None, D)
    want = np.einsum("aebf,dfce->abcd", A.astype(np.float64), B.astype(np.float64))
    assert np.array_equal(D.astype(np.float64), want)


def test_transform_order_rounding_points_and_bias():
    """gl2sh result is rounded to the shared type, sh2rf to the compute type, the bias is added
    before the last transform (reference src/epilogue.jl:67-70)."""
    M = N = K = 4
    a = np.asfortranarray(np.full((M, K), 1.0 + 2.0 ** -10, np.float16))     # 1 + ulp
    b = np.asfortranarray(np.eye(K, dtype=np.float16))
    d = np.zeros((M, N), np.float32, order="F")
    p = plain(M, N, K, zero_c=True, transforms={"global_to_shared_a": [(oracle.T_SCALE, 0.75, 0.0)],
                                                "shared_to_regs_a": [(oracle.T_SCALE, 4.0, 0.0)]})
    oracle.matmul(p, a, b, None, d)
    step1 = np.float16(np.float32(a[0, 0]) * np.float32(0.75))              # rounded to FP16 in LDS
    assert d[0, 0] == np.float32(np.float16(np.float32(step1) * np.float32(4.0)))
    assert d[0, 0] != np.float32(np.float32(a[0, 0]) * np.float32(3.0))      # a fused 3x would differ
    bias = np.array([1.0, -2.0, 3.0, -4.0], np.float32)
    p = plain(M, N, K, zero_c=True, transforms={"shared_to_global_d": [(oracle.T_RELU, 0.0, 0.0)]}, epilogue=oracle.EPI_BIAS_COL, bias=bias)
    zero = np.zeros((M, K), np.float16, order="F")
    oracle.matmul(p, zero, b, None, d)
    assert np.array_equal(d, np.broadcast_to(np.maximum(bias, 0)[None, :], (M, N)))
    p.epilogue = oracle.EPI_BIAS_ROW
    oracle.matmul(p, zero, b, None, d)
    assert np.array_equal(d, np.broadcast_to(np.maximum(bias, 0)[:, None], (M, N)))
    # relu before the bias (regs_to_shared_d) is a different function: relu(0) + bias = bias
    p = plain(M, N, K, zero_c=True, transforms={"regs_to_shared_d": [(oracle.T_RELU, 0.0, 0.0)]}, epilogue=oracle.EPI_BIAS_COL, bias=bias)
    oracle.matmul(p, zero, b, None, d)
    assert np.array_equal(d, np.broadcast_to(bias[None, :], (M, N)))


def test_alpha_beta_linearity_and_c_alias():
    M, N, K = 12, 10, 14
    a, b, c = rand((M, K), np.float16, 10), rand((K, N), np.float16, 11), rand((M, N), np.float32, 12)
    tr = {"shared_to_regs_a": [(oracle.T_SCALE, 2.0, 0.0)], "shared_to_regs_c": [(oracle.T_SCALE, 3.0, 0.0)]}
    cc = c.copy(order="F")
    oracle.matmul(plain(M, N, K, transforms=tr), a, b, cc, cc)               # d aliases c
    assert np.array_equal(cc.astype(np.float64), oracle.gemm_f64(a, b, c, 2.0, 3.0))


def test_fp32_fma_chain_is_sequential_in_k():
    """FPUOp.mma is a scalar fma chain in ascending k (reference src/operator.jl:139-153)."""
    K = 64
    rs = np.random.RandomState(13)
    a = np.asfortranarray(rs.standard_normal((1, K)).astype(np.float32))
    b = np.asfortranarray(rs.standard_normal((K, 1)).astype(np.float32))
    d = np.zeros((1, 1), np.float32, order="F")
    oracle.matmul(plain(1, 1, K, dt=F32, zero_c=True), a, b, None, d)
    acc = np.float64(0.0)
    for k in range(K):   # fma in float32 == round(float64 exact product + acc) for float32 inputs (product exact in f64)
        acc = np.float64(np.float32(np.float64(a[0, k]) * np.float64(b[k, 0]) + acc))
    assert d[0, 0] == np.float32(acc)


def test_complex_against_numpy_and_identities():
    M, N, K = 6, 5, 8
    rs = np.random.RandomState(14)
    def cplx(shape):
        return np.asfortranarray((rs.randint(-512, 512, size=shape + (2,)) / 512.0).astype(np.float16))
    a, b = cplx((M, K)), cplx((K, N))
    az = a[..., 0].astype(np.float64) + 1j * a[..., 1].astype(np.float64)
    bz = b[..., 0].astype(np.float64) + 1j * b[..., 1].astype(np.float64)
    def inter(x):   # (rows, cols, 2) logical -> interleaved col-major buffer
        return np.ascontiguousarray(np.transpose(x, (1, 0, 2)))          # memory: col, row, (re, im)
    p = Problem(M, N, K, Layout(oracle.L_ICOL, F16, M), Layout(oracle.L_ICOL, F16, K), Layout(oracle.L_ZERO, F32),
                Layout(oracle.L_ICOL, F32, M), compute_dtype=F16, accum_dtype=F32, op_kind=oracle.OP_COMPLEX)
    d = np.zeros((N, M, 2), np.float32)
    oracle.matmul(p, inter(a), inter(b), None, d)
    got = (d[..., 0] + 1j * d[..., 1]).T
    assert np.allclose(got, az @ bz, rtol=0, atol=1e-5)
    # real inputs => imaginary part exactly zero
    a0 = a.copy(); a0[..., 1] = 0
    b0 = b.copy(); b0[..., 1] = 0
    oracle.matmul(p, inter(a0), inter(b0), None, d)
    assert np.all(d[..., 1] == 0)
    # B = i * I  =>  A * B = (-im(A), re(A))
    bi = np.zeros((K, K, 2), np.float16); bi[np.arange(K), np.arange(K), 1] = 1
    p2 = Problem(M, K, K, Layout(oracle.L_ICOL, F16, M), Layout(oracle.L_ICOL, F16, K), Layout(oracle.L_ZERO, F32),
                 Layout(oracle.L_ICOL, F32, M), compute_dtype=F16, accum_dtype=F32, op_kind=oracle.OP_COMPLEX)
    d2 = np.zeros((K, M, 2), np.float32)
    oracle.matmul(p2, inter(a), inter(bi), None, d2)
    assert np.array_equal(d2[..., 0].T, -a[..., 1].astype(np.float32)) and np.array_equal(d2[..., 1].T, a[..., 0].astype(np.float32))


def test_tropical_and_dual():
    M, N, K = 5, 4, 6
    a, b, c = rand((M, K), np.float32, 15), rand((K, N), np.float32, 16), rand((M, N), np.float32, 17)
    d = np.zeros((M, N), np.float32, order="F")
    oracle.matmul(plain(M, N, K, dt=F32, op_kind=oracle.OP_TROPICAL), a, b, c, d)
    want = np.maximum(c, (a[:, :, None] + b[None, :, :]).max(axis=1))      # max-plus product (reference configs/configs.jl:226)
    assert np.array_equal(d, want)


@pytest.mark.parametrize("code,np_t,bits", [(oracle.I16, np.int16, 16), (oracle.I32, np.int32, 32), (oracle.I64, np.int64, 64)])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, True)])
def test_integer_gemm_wraps_like_julia(code, np_t, bits, ta, tb):
    """Int16 / Int32 / Int64 FPUOp (reference configs/configs.jl:495-497): alpha * A * B + beta * C
    with wrap-around, against exact Python integers reduced modulo 2^bits.  The magnitudes are
    chosen so that Int16 and Int32 really overflow."""
    M, N, K = 7, 5, 9
    rs = np.random.RandomState(bits)
    hi = {16: 300, 32: 70000, 64: 2 ** 40}[bits]
    a = np.asfortranarray(rs.randint(-hi, hi, size=(K, M) if ta else (M, K)).astype(np_t))
    b = np.asfortranarray(rs.randint(-hi, hi, size=(N, K) if tb else (K, N)).astype(np_t))
    c = np.asfortranarray(rs.randint(-hi, hi, size=(M, N)).astype(np_t))
    p = plain(M, N, K, ta, tb, dt=code, cd=code)
    p.transforms = {"shared_to_regs_a": [(oracle.T_SCALE, 2.0, 0.0)], "shared_to_regs_c": [(oracle.T_SCALE, 3.0, 0.0)]}
    d = np.zeros((M, N), np_t, order="F")
    oracle.matmul(p, a, b, c, d)
    A = [[int(x) for x in row] for row in (a.T if ta else a)]
    B = [[int(x) for x in row] for row in (b.T if tb else b)]
    mod, half = 1 << bits, 1 << (bits - 1)
    for i in range(M):
        for j in range(N):
            exact = 3 * int(c[i, j]) + sum(2 * A[i][k] * B[k][j] for k in range(K))
            want = (exact + half) % mod - half
            assert int(d[i, j]) == want, (i, j)
    if bits < 64:
        assert np.any(np.abs(np.array([[3 * int(c[i, j]) + sum(2 * A[i][k] * B[k][j] for k in range(K)) for j in range(N)] for i in range(M)], dtype=object)) >= half)


def test_float64_accumulation_of_float32_inputs():
    """(Float32, Float32, Float64) and (Float64, Float64, Float64) of the reference's FPUOp list
    (configs/configs.jl:491-492): products of two float32 values are exact in float64, so a short sum
    equals numpy's float64 matmul bit for bit when no rounding can occur, and agrees to a few ulps otherwise."""
    M, N, K = 6, 4, 8
    a, b = rand((M, K), np.float32, 1), rand((K, N), np.float32, 2)
    c = rand((M, N), np.float64, 3)
    p = plain(M, N, K, dt=F32, cd=F64)
    d = np.zeros((M, N), np.float64, order="F")
    oracle.matmul(p, a, b, c, d)
    assert np.array_equal(d, a.astype(np.float64) @ b.astype(np.float64) + c)      # 11-bit inputs: every partial sum is exact
    a64, b64 = np.asfortranarray(np.random.RandomState(4).standard_normal((M, K))), np.asfortranarray(np.random.RandomState(5).standard_normal((K, N)))
    p = plain(M, N, K, dt=F64, cd=F64, zero_c=True)
    oracle.matmul(p, a64, b64, None, d)
    assert np.allclose(d, a64 @ b64, rtol=1e-14, atol=1e-15)
    # sequential fma chain in ascending k
    import math
    acc = 0.0
    for k in range(K):
        acc = math.fma(a64[2, k], b64[k, 1], acc) if hasattr(math, "fma") else None
        if acc is None:
            break
    if acc is not None:
        assert d[2, 1] == acc


# ------------------------------------------------------------------------------------------------
# Elementwise ops (reference src/transform.jl:20-30 applies an arbitrary f; the closed vocabulary here is
# scale, add, relu, neg, abs, clamp, square).  Each op is pushed through oracle.matmul on a product with
# B = I, so that D[i, j] = f(A[i, j]) exactly (every other term of the sum is f(A[i, k]) * 0), and compared
# with values typed by hand and with numpy closed forms written from the definition of the op.
# ------------------------------------------------------------------------------------------------

def _through_identity(a32, hooks, hook_on="global_to_shared_a"):
    n = a32.shape[0]
    eye = np.asfortranarray(np.eye(n, dtype=np.float32))
    d = np.zeros((n, n), np.float32, order="F")
    p = plain(n, n, n, dt=F32, cd=F32, zero_c=True)
    p.transforms = {hook_on: hooks}
    if hook_on.endswith("_c"):
        # the hook under test sits on C: D = f(C) + 0 * I
        p = plain(n, n, n, dt=F32, cd=F32)
        p.transforms = {hook_on: hooks}
        oracle.matmul(p, np.zeros_like(eye), eye, np.asfortranarray(a32), d)
    else:
        oracle.matmul(p, np.asfortranarray(a32), eye, None, d)
    return d


_VALUES = np.array([[-2.0, -0.5, 0.25, 3.0],
                    [0.75, -1.25, 0.0, 1.5],
                    [-3.5, 2.0, 0.5, -0.125],
                    [1.0, -1.0, 4.0, -4.0]], dtype=np.float32)


def test_each_elementwise_op_against_hand_typed_values():
    T = oracle
    # add 0.75
    assert np.array_equal(_through_identity(_VALUES, [(T.T_ADD, 0.75, 0.0)]),
                          np.array([[-1.25, 0.25, 1.0, 3.75], [1.5, -0.5, 0.75, 2.25], [-2.75, 2.75, 1.25, 0.625], [1.75, -0.25, 4.75, -3.25]], np.float32))
    # neg
    assert np.array_equal(_through_identity(_VALUES, [(T.T_NEG, 0.0, 0.0)]),
                          np.array([[2.0, 0.5, -0.25, -3.0], [-0.75, 1.25, -0.0, -1.5], [3.5, -2.0, -0.5, 0.125], [-1.0, 1.0, -4.0, 4.0]], np.float32))
    # abs
    assert np.array_equal(_through_identity(_VALUES, [(T.T_ABS, 0.0, 0.0)]),
                          np.array([[2.0, 0.5, 0.25, 3.0], [0.75, 1.25, 0.0, 1.5], [3.5, 2.0, 0.5, 0.125], [1.0, 1.0, 4.0, 4.0]], np.float32))
    # clamp to [0.5, 2] (lower bound above zero; values below, inside, on and above the bounds)
    assert np.array_equal(_through_identity(_VALUES, [(T.T_CLAMP, 0.5, 2.0)]),
                          np.array([[0.5, 0.5, 0.5, 2.0], [0.75, 0.5, 0.5, 1.5], [0.5, 2.0, 0.5, 0.5], [1.0, 0.5, 2.0, 0.5]], np.float32))
    # clamp to [-1, -0.25] (both bounds negative: a swapped pair of bounds or a swapped comparison fails here)
    assert np.array_equal(_through_identity(_VALUES, [(T.T_CLAMP, -1.0, -0.25)]),
                          np.array([[-1.0, -0.5, -0.25, -0.25], [-0.25, -1.0, -0.25, -0.25], [-1.0, -0.25, -0.25, -0.25], [-0.25, -1.0, -0.25, -1.0]], np.float32))
    # square
    assert np.array_equal(_through_identity(_VALUES, [(T.T_SQUARE, 0.0, 0.0)]),
                          np.array([[4.0, 0.25, 0.0625, 9.0], [0.5625, 1.5625, 0.0, 2.25], [12.25, 4.0, 0.25, 0.015625], [1.0, 1.0, 16.0, 16.0]], np.float32))
    # relu and scale, for completeness of the table
    assert np.array_equal(_through_identity(_VALUES, [(T.T_RELU, 0.0, 0.0)]), np.maximum(_VALUES, 0))
    assert np.array_equal(_through_identity(_VALUES, [(T.T_SCALE, -1.5, 0.0)]), _VALUES * np.float32(-1.5))


@pytest.mark.parametrize("hook", ["global_to_shared_a", "shared_to_regs_a", "global_to_shared_c", "shared_to_regs_c",
                                  "regs_to_shared_d", "shared_to_global_d"])
def test_elementwise_ops_against_numpy_closed_forms_on_every_hook_kind(hook):
    """Random fp32 values (not dyadic: the roundings of every op matter), one op at a time and a chain of four,
    through hooks on A, on C and on D."""
    T = oracle
    rs = np.random.RandomState(7)
    x = np.asfortranarray((rs.standard_normal((4, 4)) * 3).astype(np.float32))
    f32 = np.float32
    cases = [
        ([(T.T_ADD, 0.3, 0.0)], lambda v: v + f32(0.3)),
        ([(T.T_NEG, 0.0, 0.0)], lambda v: -v),
        ([(T.T_ABS, 0.0, 0.0)], lambda v: np.abs(v)),
        ([(T.T_CLAMP, 0.4, 1.7)], lambda v: np.minimum(np.maximum(v, f32(0.4)), f32(1.7))),
        ([(T.T_SQUARE, 0.0, 0.0)], lambda v: v * v),
        # scale by 3, subtract 1, absolute value, clamp to [0.25, 2]: one fp32 rounding after each op
        ([(T.T_SCALE, 3.0, 0.0), (T.T_ADD, -1.0, 0.0), (T.T_ABS, 0.0, 0.0), (T.T_CLAMP, 0.25, 2.0)],
         lambda v: np.minimum(np.maximum(np.abs((v * f32(3.0)).astype(f32) + f32(-1.0)), f32(0.25)), f32(2.0))),
        # square, negate, add 2.5, relu
        ([(T.T_SQUARE, 0.0, 0.0), (T.T_NEG, 0.0, 0.0), (T.T_ADD, 2.5, 0.0), (T.T_RELU, 0.0, 0.0)],
         lambda v: np.maximum((-(v * v).astype(f32)) + f32(2.5), f32(0))),
    ]
    for ops, closed in cases:
        got = _through_identity(x, ops, hook)
        want = closed(x).astype(np.float32)
        assert np.array_equal(got, want), (hook, ops)
    # the clamp really cut on both sides, the chain really used all four ops
    assert (x < 0.4).any() and (x > 1.7).any() and ((x > 0.4) & (x < 1.7)).any()


@pytest.mark.parametrize("code,np_t,bits", [(oracle.I16, np.int16, 16), (oracle.I32, np.int32, 32), (oracle.I64, np.int64, 64)])
def test_integer_elementwise_ops_wrap(code, np_t, bits):
    """The integer evaluation of every op (Julia integer arithmetic wraps; abs and neg of typemin stay typemin)
    against exact Python integers reduced modulo 2^bits, with magnitudes that overflow, through B = I."""
    T = oracle
    mod, half = 1 << bits, 1 << (bits - 1)
    lo, hi = -half, half - 1
    big = {16: 200, 32: 50000, 64: 3_100_000_000}[bits]
    vals = [lo, hi, -big, big, -3, 0, 7, big + 1, -big - 5, 1, -1, 12, lo + 1, hi - 1, 100, -100]
    a = np.asfortranarray(np.array(vals, dtype=object).reshape(4, 4).astype(np_t))
    eye = np.asfortranarray(np.eye(4, dtype=np_t))
    wrap = lambda v: (v + half) % mod - half
    scale = {16: 300, 32: 70000, 64: 16_777_216}[bits]       # exactly representable as a binary32 parameter
    cases = [
        ([(T.T_SCALE, float(scale), 0.0)], lambda v: wrap(v * scale)),
        ([(T.T_ADD, float(scale), 0.0)], lambda v: wrap(v + scale)),
        ([(T.T_NEG, 0.0, 0.0)], lambda v: wrap(-v)),
        ([(T.T_ABS, 0.0, 0.0)], lambda v: wrap(abs(v))),
        ([(T.T_RELU, 0.0, 0.0)], lambda v: max(v, 0)),
        ([(T.T_CLAMP, 5.0, 100.0)], lambda v: min(max(v, 5), 100)),
        ([(T.T_CLAMP, -100.0, -5.0)], lambda v: min(max(v, -100), -5)),
        ([(T.T_SQUARE, 0.0, 0.0)], lambda v: wrap(v * v)),
        ([(T.T_SQUARE, 0.0, 0.0), (T.T_ADD, 3.0, 0.0), (T.T_NEG, 0.0, 0.0), (T.T_SCALE, float(scale), 0.0)],
         lambda v: wrap(wrap(-wrap(wrap(v * v) + 3)) * scale)),
    ]
    overflowed = False
    for ops, closed in cases:
        for hook in ("global_to_shared_a", "shared_to_global_d"):
            p = plain(4, 4, 4, dt=code, cd=code, zero_c=True)
            p.transforms = {hook: ops}
            d = np.zeros((4, 4), np_t, order="F")
            oracle.matmul(p, a, eye, None, d)
            for i in range(4):
                for j in range(4):
                    v = int(a[i, j])
                    assert int(d[i, j]) == closed(v), (ops, hook, v)
        overflowed |= any(not (lo <= int(v) * scale <= hi) for v in vals)
    assert overflowed


def test_bfloat16_conversions_match_torch_exhaustively():
    """float -> bfloat16 is round-to-nearest-even on the upper 16 bits: every upper half with the lower-half
    patterns just below a tie, on the tie (even and odd upper halves both occur), just above it, 0 and all ones,
    against torch.bfloat16; bfloat16 -> float for all 2^16 patterns."""
    import ctypes
    import torch
    lib = oracle.lib()
    lib.gko_float_to_bf16_n.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64]
    lib.gko_bf16_to_float_n.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64]
    upper = np.arange(65536, dtype=np.uint32) << 16
    for low in (0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF, 0x4000, 0xC000):
        bits = (upper | np.uint32(low)).astype(np.uint32)
        x = bits.view(np.float32).copy()
        out = np.zeros(x.size, np.uint16)
        lib.gko_float_to_bf16_n(x.ctypes.data, out.ctypes.data, x.size)
        want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
        nan = np.isnan(x)
        assert np.array_equal(out[~nan], want[~nan]), hex(low)
        # NaNs stay NaNs (payloads are not compared)
        back = (out[nan].astype(np.uint32) << 16).view(np.float32)
        assert np.isnan(back).all()
    h = np.arange(65536, dtype=np.uint16)
    f = np.zeros(65536, np.float32)
    lib.gko_bf16_to_float_n(h.ctypes.data, f.ctypes.data, h.size)
    want = torch.from_numpy(h.view(np.int16)).view(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(f.view(np.uint32), want.view(np.uint32))
    # the tie cases tell round-to-nearest-even from truncation and from round-half-up
    assert lib.gko_float_to_bf16_n is not None
    one_tie_even = np.array([0x3F808000], np.uint32).view(np.float32)      # 1.00390625: tie, even upper half -> stays 0x3F80
    one_tie_odd = np.array([0x3F818000], np.uint32).view(np.float32)       # tie, odd upper half -> rounds up to 0x3F82
    o = np.zeros(1, np.uint16)
    lib.gko_float_to_bf16_n(one_tie_even.ctypes.data, o.ctypes.data, 1); assert o[0] == 0x3F80
    lib.gko_float_to_bf16_n(one_tie_odd.ctypes.data, o.ctypes.data, 1); assert o[0] == 0x3F82


def test_bfloat16_gemm_rounds_its_output_once():
    """BF16 multiplicands, BF16 D: the oracle's result equals the float64 product rounded once by torch."""
    import torch
    M, N, K = 6, 5, 8
    rs = np.random.RandomState(3)
    af = (rs.randint(-128, 128, size=(M, K)) / 64.0).astype(np.float32)      # exactly representable in bfloat16
    bf = (rs.randint(-128, 128, size=(K, N)) / 64.0).astype(np.float32)
    to_bits = lambda x: np.asfortranarray((x.view(np.uint32) >> 16).astype(np.uint16))
    p = plain(M, N, K, dt=BF16, cd=F32, zero_c=True)
    p.d = Layout(oracle.L_COL, BF16, M)
    d = np.zeros((M, N), np.uint16, order="F")
    oracle.matmul(p, to_bits(np.asfortranarray(af)), to_bits(np.asfortranarray(bf)), None, d)
    exact = af.astype(np.float64) @ bf.astype(np.float64)                   # exact: small dyadic values
    want = torch.from_numpy(exact.astype(np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(d, want)


def test_dual_numbers_against_float64():
    """WMMADualOp (reference src/operator.jl:359-372): (a0 + a1 e)(b0 + b1 e) = a0 b0 + (a0 b1 + a1 b0) e, no
    a1 b1 term and no sign flip.  Against float64 matmuls of the parts; a complex product of the same data differs."""
    M, N, K = 6, 5, 7
    a = rand((M, K, 2), np.float16, 31)
    b = rand((K, N, 2), np.float16, 32)
    c = rand((M, N, 2), np.float32, 33)
    inter = lambda x: np.ascontiguousarray(np.transpose(x, (1, 0, 2)))       # column-major interleaved pairs
    def run(op, with_c):
        p = Problem(M, N, K, Layout(oracle.L_ICOL, F16, M), Layout(oracle.L_ICOL, F16, K),
                    Layout(oracle.L_ICOL, F32, M) if with_c else Layout(oracle.L_ZERO, F32), Layout(oracle.L_ICOL, F32, M),
                    compute_dtype=F16, accum_dtype=F32, op_kind=op)
        d = np.zeros((N, M, 2), np.float32)
        oracle.matmul(p, inter(a), inter(b), inter(c) if with_c else None, d)
        return np.transpose(d, (1, 0, 2))
    a0, a1 = a[..., 0].astype(np.float64), a[..., 1].astype(np.float64)
    b0, b1 = b[..., 0].astype(np.float64), b[..., 1].astype(np.float64)
    for with_c in (False, True):
        got = run(oracle.OP_DUAL, with_c)
        c0 = c[..., 0].astype(np.float64) if with_c else 0.0
        c1 = c[..., 1].astype(np.float64) if with_c else 0.0
        # dyadic inputs with 11 significant bits and K = 7: every partial sum is exact in fp32
        assert np.array_equal(got[..., 0].astype(np.float64), a0 @ b0 + c0)
        assert np.array_equal(got[..., 1].astype(np.float64), a0 @ b1 + a1 @ b0 + c1)
    assert not np.array_equal(run(oracle.OP_COMPLEX, False)[..., 0], run(oracle.OP_DUAL, False)[..., 0])


def test_hooks_on_complex_numbers_against_numpy_complex():
    """Hooks of a complex product see complex numbers (the reference hands tiles of the layout's element type to the
    transform, src/kernel.jl:167-187, 337-347): z * s and -z act on both parts, z + c (c real) and the real bias on
    the real part only.  Checked against numpy's own complex arithmetic on dyadic data (every step exact), on every
    hook, and the ops without a complex method of the same type are refused."""
    M, N, K = 5, 4, 6
    a = rand((M, K, 2), np.float16, 41)
    b = rand((K, N, 2), np.float16, 42)
    c = rand((M, N, 2), np.float32, 43)
    bias = np.array([0.5, -1.25, 2.0, -0.75, 1.5], np.float32)        # N values per column, M per row
    inter = lambda x: np.ascontiguousarray(np.transpose(x, (1, 0, 2)))
    z = lambda x: x[..., 0].astype(np.complex128) + 1j * x[..., 1].astype(np.complex128)
    def run(transforms, epilogue=0):
        p = Problem(M, N, K, Layout(oracle.L_ICOL, F16, M), Layout(oracle.L_ICOL, F16, K), Layout(oracle.L_ICOL, F32, M),
                    Layout(oracle.L_ICOL, F32, M), compute_dtype=F16, accum_dtype=F32, op_kind=oracle.OP_COMPLEX,
                    transforms=transforms, epilogue=epilogue, bias=bias if epilogue else None)
        d = np.zeros((N, M, 2), np.float32)
        oracle.matmul(p, inter(a), inter(b), inter(c), d)
        return z(np.transpose(d, (1, 0, 2)))
    A, B, C = z(a), z(b), z(c)
    assert np.array_equal(run({}), A @ B + C)
    # A and B hooks: (2 A + 0.5) and (-B), both hooks of each operand in turn
    for ha, hb in (("global_to_shared_a", "global_to_shared_b"), ("shared_to_regs_a", "shared_to_regs_b")):
        got = run({ha: [(oracle.T_SCALE, 2.0, 0.0), (oracle.T_ADD, 0.5, 0.0)], hb: [(oracle.T_NEG, 0.0, 0.0)]})
        assert np.array_equal(got, (2.0 * A + 0.5) @ (-B) + C)
    # C hooks, D hooks and the bias in the reference's order: regs_to_shared_d, bias, shared_to_global_d
    got = run({"global_to_shared_c": [(oracle.T_SCALE, 2.0, 0.0)], "shared_to_regs_c": [(oracle.T_ADD, 0.75, 0.0)],
               "regs_to_shared_d": [(oracle.T_SCALE, 0.5, 0.0), (oracle.T_NEG, 0.0, 0.0)],
               "shared_to_global_d": [(oracle.T_ADD, 0.25, 0.0)]}, epilogue=oracle.EPI_BIAS_COL)
    want = -((A @ B + (2.0 * C + 0.75)) * 0.5) + bias[None, :N].astype(np.complex128) + 0.25
    assert np.array_equal(got, want)
    assert np.array_equal(got.imag, (-((A @ B + 2.0 * C) * 0.5)).imag)          # nothing was added to the imaginary part
    got = run({}, epilogue=oracle.EPI_BIAS_ROW)
    assert np.array_equal(got, A @ B + C + bias[:M, None].astype(np.complex128))
    for kind in (oracle.T_RELU, oracle.T_ABS, oracle.T_CLAMP, oracle.T_SQUARE):
        with pytest.raises(Exception):
            run({"shared_to_global_d": [(kind, 0.0, 1.0)]})
