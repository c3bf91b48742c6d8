"""GPU parity of the complex and dual-number GEMM (benchmark config 4a; reference
configs/configs.jl:385-490, test sweep :656-695) against numpy complex128 and the CPU oracle.
Tolerance: relative Frobenius error <= 1e-3 (FP16 in, FP32 accumulate)."""
import numpy as np
import pytest
import torch

import gemmkernels as gk
from gemmkernels import Kernel, NT, configs, rng
import helpers
from oracle import oracle

pytestmark = pytest.mark.gpu
TOL = 1e-3


def to_c128(x):            # (2, rows, cols) -> complex (rows, cols)
    return x[0].astype(np.float64) + 1j * x[1].astype(np.float64)


def run(conf, a, b, c, M, N):
    ta, tb = gk.colmajor(a), gk.colmajor(b)
    tc = None if c is None else gk.colmajor(c)
    td = gk.colmajor_empty((2, M, N), torch.float32)
    td.fill_(float("nan"))
    gk.matmul(conf, ta, tb, tc, td, kernel=Kernel.matmul_pipelined)
    torch.cuda.synchronize()
    return gk.to_numpy(td)


def _tiles(ta, tb, dual=False):
    from gemmkernels import config as cfg, Operator, Float16, Float32
    op = (Operator.MFMADualOp if dual else Operator.MFMAComplexOp)[16, 16, 16, Float16, Float32]
    return [t for t, _ in cfg._complex_tiles(op, False, ta, not tb)]


TRANSPOSES = [(False, False), (False, True), (True, False), (True, True)]
CASES = [(ta, tb, block) for ta, tb in TRANSPOSES for block in _tiles(ta, tb)]


def test_complex_d_as_a_window(gpu):
    """D as a window of a larger complex matrix (leading dimension beyond M) on the four-wave kernel of 'N','N': same bits
    as in a matrix of its own, nothing written outside the window."""
    M, N, K = 256, 384, 320
    conf = configs.complex_config(M, N, K, False, False, zero_c=True, block_shape=gk.NT(M=128, N=128, K=64))
    assert "_w2x2" in gk.kernel_name(conf, Kernel.matmul_pipelined)
    a = configs.complex_matrix(71, M, K)
    b = configs.complex_matrix(72, K, N)
    plain = run(conf, a, b, None, M, N)
    want = to_c128(a) @ to_c128(b)
    assert oracle.rel_frobenius(plain[0], want.real) <= TOL and oracle.rel_frobenius(plain[1], want.imag) <= TOL
    ld = M + 24
    big = gk.colmajor_empty((2, ld, N), torch.float32)
    big.fill_(float("nan"))
    D = big[:, :M, :]
    gk.matmul(conf, gk.colmajor(a), gk.colmajor(b), None, D, kernel=Kernel.matmul_pipelined)
    torch.cuda.synchronize()
    assert np.array_equal(D.cpu().numpy(), plain)
    assert bool(torch.isnan(big[:, M:, :]).all())


@pytest.mark.parametrize("ta,tb,block", CASES)
@pytest.mark.parametrize("zero_c", [True, False])
def test_complex_all_transposes(gpu, ta, tb, block, zero_c):
    """Every compiled tile of every transpose (one real product of the real views of A and B), with and without C."""
    M, N, K = 2 * block[0], 3 * block[1], 5 * block[2]
    conf = configs.complex_config(M, N, K, ta, tb, zero_c=zero_c, block_shape=gk.NT(M=block[0], N=block[1], K=block[2]))
    a = configs.complex_matrix(61, K if ta else M, M if ta else K)
    b = configs.complex_matrix(62, N if tb else K, K if tb else N)
    c = None if zero_c else rng.matrix("upm1_f32", 63, (2, M, N))
    name = gk.kernel_name(conf, Kernel.matmul_pipelined)
    print("case", block, ta, tb, zero_c, name, flush=True)
    assert "pair" in name
    d = run(conf, a, b, c, M, N)
    A = to_c128(a).T if ta else to_c128(a)          # 'T' is a plain transpose, no conjugation (src/matmul.jl:211-213)
    B = to_c128(b).T if tb else to_c128(b)
    want = A @ B + (0 if zero_c else to_c128(c))
    assert oracle.rel_frobenius(d[0], want.real) <= TOL and oracle.rel_frobenius(d[1], want.imag) <= TOL
    # the CPU oracle restates WMMAComplexOp.mma (src/operator.jl:307-311)
    ref = np.zeros((2, M, N), np.float32, order="F")
    p = helpers.oracle_problem(conf, (a.shape[1], b.shape[1], M, M))
    oracle.matmul(p, a, b, c, ref)
    assert oracle.rel_frobenius(to_c128(d), to_c128(ref)) <= TOL


@pytest.mark.parametrize("ta,tb", TRANSPOSES)
def test_complex_default_tile_and_odd_k(gpu, ta, tb):
    """The tile the defaults pick, for a K that only the 32-deep tiles divide and for a large product."""
    for M, N, K in [(128, 192, 96), (512, 256, 320)]:
        conf = configs.complex_config(M, N, K, ta, tb)
        a = configs.complex_matrix(64, K if ta else M, M if ta else K)
        b = configs.complex_matrix(65, N if tb else K, K if tb else N)
        print("case", (M, N, K), ta, tb, gk.kernel_name(conf, Kernel.matmul_pipelined), flush=True)
        d = run(conf, a, b, None, M, N)
        A = to_c128(a).T if ta else to_c128(a)
        B = to_c128(b).T if tb else to_c128(b)
        assert oracle.rel_frobenius(to_c128(d), A @ B) <= TOL


def _hooked(conf, a, b, c, M, N, transforms, bias, cd_np=np.float32):
    """(GPU result, oracle result) of a complex product with hooks on C / D and a bias."""
    import torch
    from gemmkernels import Epilogue
    ta_, tb_ = gk.colmajor(a), gk.colmajor(b)
    tc = None if c is None else gk.colmajor(c)
    td = gk.colmajor_empty((2, M, N), torch.float16 if cd_np == np.float16 else torch.float32)
    td.fill_(float("nan"))
    tbias = None if bias is None else torch.from_numpy(bias).cuda()
    epi = None if bias is None else Epilogue.Bias(tbias)
    gk.matmul(conf, ta_, tb_, tc, td, epilogue=epi, kernel=Kernel.matmul_pipelined, **transforms)
    torch.cuda.synchronize()
    ref = np.zeros((2, M, N), cd_np, order="F")
    p = helpers.oracle_problem(conf, (a.shape[1], b.shape[1], M, M), transforms, epi, bias)
    oracle.matmul(p, a, b, c, ref)
    return gk.to_numpy(td), ref


@pytest.mark.parametrize("ta,tb", TRANSPOSES)
@pytest.mark.parametrize("dual", [False, True])
def test_hooks_and_bias_on_complex(gpu, ta, tb, dual):
    """Hooks of C and D and the bias on the complex and dual operators (the eight hooks of the reference are
    operator-agnostic, src/kernel.jl:167-187, 337-347): z * s and -z act on both parts, z + c and the (real) bias on
    the real part.  Checked against the oracle, and the oracle's complex hooks against numpy in tests/test_oracle.py."""
    from gemmkernels import Transform
    M, N, K = 128, 192, 128
    conf = configs.complex_config(M, N, K, ta, tb, zero_c=False, dual=dual)
    a = configs.complex_matrix(66, K if ta else M, M if ta else K)
    b = configs.complex_matrix(67, N if tb else K, K if tb else N)
    c = rng.matrix("upm1_f32", 68, (2, M, N))
    bias = rng.normal_f32(69, N)
    transforms = dict(transform_global_to_shared_c=Transform.Elementwise(lambda x: x * 2.0),
                      transform_shared_to_regs_c=Transform.Elementwise(lambda x: x + 0.75),
                      transform_regs_to_shared_d=Transform.Elementwise(lambda x: -(x * 0.5)),
                      transform_shared_to_global_d=Transform.Elementwise(lambda x: x + 0.25))
    print("case", ta, tb, dual, gk.kernel_name(conf, Kernel.matmul_pipelined, transforms=transforms), flush=True)
    d, ref = _hooked(conf, a, b, c, M, N, transforms, bias)
    assert np.isfinite(d).all()
    assert oracle.rel_frobenius(d[0], ref[0]) <= TOL and oracle.rel_frobenius(d[1], ref[1]) <= TOL
    if not dual:
        A = to_c128(a).T if ta else to_c128(a)
        B = to_c128(b).T if tb else to_c128(b)
        want = -((A @ B + (2.0 * to_c128(c) + 0.75)) * 0.5) + bias[None, :].astype(np.float64) + 0.25
        assert oracle.rel_frobenius(d[0], want.real) <= TOL and oracle.rel_frobenius(d[1], want.imag) <= TOL


@pytest.mark.parametrize("ta,tb", TRANSPOSES)
@pytest.mark.parametrize("dual", [False, True])
def test_scale_and_negation_of_a_and_b_on_complex(gpu, ta, tb, dual):
    """Hooks on A and B of the complex and dual operators (the reference's hooks are operator-agnostic,
    src/kernel.jl:224-236, 311-319): a scale by a power of two and a negation are real factors, act on both parts and
    commute with the product, so they are folded into the accumulators.  Against the oracle, which applies them to the
    operands, against numpy, and exactly on dyadic data (the fold must not cost a single bit)."""
    from gemmkernels import Transform
    M, N, K = 128, 192, 128
    conf = configs.complex_config(M, N, K, ta, tb, zero_c=False, dual=dual)
    a = configs.complex_matrix(166, K if ta else M, M if ta else K)
    b = configs.complex_matrix(167, N if tb else K, K if tb else N)
    c = rng.matrix("upm1_f32", 168, (2, M, N))
    transforms = dict(transform_global_to_shared_a=Transform.Elementwise(lambda x: x * 0.25),
                      transform_shared_to_regs_b=Transform.Elementwise(lambda x: -x),
                      transform_shared_to_global_d=Transform.Elementwise(lambda x: x * 2.0))
    print("case", ta, tb, dual, gk.kernel_name(conf, Kernel.matmul_pipelined, transforms=transforms), flush=True)
    d, ref = _hooked(conf, a, b, c, M, N, transforms, None)
    assert np.isfinite(d).all()
    assert oracle.rel_frobenius(d[0], ref[0]) <= 1e-5 and oracle.rel_frobenius(d[1], ref[1]) <= 1e-5
    if not dual:
        A = to_c128(a).T if ta else to_c128(a)
        B = to_c128(b).T if tb else to_c128(b)
        want = 2.0 * ((0.25 * A) @ (-B) + to_c128(c))
        assert oracle.rel_frobenius(d[0], want.real) <= TOL and oracle.rel_frobenius(d[1], want.imag) <= TOL
    # dyadic data: every product and every partial sum is exact in FP32, folded or not
    rs = np.random.RandomState(170)
    ai = np.asfortranarray(rs.randint(-4, 5, size=a.shape).astype(np.float16))
    bi = np.asfortranarray(rs.randint(-4, 5, size=b.shape).astype(np.float16))
    ci = np.asfortranarray(rs.randint(-64, 65, size=c.shape).astype(np.float32))
    di, refi = _hooked(conf, ai, bi, ci, M, N, transforms, None)
    assert np.array_equal(di, refi)


def test_complex_fp16_c_and_d(gpu):
    """Complex{Float16} C and D: fp32 accumulation, one rounding at the store."""
    from gemmkernels import Float16
    M, N, K = 128, 128, 192
    for ta, tb in TRANSPOSES:
        conf = configs.complex_config(M, N, K, ta, tb, zero_c=False, cd_type=Float16)
        a = configs.complex_matrix(70, K if ta else M, M if ta else K)
        b = configs.complex_matrix(71, N if tb else K, K if tb else N)
        c = rng.matrix("upm1_f16", 72, (2, M, N))
        d, ref = _hooked(conf, a, b, c, M, N, {}, None, np.float16)
        assert d.dtype == np.float16 and np.isfinite(d).all()
        A = to_c128(a).T if ta else to_c128(a)
        B = to_c128(b).T if tb else to_c128(b)
        assert oracle.rel_frobenius(to_c128(d), A @ B + to_c128(c)) <= 2e-3      # half an ulp of FP16 on top
        assert np.mean(d.view(np.uint16) != ref.view(np.uint16)) < 2e-3          # same rounding as the oracle's single one


def test_complex_hooks_that_are_not_defined_are_refused(gpu):
    from gemmkernels import Transform, ConfigError, _lib
    M = N = K = 128
    conf = configs.complex_config(M, N, K)
    a = gk.colmajor(configs.complex_matrix(73, M, K))
    b = gk.colmajor(configs.complex_matrix(74, K, N))
    d = gk.colmajor_empty((2, M, N), torch.float32)
    for kw in (dict(transform_shared_to_global_d=Transform.Elementwise(Transform.relu)),          # max(z, 0) has no complex method
               dict(transform_regs_to_shared_d=Transform.Elementwise(lambda x: abs(x))),         # abs(z) is real
               dict(transform_global_to_shared_a=Transform.Elementwise(lambda x: x * 3.0)),      # A / B hooks: what folds into the accumulators only
               dict(transform_shared_to_regs_b=Transform.Elementwise(lambda x: x * 64.0)),       # a power of two beyond the folded range
               dict(transform_shared_to_regs_a=Transform.Elementwise(lambda x: x + 1.0))):
        with pytest.raises(ConfigError) as ei:
            gk.matmul(conf, a, b, None, d, kernel=Kernel.matmul_pipelined, **kw)
        assert ei.value.status == _lib.GK_ERR_UNSUPPORTED, ei.value.message


def test_complex_identities_and_c(gpu):
    M = N = K = 128
    conf = configs.complex_config(M, N, K, block_shape=gk.NT(M=64, N=64, K=32))
    a = configs.complex_matrix(71, M, K)
    b = configs.complex_matrix(72, K, N)
    a_real, b_real = a.copy(order="F"), b.copy(order="F")
    a_real[1] = 0
    b_real[1] = 0
    d = run(conf, a_real, b_real, None, M, N)
    assert np.all(d[1] == 0)                                   # real inputs => imaginary part exactly zero
    bi = np.zeros((2, K, N), np.float16, order="F")
    bi[1, np.arange(K), np.arange(K)] = 1                      # B = i * I  =>  A * B = (-im A, re A)
    d = run(conf, a, bi, None, M, N)
    assert np.array_equal(d[0], -a[1].astype(np.float32)) and np.array_equal(d[1], a[0].astype(np.float32))
    conf_c = configs.complex_config(M, N, K, zero_c=False, block_shape=gk.NT(M=64, N=64, K=32))
    c = rng.matrix("upm1_f32", 73, (2, M, N))
    d = run(conf_c, a, b, c, M, N)
    assert oracle.rel_frobenius(to_c128(d), to_c128(a) @ to_c128(b) + to_c128(c)) <= TOL


@pytest.mark.parametrize("ta,tb,block", [(ta, tb, block) for ta, tb in TRANSPOSES for block in _tiles(ta, tb, dual=True)])
def test_dual_numbers(gpu, ta, tb, block):
    """(re, du): re = a_re b_re, du = a_re b_du + a_du b_re (reference src/operator.jl:366-369)."""
    M, N, K = 2 * block[0], 2 * block[1], 3 * block[2]
    conf = configs.complex_config(M, N, K, ta, tb, dual=True, block_shape=gk.NT(M=block[0], N=block[1], K=block[2]))
    a = configs.complex_matrix(81, K if ta else M, M if ta else K)
    b = configs.complex_matrix(82, N if tb else K, K if tb else N)
    print("case", block, ta, tb, gk.kernel_name(conf, Kernel.matmul_pipelined), flush=True)
    d = run(conf, a, b, None, M, N)
    a0, a1 = (x.astype(np.float64).T if ta else x.astype(np.float64) for x in (a[0], a[1]))
    b0, b1 = (x.astype(np.float64).T if tb else x.astype(np.float64) for x in (b[0], b[1]))
    assert oracle.rel_frobenius(d[0], a0 @ b0) <= TOL
    assert oracle.rel_frobenius(d[1], a0 @ b1 + a1 @ b0) <= TOL
    # and against the oracle's dual-number product (itself pinned against these float64 forms on the CPU)
    ref = np.zeros((2, M, N), np.float32, order="F")
    p = helpers.oracle_problem(conf, (a.shape[1], b.shape[1], M, M))
    assert p.op_kind == oracle.OP_DUAL
    oracle.matmul(p, a, b, None, ref)
    assert oracle.rel_frobenius(d[0], ref[0]) <= TOL and oracle.rel_frobenius(d[1], ref[1]) <= TOL


def test_config4a_full_size(gpu):
    w = configs.benchmark_config("4a")
    r = w.prepare()
    r()
    torch.cuda.synchronize()
    h = w.host()
    d = to_c128(gk.to_numpy(r.d))
    ref = (to_c128(h["a"]).astype(np.complex64) @ to_c128(h["b"]).astype(np.complex64))
    assert oracle.rel_frobenius(d, ref) <= TOL


def planar(seed, rows, cols, dtype=np.float16):
    """Planar complex matrix as a real array of logical shape (rows, cols, 2), column-major."""
    kind = "upm1_f16" if dtype == np.float16 else "upm1_f32"
    return rng.matrix(kind, seed, (rows * cols, 2)).reshape((rows, cols, 2), order="F")


def planar_to_c128(x):
    return x[:, :, 0].astype(np.float64) + 1j * x[:, :, 1].astype(np.float64)


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("zero_c", [True, False])
def test_planar_global_layouts(gpu, ta, tb, zero_c):
    """Complex GEMM on split re / im global arrays (Layout.SplitColMajor / SplitRowMajor as global
    layouts): real GEMMs on the planes with the sign pattern of WMMAComplexOp.mma (src/operator.jl:307-311)."""
    M, N, K = 256, 384, 192
    conf = configs.complex_planar_config(M, N, K, ta, tb, zero_c=zero_c)
    a = planar(81, K if ta else M, M if ta else K)
    b = planar(82, N if tb else K, K if tb else N)
    c = None if zero_c else planar(83, M, N, np.float32)
    ta_, tb_ = gk.colmajor(a), gk.colmajor(b)
    tc = None if zero_c else gk.colmajor(c)
    td = gk.colmajor_empty((M, N, 2), torch.float32)
    td.fill_(float("nan"))
    gk.matmul(conf, ta_, tb_, tc, td, kernel=Kernel.matmul_pipelined)
    torch.cuda.synchronize()
    A = planar_to_c128(a).T if ta else planar_to_c128(a)
    B = planar_to_c128(b).T if tb else planar_to_c128(b)
    ref = A @ B + (0 if zero_c else planar_to_c128(c))
    d = planar_to_c128(gk.to_numpy(td))
    assert np.isfinite(d).all()
    assert oracle.rel_frobenius(d, ref) <= TOL
    if not zero_c:      # in place, mul! style: d is c
        gk.matmul(conf, ta_, tb_, tc, tc, kernel=Kernel.matmul_pipelined)
        torch.cuda.synchronize()
        assert oracle.rel_frobenius(planar_to_c128(gk.to_numpy(tc)), ref) <= TOL


def _run_planar(M, N, K, ta, tb, zero_c, block=None, seed=90):
    kw = {} if block is None else dict(block_shape=NT(M=block[0], N=block[1], K=block[2]))
    conf = configs.complex_planar_config(M, N, K, ta, tb, zero_c=zero_c, **kw)
    a = planar(seed + 1, K if ta else M, M if ta else K)
    b = planar(seed + 2, N if tb else K, K if tb else N)
    c = None if zero_c else planar(seed + 3, M, N, np.float32)
    ta_, tb_ = gk.colmajor(a), gk.colmajor(b)
    tc = None if zero_c else gk.colmajor(c)
    td = gk.colmajor_empty((M, N, 2), torch.float32)
    td.fill_(float("nan"))
    gk.matmul(conf, ta_, tb_, tc, td, kernel=Kernel.matmul_pipelined)
    torch.cuda.synchronize()
    A = planar_to_c128(a).T if ta else planar_to_c128(a)
    B = planar_to_c128(b).T if tb else planar_to_c128(b)
    ref = A @ B + (0 if zero_c else planar_to_c128(c))
    d = planar_to_c128(gk.to_numpy(td))
    assert np.isfinite(d).all()
    return conf, oracle.rel_frobenius(d, ref), oracle.rel_frobenius(d.real, ref.real), oracle.rel_frobenius(d.imag, ref.imag)


@pytest.mark.parametrize("block", [(128, 128, 64), (64, 64, 64), (64, 64, 32), (32, 32, 32)])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_planar_kernel_every_tile(gpu, block, ta, tb):
    """The single-launch kernel for planar matrices, every compiled tile and transpose, C read: each
    plane of D is checked on its own (a wrong sign or a swapped plane leaves the other one intact)."""
    M, N, K = 2 * block[0], 3 * block[1], 5 * block[2]
    conf, err, err_re, err_im = _run_planar(M, N, K, ta, tb, False, block)
    assert "planar" in gk.kernel_name(conf, Kernel.matmul_pipelined)
    assert err <= TOL and err_re <= TOL and err_im <= TOL


@pytest.mark.parametrize("ta,tb", TRANSPOSES)
def test_planar_hooks_and_bias(gpu, ta, tb):
    """Hooks of C and D and the bias on planar matrices: the same rules as on interleaved ones (a plane is a part)."""
    from gemmkernels import Transform, Epilogue
    M, N, K = 128, 256, 128
    conf = configs.complex_planar_config(M, N, K, ta, tb, zero_c=False)
    a = planar(111, K if ta else M, M if ta else K)
    b = planar(112, N if tb else K, K if tb else N)
    c = planar(113, M, N, np.float32)
    bias = rng.normal_f32(114, N)
    tbias = torch.from_numpy(bias).cuda()
    transforms = dict(transform_global_to_shared_c=Transform.Elementwise(lambda x: x * 2.0),
                      transform_shared_to_regs_c=Transform.Elementwise(lambda x: x + 0.75),
                      transform_regs_to_shared_d=Transform.Elementwise(lambda x: -(x * 0.5)),
                      transform_shared_to_global_d=Transform.Elementwise(lambda x: x + 0.25))
    td = gk.colmajor_empty((M, N, 2), torch.float32)
    td.fill_(float("nan"))
    gk.matmul(conf, gk.colmajor(a), gk.colmajor(b), gk.colmajor(c), td, epilogue=Epilogue.Bias(tbias), kernel=Kernel.matmul_pipelined, **transforms)
    torch.cuda.synchronize()
    A = planar_to_c128(a).T if ta else planar_to_c128(a)
    B = planar_to_c128(b).T if tb else planar_to_c128(b)
    want = -((A @ B + (2.0 * planar_to_c128(c) + 0.75)) * 0.5) + bias[None, :].astype(np.float64) + 0.25
    d = planar_to_c128(gk.to_numpy(td))
    assert np.isfinite(d).all()
    assert oracle.rel_frobenius(d.real, want.real) <= TOL and oracle.rel_frobenius(d.imag, want.imag) <= TOL


@pytest.mark.parametrize("ktiles", [1, 2, 3])
def test_planar_kernel_short_k(gpu, ktiles):
    """K of one to three tiles: shorter than the pipeline is deep."""
    for block in [(128, 128, 64), (64, 64, 32)]:
        _, err, err_re, err_im = _run_planar(block[0], block[1], ktiles * block[2], False, False, True, block, seed=95)
        assert err <= TOL and err_re <= TOL and err_im <= TOL


def test_planar_operands_with_separate_planes_fall_back_to_real_gemms(gpu):
    """Planes that do not follow each other in memory (a view into a wider array) run as real GEMMs on
    the planes; same result."""
    M, N, K = 128, 256, 96
    conf = configs.complex_planar_config(M, N, K, False, False, zero_c=True)
    a, b = planar(101, M, K), planar(102, K, N)
    wide_a = gk.colmajor_empty((M, K + 8, 2), torch.float16)
    wide_a.zero_()
    wide_a[:, :K, :] = gk.colmajor(a)
    ta_ = wide_a[:, :K, :]
    assert ta_.stride(2) != ta_.stride(1) * ta_.size(1)
    td = gk.colmajor_empty((M, N, 2), torch.float32)
    gk.matmul(conf, ta_, gk.colmajor(b), None, td, kernel=Kernel.matmul_pipelined)
    torch.cuda.synchronize()
    ref = planar_to_c128(a) @ planar_to_c128(b)
    assert oracle.rel_frobenius(planar_to_c128(gk.to_numpy(td)), ref) <= TOL


def test_config4a_planar_full_size(gpu):
    """Benchmark config 4a on planar arrays at its full size (2048^3), one launch; both planes checked
    against a complex64 product of the same inputs."""
    w = configs.benchmark_config("4a-planar")
    assert "planar" in w.kernel_name
    r = w.prepare()
    r()
    torch.cuda.synchronize()
    h = w.host()
    d = planar_to_c128(gk.to_numpy(r.d))
    ref = planar_to_c128(h["a"]).astype(np.complex64) @ planar_to_c128(h["b"]).astype(np.complex64)
    assert oracle.rel_frobenius(d.real, ref.real) <= TOL
    assert oracle.rel_frobenius(d.imag, ref.imag) <= TOL


@pytest.mark.parametrize("dual", [False, True])
@pytest.mark.parametrize("zero_c", [True, False])
def test_four_waves_give_the_bits_of_eight_waves(gpu, dual, zero_c):
    """'N','N' on interleaved matrices: the 256 x 256 x 64 real tile on four waves, one per SIMD (a lane's four rows
    of a block are two complex numbers; the four real products of an element of D lie in two blocks of the lane)."""
    M, N, K = 256, 384, 320
    blk = dict(block_shape=gk.NT(M=128, N=128, K=64))
    four = configs.complex_config(M, N, K, zero_c=zero_c, dual=dual, **blk)
    eight = configs.complex_config(M, N, K, zero_c=zero_c, dual=dual, warps_per_block=8, compute_warp=gk.NT(M=64, N=32, K=16), **blk)
    n4, n8 = gk.kernel_name(four, Kernel.matmul_pipelined), gk.kernel_name(eight, Kernel.matmul_pipelined)
    print("case", dual, zero_c, n4, n8, flush=True)
    assert four.warps_per_block == 4 and n4.endswith("_w2x2") and n8.endswith("_w2x4")
    a, b = configs.complex_matrix(71, M, K), configs.complex_matrix(72, K, N)
    c = None if zero_c else rng.matrix("upm1_f32", 73, (2, M, N))
    d4, d8 = run(four, a, b, c, M, N), run(eight, a, b, c, M, N)
    assert np.array_equal(d4, d8)
    if not dual:
        want = to_c128(a) @ to_c128(b) + (0 if zero_c else to_c128(c))
        assert oracle.rel_frobenius(d4[0], want.real) <= TOL and oracle.rel_frobenius(d4[1], want.imag) <= TOL


def test_four_wave_complex_configuration_falls_back(gpu):
    """Other transposes, hooks and a bias run the eight-wave arrangement of the same tile."""
    from gemmkernels import Transform, Epilogue
    M, N, K = 256, 256, 128
    blk = dict(block_shape=gk.NT(M=128, N=128, K=64), warps_per_block=4, compute_warp=gk.NT(M=64, N=64, K=16))
    for ta, tb in [(False, True), (True, False), (True, True)]:
        conf = configs.complex_config(M, N, K, ta, tb, **blk)
        assert gk.kernel_name(conf, Kernel.matmul_pipelined).endswith("_w2x4")
    conf = configs.complex_config(M, N, K, **blk)
    assert gk.kernel_name(conf, Kernel.matmul_pipelined).endswith("_w2x2")
    hooks = dict(transform_shared_to_global_d=Transform.Elementwise(lambda x: x * 2.0))
    assert gk.kernel_name(conf, Kernel.matmul_pipelined, transforms=hooks).endswith("_w2x4")
    a, b = configs.complex_matrix(74, M, K), configs.complex_matrix(75, K, N)
    ta_, tb_ = gk.colmajor(a), gk.colmajor(b)
    td = gk.colmajor_empty((2, M, N), torch.float32)
    gk.matmul(conf, ta_, tb_, None, td, kernel=Kernel.matmul_pipelined, **hooks)
    torch.cuda.synchronize()
    want = 2.0 * (to_c128(a) @ to_c128(b))
    d = gk.to_numpy(td)
    assert oracle.rel_frobenius(d[0], want.real) <= TOL and oracle.rel_frobenius(d[1], want.imag) <= TOL


@pytest.mark.parametrize("ta,tb", TRANSPOSES)
@pytest.mark.parametrize("zero_c", [True, False])
def test_planar_four_waves_give_the_bits_of_eight_waves(gpu, ta, tb, zero_c):
    """Planar matrices on the one-wave-per-SIMD arrangement (every transpose: the planes are plain real operands)."""
    M, N, K = 256, 384, 192
    blk = dict(block_shape=NT(M=128, N=128, K=64))
    four = configs.complex_planar_config(M, N, K, ta, tb, zero_c=zero_c, **blk)
    eight = configs.complex_planar_config(M, N, K, ta, tb, zero_c=zero_c, warps_per_block=8, compute_warp=NT(M=64, N=32, K=16), **blk)
    n4, n8 = gk.kernel_name(four, Kernel.matmul_pipelined), gk.kernel_name(eight, Kernel.matmul_pipelined)
    print("case", ta, tb, zero_c, n4, n8, flush=True)
    assert four.warps_per_block == 4 and n4.endswith("_w2x2") and n8.endswith("_w2x4") and "planar" in n4
    a = planar(101, K if ta else M, M if ta else K)
    b = planar(102, N if tb else K, K if tb else N)
    c = None if zero_c else planar(103, M, N, np.float32)
    out = []
    for conf in (four, eight):
        td = gk.colmajor_empty((M, N, 2), torch.float32)
        td.fill_(float("nan"))
        gk.matmul(conf, gk.colmajor(a), gk.colmajor(b), None if zero_c else gk.colmajor(c), td, kernel=Kernel.matmul_pipelined)
        torch.cuda.synchronize()
        out.append(gk.to_numpy(td))
    assert np.array_equal(out[0], out[1])
    A = planar_to_c128(a).T if ta else planar_to_c128(a)
    B = planar_to_c128(b).T if tb else planar_to_c128(b)
    assert oracle.rel_frobenius(planar_to_c128(out[0]), A @ B + (0 if zero_c else planar_to_c128(c))) <= TOL
    # with a hook the launch runs on eight waves
    from gemmkernels import Transform
    hooks = dict(transform_shared_to_global_d=Transform.Elementwise(lambda x: x * 2.0))
    assert gk.kernel_name(four, Kernel.matmul_pipelined, transforms=hooks).endswith("_w2x4")
