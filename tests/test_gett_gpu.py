"""GPU parity of the tensor-contraction (GETT) layouts: D[a,b,c,d] = sum_{e,f} A[a,e,b,f] * B[d,f,c,e]
(benchmark config 5) and other mode permutations, against numpy einsum, the CPU oracle's own index
map, and -- bit for bit -- the plain GEMM kernel run on explicitly materialised matrices."""
import numpy as np
import pytest
import torch

import gemmkernels as gk
from gemmkernels import Kernel, Layout, configs, rng
import helpers
from oracle import oracle

pytestmark = pytest.mark.gpu


def run_gett(conf, A, B, d_shape):
    a, b = gk.colmajor(A), gk.colmajor(B)
    d = gk.colmajor_empty(d_shape, torch.float32)
    d.fill_(float("nan"))
    gk.matmul(conf, a, b, None, d, kernel=Kernel.matmul_pipelined)
    torch.cuda.synchronize()
    return gk.to_numpy(d)


def small_ints(shape, seed):
    rs = np.random.RandomState(seed)
    return np.asfortranarray(rs.randint(-4, 5, size=shape).astype(np.float16))


def test_small_contraction_is_exact_against_einsum(gpu):
    ext = dict(a=32, b=2, c=2, d=32, e=32, f=2)
    conf, gmap = configs.gett_config("aebf", "dfce", "abcd", ext, block_shape=(64, 64, 32))
    assert gk.kernel_name(conf, Kernel.matmul_pipelined).endswith("_gett")
    A = small_ints((32, 32, 2, 2), 1)     # A[a,e,b,f]
    B = small_ints((32, 2, 2, 32), 2)     # B[d,f,c,e]
    D = run_gett(conf, A, B, (32, 2, 2, 32))
    want = np.einsum("aebf,dfce->abcd", A.astype(np.float64), B.astype(np.float64))
    assert np.array_equal(D.astype(np.float64), want)          # small integers: every sum is exact
    # the CPU oracle walks the same mode tables
    ref = np.zeros((32, 2, 2, 32), np.float32, order="F")
    p = helpers.oracle_problem(conf, (0, 0, 0, 0))
    oracle.matmul(p, A, B, None, ref)
    assert np.array_equal(ref, D)


def test_distinct_extents_and_k_major_operands(gpu):
    """TCCG-style D[a,b,c] = sum_d A[b,d,a] * B[d,c] (the contraction of the reference benchmark
    script, benchmarks/tensor-contractions/run.jl:10-20): here A is contiguous along an M mode and B
    along the K mode."""
    ext = dict(a=3, b=64, c=128, d=64)
    conf, gmap = configs.gett_config("bda", "dc", "abc", ext, block_shape=(64, 64, 32))
    A = small_ints((64, 64, 3), 3)        # A[b,d,a]
    B = small_ints((64, 128), 4)          # B[d,c]
    D = run_gett(conf, A, B, (3, 64, 128))
    want = np.einsum("bda,dc->abc", A.astype(np.float64), B.astype(np.float64))
    assert np.array_equal(D.astype(np.float64), want)


def test_tccg_benchmark_at_the_reference_sizes_with_fp16_output(gpu):
    """The contraction the reference benchmarks (benchmarks/tensor-contractions/run.jl:10-21, 86-88):
    D_abc = A_bda * B_dc with a = 64, b = 32, c = d = 2048, Float16 A, B and D.  D is stored with `a`
    fastest while the GEMM's M index runs over (b, a), so the D stores are strided; accumulation is
    FP32 with one rounding at the store."""
    from gemmkernels import Layout, Float16, rng
    ext = dict(a=64, b=32, c=2048, d=2048)
    gmap = Layout.gett_map("bda", "dc", "abc", ext)
    conf, _ = configs.gett_config("bda", "dc", "abc", ext, global_d_layout=Layout.GETT[Float16, gmap],
                                  shared_d_layout=Layout.UnsafeAlignedColMajor[Float16])
    A = rng.matrix("upm1_f16", 5101, (32 * 2048, 64)).reshape((32, 2048, 64), order="F")      # A[b,d,a]
    B = rng.matrix("upm1_f16", 5102, (2048, 2048))                                              # B[d,c]
    a, b = gk.colmajor(A), gk.colmajor(B)
    d = gk.colmajor_empty((64, 32, 2048), torch.float16)
    d.fill_(float("nan"))
    print("case", gk.kernel_name(conf, Kernel.matmul_pipelined), flush=True)
    gk.matmul(conf, a, b, None, d, kernel=Kernel.matmul_pipelined)
    torch.cuda.synchronize()
    D = gk.to_numpy(d)
    assert D.dtype == np.float16 and np.isfinite(D).all()
    want = np.einsum("bda,dc->abc", A.astype(np.float32), B.astype(np.float32))
    assert oracle.rel_frobenius(D, want) <= 1e-3


def materialise(A, B, ext, gmap):
    """A_mat[m, k] and B_mat[n, k] with the kernel's own index orders (modes fastest first)."""
    a_modes, b_modes = "aebf", "dfce"
    def order(tensor_modes, dims):     # letters of the modes in `dims`, fastest first, identified by stride
        strides, s = {}, 1
        for ch in tensor_modes:
            strides[s] = ch
            s *= ext[ch]
        return strides
    sa, sb = order(a_modes, None), order(b_modes, None)
    m_letters = [sa[s0] for _, s0, _ in gmap.m]
    n_letters = [sb[s0] for _, s0, _ in gmap.n]
    k_letters = [sa[s0] for _, s0, _ in gmap.k]
    M, N, K = gmap.extent("m"), gmap.extent("n"), gmap.extent("k")
    # einsum to (m modes..., k modes...) then Fortran-reshape (first listed = fastest)
    A_mat = np.einsum(f"{a_modes}->{''.join(m_letters + k_letters)}", A).reshape((M, K), order="F")
    B_mat = np.einsum(f"{b_modes}->{''.join(n_letters + k_letters)}", B).reshape((N, K), order="F")
    return np.asfortranarray(A_mat), np.asfortranarray(B_mat), m_letters, n_letters


@pytest.mark.parametrize("extent,block", [(16, None), (64, None)])
def test_bit_exact_against_the_plain_kernel_on_materialised_matrices(gpu, extent, block):
    """Same kernel, same tile shape, same K order => the same MFMA sequence => identical bits."""
    if extent == 16:
        ext = dict(a=32, b=4, c=4, d=32, e=64, f=2)      # M = N = 128, K = 128
        block = (128, 128, 64)
    else:
        ext = dict(a=64, b=64, c=64, d=64, e=64, f=64)   # benchmark config 5
        block = (256, 256, 64)
    conf, gmap = configs.gett_config("aebf", "dfce", "abcd", ext, block_shape=block)
    shape_a = tuple(ext[ch] for ch in "aebf")
    shape_b = tuple(ext[ch] for ch in "dfce")
    A = rng.matrix("upm1_f16", 5001, shape_a)
    B = rng.matrix("upm1_f16", 5002, shape_b)
    D = run_gett(conf, A, B, tuple(ext[ch] for ch in "abcd"))
    A_mat, B_mat, m_letters, n_letters = materialise(A, B, ext, gmap)
    M, N, K = A_mat.shape[0], B_mat.shape[0], A_mat.shape[1]
    plain = configs.mfma_config(M, N, K, ta=False, tb=True, zero_c=True, block_shape=block)
    D_mat = helpers.run_gpu(plain, A_mat, B_mat, None, (M, N), kernel=Kernel.matmul_pipelined)
    # D_mat[m, n'] with m = (m_letters), n' = (n_letters), fastest first -> back to D[a,b,c,d]
    D_back = np.einsum(f"{''.join(m_letters + n_letters)}->abcd",
                       D_mat.reshape(tuple(ext[ch] for ch in m_letters + n_letters), order="F"))
    assert np.array_equal(D, D_back)
    # and the value itself, against BLAS on the materialised matrices
    ref = oracle.gemm_blas_f32(A_mat, B_mat, None, 1.0, 0.0, False, True)
    assert oracle.rel_frobenius(D_mat, ref) <= 1e-3


def test_gett_config_errors():
    from gemmkernels import ConfigError
    with pytest.raises(ConfigError):      # BLOCK_K = 32 neither divides the first K mode (24) nor is a multiple of it
        configs.gett_config("aebf", "dfce", "abcd", dict(a=32, b=2, c=2, d=32, e=24, f=4), block_shape=(64, 64, 32))
    with pytest.raises(ConfigError):      # the tile would cover e (16) whole and 2 of f, but f = 3 is not a multiple of 2
        configs.gett_config("aebf", "dfce", "abcd", dict(a=32, b=2, c=2, d=32, e=16, f=3), block_shape=(64, 64, 32))
    with pytest.raises(ConfigError):      # A has only 4 consecutive elements (a = 4, the next M mode b is not adjacent to it)
        configs.gett_config("aebf", "dfce", "abcd", dict(a=4, b=16, c=2, d=32, e=32, f=2), block_shape=(64, 64, 32))
    with pytest.raises(ConfigError):      # first N mode (d = 2) is not a multiple of 4
        configs.gett_config("aebf", "dfce", "abcd", dict(a=32, b=2, c=32, d=2, e=32, f=2), block_shape=(64, 64, 32))


# modes that the 32-wide fast path does not cover: (extents, block, what is special)
GENERAL = [
    (dict(a=32, b=2, c=2, d=32, e=16, f=4), (64, 64, 32), "a K tile = the whole first K mode (16) x 2 of the second"),
    (dict(a=32, b=4, c=4, d=32, e=16, f=4), (128, 128, 64), "a K tile = the whole first K mode x the whole second"),
    (dict(a=16, b=4, c=2, d=32, e=32, f=2), (64, 64, 32), "first M mode 16: rows of a 32-row block in two runs of D"),
    (dict(a=8, b=16, c=8, d=8, e=64, f=1), (128, 64, 32), "first M and N modes 8"),
    (dict(a=24, b=16, c=4, d=48, e=8, f=8), (128, 64, 64), "extents that are not powers of two; K tile = 8 x 8"),
]


@pytest.mark.parametrize("ext,block,what", GENERAL, ids=[g[2] for g in GENERAL])
def test_general_mode_extents_are_exact_against_einsum(gpu, ext, block, what):
    """Contractions whose modes do not come in multiples of 32 and whose K tile spans several K modes: every lane
    walks the mode tables for its own rows and columns of D, the K walker steps through the second K mode."""
    if block not in [(64, 64, 32), (128, 128, 64), (256, 256, 64)]:
        # only those tiles are compiled with contraction addressing: take the largest that divides
        M, N = ext["a"] * ext["b"], ext["c"] * ext["d"]
        block = (128, 128, 64) if (M % 128 == 0 and N % 128 == 0 and (ext["e"] * ext["f"]) % 64 == 0) else (64, 64, 32)
    conf, gmap = configs.gett_config("aebf", "dfce", "abcd", ext, block_shape=block)
    print("case", what, ext, block, gk.kernel_name(conf, Kernel.matmul_pipelined), flush=True)
    A = small_ints(tuple(ext[ch] for ch in "aebf"), 11)
    B = small_ints(tuple(ext[ch] for ch in "dfce"), 12)
    D = run_gett(conf, A, B, tuple(ext[ch] for ch in "abcd"))
    want = np.einsum("aebf,dfce->abcd", A.astype(np.float64), B.astype(np.float64))
    assert np.array_equal(D.astype(np.float64), want)
    # with C read through the same index map, and D hooks: D = 2 * (A*B + C)
    from gemmkernels import Transform, Float32
    conf_c, _ = configs.gett_config("aebf", "dfce", "abcd", ext, block_shape=block, zero_c=False)
    C = np.asfortranarray(np.random.RandomState(13).randint(-9, 10, size=D.shape).astype(np.float32))
    d = gk.colmajor_empty(D.shape, torch.float32)
    d.fill_(float("nan"))
    gk.matmul(conf_c, gk.colmajor(A), gk.colmajor(B), gk.colmajor(C), d, kernel=Kernel.matmul_pipelined,
              transform_shared_to_global_d=Transform.Elementwise(lambda x: x * 2.0))
    torch.cuda.synchronize()
    assert np.array_equal(gk.to_numpy(d).astype(np.float64), 2.0 * (want + C))


def _four_wave_case(d_modes, with_c):
    """D = sum_{e,f} A[a,e,b,f] * B[d,f,c,e] (+ C) on 256 x 256 x 64 tiles: M = a*b = 512, N = c*d = 256, K = e*f = 128."""
    ext = dict(a=64, b=8, c=4, d=64, e=64, f=2)
    kw = dict(block_shape=(256, 256, 64), zero_c=not with_c)
    conf, gmap = configs.gett_config("aebf", "dfce", d_modes, ext, **kw)
    eight, _ = configs.gett_config("aebf", "dfce", d_modes, ext, warps_per_block=8,
                                   compute_warp=gk.NT(M=128, N=64, K=16), **kw)
    A = rng.matrix("upm1_f16", 5101, tuple(ext[ch] for ch in "aebf"))
    B = rng.matrix("upm1_f16", 5102, tuple(ext[ch] for ch in "dfce"))
    d_shape = tuple(ext[ch] for ch in d_modes)
    C = rng.matrix("upm1_f32", 5103, d_shape) if with_c else None

    def run(cf):
        a, b = gk.colmajor(A), gk.colmajor(B)
        c = gk.colmajor(C) if with_c else None
        d = gk.colmajor_empty(d_shape, torch.float32)
        d.fill_(float("nan"))
        gk.matmul(cf, a, b, c, d, kernel=Kernel.matmul_pipelined)
        torch.cuda.synchronize()
        return gk.to_numpy(d)

    want = np.einsum(f"aebf,dfce->{d_modes}", A.astype(np.float64), B.astype(np.float64)) + (C.astype(np.float64) if with_c else 0.0)
    return conf, eight, run, want


@pytest.mark.parametrize("with_c", [False, True])
def test_four_waves_give_the_bits_of_eight_waves(gpu, with_c):
    """The first M mode is the contiguous one of C and D: four consecutive m of a lane are 16 bytes, and the
    contraction runs on the one-wave-per-SIMD arrangement of the 256 x 256 x 64 tile."""
    conf, eight, run, want = _four_wave_case("abcd", with_c)
    assert conf.warps_per_block == 4
    name = gk.kernel_name(conf, Kernel.matmul_pipelined)
    print("case", with_c, name, flush=True)
    assert "_w2x2_" in name and name.endswith("_gett")
    assert "_w2x4_" in gk.kernel_name(eight, Kernel.matmul_pipelined)
    d4, d8 = run(conf), run(eight)
    assert np.array_equal(d4, d8)
    assert oracle.rel_frobenius(d4, want) <= 1e-3


def test_four_wave_contraction_falls_back_where_c_and_d_are_not_contiguous_along_m(gpu):
    """D[c,a,b,d]: an N mode is the contiguous one, a lane's four rows are 4 * 4 bytes apart: eight waves."""
    conf, eight, run, want = _four_wave_case("cabd", True)
    assert "_w2x4_" in gk.kernel_name(conf, Kernel.matmul_pipelined)
    d = run(conf)
    assert np.array_equal(d, run(eight))
    assert oracle.rel_frobenius(d, want) <= 1e-3
