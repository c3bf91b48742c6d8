"""The contraction planner (TCCG-style strings -> one launch of the GEMM kernel): host logic on the
CPU, results against numpy.einsum on the GPU."""
import numpy as np
import pytest

import gemmkernels as gk
from gemmkernels import contraction

# (specification, extents): contractions of the TCCG benchmark suite's shapes, sized for a test
TCCG = [
    ("abc-bda-dc", dict(a=4, b=64, c=128, d=64)),                          # the reference's benchmark script (run.jl:10-21)
    ("abcd-dbea-ec", dict(a=4, b=2, c=64, d=32, e=64)),
    ("abcde-efbad-cf", dict(a=2, b=2, c=64, d=2, e=32, f=64)),
    ("abcd-aebf-dfce", dict(a=32, b=2, c=2, d=32, e=32, f=2)),             # benchmark config 5, reduced
    ("ab-ac-cb", dict(a=128, b=64, c=96)),                                 # a plain GEMM, A 'N', B 'N'
    ("ab-ca-cb", dict(a=64, b=128, c=64)),                                 # A transposed
    ("abcdef-dega-gfbc", dict(a=2, b=2, c=2, d=32, e=2, f=32, g=64)),
    ("abcd-dbea-ec", dict(a=64, b=4, c=64, d=2, e=64)),                    # A's leading M modes d (2) and b (4) make one run of 8
    ("abcd-dbea-ec", dict(a=64, b=3, c=64, d=2, e=64)),                    # refused: see REFUSED
]


# contractions whose operand has no run of 8 consecutive elements (here d x b = 2 x 3) for 16-byte vectors: refused, not mis-run
REFUSED = {("abcd-dbea-ec", 3)}


def test_parse_classify_and_refusals():
    assert contraction.parse("abc-bda-dc") == ("abc", "bda", "dc")
    assert contraction.classify("abc", "bda", "dc") == (["b", "a"], ["c"], ["d"])
    with pytest.raises(ValueError):
        contraction.parse("abc-bda")
    with pytest.raises(ValueError):
        contraction.parse("aab-ac-cb")
    with pytest.raises(ValueError):                       # a batch mode: in all three tensors
        contraction.classify("abn", "acn", "cbn")
    with pytest.raises(ValueError):                       # a mode summed inside A alone
        contraction.classify("ab", "acx", "cb")
    with pytest.raises(ValueError):                       # no K mode: an outer product
        contraction.classify("ab", "a", "b")


def test_fusion_of_neighbouring_modes():
    # a and b follow each other in A and in D: one mode of extent 6; e, f do so in A and B
    d, a, b, ext, groups = contraction.fuse("abc", "abef", "efc", dict(a=2, b=3, c=5, e=7, f=11))
    assert (d, a, b) == ("ac", "ae", "ec")
    assert ext == dict(a=6, c=5, e=77) and groups["a"] == "ab" and groups["e"] == "ef"
    # not neighbours in B: nothing to fuse
    d, a, b, ext, groups = contraction.fuse("abc", "abef", "fec", dict(a=2, b=3, c=5, e=7, f=11))
    assert (d, a, b) == ("ac", "aef", "fec")
    # the benchmark contraction: nothing is adjacent in both tensors
    assert contraction.fuse("abc", "bda", "dc", dict(a=4, b=64, c=128, d=64))[:3] == ("abc", "bda", "dc")


@pytest.mark.parametrize("spec,ext", TCCG, ids=[f"{t[0]}/{t[1]['a']}/{t[1]['b']}" for t in TCCG])
def test_every_benchmark_shape_maps_onto_a_compiled_kernel(spec, ext):
    found = [(swapped, info) for swapped, _, conf, info in contraction.candidates(spec, ext) if conf is not None]
    if (spec, ext["b"]) in REFUSED:
        assert not found
        return
    assert found, list(contraction.candidates(spec, ext))
    assert found[0][1].endswith("_gett")


def test_operands_are_swapped_when_only_that_assignment_fits():
    # the first input has a short leading M mode (8, not a multiple of 32) but the second input's N
    # mode is long: with the inputs swapped the short mode becomes the N side ... which has the same
    # rule, so this is refused either way, with both reasons reported
    reasons = [info for _, _, conf, info in contraction.candidates("ab-ac-cb", dict(a=8, b=64, c=64)) if conf is None]
    assert len(reasons) >= 2 and all("32" in r or "tile" in r for r in reasons)
    # K mode contiguous in neither input, M contiguous in A: fine as it stands
    ok = [s for s, _, conf, _ in contraction.candidates("ab-ac-cb", dict(a=64, b=64, c=64)) if conf is not None]
    assert ok and ok[0] is False


@pytest.mark.gpu
@pytest.mark.parametrize("spec,ext", TCCG, ids=[f"{t[0]}/{t[1]['a']}/{t[1]['b']}" for t in TCCG])
def test_contractions_against_einsum(gpu, spec, ext):
    import torch
    if (spec, ext["b"]) in REFUSED:
        pytest.skip("refused by the planner (covered on the CPU)")
    dm, am, bm = contraction.parse(spec)
    rs = np.random.RandomState(len(spec))
    A = np.asfortranarray(rs.randint(-4, 5, size=[ext[ch] for ch in am]).astype(np.float16))
    B = np.asfortranarray(rs.randint(-4, 5, size=[ext[ch] for ch in bm]).astype(np.float16))
    C = np.asfortranarray(rs.randint(-9, 10, size=[ext[ch] for ch in dm]).astype(np.float32))
    a, b, c = gk.colmajor(A), gk.colmajor(B), gk.colmajor(C)
    d = gk.colmajor_empty(tuple(ext[ch] for ch in dm), torch.float32)
    d.fill_(float("nan"))
    p = contraction.plan(spec, a, b, d)
    p()
    torch.cuda.synchronize()
    want = np.einsum(f"{am},{bm}->{dm}", A.astype(np.float64), B.astype(np.float64))
    assert np.array_equal(gk.to_numpy(d).astype(np.float64), want)          # small integers: exact
    # with C, in place: D = A*B + C
    gk.contract(spec, a, b, c, c)
    torch.cuda.synchronize()
    assert np.array_equal(gk.to_numpy(c).astype(np.float64), want + C.astype(np.float64))


@pytest.mark.gpu
def test_refused_contraction_names_the_reasons(gpu):
    import torch
    a = gk.colmajor(np.zeros((8, 64), np.float16, order="F"))
    b = gk.colmajor(np.zeros((64, 64), np.float16, order="F"))
    d = gk.colmajor_empty((8, 64), torch.float32)
    with pytest.raises(gk.ConfigError) as ei:
        contraction.plan("ab-ac-cb", a, b, d)
    assert "does not map onto the GEMM kernel" in ei.value.message
    with pytest.raises(gk.ConfigError):                   # extent of c differs between A and B
        contraction.plan("ab-ac-cb", a, gk.colmajor(np.zeros((32, 64), np.float16, order="F")), d)


def test_division_by_multiplication_is_exact():
    """The kernels divide mode indices by the extents through a multiplication by a 32-bit reciprocal (s = ceil(log2 e),
    magic = floor(2^(31+s) / e) + 1, quotient = (n * magic) >> (31 + s)): exact for every n < 2^31.  Checked here on the
    arithmetic itself, at the places where a too small or too large reciprocal would first fail."""
    rs = np.random.RandomState(5)
    extents = list(range(2, 130)) + [255, 256, 257, 1000, 4095, 4096, 4097, 65535, 65536, 65537, 2**20 + 7, 2**30 - 1, 2**30 + 1, 2**31 - 1]
    for e in extents:
        s = (e - 1).bit_length()
        magic = (1 << (31 + s)) // e + 1
        assert magic < 2**32
        span = min(4 * e + 2, 3000)                 # around 0, around the multiples of e, around 2^31
        mult = np.arange(1, 500, dtype=np.int64) * e
        ns = np.concatenate([np.arange(0, span, dtype=np.int64), (2**31 - 1) - np.arange(0, span, dtype=np.int64), mult - 1, mult,
                             ((2**31 - 1) // e - np.arange(0, 50, dtype=np.int64)) * e - 1, ((2**31 - 1) // e - np.arange(0, 50, dtype=np.int64)) * e,
                             rs.randint(0, 2**31 - 1, size=2000).astype(np.int64)])
        ns = ns[(ns >= 0) & (ns < 2**31)]
        q = [(int(n) * magic) >> (31 + s) for n in ns]
        assert q == [int(n) // e for n in ns], e
