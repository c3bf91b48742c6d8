"""The seeded input generator: fixed first values (so that any re-implementation can check itself),
ranges and exact representability."""
import numpy as np

from gemmkernels import rng


def test_splitmix_known_values():
    # splitmix64 finaliser of seed ^ (golden * (i + 1)), computed independently with Python integers
    def ref(seed, i):
        mask = (1 << 64) - 1
        z = seed ^ ((0x9E3779B97F4A7C15 * (i + 1)) & mask)
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
        return z ^ (z >> 31)
    got = rng.splitmix64(2001, 5)
    assert [int(x) for x in got] == [ref(2001, i) for i in range(5)]


def test_ranges_and_representability():
    u = rng.uniform01_f32(1, 100000)
    assert u.dtype == np.float32 and u.min() >= 0.0 and u.max() < 1.0 and abs(u.mean() - 0.5) < 0.01
    h = rng.uniform_pm1_f16(2, 100000)
    assert h.dtype == np.float16 and h.min() >= -1.0 and h.max() < 1.0
    assert np.array_equal(h.astype(np.float32) * 1024, np.round(h.astype(np.float32) * 1024))   # multiples of 2^-10
    s = rng.uniform_pm1_f32(3, 100000)
    assert s.min() >= -1.0 and s.max() < 1.0 and abs(s.mean()) < 0.01
    n = rng.normal_f32(4, 200000)
    assert abs(n.mean()) < 0.01 and abs(n.std() - 1.0) < 0.01 and np.isfinite(n).all()


def test_matrix_is_column_major_stream():
    m = rng.matrix("upm1_f16", 7, (4, 3))
    assert m.flags.f_contiguous and m.shape == (4, 3)
    assert np.array_equal(m.ravel(order="F"), rng.uniform_pm1_f16(7, 12))
