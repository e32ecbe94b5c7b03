"""The host side of the one stream of random weights (sonicboom_amd/weights/random_stream.py):
what pins it (values written down once, so that a change of the function is seen), what it must
be (standard normals), and that an element depends on (seed, tensor, element) alone."""
import numpy as np
from scipy import stats

from sonicboom_amd.sampling.philox import philox4x32_10
from sonicboom_amd.weights import random_stream as rs


def test_known_values():
    z = rs.standard_normals(7, 2, 8)
    want = ["0x1.a3b901af341d3p-3", "-0x1.1d3feab0e12a5p-2", "0x1.9b5ba08882678p-3", "0x1.58ba7745be642p+0",
            "0x1.0d948063bf72ep-4", "0x1.809637fe58eabp-2", "-0x1.1c689f090c8f4p-2", "-0x1.1ed4ddfe91636p-2"]
    assert [float(x).hex() for x in z] == want
    bits = rs.draw(7, 2, (2, 3), 1.0, 0.02).view(np.uint32)
    assert bits.tolist() == [[1065387600, 1065259745, 1065386914], [1065579137, 1065364258, 1065416227]]


def test_the_formula_from_its_parts():
    """Element 4c + 1 is sqrt(-2 ln u) sin(2 pi v) of words 0 and 1 of counter (c, 0, tensor, 0)."""
    seed, tensor, c = 99, 5, 123456
    w = philox4x32_10(np.array([c]), np.array([0]), np.array([tensor]), np.array([0]), seed)
    u, v = (float(w[0][0]) + 0.5) / 2 ** 32, (float(w[1][0]) + 0.5) / 2 ** 32
    u2, v2 = (float(w[2][0]) + 0.5) / 2 ** 32, (float(w[3][0]) + 0.5) / 2 ** 32
    z = rs.standard_normals(seed, tensor, 4, first=4 * c)
    want = [np.sqrt(-2 * np.log(u)) * np.cos(2 * np.pi * v), np.sqrt(-2 * np.log(u)) * np.sin(2 * np.pi * v),
            np.sqrt(-2 * np.log(u2)) * np.cos(2 * np.pi * v2), np.sqrt(-2 * np.log(u2)) * np.sin(2 * np.pi * v2)]
    assert np.allclose(z, want, rtol=0, atol=1e-13)


def test_logarithm_and_angles_against_the_library():
    w = np.random.default_rng(0).integers(0, 2 ** 32, 200000, dtype=np.uint64).astype(np.uint32)
    w[:4] = [0, 1, 2 ** 32 - 1, 2 ** 31]
    u = (w.astype(np.float64) + 0.5) / 2 ** 32
    assert np.max(np.abs(rs._neg2_log_u(w) / (-2 * np.log(u)) - 1)) < 2e-15
    c, s = rs._cos_sin(w)
    assert np.abs(c - np.cos(2 * np.pi * u)).max() < 2e-15 and np.abs(s - np.sin(2 * np.pi * u)).max() < 2e-15


def test_standard_normal():
    z = rs.standard_normals(11, 0, 400000)
    assert abs(z.mean()) < 0.006 and abs(z.std() - 1) < 0.005
    assert abs((z ** 3).mean()) < 0.02 and abs((z ** 4).mean() - 3) < 0.05
    assert stats.kstest(z[:100000], "norm").pvalue > 1e-3
    # neighbours (the cosine and sine of one pair, and the two pairs of a counter) do not correlate
    for lag in (1, 2, 3, 4):
        assert abs(np.corrcoef(z[:-lag], z[lag:])[0, 1]) < 0.006


def test_an_element_depends_on_seed_tensor_and_element_alone():
    whole = rs.standard_normals(3, 9, 70001)
    for first, count in ((0, 5), (1, 7), (2, 2), (65533, 11), (4 * rs.CHUNK - 3, 9)):
        whole_long = rs.standard_normals(3, 9, first + count)
        assert np.array_equal(rs.standard_normals(3, 9, count, first=first), whole_long[first:])
    assert np.array_equal(rs.draw(3, 9, (7, 10000), 0.5, 2.0),
                          (whole[:70000] * 2.0 + 0.5).astype(np.float32).reshape(7, 10000))
    assert not np.array_equal(rs.standard_normals(4, 9, 64), whole[:64])
    assert not np.array_equal(rs.standard_normals(3, 8, 64), whole[:64])
    # seeds are 64-bit keys: the high word counts
    assert not np.array_equal(rs.standard_normals(3 + 2 ** 32, 9, 64), whole[:64])
