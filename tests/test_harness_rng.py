"""The benchmark harness's input generator (oracle/harness_rng.c, mt19937_64) against the known answer
the C++ standard fixes for std::mt19937_64, and the mappings to uniform / normal / Bernoulli values."""
import numpy as np

from oracle.binding import HarnessRng


def test_mt19937_64_known_answer():
    # [rand.predef]: the 10000th consecutive invocation of a default-constructed mt19937_64 (seed 5489)
    raw = HarnessRng(base_seed=5489).raw(0, 10000)
    assert int(raw[-1]) == 9981545732273789042
    # the first outputs of the reference implementation (mt19937-64.c, init_genrand64(5489))
    assert int(raw[0]) == 14514284786278117030 and int(raw[1]) == 4620546740167642908


def test_streams_and_mappings():
    g = HarnessRng(1234)
    raw = g.raw(3, 1000)
    u = g.uniform(3, (1000,), -2.0, 6.0)
    expect = np.float32(-2.0) + np.float32(8.0) * ((raw >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -24))
    assert np.array_equal(u, expect.astype(np.float32))
    assert not np.array_equal(g.raw(4, 16), raw[:16])  # another tensor id, another stream
    assert np.array_equal(HarnessRng(1230).raw(7, 16), raw[:16])  # seed = base + tensor id
    b = g.bernoulli_u8(3, (1000,), 0.9)
    assert np.array_equal(b, ((raw >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -24) < np.float32(0.9)))
    z = g.normal(5, (200001,))
    assert abs(float(z.mean())) < 0.01 and abs(float(z.std()) - 1.0) < 0.01 and np.all(np.isfinite(z))
    r = g.raw(5, 4)
    u1 = ((r[0] >> np.uint64(40)).astype(np.float64) + 1.0) / 2.0 ** 24
    u2 = (r[1] >> np.uint64(40)).astype(np.float64) / 2.0 ** 24
    assert z[0] == np.float32(np.sqrt(-2 * np.log(u1)) * np.cos(2 * np.pi * u2))
    assert z[1] == np.float32(np.sqrt(-2 * np.log(u1)) * np.sin(2 * np.pi * u2))
    assert np.array_equal(g.index(9, 64, 10), (g.raw(9, 64) % np.uint64(10)).astype(np.uint32))
