"""The uniform weight initializers (initialize_weights_with_glorot_uniform,
glorot.cpp:225-359; Initialization__Uniform, uniform.cpp:26-90) against
tests/golden/init.npz, which the compiled reference wrote with its generator
seeded: the numpy restatement in oracle/init_oracle.py must give the same
parameter vector bit for bit, and the textbook facts the bounds reduce to must
hold on the reference's own numbers."""
import json
import os

import numpy as np
import pytest

from conftest import ROOT
from oracle import init_oracle
from oracle.binding import ACT

INFO_KEYS = ("type", "n_out", "w0", "w1", "bias", "use_bias", "n_unit", "gamma", "unit", "n_af", "depth", "padding")


def load_init_golden():
    g = np.load(os.path.join(ROOT, "tests", "golden", "init.npz"), allow_pickle=False)
    return {k: g[k] for k in g.files}


def init_cases():
    raw = json.loads(bytes(load_init_golden()["init_cases_json"]))
    return {k: ([tuple(e) for e in v[0]], {int(a): b for a, b in v[1].items()}, {int(a): b for a, b in v[2].items()},
                v[3], v[4], v[5]) for k, v in raw.items()}


def golden_info(g, name):
    table = g[name + "_info"]
    return lambda l: dict(zip(INFO_KEYS, (int(v) for v in table[l])))


@pytest.mark.parametrize("name", list(init_cases()))
def test_numpy_restatement_is_bit_identical(name):
    g = load_init_golden()
    layers, acts, norms, seed, bias, bounds = init_cases()[name]
    P, n_units = (int(v) for v in g[name + "_P"])
    lo, hi = bounds if bounds else (None, None)
    p = init_oracle.initialize(layers, {l: ACT[a] for l, a in acts.items()}, seed, bias, golden_info(g, name), P, n_units,
                               lower=lo, upper=hi)
    assert np.array_equal(p, g[name + "_params"])
    # Clear__Parameter__Normalized_Unit: moving mean 0, moving std 1, whatever they held
    assert np.array_equal(g[name + "_mov_mean"], np.zeros(n_units, np.float32))
    assert np.array_equal(g[name + "_mov_std"], np.ones(n_units, np.float32))


def test_bounds_reduce_to_the_textbook_forms():
    """He-uniform for a ReLU layer (sqrt(2) * sqrt(6 / fan_in) = sqrt(12 / fan_in)), Glorot-uniform
    sqrt(6 / (fan_in + fan_out)) for an ELU layer, fan_out = fan_in on the output layer: read off the
    reference's weights (every weight inside the bound, the largest within 2 % of it)."""
    g = load_init_golden()
    info = golden_info(g, "glorot_plain")
    p = g["glorot_plain_params"]
    expect = {1: np.sqrt(12 / 8), 2: np.sqrt(6 / (20 + 12)), 3: np.sqrt(2 / (1 + 0.01 ** 2)) * np.sqrt(6 / 30),
              4: np.sqrt(6 / (12 + 12))}
    for l, b in expect.items():
        w = p[info(l)["w0"]:info(l)["w1"]]
        assert np.abs(w).max() <= b * (1 + 1e-6), l
        assert np.abs(w).max() >= b * 0.98 or w.size < 100, l
        assert abs(w.mean()) < 4 * b / np.sqrt(3 * w.size), l  # mean of a centred uniform sample


def test_uniform_stream_is_the_mersenne_twister():
    """First output of std::mt19937 with the default seed 5489 is 3499211612 (the
    value the C++ standard fixes through its 10000th-output check belongs to the same
    sequence); the distribution maps it to word / 2^32."""
    u = init_oracle.uniform_stream(5489, 3)
    assert u[0] == np.float32(3499211612) / np.float32(2 ** 32)
    assert np.random.RandomState(5489).randint(0, 2 ** 32, size=10000, dtype=np.uint64)[-1] == 4123659995
