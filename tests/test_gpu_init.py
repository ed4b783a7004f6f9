"""The facade's weight initializers against tests/golden/init.npz (compiled
reference, generator seeded): the parameter vector in HBM after the call must be
the reference's bit for bit, scales / shifts / moving statistics reset, gradient
array and optimizer clocks cleared."""
import numpy as np
import pytest

from oracle.binding import ACT, NORM
from test_oracle_init import init_cases, load_init_golden

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def net_factory(pkg):
    from deep_learning_amd.model import Net
    lib = pkg.load_library()
    made = []

    def make(layers):
        m = Net(lib, layers)
        made.append(m)
        return m

    yield make
    for m in made:
        m.close()


@pytest.mark.parametrize("name", list(init_cases()))
def test_gpu_initializers_against_golden(net_factory, name):
    g = load_init_golden()
    layers, acts, norms, seed, bias, bounds = init_cases()[name]
    M = net_factory(layers)
    for l in sorted(set(acts) | set(norms)):
        M.set_layer(l, ACT[acts[l]] if l in acts else 0, NORM[norms.get(l, "NONE")])
    M.prepare(4)
    assert [M.P, M.n_units] == [int(v) for v in g[name + "_P"]]
    rng = np.random.default_rng(seed)
    M.set_parameters(rng.uniform(-2, 2, M.P).astype(np.float32))
    M.set_moving(rng.uniform(-2, 2, M.n_units).astype(np.float32), rng.uniform(1, 3, M.n_units).astype(np.float32))
    M.set_dparams(np.ones(M.P, np.float32))
    if bounds is None:
        M.glorot_uniform(seed, bias)
    else:
        M.init_uniform(seed, bias, *bounds)
    assert np.array_equal(M.get_parameters(), g[name + "_params"])
    mm, ms = M.get_moving()
    assert np.array_equal(mm, g[name + "_mov_mean"]) and np.array_equal(ms, g[name + "_mov_std"])
    assert not M.get_dparams().any()  # clear_training_arrays


def test_same_seed_same_weights_other_seed_other_weights(net_factory):
    layers = [("FC", 16), ("FC", 32), ("FC", 4)]
    def weights(seed):
        M = net_factory(layers)
        M.set_layer(1, ACT["RELU"])
        M.set_layer(2, ACT["SOFTMAX"])
        M.prepare(2)
        M.glorot_uniform(seed)
        return M.get_parameters()
    a, b, c = weights(42), weights(42), weights(43)
    assert np.array_equal(a, b) and not np.array_equal(a, c)


@pytest.mark.parametrize("name", [n for n, c in init_cases().items() if c[5] is None])
def test_gaussian_glorot_against_the_compiled_reference(net_factory, reference, name):
    """Initialization__Glorot__Gaussian (glorot.cpp:110-222) on the networks of the uniform cases, residual blocks
    included: the parameter vector after the call is the compiled reference's bit for bit (same walk over the
    layers, the reference's own Gaussian stream), the tail of the initialization as for the other initializers."""
    from oracle.binding import ReferenceNet
    layers, acts, norms, seed, bias, _ = init_cases()[name]
    M, R = net_factory(layers), ReferenceNet(reference, layers)
    for m in (M, R):
        for l in sorted(set(acts) | set(norms)):
            m.set_layer(l, ACT[acts[l]] if l in acts else 0, NORM[norms.get(l, "NONE")])
        m.prepare(4)
    assert [M.P, M.n_units] == [R.P, R.n_units]
    rng = np.random.default_rng(seed)
    p0 = rng.uniform(-2, 2, M.P).astype(np.float32)
    mv = rng.uniform(-2, 2, M.n_units).astype(np.float32), rng.uniform(1, 3, M.n_units).astype(np.float32)
    for m in (M, R):
        m.set_parameters(p0)
        m.set_moving(*mv)
        m.glorot_gaussian(seed, bias)
    assert np.array_equal(M.get_parameters(), R.get_parameters())
    (mm, ms), (rm, rs) = M.get_moving(), R.get_moving()
    assert np.array_equal(mm, rm) and np.array_equal(ms, rs)
    assert not np.array_equal(M.get_parameters(), p0)
    # Initialization__Identity (identity.cpp:25-103) on the same pair: zeros and the reference's ones
    for m in (M, R):
        m.set_parameters(p0)
        m.init_identity(bias)
    pi = M.get_parameters()
    assert np.array_equal(pi, R.get_parameters())
    assert set(np.unique(pi).tolist()) <= {0.0, 1.0, float(np.float32(bias))}
