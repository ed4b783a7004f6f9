"""Rows handed over as host pointers (forward_pass / compute_error of the facade): two upload slots used in
turn, gathered by several host threads above a few MB, copied on a stream of their own while the kernels of the
previous step still run.  Back-to-back steps must give what steps with a host wait after each give, bit for
bit, and what float64 arithmetic gives for the first layer."""
import numpy as np
import pytest

from oracle.binding import ACT, NORM, STATE

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def model_factory(pkg):
    from deep_learning_amd.model import Model
    lib = pkg.load_library()
    made = []

    def make(widths):
        m = Model(lib, widths)
        made.append(m)
        return m

    yield make
    for m in made:
        m.close()


def build(factory, widths, batch, seed):
    M = factory(widths)
    for l in range(1, len(widths) - 1):
        M.set_layer(l, ACT["RELU"], NORM["BRN"])
    M.set_layer(len(widths) - 1, ACT["SOFTMAX"])
    M.set_norm_hyper(0.99, 1e-5, 3.0, 5.0)
    M.prepare(batch)
    M.glorot_uniform(seed)
    return M


# a long upload behind short kernels (16 MiB of rows per step: four pieces, several gather threads) and a
# short upload behind long kernels (the slot of step i is wanted again while step i still runs)
@pytest.mark.parametrize("widths, batch", [([1024, 256, 8], 4096), ([256, 2048, 2048, 8], 4096), ([20, 16, 4], 7)])
def test_back_to_back_steps_equal_steps_with_a_wait_after_each(model_factory, widths, batch):
    n_steps = 5
    rng = np.random.default_rng(5)
    X = rng.standard_normal((n_steps * batch, widths[0]), dtype=np.float32)
    Y = np.zeros((n_steps * batch, widths[-1]), np.float32)
    Y[np.arange(len(Y)), rng.integers(0, widths[-1], len(Y))] = 1.0
    A, Bm = build(model_factory, widths, batch, 3), build(model_factory, widths, batch, 3)
    assert np.array_equal(A.get_parameters(), Bm.get_parameters())
    A.steps(STATE["TRAINING"], X, Y, batch)
    for s in range(n_steps):
        Bm.step(STATE["TRAINING"], X[s * batch:(s + 1) * batch], Y[s * batch:(s + 1) * batch])
    assert np.array_equal(A.get_dparams(), Bm.get_dparams())  # accumulated over the five steps
    assert np.array_equal(A.get_out(), Bm.get_out())
    for a, b in zip(A.get_moving(), Bm.get_moving()):
        assert np.array_equal(a, b)
    # the last step's first product against float64: the rows that were uploaded are the rows of that step
    p = A.get_parameters()
    o = A.layer_offsets(1)
    W = p[o[0]:o[0] + widths[1] * widths[0]].reshape(widths[1], widths[0]).astype(np.float64)
    Z = X[-batch:].astype(np.float64) @ W.T
    got = A.layer_buffer(1, 0)
    assert np.abs(got - Z).max() <= 1e-4 * max(1.0, np.abs(Z).max())


def test_caller_may_reuse_its_rows_once_the_call_returns(model_factory):
    widths, batch = [512, 64, 4], 4096  # 8 MiB of rows: the threaded gather
    rng = np.random.default_rng(9)
    X = rng.standard_normal((batch, widths[0]), dtype=np.float32)
    M = build(model_factory, widths, batch, 1)
    M.step(STATE["INFERENCE"], X, None, backward=False)
    want = M.get_out()
    X2 = X.copy()
    M.step(STATE["INFERENCE"], X2, None, backward=False)
    X2[:] = 0.0
    assert np.array_equal(M.get_out(), want)
