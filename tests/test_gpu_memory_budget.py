"""The memory budget given to compile() (model.hpp:2528) sizes the batch as
Allouable__Batch_Size does in the reference (update_size.cpp:26-116): the
batch buffers must fit the budget beside the model, a batch that does not fit
is reduced (and the epoch driver then walks more, smaller mini-batches), and a
budget that cannot hold the model with one example is refused.  Here the budget
counts device memory."""
import numpy as np
import pytest

from oracle.binding import ACT, NORM, OPT

pytestmark = pytest.mark.gpu

WIDTHS = [10, 16, 4]
PER_EXAMPLE = (2 * 10 + 2 * 4 + 3 * 16 + 3 * 4) * 4  # input row and target row (two upload slots each), Z / output / gradient of both layers


def build(lib, max_batch, budget=None):
    from deep_learning_amd.model import Model
    m = Model(lib, WIDTHS)
    m.set_layer(1, ACT["ELU"], NORM["BRN"])
    m.set_layer(2, ACT["SOFTMAX"])
    if budget is not None:
        m.set_allowable_memory(budget(m))
    m.prepare(max_batch)
    return m


def test_budget_defaults_to_the_device_and_sizes_are_reported(pkg):
    m = build(pkg.load_library(), 64)
    try:
        mem = m.memory()
        assert mem["budget"] > 100 * 2**30 and mem["batch_size"] == 64
        assert mem["bytes_per_example"] == PER_EXAMPLE
        P = m.P
        assert mem["model_bytes"] >= 2 * P * 4  # parameters and their gradients at least
    finally:
        m.close()


def test_a_tight_budget_reduces_the_batch_and_the_driver_follows(pkg):
    lib = pkg.load_library()
    a = build(lib, 64, budget=lambda m: m.memory()["model_bytes"] + 10 * PER_EXAMPLE + 5)
    b = build(lib, 10)  # the same mini-batches by way of the maximum batch size
    try:
        assert a.memory()["batch_size"] == 10 and b.memory()["batch_size"] == 10
        rng = np.random.default_rng(4)
        X = rng.uniform(-1, 1, (47, 10)).astype(np.float32)
        Y = np.eye(4, dtype=np.float32)[rng.integers(0, 4, 47)]
        for m in (a, b):
            m.glorot_uniform(3)
            m.set_optimizer(OPT["GD"], lr=0.05, momentum=0.0)  # no optimizer array: the model's size stays as budgeted
        for _ in range(3):
            ra, rb = a.train_epoch(X, Y), b.train_epoch(X, Y)
            assert ra == rb
            assert np.array_equal(a.get_parameters(), b.get_parameters())
        with pytest.raises(RuntimeError):  # one call with more rows than the budget allows
            a.step(1, X[:11], Y[:11], backward=True)
    finally:
        a.close()
        b.close()


@pytest.mark.parametrize("slack", [-1, PER_EXAMPLE - 1])
def test_a_budget_below_the_model_with_one_example_is_refused(pkg, slack):
    with pytest.raises(RuntimeError):
        build(pkg.load_library(), 8, budget=lambda m: m.memory()["model_bytes"] + slack)
