"""The epoch driver's recorded mini-batches: from the second epoch of a
configuration on, each mini-batch's launches are held as a HIP graph and
replayed.  Every replay is checked against a twin model that launches kernel by
kernel, with unrecorded work (an evaluation pass, parameter downloads, new
dropout masks) and synchronizations between the replays; a change of a setting
must drop the graphs and record them again."""
import numpy as np
import pytest

from oracle.binding import ACT, DROP, NORM, OPT

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib(pkg):
    return pkg.load_library()


def build(lib, widths, out_act="SOFTMAX", max_batch=16):
    from deep_learning_amd.model import Model
    m = Model(lib, widths)
    L = len(widths)
    for l in range(1, L - 1):
        m.set_layer(l, ACT["RELU" if l % 2 else "ELU"], NORM["BRN"], DROP["BERNOULLI"] if l == 1 else 0, 0.8)
    m.set_layer(L - 1, ACT[out_act])
    m.set_norm_hyper(0.9, 1e-5, 3.0, 5.0)
    m.prepare(max_batch)
    m.glorot_uniform(77)
    m.set_optimizer(OPT["ADAM"], adam_lr=0.01)
    return m


def data(n, k, h, onehot=True, seed=3):
    rng = np.random.default_rng(seed)
    X = rng.uniform(-1, 1, (n, k)).astype(np.float32)
    Y = (np.eye(h)[rng.integers(0, h, n)] if onehot else rng.uniform(-1, 1, (n, h))).astype(np.float32)
    return X, Y


def run_pair(a, b, X, Y, epochs, expect_recorded):
    """expect_recorded[e]: mini-batches of the TRAINING pass held as graphs after epoch e; the evaluation pass
    that follows each epoch is recorded on the same schedule (plain, recorded, replayed ...)."""
    for e in range(epochs):
        ra = a.train_epoch(X, Y, resample_masks=True, record_batches=False)
        rb = b.train_epoch(X, Y, resample_masks=True, record_batches=True)
        assert rb[0] == pytest.approx(ra[0], rel=1e-9) and rb[1] == ra[1], f"epoch {e}: reports {ra} / {rb}"
        assert np.array_equal(a.get_parameters(), b.get_parameters()), f"epoch {e}: parameters differ"
        ma, mb = a.get_moving(), b.get_moving()
        assert np.array_equal(ma[0], mb[0]) and np.array_equal(ma[1], mb[1]), f"epoch {e}: moving statistics differ"
        assert a.recorded_batches(X, Y) == 0
        ea, eb = a.evalt(X, Y), b.evalt(X, Y)
        assert eb[0] == pytest.approx(ea[0], rel=1e-9) and eb[1] == ea[1], f"epoch {e}: evaluation {ea} / {eb}"
        assert b.recorded_batches(X, Y) == 2 * expect_recorded[e], f"epoch {e}, after its evaluation pass"
        assert a.recorded_batches(X, Y) == 0


def test_replays_match_plain_launches_epoch_by_epoch(lib):
    widths = [20, 32, 24, 5]
    X, Y = data(50, 20, 5)  # four mini-batches of 16, the last one ragged (2 rows)
    a, b = build(lib, widths), build(lib, widths)
    try:
        run_pair(a, b, X, Y, 6, [0, 4, 4, 4, 4, 4])
        # a changed hyper-parameter is baked into the recorded launches: they must be dropped
        for m in (a, b):
            m.set_norm_hyper(0.5, 1e-5, 2.0, 1.0)
        run_pair(a, b, X, Y, 4, [0, 4, 4, 4])
        # another data set gets a driver of its own
        X2, Y2 = data(33, 20, 5, seed=9)
        run_pair(a, b, X2, Y2, 3, [0, 3, 3])
    finally:
        a.close()
        b.close()


@pytest.mark.parametrize("per_graph", [1, 3, 4])
def test_several_minibatches_per_graph(lib, per_graph, monkeypatch):
    """The driver puts up to batches_per_graph consecutive mini-batches into one graph (read from the
    environment when the driver is made): one each, a count that leaves a shorter last graph (4 = 3 + 1), and
    all of them in one graph give the plain launches' results bit for bit."""
    monkeypatch.setenv("DLMI_BATCHES_PER_GRAPH", str(per_graph))
    widths = [20, 32, 24, 5]
    X, Y = data(50, 20, 5)
    a, b = build(lib, widths), build(lib, widths)
    try:
        run_pair(a, b, X, Y, 5, [0, 4, 4, 4, 4])
    finally:
        a.close()
        b.close()


def test_regression_output_layer_is_recorded_too(lib):
    from oracle.binding import ACCU, LOSS
    widths = [12, 18, 4]
    X, Y = data(40, 12, 4, onehot=False)
    a, b = build(lib, widths, "LINEAR"), build(lib, widths, "LINEAR")
    try:
        for m in (a, b):
            m.set_loss(LOSS["MSE"], ACCU["DISTANCE"], 0.3)
        run_pair(a, b, X, Y, 5, [0, 3, 3, 3, 3])
    finally:
        a.close()
        b.close()


def test_residual_blocks_are_recorded_too(lib):
    from deep_learning_amd.model import Net

    def make():
        net = Net(lib, [("FC", 10), ("RES", 2), ("FC", 14), ("FC", 10), ("RES", 2), ("FC", 10), ("FC", 6), ("FC", 4)])
        for l in (2, 3, 5, 6):
            net.set_layer(l, ACT["ELU"], NORM["BRN"])
        net.set_layer(1, 0, NORM["BRN"])
        net.set_layer(7, ACT["SOFTMAX"])
        net.set_norm_hyper(0.9, 1e-5, 3.0, 5.0)
        net.prepare(8)
        net.glorot_uniform(5)
        net.set_optimizer(OPT["GD"], lr=0.01, momentum=0.9, nesterov=True)
        return net

    a, b = make(), make()
    try:
        X, Y = data(20, 10, 4)
        run_pair(a, b, X, Y, 5, [0, 3, 3, 3, 3])
    finally:
        a.close()
        b.close()


def test_scratch_that_moves_between_replays_drops_the_recording(lib):
    """The recorded kernels hold addresses inside the context's scratch block.  When another call on the same
    context makes the block grow (and move), the recording is stale: the next epoch must notice, launch plainly
    and record again, and every epoch must still equal the twin that never records."""
    import ctypes
    widths = [20, 32, 24, 5]
    X, Y = data(50, 20, 5)
    a, b = build(lib, widths), build(lib, widths)
    try:
        run_pair(a, b, X, Y, 3, [0, 4, 4])
        lib.dlmi_ctx_scratch_generation.restype = ctypes.c_ulonglong
        lib.dlmi_ctx_scratch_generation.argtypes = [ctypes.c_void_p]
        lib.dlmi_ctx_reserve_layer.argtypes = [ctypes.c_void_p] + [ctypes.c_size_t] * 3
        gen = lib.dlmi_ctx_scratch_generation(b.context())
        # a very tall layer's loss pairs need more than the block holds: it grows
        assert lib.dlmi_ctx_reserve_layer(b.context(), 1 << 24, 0, 8) == 0
        assert lib.dlmi_ctx_scratch_generation(b.context()) == gen + 1
        run_pair(a, b, X, Y, 4, [0, 4, 4, 4])
    finally:
        a.close()
        b.close()


@pytest.mark.parametrize("widths,max_batch,n", [([20, 32, 24, 5], 16, 50), ([1024, 1024, 512, 10], 256, 600)])
def test_weight_gradients_beside_the_chain_match_one_stream(lib, widths, max_batch, n):
    """The weight gradients run on a second stream, and the one of the layer that reads the resident input rows is
    not waited for until the next pass overwrites what it reads: a twin created with DLMI_DW_STREAM=0 issues every
    launch on one stream, and parameters, gradients and moving statistics must stay bit-identical epoch after epoch,
    with plain launches (the wide network's products are large enough to go beside the chain there too) and with
    recorded mini-batches, with evaluation passes, downloads and an optimizer step between the passes."""
    import os
    os.environ["DLMI_DW_STREAM"] = "0"
    try:
        one = build(lib, widths, max_batch=max_batch)
    finally:
        del os.environ["DLMI_DW_STREAM"]
    two, rec = build(lib, widths, max_batch=max_batch), build(lib, widths, max_batch=max_batch)
    X, Y = data(n, widths[0], widths[-1])
    try:
        for e in range(5):
            r1 = one.train_epoch(X, Y, resample_masks=True, record_batches=False)
            r2 = two.train_epoch(X, Y, resample_masks=True, record_batches=False)
            r3 = rec.train_epoch(X, Y, resample_masks=True, record_batches=True)
            assert r2 == r1 and r3[1] == r1[1] and r3[0] == pytest.approx(r1[0], rel=1e-9), f"epoch {e}: {r1} / {r2} / {r3}"
            p1 = one.get_parameters()
            assert np.array_equal(p1, two.get_parameters()), f"epoch {e}: parameters (plain launches)"
            assert np.array_equal(p1, rec.get_parameters()), f"epoch {e}: parameters (recorded)"
            m1 = one.get_moving()
            for other in (two, rec):
                mo = other.get_moving()
                assert np.array_equal(m1[0], mo[0]) and np.array_equal(m1[1], mo[1]), f"epoch {e}: moving statistics"
            if e == 2:  # gradients as the last pass left them, before anything clears them
                assert np.array_equal(one.get_dparams(), two.get_dparams())
                assert np.array_equal(one.get_dparams(), rec.get_dparams())
            assert two.evalt(X, Y) == one.evalt(X, Y)
    finally:
        one.close()
        two.close()
        rec.close()


@pytest.mark.parametrize("widths,max_batch,n", [([20, 32, 24, 5], 16, 50), ([784, 512, 512, 10], 128, 1100), ([30, 40, 7], 8, 8)])
def test_two_lanes_match_one(lib, widths, max_batch, n):
    """The driver runs the mini-batches of a training pass alternately on two sets of per-batch buffers, each with a
    stream of its own, so that a forward pass overlaps the backward pass before it; only forward-after-forward and
    backward-after-backward are ordered.  A twin created with DLMI_LANES=0 has the one set: parameters, gradients,
    moving statistics, reports, the outputs of the last mini-batch and evaluation passes must stay bit-identical
    epoch after epoch, with plain launches and with recorded mini-batches (odd and even numbers of mini-batches, a
    ragged last one, a single mini-batch)."""
    import os
    os.environ["DLMI_LANES"] = "0"
    try:
        one = build(lib, widths, max_batch=max_batch)
    finally:
        del os.environ["DLMI_LANES"]
    two, rec = build(lib, widths, max_batch=max_batch), build(lib, widths, max_batch=max_batch)
    X, Y = data(n, widths[0], widths[-1])
    try:
        for e in range(5):
            r1 = one.train_epoch(X, Y, resample_masks=True, record_batches=False)
            r2 = two.train_epoch(X, Y, resample_masks=True, record_batches=False)
            r3 = rec.train_epoch(X, Y, resample_masks=True, record_batches=True)
            assert r2 == r1 and r3[1] == r1[1] and r3[0] == pytest.approx(r1[0], rel=1e-9), f"epoch {e}: {r1} / {r2} / {r3}"
            p1 = one.get_parameters()
            assert np.array_equal(p1, two.get_parameters()), f"epoch {e}: parameters (plain launches)"
            assert np.array_equal(p1, rec.get_parameters()), f"epoch {e}: parameters (recorded)"
            m1 = one.get_moving()
            for other in (two, rec):
                mo = other.get_moving()
                assert np.array_equal(m1[0], mo[0]) and np.array_equal(m1[1], mo[1]), f"epoch {e}: moving statistics"
                assert np.array_equal(one.get_dparams(), other.get_dparams()), f"epoch {e}: gradients"
                # what the last mini-batch left in the layers: its outputs (its rows), and the batch statistics
                last_rows = n - (n - 1) // max_batch * max_batch
                for m in (one, other):
                    m.B = last_rows
                assert np.array_equal(one.get_out(), other.get_out()), f"epoch {e}: outputs of the last mini-batch"
                for k in range(4):
                    assert np.array_equal(one.layer_vector(1, k), other.layer_vector(1, k)), f"epoch {e}: batch statistic {k}"
            assert two.evalt(X, Y) == one.evalt(X, Y) and rec.evalt(X, Y) == one.evalt(X, Y)
    finally:
        one.close()
        two.close()
        rec.close()


def test_which_models_get_a_second_lane(lib):
    """Plain layers on mini-batches of at most 256 rows, when the memory budget holds a second set of buffers and
    DLMI_LANES is not 0; everything else trains on the one set (and all of them train: the epoch must succeed)."""
    import os
    X, Y = data(40, 20, 5)

    def trained(m):
        r = m.train_epoch(X, Y)
        assert np.isfinite(r[0])
        return m.lanes_enabled()

    m = build(lib, [20, 32, 24, 5])
    try:
        assert not m.lanes_enabled()  # only the driver asks for it
        assert trained(m)
    finally:
        m.close()
    m = build(lib, [20, 32, 24, 5], max_batch=512)  # more rows per mini-batch than launch latency is the bound for
    try:
        Xb, Yb = data(1100, 20, 5)
        assert np.isfinite(m.train_epoch(Xb, Yb)[0]) and not m.lanes_enabled()
    finally:
        m.close()
    os.environ["DLMI_LANES"] = "0"
    try:
        m = build(lib, [20, 32, 24, 5])
    finally:
        del os.environ["DLMI_LANES"]
    try:
        assert not trained(m)
    finally:
        m.close()
    # a budget that holds the model and its one set of buffers, but not a second set
    m = build(lib, [20, 32, 24, 5])
    try:
        mem = m.memory()
        m.set_allowable_memory(mem["model_bytes"] + mem["bytes_per_example"] * 16 + mem["bytes_per_example"] * 8)
        assert not trained(m)
        m.set_allowable_memory(mem["model_bytes"] + mem["bytes_per_example"] * 16 * 4)
        assert trained(m)
    finally:
        m.close()
