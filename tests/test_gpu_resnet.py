"""The GPU facade on layer lists with the reference's residual blocks, against
tests/golden/resnet.npz (compiled reference): structure of the compiled model,
outputs of every entry in the three propagation states, the error of every
fully-connected layer, parameter gradients and moving statistics."""
import numpy as np
import pytest

from helpers import RTOL_REDUCED as TR
from oracle.binding import ACT, NORM, STATE, OracleNet
from test_oracle_resnet import build_resnet, check_resnet, load_resnet_golden, resnet_cases

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


@pytest.mark.parametrize("name", list(resnet_cases()))
def test_gpu_resnet_against_golden(net_factory, name):
    g = load_resnet_golden()
    M = build_resnet(net_factory, g, name, 0)
    check_resnet(M, g, name, 0, TR)


def test_gpu_resnet_initialize_train_evaluate_against_golden(net_factory):
    """The caller-side chain in one piece, on the network with dropout inside its
    blocks: Glorot initialization from a seeded generator (bit-identical), two
    Driver::train epochs of 30 rows in sub-batches of 11 with one Nesterov-momentum
    step each, then Driver::evalt — parameters after every epoch, losses,
    accuracies and moving statistics as the compiled reference has them."""
    from oracle.binding import OPT
    g = load_resnet_golden()
    name = "res_dropout_wide_block"
    M = build_resnet(net_factory, g, name, 0)
    M.glorot_uniform(2024, 0.0)
    assert np.array_equal(M.get_parameters(), g["epoch_t0_init"])
    M.set_optimizer(OPT["GD"], lr=0.01, momentum=0.9, nesterov=True, weight_decay=0.01)
    X, Y = g["epoch_X"], g["epoch_Y"]
    from helpers import assert_close
    exp = g["epoch_t0_loss_accu"]
    for e in range(2):
        loss, accu = M.train_epoch(X, Y, resample_masks=False)
        assert abs(loss - exp[e, 0]) <= TR * max(1.0, abs(exp[e, 0])), (e, loss, exp[e, 0])
        assert accu == pytest.approx(exp[e, 1], abs=1e-9), (e, accu, exp[e, 1])
        assert_close(M.get_parameters(), g[f"epoch_t0_e{e}_params"], TR, f"parameters after epoch {e}")
    loss, accu = M.evalt(X, Y)
    assert abs(loss - exp[2, 0]) <= TR * max(1.0, abs(exp[2, 0])) and accu == pytest.approx(exp[2, 1], abs=1e-9)
    mm, ms = M.get_moving()
    assert_close(mm, g["epoch_t0_mov_mean"], TR, "moving mean", floor=1.0)
    assert_close(ms, g["epoch_t0_mov_std"], TR, "moving std")


def test_gpu_resnet_wide_against_oracle(net_factory, oracle):
    """Widths and a batch at which the GEMM tiles, the split reductions and the
    16-byte paths are all in play: two blocks (one widening, one narrowing the
    stream), batch renormalization on every entry, against the oracle."""
    layers = [("FC", 96), ("FC", 160), ("RES", 2), ("FC", 192), ("FC", 224), ("RES", 3), ("FC", 128), ("FC", 128), ("FC", 150),
              ("FC", 10)]
    B = 300
    rng = np.random.default_rng(7)

    def build(make):
        M = make(layers)
        M.set_layer(1, ACT["RELU"], NORM["BRN"])
        M.set_layer(2, 0, NORM["BRN"])
        for l, a in ((3, "ELU"), (4, "SELU"), (6, "ISRLU"), (7, "LEAKY_RELU"), (8, "ELU")):
            M.set_layer(l, ACT[a], NORM["BRN"] if l != 7 else 0)
        M.set_layer(9, ACT["SOFTMAX"])
        M.set_norm_hyper(0.9, 1e-5, 3.0, 5.0)
        M.prepare(B)
        return M

    G, O = build(net_factory), build(lambda ls: OracleNet(oracle, ls))
    assert G.P == O.P and G.n_units == O.n_units
    for l in range(len(layers)):
        assert G.info(l) == O.info(l), l
    p = O.get_parameters()
    nwb = O.info(0)["gamma"]
    for l in O.fc_layers():
        i = O.info(l)
        fan_in = (i["w1"] - i["w0"]) // i["n_out"]
        p[i["w0"]:i["w1"]] = rng.normal(0, 1.0 / np.sqrt(fan_in), i["w1"] - i["w0"])
    p[nwb - sum(O.info(l)["n_out"] for l in O.fc_layers()):nwb] = rng.uniform(-0.1, 0.1, sum(O.info(l)["n_out"] for l in O.fc_layers()))
    p[nwb:nwb + O.n_units] = rng.uniform(0.8, 1.2, O.n_units)
    p[nwb + O.n_units:] = rng.uniform(-0.1, 0.1, O.n_units)
    X = rng.uniform(0, 1, (B, 96)).astype(np.float32)
    Y = np.eye(10, dtype=np.float32)[rng.integers(0, 10, B)]
    from helpers import assert_close
    for M in (G, O):
        M.set_parameters(p)
    for st in ("TRAINING", "INFERENCE"):
        for M in (G, O):
            M.step(STATE[st], X, Y, backward=(st == "TRAINING"))
        for l in range(1, len(layers)):
            assert_close(G.layer_output(l), O.layer_output(l), TR, f"{st} output of entry {l}")
        if st == "TRAINING":
            for l in O.fc_layers():
                assert_close(G.layer_error(l), O.layer_error(l), TR, f"dZ of layer {l}")
            assert_close(G.get_dparams(), O.get_dparams(), TR, "parameter gradients")
            for a, b, what in zip(G.get_moving(), O.get_moving(), ("moving mean", "moving std")):
                assert_close(a, b, TR, what, floor=1.0)
