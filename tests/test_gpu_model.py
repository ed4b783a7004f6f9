"""The C++ Model facade (reference API, GPU execution) against the whole-model
golden vectors written by the real reference, and against the oracle at the
784-512-512-10 / batch 128 configuration."""
import numpy as np
import pytest

from helpers import RTOL_REDUCED as TR
from helpers import assert_close
from oracle.binding import ACT, DROP, NORM, STATE
from test_oracle_golden import MLP_CASES, build_mlp

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


@pytest.mark.parametrize("name", list(MLP_CASES))
def test_model_step_against_reference_golden(model_factory, golden_mlp, name):
    g = golden_mlp
    M, widths, hidden = build_mlp(model_factory, g, name, 0)
    L = len(widths)
    assert [M.P, M.n_units] == [int(v) for v in g[name + "_P"]]
    offs = np.array([M.layer_offsets(l) for l in range(L)])
    gold = g[name + "_offsets"]
    assert np.array_equal(offs[1:, :5], gold[1:, :5])
    assert np.array_equal(offs[1:-1, 5], gold[1:-1, 5])
    M.set_parameters(g[name + "_params"])
    q = f"{name}_t0_"
    M.step(STATE["TRAINING"], g[name + "_X"], g[name + "_Y"], backward=True)
    for l in range(1, L):
        for which, wn in ((0, "Z"), (3, "out"), (4, "dZ")):
            assert_close(M.layer_buffer(l, which), g[f"{q}L{l}_{wn}"], TR, f"L{l} {wn}")
        if l < L - 1 and hidden[l - 1][1] != "NONE":
            names = ("mean", "std", "r", "d") if hidden[l - 1][1] == "BRN" else ("mean", "std")
            for which, wn in enumerate(names):
                assert_close(M.layer_vector(l, which), g[f"{q}L{l}_{wn}"], TR, f"L{l} {wn}",
                             floor=1.0 if wn == "d" else 0.0)
    assert_close(M.get_out(), g[f"{q}L{L - 1}_out"], TR, "get_out")
    assert_close(M.get_dparams(), g[q + "dparams"], TR, "dparams")
    mm, ms = M.get_moving()
    assert_close(mm, g[q + "mov_mean"], TR, "moving mean", floor=1.0)
    assert_close(ms, g[q + "mov_std"], TR, "moving std")
    M.step(STATE["INFERENCE"], g[name + "_X"], None, backward=False)
    for l in range(1, L):
        assert_close(M.layer_buffer(l, 3), g[f"{q}infer_L{l}_out"], TR, f"inference L{l} out")


def test_setters_refuse_what_the_reference_refuses(model_factory):
    M = model_factory([8, 6, 6, 3])
    lib, h = M.lib, M.h
    import ctypes
    c_sz, c_int = ctypes.c_size_t, ctypes.c_int
    # normalization on the input / output layer (normalization.cpp:206-215)
    assert lib.dlmi_model_set_layer_normalization(h, c_sz(0), c_int(NORM["BRN"])) == 0
    assert lib.dlmi_model_set_layer_normalization(h, c_sz(3), c_int(NORM["BRN"])) == 0
    assert lib.dlmi_model_set_layer_normalization(h, c_sz(1), c_int(NORM["BRN"])) == 1
    # softmax anywhere but the output layer (train.cpp:400-406)
    assert lib.dlmi_model_set_layer_activation_function(h, c_sz(1), c_int(ACT["SOFTMAX"])) == 0
    assert lib.dlmi_model_set_layer_activation_function(h, c_sz(3), c_int(ACT["SOFTMAX"])) == 1
    # activations outside the path
    assert lib.dlmi_model_set_layer_activation_function(h, c_sz(1), c_int(19)) == 0  # SINE
    # batch size 0 (model.cpp:2652)
    assert lib.dlmi_model_prepare(h, c_sz(0)) == 0


def test_mlp_784_512_512_10_against_oracle(model_factory, oracle):
    """Configuration 1: 3-layer MLP 784-512-512-10, batch 128, FC -> batch renorm
    (rmax 3, dmax 5, momentum 0.99, eps 1e-5) -> ReLU hidden layers, softmax +
    cross-entropy output, Glorot-uniform weights, zero biases; two training
    steps accumulate gradients, then an inference pass."""
    widths, B = [784, 512, 512, 10], 128
    rng = np.random.default_rng(1234)
    X = rng.uniform(0, 1, (B, 784)).astype(np.float32)
    Y = np.eye(10, dtype=np.float32)[rng.integers(0, 10, B)]
    models = []
    for factory in (oracle.mlp, model_factory):
        M = factory(widths)
        for l in (1, 2):
            M.set_layer(l, ACT["RELU"], NORM["BRN"])
        M.set_layer(3, ACT["SOFTMAX"])
        M.set_norm_hyper(0.99, 1e-5, 3.0, 5.0)
        M.prepare(B, oracle.max_threads())
        models.append(M)
    O, G = models
    assert O.P == G.P == 673342  # W 401408 + 262144 + 5120, b 1034, gamma/beta 2 x 1818
    params = O.parameters.copy()  # gamma 1, beta 0, biases 0
    for l in range(1, 4):
        K, H = widths[l - 1], widths[l]
        lim = np.sqrt(6.0 / (K + H))
        o = O.layer_offsets(l)[0]
        params[o:o + H * K] = rng.uniform(-lim, lim, H * K).astype(np.float32)
    O.parameters[:] = params
    G.set_parameters(params)
    for _ in range(2):
        O.step(STATE["TRAINING"], X, Y, backward=True)
        G.step(STATE["TRAINING"], X, Y, backward=True)
    for l in range(1, 4):
        for which, wn in ((0, "Z"), (3, "out"), (4, "dZ")):
            assert_close(G.layer_buffer(l, which), O.layer_buffer(l, which), TR, f"L{l} {wn}")
    assert_close(G.get_dparams(), O.get_dparams(), TR, "accumulated parameter gradients")
    mo, so = O.get_moving()
    mg, sg = G.get_moving()
    assert_close(mg, mo, TR, "moving mean", floor=1.0)
    assert_close(sg, so, TR, "moving std")
    assert abs(G.loss_sum() - O.lib.dlo_mlp_loss_sum(O.h)) <= 1e-4 * abs(G.loss_sum())
    assert G.accuracy_sum() == O.lib.dlo_mlp_n_correct(O.h)
    O.step(STATE["INFERENCE"], X, None, backward=False)
    G.step(STATE["INFERENCE"], X, None, backward=False)
    assert_close(G.get_out(), O.layer_buffer(3, 3), TR, "inference output")


def test_masked_dropout_backward_mode(model_factory, oracle):
    """The facade's optional mathematically-matching dropout backward (gradient
    masked and rescaled, derivative of the pre-dropout activation), checked
    against a hand-assembled oracle pipeline on one hidden layer."""
    widths, B = [12, 16, 5], 9
    rng = np.random.default_rng(7)
    X = rng.standard_normal((B, 12)).astype(np.float32)
    Y = np.eye(5, dtype=np.float32)[rng.integers(0, 5, B)]
    keep = 0.75
    mask = (rng.uniform(size=16) < keep).astype(np.uint8)
    G = model_factory(widths)
    G.set_layer(1, ACT["SELU"], NORM["BRN"], DROP["BERNOULLI_INVERTED"], keep, mask)
    G.set_layer(2, ACT["SOFTMAX"])
    G.set_norm_hyper(0.9, 1e-5, 3.0, 5.0)
    G.set_dropout_backward_mode(True)
    G.prepare(B)
    params = G.get_parameters()
    o1, o2 = G.layer_offsets(1), G.layer_offsets(2)
    W1 = rng.uniform(-.5, .5, (16, 12)).astype(np.float32); W2 = rng.uniform(-.5, .5, (5, 16)).astype(np.float32)
    params[o1[0]:o1[0] + 192] = W1.ravel(); params[o2[0]:o2[0] + 80] = W2.ravel()
    G.set_parameters(params)
    G.step(STATE["TRAINING"], X, Y, backward=True)
    one, zero = np.ones(16, np.float32), np.zeros(16, np.float32)
    scale = np.float32(1.0) / np.float32(keep)
    Z1 = oracle.fc_fwd(X, W1)
    fw = oracle.norm_fwd_train(Z1, one, zero, zero, one, 0.9, 1e-5, 3.0, 5.0, True)
    q = oracle.act_fwd(ACT["SELU"], fw["out"])
    y1 = oracle.dropout_fwd(0, q, mask, scale)
    Z2 = oracle.bias_fwd(oracle.fc_fwd(y1, W2), np.zeros(5, np.float32))
    dZ2, _, _ = oracle.softmax_ce_seed(oracle.softmax_fwd(Z2), Y)
    dY1 = oracle.fc_bwd_dx(dZ2, W2)
    dN = oracle.act_bwd(ACT["SELU"], fw["out"], q, oracle.dropout_fwd(0, dY1, mask, scale))
    bw = oracle.norm_bwd(fw["mean"], fw["std"], one, fw["r"], Z1, fw["xhat"], dN)
    assert_close(G.layer_buffer(1, 3), y1, TR, "hidden output")
    assert_close(G.layer_buffer(1, 4), bw["dx"], TR, "dZ1 (masked backward)")
    dW1, _ = oracle.fc_bwd_dw(X, bw["dx"], with_bias=False)
    assert_close(G.get_dparams()[o1[0]:o1[0] + 192].reshape(16, 12), dW1, TR, "dW1")
