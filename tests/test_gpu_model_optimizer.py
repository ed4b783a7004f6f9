"""Model::set_optimizer / set_weight_decay / Update_Parameter of the C++ facade
against the golden vectors of the compiled reference: the optimizer step on
given gradients, and whole training steps (forward, error, backward,
derivatives, update) repeated on one batch."""
import json
import os

import numpy as np
import pytest

from conftest import ROOT
from helpers import RTOL_ELEMENTWISE as TE
from helpers import RTOL_REDUCED as TR
from helpers import assert_close
from oracle.binding import ACT, NORM, OPT, STATE
from test_oracle_optimizers import leaf_case_names

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def golden_optim():
    return np.load(os.path.join(ROOT, "tests", "golden", "optim.npz"), allow_pickle=False)


@pytest.fixture(scope="module")
def model_factory(pkg):
    from deep_learning_amd.model import Model
    lib = pkg.load_library()
    made = []

    def make(widths, batch):
        m = Model(lib, widths)
        made.append(m)
        for l in range(1, len(widths) - 1):
            m.set_layer(l, ACT["RELU"], NORM["BRN"])
        m.set_layer(len(widths) - 1, ACT["SOFTMAX"])
        m.set_norm_hyper(0.99, 1e-5, 3.0, 5.0)
        m.prepare(batch)
        return m

    yield make
    for m in made:
        m.close()


@pytest.mark.parametrize("name", leaf_case_names())
def test_update_parameter_against_golden(model_factory, golden_optim, name):
    g = golden_optim
    kind, kw = json.loads(bytes(g["opt_cases_json"]))["leaf"][name]
    B, N = (int(v) for v in g["opt_sizes"])
    M = model_factory([8, 6, 6, 3], B)
    assert M.P == g["opt_p0"].size
    M.set_parameters(g["opt_p0"])
    M.set_optimizer(OPT[kind], **kw)
    mask = g[f"opt_{name}_mask"]
    if mask.size:
        assert np.array_equal(M.opt_state(4), mask), "regularization mask: 1 on the weights only"
    steps = len(g["opt_grads"])
    for t in range(steps):
        M.set_dparams(g["opt_grads"][t])
        M.update_parameter(B, N)
        assert_close(M.get_parameters(), g[f"opt_{name}_t0_s{t}_params"], TE, f"{name} parameters after step {t}")
        assert not M.get_dparams().any(), "Update_Parameter zeroes the gradient array"
    q = f"opt_{name}_t0_s{steps - 1}_"
    for which, key in ((0, "delta"), (1, "m1"), (2, "m2"), (3, "vhat"), (5, "prev_g"), (6, "steps")):
        if q + key in g.files:
            assert_close(M.opt_state(which), g[q + key], TE, f"{name} {key}")


@pytest.mark.parametrize("name", ["traj_adam", "traj_momentum_wd"])
def test_training_trajectory_against_golden(model_factory, golden_optim, name):
    g = golden_optim
    kind, kw = json.loads(bytes(g["opt_cases_json"]))["traj"][name]
    widths = [int(w) for w in g[name + "_widths"]]
    X, Y = g[name + "_X"], g[name + "_Y"]
    B = X.shape[0]
    M = model_factory(widths, B)
    M.set_parameters(g[name + "_params"])
    M.set_optimizer(OPT[kind], **kw)
    for t in range(3):
        M.step(STATE["TRAINING"], X, Y, backward=True)
        if t == 0:
            assert_close(M.get_dparams(), g[f"{name}_t0_s0_dparams"], TR, "gradient of the first step")
        M.update_parameter(B, 5 * B)
        # one step later a rounding difference in a gradient shows up in the parameters scaled by the step size
        assert_close(M.get_parameters(), g[f"{name}_t0_s{t}_params"], (t + 1) * TR, f"parameters after step {t}")
    mm, ms = M.get_moving()
    assert_close(mm, g[f"{name}_t0_mov_mean"], 4 * TR, "moving mean", floor=1.0)
    assert_close(ms, g[f"{name}_t0_mov_std"], 4 * TR, "moving std")


def test_unsupported_optimizer_is_refused(model_factory):
    M = model_factory([8, 6, 6, 3], 4)
    with pytest.raises(Exception):
        M.set_optimizer(7)  # iRPROP-: the reference's Update_Parameter does not dispatch it either
