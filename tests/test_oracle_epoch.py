"""Epoch driver (Driver::train / Driver::evalt, drivers/driver.cpp:60-340) of the
oracle's whole-model restatement against tests/golden/epoch.npz, which the
compiled reference wrote: loss, accuracy, parameters and moving statistics over
three training epochs (sub-batches accumulate gradients, one update per epoch)
and one evaluation pass."""
import json
import os

import numpy as np
import pytest

from conftest import ROOT
from helpers import RTOL_RESTATEMENT, assert_close
from oracle.binding import ACT, DROP, NORM, OPT, OracleMLP

T = 16 * RTOL_RESTATEMENT  # three optimizer steps compound the rounding differences of the threaded sums


def load_epoch_golden():
    return np.load(os.path.join(ROOT, "tests", "golden", "epoch.npz"), allow_pickle=False)


def epoch_cases():
    return json.loads(bytes(load_epoch_golden()["epoch_cases_json"]))


def build_epoch_model(make, g, name, nt):
    """`make(widths)` returns a whole-model wrapper (oracle, reference or GPU facade)."""
    widths, n, sub, hidden, kind, kw = epoch_cases()[name]
    L = len(widths)
    M = make(widths)
    for l in range(1, L - 1):
        a, nm, dr, keep = hidden[l - 1]
        M.set_layer(l, ACT[a], NORM[nm], DROP[dr], keep, g[f"{name}_mask{l}"] if dr != "NONE" else None)
    M.set_layer(L - 1, ACT["SOFTMAX"])
    M.set_norm_hyper(0.9, 1e-5, 3.0, 5.0)
    M.prepare(sub, nt)
    M.set_parameters(g[name + "_params"])
    M.set_optimizer(OPT[kind], **kw)
    return M


def check_epochs(M, g, name, nt, tol, get_params, get_moving):
    la = g[f"{name}_t{nt}_loss_accu"]
    X, Y = g[name + "_X"], g[name + "_Y"]
    for e in range(3):
        loss, accu = M.train_epoch(X, Y)
        assert abs(loss - la[e, 0]) <= 10 * tol * abs(la[e, 0]), f"epoch {e} loss {loss} vs {la[e, 0]}"
        assert abs(accu - la[e, 1]) < 1e-9, f"epoch {e} accuracy {accu} vs {la[e, 1]}"
        assert_close(get_params(M), g[f"{name}_t{nt}_e{e}_params"], (e + 1) * tol, f"parameters after epoch {e}")
    loss, accu = M.evalt(X, Y)
    assert abs(loss - la[3, 0]) <= 100 * tol * abs(la[3, 0]), f"evaluation loss {loss} vs {la[3, 0]}"
    assert abs(accu - la[3, 1]) < 1e-9, f"evaluation accuracy {accu} vs {la[3, 1]}"
    mm, ms = get_moving(M)
    assert_close(mm, g[f"{name}_t{nt}_mov_mean"], 4 * tol, "moving mean", floor=1.0)
    assert_close(ms, g[f"{name}_t{nt}_mov_std"], 4 * tol, "moving std")


class _OracleModel(OracleMLP):
    def set_parameters(self, p):
        self.parameters[:] = p


@pytest.mark.parametrize("nt", [0, 3])
@pytest.mark.parametrize("name", list(epoch_cases()))
def test_oracle_epochs_against_golden(oracle, name, nt):
    g = load_epoch_golden()
    M = build_epoch_model(lambda w: _OracleModel(oracle, w), g, name, nt)
    check_epochs(M, g, name, nt, T, lambda m: m.parameters.copy(),
                 lambda m: (m.moving_mean.copy(), m.moving_std.copy()))


def test_one_update_per_epoch_uses_the_whole_data_set_as_batch(oracle):
    """Driver::train_st ends in update_weights_st(n_data, n_data): with normalized
    weight decay the factor is sqrt(n/(n*epoch)) = 1/sqrt(epoch) whatever the
    sub-batch size, and the time step advances once per epoch."""
    g = load_epoch_golden()
    M = build_epoch_model(lambda w: _OracleModel(oracle, w), g, "epoch_adam_brn", 0)
    X, Y = g["epoch_adam_brn_X"], g["epoch_adam_brn_Y"]
    for e in range(1, 4):
        assert abs(float(M.opt.wd(X.shape[0], X.shape[0])) - 0.01 / np.sqrt(e)) < 1e-7
        M.train_epoch(X, Y)
        assert float(M.opt.t) == e and float(M.opt.epoch_time_step) == e + 1
