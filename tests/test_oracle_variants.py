"""Layer orderings and propagation states beyond the main golden file, against
tests/golden/variants.npz (written by the compiled reference): normalization
AFTER the activation (fwp_st.cpp:466-511, 635-655; bwp_st.cpp:559-606), where
dropout then acts on the normalized values, and the UPDATE_BATCH_NORM forward
(batch statistics and moving-average update, but the inference branch of
dropout)."""
import json
import os

import numpy as np
import pytest

from conftest import ROOT
from helpers import RTOL_RESTATEMENT, assert_close
from oracle.binding import ACT, DROP, NORM, STATE, OracleMLP

T = 8 * RTOL_RESTATEMENT


def load_variants_golden():
    g = np.load(os.path.join(ROOT, "tests", "golden", "variants.npz"), allow_pickle=False)
    return {k: g[k] for k in g.files}


def variant_cases():
    return json.loads(bytes(load_variants_golden()["variant_cases_json"]))


def build_variant_model(make, g, name, nt):
    widths, B, hidden, hyper = variant_cases()[name]
    L = len(widths)
    M = make(widths)
    for l in range(1, L - 1):
        a, nm, dr, keep, before = hidden[l - 1]
        M.set_layer(l, ACT[a], NORM[nm], DROP[dr], keep, g[f"{name}_mask{l}"] if dr != "NONE" else None,
                    norm_before=before)
    M.set_layer(L - 1, ACT["SOFTMAX"])
    M.set_norm_hyper(*hyper)
    M.prepare(B, nt)
    M.set_parameters(g[name + "_params"])
    return M


def check_variant(M, g, name, nt, tol, get_moving):
    """`M.layer_buffer(l, 3)` = the layer's output, `(l, 4)` = its dZ."""
    L = len(variant_cases()[name][0])
    X, Y = g[name + "_X"], g[name + "_Y"]
    q = f"{name}_t{nt}_"
    M.step(STATE["TRAINING"], X, Y, backward=True)
    for l in range(1, L):
        assert_close(M.layer_buffer(l, 3), g[f"{q}train_L{l}_out"], tol, f"training L{l} output")
        assert_close(M.layer_buffer(l, 4), g[f"{q}train_L{l}_dZ"], tol, f"training L{l} dZ")
    assert_close(M.get_dparams(), g[q + "dparams"], tol, "dparams")
    mm, ms = get_moving(M)
    assert_close(mm, g[q + "train_mov_mean"], tol, "moving mean after the training step", floor=1.0)
    assert_close(ms, g[q + "train_mov_std"], tol, "moving std after the training step")
    M.step(STATE["UPDATE_BATCH_NORM"], X, None, backward=False)
    for l in range(1, L):
        assert_close(M.layer_buffer(l, 3), g[f"{q}ubn_L{l}_out"], tol, f"update-batch-norm L{l} output")
    mm, ms = get_moving(M)
    assert_close(mm, g[q + "ubn_mov_mean"], tol, "moving mean after the update-batch-norm pass", floor=1.0)
    assert_close(ms, g[q + "ubn_mov_std"], tol, "moving std after the update-batch-norm pass")
    M.step(STATE["INFERENCE"], X, None, backward=False)
    for l in range(1, L):
        assert_close(M.layer_buffer(l, 3), g[f"{q}infer_L{l}_out"], tol, f"inference L{l} output")


class _OracleModel(OracleMLP):
    def set_parameters(self, p):
        self.parameters[:] = p


@pytest.mark.parametrize("nt", [0, 3])
@pytest.mark.parametrize("name", list(variant_cases()))
def test_oracle_variants_against_golden(oracle, name, nt):
    g = load_variants_golden()
    M = build_variant_model(lambda w: _OracleModel(oracle, w), g, name, nt)
    check_variant(M, g, name, nt, T, lambda m: (m.moving_mean.copy(), m.moving_std.copy()))


def test_update_batch_norm_pass_moves_the_averages_but_uses_no_mask():
    """What the golden numbers say about PROPAGATION::UPDATE_BATCH_NORM: the moving
    statistics change again, and a plain-Bernoulli layer's output is the un-masked
    activation times keep (every unit non-zero where the training output had
    masked units at exactly zero)."""
    g = load_variants_golden()
    name = "var_before_dropout"
    q = name + "_t0_"
    assert not np.array_equal(g[q + "train_mov_mean"], g[q + "ubn_mov_mean"])
    mask = g[name + "_mask1"].astype(bool)
    assert (~mask).any()
    assert not g[q + "train_L1_out"][:, ~mask].any()
    assert g[q + "ubn_L1_out"][:, ~mask].all()
