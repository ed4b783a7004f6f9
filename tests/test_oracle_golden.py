"""The CPU restatement (oracle/dl_oracle.c) against golden vectors written by the
real reference sources (tests/golden/make_golden.py)."""
import numpy as np
import pytest

from helpers import RTOL_RESTATEMENT, assert_close
from oracle.binding import ACT, DROP, NORM, STATE

ACTS = ["ELU", "ISRLU", "LEAKY_RELU", "RELU", "SELU", "LINEAR"]
SETTINGS = dict(
    brn_loose=dict(fresh=True, mom=0.99, rmax=3.0, dmax=5.0, renorm=True),
    brn_tight=dict(fresh=False, mom=0.05, rmax=1.1, dmax=0.05, renorm=True),
    bn=dict(fresh=False, mom=0.3, rmax=1.0, dmax=0.0, renorm=False))
T = RTOL_RESTATEMENT


@pytest.mark.parametrize("case", [0, 1, 2])
@pytest.mark.parametrize("nt", [0, 3])
def test_leaves_against_reference_golden(oracle, golden_leaves, case, nt):
    g = golden_leaves
    p, q = f"c{case}_", f"c{case}_t{nt}_"
    B, K, H = (int(v) for v in g[p + "shape"])
    X, W, x = g[p + "X"], g[p + "W"], g[p + "x"]
    gamma, beta = g[p + "gamma"], g[p + "beta"]
    dN, dZ, mask = g[p + "dN"], g[p + "dZ"], g[p + "mask"]
    Z = oracle.fc_fwd(X, W, nt)
    assert_close(Z, g[q + "fc_fwd"], T, "fc_fwd")
    assert_close(oracle.bias_fwd(g[q + "fc_fwd"], g[p + "bias"], nt), g[q + "bias_fwd"], T, "bias_fwd")
    for sname, s in SETTINGS.items():
        mm = np.zeros(H, np.float32) if s["fresh"] else g[p + "mov_mean"]
        ms = np.ones(H, np.float32) if s["fresh"] else g[p + "mov_std"]
        fw = oracle.norm_fwd_train(x, gamma, beta, mm, ms, s["mom"], 1e-5, s["rmax"], s["dmax"], s["renorm"], nt)
        for k, v in fw.items():
            assert_close(v, g[f"{q}{sname}_fwd_{k}"], T, f"{sname} fwd {k}")
        if sname == "brn_tight":  # the clips must actually bind in this setting
            assert np.any(fw["r"] == np.float32(1.1)) or np.any(fw["r"] == np.float32(1) / np.float32(1.1))
            assert np.any(np.abs(fw["d"]) == np.float32(0.05))
        e = {k: g[f"{q}{sname}_fwd_{k}"] for k in ("mean", "std", "r", "xhat")}
        bw = oracle.norm_bwd(e["mean"], e["std"], gamma, e["r"], x, e["xhat"], dN, dgamma_init=gamma * 0.5,
                             dbeta_init=beta * 2, renorm=s["renorm"], nthreads=nt)
        for k, v in bw.items():
            assert_close(v, g[f"{q}{sname}_bwd_{k}"], 4 * T, f"{sname} bwd {k}")
    assert_close(oracle.norm_fwd_infer(x, gamma, beta, g[p + "mov_mean"], g[p + "mov_std"], nt),
                 g[q + "norm_infer"], T, "norm_infer")
    for a in ACTS:
        y = oracle.act_fwd(ACT[a], x, nt)
        assert_close(y, g[f"{q}act_fwd_{a}"], T, "act_fwd " + a)
        assert_close(oracle.act_bwd(ACT[a], x, g[f"{q}act_fwd_{a}"], dN, nt), g[f"{q}act_bwd_{a}"], T,
                     "act_bwd " + a)
    assert_close(oracle.softmax_fwd(x, nt), g[q + "softmax"], T, "softmax")
    inv = np.float32(1.0) / np.float32(0.7)
    assert np.array_equal(oracle.dropout_fwd(0, x, mask, inv, nt), g[q + "drop_inverted"])
    assert np.array_equal(oracle.dropout_fwd(1, x, mask, 0.0, nt), g[q + "drop_plain"])
    assert np.array_equal(oracle.dropout_fwd(2, x, None, 0.7, nt), g[q + "drop_infer"])
    # a [B,H] mask whose rows all equal the per-unit mask is the reference's semantics
    assert np.array_equal(oracle.dropout_fwd(0, x, np.tile(mask, (B, 1)), inv, nt), g[q + "drop_inverted"])
    assert np.array_equal(oracle.identity_add(x, dN, nt), g[q + "identity_add"])
    assert_close(oracle.fc_bwd_dx(dZ, W, nthreads=nt), g[q + "fc_bwd_dx"], 4 * T, "fc_bwd_dx")
    assert_close(oracle.fc_bwd_dx(dZ, W, dY_init=np.ones((B, K), np.float32), nthreads=nt),
                 g[q + "fc_bwd_dx_acc"], 4 * T, "fc_bwd_dx accumulate")
    dW, db = oracle.fc_bwd_dw(X, dZ, dW_init=g[p + "dW0"], db_init=g[p + "db0"], nthreads=nt)
    assert_close(dW, g[q + "fc_bwd_dw"], 4 * T, "fc_bwd_dw")
    assert_close(db, g[q + "fc_bwd_db"], 4 * T, "fc_bwd_db")


@pytest.mark.parametrize("a", ACTS)
def test_activation_special_points(oracle, golden_leaves, a):
    g = golden_leaves
    pts = g["pts"]
    y = oracle.act_fwd(ACT[a], pts)
    assert_close(y, g[f"pts_fwd_{a}"], T, "fwd " + a)
    # signed zeros come out exactly as the reference's
    assert np.array_equal(np.signbit(y), np.signbit(g[f"pts_fwd_{a}"]))
    d = oracle.act_bwd(ACT[a], pts, g[f"pts_fwd_{a}"], np.ones_like(pts))
    assert_close(d, g[f"pts_bwd_{a}"], T, "bwd " + a)


MLP_CASES = {
    "mlp_relu_brn": [("RELU", "BRN", "NONE", 1.0), ("RELU", "BRN", "NONE", 1.0)],
    "mlp_c1_small": [("RELU", "BRN", "NONE", 1.0), ("RELU", "BRN", "NONE", 1.0)],
    "mlp_mixed": [("SELU", "BRN", "BERNOULLI_INVERTED", 0.8), ("ELU", "NONE", "NONE", 1.0),
                  ("ISRLU", "BRN", "BERNOULLI", 0.6)],
    "mlp_bn": [("ISRLU", "BN", "NONE", 1.0), ("SELU", "BN", "BERNOULLI_INVERTED", 0.75)],
    "mlp_lrelu_plain": [("LEAKY_RELU", "NONE", "NONE", 1.0), ("LEAKY_RELU", "BRN", "NONE", 1.0)],
}


def build_mlp(factory, g, name, nt):
    hidden = MLP_CASES[name]
    widths = [int(w) for w in g[name + "_widths"]]
    L = len(widths)
    M = factory(widths)
    for l in range(1, L - 1):
        a, n, dr, keep = hidden[l - 1]
        M.set_layer(l, ACT[a], NORM[n], DROP[dr], keep, g[f"{name}_mask{l}"] if dr != "NONE" else None)
    M.set_layer(L - 1, ACT["SOFTMAX"])
    M.set_norm_hyper(*[float(v) for v in g[name + "_hyper"]])
    M.prepare(g[name + "_X"].shape[0], nt)
    return M, widths, hidden


@pytest.mark.parametrize("name", list(MLP_CASES))
@pytest.mark.parametrize("nt", [0, 3])
def test_mlp_step_against_reference_golden(oracle, golden_mlp, name, nt):
    g = golden_mlp
    M, widths, hidden = build_mlp(oracle.mlp, g, name, nt)
    L = len(widths)
    # packed parameter layout (weights | biases | gammas | betas)
    assert [M.P, M.n_units] == [int(v) for v in g[name + "_P"]]
    offs = np.array([M.layer_offsets(l) for l in range(L)])
    gold = g[name + "_offsets"]
    assert np.array_equal(offs[1:, :5], gold[1:, :5])
    assert np.array_equal(offs[1:-1, 5], gold[1:-1, 5])  # use_bias of the hidden layers
    M.parameters[:] = g[name + "_params"]
    q = f"{name}_t{nt}_"
    M.step(STATE["TRAINING"], g[name + "_X"], g[name + "_Y"], backward=True)
    tol = 8 * T
    for l in range(1, L):
        for which, wn in ((0, "Z"), (3, "out"), (4, "dZ")):
            assert_close(M.layer_buffer(l, which), g[f"{q}L{l}_{wn}"], tol, f"L{l} {wn}")
        if l < L - 1:
            assert_close(M.layer_buffer(l, 6), g[f"{q}L{l}_dAF"], tol, f"L{l} dAF")
            if hidden[l - 1][1] != "NONE":
                assert_close(M.layer_buffer(l, 1), g[f"{q}L{l}_xhat"], tol, f"L{l} xhat")
                assert_close(M.layer_buffer(l, 2), g[f"{q}L{l}_nrm"], tol, f"L{l} nrm")
                names = ("mean", "std", "r", "d") if hidden[l - 1][1] == "BRN" else ("mean", "std")
                for which, wn in enumerate(names):
                    assert_close(M.layer_vector(l, which), g[f"{q}L{l}_{wn}"], tol, f"L{l} {wn}")
    assert_close(M.get_dparams(), g[q + "dparams"], tol, "dparams")
    mm, ms = M.get_moving()
    assert_close(mm, g[q + "mov_mean"], tol, "moving mean")
    assert_close(ms, g[q + "mov_std"], tol, "moving std")
    M.step(STATE["INFERENCE"], g[name + "_X"], None, backward=False)
    for l in range(1, L):
        assert_close(M.layer_buffer(l, 3), g[f"{q}infer_L{l}_out"], tol, f"inference L{l} out")
