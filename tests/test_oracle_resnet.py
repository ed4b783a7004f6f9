"""Layer lists with the reference's residual blocks (Forward_Pass__Residual__Loop
and __Residual__FC__Loop, fwp_st.cpp:3876-4442; the residual branches of the
backward pass, bwp_st.cpp:80-185, 345-541, 1112-1175) against
tests/golden/resnet.npz, which the compiled reference wrote: structure
(parameter layout, unit counts, derived shortcut padding), the outputs of every
entry in the three propagation states, the error of every fully-connected layer,
parameter gradients and moving statistics."""
import json
import os

import numpy as np
import pytest

from conftest import ROOT
from helpers import RTOL_RESTATEMENT, assert_close
from oracle.binding import ACT, DROP, NORM, STATE, OracleNet

T = 8 * RTOL_RESTATEMENT


def load_resnet_golden():
    g = np.load(os.path.join(ROOT, "tests", "golden", "resnet.npz"), allow_pickle=False)
    return {k: g[k] for k in g.files}


def resnet_cases():
    raw = json.loads(bytes(load_resnet_golden()["resnet_cases_json"]))
    return {k: ([tuple(e) for e in v[0]], v[1], {int(a): b for a, b in v[2].items()}, v[3]) for k, v in raw.items()}


def build_resnet(make, g, name, nt):
    layers, B, cfg, hyper = resnet_cases()[name]
    M = make(layers)
    for l, (a, nm, dr, keep) in cfg.items():
        M.set_layer(l, ACT[a] if a else 0, NORM[nm], DROP[dr], keep, g.get(f"{name}_mask{l}"))
    M.set_layer(len(layers) - 1, ACT["SOFTMAX"])
    M.set_norm_hyper(*hyper)
    M.prepare(B, nt)
    return M


def check_resnet(M, g, name, nt, tol):
    layers = resnet_cases()[name][0]
    n = len(layers)
    keys = ("type", "n_out", "w0", "w1", "bias", "use_bias", "n_unit", "gamma", "unit", "n_af", "depth", "padding")
    for l in range(n):
        got, exp = M.info(l), dict(zip(keys, (int(v) for v in g[name + "_info"][l])))
        skip = ("w1",) if layers[l][0] != "FC" or l == 0 else ()
        if layers[l][0] == "RES" or l == 0:
            skip += ("use_bias",)  # meaningless for entries without weights
        for k in keys:
            if k not in skip:
                assert got[k] == exp[k], f"entry {l} {k}: {got[k]} != {exp[k]}"
    assert [M.P, M.n_units] == [int(v) for v in g[name + "_P"]]
    M.set_parameters(g[name + "_params"])
    X, Y = g[name + "_X"], g[name + "_Y"]
    q = f"{name}_t{nt}_"
    for st in ("TRAINING", "UPDATE_BATCH_NORM", "INFERENCE"):
        M.step(STATE[st], X, Y, backward=(st == "TRAINING"))
        for l in range(1, n):
            assert_close(M.layer_output(l), g[f"{q}{st}_L{l}_out"], tol, f"{st} output of entry {l}")
        if st == "TRAINING":
            for l in M.fc_layers():
                assert_close(M.layer_error(l), g[f"{q}L{l}_dZ"], tol, f"dZ of layer {l}")
            assert_close(M.get_dparams(), g[q + "dparams"], tol, "parameter gradients")
            mm, ms = M.get_moving()
            assert_close(mm, g[q + "mov_mean"], tol, "moving mean", floor=1.0)
            assert_close(ms, g[q + "mov_std"], tol, "moving std")


@pytest.mark.parametrize("nt", [0, 3])
@pytest.mark.parametrize("name", list(resnet_cases()))
def test_oracle_resnet_against_golden(oracle, name, nt):
    g = load_resnet_golden()
    M = build_resnet(lambda layers: OracleNet(oracle, layers), g, name, nt)
    check_resnet(M, g, name, nt, T)


def test_block_without_weights_is_the_identity_plus_block(oracle):
    """With every block weight zero and no block-level normalization the block
    contributes only its last bias, so out = shortcut + bias: the shortcut wiring
    checked without any arithmetic of its own."""
    layers = [("FC", 5), ("FC", 6), ("RES", 2), ("FC", 4), ("FC", 6), ("FC", 3)]
    M = OracleNet(oracle, layers)
    M.set_layer(1, ACT["RELU"], NORM["BN"])
    M.set_layer(3, ACT["ELU"])
    M.set_layer(4, ACT["ELU"])
    M.set_layer(5, ACT["SOFTMAX"])
    M.prepare(4)
    p = M.get_parameters()
    rng = np.random.default_rng(0)
    i1, i3, i4 = M.info(1), M.info(3), M.info(4)
    p[i1["w0"]:i1["w1"]] = rng.uniform(-1, 1, i1["w1"] - i1["w0"])
    p[i3["w0"]:i4["w1"]] = 0
    bias4 = rng.uniform(-1, 1, 6).astype(np.float32)
    p[i4["bias"]:i4["bias"] + 6] = bias4
    M.set_parameters(p)
    M.step(STATE["TRAINING"], rng.uniform(0, 1, (4, 5)).astype(np.float32), None, backward=False)
    assert np.array_equal(M.layer_output(2), M.layer_output(1) + bias4)
