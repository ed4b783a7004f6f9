"""The LSUV scaling loop (v1/ops/initializers/lsuv.cpp:108-177) of the oracle: against the reference's own loop
compiled from its sources (bit for bit), and against what the mathematics fixes.  The orthogonal
pre-initialization of the reference (Eigen QR) is NOT part of either side here: PARITY UNPINNED for it."""
import numpy as np
import pytest

from oracle.binding import ACT, NORM, STATE


def build(make, widths, acts, norms, seed=3):
    m = make(widths)
    L = len(widths)
    for l in range(1, L):
        m.set_layer(l, ACT[acts[l - 1]], NORM[norms[l - 1]] if l < L - 1 else 0)
    m.set_norm_hyper(0.9, 1e-5, 3.0, 5.0)
    m.prepare(64)
    return m


def start_parameters(P, widths, seed):
    """Weights of very different scales per layer, so every layer needs scaling."""
    rng = np.random.default_rng(seed)
    p = np.zeros(P, np.float32)
    o = 0
    for l in range(1, len(widths)):
        n = widths[l] * widths[l - 1]
        p[o:o + n] = rng.normal(0, 0.02 * 7 ** (l % 3), n)
        o += n
    nb = sum(widths[1:])
    p[o:o + nb] = rng.normal(0, 1, nb)  # LSUV overwrites the biases
    rest = P - o - nb
    if rest:
        p[o + nb:o + nb + rest // 2] = rng.uniform(0.5, 1.5, rest // 2)   # scales
        p[o + nb + rest // 2:] = rng.normal(0, 0.3, rest - rest // 2)      # shifts
    return p


CASES = [
    ([12, 40, 24, 6], ["TANH", "ELU", "LINEAR"], ["NONE", "NONE"]),
    ([9, 33, 20, 16, 4], ["RELU", "SIGMOID", "SELU", "LINEAR"], ["NONE", "NONE", "NONE"]),
    ([10, 32, 16, 5], ["RELU", "TANH", "SIGMOID"], ["BRN", "BRN"]),
]


@pytest.mark.parametrize("widths,acts,norms", CASES)
@pytest.mark.parametrize("kw", [dict(), dict(max_n_trials=2, var_target=0.5, var_tolerance=0.001, bias=0.1, max_batch_size=20)])
def test_oracle_loop_is_the_references_loop(oracle, reference, widths, acts, norms, kw):
    o = build(oracle.mlp, widths, acts, norms)
    r = build(reference.mlp, widths, acts, norms)
    p0 = start_parameters(o.P, widths, 5)
    # the reference only has scale / shift slots once a layer is normalized; the oracle always has them
    assert r.P == o.P or (all(n == "NONE" for n in norms) and r.P == o.P - 2 * o.n_units)
    o.parameters[:] = p0
    r.set_parameters(p0[:r.P])
    X = np.random.default_rng(1).normal(0, 1, (48, widths[0])).astype(np.float32)
    trials = o.lsuv(X, **kw)
    r.lsuv(X, **kw)
    assert np.array_equal(o.parameters[:r.P], r.get_parameters()), "parameters after LSUV, bit for bit"
    if r.P == o.P:
        mo, mr = o.get_moving(), r.get_moving()
        assert np.array_equal(mo[0], mr[0]) and np.array_equal(mo[1], mr[1])
    assert max(trials) <= kw.get("max_n_trials", 10) and sum(trials) > 0
    # and the two variance routines agree on the same forward pass
    n = min(kw.get("max_batch_size", 32), 48)
    o.step(STATE["INFERENCE"], X[:n], None, backward=False)
    r.step(STATE["INFERENCE"], X[:n], None, backward=False)
    for l in range(1, len(widths)):
        assert o.layer_variance(l, n) == r.layer_variance(l, n)


def test_variance_is_the_population_variance_of_all_outputs(oracle):
    o = build(oracle.mlp, [7, 19, 5], ["TANH", "LINEAR"], ["NONE"])
    o.parameters[:] = start_parameters(o.P, o.widths, 2)
    X = np.random.default_rng(0).normal(0, 2, (31, 7)).astype(np.float32)
    o.step(STATE["INFERENCE"], X, None, backward=False)
    for l in (1, 2):
        y = o.layer_buffer(l, 3).astype(np.float64)
        assert o.layer_variance(l, 31) == pytest.approx(y.var(), rel=2e-5)  # np.var: ddof = 0, all values one population


def test_positively_homogeneous_layers_need_exactly_one_scaling(oracle):
    """LINEAR and RELU are positively homogeneous: multiplying the weights by s multiplies the outputs by s
    and the variance by s^2, so ONE scaling by sqrt(target / v0) lands on the target (to rounding), whatever the
    start.  The scaled weights are the closed form, layer by layer, each on the already scaled layers before."""
    widths = [8, 30, 22, 6]
    o = build(oracle.mlp, widths, ["RELU", "LINEAR", "RELU"], ["NONE", "NONE"])
    p0 = start_parameters(o.P, widths, 9)
    o.parameters[:] = p0
    X = np.random.default_rng(4).normal(0, 1, (32, 8)).astype(np.float32)
    trials = o.lsuv(X, var_target=2.0, var_tolerance=1e-3)
    assert trials == [0, 1, 1, 1]
    # closed form in float64
    a, off, w = X.astype(np.float64), 0, []
    for l in range(1, 4):
        n = widths[l] * widths[l - 1]
        W = p0[off:off + n].astype(np.float64).reshape(widths[l], widths[l - 1])
        z = a @ W.T
        y = np.maximum(z, 0) if l != 2 else z
        s = np.sqrt(2.0 / y.var())
        w.append((W * s).ravel())
        a = y * s
        assert abs(a.var() - 2.0) < 1e-9
        off += n
    assert np.allclose(o.parameters[:off], np.concatenate(w), rtol=2e-5, atol=0)
    nb = sum(widths[1:])
    assert np.all(o.parameters[off:off + nb] == 0)  # initial_bias
    o.step(STATE["INFERENCE"], X, None, backward=False)
    for l in (1, 2, 3):
        assert abs(o.layer_variance(l, 32) - 2.0) < 1e-3


def test_trial_limit_and_tolerance(oracle):
    """A saturating activation does not land in one step: with a tight tolerance the loop runs on; the trial
    limit ends it; a loose tolerance ends it early.  At the end every layer that was not cut short is inside
    the tolerance."""
    widths = [10, 64, 48, 3]
    X = np.random.default_rng(6).normal(0, 1, (32, 10)).astype(np.float32)

    def run(**kw):
        o = build(oracle.mlp, widths, ["TANH", "SIGMOID", "TANH"], ["NONE", "NONE"])
        o.parameters[:] = start_parameters(o.P, widths, 1) * 6
        t = o.lsuv(X, **kw)
        o.step(STATE["INFERENCE"], X, None, backward=False)
        return t, [o.layer_variance(l, 32) for l in (1, 2, 3)]

    t, v = run(var_target=0.3, var_tolerance=1e-4, max_n_trials=25)
    assert max(t) > 1 and max(t) <= 25
    for l in (1, 2, 3):
        assert t[l] == 25 or abs(v[l - 1] - 0.3) < 1e-4
    t2, _ = run(var_target=0.3, var_tolerance=1e-4, max_n_trials=2)
    assert t2 == [0] + [min(k, 2) for k in t[1:]]
    t3, v3 = run(var_target=0.3, var_tolerance=0.05, max_n_trials=25)
    # (the sigmoid layer can never reach 0.3: its outputs lie in (0, 1), whose variance is below 0.25)
    assert sum(t3) < sum(t) and all(k == 25 or abs(x - 0.3) < 0.05 for k, x in zip(t3[1:], v3))
    assert t[2] == 25 and t3[2] == 25
