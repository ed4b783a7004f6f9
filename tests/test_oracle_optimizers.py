"""Optimizer steps of the oracle: against the golden vectors the compiled
reference wrote (tests/golden/optim.npz), against closed forms and torch's
library optimizers, and against the compiled reference on fresh random cases."""
import json

import numpy as np
import pytest
import torch

from helpers import RTOL_RESTATEMENT, assert_close
from oracle.binding import ACT, NORM, OPT, OptimizerHost

T = 4 * RTOL_RESTATEMENT


@pytest.fixture(scope="session")
def golden_optim():
    import os
    from conftest import ROOT
    return np.load(os.path.join(ROOT, "tests", "golden", "optim.npz"), allow_pickle=False)


def cases(g, which):
    return json.loads(bytes(g["opt_cases_json"]))[which]


def leaf_case_names():
    import os
    from conftest import ROOT
    g = np.load(os.path.join(ROOT, "tests", "golden", "optim.npz"), allow_pickle=False)
    return list(json.loads(bytes(g["opt_cases_json"]))["leaf"])


def run_leaf_case(leaves, g, name, nt):
    """Replays one golden optimizer case on `leaves`; yields (step, params, host)."""
    kind, kw = cases(g, "leaf")[name]
    mask = g[f"opt_{name}_mask"]
    p = g["opt_p0"].copy()
    rows = [tuple(int(v) for v in r) for r in g["opt_weight_rows"]]
    host = OptimizerHost(leaves, p.size, OPT[kind], mask=mask if mask.size else None, weight_rows=rows, **kw)
    B, N = (int(v) for v in g["opt_sizes"])
    for t, grad in enumerate(g["opt_grads"]):
        gg = grad.copy()
        host.update(p, gg, B, N, nt)
        assert not gg.any(), "the step zeroes the gradient it consumed"
        yield t, p, host


@pytest.mark.parametrize("nt", [0, 3])
@pytest.mark.parametrize("name", leaf_case_names())
def test_oracle_optimizer_against_golden(oracle, golden_optim, name, nt):
    g = golden_optim
    for t, p, host in run_leaf_case(oracle, g, name, nt):
        assert_close(p, g[f"opt_{name}_t{nt}_s{t}_params"], T, f"{name} parameters after step {t}")
    q = f"opt_{name}_t{nt}_s{len(g['opt_grads']) - 1}_"
    for key, arr in (("delta", host.delta), ("m1", host.m1), ("m2", host.m2), ("vhat", host.vhat),
                     ("prev_g", host.prev_g), ("steps", host.steps)):
        if q + key in g.files:
            assert arr is not None, key
            assert_close(arr, g[q + key], T, f"{name} {key}")
        else:
            assert arr is None, f"the reference allocates no {key} for {name}"


def test_regularization_mask_covers_exactly_the_weights(golden_optim):
    """8-6-6-3 network: 102 weights first, then biases and gamma / beta."""
    m = golden_optim["opt_gd_wd_mask"]
    assert m.size == 163 and m[:102].all() and not m[102:].any()
    assert golden_optim["opt_gd_plain_mask"].size == 0  # no weight decay: the reference allocates none


# ---- what the mathematics fixes ------------------------------------------------
def test_gd_closed_form(oracle64):
    rng = np.random.default_rng(1)
    p0, g = rng.standard_normal(50), rng.standard_normal(50)
    mask = (np.arange(50) < 30).astype(np.float64)
    p, gg = p0.copy(), g.copy()
    oracle64.opt_gd(p, gg, mask, 0.1, 0.0)
    np.testing.assert_allclose(p, p0 - 0.1 * g, rtol=1e-14)
    assert not gg.any()
    p, gg = p0.copy(), g.copy()
    oracle64.opt_gd(p, gg, mask, 0.1, 0.25)
    np.testing.assert_allclose(p, p0 - (0.1 * g + mask * 0.25 * p0), rtol=1e-14)
    np.testing.assert_allclose(p[30:], (p0 - 0.1 * g)[30:], rtol=1e-14)  # unmasked entries do not decay


def test_momentum_matches_torch_sgd(oracle64):
    """lr*g + mom*delta with constant lr is torch.optim.SGD's momentum buffer times lr."""
    rng = np.random.default_rng(2)
    p0 = rng.standard_normal(40)
    grads = rng.standard_normal((5, 40))
    tp = torch.tensor(p0.copy(), requires_grad=True)
    opt = torch.optim.SGD([tp], lr=0.05, momentum=0.9)
    p, delta = p0.copy(), np.zeros(40)
    for gr in grads:
        tp.grad = torch.tensor(gr.copy())
        opt.step()
        gg = gr.copy()
        oracle64.opt_gd_momentum(p, gg, delta, None, 0.05, 0.9, 0.0, False)
        np.testing.assert_allclose(p, tp.detach().numpy(), rtol=1e-12, atol=1e-14)


def test_nesterov_variant_closed_form(oracle64):
    """The reference moves the parameter by -(mom*delta - lr*g): two steps by hand."""
    p0, lr, mom = np.array([1.0, -2.0]), 0.1, 0.5
    g1, g2 = np.array([0.3, -0.7]), np.array([-1.1, 0.4])
    p, delta = p0.copy(), np.zeros(2)
    oracle64.opt_gd_momentum(p, g1.copy(), delta, None, lr, mom, 0.0, True)
    d1 = lr * g1
    e1 = p0 - (mom * d1 - lr * g1)
    np.testing.assert_allclose(p, e1, rtol=1e-14)
    oracle64.opt_gd_momentum(p, g2.copy(), delta, None, lr, mom, 0.0, True)
    d2 = lr * g2 + mom * d1
    np.testing.assert_allclose(delta, d2, rtol=1e-14)
    np.testing.assert_allclose(p, e1 - (mom * d2 - lr * g2), rtol=1e-14)


def test_adam_first_step_is_sign_of_gradient(oracle64):
    """With bias correction the first step is lr * g / (|g| + eps/sqrt(1-beta2)) ~ lr * sign(g)."""
    rng = np.random.default_rng(3)
    g = rng.standard_normal(64)
    p = np.zeros(64)
    host = OptimizerHost(oracle64, 64, OPT["ADAM"], adam_lr=0.01, eps=1e-8)
    host.m1, host.m2 = np.zeros(64), np.zeros(64)
    oracle64.opt_adam(p, g.copy(), host.m1, host.m2, None, None, 0.01 * np.sqrt(1 - 0.999) / (1 - 0.9), 0.9, 0.999,
                      1e-8, 0.0)
    np.testing.assert_allclose(p, -0.01 * g / (np.abs(g) + 1e-8 / np.sqrt(1 - 0.999)), rtol=1e-10)
    big = np.abs(g) > 0.1
    np.testing.assert_allclose(p[big], -0.01 * np.sign(g[big]), rtol=1e-5)
    np.testing.assert_allclose(host.m1, 0.1 * g, rtol=1e-12)
    np.testing.assert_allclose(host.m2, 0.001 * g * g, rtol=1e-12)


def test_adam_matches_torch_adam_when_eps_vanishes(oracle64):
    """torch puts eps next to sqrt(v_hat), the reference next to sqrt(v): identical as eps -> 0."""
    rng = np.random.default_rng(4)
    p0 = rng.standard_normal(30)
    grads = rng.standard_normal((6, 30)) + 0.1
    tp = torch.tensor(p0.copy(), requires_grad=True)
    opt = torch.optim.Adam([tp], lr=0.003, betas=(0.8, 0.95), eps=1e-30)
    p, m1, m2 = p0.copy(), np.zeros(30), np.zeros(30)
    for t, gr in enumerate(grads, 1):
        tp.grad = torch.tensor(gr.copy())
        opt.step()
        lr_t = 0.003 * np.sqrt(1 - 0.95 ** t) / (1 - 0.8 ** t)
        oracle64.opt_adam(p, gr.copy(), m1, m2, None, None, lr_t, 0.8, 0.95, 1e-30, 0.0)
        np.testing.assert_allclose(p, tp.detach().numpy(), rtol=1e-10)


def test_amsgrad_denominator_never_shrinks(oracle64):
    rng = np.random.default_rng(5)
    n = 20
    p, m1, m2, vh = np.zeros(n), np.zeros(n), np.zeros(n), np.zeros(n)
    prev = vh.copy()
    for scale in (3.0, 0.1, 2.0, 0.01):
        oracle64.opt_adam(p, scale * rng.standard_normal(n), m1, m2, vh, None, 0.01, 0.9, 0.5, 1e-8, 0.0)
        assert (vh >= prev).all() and (vh >= m2).all()
        prev = vh.copy()
    assert (vh > m2).any()  # after the small gradients the running maximum is what counts


def test_adabound_reduces_to_adam_and_to_sgd_on_the_first_moment(oracle64):
    """With a band wide enough never to bind, AdaBound is Adam; with a band of zero
    width at eta it is p -= eta * m1 (plain descent on the first moment), whatever the
    second moment says.  In between, the step size of each parameter is the clipped one."""
    rng = np.random.default_rng(6)
    n = 40
    p0, g = rng.standard_normal(n), rng.standard_normal(n) * np.exp(rng.uniform(-6, 2, n))
    pa, m1a, m2a = p0.copy(), np.zeros(n), np.zeros(n)
    oracle64.opt_adam(pa, g.copy(), m1a, m2a, None, None, 0.01, 0.9, 0.999, 1e-8, 0.0)
    pb, m1b, m2b = p0.copy(), np.zeros(n), np.zeros(n)
    oracle64.opt_adabound(pb, g.copy(), m1b, m2b, None, None, 0.01, 0.9, 0.999, 1e-8, 0.0, 0.0, 1e30)
    np.testing.assert_allclose(pb, pa, rtol=1e-14)
    pc, m1c, m2c = p0.copy(), np.zeros(n), np.zeros(n)
    oracle64.opt_adabound(pc, g.copy(), m1c, m2c, None, None, 0.01, 0.9, 0.999, 1e-8, 0.0, 0.07, 0.07)
    np.testing.assert_allclose(pc, p0 - 0.07 * 0.1 * g, rtol=1e-13)
    pd, m1d, m2d = p0.copy(), np.zeros(n), np.zeros(n)
    oracle64.opt_adabound(pd, g.copy(), m1d, m2d, None, None, 0.01, 0.9, 0.999, 1e-8, 0.0, 0.1, 2.0)
    rate = np.clip(0.01 / (np.sqrt(0.001 * g * g) + 1e-8), 0.1, 2.0)
    assert (rate == 0.1).any() and (rate == 2.0).any() and ((rate > 0.1) & (rate < 2.0)).any()
    np.testing.assert_allclose(pd, p0 - rate * 0.1 * g, rtol=1e-13)
    # AMSBound: the running maximum replaces the second moment
    vh = np.full(n, 4.0)
    pe, m1e, m2e = p0.copy(), np.zeros(n), np.zeros(n)
    oracle64.opt_adabound(pe, g.copy(), m1e, m2e, vh, None, 0.01, 0.9, 0.999, 1e-8, 0.0, 0.0, 1e30)
    assert (vh >= 4.0).all()
    np.testing.assert_allclose(pe, p0 - 0.01 / (np.sqrt(vh) + 1e-8) * 0.1 * g, rtol=1e-13)


def test_nosadam_weights_the_past_by_a_hyper_harmonic_series(oracle64):
    """NosAdam's second moment after t steps is sum_k k^-gamma g_k^2 / sum_k k^-gamma
    (Huang et al. 2019, eq. 5): the decay B_{t-1}/B_t telescopes to that."""
    rng = np.random.default_rng(8)
    n, steps, gamma = 12, 6, 0.1
    host = OptimizerHost(oracle64, n, OPT["NOSADAM"], adam_lr=0.001, adam_gamma=gamma)
    host.m1, host.m2 = np.zeros(n), np.zeros(n)
    p = np.zeros(n)
    gs = rng.standard_normal((steps, n))
    for gk in gs:
        host.update(p, gk.copy(), 1, 1)
    w = np.arange(1, steps + 1, dtype=np.float64) ** -gamma
    np.testing.assert_allclose(host.m2, (w[:, None] * gs * gs).sum(0) / w.sum(), rtol=1e-5)  # host scalars are float


def test_warm_restart_schedule_is_sgdr():
    """The rates handed to the leaf over 14 steps with a first period of 2 steps, multiplier 2 and a peak
    decaying by 0.5: eta_min + (eta_max - eta_min)(1 + cos(pi t / T)) / 2 (Loshchilov & Hutter 2017, eq. 5),
    the step that finds t == T taking the floor and restarting the clock, which the same call then advances
    to 1: the first period takes t = 0..2, the later ones t = 1..T (their peak itself is never visited)."""
    class Recorder:
        def __init__(self):
            self.rates = []

        def opt_gd(self, p, g, mask, lr, wd, nthreads=0):
            self.rates.append(float(lr))

    rec = Recorder()
    host = OptimizerHost(rec, 1, OPT["GD"], lr=0.05, momentum=0.0, warm_restarts=(0.5, 0.08, 0.001, 2.0, 2.0))
    p, g = np.zeros(1, np.float32), np.zeros(1, np.float32)
    for _ in range(14):
        host.update(p, g, 1, 1)
    expect, peak, period, first = [], 0.08, 2.0, 0
    while len(expect) < 14:
        for t in range(first, int(period) + 1):
            expect.append(0.001 + 0.5 * (peak - 0.001) * (1 + np.cos(np.pi * t / period)))
        peak, period, first = max(peak * 0.5, 0.001), period * 2, 1
    np.testing.assert_allclose(rec.rates, expect[:14], rtol=2e-6, atol=1e-9)
    assert rec.rates[0] == pytest.approx(0.08) and rec.rates[2] == pytest.approx(0.001)
    assert rec.rates[6] == pytest.approx(0.001) and rec.rates[7] == pytest.approx(0.001 + 0.5 * 0.019 * (1 + np.cos(np.pi / 8)))


def test_irprop_plus_by_hand(oracle64):
    """Four parameters through three calls, every branch, worked by hand (Igel & Hüsken 2000,
    iRPROP+): increase 1.2, decrease 0.5, step in [0.01, 0.13], start 0.1."""
    p = np.array([1.0, 1.0, 1.0, 1.0])
    prev_g, move, steps = np.zeros(4), np.zeros(4), np.full(4, 0.1)
    args = (1.2, 0.5, 0.01, 0.13)
    # call 1: no history -> plain step of the start size against the sign; zero gradient -> no move
    g = np.array([2.0, -3.0, 0.0, 5.0])
    oracle64.opt_irprop_plus(p, g, prev_g, move, steps, *args, False)
    np.testing.assert_allclose(p, [0.9, 1.1, 1.0, 0.9], rtol=1e-15)
    np.testing.assert_allclose(prev_g, [2.0, -3.0, 0.0, 5.0])
    assert not g.any()
    # call 2: same sign -> step 0.12; flipped sign with a worse loss -> last move taken back, step halved,
    # stored gradient cleared; zero history -> plain step; flipped sign again
    g = np.array([1.0, 4.0, -1.0, -2.0])
    oracle64.opt_irprop_plus(p, g, prev_g, move, steps, *args, True)
    np.testing.assert_allclose(p, [0.9 - 0.12, 1.0, 1.1, 1.0], rtol=1e-15)
    np.testing.assert_allclose(steps, [0.12, 0.05, 0.1, 0.05], rtol=1e-15)
    np.testing.assert_allclose(prev_g, [1.0, 0.0, -1.0, 0.0])
    # call 3: same sign -> 0.144 capped at 0.13; cleared history -> plain step of 0.05; same sign -> 0.12;
    # cleared history and a loss that did not get worse
    g = np.array([0.5, 4.0, -7.0, -2.0])
    oracle64.opt_irprop_plus(p, g, prev_g, move, steps, *args, False)
    np.testing.assert_allclose(p, [0.78 - 0.13, 1.0 - 0.05, 1.1 + 0.12, 1.0 + 0.05], rtol=1e-15)
    np.testing.assert_allclose(steps, [0.13, 0.05, 0.12, 0.05], rtol=1e-15)
    # a flip without a worse loss leaves the parameter where it is, and the lower limit binds
    steps[:] = 0.015
    prev_g[:] = 1.0
    before = p.copy()
    oracle64.opt_irprop_plus(p, np.full(4, -1.0), prev_g, move, steps, *args, False)
    assert np.array_equal(p, before) and np.allclose(steps, 0.01) and not prev_g.any()


def test_euclidean_norm_constraint_closed_form(oracle64, reference):
    """Above the threshold the array lands on the sphere of that radius, direction
    unchanged; below it nothing moves; row by row for the max-norm constraint.  The
    compiled reference's own helper agrees on the same arrays."""
    rng = np.random.default_rng(11)
    v = rng.standard_normal(1000)
    a = v.copy()
    oracle64.clip_gradient(a, 3.0)
    np.testing.assert_allclose(np.linalg.norm(a), 3.0, rtol=1e-12)
    np.testing.assert_allclose(a / np.linalg.norm(a), v / np.linalg.norm(v), rtol=1e-12)
    b = v.copy()
    oracle64.clip_gradient(b, 1e6)
    assert np.array_equal(b, v)
    W = rng.standard_normal((7, 50)) * rng.uniform(0.05, 2, (7, 1))
    Wc = W.copy()
    oracle64.max_norm_rows(Wc, 4.0)
    n0, n1 = np.linalg.norm(W, axis=1), np.linalg.norm(Wc, axis=1)
    assert (n0 > 4).any() and (n0 < 4).any()
    np.testing.assert_allclose(n1, np.minimum(n0, 4.0), rtol=1e-12)
    assert np.array_equal(Wc[n0 < 4], W[n0 < 4])
    for nt in (0, 3):
        r32 = v.astype(np.float32)
        reference.clip_gradient(r32, 3.0, nt)
        np.testing.assert_allclose(r32, a, rtol=2e-6)
        R = W.astype(np.float32)
        reference.max_norm_rows(R, 4.0, nt)
        np.testing.assert_allclose(R, Wc, rtol=2e-6)


def test_host_scalars(oracle):
    """Normalized weight decay wd*sqrt(B/(N*epochs)) (train.cpp:278-283) and the
    bias-corrected step size (adam.cpp:50-54), in float."""
    h = OptimizerHost(oracle, 4, OPT["ADAM"], adam_lr=0.001, weight_decay=0.04, normalized_wd=True)
    assert abs(float(h.wd(25, 100)) / (0.04 * 0.5) - 1) < 1e-6
    h.epoch_time_step = np.float32(4)
    assert abs(float(h.wd(25, 100)) / (0.04 * 0.25) - 1) < 1e-6
    h.t = np.float32(1)
    assert abs(float(h.lr_t()) / (0.001 * np.sqrt(1 - 0.999) / (1 - 0.9)) - 1) < 1e-5


# ---- against the compiled reference, fresh cases ----------------------------------
@pytest.mark.parametrize("seed", range(7))
def test_oracle_optimizer_against_reference(oracle, reference, seed):
    rng = np.random.default_rng(300 + seed)
    widths = [int(rng.integers(3, 12)) for _ in range(4)]
    nt = int(rng.integers(0, 4))
    kind = ["GD", "GD", "ADAM", "AMSGRAD", "ADABOUND", "AMSBOUND", "NOSADAM"][seed]
    kw = [dict(lr=0.03, momentum=0.0, weight_decay=0.1, normalized_wd=True),
          dict(lr=0.03, momentum=0.7, nesterov=bool(seed % 2), weight_decay=0.02, normalized_wd=False),
          dict(adam_lr=0.02, beta1=0.85, beta2=0.97, eps=1e-7, weight_decay=0.05),
          dict(adam_lr=0.02, bias_correction=False),
          dict(adam_lr=0.02, lr_final=0.04, gamma=0.4, weight_decay=0.05),
          dict(adam_lr=0.02, beta2=0.95, lr_final=0.03, gamma=0.2),
          dict(adam_lr=0.02, adam_gamma=0.05, weight_decay=0.01, normalized_wd=False)][seed]
    M = reference.mlp(widths)
    for l in (1, 2):
        M.set_layer(l, ACT["ELU"], NORM["BRN"])
    M.set_layer(3, ACT["SOFTMAX"])
    M.prepare(6, nt)
    p = rng.standard_normal(M.P).astype(np.float32)
    M.set_parameters(p)
    M.set_optimizer(OPT[kind], **kw)
    host = OptimizerHost(oracle, M.P, OPT[kind], mask=M.opt_state(4), **kw)
    for _ in range(5):
        g = rng.standard_normal(M.P).astype(np.float32)
        M.set_dparams(g)
        M.update_parameter(6, 48)
        host.update(p, g.copy(), 6, 48, nt)
        assert_close(p, M.get_parameters(), T, "parameters")
