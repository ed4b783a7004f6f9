"""LSUV on the device (Model::Initialize__LSUV / Initialization__LSUV, dlmi_layer_variance, dlmi_scale, partial
forward passes) against the oracle's loop, which tests/test_oracle_lsuv.py holds bit for bit to the reference's.
The device takes the variance sums in double in a fixed parallel order, the reference sequentially in float: the
variances agree to the float sum's own error (asserted below at 2e-5 relative), so do the scale factors, and the
trial counts are the same unless a variance sits within that error of the tolerance band's edge (the cases here
do not)."""
import numpy as np
import pytest

from oracle.binding import ACT, NORM, STATE
from test_oracle_lsuv import CASES, build, start_parameters

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib(pkg):
    return pkg.load_library()


def gpu_model(lib, widths, acts, norms):
    from deep_learning_amd.model import Model
    return build(lambda w: Model(lib, w), widths, acts, norms)


@pytest.mark.parametrize("widths,acts,norms", CASES)
@pytest.mark.parametrize("kw", [dict(), dict(max_n_trials=2, var_target=0.5, var_tolerance=0.001, bias=0.1, max_batch_size=20)])
def test_device_loop_against_the_oracle(lib, oracle, widths, acts, norms, kw):
    o = build(oracle.mlp, widths, acts, norms)
    g = gpu_model(lib, widths, acts, norms)
    try:
        p0 = start_parameters(o.P, widths, 5)
        o.parameters[:] = p0
        g.set_parameters(p0[:g.P])
        X = np.random.default_rng(1).normal(0, 1, (48, widths[0])).astype(np.float32)
        to = o.lsuv(X, **kw)
        tg = g.lsuv(X, pre_initialize=False, **kw)
        assert tg == to
        pg = g.get_parameters()
        nwb = sum(a * b + b for a, b in zip(widths[:-1], widths[1:]))
        off, worst = 0, []
        for l in range(1, len(widths)):
            n = widths[l] * widths[l - 1]
            a, b = pg[off:off + n].astype(np.float64), o.parameters[off:off + n].astype(np.float64)
            worst.append(float(np.max(np.abs(a - b) / np.abs(b))))
            off += n
        # every trial multiplies by a factor taken from a float variance; the reference's own float sums carry a
        # relative error of a few 1e-6 (more where E[y^2] - E[y]^2 cancels, as behind a sigmoid), which the
        # factors inherit and the trials compound
        for l in range(1, len(widths)):
            assert worst[l - 1] < 2e-5 * max(1, tg[l]), (worst, tg)
        assert np.array_equal(pg[off:nwb], o.parameters[off:nwb])  # the biases: initial_bias exactly
        assert np.array_equal(pg[nwb:], o.parameters[nwb:g.P])  # biases are in [:nwb]; scales 1, shifts 0 exactly
        if g.n_units:
            mg, mo = g.get_moving(), o.get_moving()
            assert np.array_equal(mg[0], mo[0]) and np.array_equal(mg[1], mo[1])
        assert np.all(g.get_dparams() == 0)
        # afterwards both see the same variances
        n = min(kw.get("max_batch_size", 32), 48)
        o.step(STATE["INFERENCE"], X[:n], None, backward=False)
        g.step(STATE["INFERENCE"], X[:n], None, backward=False)
        for l in range(1, len(widths)):
            assert g.layer_variance(l, n) == pytest.approx(o.layer_variance(l, n), rel=1e-4)
    finally:
        g.close()


def test_layer_variance_kernel(dl):
    """dlmi_layer_variance against numpy's float64 population variance; the same bits on every call; lengths
    that are not a multiple of anything."""
    import torch
    c = dl
    if True:
        for B, H, mu in [(1, 1, 0.0), (3, 7, 5.0), (32, 4096, 0.1), (1024, 4097, -2.0), (8192, 1024, 100.0)]:
            x = (torch.randn(B, H, device="cuda", generator=torch.Generator("cuda").manual_seed(B + H)) * 1.5 + mu).contiguous()
            got = [c.layer_variance(x) for _ in range(3)]
            assert got[0] == got[1] == got[2]
            want = float(x.double().var(unbiased=False).item()) if B * H > 1 else 0.0
            # the float result of var = E[x^2] - E[x]^2 taken in double: cancellation costs (mean^2 / var) ulps
            cond = 1.0 + mu * mu / max(want, 1e-30)
            assert got[0] == pytest.approx(want, rel=2e-7 * cond, abs=1e-12), (B, H)


def test_scale_kernel_is_a_float_multiply(dl):
    import torch
    c = dl
    if True:
        for n in (1, 5, 4096, 1000003):
            x = torch.randn(n + 3, device="cuda")
            ref = x.clone()
            f = np.float32(0.8371)
            c.scale(x, f, n)
            c.synchronize()
            assert torch.equal(x[:n], ref[:n] * float(f)) and torch.equal(x[n:], ref[n:])


def test_partial_forward_pass_stops_where_asked(lib):
    widths = [6, 20, 14, 9, 4]
    g = gpu_model(lib, widths, ["ELU", "TANH", "RELU", "LINEAR"], ["BRN", "NONE", "BRN"])
    try:
        g.glorot_uniform(3)
        X = np.random.default_rng(0).normal(0, 1, (16, 6)).astype(np.float32)
        X2 = np.random.default_rng(1).normal(0, 1, (16, 6)).astype(np.float32)
        g.step(STATE["INFERENCE"], X, None, backward=False)
        full = [g.layer_buffer(l, 3) for l in range(1, 5)]
        g.step(STATE["INFERENCE"], X2, None, backward=False)
        other = [g.layer_buffer(l, 3) for l in range(1, 5)]
        g.forward_to(STATE["INFERENCE"], X, 3)  # layers 1 and 2 only
        assert np.array_equal(g.layer_buffer(1, 3), full[0]) and np.array_equal(g.layer_buffer(2, 3), full[1])
        assert np.array_equal(g.layer_buffer(3, 3), other[2]) and np.array_equal(g.layer_buffer(4, 3), other[3])
        with pytest.raises(RuntimeError):
            g.forward_to(STATE["INFERENCE"], X, 1)   # no layer at all
        with pytest.raises(RuntimeError):
            g.forward_to(STATE["INFERENCE"], X, 6)   # past the output layer
        g.forward_to(STATE["INFERENCE"], X, 5)       # the whole network; an earlier refusal does not stick
        assert np.array_equal(g.layer_buffer(4, 3), full[3])
    finally:
        g.close()


def test_residual_network_layers_meet_the_target(lib):
    """Every fully-connected entry is scaled, inside blocks too; a RESIDUAL entry has no weights and is skipped.
    RELU blocks are positively homogeneous in each layer's weights: one scaling per layer."""
    from deep_learning_amd.model import Net
    layers = [("FC", 10), ("FC", 24), ("RES", 2), ("FC", 24), ("FC", 24), ("FC", 5)]
    g = Net(lib, layers)
    try:
        for l in g.fc_layers()[:-1]:
            g.set_layer(l, ACT["RELU"])
        g.set_layer(5, ACT["LINEAR"])
        g.prepare(32)
        g.init_uniform(2, 0.0, -0.3, 0.3)
        X = np.random.default_rng(5).normal(0, 1, (32, 10)).astype(np.float32)
        trials = g.lsuv(X, var_target=1.5, var_tolerance=1e-3, pre_initialize=False)
        assert trials[2] == 0 and all(trials[l] >= 1 for l in (1, 3, 4, 5)) and max(trials) <= 10
        for l in (1, 3, 4, 5):
            g.forward_to(STATE["INFERENCE"], X, l + 1)
            assert trials[l] == 10 or abs(g.layer_variance(l, 32) - 1.5) < 1e-3, (l, trials)
    finally:
        g.close()


def test_settings_are_checked(lib):
    g = gpu_model(lib, [4, 5, 3], ["TANH", "LINEAR"], ["NONE"])
    try:
        X = np.zeros((8, 4), np.float32)
        for bad in (dict(max_batch_size=0), dict(var_target=-1.0), dict(var_tolerance=-0.5)):
            with pytest.raises(RuntimeError):
                g.lsuv(X, pre_initialize=False, **bad)
        # all-zero inputs: every variance is 0, replaced by epsilon (lsuv.cpp:140), the loop still ends
        g.glorot_uniform(1)
        t = g.lsuv(X, max_n_trials=3, pre_initialize=False)
        assert max(t) <= 3 and np.all(np.isfinite(g.get_parameters()))
    finally:
        g.close()


def test_the_loop_alone_without_weights_is_refused(lib):
    """With pre_initialize=False the call scales the weights it finds.  On a model whose weights nobody has set it
    says so instead of scaling zeros."""
    g = gpu_model(lib, [12, 16, 4], ["RELU", "LINEAR"], ["NONE"])
    try:
        X = np.random.default_rng(2).normal(0, 1, (16, 12)).astype(np.float32)
        with pytest.raises(RuntimeError, match="no weights have been set"):
            g.lsuv(X, pre_initialize=False)
        g.glorot_uniform(3)
        g.lsuv(X, pre_initialize=False)  # an initializer has run: accepted
    finally:
        g.close()


def layer_weights(p, widths):
    off = 0
    for a, b in zip(widths[:-1], widths[1:]):
        yield a, b, p[off:off + a * b]
        off += a * b


def test_orthogonal_initializer(lib):
    """layers_initialize_orthogonal(false, bias): per layer, the weights as they lie are gain x a matrix with
    orthonormal columns - max(fan-in, units) x min(fan-in, units), row-major when fan-in >= units (the reference
    transposes in place), column-major otherwise; biases as given, scales 1, shifts 0, moving statistics 0 / 1,
    gradients cleared.  The draws continue from layer to layer and repeat for a seed.  (The factorization itself is
    held to LAPACK's in tests/test_orthogonal_weights.py.)"""
    widths, acts = [12, 16, 16, 8, 5], ["RELU", "TANH", "LEAKY_RELU", "LINEAR"]
    gains = [np.sqrt(2.0), 5.0 / 3.0, np.sqrt(2.0 / (1.0 + 0.01 ** 2)), 1.0]
    g = gpu_model(lib, widths, acts, ["BRN", "NONE", "BN"])
    h = gpu_model(lib, widths, acts, ["BRN", "NONE", "BN"])
    try:
        g.orthogonal(3, bias=0.25)
        p = g.get_parameters()
        nw = sum(a * b for a, b in zip(widths[:-1], widths[1:]))
        nb = sum(widths[1:])
        for (fan_in, units, w), gain in zip(layer_weights(p, widths), gains):
            hi, lo = max(fan_in, units), min(fan_in, units)
            W = (w.reshape(hi, lo) if fan_in >= units else w.reshape(lo, hi).T).astype(np.float64) / gain
            assert np.max(np.abs(W.T @ W - np.eye(lo))) < 1e-5, (fan_in, units)
        assert np.all(p[nw:nw + nb] == np.float32(0.25))
        nu = g.n_units
        assert np.all(p[nw + nb:nw + nb + nu] == 1.0) and np.all(p[nw + nb + nu:nw + nb + 2 * nu] == 0.0)
        mm, ms = g.get_moving()
        assert np.all(mm == 0.0) and np.all(ms == 1.0) and np.all(g.get_dparams() == 0)
        h.orthogonal(3, bias=0.25)
        assert np.array_equal(h.get_parameters(), p)
        h.orthogonal(4, bias=0.25)
        assert not np.array_equal(h.get_parameters()[:nw], p[:nw])
        # the second layer's draws follow the first's: a model that starts at the second layer's shape with the
        # same seed holds other weights there
        k = gpu_model(lib, widths[1:], acts[1:], ["NONE", "BN"])
        try:
            k.orthogonal(3, bias=0.25)
            assert not np.array_equal(k.get_parameters()[:16 * 16], p[12 * 16:12 * 16 + 16 * 16])
        finally:
            k.close()
    finally:
        g.close()
        h.close()


def test_lsuv_starts_from_the_orthogonal_initializer(lib):
    """Initialization__LSUV as the reference runs it (lsuv.cpp:55): on a model whose weights nobody has set, the
    orthogonal initializer first, then the scaling loop - the same bits as the two steps taken by hand - and every
    layer's output variance ends within the tolerance of the target."""
    widths, acts = [20, 32, 24, 6], ["RELU", "TANH", "LINEAR"]
    a = gpu_model(lib, widths, acts, ["NONE", "NONE"])
    b = gpu_model(lib, widths, acts, ["NONE", "NONE"])
    try:
        X = np.random.default_rng(8).normal(0, 1, (40, 20)).astype(np.float32)
        a.seed_gaussian(7)
        ta = a.lsuv(X, bias=0.05, var_tolerance=1e-3)
        b.orthogonal(7, bias=0.05)
        tb = b.lsuv(X, bias=0.05, var_tolerance=1e-3, pre_initialize=False)
        assert ta == tb and max(ta) <= 10
        assert np.array_equal(a.get_parameters(), b.get_parameters())
        for l in range(1, len(widths)):
            a.forward_to(STATE["INFERENCE"], X[:32], l + 1)
            assert ta[l] == 10 or abs(a.layer_variance(l, 32) - 1.0) < 1e-3, (l, ta)
    finally:
        a.close()
        b.close()


def test_gaussian_draws_are_the_references(lib, reference):
    """The N(0, 1) draws the orthogonal initializer starts from, against the compiled reference's own
    gaussian.seed(seed) + weights_initialize_gaussian (model.cpp:5401-5409), bit for bit: an odd count first, so
    that the distribution's spare value crosses from one call into the next, as it does from layer to layer."""
    g = gpu_model(lib, [6, 5, 3], ["TANH", "LINEAR"], ["NONE"])
    r = build(reference.mlp, [6, 5, 3], ["TANH", "LINEAR"], ["NONE"])
    try:
        g.seed_gaussian(123)
        a = np.concatenate([g.gaussian_draws(7), g.gaussian_draws(30)])
        b = r.gaussian_draws(123, 37)
        assert np.array_equal(a, b)
        assert abs(float(a.mean())) < 0.6 and 0.5 < float(a.std()) < 1.6
    finally:
        g.close()
