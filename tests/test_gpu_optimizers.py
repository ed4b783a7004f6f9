"""dlmi_opt_* through the C ABI: against the golden vectors of the compiled
reference (tests/golden/optim.npz), and against the oracle on larger, ragged
and unaligned arrays."""
import numpy as np
import pytest
import torch

from helpers import RTOL_ELEMENTWISE as TE
from helpers import assert_close
from oracle.binding import OPT, OptimizerHost
from test_oracle_optimizers import leaf_case_names, run_leaf_case

pytestmark = pytest.mark.gpu


class GpuLeaves:
    """opt_gd / opt_gd_momentum / opt_adam on numpy arrays, in place, computed on
    the GPU: every array goes to the device, through the C ABI and back."""

    def __init__(self, dl):
        self.dl = dl

    def _run(self, fn, arrays, *scalars):
        dev = [None if a is None else torch.from_numpy(a).cuda() for a in arrays]
        fn(*dev, *scalars)
        torch.cuda.synchronize()
        for a, d in zip(arrays, dev):
            if a is not None:
                a[...] = d.cpu().numpy()

    def opt_gd(self, p, g, mask, lr, wd, nthreads=0):
        self._run(self.dl.opt_gd, [p, g, mask], float(lr), float(wd))

    def opt_gd_momentum(self, p, g, delta, mask, lr, mom, wd, nesterov, nthreads=0):
        self._run(self.dl.opt_gd_momentum, [p, g, delta, mask], float(lr), float(mom), float(wd), nesterov)

    def opt_adam(self, p, g, m1, m2, vhat, mask, lr_t, b1, b2, eps, wd, nthreads=0):
        self._run(self.dl.opt_adam, [p, g, m1, m2, vhat, mask], float(lr_t), float(b1), float(b2), float(eps),
                  float(wd))

    def opt_irprop_plus(self, p, g, prev_g, prev_move, steps, incr, decr, step_min, step_max, worse, nthreads=0):
        self._run(self.dl.opt_irprop_plus, [p, g, prev_g, prev_move, steps], float(incr), float(decr), float(step_min),
                  float(step_max), bool(worse))

    def clip_gradient(self, g, max_norm, nthreads=0):
        self._run(self.dl.clip_gradient, [g], float(max_norm))

    def max_norm_rows(self, W, max_norm, nthreads=0):
        self._run(self.dl.max_norm_rows, [W], float(max_norm))

    def opt_adabound(self, p, g, m1, m2, vhat, mask, lr_t, b1, b2, eps, wd, lower, upper, nthreads=0):
        self._run(self.dl.opt_adabound, [p, g, m1, m2, vhat, mask], float(lr_t), float(b1), float(b2), float(eps),
                  float(wd), float(lower), float(upper))


@pytest.fixture(scope="module")
def golden_optim():
    import os
    from conftest import ROOT
    return np.load(os.path.join(ROOT, "tests", "golden", "optim.npz"), allow_pickle=False)


@pytest.mark.parametrize("name", leaf_case_names())
def test_gpu_optimizer_against_golden(dl, golden_optim, name):
    g = golden_optim
    for t, p, host in run_leaf_case(GpuLeaves(dl), g, name, 0):
        assert_close(p, g[f"opt_{name}_t0_s{t}_params"], TE, f"{name} parameters after step {t}")
    q = f"opt_{name}_t0_s{len(g['opt_grads']) - 1}_"
    for key, arr in (("delta", host.delta), ("m1", host.m1), ("m2", host.m2), ("vhat", host.vhat),
                     ("prev_g", host.prev_g), ("steps", host.steps)):
        if q + key in g.files:
            assert_close(arr, g[q + key], TE, f"{name} {key}")


@pytest.mark.parametrize("n", [1, 3, 4, 1000, 4099, 1 << 20])
@pytest.mark.parametrize("kind,kw", [
    ("GD", dict(lr=0.05, momentum=0.0, weight_decay=0.1, normalized_wd=False)),
    ("GD", dict(lr=0.05, momentum=0.9)),
    ("GD", dict(lr=0.05, momentum=0.9, nesterov=True, weight_decay=0.1, normalized_wd=True)),
    ("ADAM", dict(adam_lr=0.01, weight_decay=0.05)),
    ("AMSGRAD", dict(adam_lr=0.01, beta2=0.9)),
    ("ADABOUND", dict(adam_lr=0.01, lr_final=0.05, gamma=0.5, weight_decay=0.05)),
    ("AMSBOUND", dict(adam_lr=0.01, beta2=0.9, lr_final=0.02, gamma=0.3)),
    ("NOSADAM", dict(adam_lr=0.01, adam_gamma=0.1, weight_decay=0.02, normalized_wd=False)),
    ("IRPROP_PLUS", dict(rprop=[1.5, 0.4, 0.01, 0.3, 0.1], rprop_losses=[[2.0, 1.0], [1.0, 2.0], [3.0, 1.0]])),
])
def test_gpu_optimizer_against_oracle(dl, oracle, n, kind, kw):
    rng = np.random.default_rng(n + len(kind))
    p0 = rng.standard_normal(n).astype(np.float32)
    mask = (rng.uniform(size=n) < 0.7).astype(np.float32)
    ho = OptimizerHost(oracle, n, OPT[kind], mask=mask, **kw)
    hg = OptimizerHost(GpuLeaves(dl), n, OPT[kind], mask=mask, **kw)
    po, pg = p0.copy(), p0.copy()
    for _ in range(3):
        g = rng.standard_normal(n).astype(np.float32)
        go, gg = g.copy(), g.copy()
        ho.update(po, go, 32, 4096)
        hg.update(pg, gg, 32, 4096)
        assert not gg.any(), "gradient zeroed"
        assert_close(pg, po, TE, "parameters")
    for a, b, what in ((hg.delta, ho.delta, "delta"), (hg.m1, ho.m1, "m1"), (hg.m2, ho.m2, "m2"),
                       (hg.vhat, ho.vhat, "vhat")):
        if b is not None:
            assert_close(a, b, TE, what)


@pytest.mark.parametrize("n", [1, 5, 4099, 1 << 22])
def test_gpu_clip_gradient_against_oracle(dl, oracle64, n):
    """float64 arbitrates: over four million terms the oracle's own float sum drifts."""
    rng = np.random.default_rng(n)
    g = rng.standard_normal(n).astype(np.float32)
    norm = float(np.linalg.norm(g.astype(np.float64)))
    for c in (0.5 * norm, 2.0 * norm):
        exp = g.astype(np.float64)
        oracle64.clip_gradient(exp, c)
        t = torch.from_numpy(g.copy()).cuda()
        dl.clip_gradient(t, c)
        assert_close(t.cpu().numpy(), exp, TE, f"clip at {c:.3g}")
        if c > norm:
            assert np.array_equal(t.cpu().numpy(), g), "below the threshold nothing is rewritten"
    # a range that does not start on a 16-byte boundary
    if n > 1:
        t = torch.from_numpy(g.copy()).cuda()
        exp = g[1:].astype(np.float64)
        oracle64.clip_gradient(exp, 0.25 * norm)
        dl.clip_gradient(t[1:], 0.25 * norm)
        assert_close(t[1:].cpu().numpy(), exp, TE, "unaligned view")
        assert float(t[0]) == float(g[0])


@pytest.mark.parametrize("rows,cols", [(1, 1), (7, 50), (512, 784), (10, 4097), (3000, 33)])
def test_gpu_max_norm_rows_against_oracle(dl, oracle64, rows, cols):
    rng = np.random.default_rng(rows * 31 + cols)
    W = (rng.standard_normal((rows, cols)) * rng.uniform(0.05, 2, (rows, 1))).astype(np.float32)
    c = float(np.median(np.linalg.norm(W.astype(np.float64), axis=1))) * 1.001
    exp = W.astype(np.float64)
    oracle64.max_norm_rows(exp, c)
    t = torch.from_numpy(W.copy()).cuda()
    dl.max_norm_rows(t, c)
    got = t.cpu().numpy()
    assert_close(got, exp, TE, "rows")
    untouched = np.linalg.norm(W.astype(np.float64), axis=1) < c * 0.999
    assert np.array_equal(got[untouched], W[untouched])


def test_gpu_optimizer_on_unaligned_views(dl, oracle):
    """A parameter range that does not start on a 16-byte boundary (str/end of the
    reference's Update_Parameters__*(…, str, end)) takes the scalar path."""
    n = 1001
    rng = np.random.default_rng(9)
    base = [torch.from_numpy(rng.standard_normal(n + 1).astype(np.float32)).cuda() for _ in range(4)]
    first = [float(b[0]) for b in base]
    p, g, m1, m2 = (b[1:] for b in base)
    po, go, m1o, m2o = (t.cpu().numpy().copy() for t in (p, g, m1, m2))
    m1o, m2o = np.abs(m1o), np.abs(m2o)
    m1.copy_(torch.from_numpy(m1o)); m2.copy_(torch.from_numpy(m2o))
    dl.opt_adam(p, g, m1, m2, None, None, 0.01, 0.9, 0.999, 1e-8, 0.0)
    oracle.opt_adam(po, go, m1o, m2o, None, None, 0.01, 0.9, 0.999, 1e-8, 0.0)
    assert_close(p.cpu().numpy(), po, TE, "parameters")
    assert_close(m2.cpu().numpy(), m2o, TE, "m2")
    assert not g.cpu().numpy().any()
    assert first == [float(b[0]) for b in base], "the element before the range is untouched"


def test_weight_decay_without_mask_is_refused(dl):
    p = torch.zeros(8, device="cuda")
    with pytest.raises(RuntimeError):
        dl.opt_gd(p, p.clone(), None, 0.1, 0.5)
