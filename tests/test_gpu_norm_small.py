"""The small-batch normalization kernels (at most 256 rows and 2^20 elements: one launch per direction, a
workgroup owns 8 columns for all rows) against the multi-launch kernels of the same library and against
float64 closed forms.  Same per-unit arithmetic, other summation order: the two paths agree to rounding of
the column sums, not bit for bit.  A context created with DLMI_NORM_SMALL=0 never takes the small-batch
kernels; that is the twin here."""
import os

import numpy as np
import pytest
import torch

from helpers import assert_close
from oracle.binding import ACT, DROP
from test_gpu_norm_panel import dev, make, run_bwd, run_fwd

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def twins(pkg):
    os.environ["DLMI_NORM_SMALL"] = "0"
    try:
        plain = pkg.Dlmi(0)
    finally:
        del os.environ["DLMI_NORM_SMALL"]
    small = pkg.Dlmi(0)
    yield small, plain
    small.close()
    plain.close()


CASES = [  # B, H, act, dropout, per element, shortcut
    (128, 512, "RELU", "NONE", False, False),                  # the reference's own mini-batch
    (128, 512, "ELU", "BERNOULLI_INVERTED", True, True),
    (37, 10, "SELU", "BERNOULLI", False, False),               # ragged: 2 workgroups, the second half empty
    (1, 8, "LEAKY_RELU", "NONE", False, False),                # one row: variance 0 + epsilon
    (200, 36, "ISRLU", "BERNOULLI_INVERTED", False, True),
    (256, 4096, "TANH", "NONE", False, False),                 # the largest shape the kernels take
    (255, 1001, "SIGMOID", "BERNOULLI", True, False),
    (33, 7, "LINEAR", "NONE", False, False),
]


@pytest.mark.parametrize("B,H,act,drop,per_element,shortcut", CASES)
def test_forward_small_equals_multi_launch_to_rounding(twins, pkg, B, H, act, drop, per_element, shortcut):
    small, plain = twins
    d = make(B, H, B + H)
    a, *_ = run_fwd(small, pkg, d, act, drop, per_element, shortcut)
    b, *_ = run_fwd(plain, pkg, d, act, drop, per_element, shortcut)
    for k in ("mean", "std", "mov_mean", "mov_std", "r"):
        assert_close(a[k], b[k], 2e-6, f"{k} [{B}x{H}]", floor=1e-3 if B == 1 else 0.0)
    assert_close(a["d"], b["d"], 1e-5, f"d [{B}x{H}]", floor=1.0)   # a shift in units of sigma: a difference of means
    assert_close(a["y"], b["y"], 1e-5, f"y [{B}x{H}]", floor=1.0)


@pytest.mark.parametrize("B,H,act,drop,per_element,shortcut", CASES)
def test_backward_small_equals_multi_launch_to_rounding(twins, pkg, B, H, act, drop, per_element, shortcut):
    small, plain = twins
    d = make(B, H, B + H + 1)
    _, desc, mask, st = run_fwd(plain, pkg, d, act, drop, per_element, False)  # both start from the same forward
    a = run_bwd(small, pkg, d, desc, mask, st)
    b = run_bwd(plain, pkg, d, desc, mask, st)
    assert_close(a["dx"], b["dx"], 1e-4, f"dX [{B}x{H}]", floor=1.0)
    assert_close(a["dgamma"], b["dgamma"], 1e-4, "dgamma", floor=1.0)
    assert_close(a["dbeta"], b["dbeta"], 1e-4, "dbeta", floor=1.0)


def test_small_against_float64(twins, pkg):
    """128 x 512, batch renormalization + ELU, forward and backward from the closed forms in float64."""
    small, _ = twins
    B, H = 128, 512
    d = make(B, H, 15)
    a, desc, mask, st = run_fwd(small, pkg, d, "ELU", "NONE", False, False)
    x = d["x"].astype(np.float64)
    mean = x.mean(0)
    std = np.sqrt((x * x).mean(0) - mean * mean + 1e-5)
    mm = d["mm"] + 0.9 * (mean - d["mm"])
    ms = d["ms"] + 0.9 * (std - d["ms"])
    r = np.clip(std / ms, 1 / 3.0, 3.0)
    dd = np.clip((mean - mm) / ms, -5.0, 5.0)
    xh = (x - mean) / std * r + dd
    n = d["gamma"] * xh + d["beta"]
    assert_close(a["mean"], mean, 2e-6, "mean")
    assert_close(a["std"], std, 2e-6, "std")
    assert_close(a["mov_mean"], mm, 2e-6, "moving mean")
    assert_close(a["mov_std"], ms, 2e-6, "moving std")
    assert_close(a["r"], r, 2e-6, "r")
    assert_close(a["d"], dd, 1e-5, "d", floor=1.0)
    assert_close(a["y"], np.where(n > 0, n, np.expm1(n)), 1e-5, "y", floor=1.0)
    keep = np.abs(n) > 1e-4   # the derivative of ELU jumps at 0
    dy = d["dy"].astype(np.float64) * keep
    g = run_bwd(small, pkg, dict(d, dy=dy.astype(np.float32)), desc, mask, st)
    # the reference's ELU derivative for n < 0 is the activation value itself (functions.hpp:92)
    dn = dy * np.where(n > 0, 1.0, np.expm1(n))
    e = dn * d["gamma"]
    dmean = (e * (-r / std)).sum(0)
    dstd = (e * (x - mean) * (-r / std ** 2)).sum(0)
    dx = e * (r / std) + dstd * (x - mean) / (B * std) + dmean / B
    assert_close(g["dx"], dx, 1e-4, "dX", floor=1.0)
    assert_close(g["dgamma"], 0.25 + (dn * xh).sum(0), 1e-4, "dgamma", floor=1.0)
    assert_close(g["dbeta"], -0.5 + dn.sum(0), 1e-4, "dbeta", floor=1.0)


def test_small_is_reproducible(twins, pkg):
    small, _ = twins
    d = make(100, 300, 3)
    first, desc, mask, st = run_fwd(small, pkg, d, "SELU", "NONE", False, False)
    g0 = run_bwd(small, pkg, d, desc, mask, st)
    for _ in range(3):
        again, desc, mask, st2 = run_fwd(small, pkg, d, "SELU", "NONE", False, False)
        for k in first:
            assert np.array_equal(first[k], again[k]), k
        g = run_bwd(small, pkg, d, desc, mask, st2)
        for k in g0:
            assert np.array_equal(g0[k], g[k]), k


@pytest.mark.parametrize("B,K,H", [(128, 784, 512), (128, 512, 512), (64, 100, 24), (256, 2048, 128), (130, 33, 70)])
def test_fc_forward_whose_k_slices_the_small_kernel_adds(twins, pkg, B, K, H):
    """dlmi_fc_norm_act_fwd on a mini-batch: a product that runs split over K leaves its slices to the
    normalization kernel, which adds them in slice order, stores Z and carries on.  Against the twin (GEMM +
    its own slice reduction + multi-launch normalization): Z bit-identical where both split the same way
    (same slices, same order), everything else to rounding; and Z against float64."""
    small, plain = twins
    rng = np.random.default_rng(B + K + H)
    X = rng.standard_normal((B, K)).astype(np.float32)
    W = (rng.standard_normal((H, K)) / np.sqrt(K)).astype(np.float32)
    d = make(B, H, 77)
    desc = pkg.Dlmi.desc(ACT["RELU"], renorm=True, momentum=0.9, eps=1e-5, r_max=3.0, d_max=5.0)
    res = []
    for dl in (small, plain):
        mm, ms = dev(d["mm"]), dev(d["ms"])
        Z, y, st = dl.fc_norm_act_fwd(desc, dev(X), dev(W), dev(d["gamma"]), dev(d["beta"]), mm, ms)
        dl.synchronize()
        out = {k: v.cpu().numpy() for k, v in st.items()}
        out.update(Z=Z.cpu().numpy(), y=y.cpu().numpy(), mov_mean=mm.cpu().numpy(), mov_std=ms.cpu().numpy())
        res.append(out)
    a, b = res
    assert np.array_equal(a["Z"], b["Z"]), "same slices added in the same order"
    assert_close(a["Z"], X.astype(np.float64) @ W.astype(np.float64).T, 1e-4, "Z")
    for k in ("mean", "std", "mov_mean", "mov_std", "r"):
        assert_close(a[k], b[k], 2e-6, k, floor=1e-3)
    assert_close(a["d"], b["d"], 1e-5, "d", floor=1.0)
    assert_close(a["y"], b["y"], 1e-5, "y", floor=1.0)


@pytest.mark.parametrize("B,H", [(128, 10), (256, 513), (5, 3)])
def test_bias_gradient_of_a_mini_batch(twins, pkg, B, H):
    small, plain = twins
    rng = np.random.default_rng(B * H)
    dZ = rng.standard_normal((B, H)).astype(np.float32)
    Xin = rng.standard_normal((B, 16)).astype(np.float32)
    out = []
    for dl in (small, plain):
        dW, db = dl.fc_bwd_dw(dev(Xin), dev(dZ), with_bias=True)
        db0 = db.cpu().numpy()
        dl.fc_bwd_dw(dev(Xin), dev(dZ), dW=dW, db=db, accumulate=True)   # accumulates on top
        out.append((db0, db.cpu().numpy()))
    exact = dZ.astype(np.float64).sum(0)
    for db0, db1 in out:
        assert_close(db0, exact, 1e-5, "db", floor=1.0)
        assert_close(db1, 2 * exact, 1e-5, "db accumulated", floor=1.0)
    assert_close(out[0][0], out[1][0], 1e-5, "db small vs multi-launch", floor=1.0)
