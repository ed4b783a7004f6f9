"""Pins the CPU restatement with what the mathematics fixes, independently of
any run of the reference: brute force in float64, closed forms, invariants,
finite differences and library routines (torch.nn.functional)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import assert_close
from oracle.binding import ACT


def rnd(seed, *shape):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


# ---------------------------------------------------------------- GEMMs (a7, a18, a23)
@pytest.mark.parametrize("B,K,H", [(1, 1, 1), (3, 7, 5), (17, 33, 9), (8, 64, 64)])
@pytest.mark.parametrize("nt", [0, 4])
def test_gemms_brute_force_and_adjoint(oracle, B, K, H, nt):
    X, W, dZ = rnd(1, B, K), rnd(2, H, K), rnd(3, B, H)
    X64, W64, dZ64 = X.astype(np.float64), W.astype(np.float64), dZ.astype(np.float64)
    Z = oracle.fc_fwd(X, W, nt)
    assert_close(Z, np.einsum("bk,hk->bh", X64, W64), 2e-6, "Z = X W^T")
    dX = oracle.fc_bwd_dx(dZ, W, nthreads=nt)
    assert_close(dX, np.einsum("bh,hk->bk", dZ64, W64), 2e-6, "dX = dZ W")
    dW, db = oracle.fc_bwd_dw(X, dZ, nthreads=nt)
    assert_close(dW, np.einsum("bh,bk->hk", dZ64, X64), 2e-6, "dW = dZ^T X")
    assert_close(db, dZ64.sum(0), 2e-6, "db = sum_b dZ")
    # <dZ, X W^T> = <dZ W, X> = <dZ^T X, W>: a transposed operand breaks one of them
    a = float(np.sum(dZ64 * Z)); b = float(np.sum(dX.astype(np.float64) * X64)); c = float(np.sum(dW.astype(np.float64) * W64))
    s = np.sqrt(B * K * H)
    assert abs(a - b) <= 1e-5 * s and abs(a - c) <= 1e-5 * s


def test_gemm_identity_and_accumulation(oracle):
    X = rnd(4, 6, 5)
    assert np.array_equal(oracle.fc_fwd(X, np.eye(5, dtype=np.float32)), X)
    # dX accumulates into what is already there; dW too
    base = rnd(5, 6, 5)
    dZ, W = rnd(6, 6, 3), rnd(7, 3, 5)
    assert_close(oracle.fc_bwd_dx(dZ, W, dY_init=base), base + oracle.fc_bwd_dx(dZ, W), 1e-6, "dX +=")
    dW0 = rnd(8, 3, 5)
    assert_close(oracle.fc_bwd_dw(X, dZ, dW_init=dW0)[0], dW0 + oracle.fc_bwd_dw(X, dZ)[0], 1e-6, "dW +=")


# ---------------------------------------------------------------- BN / BRN forward (a9-a11)
def brn_closed_form(x, gamma, beta, mm, ms, m, eps, rmax, dmax, renorm=True):
    x = x.astype(np.float64)
    mu = x.mean(0)
    sd = np.sqrt((x * x).mean(0) - mu * mu + eps)
    mm2 = mm + m * (mu - mm)
    ms2 = ms + m * (sd - ms)
    r = np.clip(sd / ms2, 1 / rmax, rmax) if renorm else np.ones_like(mu)
    d = np.clip((mu - mm2) / ms2, -dmax, dmax) if renorm else np.zeros_like(mu)
    xhat = (x - mu) / sd * r + d
    return dict(mean=mu, std=sd, mov_mean=mm2, mov_std=ms2, r=r, d=d, xhat=xhat, out=gamma * xhat + beta)


@pytest.mark.parametrize("B,H", [(2, 1), (16, 7), (64, 33)])
@pytest.mark.parametrize("nt", [0, 5])
@pytest.mark.parametrize("hyper", [(0.99, 3.0, 5.0), (0.01, 1.05, 0.02), (1.0, 2.0, 1.0)])
def test_brn_forward_closed_form(oracle, B, H, nt, hyper):
    m, rmax, dmax = hyper
    rng = np.random.default_rng(B * 100 + H)
    x = (rng.standard_normal((B, H)) * rng.uniform(0.5, 2, H) + rng.uniform(-1, 1, H)).astype(np.float32)
    gamma = rng.uniform(0.8, 1.2, H).astype(np.float32); beta = rng.uniform(-.1, .1, H).astype(np.float32)
    mm = rng.uniform(-1, 1, H).astype(np.float32); ms = rng.uniform(0.5, 2, H).astype(np.float32)
    got = oracle.norm_fwd_train(x, gamma, beta, mm, ms, m, 1e-5, rmax, dmax, True, nt)
    exp = brn_closed_form(x, gamma, beta, mm, ms, m, 1e-5, rmax, dmax)
    for k in exp:
        assert_close(got[k], exp[k], 2e-5, k, floor=1.0 if k == "d" else 0.0)
    # "variance" outputs are standard deviations, updated before r and d are formed
    if m == 1.0:  # then the moving stats equal the batch stats: r = 1, d = 0 -> plain BN
        assert np.max(np.abs(got["r"] - 1.0)) < 1e-6 and np.max(np.abs(got["d"])) < 1e-6
        t = F.batch_norm(torch.from_numpy(x), None, None, torch.from_numpy(gamma), torch.from_numpy(beta),
                         training=True, eps=1e-5).numpy()
        assert_close(got["out"], t, 2e-5, "torch batch_norm")


def test_bn_is_brn_with_r1_d0_and_invariants(oracle):
    rng = np.random.default_rng(11)
    B, H = 40, 9
    x = (rng.standard_normal((B, H)) * 3 + 1).astype(np.float32)
    one, zero = np.ones(H, np.float32), np.zeros(H, np.float32)
    bn = oracle.norm_fwd_train(x, one, zero, zero, one, 0.5, 1e-5, renorm=False)
    brn = oracle.norm_fwd_train(x, one, zero, zero, one, 0.5, 1e-5, r_max=1.0, d_max=0.0, renorm=True)
    assert_close(bn["xhat"], brn["xhat"], 1e-6, "BN == BRN(r_max=1, d_max=0)")
    xh = bn["xhat"].astype(np.float64)
    assert np.max(np.abs(xh.mean(0))) < 1e-6                       # column mean 0
    sd = bn["std"].astype(np.float64)
    assert_close((xh * xh).mean(0), 1 - 1e-5 / sd ** 2, 1e-5, "mean square = 1 - eps/sigma^2")
    # a constant column has sigma = sqrt(eps) (B = 32: every sum and 1/B is exact in fp32,
    # so E[x^2] - mu^2 cancels exactly; for other B the fp32 cancellation error dominates eps)
    c = np.full((32, 3), 2.5, np.float32)
    cs = oracle.norm_fwd_train(c, one[:3], zero[:3], zero[:3], one[:3], 0.5, 1e-5, renorm=False)
    assert_close(cs["std"], np.full(3, np.sqrt(1e-5)), 1e-6, "sigma of a constant column")


def test_bn_inference_uses_moving_std_without_eps(oracle):
    rng = np.random.default_rng(12)
    x = rng.standard_normal((9, 4)).astype(np.float32)
    g = rng.uniform(.8, 1.2, 4).astype(np.float32); b = rng.uniform(-.1, .1, 4).astype(np.float32)
    mm = rng.uniform(-1, 1, 4).astype(np.float32); ms = rng.uniform(.5, 2, 4).astype(np.float32)
    exp = g.astype(np.float64) * ((x.astype(np.float64) - mm) / ms) + b
    assert_close(oracle.norm_fwd_infer(x, g, b, mm, ms), exp, 2e-6, "inference")


# ---------------------------------------------------------------- activations (a12, a19)
def test_activation_forward_library_and_closed_forms(oracle):
    x = np.concatenate([rnd(20, 1, 200) * 3, np.array([[0.0, -0.0, 1e-6, -1e-6, 30.0, -30.0]], np.float32)], 1)
    t = torch.from_numpy(x)
    assert np.array_equal(oracle.act_fwd(ACT["RELU"], x), F.relu(t).numpy())
    assert_close(oracle.act_fwd(ACT["LEAKY_RELU"], x), F.leaky_relu(t, 0.01).numpy(), 1e-6, "lrelu")
    x64 = x.astype(np.float64)
    assert_close(oracle.act_fwd(ACT["ELU"], x), np.where(x64 < 0, np.exp(x64) - 1, x64), 2e-6, "elu")
    a, s = 1.6732632423543772, 1.0507009873554805
    assert_close(oracle.act_fwd(ACT["SELU"], x), s * np.where(x64 <= 0, a * np.exp(x64) - a, x64), 2e-6, "selu")
    assert_close(oracle.act_fwd(ACT["SELU"], x), F.selu(t).numpy(), 2e-6, "selu torch")
    assert_close(oracle.act_fwd(ACT["ISRLU"], x), np.where(x64 < 0, x64 / np.sqrt(1 + x64 * x64), x64), 2e-6, "isrlu")
    assert np.array_equal(oracle.act_fwd(ACT["LINEAR"], x), x)


def test_activation_derivatives_reference_quirks(oracle):
    """The derivative the backward pass uses is a function of (pre, post):
    ELU' = post for x<0 (i.e. exp(x)-1, not exp(x)), SELU' = scale*(post+alpha)
    for x<=0 (not post + scale*alpha), ISRLU' = (post/pre)^3.  ReLU / leaky
    ReLU / ISRLU coincide with the textbook derivative (finite differences)."""
    x = (rnd(21, 1, 300) * 2).astype(np.float32)
    x = x[np.abs(x) > 1e-2].reshape(1, -1)
    one = np.ones_like(x)
    x64 = x.astype(np.float64)
    a, s = 1.6732632423543772, 1.0507009873554805

    def deriv(name):
        return oracle.act_bwd(ACT[name], x, oracle.act_fwd(ACT[name], x), one)

    assert_close(deriv("ELU"), np.where(x64 < 0, np.exp(x64) - 1, 1.0), 2e-6, "elu'")
    assert_close(deriv("SELU"), s * np.where(x64 <= 0, s * (a * np.exp(x64) - a) + a, 1.0), 2e-6, "selu'")
    assert np.array_equal(deriv("RELU"), (x >= 0).astype(np.float32))
    assert_close(deriv("LEAKY_RELU"), np.where(x64 < 0, 0.01, 1.0), 1e-6, "lrelu'")
    assert np.array_equal(deriv("LINEAR"), one)
    f = lambda v: np.where(v < 0, v / np.sqrt(1 + v * v), v)
    h = 1e-6
    assert_close(deriv("ISRLU"), (f(x64 + h) - f(x64 - h)) / (2 * h), 1e-4, "isrlu' finite difference")
    # dN = dY * f': linear in dY
    dY = rnd(22, *x.shape)
    y = oracle.act_fwd(ACT["SELU"], x)
    assert_close(oracle.act_bwd(ACT["SELU"], x, y, dY), dY * oracle.act_bwd(ACT["SELU"], x, y, one), 1e-6, "linear")


# ---------------------------------------------------------------- BRN backward (a20, a21)
@pytest.mark.parametrize("renorm", [True, False])
@pytest.mark.parametrize("nt", [0, 3])
def test_norm_backward_finite_difference(oracle, oracle64, renorm, nt):
    """dx must be the gradient of sum(dN * out) w.r.t. x with r and d frozen
    (the reference treats them as constants).  Checked against central
    differences of the float64 forward."""
    rng = np.random.default_rng(30)
    B, H = 7, 4
    x = rng.standard_normal((B, H)) * 1.5 + 0.3
    gamma = rng.uniform(.8, 1.2, H); beta = rng.uniform(-.1, .1, H)
    mm = rng.uniform(-1, 1, H); ms = rng.uniform(.5, 2, H)
    dN = rng.standard_normal((B, H))
    hyper = (0.3, 1e-5, 1.3, 0.3)
    fw = oracle64.norm_fwd_train(x, gamma, beta, mm, ms, *hyper, renorm)
    r, d = fw["r"], fw["d"]

    def loss(xv):
        mu = xv.mean(0); sd = np.sqrt((xv * xv).mean(0) - mu * mu + hyper[1])
        return float(np.sum(dN * (gamma * ((xv - mu) / sd * r + d) + beta)))

    num = np.zeros_like(x)
    h = 1e-6
    for i in range(B):
        for j in range(H):
            xp = x.copy(); xp[i, j] += h
            xm = x.copy(); xm[i, j] -= h
            num[i, j] = (loss(xp) - loss(xm)) / (2 * h)
    fw32 = oracle.norm_fwd_train(x, gamma, beta, mm, ms, *hyper, renorm, nt)
    bw = oracle.norm_bwd(fw32["mean"], fw32["std"], gamma, fw32["r"], x, fw32["xhat"], dN, renorm=renorm, nthreads=nt)
    assert_close(bw["dx"], num, 2e-4, "dx vs finite differences")
    assert_close(bw["dbeta"], dN.sum(0), 1e-5, "dbeta")
    assert_close(bw["dgamma"], (dN * fw["xhat"]).sum(0), 1e-5, "dgamma")
    dx = bw["dx"].astype(np.float64)
    assert np.max(np.abs(dx.sum(0))) < 1e-5                       # sum_b dx = 0
    # sum_b dx (x - mu) = r * S * eps / sigma^3 with S = sum_b gamma dN (x - mu): zero but for eps
    xc = x - x.mean(0)
    S = (gamma * dN * xc).sum(0)
    assert np.max(np.abs((dx * xc).sum(0) - fw["r"] * S * hyper[1] / fw["std"] ** 3)) < 2e-6


# ---------------------------------------------------------------- dropout, add, softmax, seed gradient
def test_dropout_and_identity_closed_forms(oracle):
    v = rnd(40, 5, 6)
    mask = np.array([1, 0, 1, 1, 0, 1], np.uint8)
    s = np.float32(1 / 0.75)
    assert np.array_equal(oracle.dropout_fwd(0, v, mask, s), np.where(mask, v * s, 0).astype(np.float32))
    assert np.array_equal(oracle.dropout_fwd(1, v, mask, 0.0), np.where(mask, v, 0).astype(np.float32))
    assert np.array_equal(oracle.dropout_fwd(2, v, None, 0.75), v * np.float32(0.75))
    m2 = (np.random.default_rng(41).uniform(size=(5, 6)) < 0.5).astype(np.uint8)
    assert np.array_equal(oracle.dropout_fwd(0, v, m2, s), np.where(m2, v * s, 0).astype(np.float32))
    assert np.array_equal(oracle.identity_add(v, 2 * v), v + 2 * v)


def test_softmax_and_ce_seed_gradient(oracle):
    x = rnd(50, 6, 10) * 4
    q = oracle.softmax_fwd(x)
    assert_close(q, F.softmax(torch.from_numpy(x), 1).numpy(), 2e-6, "softmax")
    labels = np.arange(6) % 10
    y = np.eye(10, dtype=np.float32)[labels]
    dZ, loss, correct = oracle.softmax_ce_seed(q, y)
    assert_close(dZ, (q.astype(np.float64) - y) / 6, 2e-5, "(q - y)/B")
    assert abs(loss - float(-np.log(q[np.arange(6), labels].astype(np.float64)).sum())) < 1e-5
    assert correct == float(np.sum(np.argmax(q, 1) == labels))


def test_softmax_ce_known_answer_of_the_reference_tests(oracle):
    """Constants of the reference's own Dense1x3SoftmaxCCELoss test
    (test/deep-learning/array_grad_adept_test.cpp:152-158): X=0.5,
    W={1.3,-5.3,4.3}, B=0.4, Y={1,0,0}.  That test asserts the hand-derived
    softmax-Jacobian x CCE back-prop equals reverse-mode AD; here the same
    forward is pushed through the leaves and the seed gradient compared with
    the analytic dL/dz = q - y (batch of one), and dW = dz * X, db = dz."""
    X = np.array([[0.5]], np.float32)
    W = np.array([[1.3], [-5.3], [4.3]], np.float32)
    bias = np.full(3, 0.4, np.float32)
    Y = np.array([[1, 0, 0]], np.float32)
    z = oracle.bias_fwd(oracle.fc_fwd(X, W), bias)
    assert_close(z, np.array([[1.05, -2.25, 2.55]]), 1e-6, "pre-activation")
    q = oracle.softmax_fwd(z)
    e = np.exp(np.array([1.05, -2.25, 2.55]))
    assert_close(q, (e / e.sum())[None], 1e-6, "softmax")
    dz, loss, _ = oracle.softmax_ce_seed(q, Y)
    assert_close(dz, (e / e.sum() - Y[0])[None], 1e-6, "q - y")
    assert abs(loss + np.log(e[0] / e.sum())) < 1e-6
    dW, db = oracle.fc_bwd_dw(X, dz)
    assert_close(dW, (dz.T * 0.5), 1e-6, "dW")
    assert_close(db, dz[0], 1e-6, "db")
