"""The narrow-layer kernels (a layer of at most 16 units on a mini-batch: one launch for product + bias
+ softmax, one launch for dW + db) and the backward that takes its upstream gradient as K slices, against
the tiled-GEMM path of the same library (a context created with DLMI_FC_NARROW=0 / DLMI_NORM_SMALL=0 is the
twin) and against float64."""
import os

import numpy as np
import pytest
import torch

from helpers import assert_close
from oracle.binding import ACT
from test_gpu_norm_panel import dev, make, run_fwd

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def twins(pkg):
    os.environ["DLMI_FC_NARROW"] = "0"
    os.environ["DLMI_NORM_SMALL"] = "0"
    try:
        plain = pkg.Dlmi(0)
    finally:
        del os.environ["DLMI_FC_NARROW"]
        del os.environ["DLMI_NORM_SMALL"]
    fast = pkg.Dlmi(0)
    yield fast, plain
    fast.close()
    plain.close()


def softmax64(z):
    e = np.exp(z - z.max(1, keepdims=True))
    return e / e.sum(1, keepdims=True)


@pytest.mark.parametrize("B,K,H", [(128, 512, 10), (1000, 33, 16), (7, 5, 1), (1024, 784, 3), (64, 1, 16), (3, 1000, 2)])
def test_narrow_forward_with_softmax(twins, pkg, B, K, H):
    fast, plain = twins
    rng = np.random.default_rng(B + K + H)
    X = rng.standard_normal((B, K)).astype(np.float32)
    W = (rng.standard_normal((H, K)) / np.sqrt(K)).astype(np.float32)
    b = rng.uniform(-.5, .5, H).astype(np.float32)
    z64 = X.astype(np.float64) @ W.astype(np.float64).T + b
    for bias in (b, None):
        exact = z64 if bias is not None else z64 - b
        Z, Q = fast.fc_softmax_fwd(dev(X), dev(W), None if bias is None else dev(bias))
        Zp, Qp = plain.fc_softmax_fwd(dev(X), dev(W), None if bias is None else dev(bias))
        Zf = fast.fc_fwd(dev(X), dev(W), None if bias is None else dev(bias))
        assert_close(Z.cpu().numpy(), exact, 1e-4, "Z vs float64", floor=1e-3)
        assert_close(Q.cpu().numpy(), softmax64(exact), 1e-4, "softmax vs float64")
        assert_close(Z.cpu().numpy(), Zp.cpu().numpy(), 1e-4, "Z vs tiled GEMM", floor=1e-3)
        assert_close(Q.cpu().numpy(), Qp.cpu().numpy(), 1e-4, "softmax vs GEMM + softmax leaf")
        assert torch.equal(Z, Zf), "dlmi_fc_fwd takes the same kernel"
        # the softmax is the leaf's arithmetic on the same Z
        assert torch.equal(Q, fast.softmax_fwd(Z))
        assert np.allclose(Q.cpu().numpy().sum(1), 1.0, atol=1e-6)


def test_wider_or_taller_layers_take_the_tiled_path(twins, pkg):
    fast, plain = twins
    rng = np.random.default_rng(4)
    for B, K, H in [(128, 64, 17), (1025, 64, 10)]:
        X, W = rng.standard_normal((B, K)).astype(np.float32), rng.standard_normal((H, K)).astype(np.float32)
        Z, Q = fast.fc_softmax_fwd(dev(X), dev(W))
        Zp, Qp = plain.fc_softmax_fwd(dev(X), dev(W))
        assert torch.equal(Z, Zp) and torch.equal(Q, Qp)


@pytest.mark.parametrize("B,K,H", [(128, 512, 10), (256, 100, 16), (5, 3, 2), (77, 1000, 1), (200, 9, 13)])
def test_narrow_weight_and_bias_gradient(twins, pkg, B, K, H):
    fast, plain = twins
    rng = np.random.default_rng(B * K + H)
    X = rng.standard_normal((B, K)).astype(np.float32)
    dZ = rng.standard_normal((B, H)).astype(np.float32)
    dW64 = dZ.astype(np.float64).T @ X.astype(np.float64)
    db64 = dZ.astype(np.float64).sum(0)
    dW, db = fast.fc_bwd_dw(dev(X), dev(dZ), with_bias=True)
    dWp, dbp = plain.fc_bwd_dw(dev(X), dev(dZ), with_bias=True)
    assert_close(dW.cpu().numpy(), dW64, 1e-4, "dW vs float64", floor=1e-3)
    assert_close(db.cpu().numpy(), db64, 1e-5, "db vs float64", floor=1.0)
    assert_close(dW.cpu().numpy(), dWp.cpu().numpy(), 1e-4, "dW vs tiled GEMM", floor=1e-3)
    assert_close(db.cpu().numpy(), dbp.cpu().numpy(), 1e-5, "db vs column-sum kernels", floor=1.0)
    # accumulating on top, and without a bias gradient
    fast.fc_bwd_dw(dev(X), dev(dZ), dW=dW, db=db, accumulate=True)
    assert_close(dW.cpu().numpy(), 2 * dW64, 1e-4, "dW accumulated", floor=1e-3)
    assert_close(db.cpu().numpy(), 2 * db64, 1e-5, "db accumulated", floor=1.0)
    dW2, none = fast.fc_bwd_dw(dev(X), dev(dZ))
    assert none is None
    assert_close(dW2.cpu().numpy(), dW64, 1e-4, "dW alone", floor=1e-3)


@pytest.mark.parametrize("B,Hn,H,act,drop", [
    (128, 512, 512, "RELU", "NONE"),                  # runs split over K: the normalization kernel adds the slices
    (128, 10, 512, "RELU", "NONE"),                   # a narrow layer above: the normalization kernel forms dY itself
    (256, 16, 36, "SELU", "BERNOULLI_INVERTED"),      # ... the widest it takes, 8 rows per thread, ragged width
    (7, 1, 100, "TANH", "NONE"),
    (33, 3, 8, "LEAKY_RELU", "BERNOULLI"),
    (128, 17, 512, "RELU", "NONE"),                   # one unit too many: product launch, then the normalization kernel
    (200, 300, 36, "ELU", "BERNOULLI_INVERTED"),
    (256, 1024, 64, "TANH", "BERNOULLI"),
    (512, 256, 256, "SELU", "NONE"),                  # more rows than the small-batch kernels take
])
def test_backward_with_the_product_above_it(twins, pkg, B, Hn, H, act, drop):
    """dlmi_fc_bwd_dx_norm_act_bwd against dlmi_fc_bwd_dx followed by dlmi_fused_norm_act_bwd on the twin."""
    fast, plain = twins
    d = make(B, H, B + Hn + H)
    rng = np.random.default_rng(B + H)
    dZn = rng.standard_normal((B, Hn)).astype(np.float32)
    Wn = (rng.standard_normal((Hn, H)) / np.sqrt(Hn)).astype(np.float32)
    _, desc, mask, st = run_fwd(plain, pkg, d, act, drop, False, False)
    dg, db = torch.full((H,), 0.25, device="cuda"), torch.full((H,), -0.5, device="cuda")
    dX = fast.fc_bwd_dx_fused_bwd(desc, dev(dZn), dev(Wn), dev(d["x"]), dev(d["gamma"]), dev(d["beta"]), st, dg, db, mask=mask)
    dgp, dbp = torch.full((H,), 0.25, device="cuda"), torch.full((H,), -0.5, device="cuda")
    dY = plain.fc_bwd_dx(dev(dZn), dev(Wn))
    dXp = plain.fused_bwd(desc, dev(d["x"]), dev(d["gamma"]), dev(d["beta"]), st, dY, dgp, dbp, mask=mask)
    assert_close(dX.cpu().numpy(), dXp.cpu().numpy(), 1e-4, "dX", floor=1.0)
    assert_close(dg.cpu().numpy(), dgp.cpu().numpy(), 1e-4, "dgamma", floor=1.0)
    assert_close(db.cpu().numpy(), dbp.cpu().numpy(), 1e-4, "dbeta", floor=1.0)


@pytest.mark.parametrize("B,K,H", [(128, 512, 10), (1000, 33, 16), (7, 5, 1), (64, 257, 3), (300, 64, 40)])
def test_output_layer_forward_with_the_seed_gradient(twins, pkg, B, K, H):
    """dlmi_fc_softmax_ce_fwd against dlmi_fc_softmax_fwd followed by dlmi_softmax_ce_seed: Z, Q and dZ bit for bit
    (the seed is formed by the same per-row code), the loss and accuracy sums to the rounding of a double sum in
    another grouping; the accumulators accumulate, launch after launch; 40 units: the two-call path inside."""
    fast, _ = twins
    rng = np.random.default_rng(B * 3 + K + H)
    X = dev(rng.standard_normal((B, K)).astype(np.float32))
    W = dev((rng.standard_normal((H, K)) / np.sqrt(K)).astype(np.float32))
    b = dev(rng.uniform(-.5, .5, H).astype(np.float32))
    Y = dev(np.eye(H, dtype=np.float32)[rng.integers(0, H, B)])
    for bias in (b, None):
        st_two = torch.tensor([0.5, 3.0], dtype=torch.float64, device="cuda")
        st_one = st_two.clone()
        Z2, Q2 = fast.fc_softmax_fwd(X, W, bias)
        dZ2 = fast.softmax_ce_seed(Q2, Y, stats=st_two)
        for rep in range(2):  # the ticket and the pairs are left ready for the next launch
            Z1, Q1, dZ1 = fast.fc_softmax_ce_fwd(X, W, Y, bias=bias, stats=st_one)
            assert torch.equal(Z1, Z2) and torch.equal(Q1, Q2) and torch.equal(dZ1, dZ2)
        fast.softmax_ce_seed(Q2, Y, stats=st_two)
        fast.synchronize()
        a, c = st_one.cpu().numpy(), st_two.cpu().numpy()
        assert a[1] == c[1], "correct predictions"
        assert abs(a[0] - c[0]) <= 1e-12 * abs(c[0]), "loss sum"
    # without accumulators
    Z1, Q1, dZ1 = fast.fc_softmax_ce_fwd(X, W, Y, bias=b)
    assert torch.equal(dZ1, fast.softmax_ce_seed(fast.fc_softmax_fwd(X, W, b)[1], Y))


@pytest.mark.parametrize("B,K,H", [(128, 784, 512), (128, 512, 512), (256, 64, 64), (1, 4, 20), (7, 100, 36), (130, 68, 132),
                                   (255, 1000, 24), (64, 2048, 512), (3, 8, 4)])
@pytest.mark.parametrize("accumulate", [False, True])
def test_minibatch_weight_gradient(pkg, B, K, H, accumulate):
    """dW (+)= dZ^T X of a layer of any width on a mini-batch (k_minibatch_dw: one workgroup per 64 x 64 block of dW,
    the batch staged in LDS, the sum over the rows on the matrix pipe) against float64 and against the tiled GEMM
    of the same library (a context created with DLMI_MINIBATCH_DW=0); ragged blocks, batches that are no multiple of
    four, more than one staging pass; bit-reproducible; the bias gradient behind it unchanged."""
    os.environ["DLMI_MINIBATCH_DW"] = "0"
    try:
        plain = pkg.Dlmi(0)
    finally:
        del os.environ["DLMI_MINIBATCH_DW"]
    fast = pkg.Dlmi(0)
    try:
        rng = np.random.default_rng(B + 3 * K + 7 * H)
        X = rng.standard_normal((B, K)).astype(np.float32)
        dZ = rng.standard_normal((B, H)).astype(np.float32)
        dW0 = rng.standard_normal((H, K)).astype(np.float32)
        db0 = rng.standard_normal(H).astype(np.float32)
        want = dZ.astype(np.float64).T @ X.astype(np.float64) + (dW0 if accumulate else 0.0)
        want_db = dZ.astype(np.float64).sum(0) + (db0 if accumulate else 0.0)
        outs = []
        for dl in (fast, plain, fast):
            dW, db = dev(dW0), dev(db0)
            dl.fc_bwd_dw(dev(X), dev(dZ), dW=dW, db=db, accumulate=accumulate)
            dl.synchronize()
            outs.append((dW.cpu().numpy(), db.cpu().numpy()))
        assert_close(outs[0][0], want, 1e-5, "dW vs float64", floor=1.0)
        assert_close(outs[0][0], outs[1][0], 1e-5, "dW vs tiled GEMM", floor=1.0)
        assert_close(outs[0][1], want_db, 1e-5, "db vs float64", floor=1.0)
        assert np.array_equal(outs[0][0], outs[2][0]) and np.array_equal(outs[0][1], outs[2][1]), "not reproducible"
    finally:
        fast.close()
        plain.close()
