"""The CPU restatement against the real reference, compiled (oracle/_ref), on
randomized shapes and thread counts beyond what the golden files hold.  Skipped
where that library was not built."""
import numpy as np
import pytest

from helpers import RTOL_RESTATEMENT, assert_close
from oracle.binding import ACT

T = 4 * RTOL_RESTATEMENT


@pytest.mark.parametrize("seed", range(6))
def test_random_leaves(oracle, reference, seed):
    rng = np.random.default_rng(1000 + seed)
    B, K, H = int(rng.integers(1, 40)), int(rng.integers(1, 70)), int(rng.integers(1, 70))
    nt = int(rng.integers(0, 7))
    f = lambda *s: rng.standard_normal(s).astype(np.float32)
    X, W, x, dN = f(B, K), f(H, K), f(B, H) * 2 + 0.5, f(B, H)
    gamma, beta = rng.uniform(.8, 1.2, H).astype(np.float32), rng.uniform(-.1, .1, H).astype(np.float32)
    mm, ms = rng.uniform(-1, 1, H).astype(np.float32), rng.uniform(.5, 2, H).astype(np.float32)
    assert_close(oracle.fc_fwd(X, W, nt), reference.fc_fwd(X, W, nt), T, "fc_fwd")
    assert_close(oracle.fc_bwd_dx(dN, W, nthreads=nt), reference.fc_bwd_dx(dN, W, nthreads=nt), T, "dx")
    a, b = oracle.fc_bwd_dw(X, dN, nthreads=nt), reference.fc_bwd_dw(X, dN, nthreads=nt)
    assert_close(a[0], b[0], T, "dW"); assert_close(a[1], b[1], T, "db")
    for renorm in (True, False):
        hyper = (float(rng.uniform(0.01, 1)), 1e-5, float(rng.uniform(1, 3)), float(rng.uniform(0, 1)))
        fo = oracle.norm_fwd_train(x, gamma, beta, mm, ms, *hyper, renorm, nt)
        fr = reference.norm_fwd_train(x, gamma, beta, mm, ms, *hyper, renorm, nt)
        for k in fo:
            assert_close(fo[k], fr[k], T, f"norm fwd {k}")
        bo = oracle.norm_bwd(fr["mean"], fr["std"], gamma, fr["r"], x, fr["xhat"], dN, renorm=renorm, nthreads=nt)
        br = reference.norm_bwd(fr["mean"], fr["std"], gamma, fr["r"], x, fr["xhat"], dN, renorm=renorm, nthreads=nt)
        for k in bo:
            assert_close(bo[k], br[k], T, f"norm bwd {k}")
    assert_close(oracle.norm_fwd_infer(x, gamma, beta, mm, ms, nt), reference.norm_fwd_infer(x, gamma, beta, mm, ms, nt), T, "infer")
    for name in ("ELU", "ISRLU", "LEAKY_RELU", "RELU", "SELU", "LINEAR"):
        y = reference.act_fwd(ACT[name], x, nt)
        assert_close(oracle.act_fwd(ACT[name], x, nt), y, T, name)
        assert_close(oracle.act_bwd(ACT[name], x, y, dN, nt), reference.act_bwd(ACT[name], x, y, dN, nt), T, name + "'")
    assert_close(oracle.softmax_fwd(x, nt), reference.softmax_fwd(x, nt), T, "softmax")


def test_reference_layout_8_6_6_3(reference):
    """Parameter-array layout of the reference itself: weights, then biases,
    then a gamma slot and a beta slot for EVERY layer including the input
    (8-6-6-3 net: 102 + 15 + 2*23 = 163)."""
    M = reference.mlp([8, 6, 6, 3])
    M.set_layer(1, ACT["RELU"], 2); M.set_layer(2, ACT["RELU"], 2); M.set_layer(3, ACT["SOFTMAX"])
    M.prepare(4, 0)
    assert M.P == 163 and M.n_units == 23
    assert [M.layer_offsets(l)[:5] for l in range(1, 4)] == [[0, 102, 125, 148, 8], [48, 108, 131, 154, 14],
                                                             [84, 114, 137, 160, 20]]
