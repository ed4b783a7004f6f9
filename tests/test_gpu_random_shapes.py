"""Seeded sweep over irregular shapes, through the C ABI, against the oracle: the
three fully-connected products and the fused normalization + activation +
dropout forward / backward on shapes drawn at random (odd sizes, sizes just
around the tile edges and the 16-byte vector width, very thin and very wide
tensors).  The fixed list in test_gpu_parity.py pins the named cases; this one
looks for an index or tail mistake that only an unplanned shape would meet."""
import numpy as np
import pytest

from helpers import RTOL_REDUCED as TR
from helpers import assert_close
from oracle.binding import ACT, DROP
from test_gpu_parity import dev, host, oracle_fused

pytestmark = pytest.mark.gpu

EDGES = [1, 2, 3, 4, 5, 7, 8, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 513]


def draw_shapes(seed, n, ndim, cap):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < n:
        dims = [int(rng.choice(EDGES)) if rng.uniform() < 0.6 else int(rng.integers(1, 700)) for _ in range(ndim)]
        if np.prod(dims) <= cap:
            out.append(tuple(dims))
    return out


@pytest.mark.parametrize("B,K,H", draw_shapes(2024, 40, 3, 6_000_000))
def test_products_on_random_shapes(dl, oracle, B, K, H):
    rng = np.random.default_rng(B * 1009 + K * 31 + H)
    X = rng.standard_normal((B, K)).astype(np.float32)
    W = rng.uniform(-1, 1, (H, K)).astype(np.float32)
    bias = rng.uniform(-1, 1, H).astype(np.float32)
    dZ = rng.standard_normal((B, H)).astype(np.float32)
    nt = oracle.max_threads()
    assert_close(host(dl.fc_fwd(dev(X), dev(W), dev(bias))), oracle.bias_fwd(oracle.fc_fwd(X, W, nt), bias), TR, "Z")
    dY0 = rng.standard_normal((B, K)).astype(np.float32)
    got = dl.fc_bwd_dx(dev(dZ), dev(W), out=dev(dY0), accumulate=True)
    assert_close(host(got), oracle.fc_bwd_dx(dZ, W, dY_init=dY0, nthreads=nt), TR, "dX accumulated")
    dW0, db0 = rng.standard_normal((H, K)).astype(np.float32), rng.standard_normal(H).astype(np.float32)
    dWo, dbo = oracle.fc_bwd_dw(X, dZ, dW_init=dW0, db_init=db0, nthreads=nt)
    dW, db = dl.fc_bwd_dw(dev(X), dev(dZ), dW=dev(dW0), db=dev(db0), accumulate=True)
    assert_close(host(dW), dWo, TR, "dW accumulated")
    assert_close(host(db), dbo, TR, "db accumulated")


@pytest.mark.parametrize("B,H", [s for s in draw_shapes(7, 40, 2, 3_000_000) if s[0] >= 2])
def test_fused_norm_on_random_shapes(dl, oracle, pkg, B, H):
    rng = np.random.default_rng(B * 1013 + H)
    act = ["SELU", "ELU", "ISRLU", "RELU", "LEAKY_RELU", "SIGMOID", "TANH"][(B + H) % 7]
    drop = ["NONE", "BERNOULLI", "BERNOULLI_INVERTED"][(B * 7 + H) % 3]
    renorm = bool((B + 3 * H) % 2)
    x = (rng.standard_normal((B, H)) * rng.uniform(.5, 2, H) + rng.uniform(-1, 1, H)).astype(np.float32)
    gamma = rng.uniform(.8, 1.2, H).astype(np.float32)
    beta = rng.uniform(-.1, .1, H).astype(np.float32)
    dY = rng.standard_normal((B, H)).astype(np.float32)
    dg0, db0 = rng.standard_normal(H).astype(np.float32), rng.standard_normal(H).astype(np.float32)
    hyper = (0.9, 1e-3, 2.0, 1.0)
    mm, ms = rng.uniform(-.5, .5, H).astype(np.float32), rng.uniform(.5, 2, H).astype(np.float32)
    mask = (rng.uniform(size=H) < 0.7).astype(np.uint8)
    scale = float(np.float32(1) / np.float32(0.7)) if drop == "BERNOULLI_INVERTED" else 1.0
    pre = oracle.norm_fwd_train(x, gamma, beta, mm, ms, *hyper, renorm, 2)["out"]
    dY[np.abs(pre) < 1e-5] = 0  # the derivatives jump at 0
    fw, y, bw = oracle_fused(oracle, ACT[act], x, gamma, beta, mm, ms, hyper, renorm, DROP[drop],
                             None if drop == "NONE" else mask, scale, False, dY, dg0, db0, nt=2)
    desc = pkg.Dlmi.desc(ACT[act], renorm=renorm, dropout=DROP[drop], momentum=hyper[0], eps=hyper[1], r_max=hyper[2],
                         d_max=hyper[3], drop_scale=scale)
    dmask = None if drop == "NONE" else dev(mask, dtype=__import__("torch").uint8)
    dmm, dms = dev(mm), dev(ms)
    yg, st = dl.fused_fwd(desc, dev(x), dev(gamma), dev(beta), dmm, dms, mask=dmask)
    assert_close(host(yg), y, TR, "y")
    assert_close(host(dmm), fw["mov_mean"], TR, "moving mean", floor=1.0)
    assert_close(host(dms), fw["mov_std"], TR, "moving std")
    dg, db = dev(dg0), dev(db0)
    dX = dl.fused_bwd(desc, dev(x), dev(gamma), dev(beta), st, dev(dY), dg, db, mask=dmask)
    assert_close(host(dX), bw["dx"], TR, "dX", floor=1e-3)
    assert_close(host(dg), bw["dgamma"], TR, "dgamma", floor=1.0)
    assert_close(host(db), bw["dbeta"], TR, "dbeta", floor=1.0)
