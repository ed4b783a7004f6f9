"""A weight gradient that is split over K (few output tiles, a long batch) forms the bias gradient on its way: the
workgroups of one tile column add up the rows of dZ they stage, per slice, and the slice sum adds the shares up
(dlmi_fc_bwd_dw with db).  Checked against float64 column sums and against a context created with
DLMI_DB_IN_PRODUCT=0, which passes over dZ once more: dW must be the same bit for bit (the products are the same
code), db equal to the rounding of two summation orders."""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def second_pass(pkg):
    os.environ["DLMI_DB_IN_PRODUCT"] = "0"
    try:
        ctx = pkg.Dlmi(0)
    finally:
        del os.environ["DLMI_DB_IN_PRODUCT"]
    yield ctx
    ctx.close()


# (B, K, H): split products of 128 x 128 tiles with 4 and 8 wavefronts, one and two register stages, one to four
# tile columns; the last two are not split (the bias gradient then takes the pass over dZ in both contexts)
SHAPES = [(65536, 256, 256), (8192, 128, 128), (16384, 256, 128), (4096, 512, 128), (32768, 128, 384), (2048, 384, 256),
          (512, 256, 256), (1024, 2048, 2048)]


@pytest.mark.parametrize("B,K,H", SHAPES)
@pytest.mark.parametrize("accumulate", [False, True])
def test_bias_gradient_of_a_split_weight_gradient(dl, second_pass, B, K, H, accumulate):
    g = torch.Generator(device="cuda").manual_seed(B + K + H)
    X = torch.randn(B, K, device="cuda", generator=g)
    dZ = torch.randn(B, H, device="cuda", generator=g) + 0.25
    dW0 = torch.randn(H, K, device="cuda", generator=g)
    db0 = torch.randn(H, device="cuda", generator=g)
    out = []
    for ctx in (dl, second_pass):
        dW, db = dW0.clone(), db0.clone()
        ctx.fc_bwd_dw(X, dZ, dW=dW, db=db, accumulate=accumulate)
        ctx.synchronize()
        out.append((dW, db))
    assert torch.equal(out[0][0], out[1][0])
    want = dZ.double().sum(0) + (db0.double() if accumulate else 0.0)
    scale = dZ.double().abs().sum(0)  # the size of what a float sum of B terms can lose
    for _, db in out:
        assert float(((db.double() - want).abs() / scale).max()) < 2e-6
    # and without a bias gradient asked for nothing changes in dW
    dW = dW0.clone()
    dl.fc_bwd_dw(X, dZ, dW=dW, accumulate=accumulate)
    assert torch.equal(dW, out[0][0])


def test_repeated_calls_give_the_same_bits(dl):
    B, K, H = 16384, 256, 256
    g = torch.Generator(device="cuda").manual_seed(1)
    X, dZ = torch.randn(B, K, device="cuda", generator=g), torch.randn(B, H, device="cuda", generator=g)
    first = None
    for _ in range(3):
        dW, db = torch.empty(H, K, device="cuda"), torch.empty(H, device="cuda")
        dl.fc_bwd_dw(X, dZ, dW=dW, db=db)
        dl.synchronize()
        if first is None:
            first = (dW, db)
        else:
            assert torch.equal(dW, first[0]) and torch.equal(db, first[1])
