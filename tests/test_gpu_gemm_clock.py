"""The measurement aid of the products: a context created with DLMI_GEMM_CLOCK=1 has every workgroup of a product
launch leave its own time stamps (dlmi_ctx_gemm_clock, dlmi_ctx_gemm_timeline).  Checked here: the stamps are
ordered, every workgroup reports a place on the device, the product itself is the same bit for bit as in a context
without the aid, and a context without it refuses the read-out."""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def clocked(pkg):
    os.environ["DLMI_GEMM_CLOCK"] = "1"
    try:
        ctx = pkg.Dlmi(0)
    finally:
        del os.environ["DLMI_GEMM_CLOCK"]
    yield ctx
    ctx.close()


def test_every_workgroup_leaves_ordered_stamps(clocked, dl):
    B, K, H = 16384, 256, 256  # 128 x 2 tiles of 128 x 128
    g = torch.Generator(device="cuda").manual_seed(5)
    X = torch.randn(B, K, device="cuda", generator=g)
    W = torch.randn(H, K, device="cuda", generator=g) * 0.05
    bias = torch.randn(H, device="cuda", generator=g)
    Z, Z0 = torch.empty(B, H, device="cuda"), torch.empty(B, H, device="cuda")
    clocked.fc_fwd(X, W, bias, out=Z)
    dl.fc_fwd(X, W, bias, out=Z0)
    mhz, us = clocked.gemm_clock()
    assert 500.0 < mhz < 3000.0 and 1.0 < us < 1000.0
    n = 256
    a = clocked.gemm_timeline(n)
    torch.cuda.synchronize()
    assert torch.equal(Z, Z0)
    start, issued, done = a[:, 0], a[:, 1], a[:, 2]
    assert (start > 0).all() and (start <= issued).all() and (issued <= done).all()
    assert (done - start).max() < 100 * 1000 * 1000  # ticks of 10 ns: well under a second
    assert done.max() - start.min() < 100 * 1000 * 1000
    xcd = a[:, 3] >> 32
    assert set(xcd.tolist()) == set(range(8))  # the workgroups of a launch go to the XCDs in turn
    assert len(set(a[:, 3].tolist())) > 8


def test_a_context_without_the_aid_refuses(dl):
    with pytest.raises(RuntimeError, match="DLMI_GEMM_CLOCK"):
        dl.gemm_timeline(4)
    with pytest.raises(RuntimeError, match="DLMI_GEMM_CLOCK"):
        dl.gemm_clock()


def test_too_many_workgroups_are_refused(clocked):
    with pytest.raises(RuntimeError, match="4096"):
        clocked.gemm_timeline(4097)
