"""Degenerate shapes and refused arguments, through the C ABI.

Shapes: the smallest and the most lopsided tensors the kernels' grids and tails
can meet (two rows, one unit, one very tall column), against the oracle.  A
single row is left out on purpose: its variance E[x^2] - mean^2 is an exact
cancellation, so sigma = sqrt(eps + rounding noise) depends on whether the
compiler fuses the multiply-add, on either side.

Refusals: every size or pointer check happens on the host before any launch, so
these calls must come back with DLMI_E_INVALID and a message, and the context
must stay usable afterwards."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import RTOL_REDUCED as TR
from helpers import assert_close
from oracle.binding import ACT, DROP
from test_gpu_parity import dev, host, oracle_fused

pytestmark = pytest.mark.gpu

c_sz = ctypes.c_size_t
vp = ctypes.c_void_p


@pytest.mark.parametrize("B,H", [(2, 1), (2, 7), (3, 1), (5000, 1), (40000, 3), (2, 4100),
                                 # a million units (odd: the scalar path; partial sums beyond the first scratch block)
                                 (16, 1_000_003), (24, 600_000)])
@pytest.mark.parametrize("renorm", [True, False])
def test_fused_degenerate_shapes(dl, oracle, pkg, B, H, renorm):
    rng = np.random.default_rng(B * 13 + H)
    x = (rng.standard_normal((B, H)) * rng.uniform(.5, 2, H) + rng.uniform(-1, 1, H)).astype(np.float32)
    gamma = rng.uniform(.8, 1.2, H).astype(np.float32)
    beta = rng.uniform(-.1, .1, H).astype(np.float32)
    dY = rng.standard_normal((B, H)).astype(np.float32)
    dg0, db0 = rng.standard_normal(H).astype(np.float32), rng.standard_normal(H).astype(np.float32)
    hyper = (0.9, 1e-3, 3.0, 5.0)  # eps large enough that two nearly equal rows stay well conditioned
    mm, ms = rng.uniform(-.5, .5, H).astype(np.float32), rng.uniform(.5, 2, H).astype(np.float32)
    pre = oracle.norm_fwd_train(x, gamma, beta, mm, ms, *hyper, renorm, 2)["out"]
    dY[np.abs(pre) < 1e-5] = 0
    fw, y, bw = oracle_fused(oracle, ACT["ELU"], x, gamma, beta, mm, ms, hyper, renorm, DROP["NONE"], None, 1.0, False,
                             dY, dg0, db0, nt=2)
    desc = pkg.Dlmi.desc(ACT["ELU"], renorm=renorm, momentum=hyper[0], eps=hyper[1], r_max=hyper[2], d_max=hyper[3])
    dmm, dms = dev(mm), dev(ms)
    yg, st = dl.fused_fwd(desc, dev(x), dev(gamma), dev(beta), dmm, dms)
    # E[x^2] - mean^2 in fp32 loses log2(E[x^2] / variance) bits: with two or three rows whose values
    # nearly agree the variance is as small as eps, and every order of evaluation (the reference's own
    # OpenMP path included) lands within a few roundings of E[x^2], not of the variance
    x64 = x.astype(np.float64)
    cond = float(np.max(((x64 * x64).mean(0) + hyper[1]) / (x64.var(0) + hyper[1])))
    TRC = max(TR, 4 * 2.0 ** -24 * cond)
    assert_close(host(yg), y, TRC, "y")
    for k in ("mean", "std", "r", "d"):
        assert_close(host(st[k]), fw[k], TRC, k, floor=1.0)
    assert_close(host(dmm), fw["mov_mean"], TR, "moving mean", floor=1.0)
    assert_close(host(dms), fw["mov_std"], TRC, "moving std")
    dg, db = dev(dg0), dev(db0)
    dX = dl.fused_bwd(desc, dev(x), dev(gamma), dev(beta), st, dev(dY), dg, db)
    assert_close(host(dX), bw["dx"], TRC, "dX", floor=1e-3)
    assert_close(host(dg), bw["dgamma"], TRC, "dgamma", floor=1.0)
    assert_close(host(db), bw["dbeta"], TRC, "dbeta", floor=1.0)
    yi = dl.fused_infer(desc, dev(x), dev(gamma), dev(beta), dev(mm), dev(ms))
    assert_close(host(yi), oracle.act_fwd(ACT["ELU"], oracle.norm_fwd_infer(x, gamma, beta, mm, ms)), TR, "inference")


def test_three_million_rows_against_float64(dl, oracle, oracle64, pkg):
    """[3 000 000 x 8]: the batch is cut into the largest number of chunks the grid takes.  At this
    length the reference's single fp32 accumulator per thread is itself off by more than the
    tolerance (about 7e-4 on the outputs), so float64 arbitrates: the GPU's chunked sums must
    meet the tolerance against it, and be nearer to it than the fp32 restatement is."""
    from helpers import max_rel_err
    B, H = 3_000_000, 8
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((B, H)) * rng.uniform(.5, 2, H) + rng.uniform(-1, 1, H)).astype(np.float32)
    gamma, beta = rng.uniform(.8, 1.2, H).astype(np.float32), rng.uniform(-.1, .1, H).astype(np.float32)
    dY = rng.standard_normal((B, H)).astype(np.float32)
    zero, one = np.zeros(H, np.float32), np.ones(H, np.float32)
    hyper = (0.9, 1e-5, 3.0, 5.0)
    a = ACT["LEAKY_RELU"]
    args = (a, x, gamma, beta, zero, one, hyper, True, DROP["NONE"], None, 1.0, False, dY, zero, zero)
    fw32, y32, bw32 = oracle_fused(oracle, *args, nt=oracle.max_threads())
    fw64, y64, bw64 = oracle_fused(oracle64, *args, nt=oracle.max_threads())
    desc = pkg.Dlmi.desc(a, momentum=hyper[0], eps=hyper[1], r_max=hyper[2], d_max=hyper[3])
    dmm, dms = dev(zero), dev(one)
    yg, st = dl.fused_fwd(desc, dev(x), dev(gamma), dev(beta), dmm, dms)
    dg, db = dev(zero), dev(zero)
    dX = dl.fused_bwd(desc, dev(x), dev(gamma), dev(beta), st, dev(dY), dg, db)
    assert_close(host(st["mean"]), fw64["mean"], TR, "mean vs float64", floor=1.0)
    assert_close(host(st["std"]), fw64["std"], TR, "std vs float64")
    assert_close(host(yg), y64, TR, "y vs float64")
    assert_close(host(dX), bw64["dx"], TR, "dX vs float64", floor=1e-3)
    assert_close(host(dg), bw64["dgamma"], TR, "dgamma vs float64", floor=1.0)
    assert_close(host(db), bw64["dbeta"], TR, "dbeta vs float64", floor=1.0)
    assert max_rel_err(host(yg), y64, 0.0) <= max_rel_err(y32, y64, 0.0)


@pytest.mark.parametrize("B,K,H", [(1, 4096, 1), (1, 1, 300), (4097, 1, 1), (2, 3, 4099), (3, 5000, 2)])
def test_gemm_degenerate_shapes(dl, oracle, B, K, H):
    rng = np.random.default_rng(B + 3 * K + 7 * H)
    X = rng.standard_normal((B, K)).astype(np.float32)
    W = rng.uniform(-1, 1, (H, K)).astype(np.float32)
    dZ = rng.standard_normal((B, H)).astype(np.float32)
    assert_close(host(dl.fc_fwd(dev(X), dev(W))), oracle.fc_fwd(X, W), TR, "Z")
    assert_close(host(dl.fc_bwd_dx(dev(dZ), dev(W))), oracle.fc_bwd_dx(dZ, W), TR, "dX")
    dWo, dbo = oracle.fc_bwd_dw(X, dZ)
    dW, db = dl.fc_bwd_dw(dev(X), dev(dZ), with_bias=True)
    assert_close(host(dW), dWo, TR, "dW")
    assert_close(host(db), dbo, TR, "db")


def test_refused_arguments_leave_the_context_usable(dl, pkg):
    lib, ctx = dl.lib, dl.ctx
    lib.dlmi_last_error.restype = ctypes.c_char_p
    a = torch.ones(4, 4, device="cuda")
    v = torch.ones(4, device="cuda")
    p = lambda t: vp(t.data_ptr())
    desc = pkg.Dlmi.desc(ACT["RELU"])
    OFF_PATH = 19  # ACTIVATION::SINE: not one of the path's activations
    bad_act = pkg.Dlmi.desc(OFF_PATH)
    INVALID, UNSUPPORTED = -1, -4
    calls = {
        "fc_fwd, no rows": lambda: lib.dlmi_fc_fwd(ctx, c_sz(0), c_sz(4), c_sz(4), p(a), p(a), None, p(a)),
        "fc_fwd, null W": lambda: lib.dlmi_fc_fwd(ctx, c_sz(4), c_sz(4), c_sz(4), p(a), None, None, p(a)),
        "fc_bwd_dx, no units": lambda: lib.dlmi_fc_bwd_dx(ctx, c_sz(4), c_sz(4), c_sz(0), p(a), p(a), p(a), 0),
        "fc_bwd_dw, null dW": lambda: lib.dlmi_fc_bwd_dw(ctx, c_sz(4), c_sz(4), c_sz(4), p(a), p(a), None, None, 0),
        "fused fwd, no rows": lambda: lib.dlmi_fused_norm_act_fwd(ctx, ctypes.byref(desc), c_sz(0), c_sz(4), p(a), p(v), p(v),
                                                                  None, p(v), p(v), p(v), p(v), p(v), p(v), p(a)),
        "fused fwd, null statistics": lambda: lib.dlmi_fused_norm_act_fwd(ctx, ctypes.byref(desc), c_sz(4), c_sz(4), p(a),
                                                                          p(v), p(v), None, None, p(v), p(v), p(v), p(v),
                                                                          p(v), p(a)),
        "fused fwd, null descriptor": lambda: lib.dlmi_fused_norm_act_fwd(ctx, None, c_sz(4), c_sz(4), p(a), p(v), p(v), None,
                                                                          p(v), p(v), p(v), p(v), p(v), p(v), p(a)),
        "fused fwd, activation off the path": lambda: lib.dlmi_fused_norm_act_fwd(
            ctx, ctypes.byref(bad_act), c_sz(4), c_sz(4), p(a), p(v), p(v), None, p(v), p(v), p(v), p(v), p(v), p(v), p(a)),
        "act_fwd, activation off the path": lambda: lib.dlmi_act_fwd(ctx, OFF_PATH, c_sz(4), c_sz(4), p(a), p(a)),
        "zero-padded identity, padding past the wider operand": lambda: lib.dlmi_zero_padded_identity_fwd(
            ctx, c_sz(4), c_sz(4), c_sz(2), c_sz(3), p(a), p(a), p(a)),
    }
    for what, call in calls.items():
        rc = call()
        assert rc in (INVALID, UNSUPPORTED), f"{what}: returned {rc}"
        if "null descriptor" not in what:  # that one cannot even look the message buffer up
            assert lib.dlmi_last_error(ctx), what
    # nothing was launched and nothing is poisoned: a good call still works
    out = dl.fc_fwd(a, a)
    assert torch.equal(out, torch.full((4, 4), 4.0, device="cuda"))
