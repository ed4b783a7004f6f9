"""dlmi_fc_norm_act_fwd — the FC forward whose GEMM epilogue supplies the batch
statistics — against the oracle's FC -> batch renorm -> activation -> dropout
composition, on tile-aligned and ragged shapes."""
import numpy as np
import pytest
import torch

from helpers import RTOL_REDUCED as TR
from helpers import assert_close
from oracle.binding import ACT, DROP

pytestmark = pytest.mark.gpu


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.ascontiguousarray(a)).to("cuda", dtype=dtype).contiguous()


def host(t):
    return t.detach().cpu().numpy()


@pytest.mark.parametrize("B,K,H", [(256, 64, 256), (512, 128, 1024), (100, 70, 36), (1024, 32, 512), (33, 5, 7)])
@pytest.mark.parametrize("act,drop", [("ELU", "NONE"), ("ISRLU", "BERNOULLI_INVERTED"), ("RELU", "BERNOULLI")])
def test_fc_norm_act_fwd_against_oracle(dl, oracle, pkg, B, K, H, act, drop):
    rng = np.random.default_rng(B + K + H)
    X = rng.standard_normal((B, K)).astype(np.float32)
    W = (rng.uniform(-1, 1, (H, K)) * np.sqrt(6.0 / (K + H))).astype(np.float32)
    gamma = rng.uniform(.8, 1.2, H).astype(np.float32); beta = rng.uniform(-.1, .1, H).astype(np.float32)
    mm = rng.uniform(-.1, .1, H).astype(np.float32); ms = rng.uniform(.5, 1.5, H).astype(np.float32)
    keep = 0.9
    mask = (rng.uniform(size=(B, H)) < keep).astype(np.uint8)
    scale = float(np.float32(1) / np.float32(keep)) if drop == "BERNOULLI_INVERTED" else 1.0
    hyper = (0.99, 1e-5, 3.0, 5.0)
    nt = 4
    Zo = oracle.fc_fwd(X, W, nt)
    fw = oracle.norm_fwd_train(Zo, gamma, beta, mm, ms, *hyper, True, nt)
    yo = oracle.act_fwd(ACT[act], fw["out"], nt)
    if drop != "NONE":
        yo = oracle.dropout_fwd(0 if drop == "BERNOULLI_INVERTED" else 1, yo, mask, scale, nt)
    desc = pkg.Dlmi.desc(ACT[act], renorm=True, dropout=DROP[drop], mask_per_element=True, momentum=hyper[0],
                         eps=hyper[1], r_max=hyper[2], d_max=hyper[3], drop_scale=scale)
    dmm, dms = dev(mm), dev(ms)
    Z, y, st = dl.fc_norm_act_fwd(desc, dev(X), dev(W), dev(gamma), dev(beta), dmm, dms,
                                  mask=dev(mask, torch.uint8) if drop != "NONE" else None)
    assert_close(host(Z), Zo, TR, "Z")
    for k in ("mean", "std", "r", "d"):
        assert_close(host(st[k]), fw[k], TR, k, floor=1.0 if k in ("d", "mean") else 0.0)
    assert_close(host(dmm), fw["mov_mean"], TR, "moving mean", floor=1.0)
    assert_close(host(dms), fw["mov_std"], TR, "moving std")
    assert_close(host(y), yo, TR, "y")
    # same result as the two-call sequence on the GPU (GEMM, then the statistics pass over Z)
    dmm2, dms2 = dev(mm), dev(ms)
    y2, st2 = dl.fused_fwd(desc, Z, dev(gamma), dev(beta), dmm2, dms2,
                           mask=dev(mask, torch.uint8) if drop != "NONE" else None)
    assert_close(host(y), host(y2), TR, "epilogue statistics vs statistics pass")


@pytest.mark.parametrize("B,K,H", [(256, 64, 256), (1024, 96, 2048), (100, 70, 36), (33, 5, 7)])
@pytest.mark.parametrize("act,drop", [("ISRLU", "BERNOULLI_INVERTED"), ("SELU", "NONE")])
def test_shortcut_in_the_same_pass_equals_the_separate_add(dl, oracle, pkg, B, K, H, act, drop):
    """y = shortcut + dropout(f(norm(Z))) from dlmi_fused_norm_act_residual_fwd and
    dlmi_fc_norm_act_residual_fwd: bit-identical to the un-fused call followed by dlmi_identity_add
    (the same sum, formed once), and within tolerance of the oracle's leaves
    (Forward_Pass__Zero_Padded_Identity, fwp_st.cpp:5051-5112)."""
    rng = np.random.default_rng(B * 7 + K + H)
    X = rng.standard_normal((B, K)).astype(np.float32)
    W = (rng.uniform(-1, 1, (H, K)) * np.sqrt(6.0 / (K + H))).astype(np.float32)
    S = rng.standard_normal((B, H)).astype(np.float32)
    gamma = rng.uniform(.8, 1.2, H).astype(np.float32); beta = rng.uniform(-.1, .1, H).astype(np.float32)
    mm = rng.uniform(-.1, .1, H).astype(np.float32); ms = rng.uniform(.5, 1.5, H).astype(np.float32)
    keep = 0.9
    mask = (rng.uniform(size=(B, H)) < keep).astype(np.uint8)
    scale = float(np.float32(1) / np.float32(keep))
    hyper = (0.99, 1e-5, 3.0, 5.0)
    desc = pkg.Dlmi.desc(ACT[act], renorm=True, dropout=DROP[drop], mask_per_element=True, momentum=hyper[0],
                         eps=hyper[1], r_max=hyper[2], d_max=hyper[3], drop_scale=scale)
    dmask = dev(mask, torch.uint8) if drop != "NONE" else None
    dX, dW, dS, dg, db = dev(X), dev(W), dev(S), dev(gamma), dev(beta)
    # reference composition on the GPU
    m0, s0 = dev(mm), dev(ms)
    Z0, y0, st0 = dl.fc_norm_act_fwd(desc, dX, dW, dg, db, m0, s0, mask=dmask)
    sum0 = dl.identity_add(dS, y0)
    # GEMM + statistics in the epilogue + shortcut in the apply pass
    m1, s1 = dev(mm), dev(ms)
    Z1, y1, st1 = dl.fc_norm_act_fwd(desc, dX, dW, dg, db, m1, s1, mask=dmask, shortcut=dS)
    assert torch.equal(Z1, Z0) and torch.equal(y1, sum0) and torch.equal(m1, m0) and torch.equal(s1, s0)
    for k in st0:
        assert torch.equal(st1[k], st0[k]), k
    # statistics pass over Z + shortcut
    m2, s2 = dev(mm), dev(ms)
    y2, st2 = dl.fused_fwd(desc, Z0, dg, db, m2, s2, mask=dmask, shortcut=dS)
    m3, s3 = dev(mm), dev(ms)
    y3, _ = dl.fused_fwd(desc, Z0, dg, db, m3, s3, mask=dmask)
    assert torch.equal(y2, dl.identity_add(dS, y3)) and torch.equal(m2, m3)
    # and in place on the shortcut
    S_inplace = dS.clone()
    dl.fused_fwd(desc, Z0, dg, db, dev(mm), dev(ms), mask=dmask, shortcut=S_inplace, out=S_inplace)
    assert torch.equal(S_inplace, y2)
    # the oracle's leaves
    nt = 4
    Zo = oracle.fc_fwd(X, W, nt)
    fw = oracle.norm_fwd_train(Zo, gamma, beta, mm, ms, *hyper, True, nt)
    yo = oracle.act_fwd(ACT[act], fw["out"], nt)
    if drop != "NONE":
        yo = oracle.dropout_fwd(0, yo, mask, scale, nt)
    assert_close(host(y1), oracle.identity_add(S, yo, nt), TR, "shortcut + y")
