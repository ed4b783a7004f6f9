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
