"""The remaining benchmark configurations as parity tests.

Configuration 4: deep residual MLP, blocks x + Dropout(ISRLU(BRN(FC(x)))) with a
host-generated per-element uint8 keep-mask, forward + backward — against the
oracle at a reduced size and against a float64 evaluation at the full size
(16 blocks, width 2048, batch 1024).

Configuration 5: tall-skinny FC 256->256 on batch 65536 (1% outliers x50) + BRN +
leaky ReLU, forward + backward at FULL size against the oracle, plus the
inference-mode forward with given moving statistics.
"""
import numpy as np
import pytest
import torch

from helpers import RTOL_ELEMENTWISE as TE
from helpers import RTOL_REDUCED as TR
from helpers import assert_close
from oracle.binding import ACT, DROP

pytestmark = pytest.mark.gpu
HYPER = (0.99, 1e-5, 3.0, 5.0)


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.ascontiguousarray(a)).to("cuda", dtype=dtype).contiguous()


def host(t):
    return t.detach().cpu().numpy()


def residual_gpu(dl, pkg, x, Ws, masks, dOut, keep, bwd_masked):
    """x + Dropout(ISRLU(BRN(FC(x)))) blocks through the C ABI leaves."""
    scale = float(np.float32(1) / np.float32(keep))
    desc = pkg.Dlmi.desc(ACT["ISRLU"], renorm=True, dropout=DROP["BERNOULLI_INVERTED"], mask_per_element=True,
                         dropout_bwd=1 if bwd_masked else 0, momentum=HYPER[0], eps=HYPER[1], r_max=HYPER[2],
                         d_max=HYPER[3], drop_scale=scale)
    H = x.shape[1]
    one, zero = torch.ones(H, device="cuda"), torch.zeros(H, device="cuda")
    saved = []
    cur = x
    for W, m in zip(Ws, masks):
        Z, y, st = dl.fc_norm_act_fwd(desc, cur, W, one, zero, zero.clone(), one.clone(), mask=m)
        saved.append((cur, Z, st))
        cur = dl.identity_add(cur, y)
    out = cur
    g = dOut
    dWs, dgs, dbs = [], [], []
    for (xin, Z, st), W, m in zip(reversed(saved), reversed(Ws), reversed(masks)):
        dg, db = zero.clone(), zero.clone()
        dZ = dl.fused_bwd(desc, Z, one, zero, st, g, dg, db, mask=m)
        dXb = dl.fc_bwd_dx(dZ, W)
        dW, _ = dl.fc_bwd_dw(xin, dZ)
        g = dl.identity_add(g, dXb)  # the shortcut carries dOut, the block adds dX
        dWs.append(dW); dgs.append(dg); dbs.append(db)
    return out, g, dWs[::-1], dgs[::-1], dbs[::-1]


def residual_oracle(oracle, x, Ws, masks, dOut, keep, bwd_masked, nt):
    scale = np.float32(1) / np.float32(keep)
    H = x.shape[1]
    one, zero = np.ones(H, np.float32), np.zeros(H, np.float32)
    saved = []
    cur = x
    for W, m in zip(Ws, masks):
        Z = oracle.fc_fwd(cur, W, nt)
        fw = oracle.norm_fwd_train(Z, one, zero, zero, one, *HYPER, True, nt)
        q = oracle.act_fwd(ACT["ISRLU"], fw["out"], nt)
        y = oracle.dropout_fwd(0, q, m, scale, nt)
        saved.append((cur, Z, fw, q, y))
        cur = oracle.identity_add(cur, y, nt)
    out = cur
    g = dOut
    dWs, dgs = [], []
    for (xin, Z, fw, q, y), W, m in zip(reversed(saved), reversed(Ws), reversed(masks)):
        if bwd_masked:
            dN = oracle.act_bwd(ACT["ISRLU"], fw["out"], q, oracle.dropout_fwd(0, g, m, scale, nt), nt)
        else:
            dN = oracle.act_bwd(ACT["ISRLU"], fw["out"], y, g, nt)
        bw = oracle.norm_bwd(fw["mean"], fw["std"], one, fw["r"], Z, fw["xhat"], dN, renorm=True, nthreads=nt)
        dXb = oracle.fc_bwd_dx(bw["dx"], W, nthreads=nt)
        dW, _ = oracle.fc_bwd_dw(xin, bw["dx"], with_bias=False, nthreads=nt)
        g = oracle.identity_add(g, dXb, nt)
        dWs.append(dW); dgs.append(bw["dgamma"])
    return out, g, dWs[::-1], dgs[::-1]


@pytest.mark.parametrize("bwd_masked", [False, True])
def test_config4_residual_blocks_reduced_against_oracle(dl, oracle, pkg, bwd_masked):
    rng = np.random.default_rng(4)
    nblk, H, B, keep = 4, 256, 128, 0.9
    x = rng.standard_normal((B, H)).astype(np.float32)
    lim = np.sqrt(6.0 / (2 * H))
    Ws = [rng.uniform(-lim, lim, (H, H)).astype(np.float32) for _ in range(nblk)]
    masks = [(rng.uniform(size=(B, H)) < keep).astype(np.uint8) for _ in range(nblk)]
    dOut = rng.standard_normal((B, H)).astype(np.float32)
    nt = oracle.max_threads()
    oo, og, odW, odg = residual_oracle(oracle, x, Ws, masks, dOut, keep, bwd_masked, nt)
    go, gg, gdW, gdg, _ = residual_gpu(dl, pkg, dev(x), [dev(w) for w in Ws], [dev(m, torch.uint8) for m in masks],
                                       dev(dOut), keep, bwd_masked)
    assert_close(host(go), oo, TR, "output of the last block")
    # ISRLU's derivative is continuous, so no element needs to be excluded; the error budget grows with depth
    assert_close(host(gg), og, 4 * TR, "gradient with respect to the input")
    for i in range(nblk):
        assert_close(host(gdW[i]), odW[i], 4 * TR, f"dW block {i}")
        assert_close(host(gdg[i]), odg[i], 4 * TR, f"dgamma block {i}")


def test_config4_residual_blocks_full_size_float64(dl, pkg):
    """16 blocks, width 2048, batch 1024, dropout p=0.1 with a uint8 [16,1024,2048]
    mask: the GPU pipeline against the same formulas in float64 (torch on the
    GPU), masked backward."""
    torch.manual_seed(44)
    nblk, H, B, keep = 16, 2048, 1024, 0.9
    x = torch.randn(B, H, device="cuda")
    lim = float(np.sqrt(6.0 / (2 * H)))
    Ws = [(torch.rand(H, H, device="cuda") * 2 - 1) * lim for _ in range(nblk)]
    mask = (torch.rand(nblk, B, H, device="cuda") < keep).to(torch.uint8)
    dOut = torch.randn(B, H, device="cuda")
    go, gg, gdW, gdg, gdb = residual_gpu(dl, pkg, x, Ws, [mask[i] for i in range(nblk)], dOut, keep, True)
    scale = float(np.float32(1) / np.float32(keep))
    m_, eps, rmax, dmax = HYPER
    cur = x.double()
    saved = []
    for i in range(nblk):
        Z = cur @ Ws[i].double().T
        mu = Z.mean(0); sd = ((Z * Z).mean(0) - mu * mu + eps).sqrt()
        mm = m_ * mu; ms = 1 + m_ * (sd - 1)
        r = (sd / ms).clamp(1 / rmax, rmax); d = ((mu - mm) / ms).clamp(-dmax, dmax)
        xh = (Z - mu) / sd * r + d
        q = torch.where(xh < 0, xh / (1 + xh * xh).sqrt(), xh)
        mk = mask[i].double() * scale
        saved.append((cur, Z, mu, sd, r, xh, q, mk))
        cur = cur + q * mk
    assert_close(host(go), host(cur), 4 * TR, "output of block 16")
    g = dOut.double()
    for i in reversed(range(nblk)):
        xin, Z, mu, sd, r, xh, q, mk = saved[i]
        dn = g * mk * torch.where(xh < 0, (q / xh) ** 3, torch.ones_like(xh))
        dmu = (dn * (-r / sd)).sum(0); dsd = (dn * (Z - mu) * (-r / (sd * sd))).sum(0)
        dZ = dn * (r / sd) + dsd * ((Z - mu) / (B * sd)) + dmu / B
        if i in (0, nblk - 1):
            assert_close(host(gdW[i]), host(dZ.T @ xin), 8 * TR, f"dW block {i}")
            assert_close(host(gdg[i]), host((dn * xh).sum(0)), 8 * TR, f"dgamma block {i}")
            assert_close(host(gdb[i]), host(dn.sum(0)), 8 * TR, f"dbeta block {i}")
        g = g + dZ @ Ws[i].double()
    assert_close(host(gg), host(g), 8 * TR, "gradient with respect to the input")


def test_config5_tall_skinny_full_size_against_oracle(dl, oracle, pkg):
    rng = np.random.default_rng(5)
    B, K, H = 65536, 256, 256
    X = rng.standard_normal((B, K), dtype=np.float32)
    X[rng.random((B, K)) < 0.01] *= 50
    lim = np.sqrt(6.0 / (K + H))
    W = rng.uniform(-lim, lim, (H, K)).astype(np.float32)
    gamma = rng.uniform(.8, 1.2, H).astype(np.float32); beta = rng.uniform(-.1, .1, H).astype(np.float32)
    dY = rng.standard_normal((B, H), dtype=np.float32)
    zero, one = np.zeros(H, np.float32), np.ones(H, np.float32)
    a = ACT["LEAKY_RELU"]
    nt = oracle.max_threads()
    Zo = oracle.fc_fwd(X, W, nt)
    fw = oracle.norm_fwd_train(Zo, gamma, beta, zero, one, *HYPER, True, nt)
    dY[np.abs(fw["out"]) < 1e-5] = 0  # leaky ReLU's derivative jumps at 0
    yo = oracle.act_fwd(a, fw["out"], nt)
    dN = oracle.act_bwd(a, fw["out"], yo, dY, nt)
    bw = oracle.norm_bwd(fw["mean"], fw["std"], gamma, fw["r"], Zo, fw["xhat"], dN, renorm=True, nthreads=nt)
    dXo = oracle.fc_bwd_dx(bw["dx"], W, nthreads=nt)
    dWo, _ = oracle.fc_bwd_dw(X, bw["dx"], with_bias=False, nthreads=nt)

    desc = pkg.Dlmi.desc(a, renorm=True, momentum=HYPER[0], eps=HYPER[1], r_max=HYPER[2], d_max=HYPER[3])
    dXd, dWd = dev(X), dev(W)
    mm, ms = dev(zero), dev(one)
    Z, y, st = dl.fc_norm_act_fwd(desc, dXd, dWd, dev(gamma), dev(beta), mm, ms)
    dg, db = dev(zero), dev(zero)
    dZ = dl.fused_bwd(desc, Z, dev(gamma), dev(beta), st, dev(dY), dg, db)
    dX = dl.fc_bwd_dx(dZ, dWd)
    dW, _ = dl.fc_bwd_dw(dXd, dZ)
    assert_close(host(Z), Zo, TR, "Z")
    assert_close(host(st["mean"]), fw["mean"], TR, "mean", floor=1.0)
    assert_close(host(st["std"]), fw["std"], TR, "std")
    assert_close(host(y), yo, TR, "y")
    assert_close(host(dZ), bw["dx"], TR, "dZ")
    assert_close(host(dg), bw["dgamma"], TR, "dgamma")
    assert_close(host(db), bw["dbeta"], TR, "dbeta")
    assert_close(host(dX), dXo, TR, "dX")
    assert_close(host(dW), dWo, TR, "dW (split-K over the batch)")
    # inference-mode forward with given moving statistics ("variance" consumed as a standard deviation)
    mvm = rng.uniform(-1, 1, H).astype(np.float32); mvs = rng.uniform(.5, 2, H).astype(np.float32)
    yi = oracle.act_fwd(a, oracle.norm_fwd_infer(Zo, gamma, beta, mvm, mvs, nt), nt)
    assert_close(host(dl.fused_infer(desc, Z, dev(gamma), dev(beta), dev(mvm), dev(mvs))), yi, TE, "inference")
