"""dlmi_fused_norm_act_bwd_db: the fused backward that also forms the bias gradient db[j] = sum_b dX[b, j] in the
pass that writes dX.  dgamma and dbeta must be bit-identical to the plain call and dX equal to the last place or
two (the two apply kernels are separate instantiations, in which the compiler may contract the same expression
into fused multiply-adds differently); db must be the column sums of the dX this call stored (float32 sums in another order than numpy's: compared with the float64 sums to the rounding of B terms),
on every path: multi-launch and single-launch panel kernels (the by-product: per-block / per-workgroup partial sums and
one small launch), tall tensors, mini-batch kernels and ragged widths (a pass over dX after them), with and without
accumulation."""
import numpy as np
import pytest
import torch

from helpers import assert_close
from oracle.binding import ACT, DROP

pytestmark = pytest.mark.gpu

CASES = [  # B, H, activation, dropout, per element
    (8192, 512, "ELU", "NONE", False),        # multi-launch, folded finalize
    (65536, 256, "LEAKY_RELU", "NONE", False),  # tall: finalize kernels
    (2048, 1024, "SELU", "NONE", False),      # single-launch panel kernel, 64-column panels, 2 rows per thread
    (4096, 1536, "TANH", "NONE", False),      # ... 4 rows per thread, 3 panels per XCD
    (8192, 1024, "SIGMOID", "NONE", False),   # ... 32-column panels
    (4096, 1024, "LEAKY_RELU", "BERNOULLI_INVERTED", True),  # ... with the per-element mask stream
    (128, 512, "RELU", "NONE", False),        # mini-batch kernel
    (1000, 250, "TANH", "NONE", False),       # ragged width: no 16-byte path
    (3000, 768, "ISRLU", "BERNOULLI_INVERTED", True),
    (4096, 1024, "ELU", "BERNOULLI", False),
]


@pytest.mark.parametrize("B,H,act,drop,per_element", CASES)
@pytest.mark.parametrize("accumulate", [False, True])
def test_bias_gradient_by_product(dl, pkg, B, H, act, drop, per_element, accumulate):
    rng = np.random.default_rng(B + 7 * H)
    dev = lambda a: torch.as_tensor(np.ascontiguousarray(a), device="cuda")
    x = dev((rng.standard_normal((B, H)) * rng.uniform(.5, 2, H) + rng.uniform(-1, 1, H)).astype(np.float32))
    gamma, beta = dev(rng.uniform(.8, 1.2, H).astype(np.float32)), dev(rng.uniform(-.1, .1, H).astype(np.float32))
    dY = dev(rng.standard_normal((B, H)).astype(np.float32))
    mask = None
    if drop != "NONE":
        mask = dev((rng.uniform(size=(B, H) if per_element else H) < 0.9).astype(np.uint8))
    desc = pkg.Dlmi.desc(ACT[act], renorm=True, dropout=DROP[drop], mask_per_element=per_element, momentum=0.9,
                         drop_scale=float(np.float32(1) / np.float32(0.9)))
    _, st = dl.fused_fwd(desc, x, gamma, beta, torch.zeros(H, device="cuda"), torch.ones(H, device="cuda"), mask=mask)
    dg0, db0 = rng.standard_normal(H).astype(np.float32), rng.standard_normal(H).astype(np.float32)
    bias0 = rng.standard_normal(H).astype(np.float32)
    dg_a, dbeta_a = dev(dg0), dev(db0)
    dX_a = dl.fused_bwd(desc, x, gamma, beta, st, dY, dg_a, dbeta_a, mask=mask)
    dg_b, dbeta_b, db = dev(dg0), dev(db0), dev(bias0)
    dX_b = dl.fused_bwd(desc, x, gamma, beta, st, dY, dg_b, dbeta_b, mask=mask, db=db, accumulate_db=accumulate)
    dl.synchronize()
    assert torch.equal(dg_a, dg_b) and torch.equal(dbeta_a, dbeta_b)
    assert_close(dX_b.cpu().numpy(), dX_a.cpu().numpy(), 1e-6, "dX", floor=1.0)
    dx = dX_b.cpu().numpy().astype(np.float64)
    want = dx.sum(0) + (bias0 if accumulate else 0.0)
    # a float32 sum of B terms: error at most a few ulp of the sum of |terms|
    bound = 4 * np.finfo(np.float32).eps * (np.abs(dx).sum(0) + np.abs(bias0)) * max(1.0, np.log2(B))
    assert np.all(np.abs(db.cpu().numpy() - want) <= bound + 1e-30)
    # reproducible
    db2 = dev(bias0)
    dl.fused_bwd(desc, x, gamma, beta, st, dY, dev(dg0), dev(db0), mask=mask, db=db2, accumulate_db=accumulate)
    assert torch.equal(db, db2)
