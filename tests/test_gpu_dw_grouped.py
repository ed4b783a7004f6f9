"""dlmi_fc_bwd_dw_grouped: the weight gradients of several layers in one launch per kernel variant.  Every
product is computed by the same tile code in the same order as by dlmi_fc_bwd_dw, so the results must be
bit-identical to the one-by-one calls, whatever the mix of shapes (grouped variants, products that go alone:
ragged, split over K, narrow), with and without accumulation and bias gradients; and equal to the oracle."""
import numpy as np
import pytest
import torch

from helpers import RTOL_REDUCED as TR
from helpers import assert_close

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.as_tensor(np.ascontiguousarray(a), device="cuda")


def problems(shapes, seed):
    rng = np.random.default_rng(seed)
    out = []
    for B, K, H in shapes:
        out.append(dict(X=rng.standard_normal((B, K)).astype(np.float32), dZ=rng.standard_normal((B, H)).astype(np.float32),
                        dW0=rng.standard_normal((H, K)).astype(np.float32), db0=rng.standard_normal(H).astype(np.float32)))
    return out


MIXES = {
    # four equal layers of a residual stack (one group of 128 x 128 tiles) and two more of another variant
    "equal layers": [(1024, 512, 512)] * 4 + [(512, 256, 256)] * 2,
    # different shapes of ONE variant share a launch; a ragged layer, a narrow output layer and a product that is
    # split over K go alone
    "mixed": [(256, 512, 256), (256, 256, 512), (128, 784, 512), (128, 512, 10), (8192, 128, 128), (256, 512, 256)],
    "single": [(512, 256, 256)],
    # the layers of a network on a mini-batch: the products of any width share one launch of the mini-batch kernel
    # (ragged blocks, a batch that is no multiple of four among them); the first narrow layer (the output layer, with
    # its bias gradient) rides along in that launch, a second one goes alone
    "mini-batch": [(128, 784, 512), (128, 512, 512), (128, 512, 10), (100, 36, 24), (255, 64, 64), (128, 512, 512),
                   (77, 130, 16)],
    # one hidden layer and the output layer: one launch for both
    "mini-batch pair": [(128, 784, 512), (128, 512, 10)],
    # more mini-batch products than one launch of their kernel holds (8), and a narrow layer with the first launch
    "mini-batch many": [(64, 64, 64)] * 9 + [(64, 64, 3)],
}


@pytest.mark.parametrize("name", sorted(MIXES))
@pytest.mark.parametrize("accumulate", [False, True])
@pytest.mark.parametrize("with_bias", [False, True])
def test_grouped_equals_one_by_one(dl, oracle, name, accumulate, with_bias):
    ps = problems(MIXES[name], len(name))
    one, grp = [], []
    for p in ps:
        X, dZ = dev(p["X"]), dev(p["dZ"])
        dWa, dba = dev(p["dW0"]), dev(p["db0"]) if with_bias else None
        dl.fc_bwd_dw(X, dZ, dW=dWa, db=dba, accumulate=accumulate)
        one.append((dWa, dba))
        grp.append((X, dZ, dev(p["dW0"]), dev(p["db0"]) if with_bias else None))
    dl.fc_bwd_dw_grouped(grp, accumulate=accumulate)
    dl.synchronize()
    nt = oracle.max_threads()
    for p, (dWa, dba), (_, _, dWg, dbg) in zip(ps, one, grp):
        assert torch.equal(dWa, dWg), (name, p["X"].shape, p["dZ"].shape)
        if with_bias:
            assert torch.equal(dba, dbg)
        dWo, dbo = oracle.fc_bwd_dw(p["X"], p["dZ"], dW_init=p["dW0"] if accumulate else None,
                                    db_init=p["db0"] if accumulate else None, nthreads=nt)
        assert_close(dWg.cpu().numpy(), dWo, TR, "dW")
        if with_bias:
            assert_close(dbg.cpu().numpy(), dbo, TR, "db")


def test_more_problems_than_one_launch_holds(dl):
    """40 equal products: two launches of the group kernel (32 + 8)."""
    ps = problems([(256, 128, 128)] * 40, 3)
    grp = [(dev(p["X"]), dev(p["dZ"]), torch.empty(128, 128, device="cuda"), None) for p in ps]
    dl.fc_bwd_dw_grouped(grp)
    for p, (X, dZ, dWg, _) in zip(ps, grp):
        want, _ = dl.fc_bwd_dw(X, dZ)
        assert torch.equal(want, dWg)
