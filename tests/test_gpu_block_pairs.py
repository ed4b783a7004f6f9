"""The loss / accuracy sums of the seed-gradient kernels (one pair per block, added in block order by the block that
draws the last ticket: csrc/block_pairs.hpp) on batches of many blocks, launch after launch on one context - the ticket
word must be back at zero after every launch -, and the strip-streaming measurement aid."""
import numpy as np
import pytest
import torch

from oracle.binding import ACCU, ACT, LOSS

pytestmark = pytest.mark.gpu


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.ascontiguousarray(a)).to("cuda", dtype=dtype).contiguous()


@pytest.mark.parametrize("B,H", [(1, 10), (4, 3), (5, 10), (1000, 10), (4099, 7), (70001, 4)])
def test_softmax_seed_sums_over_many_blocks(dl, B, H):
    rng = np.random.default_rng(B + H)
    z = rng.standard_normal((B, H))
    q = np.exp(z - z.max(1, keepdims=True))
    q = (q / q.sum(1, keepdims=True)).astype(np.float32)
    target = rng.integers(0, H, B)
    y = np.eye(H, dtype=np.float32)[target]
    qc = np.clip(q.astype(np.float64), 1e-7, 1 - 1e-7)
    loss = -np.log(qc[np.arange(B), target].astype(np.float32).astype(np.float64)).sum()
    # ">=" scan: the last maximal index wins
    correct = float((H - 1 - np.argmax(q[:, ::-1], axis=1) == target).sum())
    stats = torch.zeros(2, dtype=torch.float64, device="cuda")
    first = None
    for launch in range(1, 4):  # the sums accumulate; a ticket that was not reset would leave a launch without its sum
        dl.softmax_ce_seed(dev(q), dev(y), stats)
        got = stats.cpu().numpy()
        assert got[1] == launch * correct, f"launch {launch}: accuracy count {got[1]} != {launch * correct}"
        assert abs(got[0] - launch * loss) <= 1e-6 * launch * abs(loss) + 1e-9, f"launch {launch}: loss {got[0]} vs {launch * loss}"
        if first is None:
            first = got.copy()
    # bit-reproducible: a fresh accumulator gets the first launch's sums again
    again = torch.zeros(2, dtype=torch.float64, device="cuda")
    dl.softmax_ce_seed(dev(q), dev(y), again)
    assert np.array_equal(again.cpu().numpy(), first)


@pytest.mark.parametrize("B,H", [(3, 5), (2049, 16), (30000, 3)])
def test_regression_seed_sums_over_many_blocks(dl, B, H):
    rng = np.random.default_rng(B * H)
    z = rng.standard_normal((B, H)).astype(np.float32)
    y = rng.standard_normal((B, H)).astype(np.float32)
    stats = torch.zeros(2, dtype=torch.float64, device="cuda")
    for launch in range(1, 4):
        dl.loss_seed(LOSS["MSE"], ACCU["DISTANCE"], 0.5, ACT["LINEAR"], dev(z), dev(z), dev(y), stats)
        got = stats.cpu().numpy()
        d = z.astype(np.float64) - y.astype(np.float64)
        want_loss = launch * (np.float32(1) * (z - y) * (z - y)).astype(np.float64).sum()
        want_acc = launch * float((np.abs(z - y) <= np.float32(0.5)).sum())
        assert got[1] == want_acc
        assert abs(got[0] - want_loss) <= 1e-6 * want_loss, (got[0], want_loss, (d * d).sum())


def test_strip_stream_probe_copies_and_adds(dl):
    B, H = 4096, 1024
    x = torch.randn(B, H, device="cuda")
    x2 = torch.randn(B, H, device="cuda")
    y = torch.empty(B, H, device="cuda")
    dl.probe_strip_stream(x, y)
    assert torch.equal(y, x)
    dl.probe_strip_stream(x, y, x2=x2)
    assert torch.equal(y, x + x2)
    with pytest.raises(Exception):
        dl.probe_strip_stream(x[:1000].contiguous(), y[:1000].contiguous())  # B not a multiple of 4096
    with pytest.raises(Exception):
        dl.probe_strip_stream(torch.randn(4096, 500, device="cuda"), torch.empty(4096, 500, device="cuda"))
