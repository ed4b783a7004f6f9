"""The facade's Dropout_Bernoulli against tests/golden/masks.npz (compiled reference, seeded
generator): the same masks, call after call, and the device copy is the one the forward pass uses."""
import numpy as np
import pytest

from oracle.binding import ACT, DROP, NORM, STATE
from test_oracle_masks import load_masks_golden, mask_case

pytestmark = pytest.mark.gpu


def test_gpu_dropout_bernoulli_against_golden(pkg):
    from deep_learning_amd.model import Model
    g, c = load_masks_golden(), mask_case()
    M = Model(pkg.load_library(), c["widths"])
    try:
        for l, (kind, keep) in c["dropout"].items():
            M.set_layer(l, ACT["RELU"], NORM["NONE"], DROP[kind], keep)
        M.set_layer(len(c["widths"]) - 1, ACT["SOFTMAX"])
        M.prepare(4)
        for l in c["dropout"]:
            assert np.array_equal(M.dropout_mask(l, c["widths"][l]), g[f"mask_initial_L{l}"])
        for call in range(2):
            M.dropout_bernoulli(c["seed"] if call == 0 else None)
            for l in c["dropout"]:
                assert np.array_equal(M.dropout_mask(l, c["widths"][l]), g[f"mask_call{call}_L{l}"]), (call, l)
        # the forward pass in TRAINING state drops exactly the units of the installed mask
        rng = np.random.default_rng(0)
        p = M.get_parameters()
        p[:] = rng.uniform(0.05, 0.3, p.size)  # positive weights and inputs: every kept ReLU unit is > 0
        M.set_parameters(p)
        M.step(STATE["TRAINING"], rng.uniform(0.1, 1, (4, c["widths"][0])).astype(np.float32), None, backward=False)
        out1 = M.layer_buffer(1, 3)
        assert np.array_equal(out1 != 0, np.broadcast_to(g["mask_call1_L1"].astype(bool), out1.shape))
    finally:
        M.close()
