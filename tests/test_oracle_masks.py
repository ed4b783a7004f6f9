"""Dropout mask resampling (Model::Dropout_Bernoulli, bernoulli_st.cpp:27-100) against
tests/golden/masks.npz, which the compiled reference wrote from a seeded generator:
the numpy restatement in oracle/init_oracle.py reproduces every mask, and the fixture
shows the reference's own rules (inverted-Bernoulli layers are never resampled, a keep
probability of 0 clears the mask, the generator runs on across calls)."""
import json
import os

import numpy as np

from conftest import ROOT
from oracle import init_oracle


def load_masks_golden():
    g = np.load(os.path.join(ROOT, "tests", "golden", "masks.npz"), allow_pickle=False)
    return {k: g[k] for k in g.files}


def mask_case():
    c = json.loads(bytes(load_masks_golden()["mask_case_json"]))
    c["dropout"] = {int(k): tuple(v) for k, v in c["dropout"].items()}
    return c


def test_numpy_restatement_reproduces_the_masks():
    g, c = load_masks_golden(), mask_case()
    units = {l: c["widths"][l] for l in c["dropout"]}
    masks = {l: g[f"mask_initial_L{l}"].copy() for l in c["dropout"]}
    stream = init_oracle.BernoulliStream(c["seed"])
    for call in range(2):
        init_oracle.dropout_bernoulli(stream, units, c["dropout"], masks)
        for l in c["dropout"]:
            assert np.array_equal(masks[l], g[f"mask_call{call}_L{l}"]), (call, l)


def test_what_the_reference_does_with_each_kind():
    g, c = load_masks_golden(), mask_case()
    for l, (kind, keep) in c["dropout"].items():
        assert g[f"mask_initial_L{l}"].all(), "masks are allocated all ones (allocate.cpp:182-193)"
        if kind == "BERNOULLI_INVERTED":
            assert g[f"mask_call0_L{l}"].all() and g[f"mask_call1_L{l}"].all(), "never resampled"
        elif keep == 0:
            assert not g[f"mask_call0_L{l}"].any()
        else:
            m0, m1 = g[f"mask_call0_L{l}"], g[f"mask_call1_L{l}"]
            assert 0 < m0.sum() < m0.size and not np.array_equal(m0, m1), "the stream runs on across calls"


def test_keep_fraction_converges():
    """Law of large numbers on the restated stream: the kept fraction of 200 000 draws is within
    four standard deviations of p."""
    for p in (0.1, 0.5, 0.9):
        m = init_oracle.BernoulliStream(7).draw(200_000, p)
        assert abs(m.mean() - p) < 4 * np.sqrt(p * (1 - p) / m.size)
