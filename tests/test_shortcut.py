"""Zero-padded identity shortcut of a residual block and the routing of its
gradient (Forward_Pass__Zero_Padded_Identity__*, fwp_st.cpp:5051-5112;
Backward_Pass__Residual__* / __Identity__*, bwp_st.cpp:1047-1068, 1112-1175):
oracle and GPU leaves against tests/golden/shortcut.npz (compiled reference) and
against the slicing the definition amounts to."""
import os

import numpy as np
import pytest

from conftest import ROOT


def golden():
    g = np.load(os.path.join(ROOT, "tests", "golden", "shortcut.npz"), allow_pickle=False)
    return {k: g[k] for k in g.files}


def case_ids():
    return list(range(len(golden()["shortcut_cases"])))


def by_slicing(a, b, g, da0, db0, pad):
    """The leaves written with numpy slices: the wider operand, plus the narrower
    one at column offset pad; each operand's gradient is its window of g."""
    HA, HB = a.shape[1], b.shape[1]
    wide, narrow = (a, b) if HA >= HB else (b, a)
    out = wide.copy()
    out[:, pad:pad + narrow.shape[1]] += narrow
    win = lambda H: g if H == g.shape[1] else g[:, pad:pad + H]
    return out, da0 + win(HA), db0 + win(HB)


@pytest.mark.parametrize("nt", [0, 3])
@pytest.mark.parametrize("ci", case_ids())
def test_oracle_shortcut_against_golden(oracle, ci, nt):
    g = golden()
    B, HA, HB, pad = (int(v) for v in g["shortcut_cases"][ci])
    a, b, gr, da0, db0 = (g[f"sc{ci}_{k}"] for k in ("a", "b", "g", "da0", "db0"))
    assert np.array_equal(oracle.zero_padded_identity_fwd(a, b, pad, nt), g[f"sc{ci}_t{nt}_out"])
    assert np.array_equal(oracle.residual_bwd(gr, da0, pad, nt), g[f"sc{ci}_t{nt}_da"])
    assert np.array_equal(oracle.residual_bwd(gr, db0, pad, nt), g[f"sc{ci}_t{nt}_db"])


@pytest.mark.parametrize("ci", case_ids())
def test_golden_shortcut_is_window_arithmetic(ci):
    g = golden()
    B, HA, HB, pad = (int(v) for v in g["shortcut_cases"][ci])
    out, da, db = by_slicing(*(g[f"sc{ci}_{k}"] for k in ("a", "b", "g", "da0", "db0")), pad)
    assert np.array_equal(out, g[f"sc{ci}_t0_out"])
    assert np.array_equal(da, g[f"sc{ci}_t0_da"])
    assert np.array_equal(db, g[f"sc{ci}_t0_db"])


@pytest.mark.gpu
@pytest.mark.parametrize("ci", case_ids())
def test_gpu_shortcut_against_golden(dl, ci):
    import torch
    g = golden()
    B, HA, HB, pad = (int(v) for v in g["shortcut_cases"][ci])
    dev = lambda x: torch.from_numpy(np.ascontiguousarray(x)).cuda()
    a, b, gr = dev(g[f"sc{ci}_a"]), dev(g[f"sc{ci}_b"]), dev(g[f"sc{ci}_g"])
    out = dl.zero_padded_identity_fwd(a, b, pad)
    assert np.array_equal(out.cpu().numpy(), g[f"sc{ci}_t0_out"])  # one rounding per element: bit-exact
    da = dl.residual_bwd(gr, dev(g[f"sc{ci}_da0"]), pad)
    db = dl.residual_bwd(gr, dev(g[f"sc{ci}_db0"]), pad)
    assert np.array_equal(da.cpu().numpy(), g[f"sc{ci}_t0_da"])
    assert np.array_equal(db.cpu().numpy(), g[f"sc{ci}_t0_db"])


@pytest.mark.gpu
def test_gpu_shortcut_large_and_refusals(dl):
    import torch
    torch.manual_seed(3)
    a, b = torch.randn(1024, 2048, device="cuda"), torch.randn(1024, 1536, device="cuda")
    out = dl.zero_padded_identity_fwd(a, b, 256)
    exp = a.clone()
    exp[:, 256:256 + 1536] += b
    assert torch.equal(out, exp)
    gr = torch.randn(1024, 2048, device="cuda")
    db = torch.zeros(1024, 1536, device="cuda")
    dl.residual_bwd(gr, db, 256)
    assert torch.equal(db, gr[:, 256:256 + 1536])
    with pytest.raises(RuntimeError):
        dl.zero_padded_identity_fwd(a, b, 1024)  # 1024 + 1536 > 2048: does not fit
    with pytest.raises(RuntimeError):
        dl.zero_padded_identity_fwd(a, b, 0)     # no padding needs equal widths
