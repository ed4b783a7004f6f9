"""The single-launch (column panel) normalization kernels (forward: 1024 - 8192 rows, backward: 2048 - 8192 rows; the
other backward cases below run the multi-launch kernels in both contexts) against the multi-launch path of the same library
and against the oracle: same per-unit arithmetic, the batch summed in 32 chunks instead of <= 16, so the two
paths agree to rounding of the column sums (1e-6 relative on the statistics), not bit for bit.  A context
created with DLMI_NORM_PANEL=0 never takes the panel path; that is the twin here."""
import os

import numpy as np
import pytest
import torch

from helpers import assert_close
from oracle.binding import ACT, DROP

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def twins(pkg):
    os.environ["DLMI_NORM_PANEL"] = "0"
    try:
        plain = pkg.Dlmi(0)
    finally:
        del os.environ["DLMI_NORM_PANEL"]
    panel = pkg.Dlmi(0)
    yield panel, plain
    panel.close()
    plain.close()


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.ascontiguousarray(a), dtype=dtype, device="cuda")


def make(B, H, seed):
    rng = np.random.default_rng(seed)
    s = rng.uniform(0.5, 2.0, H).astype(np.float32)
    m = rng.uniform(-1, 1, H).astype(np.float32)
    x = (rng.standard_normal((B, H)).astype(np.float32) * s + m).astype(np.float32)
    return dict(x=x, gamma=rng.uniform(.8, 1.2, H).astype(np.float32), beta=rng.uniform(-.1, .1, H).astype(np.float32),
                mm=rng.uniform(-.2, .2, H).astype(np.float32), ms=rng.uniform(.6, 1.6, H).astype(np.float32),
                dy=rng.standard_normal((B, H)).astype(np.float32), short=rng.standard_normal((B, H)).astype(np.float32),
                emask=(rng.uniform(size=(B, H)) < 0.9).astype(np.uint8), umask=(rng.uniform(size=H) < 0.8).astype(np.uint8))


def run_fwd(dl, pkg, d, act, drop, per_element, shortcut, renorm=True):
    desc = pkg.Dlmi.desc(ACT[act], renorm=renorm, dropout=DROP[drop], mask_per_element=per_element, momentum=0.9, eps=1e-5,
                         r_max=3.0, d_max=5.0, drop_scale=float(np.float32(1) / np.float32(0.9)))
    mask = None if drop == "NONE" else dev(d["emask"] if per_element else d["umask"], torch.uint8)
    mm, ms = dev(d["mm"]), dev(d["ms"])
    y, st = dl.fused_fwd(desc, dev(d["x"]), dev(d["gamma"]), dev(d["beta"]), mm, ms, mask=mask,
                         shortcut=dev(d["short"]) if shortcut else None)
    dl.synchronize()
    out = {k: v.cpu().numpy() for k, v in st.items()}
    out.update(y=y.cpu().numpy(), mov_mean=mm.cpu().numpy(), mov_std=ms.cpu().numpy())
    return out, desc, mask, st


CASES = [  # B, H, act, dropout, per element, shortcut
    (1024, 1024, "RELU", "NONE", False, False),
    (1024, 2048, "ISRLU", "BERNOULLI_INVERTED", True, True),    # a block of workload c4
    (2048, 1024, "ELU", "BERNOULLI", False, False),              # per-unit mask
    (2048, 3072, "TANH", "NONE", False, True),
    (4096, 1024, "SELU", "NONE", False, False),
    (4096, 2048, "LEAKY_RELU", "BERNOULLI_INVERTED", True, False),
    (8192, 1024, "ELU", "NONE", False, False),
    (8192, 2048, "SIGMOID", "BERNOULLI", False, False),
]


@pytest.mark.parametrize("B,H,act,drop,per_element,shortcut", CASES)
def test_forward_panel_equals_multi_launch_to_rounding(twins, pkg, B, H, act, drop, per_element, shortcut):
    panel, plain = twins
    d = make(B, H, B + H)
    a, *_ = run_fwd(panel, pkg, d, act, drop, per_element, shortcut)
    b, *_ = run_fwd(plain, pkg, d, act, drop, per_element, shortcut)
    for k in ("mean", "std", "mov_mean", "mov_std", "r", "d"):
        assert_close(a[k], b[k], 2e-6, f"{k} [{B}x{H}]")
    assert_close(a["y"], b["y"], 1e-5, f"y [{B}x{H}]", floor=1.0)


def test_forward_panel_against_float64(twins, pkg):
    """4096 x 1024, batch renormalization + SELU: the closed form in float64."""
    panel, _ = twins
    B, H = 4096, 1024
    d = make(B, H, 5)
    a, *_ = run_fwd(panel, pkg, d, "SELU", "NONE", False, False)
    x = d["x"].astype(np.float64)
    mean = x.mean(0)
    std = np.sqrt((x * x).mean(0) - mean * mean + 1e-5)
    mm = d["mm"] + 0.9 * (mean - d["mm"])
    ms = d["ms"] + 0.9 * (std - d["ms"])
    r = np.clip(std / ms, 1 / 3.0, 3.0)
    dd = np.clip((mean - mm) / ms, -5.0, 5.0)
    n = d["gamma"] * ((x - mean) / std * r + dd) + d["beta"]
    al, sc = 1.6732632423543772, 1.0507009873554805
    y = sc * np.where(n > 0, n, al * np.expm1(n))
    assert_close(a["mean"], mean, 2e-6, "mean")
    assert_close(a["std"], std, 2e-6, "std")
    assert_close(a["mov_mean"], mm, 2e-6, "moving mean")
    assert_close(a["mov_std"], ms, 2e-6, "moving std")
    assert_close(a["r"], r, 2e-6, "r")
    assert_close(a["d"], dd, 1e-5, "d", floor=1.0)
    assert_close(a["y"], y, 1e-5, "y", floor=1.0)


def test_forward_panel_is_reproducible_and_leaves_no_state(twins, pkg):
    """Same bits on every call (fixed summation order), also after a call of another shape in between: the
    barrier words are back at zero when a launch ends."""
    panel, _ = twins
    d = make(2048, 1024, 9)
    first, *_ = run_fwd(panel, pkg, d, "ELU", "NONE", False, False)
    other = make(1024, 2048, 10)
    run_fwd(panel, pkg, other, "RELU", "NONE", False, False)
    for _ in range(3):
        again, *_ = run_fwd(panel, pkg, d, "ELU", "NONE", False, False)
        for k in first:
            assert np.array_equal(first[k], again[k]), k


def test_shapes_outside_the_panel_geometry_take_the_multi_launch_path(twins, pkg):
    """Batches that are not 1024 / 2048 / 4096 / 8192 rows or widths that are not multiples of 1024: bit-identical
    results from both contexts, because both run the same kernels."""
    panel, plain = twins
    for B, H in [(1536, 1024), (1024, 1536), (512, 1024), (4096, 1000)]:
        d = make(B, H, B * 3 + H)
        a, *_ = run_fwd(panel, pkg, d, "ELU", "NONE", False, False)
        b, *_ = run_fwd(plain, pkg, d, "ELU", "NONE", False, False)
        for k in a:
            assert np.array_equal(a[k], b[k]), (B, H, k)


def run_bwd(dl, pkg, d, desc, mask, st):
    B, H = d["x"].shape
    dg, db = torch.full((H,), 0.25, device="cuda"), torch.full((H,), -0.5, device="cuda")  # they accumulate
    dx = dl.fused_bwd(desc, dev(d["x"]), dev(d["gamma"]), dev(d["beta"]), st, dev(d["dy"]), dg, db, mask=mask)
    dl.synchronize()
    return dict(dx=dx.cpu().numpy(), dgamma=dg.cpu().numpy(), dbeta=db.cpu().numpy())


@pytest.mark.parametrize("B,H,act,drop,per_element,shortcut", CASES)
def test_backward_panel_equals_multi_launch_to_rounding(twins, pkg, B, H, act, drop, per_element, shortcut):
    panel, plain = twins
    d = make(B, H, B + H + 1)
    # both backward passes start from the SAME forward results (the multi-launch context's)
    _, desc, mask, st = run_fwd(plain, pkg, d, act, drop, per_element, False)
    a = run_bwd(panel, pkg, d, desc, mask, st)
    b = run_bwd(plain, pkg, d, desc, mask, st)
    assert_close(a["dx"], b["dx"], 1e-4, f"dX [{B}x{H}]", floor=1.0)
    assert_close(a["dgamma"], b["dgamma"], 1e-4, "dgamma", floor=1.0)
    assert_close(a["dbeta"], b["dbeta"], 1e-4, "dbeta", floor=1.0)


ALL_ACTS = ["LINEAR", "RELU", "LEAKY_RELU", "ELU", "SELU", "ISRLU", "SIGMOID", "TANH"]


@pytest.mark.parametrize("act", ALL_ACTS)
@pytest.mark.parametrize("B,per_element", [(2048, False), (2048, True), (4096, False), (4096, True)])
def test_every_backward_panel_kernel_variant(twins, pkg, B, per_element, act):
    """The backward panel kernel issues its loads as explicit instructions behind explicit waits, which the
    compiler cannot check: every compiled variant (activation x rows per thread x with / without the per-element
    mask stream) is therefore run against the multi-launch kernels, over several panels per XCD."""
    panel, plain = twins
    H = 1536 if B == 2048 else 1024  # 3 and 2 panels of 64 columns per XCD (4 with the 32-column variant)
    d = make(B, H, B + len(act))
    drop = "BERNOULLI_INVERTED" if per_element else "NONE"
    _, desc, mask, st = run_fwd(plain, pkg, d, act, drop, per_element, False)
    a = run_bwd(panel, pkg, d, desc, mask, st)
    b = run_bwd(plain, pkg, d, desc, mask, st)
    assert_close(a["dx"], b["dx"], 1e-4, f"dX [{B}x{H}] {act}", floor=1.0)
    assert_close(a["dgamma"], b["dgamma"], 1e-4, "dgamma", floor=1.0)
    assert_close(a["dbeta"], b["dbeta"], 1e-4, "dbeta", floor=1.0)
    again = run_bwd(panel, pkg, d, desc, mask, st)
    for k in a:
        assert np.array_equal(a[k], again[k]), f"{k}: not reproducible"


@pytest.mark.parametrize("B,H", [(4096, 1024), (8192, 1536)])
def test_backward_panel_against_float64(twins, pkg, B, H):
    """Batch renormalization + ELU (64-column panels at 4096 rows, 32-column panels at 8192): dX, dgamma, dbeta from
    the closed form in float64, and the invariant that r-corrected batch normalization removes the column mean of dX."""
    panel, _ = twins
    d = make(B, H, 6)
    a, desc, mask, st = run_fwd(panel, pkg, d, "ELU", "NONE", False, False)
    g = run_bwd(panel, pkg, d, desc, mask, st)
    x, dy = d["x"].astype(np.float64), d["dy"].astype(np.float64)
    mean, std, r, dd = (a[k].astype(np.float64) for k in ("mean", "std", "r", "d"))
    xh = (x - mean) / std * r + dd
    n = d["gamma"] * xh + d["beta"]
    keep = np.abs(n) > 1e-4  # the derivative of ELU jumps at 0: leave the few elements within rounding of it out
    # the reference's ELU derivative for n < 0 is the activation value itself, alpha * (exp(n) - 1), not
    # alpha * exp(n) (v1/ops/activations/functions.hpp:92): the kernels keep that
    dn = dy * np.where(n > 0, 1.0, np.expm1(n)) * keep
    # the GPU sees the same zeros
    dyk = (dy * keep).astype(np.float32)
    d2 = dict(d, dy=dyk)
    g = run_bwd(panel, pkg, d2, desc, mask, st)
    e = dn * d["gamma"]
    dmean = (e * (-r / std)).sum(0)
    dstd = (e * (x - mean) * (-r / std ** 2)).sum(0)
    dx = e * (r / std) + dstd * (x - mean) / (B * std) + dmean / B
    assert_close(g["dx"], dx, 1e-4, "dX", floor=1.0)
    assert_close(g["dgamma"], 0.25 + (dn * xh).sum(0), 1e-4, "dgamma", floor=1.0)
    assert_close(g["dbeta"], -0.5 + dn.sum(0), 1e-4, "dbeta", floor=1.0)
    assert np.max(np.abs(g["dx"].astype(np.float64).sum(0))) < 1e-2  # sum_b dX = 0 up to rounding of B terms


def test_a_destroyed_stream_is_not_touched_by_the_next_launch(twins, pkg):
    """Launches of different streams are ordered through the stream of the previous launch.  A model owns its
    stream and destroys it when it is closed: the next launch, from another stream, must not look at it."""
    from deep_learning_amd.model import Model
    from oracle.binding import NORM, STATE
    panel, _ = twins
    M = Model(pkg.load_library(), [64, 1024, 4])
    M.set_layer(1, ACT["RELU"], NORM["BRN"])
    M.set_layer(2, ACT["SOFTMAX"])
    M.set_norm_hyper(0.99, 1e-5, 3.0, 5.0)
    M.prepare(1024)
    M.glorot_uniform(1)
    rng = np.random.default_rng(0)
    Y = np.zeros((1024, 4), np.float32)
    Y[:, 0] = 1.0
    M.step(STATE["TRAINING"], rng.standard_normal((1024, 64), dtype=np.float32), Y)  # [1024 x 1024]: a panel launch
    M.close()
    d = make(1024, 1024, 3)
    a, *_ = run_fwd(panel, pkg, d, "RELU", "NONE", False, False)
    assert np.isfinite(a["y"]).all()


def test_panel_kernels_beside_another_kernel(twins, pkg):
    """A product on another stream holds compute units while a panel kernel starts, so some of its workgroups
    begin late.  A workgroup counts itself in for panel p+1 before it waits for panel p; with one running
    arrival total the ones ahead could complete the count for p on their own, and a late workgroup's sums were
    read before it had stored them.  Arrivals are counted per panel parity now: the results beside a running
    product must be those of a quiet device, bit for bit."""
    panel, _ = twins
    B, H = 4096, 2048
    d = make(B, H, 77)
    quiet_f, desc, mask, st = run_fwd(panel, pkg, d, "ELU", "NONE", False, False)
    quiet_b = run_bwd(panel, pkg, d, desc, mask, st)
    side = torch.cuda.Stream()
    other = pkg.Dlmi(0)
    other.set_stream(side)
    X = torch.randn(4096, 4096, device="cuda")
    W = torch.randn(4096, 4096, device="cuda") * 0.01
    Z = torch.empty(4096, 4096, device="cuda")
    torch.cuda.synchronize()
    try:
        for _ in range(4):
            for _ in range(3):
                other.fc_fwd(X, W, None, out=Z)  # 256 x 256 tiles: every compute unit held for about 0.5 ms each
            busy_f, desc2, mask2, st2 = run_fwd(panel, pkg, d, "ELU", "NONE", False, False)
            for _ in range(3):
                other.fc_fwd(X, W, None, out=Z)
            busy_b = run_bwd(panel, pkg, d, desc, mask, st)
            torch.cuda.synchronize()
            for k in quiet_f:
                assert np.array_equal(quiet_f[k], busy_f[k]), k
            for k in quiet_b:
                assert np.array_equal(quiet_b[k], busy_b[k]), k
    finally:
        torch.cuda.synchronize()
        other.close()


# ---------------------------------------------------------------- the bounded wait's give-up branch
def spin_limited(pkg, limit=64):
    os.environ["DLMI_PANEL_SPIN_LIMIT"] = str(limit)
    try:
        return pkg.Dlmi(0)
    finally:
        del os.environ["DLMI_PANEL_SPIN_LIMIT"]


def test_a_give_up_is_reported_once_and_the_context_falls_back(twins, pkg):
    """The give-up branch, driven from the host so that every kernel still exits normally: one rank ticket of
    XCD 0 is taken before the launch, so one of that XCD's 32 workgroups is told it is the 33rd and leaves at
    once, and the count of the other 31 can never complete; with a spin limit of 64 polls they give up within
    microseconds.  The synchronization after the call reports it, once; the context then runs the multi-launch
    kernels (same bits as a context that never had the panel path), and its barrier words are back at zero."""
    _, plain = twins
    ctx = spin_limited(pkg)
    try:
        assert ctx.norm_panel_enabled()
        d = make(4096, 1024, 21)
        good, *_ = run_fwd(ctx, pkg, d, "ELU", "NONE", False, False)  # a normal panel launch first
        ctx.norm_panel_poke(0, 0, 1)
        with pytest.raises(pkg.DlmiError, match="gave up"):
            run_fwd(ctx, pkg, d, "ELU", "NONE", False, False)
        assert not ctx.norm_panel_enabled()
        ctx.synchronize()  # reported once
        again, desc, mask, st = run_fwd(ctx, pkg, d, "ELU", "NONE", False, False)
        want, *_ = run_fwd(plain, pkg, d, "ELU", "NONE", False, False)
        for k in want:
            assert np.array_equal(again[k], want[k]), k
        for k in ("mean", "std", "r", "d"):
            assert_close(again[k], good[k], 2e-6, k)
        # backward: also the multi-launch kernels now
        a = run_bwd(ctx, pkg, d, desc, mask, st)
        b = run_bwd(plain, pkg, d, desc, mask, st)
        for k in a:
            assert np.array_equal(a[k], b[k]), k
    finally:
        ctx.close()


def test_a_launch_that_finds_stale_barrier_words_is_reported(pkg):
    """What a give-up leaves behind (tickets beyond 32) makes every workgroup of a later launch leave at once.
    That launch says so through the host word, so the call is reported like the give-up itself."""
    ctx = spin_limited(pkg)
    try:
        d = make(2048, 1024, 22)
        for x in range(8):
            ctx.norm_panel_poke(x, 0, 32)
        with pytest.raises(pkg.DlmiError, match="not valid"):
            run_fwd(ctx, pkg, d, "RELU", "NONE", False, False)
        assert not ctx.norm_panel_enabled()
        a, *_ = run_fwd(ctx, pkg, d, "RELU", "NONE", False, False)
        assert np.isfinite(a["y"]).all()
    finally:
        ctx.close()


def test_a_give_up_inside_a_model_fails_the_step_and_the_next_one_is_right(pkg):
    """Through the facade: the step whose normalization kernel gave up returns false (every read of results
    waits through the context), the model then matches a twin that never used the panel kernels, bit for bit."""
    import ctypes
    from deep_learning_amd.model import Model
    from oracle.binding import NORM, STATE
    lib = pkg.load_library()
    lib.dlmi_model_context.restype = ctypes.c_void_p

    def build(env):
        os.environ.update(env)
        try:
            M = Model(lib, [64, 1024, 4])
        finally:
            for k in env:
                del os.environ[k]
        M.set_layer(1, ACT["ELU"], NORM["BRN"])
        M.set_layer(2, ACT["SOFTMAX"])
        M.set_norm_hyper(0.99, 1e-5, 3.0, 5.0)
        M.prepare(2048)
        M.glorot_uniform(1)
        return M

    M, T = build({"DLMI_PANEL_SPIN_LIMIT": "64"}), build({"DLMI_NORM_PANEL": "0"})
    try:
        rng = np.random.default_rng(3)
        X = rng.standard_normal((2048, 64), dtype=np.float32)
        Y = np.eye(4, dtype=np.float32)[rng.integers(0, 4, 2048)]
        ctx = ctypes.c_void_p(lib.dlmi_model_context(M.h))
        assert lib.dlmi_ctx_norm_panel_enabled(ctx) == 1
        assert lib.dlmi_ctx_norm_panel_poke(ctx, ctypes.c_uint(0), ctypes.c_uint(0), ctypes.c_uint(1)) == 0
        with pytest.raises(RuntimeError, match="gave up"):
            M.step(STATE["TRAINING"], X, Y)
        assert lib.dlmi_ctx_norm_panel_enabled(ctx) == 0
        # start both from the same state again
        for m in (M, T):
            m.clear_training_arrays()
            mv = m.get_moving()
            m.set_moving(np.zeros_like(mv[0]), np.ones_like(mv[1]))
            m.step(STATE["TRAINING"], X, Y)
        assert np.array_equal(np.array(M.get_dparams()), np.array(T.get_dparams()))
        assert np.array_equal(np.array(M.layer_buffer(2, 3)), np.array(T.layer_buffer(2, 3)))
    finally:
        M.close()
        T.close()


def test_recorded_panel_kernels_keep_other_streams_on_the_multi_launch_path(twins, pkg):
    """A panel kernel recorded into a HIP graph runs whenever the graph is replayed, where no event of this
    library can order it against panel kernels of other streams.  The stream that records one therefore becomes
    the only stream of the device that launches them: another context's call, on another stream, takes the
    multi-launch kernels (bit-identical to a context without the panel path) while the graph's owner lives, and
    every replay - with eager work of both contexts between the replays - gives the eager result."""
    _, plain = twins
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    owner, other = pkg.Dlmi(0), pkg.Dlmi(0)
    try:
        owner.set_stream(s1)
        other.set_stream(s2)
        B, H = 2048, 1024
        d = make(B, H, 31)
        desc = pkg.Dlmi.desc(ACT["ELU"], renorm=True, momentum=0.9, eps=1e-5, r_max=3.0, d_max=5.0)
        x, ga, be = dev(d["x"]), dev(d["gamma"]), dev(d["beta"])
        y = torch.empty(B, H, device="cuda")
        st = {k: torch.empty(H, device="cuda") for k in ("mean", "std", "r", "d")}
        mm0, ms0 = dev(d["mm"]), dev(d["ms"])
        mm, ms = mm0.clone(), ms0.clone()
        torch.cuda.synchronize()
        with torch.cuda.stream(s1):
            owner.fused_fwd(desc, x, ga, be, mm, ms, out=y, stats=st)  # eager: a panel launch
        owner.synchronize()
        eager = dict(y=y.cpu().numpy(), mean=st["mean"].cpu().numpy(), mov_mean=mm.cpu().numpy())
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s1):
            owner.fused_fwd(desc, x, ga, be, mm, ms, out=y, stats=st)
        for _ in range(3):
            mm.copy_(mm0)
            ms.copy_(ms0)
            y.zero_()
            torch.cuda.synchronize()
            g.replay()
            # the other stream's call while the owner's graph may be running: multi-launch kernels
            with torch.cuda.stream(s2):
                a, *_ = run_fwd(other, pkg, d, "ELU", "NONE", False, False)
            torch.cuda.synchronize()
            owner.synchronize()
            assert np.array_equal(y.cpu().numpy(), eager["y"])
            assert np.array_equal(st["mean"].cpu().numpy(), eager["mean"])
            assert np.array_equal(mm.cpu().numpy(), eager["mov_mean"])
            b, *_ = run_fwd(plain, pkg, d, "ELU", "NONE", False, False)
            for k in a:
                assert np.array_equal(a[k], b[k]), k
        del g
    finally:
        torch.cuda.synchronize()
        owner.close()
        other.close()
