"""dlmi_fused_norm_act_fwd_noalloc (the entry point that allocates nothing: its reduction partials
live in a fixed array inside the library's code object) against dlmi_fused_norm_act_fwd, through the
C ABI, on two calls in a row, the second on a smaller input.

Both entry points launch the same kernels with the same geometry; only where the partial sums are
kept differs, so the results must agree bit for bit - which is well inside the path's tolerance
(1e-5 element-wise, 1e-4 after the column reductions)."""
import numpy as np
import pytest
import torch

from helpers import RTOL_REDUCED as TR
from helpers import assert_close

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.as_tensor(np.ascontiguousarray(a)).cuda().contiguous()


def host(t):
    return t.detach().cpu().numpy()


def run_both(dl, pkg, B, H, act, seed, unit_mask):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((B, H)) * rng.uniform(.5, 2, H) + rng.uniform(-1, 1, H)).astype(np.float32)
    gamma = rng.uniform(.8, 1.2, H).astype(np.float32)
    beta = rng.uniform(-.1, .1, H).astype(np.float32)
    mm, ms = rng.uniform(-.5, .5, H).astype(np.float32), rng.uniform(.5, 2, H).astype(np.float32)
    mask = dev((rng.uniform(size=H) < 0.8).astype(np.uint8)) if unit_mask else None
    desc = pkg.Dlmi.desc(pkg.ACT[act], renorm=True, momentum=0.9, eps=1e-5, r_max=3.0, d_max=5.0,
                         dropout=pkg.DROP["BERNOULLI_INVERTED"] if unit_mask else 0, drop_scale=1.25)
    xd, gd, bd = dev(x), dev(gamma), dev(beta)
    out = {}
    for name, noalloc in (("alloc", False), ("noalloc", True)):
        m, s = dev(mm), dev(ms)
        y = torch.empty((B, H), device="cuda")
        st = {k: torch.empty(H, device="cuda") for k in ("mean", "std", "r", "d")}
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info()[0]
        dl.fused_fwd(desc, xd, gd, bd, m, s, mask=mask, out=y, stats=st, noalloc=noalloc)
        torch.cuda.synchronize()
        free1 = torch.cuda.mem_get_info()[0]
        if noalloc:
            assert free1 == free0, "the call changed the device's free memory: it allocated"
        out[name] = dict(y=host(y), mov_mean=host(m), mov_std=host(s), **{k: host(v) for k, v in st.items()})
    return out


@pytest.mark.parametrize("act", ["SELU", "RELU"])
def test_noalloc_entry_matches_the_allocating_one_twice_in_a_row(dl, pkg, act):
    # the second call is smaller, takes the scalar path (H % 4 != 0) and finds the first call's
    # partial sums still in the array
    for B, H, seed, unit_mask in ((1500, 1024, 1, False), (333, 250, 2, True)):
        o = run_both(dl, pkg, B, H, act, seed, unit_mask)
        for k, v in o["alloc"].items():
            assert np.all(np.isfinite(v)), k
            assert_close(o["noalloc"][k], v, 1e-5 if k == "y" else TR, f"[{B}x{H}] {k}", floor=1.0)
            assert np.array_equal(o["noalloc"][k], v), f"[{B}x{H}] {k}: same kernels, same geometry, yet not identical"


def test_noalloc_entry_on_single_launch_shapes(dl, pkg):
    """A few thousand rows: the allocating entry point runs the single-launch panel kernel, whose chunk
    partials need 384 bytes per unit.  The entry point that allocates nothing runs the same kernel while
    they fit its fixed array (bit-identical then) and the multi-launch kernels beyond (same tolerance as
    any two summation orders)."""
    o = run_both(dl, pkg, 2048, 1024, "ELU", 5, True)
    for k, v in o["alloc"].items():
        assert np.array_equal(o["noalloc"][k], v), k
    o = run_both(dl, pkg, 1024, 8192, "ELU", 6, False)   # 3 MiB of panel partials: more than the array
    for k, v in o["alloc"].items():
        assert np.all(np.isfinite(v)), k
        assert_close(o["noalloc"][k], v, 1e-5 if k == "y" else TR, f"[1024x8192] {k}", floor=1.0)


def test_noalloc_entry_never_touches_the_context_scratch(pkg):
    """On a context of its own, whose scratch block nothing has grown yet: the block's generation and the
    device's free memory stay what they were across calls of every kernel family.  (Each shape is called once
    before the measured call: the first launch of a kernel makes the HIP runtime load that kernel's code object
    into device memory, once per process, which is the loader's doing and not the call's.)"""
    import ctypes
    d = pkg.Dlmi(0)
    try:
        d.lib.dlmi_ctx_scratch_generation.restype = ctypes.c_ulonglong
        gen0 = d.lib.dlmi_ctx_scratch_generation(d.ctx)
        desc = pkg.Dlmi.desc(pkg.ACT["RELU"], renorm=True)
        for B, H in ((4096, 4096), (64, 65536), (8192, 1024), (100, 36)):
            x = torch.randn((B, H), device="cuda")
            v = lambda: torch.ones(H, device="cuda")
            args = (desc, x, v(), v() * 0, v() * 0, v())
            kw = dict(out=torch.empty_like(x), stats={k: v() for k in ("mean", "std", "r", "d")}, noalloc=True)
            d.fused_fwd(*args, **kw)
            torch.cuda.synchronize()
            free0 = torch.cuda.mem_get_info()[0]
            d.fused_fwd(*args, **kw)
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free0, (B, H)
            assert d.lib.dlmi_ctx_scratch_generation(d.ctx) == gen0, (B, H)
            assert torch.isfinite(kw["out"]).all()
    finally:
        d.close()


def test_noalloc_entry_refuses_more_units_than_its_array_holds(dl, pkg):
    H = 65536 + 4
    desc = pkg.Dlmi.desc(pkg.ACT["RELU"])
    x = torch.zeros((2, H), device="cuda")
    v = lambda: torch.ones(H, device="cuda")
    with pytest.raises(pkg.DlmiError, match="exceed"):
        dl.fused_fwd(desc, x, v(), v(), v(), v(), out=torch.empty_like(x),
                     stats={k: v() for k in ("mean", "std", "r", "d")}, noalloc=True)
    # the limit itself is accepted, and the context stays usable
    H = 65536
    x = torch.randn((8, H), device="cuda")
    a = dl.fused_fwd(desc, x, v(), v() * 0, v() * 0, v(), noalloc=True)[0]
    b = dl.fused_fwd(desc, x, v(), v() * 0, v() * 0, v(), noalloc=False)[0]
    assert torch.equal(a, b)


def test_noalloc_calls_from_two_streams_are_ordered(pkg):
    """Every call on one GPU uses the same fixed array.  Calls from two contexts on two streams, issued
    alternately without any host wait, would trample each other's partial sums; the library makes a call from
    another stream than the previous one wait (on the device) for that one.  Results: those of each input alone."""
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    a, b = pkg.Dlmi(0), pkg.Dlmi(0)
    try:
        a.set_stream(s1)
        b.set_stream(s2)
        desc = pkg.Dlmi.desc(pkg.ACT["ELU"], renorm=True, momentum=0.9)
        H = 8192  # multi-launch kernels: statistics, finalize and apply all go through the array
        rng = np.random.default_rng(4)
        xs = [dev(rng.standard_normal((300 + 40 * i, H)).astype(np.float32) * (1 + i)) for i in range(6)]
        one, zero = torch.ones(H, device="cuda"), torch.zeros(H, device="cuda")

        def call(ctx, x):
            y = torch.empty_like(x)
            st = {k: torch.empty(H, device="cuda") for k in ("mean", "std", "r", "d")}
            ctx.fused_fwd(desc, x, one, zero, zero.clone(), one.clone(), out=y, stats=st, noalloc=True)
            return y, st

        torch.cuda.synchronize()
        want = []
        for x in xs:
            with torch.cuda.stream(s1):
                want.append(call(a, x))
            torch.cuda.synchronize()
        for _ in range(5):
            got = []
            for i, x in enumerate(xs):  # alternating streams, nothing waits on the host
                with torch.cuda.stream(s1 if i % 2 == 0 else s2):
                    got.append(call(a if i % 2 == 0 else b, x))
            torch.cuda.synchronize()
            for (y, st), (yw, sw) in zip(got, want):
                assert torch.equal(y, yw)
                assert torch.equal(st["mean"], sw["mean"]) and torch.equal(st["std"], sw["std"])
    finally:
        torch.cuda.synchronize()
        a.close()
        b.close()
