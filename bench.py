"""Benchmark of the fully-connected + batch-renorm + activation hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|c1|c2|c3|c4|c5] [--report FILE]

The default run times workload c3 (configuration 3 of the benchmark: the one the metric is quoted on) as the
headline and the other four configurations under detail.workloads, each with its step time, the roofline
of its dominant kernels and the reference's CPU path timed beside it.

A "step" is one forward + backward pass over one synthetic batch resident in HBM.  Every input tensor
is drawn ONCE on the host from a seeded mt19937_64 stream of its own (oracle/harness_rng.c) and the same
bits go to the GPU and to the CPU baseline; the GPU results of the first step are checked in the run
against that CPU pass and both against a float64 evaluation of the same arithmetic on row / column slabs.

Prints ONE compact JSON line on stdout (short keys, numbers to five digits: the whole line stays below
6 KB): samples/s of the whole step, the roofline of the dominant kernel (fp32 MFMA GEMM), the HBM roofline of
the fused normalization + activation kernels, the CPU baseline measured on the host cores (the compiled
reference's OpenMP leaves when oracle/_ref is present, else this repository's restatement of them) and the
parity figures.  The unabridged figures (every timing, every tensor's errors) go to stderr as a second JSON
object and, with --report, to a file.

--steps / --warmup govern the headline workload.  The side workloads always take as many steps as make a
sustained load (an idle GPU's clock needs about 15 ms of it) and report the counts they used.
"""
import os

# The CPU baseline's protocol: threads bound to cores, neighbours first.  Set before any OpenMP runtime is
# loaded (numpy's, torch's, the baseline library's), which is when they are read.
os.environ.setdefault("OMP_PROC_BIND", "close")
os.environ.setdefault("OMP_PLACES", "cores")

import argparse  # noqa: E402
import json  # noqa: E402
import sys  # noqa: E402
import time  # noqa: E402

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "FC+BRN+act fwd+bwd samples/sec; % HBM peak (norm/act), % FP32 MFMA peak (GEMM)"
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_FP32_PEAK_TFLOPS = 157.3  # MI355X dense FP32 matrix
HYPER = dict(momentum=0.99, eps=1e-5, r_max=3.0, d_max=5.0)

LAYER_WORKLOADS = {
    # name: (B, K, H, activation, description)
    "c3": (8192, 4096, 4096, "ELU", "FC 4096->4096, batch 8192, BRN + ELU, fwd+bwd (dX,dW,db,dgamma,dbeta)"),
    "c2": (4096, 0, 4096, "SELU", "BRN + SELU fwd+bwd on [4096 x 4096]"),
    "c5": (65536, 256, 256, "LEAKY_RELU", "FC 256->256, batch 65536, BRN + leaky ReLU, fwd+bwd (+ inference fwd)"),
}

# HBM-side bytes per launch (sequence) from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this file's --only
# parts, calibrated against the plain copy of --only copy.  Hardware counters cannot be read from inside this
# process: these are the figures of the committed profile, tied to a digest of the kernel sources at the time
# the counters were read (`python bench.py --traffic-digest` prints the current one).  When a source has
# changed since, `traffic` is null instead of a figure that may no longer hold.
MIB = 1024.0 * 1024.0
TRAFFIC_PROFILE = "profiles/hbm_traffic_pmc.md"
MEASURED_TRAFFIC_BYTES = {
    "c3": {"gemm": (898.0 + 898.4 + 832.8) / 3.0 * MIB, "norm_act": (259.1 + 388.4) * MIB},
    "c2": {"norm_act": 326.8 * MIB},
    "c4": {"gemm": (72.5 + 72.1 + 64.1) / 3.0 * MIB, "norm_act": 73.6 * MIB},
    "c5": {"gemm": (132.1 + 132.3 + 144.1 + 16.3) / 3.0 * MIB, "norm_act": 513.6 * MIB},
}
TRAFFIC_SOURCES = ("gemm_f32_mfma.hip", "norm_kernels.hip", "norm_panel_fwd.hip", "norm_panel_bwd.hip",
                   "norm_panel_common.hpp", "norm_shared.hpp", "activations.hpp")
TRAFFIC_SOURCES_SHA256 = "3f8482c1a956161b8b809770a17f35365877b6bd5396f7d78e2b73a29270ba20"


def traffic_sources_digest():
    import hashlib
    h = hashlib.sha256()
    for name in TRAFFIC_SOURCES:
        with open(os.path.join(ROOT, "deep-learning_amd", "csrc", name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()


def measured_traffic(workload, key):
    """The profile's figure while the kernels are the measured ones, else None."""
    v = MEASURED_TRAFFIC_BYTES.get(workload, {}).get(key)
    if v is None or traffic_sources_digest() != TRAFFIC_SOURCES_SHA256:
        return None
    return v


# ---------------------------------------------------------------- helpers
def host_info():
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            model = next(l.split(":", 1)[1].strip() for l in f if l.startswith("model name"))
    except Exception:
        pass
    ncpu = os.cpu_count() or 1
    # the reference's default is every processor (update_size.cpp:76, pct_threads = 100); the GPU box hands a
    # job a share of the host and says so through OMP_NUM_THREADS
    share = int(os.environ.get("OMP_NUM_THREADS", "0")) or ncpu
    return model, ncpu, max(1, min(share, ncpu, 64))


def cpu_engine():
    from oracle.binding import Oracle, Reference, reference_available
    kind = "reference" if reference_available() else "port"
    return kind, (Reference() if kind == "reference" else Oracle())


def rel_errors(got, exp):
    """(max |got-exp| / max(|exp|, rms(exp)), max |got-exp| / max(|exp|, 1e-6 max|exp|)): the tolerance the
    parity tests assert behind reductions and GEMMs, and the strict per-element metric (chunked: the
    largest tensors are 128 MiB)."""
    import numpy as np
    g = np.asarray(got).ravel()
    e = np.asarray(exp).ravel()
    if e.size == 0:
        return 0.0, 0.0
    step = 1 << 22
    ss, mx = 0.0, 0.0
    for i in range(0, e.size, step):
        c = e[i:i + step].astype(np.float64)
        ss += float(np.dot(c, c))
        mx = max(mx, float(np.max(np.abs(c))))
    rms = max((ss / e.size) ** 0.5, 1e-30)
    floor = max(1e-6 * mx, 1e-300)
    a = b = 0.0
    for i in range(0, e.size, step):
        c = e[i:i + step].astype(np.float64)
        d = np.abs(g[i:i + step].astype(np.float64) - c)
        ac = np.abs(c)
        a = max(a, float(np.max(d / np.maximum(ac, rms))))
        b = max(b, float(np.max(d / np.maximum(ac, floor))))
    return a, b


def parity_block(pairs, limit, f64=None, extra=None, ref_rms_floor=None):
    """pairs: name -> (gpu array, cpu array).  The rms-floored error must meet `limit` (1e-4 behind
    reductions and GEMMs, as the parity tests assert); the strict per-element error is reported beside it.
    f64: name -> (gpu slab, its float64 target, cpu slab, its float64 target): the arbitration of the strict
    metric on the same elements (the two targets differ only where a stage is evaluated on each side's own
    inputs).  Reported: the strict error of each side against float64 (`gpu`, `ref`: maxima, i.e. the error of
    whichever element cancels most, divided by that element) and `rms_ratio`, the largest ratio over the
    tensors of the GPU's root-mean-square error against float64 to the CPU baseline's.  `ok` is judged on the
    ratio (at most 2): the two maxima are single-element errors, whose quotient scatters by more than that
    between two summation orders of equal accuracy.
    ref_rms_floor: name -> rms error of the reference's OTHER summation order for that tensor (its single-thread
    leaf, where the timed baseline is its OpenMP path): the baseline error of the ratio is the larger of the two,
    so the GPU is asked to be no worse than the reference's less accurate own order (`f64.baseline` says which
    tensors took it).
    Returns (compact block for the line, per-tensor block for the report)."""
    full, ok, worst = {}, True, ("", 0.0, 0.0)
    for k, (g, e) in pairs.items():
        a, b = rel_errors(g, e)
        full[k] = {"max_rel_err": a, "max_rel_err_strict": b}
        ok = ok and a <= limit
        if a >= worst[1]:
            worst = (k, a, b)
    out = {"tol": limit, "ok": ok, "max_rel_err": worst[1], "worst": worst[0],
           "max_rel_err_strict": max(v["max_rel_err_strict"] for v in full.values())}
    if f64:
        import numpy as np
        rms = lambda a: float(np.sqrt(np.mean(np.square(np.asarray(a, np.float64)))))
        g_max, r_max, ratio, worst64, floored = 0.0, 0.0, 0.0, "", []
        for k, (g, xg, e, xe) in f64.items():
            eg, er = rel_errors(g, xg)[1], rel_errors(e, xe)[1]
            rg, rr = rms(np.asarray(g, np.float64) - xg), rms(np.asarray(e, np.float64) - xe)
            floor = (ref_rms_floor or {}).get(k, 0.0)
            if floor > rr:
                floored.append(k)
            q = rg / max(rr, floor, 1e-7 * rms(xg), 1e-300)  # a baseline that is exact leaves the float's own rounding
            full.setdefault(k, {}).update({"strict_gpu_vs_f64": eg, "strict_ref_vs_f64": er, "rms_err_gpu_vs_f64": rg,
                                           "rms_err_ref_vs_f64": rr})
            g_max, r_max = max(g_max, eg), max(r_max, er)
            if q >= ratio:
                ratio, worst64 = q, k
        out["f64"] = {"gpu": g_max, "ref": r_max, "rms_ratio": ratio, "worst": worst64, "ok": ratio <= 2.0}
        if floored:
            out["f64"]["baseline"] = "single-thread order for " + ",".join(floored)
    if extra:
        out.update(extra)
    return out, full


# The engine clock of an idle GPU takes about 15 ms of sustained load to reach its working point: a 70 us
# kernel timed over 20 back-to-back calls reads 10-12 % slower than over 2000.  Timed regions shorter than
# this are therefore repeated until they are a sustained load (the step counts used are reported).
SUSTAINED_MS = 40.0


def time_events(torch, fn, reps, warmup=2, min_ms=SUSTAINED_MS):
    """Average duration (ms) of fn() over at least `reps` back-to-back calls, measured with HIP events recorded
    on the stream the kernels are launched on.  A region shorter than `min_ms` is measured again with as many
    calls as fill `min_ms`, after as many untimed ones."""
    def region(n):
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(n):
            fn()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / n

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ms = region(reps)
    if ms * reps >= min_ms:
        return ms
    n = int(min_ms / max(ms, 1e-4)) + 1
    region(n)
    return region(n)


def sustained_steps(torch, fn):
    """(steps, warmup) of a side workload: enough of both for a sustained load."""
    ms = time_wall(torch, fn, 5, 2)
    return max(20, int(1.5 * SUSTAINED_MS / ms) + 1), max(3, int(SUSTAINED_MS / ms) + 1)


def time_wall(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e3


def median_time(fn, reps, warmup=1):
    """Median wall time (s) of fn() over `reps` calls after `warmup` untimed ones."""
    for _ in range(warmup):
        fn()
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[len(ts) // 2]


def gave_up(*contexts):
    """Waits for every context's stream the way a caller of the library does; True when a single-launch
    normalization kernel gave up its bounded wait since the last check (the timings are then not valid)."""
    from deep_learning_amd import DlmiError
    bad = False
    for c in contexts:
        try:
            c.synchronize()
        except DlmiError:
            bad = True
    return bad


def rnd(x, digits=5):
    """Numbers to `digits` significant digits, recursively (the line's size)."""
    if isinstance(x, float):
        return float("%.*g" % (digits, x)) if x == x and abs(x) != float("inf") else None
    if isinstance(x, dict):
        return {k: rnd(v, digits) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return [rnd(v, digits) for v in x]
    return x


def line(value, ms, steps, warmup, config, roof, hbm, cpu, detail, parity, report):
    out = {"metric": METRIC, "value": value, "unit": "samples/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
           "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
           "data": "synthetic", "config": config, "roofline": roof}
    if hbm is not None:
        out["roofline_norm_act"] = hbm
    out["cpu_baseline"] = cpu
    out["parity"] = parity
    out["detail"] = detail
    out["_report"] = report  # unabridged figures: stripped from the line, printed to stderr
    return out


# ---------------------------------------------------------------- c2, c3, c5: one layer
def layer_inputs(name):
    """Host tensors of a layer workload, one seeded stream per tensor."""
    import numpy as np
    from oracle.binding import HarnessRng
    B, K, H, act, _ = LAYER_WORKLOADS[name]
    rng = HarnessRng(1234 + {"c2": 200, "c3": 300, "c5": 500}.get(name, 900))
    t = {}
    if K:
        t["X"] = rng.normal(1, (B, K))
        if name == "c5":  # 1 % of the elements are outliers x 50
            t["X"] = np.where(rng.uniform(2, (B, K)) < np.float32(0.01), t["X"] * np.float32(50), t["X"])
        lim = (6.0 / (K + H)) ** 0.5
        t["W"] = rng.uniform(3, (H, K), -lim, lim)
        t["bias"] = np.zeros(H, np.float32)
        t["gamma"] = np.ones(H, np.float32)
        t["beta"] = np.zeros(H, np.float32)
    else:
        s, m = rng.uniform(4, (H,), 0.5, 2.0), rng.uniform(5, (H,), -1.0, 1.0)
        t["Z"] = rng.normal(6, (B, H)) * s + m
        t["gamma"] = rng.uniform(7, (H,), 0.8, 1.2)
        t["beta"] = rng.uniform(8, (H,), -0.1, 0.1)
    t["dY"] = rng.normal(9, (B, H))
    t["mov_mean"] = np.zeros(H, np.float32)
    t["mov_std"] = np.ones(H, np.float32)
    if name == "c5":  # moving statistics of the inference-mode forward
        t["inf_mean"] = rng.uniform(10, (H,), -1.0, 1.0)
        t["inf_std"] = rng.uniform(11, (H,), 0.5, 2.0)  # the "variance" array holds standard deviations
    return t


def workgroup_timeline(dl, step, part):
    """Profiling aid: when the workgroups of the last product launch started and ended, by the kernel's own stamps."""
    import ctypes
    import numpy as np
    M, N, K = {"gemm_fwd": (step.B, step.H, step.K), "gemm_dx": (step.B, step.K, step.H)}.get(part, (step.H, step.K, step.B))
    tm, tn, ks, rs = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_uint(0), ctypes.c_int(0)
    sz = ctypes.c_size_t
    dl._ck(dl.lib.dlmi_gemm_plan(ctypes.c_int(dl.compute_units()), sz(M), sz(N), sz(K), ctypes.byref(tm), ctypes.byref(tn),
                                 ctypes.byref(ks), ctypes.byref(rs)))
    n = min(4096, -(-M // tm.value) * -(-N // tn.value))
    a = dl.gemm_timeline(n)
    t0 = a[:, 0].min()
    start, issued, done = ((a[:, i] - t0) / 100.0 for i in range(3))
    where = a[:, 3] >> 32 << 16 | (a[:, 3] >> 8 & 0xff)  # XCD, shader engine / array / CU
    cus = dl.compute_units()
    out = ["%s %d x %d x %d: %d workgroups of %d x %d (%d K slices) on %d CUs; first start to last acknowledged store %.1f us; "
           "tile at the matrix peak %.2f us" % (part, M, N, K, n, tm.value, tn.value, ks.value, len(set(where.tolist())),
                                                done.max(), 2.0 * tm.value * tn.value * K / ks.value / (157.3e12 / cus) * 1e6)]
    for lo in range(0, n, cus):
        sl = slice(lo, min(n, lo + cus))
        out.append("  workgroups %4d..%4d: start %5.1f / %5.1f / %5.1f us, lifetime %5.1f / %5.1f / %5.1f us (min / median / max), "
                   "last store acknowledged %.2f us after its issue"
                   % (lo, sl.stop - 1, start[sl].min(), np.median(start[sl]), start[sl].max(), (done - start)[sl].min(),
                      np.median((done - start)[sl]), (done - start)[sl].max(), np.median((done - issued)[sl])))
    return "\n".join(out)


class LayerStep:
    """The pieces of one step of a layer workload, callable separately so each can be timed."""

    def __init__(self, dl, pkg, torch, name, h):
        self.dl, self.torch = dl, torch
        self.B, self.K, self.H, act, _ = LAYER_WORKLOADS[name]
        self.desc = pkg.Dlmi.desc(pkg.ACT[act], renorm=True, **HYPER)
        dev = lambda a: torch.from_numpy(a).cuda()
        t = {k: dev(v) for k, v in h.items()}
        B, K, H = self.B, self.K, self.H
        e = lambda *s: torch.empty(*s, device="cuda")
        if K:
            t["Z"], t["dX"], t["dW"], t["db"] = e(B, H), e(B, K), e(H, K), e(H)
        t["y"], t["dZ"] = e(B, H), e(B, H)
        t["dgamma"], t["dbeta"] = torch.zeros(H, device="cuda"), torch.zeros(H, device="cuda")
        t["stats"] = {k: e(H) for k in ("mean", "std", "r", "d")}
        self.t = t

    def gemm_fwd(self):
        t = self.t
        self.dl.fc_fwd(t["X"], t["W"], t["bias"], out=t["Z"])

    def norm_fwd(self):
        t = self.t
        self.dl.fused_fwd(self.desc, t["Z"], t["gamma"], t["beta"], t["mov_mean"], t["mov_std"], out=t["y"],
                          stats=t["stats"])

    def norm_bwd(self):
        t = self.t
        self.dl.fused_bwd(self.desc, t["Z"], t["gamma"], t["beta"], t["stats"], t["dY"], t["dgamma"], t["dbeta"],
                          out=t["dZ"])

    def norm_bwd_db(self):
        """The backward of the normalization that also forms the bias gradient db = sum_b dZ while it writes dZ."""
        t = self.t
        self.dl.fused_bwd(self.desc, t["Z"], t["gamma"], t["beta"], t["stats"], t["dY"], t["dgamma"], t["dbeta"],
                          out=t["dZ"], db=t["db"])

    def gemm_dx(self):
        t = self.t
        self.dl.fc_bwd_dx(t["dZ"], t["W"], out=t["dX"])

    def gemm_dw(self):
        t = self.t
        self.dl.fc_bwd_dw(t["X"], t["dZ"], dW=t["dW"], db=t["db"])

    def gemm_dw_only(self):
        t = self.t
        self.dl.fc_bwd_dw(t["X"], t["dZ"], dW=t["dW"])

    def fc_norm_fwd(self):
        """Forward of the layer in one call: the GEMM epilogue accumulates the batch statistics, so the
        normalization reads Z only once."""
        t = self.t
        self.dl.fc_norm_act_fwd(self.desc, t["X"], t["W"], t["gamma"], t["beta"], t["mov_mean"], t["mov_std"],
                                Z=t["Z"], out=t["y"], stats=t["stats"])

    def infer_fwd(self):
        t = self.t
        self.dl.fused_infer(self.desc, t["Z"], t["gamma"], t["beta"], t["inf_mean"], t["inf_std"], out=t["y"])

    def adam(self):
        """Adam step over the layer's weights (not part of the timed step: the metric is forward + backward;
        reported under detail)."""
        t = self.t
        if "m1" not in t:
            t["m1"], t["m2"] = self.torch.zeros_like(t["W"]), self.torch.zeros_like(t["W"])
        self.dl.opt_adam(t["W"], t["dW"], t["m1"], t["m2"], None, None, 1e-6, 0.9, 0.999, 1e-8, 0.0)

    def copy(self):
        """A plain device copy of one [B, H] tensor (known size): calibrates the FETCH_SIZE / WRITE_SIZE
        counters of a rocprofv3 --pmc run."""
        self.t["y"].copy_(self.t["dY"])

    def strip_fwd(self):
        """One tensor in, one out, walked like the single-launch normalization kernels walk theirs and nothing
        else done with the data: the memory floor of the forward kernel's access pattern (measurement aid)."""
        self.dl.probe_strip_stream(self.t["dY"], self.t["y"])

    def strip_bwd(self):
        """Two tensors in, one out, same pattern: the memory floor of the backward kernel's."""
        self.dl.probe_strip_stream(self.t["dY"], self.t["dZ"], x2=self.t["y"])

    def parts(self):
        if self.K:
            return [self.fc_norm_fwd, self.norm_bwd_db, self.gemm_dx, self.gemm_dw_only]
        return [self.norm_fwd, self.norm_bwd]

    def __call__(self):
        for p in self.parts():
            p()


KINK = 1e-5  # |pre-activation| below which an activation whose derivative jumps at 0 may take either branch


class CpuLayerPass:
    """One forward + backward pass of a layer workload through the CPU baseline's OpenMP leaves, on buffers
    allocated once: a timed pass allocates nothing.  The leaves accumulate into dX, dW, dgamma and dbeta like
    the reference's, which clears those arrays first (bwp_st.cpp:96-115): the clears are part of the pass."""

    def __init__(self, name, h, rows):
        import numpy as np
        from oracle.binding import ACT, _ptr, c_f, c_int, c_sz
        self.np, self.ptr, self.c = np, _ptr, (c_int, c_sz, c_f)
        B, K, H, act, _ = LAYER_WORKLOADS[name]
        self.name, self.h, self.act = name, h, ACT[act]
        self.kind, self.eng = cpu_engine()
        self.model, self.ncpu, self.nt = host_info()
        self.B, self.K, self.H, self.Bs = B, K, H, min(B, rows)
        Bs = self.Bs
        f = lambda *s: np.empty(s, np.float32)
        b = {"xhat": f(Bs, H), "out": f(Bs, H), "y": f(Bs, H), "dN": f(Bs, H), "dZ": f(Bs, H)}
        for k in ("mean", "std", "r", "d", "mov_mean", "mov_std", "dgamma", "dbeta", "dmean", "dstd"):
            b[k] = f(H)
        if K:
            b["Z"], b["dX"], b["dW"] = f(Bs, H), f(Bs, K), f(H, K)
            self.X = np.ascontiguousarray(h["X"][:Bs])
        else:
            b["Z"] = np.ascontiguousarray(h["Z"][:Bs])
        if name == "c5":
            b["n_inf"], b["y_inference"] = f(Bs, H), f(Bs, H)
        self.b = b
        self.dY = np.ascontiguousarray(h["dY"][:Bs])

    def _call(self, leaf, *args):
        self.eng._f(leaf)(*args)

    def forward(self):
        c_int, c_sz, c_f = self.c
        p, b, h, nt, Bs, K, H = self.ptr, self.b, self.h, self.nt, self.Bs, self.K, self.H
        if K:
            self._call("fc_fwd", c_int(nt), c_sz(Bs), c_sz(K), c_sz(H), p(self.X), p(h["W"]), p(b["Z"]))
        b["mov_mean"][:] = h["mov_mean"]
        b["mov_std"][:] = h["mov_std"]
        b["r"][:] = 1.0
        b["d"][:] = 0.0
        self._call("norm_fwd_train", c_int(nt), c_int(1), c_sz(Bs), c_sz(H), c_f(HYPER["momentum"]), c_f(HYPER["eps"]),
                   c_f(HYPER["r_max"]), c_f(HYPER["d_max"]), p(b["Z"]), p(h["gamma"]), p(h["beta"]), p(b["mean"]),
                   p(b["std"]), p(b["mov_mean"]), p(b["mov_std"]), p(b["r"]), p(b["d"]), p(b["xhat"]), p(b["out"]))
        self._call("act_fwd", c_int(nt), c_int(self.act), c_sz(Bs), c_sz(H), p(b["out"]), p(b["y"]))

    def backward(self):
        c_int, c_sz, c_f = self.c
        p, b, h, nt, Bs, K, H = self.ptr, self.b, self.h, self.nt, self.Bs, self.K, self.H
        self._call("act_bwd", c_int(nt), c_int(self.act), c_sz(Bs), c_sz(H), p(b["out"]), p(b["y"]), p(self.dY), p(b["dN"]))
        b["dgamma"][:] = 0.0
        b["dbeta"][:] = 0.0
        self._call("norm_bwd", c_int(nt), c_int(1), c_sz(Bs), c_sz(H), p(b["mean"]), p(b["std"]), p(h["gamma"]), p(b["r"]),
                   p(b["Z"]), p(b["xhat"]), p(b["dN"]), p(b["dgamma"]), p(b["dbeta"]), p(b["dmean"]), p(b["dstd"]),
                   p(b["dZ"]))
        if K:
            b["dX"][:] = 0.0
            self._call("fc_bwd_dx", c_int(nt), c_sz(Bs), c_sz(H), c_sz(K), p(b["dZ"]), p(h["W"]), p(b["dX"]))
            b["dW"][:] = 0.0
            self._call("fc_bwd_dw", c_int(nt), c_sz(Bs), c_sz(K), c_sz(H), p(self.X), p(b["dZ"]), p(b["dW"]), None)

    def step(self):
        self.forward()
        self.backward()

    def inference(self):
        c_int, c_sz, _ = self.c
        p, b, h, nt = self.ptr, self.b, self.h, self.nt
        self._call("norm_fwd_infer", c_int(nt), c_sz(self.Bs), c_sz(self.H), p(b["Z"]), p(h["gamma"]), p(h["beta"]),
                   p(h["inf_mean"]), p(h["inf_std"]), p(b["n_inf"]))
        self._call("act_fwd", c_int(nt), c_int(self.act), c_sz(self.Bs), c_sz(self.H), p(b["n_inf"]), p(b["y_inference"]))

    def baseline(self, reps):
        """cpu_baseline object: one untimed pass, then the median of `reps` timed ones."""
        dt = median_time(self.step, reps, warmup=1)
        return {"value": self.Bs / dt, "unit": "samples/s", "cores": self.nt, "kind": self.kind,
                "sample": "%d of %d rows, 1 warm-up + median of %d passes" % (self.Bs, self.B, reps)}, \
               {"seconds_per_pass": dt, "host_cpu_count": self.ncpu, "cpu_model": self.model,
                "omp_proc_bind": os.environ.get("OMP_PROC_BIND"), "omp_places": os.environ.get("OMP_PLACES")}

    def results(self):
        b = self.b
        keys = ["y", "dZ", "dgamma", "dbeta", "mean", "std", "mov_mean", "mov_std"] + (["Z", "dX", "dW"] if self.K else [])
        if self.name == "c5":
            keys.append("y_inference")
        return {k: b[k] for k in keys}


def layer_f64_slabs(name, h, gpu, ref):
    """name -> (gpu slab, float64, cpu slab, float64) on 64 rows / 64 columns of a layer workload's results.  Each
    implementation's stage is evaluated in float64 on that implementation's OWN stage inputs (its Z for the
    normalization, its dZ for dX and dW), so a stage's error is not charged with the stages before it."""
    import numpy as np
    from oracle.binding import ACT, Oracle
    B, K, H, act, _ = LAYER_WORKLOADS[name]
    o64 = Oracle(np.float64)
    rows = np.arange(0, B, B // 64)[:64]
    cols = np.arange(0, H, H // 64)[:64]
    out = {}
    d = lambda a: np.asarray(a, np.float64)
    if K:
        z64 = d(h["X"][rows]) @ d(h["W"]).T
        out["Z"] = (gpu["Z"][rows], z64, ref["Z"][rows], z64)
    per_side = {}
    for side, res in (("gpu", gpu), ("ref", ref)):
        Zs = res["Z"] if K else h["Z"]
        zc = np.ascontiguousarray(d(Zs[:, cols]))
        ga, be = d(h["gamma"][cols]), d(h["beta"][cols])
        fw = o64.norm_fwd_train(zc, ga, be, d(h["mov_mean"][cols]), d(h["mov_std"][cols]), HYPER["momentum"], HYPER["eps"],
                                HYPER["r_max"], HYPER["d_max"], True)
        y = o64.act_fwd(ACT[act], fw["out"])
        dN = o64.act_bwd(ACT[act], fw["out"], y, d(h["dY"][:, cols]))
        bw = o64.norm_bwd(fw["mean"], fw["std"], ga, fw["r"], zc, fw["xhat"], dN, renorm=True)
        s = dict(y=y, dZ=bw["dx"], dgamma=bw["dgamma"], dbeta=bw["dbeta"], mean=fw["mean"], std=fw["std"])
        if K:
            s["dX"] = d(res["dZ"][rows]) @ d(h["W"])
            s["dW"] = d(res["dZ"][:, cols]).T @ d(h["X"])
        per_side[side] = s
    pick = {"y": lambda a: a[:, cols], "dZ": lambda a: a[:, cols], "dgamma": lambda a: a[cols], "dbeta": lambda a: a[cols],
            "mean": lambda a: a[cols], "std": lambda a: a[cols], "dX": lambda a: a[rows], "dW": lambda a: a[cols]}
    for k, f in pick.items():
        if k in per_side["gpu"]:
            out[k] = (f(gpu[k]), per_side["gpu"][k], f(ref[k]), per_side["ref"][k])
    return out


def dw_single_chain(h, gpu, ref, B, H, K):
    """The weight gradient sums over the batch.  The CPU baseline's OpenMP path adds one partial sum per thread
    (merge.cpp:76-100), the GPU kernel one chain over all B rows per output, like the reference's single-thread
    leaf (update_derivative_fwp_st.cpp:246-281).  On 8 units x 512 inputs: the float32 sum in the single-thread
    leaf's order (row after row into one accumulator) against float64, beside the GPU's and the OpenMP pass's."""
    import numpy as np
    units, kc = np.arange(0, H, H // 8)[:8], min(K, 512)
    rms = lambda a: float(np.sqrt(np.mean(np.square(a))))
    dz, x = ref["dZ"][:, units], h["X"][:, :kc]
    chain = np.cumsum(dz[:, :, None] * x[:, None, :], axis=0, dtype=np.float32)[-1]
    exact = dz.astype(np.float64).T @ x.astype(np.float64)
    exact_gpu = gpu["dZ"][:, units].astype(np.float64).T @ x.astype(np.float64)
    return {"rms_err_single_chain_vs_f64": rms(chain - exact), "rms_err_openmp_vs_f64": rms(ref["dW"][units][:, :kc] - exact),
            "rms_err_gpu_vs_f64": rms(gpu["dW"][units][:, :kc] - exact_gpu), "rows": B}


def run_layer(args, torch, pkg, dl, name, full):
    """One layer workload.  full: the headline run (all detail timings)."""
    import numpy as np
    B, K, H, act, descr = LAYER_WORKLOADS[name]
    h = layer_inputs(name)
    cpu_rows = 0 if args.only else (args.cpu_rows if args.cpu_rows >= 0 else B)
    cp, kinks = None, None
    if cpu_rows:
        # The CPU forward runs first: where a pre-activation lies within rounding of 0, an activation whose
        # derivative jumps there (all of these) may take the other branch on the other side, which changes
        # that element's gradient by all of itself and, through the GEMMs, a whole row of dX and dW.  The
        # upstream gradient of those few elements is set to zero for BOTH sides, as in the parity tests.
        cp = CpuLayerPass(name, h, cpu_rows)
        if cp.Bs == B:
            cp.forward()
            near = np.abs(cp.b["out"]) < KINK
            kinks = int(near.sum())
            h["dY"][near] = 0.0
            cp.dY = h["dY"]
    step = LayerStep(dl, pkg, torch, name, h)
    t = step.t

    if args.only:
        step()  # every buffer a part reads has been produced once
        ms = time_events(torch, getattr(step, args.only), args.steps, warmup=args.warmup, min_ms=0.0)
        print("%s: %.4f ms per call over %d calls" % (args.only, ms, args.steps), file=sys.stderr)
        if os.environ.get("DLMI_GEMM_CLOCK") == "1" and args.only.startswith("gemm"):
            # the engine clock inside the last of those launches, from the kernel's own counters (no profiler)
            mhz, us = dl.gemm_clock()
            print("%s: engine clock inside the launch %.0f MHz (first tile's workgroup lived %.1f us)" % (args.only, mhz, us),
                  file=sys.stderr)
            print(workgroup_timeline(dl, step, args.only), file=sys.stderr)
        return None

    # ---- one clean step on the fresh inputs: the results the CPU baseline is compared with
    step()
    bad = gave_up(dl)
    host = lambda x: x.cpu().numpy()
    gpu = dict(y=host(t["y"]), dZ=host(t["dZ"]), dgamma=host(t["dgamma"]), dbeta=host(t["dbeta"]),
               **({"db": host(t["db"])} if K else {}),
               mean=host(t["stats"]["mean"]), std=host(t["stats"]["std"]), mov_mean=host(t["mov_mean"]),
               mov_std=host(t["mov_std"]))
    if K:
        gpu.update(Z=host(t["Z"]), dX=host(t["dX"]), dW=host(t["dW"]))
    if name == "c5":
        step.infer_fwd()
        gpu["y_inference"] = host(t["y"])
        step.norm_fwd()

    # ---- timed steps, then per-kernel-group timings with HIP events on the launch stream
    # the headline workload times exactly --steps steps after --warmup (117 ms: a sustained load by itself)
    steps, warmup = (args.steps, args.warmup) if (name == "c3" or args.explicit_steps) else sustained_steps(torch, step)
    ms_per_step = time_wall(torch, step, steps, warmup)
    bad = gave_up(dl) or bad
    E = B * H
    t_nf = time_events(torch, step.norm_fwd, 20)
    t_nb = time_events(torch, step.norm_bwd, 20)
    hbm = {"bound": "hbm", "achieved": 32.0 * E / ((t_nf + t_nb) * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
           "traffic": measured_traffic(name, "norm_act")}
    hbm["frac"] = hbm["achieved"] / hbm["peak"]
    ms = {"norm_fwd": t_nf, "norm_bwd": t_nb}
    report = {"roofline_norm_act": {"kernels": "dlmi_fused_norm_act_fwd + dlmi_fused_norm_act_bwd; `achieved` counts the "
                                               "two-pass accounting of 12 + 20 B/element whatever the kernels move",
                                    "bytes_fwd": 12.0 * E, "bytes_bwd": 20.0 * E}}
    detail = {"ms": ms}
    if K:
        t_gf = time_events(torch, step.gemm_fwd, 10)
        t_gx = time_events(torch, step.gemm_dx, 10)
        t_gw = time_events(torch, step.gemm_dw_only, 10)
        flops = 2.0 * B * K * H
        avg = (t_gf + t_gx + t_gw) / 3.0
        roof = {"bound": "mfma", "achieved": flops / (avg * 1e-3) / 1e12, "peak": MFMA_FP32_PEAK_TFLOPS,
                "unit": "TFLOP/s", "traffic": measured_traffic(name, "gemm"),
                "kernel": "k_gemm_f32 (avg of fwd, dX, dW)"}
        roof["frac"] = roof["achieved"] / roof["peak"]
        t_ff = time_events(torch, step.fc_norm_fwd, 10)
        t_nbd = time_events(torch, step.norm_bwd_db, 10)
        ms.update({"gemm_fwd": t_gf, "gemm_dx": t_gx, "gemm_dw": t_gw, "fc_norm_fwd": t_ff, "norm_bwd_db": t_nbd})
        # epilogue-fused accounting (kept apart from roofline_norm_act): the normalization forward costs what
        # the fused call takes beyond the plain GEMM and moves 8 B/element
        report["epilogue_fused_norm_fwd"] = {"ms": t_ff - t_gf, "bytes": 8.0 * E,
                                             "GBps": 8.0 * E / max(t_ff - t_gf, 1e-6) / 1e6}
        if name == "c5":
            t_in = time_events(torch, step.infer_fwd, 20)
            ms["inference_fwd"] = t_in
            detail["inference_fwd_frac_hbm"] = 8.0 * E / t_in / 1e6 / HBM_PEAK_GBS
        if full:
            # the optimizer step that follows a training step (Adam over the H x K weights: reads and writes
            # parameter, gradient and both moments = 32 B/parameter), timed last because it consumes dW
            t_ad = time_events(torch, step.adam, 10)
            ms["adam_step"] = t_ad
            report["adam_step"] = {"ms": t_ad, "bytes": 32.0 * H * K, "frac_hbm_peak": 32.0 * H * K / t_ad / 1e6 / HBM_PEAK_GBS}
            # What a caller pays who hands over host rows every step, as the facade's forward_pass(batch, rows)
            # does: the [B, K] input block from pinned host memory over PCIe, on top of the step.  Not `value`.
            pinned = torch.empty((B, K), dtype=torch.float32, pin_memory=True)
            pinned.copy_(t["X"])
            staging = torch.empty_like(t["X"])
            t_up = time_events(torch, lambda: staging.copy_(pinned, non_blocking=True), 5, warmup=1)
            ms["host_rows_upload"] = t_up
            report["host_rows_upload"] = {"ms": t_up, "GBps": 4.0 * B * K / t_up / 1e6,
                                          "samples_per_s_with_upload": B / ((ms_per_step + t_up) * 1e-3)}
            del pinned, staging
    else:
        roof = dict(hbm)
    bad = gave_up(dl) or bad

    cpu = parity = None
    if cp is not None:
        # the bounded CPU sample: c3's pass takes seconds (1 warm-up + 1), the others 1 warm-up + median of 5
        cpu, cpu_report = cp.baseline(1 if name == "c3" else 5)
        report["cpu_baseline"] = cpu_report
        if cp.Bs == B:  # batch statistics of a row sample differ from the full batch's: compare full passes only
            if name == "c5":
                cp.inference()
            ref = cp.results()
            chain = dw_single_chain(h, gpu, ref, B, H, K) if K else None
            parity, per_tensor = parity_block({k: (gpu[k], ref[k]) for k in ref}, 1e-4, layer_f64_slabs(name, h, gpu, ref),
                                              {"kinks_zeroed": kinks},
                                              {"dW": chain["rms_err_single_chain_vs_f64"]} if chain else None)
            report["parity_tensors"] = per_tensor
            if chain:
                report["dW_summation_order"] = chain
    config = {"workload": name + ": " + descr, "batch": B, "fan_in": K, "units": H}
    detail["panel_gave_up"] = bad
    del step, t
    torch.cuda.empty_cache()
    return line(B / (ms_per_step * 1e-3), ms_per_step, steps, warmup, config, roof, hbm, cpu, detail, parity, report)


# ---------------------------------------------------------------- c4: residual blocks
def run_c4(args, torch, pkg, dl):
    """Workload c4: 16 residual blocks x + Dropout(ISRLU(BRN(FC(x)))), width 2048, batch 1024, per-element
    uint8 keep-mask [16, 1024, 2048] (p_drop 0.1), masked backward; forward + backward (dX, dW, dgamma, dbeta
    per block) assembled from the C ABI leaves: per block one call forward (GEMM with the statistics in its
    epilogue, then normalization + activation + mask + shortcut in one pass), three backward (fused
    normalization backward, dX accumulated into the running gradient, dW).  Everything pre-allocated and
    resident in HBM; the host only enqueues."""
    import numpy as np
    from oracle.binding import ACT, HarnessRng, Oracle
    nblk, H, B, keep = 16, 2048, 1024, 0.9
    rng = HarnessRng(1234 + 400)
    hx0 = rng.normal(1, (B, H))
    lim = (6.0 / (2 * H)) ** 0.5
    hW = [rng.uniform(10 + i, (H, H), -lim, lim) for i in range(nblk)]
    hmask = rng.bernoulli_u8(2, (nblk, B, H), keep)
    hdOut = rng.normal(3, (B, H))
    dev = dict(device="cuda")
    up = lambda a: torch.from_numpy(a).cuda()
    x0, Ws, mask, dOut = up(hx0), [up(w) for w in hW], up(hmask), up(hdOut)
    scale = float(np.float32(1) / np.float32(keep))
    desc = pkg.Dlmi.desc(pkg.ACT["ISRLU"], renorm=True, dropout=pkg.DROP["BERNOULLI_INVERTED"], mask_per_element=True,
                         dropout_bwd=1, drop_scale=scale, **HYPER)
    one, zero = torch.ones(H, **dev), torch.zeros(H, **dev)
    xs = [x0] + [torch.empty(B, H, **dev) for _ in range(nblk)]       # block inputs / outputs
    Zs = [torch.empty(B, H, **dev) for _ in range(nblk)]
    stats = [{k: torch.empty(H, **dev) for k in ("mean", "std", "r", "d")} for _ in range(nblk)]
    mm, ms = [zero.clone() for _ in range(nblk)], [one.clone() for _ in range(nblk)]
    dWs = [torch.empty(H, H, **dev) for _ in range(nblk)]
    dgs, dbs = [zero.clone() for _ in range(nblk)], [zero.clone() for _ in range(nblk)]
    dZ, g = torch.empty(B, H, **dev), torch.empty(B, H, **dev)
    # The weight gradient of a block depends on nothing that follows it, so it runs on a second stream (a context
    # of its own: its scratch) beside the chain dX -> normalization backward of the block below -> ...: a product
    # of this size leaves the matrix pipes idle for 15-20 % of its launch (dispatch, first operands, stores), which
    # the other stream's product fills.  dZ alternates between two buffers; an event per buffer says when the
    # weight gradient has read it.
    two_streams = args.c4_streams == 2 and args.c4_dw == "layer"
    grouped = args.c4_dw == "grouped"
    main = torch.cuda.current_stream()
    side = torch.cuda.Stream() if two_streams else None  # default priority
    dl_side = pkg.Dlmi(0) if two_streams else None
    if two_streams:
        dl_side.set_stream(side)
    dZs = [dZ, torch.empty(B, H, **dev)] if two_streams else [dZ, dZ]
    if grouped:  # every block keeps its dZ until the one launch that forms all the weight gradients
        dZs = [dZ] + [torch.empty(B, H, **dev) for _ in range(nblk - 1)]
    ready = [torch.cuda.Event(), torch.cuda.Event()]
    read = [torch.cuda.Event(), torch.cuda.Event()]
    used = [False, False]

    def step(two_streams=two_streams):
        for i in range(nblk):
            dl.fc_norm_act_fwd(desc, xs[i], Ws[i], one, zero, mm[i], ms[i], mask=mask[i], Z=Zs[i], out=xs[i + 1],
                               stats=stats[i], shortcut=xs[i])
        g.copy_(dOut)
        for k, i in enumerate(reversed(range(nblk))):
            b = i if grouped else k & 1
            if two_streams and used[b]:
                main.wait_event(read[b])  # the weight gradient two blocks up has read this buffer
            dl.fused_bwd(desc, Zs[i], one, zero, stats[i], g, dgs[i], dbs[i], mask=mask[i], out=dZs[b])
            if two_streams:
                ready[b].record(main)
            dl.fc_bwd_dx(dZs[b], Ws[i], out=g, accumulate=True)  # the shortcut carries g on, the block adds dZ W
            if two_streams:
                side.wait_event(ready[b])
                dl_side.fc_bwd_dw(xs[i], dZs[b], dW=dWs[i])
                read[b].record(side)
                used[b] = True
            elif not grouped:
                dl.fc_bwd_dw(xs[i], dZs[b], dW=dWs[i])
        if grouped:
            dl.fc_bwd_dw_grouped([(xs[i], dZs[i], dWs[i], None) for i in range(nblk)])
        if two_streams:
            main.wait_stream(side)  # the step ends when both streams have

    ctxs = [dl] + ([dl_side] if two_streams else [])
    step()
    bad = gave_up(*ctxs)
    host = lambda x: x.cpu().numpy()
    gpu = {"out": host(xs[nblk]), "dX": host(g), "dW_first": host(dWs[0]), "dW_last": host(dWs[-1]),
           "dgamma_first": host(dgs[0]), "dgamma_last": host(dgs[-1]), "dbeta_first": host(dbs[0])}
    for v in dgs + dbs:
        v.zero_()
    steps, warmup = (args.steps, args.warmup) if args.explicit_steps else sustained_steps(torch, step)
    ms_step = time_wall(torch, step, steps, warmup)
    ms_one_stream = time_wall(torch, lambda: step(False), steps, warmup) if two_streams else ms_step
    bad = gave_up(*ctxs) or bad
    E = B * H
    t_f = time_events(torch, lambda: dl.fc_fwd(xs[0], Ws[0], None, out=Zs[0]), 20)
    t_x = time_events(torch, lambda: dl.fc_bwd_dx(dZ, Ws[0], out=g), 20)
    t_w = time_events(torch, lambda: dl.fc_bwd_dw(xs[0], dZ, dW=dWs[0]), 20)
    flops = 2.0 * B * H * H
    avg = (t_f + t_x + t_w) / 3.0
    roof = {"bound": "mfma", "achieved": flops / (avg * 1e-3) / 1e12, "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
            "traffic": measured_traffic("c4", "gemm"),
            "kernel": "k_gemm_f32 1024x2048x2048 (avg of fwd, dX, dW; operands cache-resident)"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    ytmp = torch.empty(B, H, **dev)
    t_nf = time_events(torch, lambda: dl.fused_fwd(desc, Zs[0], one, zero, mm[0], ms[0], mask=mask[0], out=ytmp,
                                                   stats=stats[0], shortcut=xs[0]), 50, warmup=5)
    t_nb = time_events(torch, lambda: dl.fused_bwd(desc, Zs[0], one, zero, stats[0], dOut, dgs[0], dbs[0], mask=mask[0],
                                                   out=dZ), 50, warmup=5)
    # 32 B/element + 3 (mask read by three passes) + 4 (shortcut read by the forward apply pass); the 8 MiB
    # tensors are cache-resident and the chain is bound by launch latency, not by bandwidth
    hbm = {"bound": "hbm", "achieved": 39.0 * E / ((t_nf + t_nb) * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
           "traffic": measured_traffic("c4", "norm_act")}
    hbm["frac"] = hbm["achieved"] / hbm["peak"]
    bad = gave_up(*ctxs) or bad
    detail = {"ms": {"gemm_fwd": t_f, "gemm_dx": t_x, "gemm_dw": t_w, "norm_fwd": t_nf, "norm_bwd": t_nb,
                     "step_one_stream": ms_one_stream},
              "whole_step_frac_mfma_peak": 3.0 * nblk * flops / (ms_step * 1e-3) / 1e12 / MFMA_FP32_PEAK_TFLOPS,
              "streams": 2 if two_streams else 1, "weight_gradients": args.c4_dw, "panel_gave_up": bad}
    report = {"gemm_ms_per_step": 16 * (t_f + t_x + t_w), "norm_ms_per_step": 16 * (t_nf + t_nb),
              "calls_per_step": 4 * nblk + 1}

    cpu = parity = None
    if args.cpu_rows != 0:
        kind, eng = cpu_engine()
        model, ncpu, nt = host_info()
        onev, zerov = np.ones(H, np.float32), np.zeros(H, np.float32)
        hyper = (HYPER["momentum"], HYPER["eps"], HYPER["r_max"], HYPER["d_max"])
        keepf = [hmask[i].astype(np.float32) * np.float32(scale) for i in range(nblk)]  # outside the timed passes

        keep_of = lambda i, dt: keepf[i] if dt == np.float32 else keepf[i].astype(dt)

        def network(eng, matmul_nt, matmul_nn, matmul_tn, dt, nth):
            """The whole step from leaves; returns the tensors the GPU's are compared with."""
            one_, zero_ = onev.astype(dt), zerov.astype(dt)
            saved, cur = [], hx0.astype(dt)
            for i in range(nblk):
                Z = matmul_nt(cur, hW[i])
                fw = eng.norm_fwd_train(Z, one_, zero_, zero_, one_, *hyper, True, nth)
                q = eng.act_fwd(ACT["ISRLU"], fw["out"], nth)
                y = q * keep_of(i, dt)  # the reference's dropout leaf takes one mask per unit
                saved.append((cur, Z, fw, q))
                cur = eng.identity_add(cur, y, nth)
            gg = hdOut.astype(dt)
            cdW, cdg, cdb = [None] * nblk, [None] * nblk, [None] * nblk
            for i in reversed(range(nblk)):
                xin, Z, fw, q = saved[i]
                dN = eng.act_bwd(ACT["ISRLU"], fw["out"], q, gg * keep_of(i, dt), nth)
                bw = eng.norm_bwd(fw["mean"], fw["std"], one_, fw["r"], Z, fw["xhat"], dN, renorm=True, nthreads=nth)
                dXb = matmul_nn(bw["dx"], hW[i])
                if i in (0, nblk - 1) or dt == np.float32:  # the timed pass forms every block's; two are compared
                    cdW[i] = matmul_tn(bw["dx"], xin)
                cdg[i], cdb[i] = bw["dgamma"], bw["dbeta"]
                gg = eng.identity_add(gg, dXb, nth)
            return {"out": cur, "dX": gg, "dW_first": cdW[0], "dW_last": cdW[-1], "dgamma_first": cdg[0],
                    "dgamma_last": cdg[-1], "dbeta_first": cdb[0]}

        ref_pass = lambda: network(eng, lambda a, w: eng.fc_fwd(a, w, nt), lambda a, w: eng.fc_bwd_dx(a, w, nthreads=nt),
                                   lambda dz, x: eng.fc_bwd_dw(x, dz, with_bias=False, nthreads=nt)[0], np.float32, nt)
        out = {}
        dt = median_time(lambda: out.update(ref=ref_pass()), 5, warmup=1)
        cpu = {"value": B / dt, "unit": "samples/s", "cores": nt, "kind": kind,
               "sample": "whole step, all %d rows, 1 warm-up + median of 5 passes" % B}
        report["cpu_baseline"] = {"seconds_per_pass": dt, "host_cpu_count": ncpu, "cpu_model": model,
                                  "note": "16 blocks assembled from the OpenMP leaves, the per-element mask applied with numpy"}
        ref = out["ref"]
        # float64 arbiter: the same network with float64 leaves and float64 library products
        d = lambda a: np.asarray(a, np.float64)
        o64 = Oracle(np.float64)
        f64 = network(o64, lambda a, w: d(a) @ d(w).T, lambda a, w: d(a) @ d(w), lambda dz, x: d(dz).T @ d(x), np.float64, 0)
        parity, per_tensor = parity_block({k: (gpu[k], ref[k]) for k in ref}, 1e-4,
                                          {k: (gpu[k], f64[k], ref[k], f64[k]) for k in ref})
        report["parity_tensors"] = per_tensor
    config = {"workload": "c4: 16 residual blocks x + Dropout(ISRLU(BRN(FC x))), width 2048, batch 1024, uint8 mask per "
                          "element, fwd+bwd", "batch": B, "units": H, "blocks": nblk}
    if two_streams:
        dl_side.close()
    return line(B / (ms_step * 1e-3), ms_step, steps, warmup, config, roof, hbm, cpu, detail, parity, report)


# ---------------------------------------------------------------- c1: the MLP through the facade
def c1_f64(widths, p, offsets, X, Y):
    """One training step of workload c1 in float64 from the initial parameters: (gradient array, output)."""
    import numpy as np
    from oracle.binding import ACT, Oracle
    o = Oracle(np.float64)
    d = lambda a: np.asarray(a, np.float64)
    L = len(widths) - 1
    Ws = [d(p[offsets[l][0]:offsets[l][0] + widths[l] * widths[l - 1]]).reshape(widths[l], widths[l - 1]) for l in range(1, L + 1)]
    hyper = (HYPER["momentum"], HYPER["eps"], HYPER["r_max"], HYPER["d_max"])
    a, saved = d(X), []
    for l in range(1, L):
        H = widths[l]
        Z = a @ Ws[l - 1].T
        fw = o.norm_fwd_train(Z, np.ones(H), np.zeros(H), np.zeros(H), np.ones(H), *hyper, True)
        y = o.act_fwd(ACT["RELU"], fw["out"])
        saved.append((a, Z, fw, y))
        a = y
    bias_out = d(p[offsets[L][1]:offsets[L][1] + widths[L]])
    q = o.softmax_fwd(a @ Ws[L - 1].T + bias_out)
    dZ, _, _ = o.softmax_ce_seed(q, d(Y))
    g = np.zeros(p.size, np.float64)

    def put(l, dz, xin):
        g[offsets[l][0]:offsets[l][0] + widths[l] * widths[l - 1]] = (dz.T @ xin).ravel()

    put(L, dZ, a)
    g[offsets[L][1]:offsets[L][1] + widths[L]] = dZ.sum(0)
    dY = dZ @ Ws[L - 1]
    for l in range(L - 1, 0, -1):
        xin, Z, fw, y = saved[l - 1]
        H = widths[l]
        dN = o.act_bwd(ACT["RELU"], fw["out"], y, dY)
        bw = o.norm_bwd(fw["mean"], fw["std"], np.ones(H), fw["r"], Z, fw["xhat"], dN, renorm=True)
        put(l, bw["dx"], xin)
        g[offsets[l][2]:offsets[l][2] + H] = bw["dgamma"]
        g[offsets[l][3]:offsets[l][3] + H] = bw["dbeta"]
        if l > 1:
            dY = bw["dx"] @ Ws[l - 1]
    return g, q


def run_c1(args, torch, pkg):
    """Workload c1: MLP 784-512-512-10, batch 128, batch renorm + ReLU hidden layers, softmax +
    cross-entropy output, through the Model / Driver facade.  A step is one forward + error + backward +
    parameter-gradient pass over one batch of 128 rows (data set resident in HBM); every 64 steps
    Driver::train ends in one Adam update.  Latency-bound: a dozen kernels of a few microseconds each per
    step, replayed as one recorded HIP graph per batch."""
    import numpy as np
    from oracle.binding import ACT, NORM, OPT, HarnessRng
    from deep_learning_amd.model import Model
    widths, B, per_epoch = [784, 512, 512, 10], 128, 64
    n = B * per_epoch
    rng = HarnessRng(1234 + 100)
    X = rng.uniform(1, (n, widths[0]))
    Y = np.eye(widths[-1], dtype=np.float32)[rng.index(2, n, widths[-1])]

    def build(make):
        M = make(widths)
        for l in (1, 2):
            M.set_layer(l, ACT["RELU"], NORM["BRN"])
        M.set_layer(3, ACT["SOFTMAX"])
        M.set_norm_hyper(HYPER["momentum"], HYPER["eps"], HYPER["r_max"], HYPER["d_max"])
        return M

    M = build(lambda w: Model(pkg.load_library(), w))  # raises without the HIP library or a GPU
    M.prepare(B)
    p = M.get_parameters()
    offsets = {l: M.layer_offsets(l) for l in range(1, 4)}
    for l in range(1, 4):
        K, H = widths[l - 1], widths[l]
        lim = (6.0 / (K + H)) ** 0.5
        p[offsets[l][0]:offsets[l][0] + H * K] = rng.uniform(10 + l, (H * K,), -lim, lim)
    M.set_parameters(p)
    M.set_optimizer(OPT["ADAM"], adam_lr=1e-3)
    R = kind = None
    pb = 0  # the batch the parity check uses
    if args.cpu_rows != 0:
        from oracle.binding import Oracle, OracleMLP, Reference, reference_available
        kind = "reference" if reference_available() else "port"
        model, ncpu, nt = host_info()
        R = build((lambda w: Reference().mlp(w)) if kind == "reference" else (lambda w: OracleMLP(Oracle(), w)))
        R.prepare(B, nt)

        def reset_reference():
            if kind == "reference":
                R.set_parameters(p)
                R.set_moving(np.zeros(sum(widths), np.float32), np.ones(sum(widths), np.float32))
            else:
                R.parameters[:] = p
                R.moving_mean[:] = 0
                R.moving_std[:] = 1
        # ReLU's derivative jumps at 0: a hidden pre-activation within rounding of it may take the other branch on
        # the other side and move every gradient below it.  The check uses the first batch that has none.
        for pb in range(per_epoch):
            reset_reference()
            R.step(1, X[pb * B:(pb + 1) * B], Y[pb * B:(pb + 1) * B], backward=False)
            if all(float(np.min(np.abs(R.layer_buffer(l, 2)))) >= KINK for l in (1, 2)):
                break
        reset_reference()
    # one step on that batch from the initial parameters: the gradients the CPU baseline is compared with
    Xp, Yp = X[pb * B:(pb + 1) * B], Y[pb * B:(pb + 1) * B]
    M.step(1, Xp, Yp)
    gpu = {"dparameters": np.array(M.get_dparams()).copy(), "output": np.array(M.layer_buffer(3, 3)).copy()}
    M.clear_training_arrays()
    M.set_parameters(p)
    mz = M.get_moving()
    M.set_moving(np.zeros_like(mz[0]), np.ones_like(mz[1]))
    # ten epochs of 64 batches: 60 ms of replayed graphs, a sustained load.  The driver launches the first epoch
    # kernel by kernel, records the second into one HIP graph per batch and replays from the third on: those
    # two stay outside the timed region, and so do as many replayed epochs as bring the clock to its working point
    epochs = max(1, args.steps // per_epoch) if args.explicit_steps else 10
    warm_epochs = max(2, -(-args.warmup // per_epoch)) if args.explicit_steps else 2 + 6
    for _ in range(warm_epochs):
        M.train_epoch(X, Y)
    t0 = time.perf_counter()
    for _ in range(epochs):
        loss, accu = M.train_epoch(X, Y)  # returns after the loss has been read back: the stream is idle
    dt = time.perf_counter() - t0  # a kernel that gave up makes train_epoch raise
    steps = epochs * per_epoch
    ms = dt / steps * 1e3
    flops = 2.0 * B * (784 * 512 + 512 * 512 + 512 * 10) * 2 + 2.0 * B * (512 * 512 + 512 * 10)  # fwd + dW, dX of layers 2, 3
    roof = {"bound": "mfma", "achieved": flops / (ms * 1e-3) / 1e12, "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
            "traffic": None, "kernel": "whole step (latency-bound; one HIP graph replay per batch)"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    cpu = parity = None
    report = {}
    if R is not None:
        R.step(1, Xp, Yp)
        ref = {"dparameters": np.array(R.get_dparams()).copy(), "output": np.array(R.layer_buffer(3, 3)).copy()}
        g64, q64 = c1_f64(widths, p, offsets, Xp, Yp)
        parity, per_tensor = parity_block({k: (gpu[k], ref[k]) for k in ref}, 1e-4,
                                          {"dparameters": (gpu["dparameters"], g64, ref["dparameters"], g64),
                                           "output": (gpu["output"], q64, ref["output"], q64)}, {"batch": pb})
        report["parity_tensors"] = per_tensor
        if kind == "reference":
            R.set_dparams(np.zeros_like(ref["dparameters"]))
        else:
            R.dparameters[:] = 0
        reset_reference()
        R.set_optimizer(OPT["ADAM"], adam_lr=1e-3)
        dtc = median_time(lambda: R.train_epoch(X, Y), 5, warmup=1)
        cpu = {"value": n / dtc, "unit": "samples/s", "cores": nt, "kind": kind,
               "sample": "Driver::train epoch, %d rows in batches of %d, 1 warm-up + median of 5" % (n, B)}
        report["cpu_baseline"] = {"seconds_per_epoch": dtc, "host_cpu_count": ncpu, "cpu_model": model}
    config = {"workload": "c1: MLP 784-512-512-10, batch 128, BRN + ReLU, softmax cross-entropy, fwd+bwd per batch, "
                          "Adam every 64 batches (Driver::train)", "batch": B}
    out = line(B / (ms * 1e-3), ms, steps, warm_epochs * per_epoch, config, roof, None, cpu,
               {"final_loss": loss, "final_accuracy": accu, "panel_gave_up": False}, parity, report)
    M.close()
    return out


# ---------------------------------------------------------------- main
def brief(o):
    """A side workload's line reduced to what the headline's detail.workloads carries: fixed short keys."""
    r, h = o["roofline"], o.get("roofline_norm_act")
    out = {"w": o["config"]["workload"].split(":")[0], "value": o["value"], "ms_per_step": o["ms_per_step"],
           "steps": o["steps"], "warmup": o["warmup"],
           "roofline": {"bound": r["bound"], "achieved": r["achieved"], "unit": r["unit"], "frac": r["frac"],
                        "traffic": r.get("traffic")}}
    if h is not None and r["bound"] != "hbm":
        out["norm_act"] = {"achieved": h["achieved"], "frac": h["frac"], "traffic": h.get("traffic")}
    c = o.get("cpu_baseline")
    if c:
        out["cpu"] = {"value": c["value"], "cores": c["cores"], "kind": c["kind"]}
    if o.get("parity"):
        out["parity"] = o["parity"]
    out["detail"] = o["detail"]
    return out


def emit(head, report_path):
    """The compact line on stdout, the unabridged report on stderr (and in `report_path`)."""
    def strip(o):
        rep = o.pop("_report", None)
        return rep
    report = {"headline": strip(head)}
    for name, w in head["detail"].get("workloads", {}).items():
        if isinstance(w, dict) and "_report" in w:
            report[name] = w.pop("_report")
    text = json.dumps(rnd(head), separators=(",", ":"))
    full = json.dumps({"line_bytes": len(text), "report": report})
    print("bench report: " + full, file=sys.stderr)
    if report_path:
        with open(report_path, "w") as f:
            f.write(full + "\n")
    print(text)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps of the headline workload (default 20)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps before them (default 3)")
    ap.add_argument("--workload", default="all", choices=["all", "c1", "c2", "c3", "c4", "c5"])
    ap.add_argument("--c4-streams", type=int, default=2, choices=[1, 2],
                    help="workload c4: 2 = the weight gradients run on a second stream beside the backward chain")
    ap.add_argument("--c4-dw", default="layer", choices=["layer", "grouped"],
                    help="workload c4: the weight gradients block by block (beside the chain with --c4-streams 2), or "
                         "all sixteen in one grouped launch after the backward chain")
    ap.add_argument("--cpu-rows", type=int, default=-1, help="rows of the CPU baseline sample (0 = skip the CPU legs "
                                                             "and the in-run parity check)")
    ap.add_argument("--only", default="", help="profiling aid (layer workloads): run just this part (gemm_fwd, gemm_dx, "
                                               "gemm_dw, gemm_dw_only, norm_fwd, norm_bwd, norm_bwd_db, fc_norm_fwd, infer_fwd, adam, copy, "
                                               "strip_fwd, strip_bwd) "
                                               "--steps times and exit without a JSON line")
    ap.add_argument("--shape", default="", help="profiling aid, with --only: B,K,H of the layer to run the part on instead "
                                                "of a workload's (e.g. 1024,2048,2048: one block of c4)")
    ap.add_argument("--report", default="", help="also write the unabridged figures to this file")
    ap.add_argument("--traffic-digest", action="store_true", help="print the digest of the kernel sources the "
                                                                  "`traffic` figures are tied to and exit")
    args = ap.parse_args()
    if args.traffic_digest:
        print(traffic_sources_digest())
        return
    # --steps / --warmup always govern the headline workload c3; a side workload follows them only when it is run
    # on its own (profiling runs name their counts), otherwise it takes what makes a sustained load
    args.explicit_steps = args.steps is not None and args.workload not in ("all", "c3")
    args.steps = 20 if args.steps is None else args.steps
    args.warmup = 3 if args.warmup is None else args.warmup
    if args.shape:
        if not args.only:
            ap.error("--shape needs --only")
        LAYER_WORKLOADS["shape"] = tuple(int(v) for v in args.shape.split(",")) + ("ELU", "profiling shape " + args.shape)
        args.workload = "shape"
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    from __graft_entry__ import load_package
    pkg = load_package()
    dl = pkg.Dlmi(0)  # raises if the HIP library or the GPU is missing: no fallback

    def run(name, full):
        if name in LAYER_WORKLOADS:
            return run_layer(args, torch, pkg, dl, name, full)
        if name == "c4":
            return run_c4(args, torch, pkg, dl)
        return run_c1(args, torch, pkg)

    if args.workload != "all":
        if args.only and args.workload not in LAYER_WORKLOADS:
            ap.error("--only applies to the layer workloads c2, c3, c5")
        out = run(args.workload, True)
        if out is not None:
            emit(out, args.report)
        dl.close()
        return
    if args.only:
        args.workload = "c3"
        run("c3", True)
        dl.close()
        return

    head = run("c3", True)
    others = {}
    for name in ("c1", "c2", "c4", "c5"):
        try:
            o = run(name, False)
            others[name] = brief(o)
            others[name]["_report"] = o["_report"]
        except Exception as e:  # a failing side workload must not take the headline down with it
            others[name] = {"error": "%s: %s" % (type(e).__name__, str(e)[:200])}
    head["detail"]["workloads"] = others
    head["detail"]["panel_gave_up"] = bool(head["detail"].get("panel_gave_up")) or any(
        isinstance(w, dict) and w.get("detail", {}).get("panel_gave_up") for w in others.values())
    emit(head, args.report)
    dl.close()


if __name__ == "__main__":
    main()
