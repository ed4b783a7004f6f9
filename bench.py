"""Benchmark of the fully-connected + batch-renorm + activation hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|c1|c2|c3|c4|c5]

The default run times workload c3 (configuration 3 of the benchmark: the one the metric is quoted on) as the
headline and the other four configurations under detail.workloads, each with its step time, the roofline
of its dominant kernels and the reference's CPU path timed beside it.

A "step" is one forward + backward pass over one synthetic batch resident in HBM.  Every input tensor
is drawn ONCE on the host from a seeded mt19937_64 stream of its own (oracle/harness_rng.c) and the same
bits go to the GPU and to the CPU baseline; the GPU results of the first step are checked in the run
against that CPU pass (max relative errors in the JSON line).

Prints ONE JSON line: samples/s of the whole step, the roofline of the dominant kernel (fp32 MFMA GEMM),
the HBM roofline of the fused normalization + activation kernels, and the CPU baseline measured on the host
cores (the compiled reference's OpenMP leaves when oracle/_ref is present, else this repository's
restatement of them).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "FC+BRN+act fwd+bwd samples/sec; % HBM peak (norm/act), % FP32 MFMA peak (GEMM)"
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_FP32_PEAK_TFLOPS = 157.3  # MI355X dense FP32 matrix
HYPER = dict(momentum=0.99, eps=1e-5, r_max=3.0, d_max=5.0)
NORM_TEXT = "batch renorm rmax=3 dmax=5 momentum=0.99 eps=1e-5"

LAYER_WORKLOADS = {
    # name: (B, K, H, activation, description)
    "c3": (8192, 4096, 4096, "ELU", "FC 4096->4096 on batch 8192 + batch renorm + ELU, fwd+bwd (dX,dW,db,dgamma,dbeta)"),
    "c2": (4096, 0, 4096, "SELU", "batch renorm + SELU fwd+bwd on [4096 x 4096] (no FC)"),
    "c5": (65536, 256, 256, "LEAKY_RELU", "FC 256->256 on batch 65536 + batch renorm + leaky ReLU, fwd+bwd, and the "
                                          "inference-mode forward on moving statistics"),
}

# HBM-side bytes per launch (sequence) from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this file's --only
# parts, calibrated against the plain copy of --only copy (profiles/c3_c2_hbm_traffic_pmc.md).  Hardware
# counters cannot be read from inside this process: these are the figures of the committed profile, and
# TRAFFIC_PROFILE names it so that a reader can tell which build they belong to.
MIB = 1024.0 * 1024.0
TRAFFIC_PROFILE = "profiles/c3_c2_hbm_traffic_pmc.md"
MEASURED_TRAFFIC_BYTES = {
    "c3": {"gemm": (897.8 + 897.3 + 832.8) / 3.0 * MIB, "norm_act": 901.8 * MIB},
    "c2": {"norm_act": 326.4 * MIB},
}
# The figures above belong to the kernels as they were when the counters were read: the digest of their
# sources at that time (`python bench.py --traffic-digest` prints the current one).  When a source has
# changed since, `traffic` is reported as null instead of a figure that may no longer hold.
TRAFFIC_SOURCES = ("gemm_f32_mfma.hip", "norm_kernels.hip", "norm_panel_fwd.hip", "norm_panel_bwd.hip",
                   "norm_panel_common.hpp", "norm_shared.hpp", "activations.hpp", "dlmi_common.hpp")
TRAFFIC_SOURCES_SHA256 = "bac12d74dbe0450cca72c0468c1f8a926ba5a3cdf475be4b3daf00067df1171a"


def traffic_sources_digest():
    import hashlib
    h = hashlib.sha256()
    for name in TRAFFIC_SOURCES:
        with open(os.path.join(ROOT, "deep-learning_amd", "csrc", name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()


def measured_traffic(workload, key):
    """(bytes, source) for the roofline's `traffic`: the profile's figure while the kernels are the measured ones."""
    v = MEASURED_TRAFFIC_BYTES.get(workload, {}).get(key)
    if v is None:
        return None, None
    if traffic_sources_digest() != TRAFFIC_SOURCES_SHA256:
        return None, "not reported: the kernel sources have changed since %s was taken" % TRAFFIC_PROFILE
    return v, TRAFFIC_PROFILE


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
    parity tests assert behind reductions and GEMMs, and the strict per-element metric, on float32 arrays
    (chunked: the largest tensors are 128 MiB)."""
    import numpy as np
    g = np.asarray(got, np.float32).ravel()
    e = np.asarray(exp, np.float32).ravel()
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


def parity_block(pairs, limit):
    """pairs: name -> (gpu array, cpu array).  The rms-floored error must meet `limit` (1e-4 behind
    reductions and GEMMs, as the parity tests assert); the strict per-element error is reported beside it."""
    out, ok = {}, True
    for k, (g, e) in pairs.items():
        a, b = rel_errors(g, e)
        out[k] = {"max_rel_err": a, "max_rel_err_strict": b}
        ok = ok and a <= limit
    return {"tolerance": limit, "within_tolerance": ok, "against": "the CPU baseline of this run, same input bits",
            "tensors": out}


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


def sustained_steps(torch, fn, args):
    """(steps, warmup) of a side workload: the command line's when given, otherwise enough of both for a
    sustained load."""
    if args.steps_given:
        return args.steps, args.warmup
    ms = time_wall(torch, fn, 5, 2)
    return max(args.steps, int(1.5 * SUSTAINED_MS / ms) + 1), max(args.warmup, int(SUSTAINED_MS / ms) + 1)


def time_wall(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e3


def line(value, ms, steps, warmup, config, roof, hbm, cpu, detail, parity):
    out = {"metric": METRIC, "value": value, "unit": "samples/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
           "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
           "data": "synthetic", "config": config, "roofline": roof}
    if hbm is not None:
        out["roofline_norm_act"] = hbm
    out["cpu_baseline"] = cpu
    out["parity"] = parity
    out["detail"] = detail
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

    def parts(self):
        if self.K:
            return [self.fc_norm_fwd, self.norm_bwd, self.gemm_dx, self.gemm_dw]
        return [self.norm_fwd, self.norm_bwd]

    def __call__(self):
        for p in self.parts():
            p()


KINK = 1e-5  # |pre-activation| below which an activation whose derivative jumps at 0 may take either branch


def layer_cpu_forward(name, h, rows):
    """Forward half of the reference's OpenMP CPU path on the first `rows` rows of the same tensors."""
    from oracle.binding import ACT
    B, K, H, act, _ = LAYER_WORKLOADS[name]
    kind, cpu = cpu_engine()
    model, ncpu, nt = host_info()
    Bs = min(B, rows)
    t0 = time.perf_counter()
    Z = cpu.fc_fwd(h["X"][:Bs], h["W"], nt) if K else h["Z"][:Bs]
    fw = cpu.norm_fwd_train(Z, h["gamma"], h["beta"], h["mov_mean"], h["mov_std"], HYPER["momentum"], HYPER["eps"],
                            HYPER["r_max"], HYPER["d_max"], True, nt)
    y = cpu.act_fwd(ACT[act], fw["out"], nt)
    return dict(cpu=cpu, kind=kind, nt=nt, ncpu=ncpu, model=model, Bs=Bs, Z=Z, fw=fw, y=y, seconds=time.perf_counter() - t0)


def layer_cpu_backward(name, h, f):
    """Backward half; returns the cpu_baseline object and every output of the step."""
    from oracle.binding import ACT
    B, K, H, act, _ = LAYER_WORKLOADS[name]
    cpu, nt, Bs, Z, fw, y = f["cpu"], f["nt"], f["Bs"], f["Z"], f["fw"], f["y"]
    o = {}
    t0 = time.perf_counter()
    dN = cpu.act_bwd(ACT[act], fw["out"], y, h["dY"][:Bs], nt)
    bw = cpu.norm_bwd(fw["mean"], fw["std"], h["gamma"], fw["r"], Z, fw["xhat"], dN, renorm=True, nthreads=nt)
    if K:
        o["dX"] = cpu.fc_bwd_dx(bw["dx"], h["W"], nthreads=nt)
        o["dW"], _ = cpu.fc_bwd_dw(h["X"][:Bs], bw["dx"], with_bias=False, nthreads=nt)
    dt = f["seconds"] + time.perf_counter() - t0
    if K:
        o["Z"] = Z
    o.update(y=y, dZ=bw["dx"], dgamma=bw["dgamma"], dbeta=bw["dbeta"], mean=fw["mean"], std=fw["std"],
             mov_mean=fw["mov_mean"], mov_std=fw["mov_std"])
    if name == "c5":
        o["y_inference"] = cpu.act_fwd(ACT[act], cpu.norm_fwd_infer(Z, h["gamma"], h["beta"], h["inf_mean"],
                                                                    h["inf_std"], nt), nt)
    base = {"value": Bs / dt, "unit": "samples/s", "cores": nt, "host_cpu_count": f["ncpu"], "kind": f["kind"],
            "sample": "first %d of %d rows of the same tensors, one fwd+bwd pass, %.1f s, OpenMP leaves on %d "
                      "threads of %d processors (%s)" % (Bs, B, dt, nt, f["ncpu"], f["model"])}
    return base, o


def run_layer(args, torch, pkg, dl, name, full):
    """One layer workload.  full: the headline run (all detail timings)."""
    import numpy as np
    B, K, H, act, descr = LAYER_WORKLOADS[name]
    h = layer_inputs(name)
    cpu_rows = 0 if args.only else (args.cpu_rows if args.cpu_rows >= 0 else B)
    cf, kinks = None, None
    if cpu_rows:
        # The CPU forward runs first: where a pre-activation lies within rounding of 0, an activation whose
        # derivative jumps there (all of these) may take the other branch on the other side, which changes
        # that element's gradient by all of itself and, through the GEMMs, a whole row of dX and dW.  The
        # upstream gradient of those few elements is set to zero for BOTH sides, as in the parity tests.
        cf = layer_cpu_forward(name, h, cpu_rows)
        if cf["Bs"] == B:
            near = np.abs(cf["fw"]["out"]) < KINK
            kinks = int(near.sum())
            h["dY"][near] = 0.0
    step = LayerStep(dl, pkg, torch, name, h)
    t = step.t

    if args.only:
        step()  # every buffer a part reads has been produced once
        ms = time_events(torch, getattr(step, args.only), args.steps, warmup=args.warmup, min_ms=0.0)
        print("%s: %.4f ms per call over %d calls" % (args.only, ms, args.steps), file=sys.stderr)
        return None

    # ---- one clean step on the fresh inputs: the results the CPU baseline is compared with
    step()
    torch.cuda.synchronize()
    host = lambda x: x.cpu().numpy()
    gpu = dict(y=host(t["y"]), dZ=host(t["dZ"]), dgamma=host(t["dgamma"]), dbeta=host(t["dbeta"]),
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
    steps, warmup = (args.steps, args.warmup) if name == "c3" else sustained_steps(torch, step, args)
    ms_per_step = time_wall(torch, step, steps, warmup)
    E = B * H
    t_nf = time_events(torch, step.norm_fwd, 20)
    t_nb = time_events(torch, step.norm_bwd, 20)
    norm_traffic, norm_traffic_source = measured_traffic(name, "norm_act")
    hbm = {"bound": "hbm", "achieved": 32.0 * E / ((t_nf + t_nb) * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
           "traffic": norm_traffic, "traffic_source": norm_traffic_source,
           "kernels": "dlmi_fused_norm_act_fwd + dlmi_fused_norm_act_bwd; `achieved` counts the two-pass accounting "
                      "of 12 + 20 B/element.  Batches of 1024-8192 rows (forward) / 2048-4096 rows (backward) with a "
                      "width that is a multiple of 1024 run the single-launch panel kernels, which read every tensor "
                      "once (8 + 12 B/element of actual traffic, see `traffic`); other shapes run k_col_stats -> "
                      "k_fwd_apply / k_bwd_reduce -> k_bwd_apply",
           "ms_fwd": t_nf, "ms_bwd": t_nb, "bytes_fwd": 12.0 * E, "bytes_bwd": 20.0 * E}
    hbm["frac"] = hbm["achieved"] / hbm["peak"]
    detail = {"ms_norm_fwd": t_nf, "ms_norm_bwd": t_nb}
    if K:
        t_gf = time_events(torch, step.gemm_fwd, 10)
        t_gx = time_events(torch, step.gemm_dx, 10)
        t_gw = time_events(torch, step.gemm_dw_only, 10)
        flops = 2.0 * B * K * H
        avg = (t_gf + t_gx + t_gw) / 3.0
        gemm_traffic, gemm_traffic_source = measured_traffic(name, "gemm")
        roof = {"bound": "mfma", "achieved": flops / (avg * 1e-3) / 1e12, "peak": MFMA_FP32_PEAK_TFLOPS,
                "unit": "TFLOP/s", "traffic": gemm_traffic, "traffic_source": gemm_traffic_source,
                "kernel": "k_gemm_f32 (avg of fwd NT, dX NN, dW TN launches)",
                "tflops_fwd": flops / (t_gf * 1e-3) / 1e12, "tflops_dx": flops / (t_gx * 1e-3) / 1e12,
                "tflops_dw": flops / (t_gw * 1e-3) / 1e12}
        roof["frac"] = roof["achieved"] / roof["peak"]
        t_ff = time_events(torch, step.fc_norm_fwd, 10)
        detail.update({"ms_gemm_fwd": t_gf, "ms_gemm_dx": t_gx, "ms_gemm_dw": t_gw, "ms_fc_norm_fwd": t_ff,
                       # epilogue-fused accounting (kept apart from roofline_norm_act): the normalization
                       # forward costs what the fused call takes beyond the plain GEMM and moves 8 B/element
                       "epilogue_fused_norm_fwd": {"ms": t_ff - t_gf, "bytes": 8.0 * E,
                                                   "GBps": 8.0 * E / max(t_ff - t_gf, 1e-6) / 1e6}})
        if name == "c5":
            t_in = time_events(torch, step.infer_fwd, 20)
            detail["inference_fwd"] = {"ms": t_in, "bytes": 8.0 * E, "GBps": 8.0 * E / t_in / 1e6,
                                       "frac_hbm_peak": 8.0 * E / t_in / 1e6 / HBM_PEAK_GBS}
        if full:
            # the optimizer step that follows a training step (Adam over the H x K weights: reads and writes
            # parameter, gradient and both moments = 32 B/parameter), timed last because it consumes dW
            t_ad = time_events(torch, step.adam, 10)
            detail["adam_step"] = {"ms": t_ad, "bytes": 32.0 * H * K, "GBps": 32.0 * H * K / t_ad / 1e6,
                                   "frac_hbm_peak": 32.0 * H * K / t_ad / 1e6 / HBM_PEAK_GBS}
            # What a caller pays who hands over host rows every step, as the facade's forward_pass(batch, rows)
            # does: the [B, K] input block from pinned host memory over PCIe, on top of the step.  Not `value`.
            pinned = torch.empty((B, K), dtype=torch.float32, pin_memory=True)
            pinned.copy_(t["X"])
            staging = torch.empty_like(t["X"])
            t_up = time_events(torch, lambda: staging.copy_(pinned, non_blocking=True), 5, warmup=1)
            detail["host_rows_upload"] = {"ms": t_up, "GBps": 4.0 * B * K / t_up / 1e6,
                                          "samples_per_s_with_upload": B / ((ms_per_step + t_up) * 1e-3)}
            del pinned, staging
    else:
        roof = dict(hbm)

    cpu = parity = None
    if cf is not None:
        cpu, ref = layer_cpu_backward(name, h, cf)
        if cf["Bs"] == B:  # batch statistics of a row sample differ from the full batch's: compare full passes only
            parity = parity_block({k: (gpu[k], ref[k]) for k in ref}, 1e-4)
            parity["upstream_gradient_zeroed_at_kinks"] = kinks
    config = {"workload": name + ": " + descr, "batch": B, "fan_in": K, "units": H, "activation": act,
              "norm": NORM_TEXT, "inputs": "resident in HBM"}
    del step, t
    torch.cuda.empty_cache()
    return line(B / (ms_per_step * 1e-3), ms_per_step, steps, warmup, config, roof, hbm, cpu, detail, parity)


# ---------------------------------------------------------------- c4: residual blocks
def run_c4(args, torch, pkg, dl):
    """Workload c4: 16 residual blocks x + Dropout(ISRLU(BRN(FC(x)))), width 2048, batch 1024, per-element
    uint8 keep-mask [16, 1024, 2048] (p_drop 0.1), masked backward; forward + backward (dX, dW, dgamma, dbeta
    per block) assembled from the C ABI leaves: per block one call forward (GEMM with the statistics in its
    epilogue, then normalization + activation + mask + shortcut in one pass), three backward (fused
    normalization backward, dX accumulated into the running gradient, dW).  Everything pre-allocated and
    resident in HBM; the host only enqueues."""
    import numpy as np
    from oracle.binding import ACT, HarnessRng
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
    # the other stream's product fills (dX + dW of one block: 145 us one after the other, 129 us side by side).
    # dZ alternates between two buffers; an event per buffer says when the weight gradient has read it.
    two_streams = args.c4_streams == 2
    main = torch.cuda.current_stream()
    side = torch.cuda.Stream() if two_streams else None  # default priority
    dl_side = pkg.Dlmi(0) if two_streams else None
    if two_streams:
        dl_side.set_stream(side)
    dZs = [dZ, torch.empty(B, H, **dev)] if two_streams else [dZ, dZ]
    ready = [torch.cuda.Event(), torch.cuda.Event()]
    read = [torch.cuda.Event(), torch.cuda.Event()]
    used = [False, False]

    def step(two_streams=two_streams):
        for i in range(nblk):
            dl.fc_norm_act_fwd(desc, xs[i], Ws[i], one, zero, mm[i], ms[i], mask=mask[i], Z=Zs[i], out=xs[i + 1],
                               stats=stats[i], shortcut=xs[i])
        g.copy_(dOut)
        for k, i in enumerate(reversed(range(nblk))):
            b = k & 1
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
            else:
                dl.fc_bwd_dw(xs[i], dZs[b], dW=dWs[i])
        if two_streams:
            main.wait_stream(side)  # the step ends when both streams have

    step()
    torch.cuda.synchronize()
    host = lambda x: x.cpu().numpy()
    gpu = {"out": host(xs[nblk]), "dX": host(g), "dW_first": host(dWs[0]), "dW_last": host(dWs[-1]),
           "dgamma_first": host(dgs[0]), "dgamma_last": host(dgs[-1]), "dbeta_first": host(dbs[0])}
    for v in dgs + dbs:
        v.zero_()
    ms_step = time_wall(torch, step, args.steps, args.warmup)
    ms_one_stream = time_wall(torch, lambda: step(False), args.steps, args.warmup) if two_streams else ms_step
    E = B * H
    t_f = time_events(torch, lambda: dl.fc_fwd(xs[0], Ws[0], None, out=Zs[0]), 20)
    t_x = time_events(torch, lambda: dl.fc_bwd_dx(dZ, Ws[0], out=g), 20)
    t_w = time_events(torch, lambda: dl.fc_bwd_dw(xs[0], dZ, dW=dWs[0]), 20)
    flops = 2.0 * B * H * H
    avg = (t_f + t_x + t_w) / 3.0
    roof = {"bound": "mfma", "achieved": flops / (avg * 1e-3) / 1e12, "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
            "traffic": None, "kernel": "k_gemm_f32 at 1024 x 2048 x 2048 (avg of fwd, dX, dW launches; operands cache-resident)"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    ytmp = torch.empty(B, H, **dev)
    t_nf = time_events(torch, lambda: dl.fused_fwd(desc, Zs[0], one, zero, mm[0], ms[0], mask=mask[0], out=ytmp,
                                                   stats=stats[0], shortcut=xs[0]), 50, warmup=5)
    t_nb = time_events(torch, lambda: dl.fused_bwd(desc, Zs[0], one, zero, stats[0], dOut, dgs[0], dbs[0], mask=mask[0],
                                                   out=dZ), 50, warmup=5)
    hbm = {"bound": "hbm", "achieved": 39.0 * E / ((t_nf + t_nb) * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
           "traffic": None, "kernels": "fused normalization kernels of one block: 32 B/element + 3 (mask read by three "
                                       "passes) + 4 (shortcut read by the forward apply pass); the 8 MiB tensors are "
                                       "cache-resident and the chain is bound by launch latency, not by bandwidth",
           "ms_fwd": t_nf, "ms_bwd": t_nb}
    hbm["frac"] = hbm["achieved"] / hbm["peak"]
    detail = {"ms_gemm_fwd": t_f, "ms_gemm_dx": t_x, "ms_gemm_dw": t_w, "ms_norm_fwd": t_nf, "ms_norm_bwd": t_nb,
              "gemm_ms_per_step": 16 * (t_f + t_x + t_w), "norm_ms_per_step": 16 * (t_nf + t_nb),
              "calls_per_step": 4 * nblk + 1, "ms_per_step_one_stream": ms_one_stream}

    cpu = parity = None
    if args.cpu_rows != 0:
        kind, eng = cpu_engine()
        model, ncpu, nt = host_info()
        onev, zerov = np.ones(H, np.float32), np.zeros(H, np.float32)
        hyper = (HYPER["momentum"], HYPER["eps"], HYPER["r_max"], HYPER["d_max"])
        sc = np.float32(scale)
        t0 = time.perf_counter()
        saved, cur = [], hx0
        for i in range(nblk):
            Z = eng.fc_fwd(cur, hW[i], nt)
            fw = eng.norm_fwd_train(Z, onev, zerov, zerov, onev, *hyper, True, nt)
            q = eng.act_fwd(ACT["ISRLU"], fw["out"], nt)
            y = q * (hmask[i].astype(np.float32) * sc)  # the reference's dropout leaf takes one mask per unit
            saved.append((cur, Z, fw, q))
            cur = eng.identity_add(cur, y, nt)
        gg = hdOut
        cdW, cdg, cdb = [None] * nblk, [None] * nblk, [None] * nblk
        for i in reversed(range(nblk)):
            xin, Z, fw, q = saved[i]
            dN = eng.act_bwd(ACT["ISRLU"], fw["out"], q, gg * (hmask[i].astype(np.float32) * sc), nt)
            bw = eng.norm_bwd(fw["mean"], fw["std"], onev, fw["r"], Z, fw["xhat"], dN, renorm=True, nthreads=nt)
            dXb = eng.fc_bwd_dx(bw["dx"], hW[i], nthreads=nt)
            cdW[i], _ = eng.fc_bwd_dw(xin, bw["dx"], with_bias=False, nthreads=nt)
            cdg[i], cdb[i] = bw["dgamma"], bw["dbeta"]
            gg = eng.identity_add(gg, dXb, nt)
        dt = time.perf_counter() - t0
        cpu = {"value": B / dt, "unit": "samples/s", "cores": nt, "host_cpu_count": ncpu, "kind": kind,
               "sample": "the whole step (16 blocks, all %d rows) assembled from the OpenMP leaves, the per-element "
                         "mask applied with numpy, %.1f s, %d threads of %d processors (%s)" % (B, dt, nt, ncpu, model)}
        ref = {"out": cur, "dX": gg, "dW_first": cdW[0], "dW_last": cdW[-1], "dgamma_first": cdg[0],
               "dgamma_last": cdg[-1], "dbeta_first": cdb[0]}
        # 16 layers deep: the error budget of the parity tests grows with depth (4 x 1e-4 there at depth 4)
        parity = parity_block({k: (gpu[k], ref[k]) for k in ref}, 1e-3)
    config = {"workload": "c4: 16 residual blocks x + Dropout(ISRLU(BRN(FC x))), width 2048, batch 1024, "
                          "uint8 keep-mask per element, fwd+bwd", "batch": B, "units": H, "blocks": nblk,
              "norm": NORM_TEXT, "inputs": "resident in HBM",
              "streams": "2: weight gradients on a second stream beside the backward chain" if two_streams else "1"}
    if two_streams:
        dl_side.close()
    return line(B / (ms_step * 1e-3), ms_step, args.steps, args.warmup, config, roof, hbm, cpu, detail, parity)


# ---------------------------------------------------------------- c1: the MLP through the facade
def run_c1(args, torch, pkg):
    """Workload c1: MLP 784-512-512-10, batch 128, batch renorm + ReLU hidden layers, softmax +
    cross-entropy output, through the Model / Driver facade.  A step is one forward + error + backward +
    parameter-gradient pass over one batch of 128 rows (data set resident in HBM); every 64 steps
    Driver::train ends in one Adam update.  Latency-bound: about 20 kernels of a few microseconds each per
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
    for l in range(1, 4):
        o = M.layer_offsets(l)
        K, H = widths[l - 1], widths[l]
        lim = (6.0 / (K + H)) ** 0.5
        p[o[0]:o[0] + H * K] = rng.uniform(10 + l, (H * K,), -lim, lim)
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
    steps = args.steps if args.steps_given else 640  # ten epochs of 64 batches unless told otherwise
    epochs = max(1, steps // per_epoch)
    # the driver launches the first epoch kernel by kernel, records the second into one HIP graph per
    # batch and replays from the third on: at least those two stay outside the timed region
    warm_epochs = max(2, -(-args.warmup // per_epoch))
    for _ in range(warm_epochs):
        M.train_epoch(X, Y)
    t0 = time.perf_counter()
    for _ in range(epochs):
        loss, accu = M.train_epoch(X, Y)  # returns after the loss has been read back: the stream is idle
    dt = time.perf_counter() - t0
    steps = epochs * per_epoch
    ms = dt / steps * 1e3
    flops = 2.0 * B * (784 * 512 + 512 * 512 + 512 * 10) * 2 + 2.0 * B * (512 * 512 + 512 * 10)  # fwd + dW, dX of layers 2, 3
    roof = {"bound": "mfma", "achieved": flops / (ms * 1e-3) / 1e12, "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
            "traffic": None, "kernel": "whole step (latency-bound: the GEMMs are 128 x 512 x 784 and smaller; each batch is one HIP graph replay)"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    cpu = parity = None
    if R is not None:
        R.step(1, Xp, Yp)
        ref = {"dparameters": np.array(R.get_dparams()).copy(), "output": np.array(R.layer_buffer(3, 3)).copy()}
        parity = parity_block({k: (gpu[k], ref[k]) for k in ref}, 1e-4)
        parity["batch"] = pb
        if kind == "reference":
            R.set_dparams(np.zeros_like(ref["dparameters"]))
        else:
            R.dparameters[:] = 0
        reset_reference()
        R.set_optimizer(OPT["ADAM"], adam_lr=1e-3)
        R.train_epoch(X[:B * 4], Y[:B * 4])
        t1 = time.perf_counter()
        R.train_epoch(X, Y)
        dtc = time.perf_counter() - t1
        cpu = {"value": n / dtc, "unit": "samples/s", "cores": nt, "host_cpu_count": ncpu, "kind": kind,
               "sample": "one Driver::train epoch over the same %d rows in batches of %d, %.1f s, %d OpenMP threads of "
                         "%d processors (%s)" % (n, B, dtc, nt, ncpu, model)}
    config = {"workload": "c1: MLP 784-512-512-10, batch 128, batch renorm + ReLU, softmax cross-entropy, "
                          "fwd+bwd per batch, Adam update every 64 batches (Driver::train)",
              "batch": B, "norm": NORM_TEXT, "inputs": "resident in HBM"}
    out = line(B / (ms * 1e-3), ms, steps, warm_epochs * per_epoch, config, roof, None, cpu,
               {"final_loss": loss, "final_accuracy": accu}, parity)
    M.close()
    return out


# ---------------------------------------------------------------- main
def brief(o):
    """A workload's line reduced to what the headline's detail.workloads carries."""
    keep = ("value", "unit", "ms_per_step", "steps", "warmup", "config", "roofline", "roofline_norm_act", "cpu_baseline",
            "parity", "detail")
    return {k: o[k] for k in keep if k in o}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default 20; the short side workloads "
                                                            "then take as many as make a sustained load)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps before them (default 3)")
    ap.add_argument("--workload", default="all", choices=["all", "c1", "c2", "c3", "c4", "c5"])
    ap.add_argument("--c4-streams", type=int, default=2, choices=[1, 2],
                    help="workload c4: 2 = the weight gradients run on a second stream beside the backward chain")
    ap.add_argument("--cpu-rows", type=int, default=-1, help="rows of the CPU baseline sample (0 = skip the CPU legs "
                                                             "and the in-run parity check)")
    ap.add_argument("--only", default="", help="profiling aid (layer workloads): run just this part (gemm_fwd, gemm_dx, "
                                               "gemm_dw, norm_fwd, norm_bwd, fc_norm_fwd, infer_fwd, adam, copy) "
                                               "--steps times and exit without a JSON line")
    ap.add_argument("--shape", default="", help="profiling aid, with --only: B,K,H of the layer to run the part on instead "
                                                "of a workload's (e.g. 1024,2048,2048: one block of c4)")
    ap.add_argument("--traffic-digest", action="store_true", help="print the digest of the kernel sources the "
                                                                  "`traffic` figures are tied to and exit")
    args = ap.parse_args()
    if args.traffic_digest:
        print(traffic_sources_digest())
        return
    args.steps_given = args.steps is not None
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
            print(json.dumps(out))
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
            others[name] = brief(run(name, False))
        except Exception as e:  # a failing side workload must not take the headline down with it
            others[name] = {"error": "%s: %s" % (type(e).__name__, e)}
    head["detail"]["workloads"] = others
    print(json.dumps(head))
    dl.close()


if __name__ == "__main__":
    main()
