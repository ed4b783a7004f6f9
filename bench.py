"""Benchmark of the fully-connected + batch-renorm + activation hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c2|c5|c1]

A "step" is one forward + backward pass of the layer over one synthetic batch
resident in HBM:  Z = X W^T (+bias) -> batch renorm -> activation, then
dZ = d(activation, batch renorm), dX = dZ W, dW = dZ^T X, db, dgamma, dbeta.
Prints ONE JSON line: samples/s of the whole step, the roofline of the dominant
kernel (fp32 MFMA GEMM for c3/c5, the fused normalization kernels for c2), the
HBM roofline of the fused normalization + activation kernels, and the CPU
baseline measured on the host cores on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0         # MI355X HBM3E
MFMA_FP32_PEAK_TFLOPS = 157.3  # MI355X dense FP32 matrix

WORKLOADS = {
    # name: (B, K, H, activation, description)
    "c3": (8192, 4096, 4096, "ELU", "FC 4096->4096 on batch 8192 + batch renorm + ELU, fwd+bwd (dX,dW,db,dgamma,dbeta)"),
    "c2": (4096, 0, 4096, "SELU", "batch renorm + SELU fwd+bwd on [4096 x 4096] (no FC)"),
    "c5": (65536, 256, 256, "LEAKY_RELU", "FC 256->256 on batch 65536 + batch renorm + leaky ReLU, fwd+bwd"),
}
HYPER = dict(momentum=0.99, eps=1e-5, r_max=3.0, d_max=5.0)

# HBM-side bytes per launch (sequence) from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# file's --only parts, calibrated against the plain copy of --only copy
# (profiles/c3_c2_hbm_traffic_pmc.md).  They cannot be measured from inside this process.
MIB = 1024.0 * 1024.0
MEASURED_TRAFFIC_BYTES = {
    "c3": {"gemm": (897.9 + 897.3 + 832.8) / 3.0 * MIB, "norm_act": 1047.0 * MIB},
    "c2": {"norm_act": 528.8 * MIB},
}


def make_inputs(torch, name):
    B, K, H, act, _ = WORKLOADS[name]
    g = torch.Generator(device="cuda")
    g.manual_seed(1234)
    t = {}
    if K:
        t["X"] = torch.randn(B, K, device="cuda", generator=g)
        if name == "c5":  # 1% outliers x50
            t["X"] = torch.where(torch.rand(B, K, device="cuda", generator=g) < 0.01, t["X"] * 50, t["X"])
        lim = (6.0 / (K + H)) ** 0.5
        t["W"] = (torch.rand(H, K, device="cuda", generator=g) * 2 - 1) * lim
        t["bias"] = torch.zeros(H, device="cuda")
        t["gamma"] = torch.ones(H, device="cuda")
        t["beta"] = torch.zeros(H, device="cuda")
        t["Z"] = torch.empty(B, H, device="cuda")
        t["dX"] = torch.empty(B, K, device="cuda")
        t["dW"] = torch.empty(H, K, device="cuda")
        t["db"] = torch.empty(H, device="cuda")
    else:
        s = torch.rand(H, device="cuda", generator=g) * 1.5 + 0.5
        m = torch.rand(H, device="cuda", generator=g) * 2 - 1
        t["Z"] = torch.randn(B, H, device="cuda", generator=g) * s + m
        t["gamma"] = torch.rand(H, device="cuda", generator=g) * 0.4 + 0.8
        t["beta"] = torch.rand(H, device="cuda", generator=g) * 0.2 - 0.1
    t["dY"] = torch.randn(B, H, device="cuda", generator=g)
    t["y"] = torch.empty(B, H, device="cuda")
    t["dZ"] = torch.empty(B, H, device="cuda")
    t["mov_mean"] = torch.zeros(H, device="cuda")
    t["mov_std"] = torch.ones(H, device="cuda")
    t["dgamma"] = torch.zeros(H, device="cuda")
    t["dbeta"] = torch.zeros(H, device="cuda")
    t["stats"] = {k: torch.empty(H, device="cuda") for k in ("mean", "std", "r", "d")}
    return t


class Step:
    """The pieces of one step, callable separately so each can be timed."""

    def __init__(self, dl, pkg, name, t):
        self.dl, self.t = dl, t
        self.B, self.K, self.H, act, _ = WORKLOADS[name]
        self.desc = pkg.Dlmi.desc(pkg.ACT[act], renorm=True, **HYPER)

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

    def fc_norm_fwd(self):
        """Forward of the layer in one call: the GEMM epilogue accumulates the
        batch statistics, so the normalization reads Z only once."""
        t = self.t
        self.dl.fc_norm_act_fwd(self.desc, t["X"], t["W"], t["gamma"], t["beta"], t["mov_mean"], t["mov_std"],
                                Z=t["Z"], out=t["y"], stats=t["stats"])

    def adam(self):
        """Adam step over the layer's weights (not part of the timed step: the
        metric is forward + backward; reported under detail)."""
        t = self.t
        if "m1" not in t:
            import torch
            t["m1"], t["m2"] = torch.zeros_like(t["W"]), torch.zeros_like(t["W"])
        self.dl.opt_adam(t["W"], t["dW"], t["m1"], t["m2"], None, None, 1e-6, 0.9, 0.999, 1e-8, 0.0)

    def copy(self):
        """A plain device copy of one [B, H] tensor (known size): calibrates the
        FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run."""
        self.t["y"].copy_(self.t["dY"])

    def parts(self):
        if self.K:
            return [self.fc_norm_fwd, self.norm_bwd, self.gemm_dx, self.gemm_dw]
        return [self.norm_fwd, self.norm_bwd]

    def __call__(self):
        for p in self.parts():
            p()


def time_events(torch, fn, reps, warmup=2):
    """Average duration (ms) of fn() over `reps` back-to-back calls, measured
    with HIP events recorded on the stream the kernels are launched on."""
    for _ in range(warmup):
        fn()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    s.record()
    for _ in range(reps):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) / reps


def cpu_baseline(name, budget_rows):
    """The reference's OpenMP CPU path (the real reference compiled, if
    oracle/_ref is present; else this repository's restatement of it) on the
    first `budget_rows` rows of the same workload shape, host cores only."""
    import numpy as np
    from oracle.binding import ACT, Oracle, Reference, reference_available
    B, K, H, act, _ = WORKLOADS[name]
    Bs = min(B, budget_rows)
    kind = "reference" if reference_available() else "port"
    cpu = Reference() if kind == "reference" else Oracle()
    nt = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(16, os.cpu_count() or 1)
    nt = max(1, min(nt, os.cpu_count() or 1, 64))
    rng = np.random.default_rng(1234)
    zero, one = np.zeros(H, np.float32), np.ones(H, np.float32)
    dY = rng.standard_normal((Bs, H), dtype=np.float32)
    if K:
        X = rng.standard_normal((Bs, K), dtype=np.float32)
        W = ((rng.random((H, K), dtype=np.float32) * 2 - 1) * np.float32((6.0 / (K + H)) ** 0.5))
    else:
        Z = rng.standard_normal((Bs, H), dtype=np.float32)
    t0 = time.perf_counter()
    if K:
        Z = cpu.fc_fwd(X, W, nt)
    fw = cpu.norm_fwd_train(Z, one, zero, zero, one, HYPER["momentum"], HYPER["eps"], HYPER["r_max"],
                            HYPER["d_max"], True, nt)
    y = cpu.act_fwd(ACT[act], fw["out"], nt)
    dN = cpu.act_bwd(ACT[act], fw["out"], y, dY, nt)
    bw = cpu.norm_bwd(fw["mean"], fw["std"], one, fw["r"], Z, fw["xhat"], dN, renorm=True, nthreads=nt)
    if K:
        cpu.fc_bwd_dx(bw["dx"], W, nthreads=nt)
        cpu.fc_bwd_dw(X, bw["dx"], with_bias=False, nthreads=nt)
    dt = time.perf_counter() - t0
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            model = next(l.split(":", 1)[1].strip() for l in f if l.startswith("model name"))
    except Exception:
        pass
    return {"value": Bs / dt, "unit": "samples/s", "cores": nt, "kind": kind,
            "sample": "first %d of %d rows of the same layer shape, one fwd+bwd pass, %.1f s, OpenMP leaves on %d threads (%s)"
                      % (Bs, B, dt, nt, model)}


def bench_c1(args):
    """Workload c1: MLP 784-512-512-10, batch 128, batch renorm + ReLU hidden layers, softmax +
    cross-entropy output, through the Model / Driver facade.  A step is one forward + error +
    backward + parameter-gradient pass over one batch of 128 rows (data set resident in HBM); every
    64 steps Driver::train ends in one Adam update.  Latency-bound: about 25 kernels of a few
    microseconds each per step, replayed as one recorded HIP graph per batch."""
    import numpy as np
    from __graft_entry__ import load_package
    from oracle.binding import ACT, NORM, OPT
    pkg = load_package()
    from deep_learning_amd.model import Model
    widths, B, per_epoch = [784, 512, 512, 10], 128, 64
    n = B * per_epoch
    rng = np.random.default_rng(1234)
    X = rng.random((n, widths[0]), dtype=np.float32)
    Y = np.eye(widths[-1], dtype=np.float32)[rng.integers(0, widths[-1], n)]

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
        p[o[0]:o[0] + H * K] = ((rng.random(H * K, dtype=np.float32) * 2 - 1) * np.float32((6.0 / (K + H)) ** 0.5))
    M.set_parameters(p)
    M.set_optimizer(OPT["ADAM"], adam_lr=1e-3)
    epochs = max(1, args.steps // per_epoch)
    # the driver launches the first epoch kernel by kernel, records the second into one HIP graph per
    # batch and replays from the third on: at least those two stay outside the timed region
    args.warmup = max(args.warmup, 2 * per_epoch)
    for _ in range(args.warmup // per_epoch):
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
    cpu = None
    if args.cpu_rows != 0:
        from oracle.binding import Oracle, OracleMLP, Reference, reference_available
        kind = "reference" if reference_available() else "port"
        nt = max(1, min(int(os.environ.get("OMP_NUM_THREADS", "0")) or 16, os.cpu_count() or 1, 64))
        R = build((lambda w: Reference().mlp(w)) if kind == "reference" else (lambda w: OracleMLP(Oracle(), w)))
        R.prepare(B, nt)
        if kind == "reference":
            R.set_parameters(p)
        else:
            R.parameters[:] = p
        R.set_optimizer(OPT["ADAM"], adam_lr=1e-3)
        R.train_epoch(X[:B * 4], Y[:B * 4])
        t1 = time.perf_counter()
        R.train_epoch(X, Y)
        dtc = time.perf_counter() - t1
        cpu = {"value": n / dtc, "unit": "samples/s", "cores": nt, "kind": kind,
               "sample": "one Driver::train epoch over the same %d rows in batches of %d, %.1f s, %d OpenMP threads"
                         % (n, B, dtc, nt)}
    out = {"metric": "FC+BRN+act fwd+bwd samples/sec; % HBM peak (norm/act), % FP32 MFMA peak (GEMM)",
           "value": B / (ms * 1e-3), "unit": "samples/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
           "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
           "data": "synthetic",
           "config": {"workload": "c1: MLP 784-512-512-10, batch 128, batch renorm + ReLU, softmax cross-entropy, "
                                  "fwd+bwd per batch, Adam update every 64 batches (Driver::train)",
                      "batch": B, "inputs": "resident in HBM"},
           "roofline": roof, "cpu_baseline": cpu, "detail": {"final_loss": loss, "final_accuracy": accu}}
    print(json.dumps(out))
    M.close()


def bench_c4(args):
    """Workload c4: 16 residual blocks x + Dropout(ISRLU(BRN(FC(x)))), width 2048, batch 1024,
    per-element uint8 keep-mask [16, 1024, 2048] (p_drop 0.1), masked backward; forward + backward
    (dX, dW, dgamma, dbeta per block) assembled from the C ABI leaves.  Everything pre-allocated and
    resident in HBM; the host only enqueues (about 100 calls per step)."""
    import torch
    from __graft_entry__ import load_package
    pkg = load_package()
    dl = pkg.Dlmi(0)  # raises without the HIP library or a GPU
    nblk, H, B, keep = 16, 2048, 1024, 0.9
    g = torch.Generator(device="cuda")
    g.manual_seed(1234)
    dev = dict(device="cuda")
    x0 = torch.randn(B, H, generator=g, **dev)
    lim = (6.0 / (2 * H)) ** 0.5
    Ws = [(torch.rand(H, H, generator=g, **dev) * 2 - 1) * lim for _ in range(nblk)]
    mask = (torch.rand(nblk, B, H, generator=g, **dev) < keep).to(torch.uint8)
    dOut = torch.randn(B, H, generator=g, **dev)
    desc = pkg.Dlmi.desc(pkg.ACT["ISRLU"], renorm=True, dropout=pkg.DROP["BERNOULLI_INVERTED"], mask_per_element=True,
                         dropout_bwd=1, drop_scale=1.0 / keep, **HYPER)
    one, zero = torch.ones(H, **dev), torch.zeros(H, **dev)
    xs = [x0] + [torch.empty(B, H, **dev) for _ in range(nblk)]       # block inputs / outputs
    Zs = [torch.empty(B, H, **dev) for _ in range(nblk)]
    ys = [torch.empty(B, H, **dev) for _ in range(nblk)]
    stats = [{k: torch.empty(H, **dev) for k in ("mean", "std", "r", "d")} for _ in range(nblk)]
    mm, ms = [zero.clone() for _ in range(nblk)], [one.clone() for _ in range(nblk)]
    dWs = [torch.empty(H, H, **dev) for _ in range(nblk)]
    dgs, dbs = [zero.clone() for _ in range(nblk)], [zero.clone() for _ in range(nblk)]
    dZ, dXb = torch.empty(B, H, **dev), torch.empty(B, H, **dev)
    gbuf = [torch.empty(B, H, **dev), torch.empty(B, H, **dev)]

    def step():
        for i in range(nblk):
            dl.fc_norm_act_fwd(desc, xs[i], Ws[i], one, zero, mm[i], ms[i], mask=mask[i], Z=Zs[i], out=ys[i],
                               stats=stats[i])
            dl.identity_add(xs[i], ys[i], out=xs[i + 1])
        gcur = dOut
        for i in reversed(range(nblk)):
            dl.fused_bwd(desc, Zs[i], one, zero, stats[i], gcur, dgs[i], dbs[i], mask=mask[i], out=dZ)
            dl.fc_bwd_dx(dZ, Ws[i], out=dXb)
            dl.fc_bwd_dw(xs[i], dZ, dW=dWs[i])
            nxt = gbuf[i & 1]
            dl.identity_add(gcur, dXb, out=nxt)
            gcur = nxt

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) / args.steps * 1e3
    E = B * H
    t_f = time_events(torch, lambda: dl.fc_fwd(xs[0], Ws[0], None, out=Zs[0]), 20)
    t_x = time_events(torch, lambda: dl.fc_bwd_dx(dZ, Ws[0], out=dXb), 20)
    t_w = time_events(torch, lambda: dl.fc_bwd_dw(xs[0], dZ, dW=dWs[0]), 20)
    flops = 2.0 * B * H * H
    avg = (t_f + t_x + t_w) / 3.0
    roof = {"bound": "mfma", "achieved": flops / (avg * 1e-3) / 1e12, "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
            "traffic": None, "kernel": "k_gemm_f32 at 1024 x 2048 x 2048 (avg of fwd, dX, dW launches; operands cache-resident)"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    t_nf = time_events(torch, lambda: dl.fused_fwd(desc, Zs[0], one, zero, mm[0], ms[0], mask=mask[0], out=ys[0],
                                                   stats=stats[0]), 20)
    t_nb = time_events(torch, lambda: dl.fused_bwd(desc, Zs[0], one, zero, stats[0], dOut, dgs[0], dbs[0], mask=mask[0],
                                                   out=dZ), 20)
    hbm = {"bound": "hbm", "achieved": 35.0 * E / ((t_nf + t_nb) * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
           "traffic": None, "kernels": "fused normalization kernels of one block, 32 + 3 (mask) B/element; the 8 MiB "
                                       "tensors are cache-resident", "ms_fwd": t_nf, "ms_bwd": t_nb}
    hbm["frac"] = hbm["achieved"] / hbm["peak"]
    out = {"metric": "FC+BRN+act fwd+bwd samples/sec; % HBM peak (norm/act), % FP32 MFMA peak (GEMM)",
           "value": B / (ms_step * 1e-3), "unit": "samples/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
           "data": "synthetic",
           "config": {"workload": "c4: 16 residual blocks x + Dropout(ISRLU(BRN(FC x))), width 2048, batch 1024, "
                                  "uint8 keep-mask per element, fwd+bwd", "batch": B, "inputs": "resident in HBM"},
           "roofline": roof, "roofline_norm_act": hbm, "cpu_baseline": None,
           "detail": {"ms_gemm_fwd": t_f, "ms_gemm_dx": t_x, "ms_gemm_dw": t_w, "ms_norm_fwd": t_nf, "ms_norm_bwd": t_nb,
                      "gemm_ms_per_step": 16 * (t_f + t_x + t_w), "norm_ms_per_step": 16 * (t_nf + t_nb)}}
    print(json.dumps(out))
    dl.close()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS) + ["c1", "c4"])
    ap.add_argument("--cpu-rows", type=int, default=-1, help="rows of the CPU baseline sample (0 = skip)")
    ap.add_argument("--only", default="", help="profiling aid: run just this part (gemm_fwd, gemm_dx, gemm_dw, "
                                               "norm_fwd, norm_bwd, fc_norm_fwd, adam, copy) --steps times and exit "
                                               "without a JSON line")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    if args.workload == "c4":
        bench_c4(args)
        return
    if args.workload == "c1":
        if args.steps == 20:
            args.steps = 640  # ten epochs of 64 batches unless told otherwise
        bench_c1(args)
        return

    import torch
    from __graft_entry__ import load_package
    pkg = load_package()
    dl = pkg.Dlmi(0)  # raises if the HIP library or the GPU is missing: no fallback
    name = args.workload
    B, K, H, act, descr = WORKLOADS[name]
    t = make_inputs(torch, name)
    step = Step(dl, pkg, name, t)

    if args.only:
        step()  # every buffer a part reads has been produced once
        part = getattr(step, args.only)
        ms = time_events(torch, part, args.steps, warmup=args.warmup)
        print("%s: %.4f ms per call over %d calls" % (args.only, ms, args.steps), file=sys.stderr)
        dl.close()
        return

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3

    # per-kernel-group timings with HIP events on the launch stream
    E = B * H
    t_nf = time_events(torch, step.norm_fwd, 20)
    t_nb = time_events(torch, step.norm_bwd, 20)
    hbm_bytes = 32.0 * E  # fwd 12 B/element + bwd 20 B/element
    hbm = {"bound": "hbm", "achieved": hbm_bytes / ((t_nf + t_nb) * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
           "traffic": MEASURED_TRAFFIC_BYTES.get(name, {}).get("norm_act"), "kernels": "k_col_stats+k_fwd_finalize+k_fwd_apply / k_bwd_reduce+k_bwd_finalize+k_bwd_apply",
           "ms_fwd": t_nf, "ms_bwd": t_nb, "bytes_fwd": 12.0 * E, "bytes_bwd": 20.0 * E}
    hbm["frac"] = hbm["achieved"] / hbm["peak"]
    detail = {"ms_norm_fwd": t_nf, "ms_norm_bwd": t_nb}
    if K:
        t_gf = time_events(torch, step.gemm_fwd, 10)
        t_gx = time_events(torch, step.gemm_dx, 10)
        t_gw = time_events(torch, lambda: dl.fc_bwd_dw(t["X"], t["dZ"], dW=t["dW"]), 10)
        flops = 2.0 * B * K * H
        avg = (t_gf + t_gx + t_gw) / 3.0
        roof = {"bound": "mfma", "achieved": flops / (avg * 1e-3) / 1e12, "peak": MFMA_FP32_PEAK_TFLOPS,
                "unit": "TFLOP/s", "traffic": MEASURED_TRAFFIC_BYTES.get(name, {}).get("gemm"), "kernel": "k_gemm_f32 (avg of fwd NT, dX NN, dW TN launches)",
                "tflops_fwd": flops / (t_gf * 1e-3) / 1e12, "tflops_dx": flops / (t_gx * 1e-3) / 1e12,
                "tflops_dw": flops / (t_gw * 1e-3) / 1e12}
        roof["frac"] = roof["achieved"] / roof["peak"]
        t_ff = time_events(torch, step.fc_norm_fwd, 10)
        detail.update({"ms_gemm_fwd": t_gf, "ms_gemm_dx": t_gx, "ms_gemm_dw": t_gw, "ms_fc_norm_fwd": t_ff,
                       # epilogue-fused accounting (kept apart from roofline_norm_act): the normalization
                       # forward costs what the fused call takes beyond the plain GEMM and moves 8 B/element
                       "epilogue_fused_norm_fwd": {"ms": t_ff - t_gf, "bytes": 8.0 * E,
                                                   "GBps": 8.0 * E / max(t_ff - t_gf, 1e-6) / 1e6}})
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
    else:
        roof = dict(hbm)

    cpu_rows = args.cpu_rows if args.cpu_rows >= 0 else {"c3": 8192, "c2": 4096, "c5": 65536}[name]  # c3: ~10 s on 16 cores
    cpu = cpu_baseline(name, cpu_rows) if cpu_rows else None

    out = {
        "metric": "FC+BRN+act fwd+bwd samples/sec; % HBM peak (norm/act), % FP32 MFMA peak (GEMM)",
        "value": B / (ms_per_step * 1e-3), "unit": "samples/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": name + ": " + descr, "batch": B, "fan_in": K, "units": H, "activation": act,
                   "norm": "batch renorm rmax=3 dmax=5 momentum=0.99 eps=1e-5", "inputs": "resident in HBM"},
        "roofline": roof, "roofline_norm_act": hbm, "cpu_baseline": cpu, "detail": detail,
    }
    print(json.dumps(out))
    dl.close()


if __name__ == "__main__":
    main()
