"""Writes the golden vectors under tests/golden/ by running the REAL reference
sources (compiled by oracle/Makefile.ref into oracle/_ref/libdlref.so) on
seeded inputs.  Run from the repository root, in a container that holds
/root/reference:

    make -f oracle/Makefile.ref -j8 && python tests/golden/make_golden.py

The fixtures are data only: inputs and the reference's outputs (npz, float32 /
uint8 arrays, loaded with allow_pickle=False).  Every value in an "exp_*" array
was produced by a member function of the reference's DL::v1::Model.
"""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle.binding import ACCU, ACT, DROP, LOSS, NORM, OPT, STATE, Reference, ReferenceNet  # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))
ACTS = ["ELU", "ISRLU", "LEAKY_RELU", "RELU", "SELU", "LINEAR"]
LEAF_SHAPES = [(4, 5, 3), (7, 130, 5), (33, 24, 66)]  # (B, K, H)
THREADS = [0, 3]  # 0 = single-thread leaves, 3 = OpenMP leaves on 3 threads


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def save(name, d):
    """Writes tests/golden/<name> unless the file already holds exactly these
    arrays (an npz is a zip: rewriting it would change its bytes for nothing)."""
    path = os.path.join(OUT, name)
    if os.path.exists(path):
        old = np.load(path, allow_pickle=False)
        if set(old.files) == set(d) and all(np.array_equal(old[k], np.asarray(d[k])) for k in d):
            return
    np.savez_compressed(path, **d)


def leaves(R):
    rng = np.random.default_rng(20240607)
    d = {}
    for ci, (B, K, H) in enumerate(LEAF_SHAPES):
        p = f"c{ci}_"
        X = f32(rng.standard_normal((B, K)))
        W = f32(rng.uniform(-1, 1, (H, K)) * np.sqrt(6.0 / (K + H)))
        bias = f32(rng.uniform(-0.5, 0.5, H))
        x = f32(rng.standard_normal((B, H)) * rng.uniform(0.5, 2, H) + rng.uniform(-1, 1, H))
        gamma = f32(rng.uniform(0.8, 1.2, H))
        beta = f32(rng.uniform(-0.1, 0.1, H))
        mov_mean = f32(rng.uniform(-1, 1, H))
        mov_std = f32(rng.uniform(0.5, 2, H))
        dN = f32(rng.standard_normal((B, H)))
        dZ = f32(rng.standard_normal((B, H)))
        dW0 = f32(rng.standard_normal((H, K)))
        db0 = f32(rng.standard_normal(H))
        mask = (rng.uniform(size=H) < 0.7).astype(np.uint8)
        d.update({p + "shape": np.array([B, K, H]), p + "X": X, p + "W": W, p + "bias": bias, p + "x": x,
                  p + "gamma": gamma, p + "beta": beta, p + "mov_mean": mov_mean, p + "mov_std": mov_std,
                  p + "dN": dN, p + "dZ": dZ, p + "dW0": dW0, p + "db0": db0, p + "mask": mask})
        for nt in THREADS:
            q = f"{p}t{nt}_"
            Z = R.fc_fwd(X, W, nt)
            d[q + "fc_fwd"] = Z
            d[q + "bias_fwd"] = R.bias_fwd(Z, bias, nt)
            # three normalization settings: (a) fresh moving stats, clips do not
            # bind; (b) warm moving stats + tight clips, both bind; (c) plain BN
            settings = dict(
                brn_loose=dict(mm=np.zeros(H), ms=np.ones(H), mom=0.99, rmax=3.0, dmax=5.0, renorm=True),
                brn_tight=dict(mm=mov_mean, ms=mov_std, mom=0.05, rmax=1.1, dmax=0.05, renorm=True),
                bn=dict(mm=mov_mean, ms=mov_std, mom=0.3, rmax=1.0, dmax=0.0, renorm=False))
            for sname, s in settings.items():
                fw = R.norm_fwd_train(x, gamma, beta, s["mm"], s["ms"], s["mom"], 1e-5, s["rmax"],
                                      s["dmax"], s["renorm"], nt)
                for k, v in fw.items():
                    d[f"{q}{sname}_fwd_{k}"] = v
                bw = R.norm_bwd(fw["mean"], fw["std"], gamma, fw["r"], x, fw["xhat"], dN,
                                dgamma_init=gamma * 0.5, dbeta_init=beta * 2, renorm=s["renorm"], nthreads=nt)
                for k, v in bw.items():
                    d[f"{q}{sname}_bwd_{k}"] = v
            d[q + "norm_infer"] = R.norm_fwd_infer(x, gamma, beta, mov_mean, mov_std, nt)
            for a in ACTS:
                y = R.act_fwd(ACT[a], x, nt)
                d[f"{q}act_fwd_{a}"] = y
                d[f"{q}act_bwd_{a}"] = R.act_bwd(ACT[a], x, y, dN, nt)
            d[q + "softmax"] = R.softmax_fwd(x, nt)
            d[q + "drop_inverted"] = R.dropout_fwd(0, x, mask, np.float32(1.0) / np.float32(0.7), nt)
            d[q + "drop_plain"] = R.dropout_fwd(1, x, mask, 0.0, nt)
            d[q + "drop_infer"] = R.dropout_fwd(2, x, None, 0.7, nt)
            d[q + "identity_add"] = R.identity_add(x, dN, nt)
            d[q + "fc_bwd_dx"] = R.fc_bwd_dx(dZ, W, nthreads=nt)
            d[q + "fc_bwd_dx_acc"] = R.fc_bwd_dx(dZ, W, dY_init=f32(np.ones((B, K))), nthreads=nt)
            dW, db = R.fc_bwd_dw(X, dZ, dW_init=dW0, db_init=db0, nthreads=nt)
            d[q + "fc_bwd_dw"] = dW
            d[q + "fc_bwd_db"] = db
    # activation special points (one row): signed zeros, tiny, large, around the knees
    pts = f32([[-0.0, 0.0, -1e-30, 1e-30, -1e-6, 1e-6, -0.5, 0.5, -1.0, 1.0, -5.0, 5.0, -20.0, 20.0,
                -88.0, 88.0, -1e4, 1e4]])
    d["pts"] = pts
    ones = np.ones_like(pts)
    for a in ACTS:
        y = R.act_fwd(ACT[a], pts, 0)
        d[f"pts_fwd_{a}"] = y
        d[f"pts_bwd_{a}"] = R.act_bwd(ACT[a], pts, y, ones, 0)
    save("leaves.npz", d)
    return len(d)


MLP_CASES = {
    # name: (widths, B, per-layer (act, norm, drop, keep), hyper(m, eps, rmax, dmax))
    "mlp_relu_brn": ([8, 6, 6, 3], 5, [("RELU", "BRN", "NONE", 1.0), ("RELU", "BRN", "NONE", 1.0)],
                     (0.99, 1e-5, 3.0, 5.0)),
    "mlp_c1_small": ([20, 16, 16, 10], 12, [("RELU", "BRN", "NONE", 1.0), ("RELU", "BRN", "NONE", 1.0)],
                     (0.99, 1e-5, 3.0, 5.0)),
    "mlp_mixed": ([9, 7, 12, 5, 4], 11,
                  [("SELU", "BRN", "BERNOULLI_INVERTED", 0.8), ("ELU", "NONE", "NONE", 1.0),
                   ("ISRLU", "BRN", "BERNOULLI", 0.6)], (0.3, 1e-3, 1.2, 0.1)),
    # the reference refuses BN and BRN layers in one model (the first BN layer
    # re-allocates arrays the BRN layers already own, normalization.cpp:351), so
    # plain batch normalization gets a model of its own
    "mlp_bn": ([7, 9, 8, 3], 10, [("ISRLU", "BN", "NONE", 1.0), ("SELU", "BN", "BERNOULLI_INVERTED", 0.75)],
               (0.2, 1e-5, 1.0, 0.0)),
    "mlp_lrelu_plain": ([6, 10, 10, 4], 9, [("LEAKY_RELU", "NONE", "NONE", 1.0), ("LEAKY_RELU", "BRN", "NONE", 1.0)],
                        (0.5, 1e-5, 2.0, 1.0)),
}


def glorot(rng, H, K):
    lim = np.sqrt(6.0 / (K + H))
    return f32(rng.uniform(-lim, lim, (H, K)))


def mlps(R):
    d = {}
    for name, (widths, B, hidden, hyper) in MLP_CASES.items():
        rng = np.random.default_rng(sum(map(ord, name)))
        L = len(widths)
        X = f32(rng.uniform(0, 1, (B, widths[0])))
        labels = rng.integers(0, widths[-1], B)
        Y = f32(np.eye(widths[-1])[labels])
        masks = {l: (rng.uniform(size=widths[l]) < hidden[l - 1][3]).astype(np.uint8) for l in range(1, L - 1)}
        d[name + "_widths"] = np.array(widths)
        d[name + "_X"] = X
        d[name + "_Y"] = Y
        d[name + "_hyper"] = f32(hyper)
        for l, mk in masks.items():
            d[f"{name}_mask{l}"] = mk
        params = None
        for nt in THREADS:
            M = R.mlp(widths)
            for l in range(1, L - 1):
                a, n, dr, keep = hidden[l - 1]
                M.set_layer(l, ACT[a], NORM[n], DROP[dr], keep, masks[l] if dr != "NONE" else None)
            M.set_layer(L - 1, ACT["SOFTMAX"])
            M.set_norm_hyper(*hyper)
            M.prepare(B, nt)
            if params is None:
                # harness-generated parameters in the reference's packed layout
                params = M.get_parameters()  # gamma=1, beta=0 from the reference's allocator
                offs = [M.layer_offsets(l) for l in range(L)]
                d[name + "_offsets"] = np.array(offs)
                for l in range(1, L):
                    K, H = widths[l - 1], widths[l]
                    params[offs[l][0]:offs[l][0] + H * K] = glorot(rng, H, K).ravel()
                    params[offs[l][1]:offs[l][1] + H] = f32(rng.uniform(-0.2, 0.2, H))
                    params[offs[l][2]:offs[l][2] + H] = f32(rng.uniform(0.8, 1.2, H))
                    params[offs[l][3]:offs[l][3] + H] = f32(rng.uniform(-0.1, 0.1, H))
                d[name + "_params"] = params.copy()
                d[name + "_P"] = np.array([M.P, M.n_units])
            M.set_parameters(params)
            q = f"{name}_t{nt}_"
            M.step(STATE["TRAINING"], X, Y, backward=True)
            for l in range(1, L):
                for which, wn in ((0, "Z"), (3, "out"), (4, "dZ")):
                    d[f"{q}L{l}_{wn}"] = M.layer_buffer(l, which)
                if l < L - 1:
                    # derivative_outputs aliases the AF units' error array
                    # (ordering.cpp:165), so after the backward pass it holds
                    # dY * f'(pre, post), not dY
                    d[f"{q}L{l}_dAF"] = M.layer_buffer(l, 5)
                    if hidden[l - 1][1] != "NONE":
                        d[f"{q}L{l}_xhat"] = M.layer_buffer(l, 1)
                        d[f"{q}L{l}_nrm"] = M.layer_buffer(l, 2)
                        vecs = ((0, "mean"), (1, "std"), (2, "r"), (3, "d"))
                        for which, wn in vecs if hidden[l - 1][1] == "BRN" else vecs[:2]:
                            d[f"{q}L{l}_{wn}"] = M.layer_vector(l, which)
            d[q + "dparams"] = M.get_dparams()
            mm, ms = M.get_moving()
            d[q + "mov_mean"] = mm
            d[q + "mov_std"] = ms
            # inference forward with the moving statistics just updated
            M.step(STATE["INFERENCE"], X, None, backward=False)
            for l in range(1, L):
                d[f"{q}infer_L{l}_out"] = M.layer_buffer(l, 3)
    save("mlp.npz", d)
    return len(d)


OPT_CASES = {
    # name: (optimizer, keyword settings of ReferenceMLP.set_optimizer)
    "gd_plain": ("GD", dict(lr=0.05, momentum=0.0)),
    "gd_wd": ("GD", dict(lr=0.05, momentum=0.0, weight_decay=0.02, normalized_wd=False)),
    "gd_momentum": ("GD", dict(lr=0.02, momentum=0.9)),
    "gd_momentum_wd_norm": ("GD", dict(lr=0.02, momentum=0.8, weight_decay=0.05, normalized_wd=True)),
    "gd_nesterov": ("GD", dict(lr=0.02, momentum=0.9, nesterov=True)),
    "adam": ("ADAM", dict(adam_lr=0.001)),
    "adam_nobias_wd": ("ADAM", dict(adam_lr=0.01, beta1=0.8, beta2=0.99, eps=1e-6, bias_correction=False,
                                    weight_decay=0.03, normalized_wd=True)),
    "amsgrad": ("AMSGRAD", dict(adam_lr=0.005, beta1=0.7, beta2=0.9)),
    "amsgrad_wd": ("AMSGRAD", dict(adam_lr=0.005, weight_decay=0.01, normalized_wd=False)),
    # a fast-closing band (gamma large), so that both clips bind within the four steps
    "adabound": ("ADABOUND", dict(adam_lr=0.01, lr_final=0.05, gamma=0.5)),
    "adabound_wd_norm": ("ADABOUND", dict(adam_lr=0.01, beta1=0.8, beta2=0.99, lr_final=0.1, gamma=1e-3,
                                          weight_decay=0.03, normalized_wd=True)),
    "amsbound": ("AMSBOUND", dict(adam_lr=0.005, beta1=0.7, beta2=0.9, lr_final=0.02, gamma=0.3)),
    "nosadam": ("NOSADAM", dict(adam_lr=0.002, adam_gamma=0.1)),
    "nosadam_wd": ("NOSADAM", dict(adam_lr=0.002, adam_gamma=0.05, bias_correction=False, weight_decay=0.02,
                                   normalized_wd=False)),
    # the Euclidean-norm constraints around the step.  The gradients have norm ~ sqrt(163) ~ 12.8, the
    # parameter rows ~ sqrt(fan-in): thresholds well away from both, binding and not binding
    "gd_clip_binding": ("GD", dict(lr=0.05, momentum=0.0, clip=4.0)),
    "gd_clip_loose": ("GD", dict(lr=0.05, momentum=0.9, clip=40.0)),
    "adam_maxnorm": ("ADAM", dict(adam_lr=0.05, max_norm=2.0)),
    "gd_clip_maxnorm_wd": ("GD", dict(lr=0.1, momentum=0.5, weight_decay=0.02, clip=6.0, max_norm=2.5)),
    # cosine annealing with warm restarts, (decay of the peak, peak, floor, first period, multiplier): a period
    # of two steps, so the four updates see the peak, the middle, the floor + restart, and the stretched period
    "gd_warm_restarts": ("GD", dict(lr=0.05, momentum=0.9, weight_decay=0.02, normalized_wd=False,
                                    warm_restarts=[0.5, 0.08, 0.001, 2.0, 2.0])),
    "adam_warm_restarts": ("ADAM", dict(adam_lr=0.01, weight_decay=0.01, warm_restarts=[0.7, 0.02, 1e-4, 2.0, 1.5])),
    "amsbound_warm_restarts": ("AMSBOUND", dict(adam_lr=0.005, beta2=0.9, lr_final=0.02, gamma=0.3,
                                                warm_restarts=[1.0, 0.01, 1e-3, 3.0, 2.0])),
    # iRPROP+: [loss, previous loss] installed before each of the four updates (worse on the third);
    # the second case makes both limits of the step size bind and the loss always worse
    "irprop_plus": ("IRPROP_PLUS", dict(rprop_losses=[[3e38, 3e38], [0.9, 1.0], [1.1, 0.9], [1.0, 1.1]])),
    "irprop_plus_limits": ("IRPROP_PLUS", dict(rprop=[3.0, 0.01, 0.02, 0.25, 0.1],
                                               rprop_losses=[[2.0, 1.0], [3.0, 2.0], [4.0, 3.0], [5.0, 4.0]])),
}
OPT_STEPS = 4
OPT_BATCH, OPT_TRAINING_SIZE = 5, 60


def small_brn_model(R, widths, B, nt):
    M = R.mlp(widths)
    for l in range(1, len(widths) - 1):
        M.set_layer(l, ACT["RELU"], NORM["BRN"])
    M.set_layer(len(widths) - 1, ACT["SOFTMAX"])
    M.set_norm_hyper(0.99, 1e-5, 3.0, 5.0)
    M.prepare(B, nt)
    return M


def optimizers(R):
    """(a) Model::Update_Parameter on given gradients, OPT_STEPS times in a row;
    (b) whole training steps (forward, error, backward, derivatives, update) on
    one batch with Adam and with momentum + weight decay."""
    d = {}
    widths = [8, 6, 6, 3]
    rng = np.random.default_rng(77)
    M0 = small_brn_model(R, widths, OPT_BATCH, 0)
    P = M0.P
    p0 = f32(rng.standard_normal(P))
    grads = f32(rng.standard_normal((OPT_STEPS, P)))
    grads[1, ::7] = 0  # zero gradients: second moments stay where they are
    d["opt_p0"], d["opt_grads"] = p0, grads
    d["opt_sizes"] = np.array([OPT_BATCH, OPT_TRAINING_SIZE])
    # (first weight index, units, fan-in) of every layer: what the max-norm constraint walks
    d["opt_weight_rows"] = np.array([[M0.layer_offsets(l)[0], widths[l], widths[l - 1]] for l in range(1, len(widths))])
    # the settings travel with the vectors (JSON text as bytes)
    traj = {"traj_adam": ("ADAM", dict(adam_lr=0.01)),
            "traj_momentum_wd": ("GD", dict(lr=0.1, momentum=0.9, weight_decay=0.01, normalized_wd=True))}
    d["opt_cases_json"] = np.frombuffer(json.dumps({"leaf": OPT_CASES, "traj": traj}).encode(), dtype=np.uint8)
    for name, (kind, kw) in OPT_CASES.items():
        for nt in THREADS:
            M = small_brn_model(R, widths, OPT_BATCH, nt)
            M.set_parameters(p0)
            M.set_optimizer(OPT[kind], **kw)
            if nt == 0:
                mask = M.opt_state(4)
                d[f"opt_{name}_mask"] = mask if mask is not None else np.zeros(0, np.float32)
            for t in range(OPT_STEPS):
                M.set_dparams(grads[t])
                M.update_parameter(OPT_BATCH, OPT_TRAINING_SIZE)
                q = f"opt_{name}_t{nt}_s{t}_"
                d[q + "params"] = M.get_parameters()
                assert not M.get_dparams().any(), "the reference zeroes the consumed gradient"
                for which, wn in ((0, "delta"), (1, "m1"), (2, "m2"), (3, "vhat"), (5, "prev_g"), (6, "steps")):
                    st = M.opt_state(which)
                    if st is not None and t == OPT_STEPS - 1:
                        d[q + wn] = st
    # (b) training trajectories
    for name, (kind, kw) in traj.items():
        widths, B = [20, 16, 16, 10], 12
        rng = np.random.default_rng(sum(map(ord, name)))
        X = f32(rng.uniform(0, 1, (B, widths[0])))
        Y = f32(np.eye(widths[-1])[rng.integers(0, widths[-1], B)])
        d[name + "_X"], d[name + "_Y"], d[name + "_widths"] = X, Y, np.array(widths)
        params = None
        for nt in THREADS:
            M = small_brn_model(R, widths, B, nt)
            if params is None:
                params = M.get_parameters()
                for l in range(1, len(widths)):
                    o = M.layer_offsets(l)
                    K, H = widths[l - 1], widths[l]
                    params[o[0]:o[0] + H * K] = glorot(rng, H, K).ravel()
                d[name + "_params"] = params.copy()
            M.set_parameters(params)
            M.set_optimizer(OPT[kind], **kw)
            for t in range(3):
                M.step(STATE["TRAINING"], X, Y, backward=True)
                if t == 0:
                    d[f"{name}_t{nt}_s0_dparams"] = M.get_dparams()
                M.update_parameter(B, 5 * B)
                d[f"{name}_t{nt}_s{t}_params"] = M.get_parameters()
            mm, ms = M.get_moving()
            d[f"{name}_t{nt}_mov_mean"], d[f"{name}_t{nt}_mov_std"] = mm, ms
    save("optim.npz", d)
    return len(d)


EPOCH_CASES = {
    # name: (widths, n_data, sub-batch, hidden (act, norm, drop, keep), optimizer, settings)
    "epoch_adam_brn": ([20, 16, 16, 10], 50, 16, [("RELU", "BRN", "NONE", 1.0)] * 2, "ADAM",
                       dict(adam_lr=0.01, weight_decay=0.01)),
    "epoch_nesterov_dropout": ([12, 24, 9, 5], 37, 37, [("ELU", "BRN", "BERNOULLI_INVERTED", 0.8),
                                                         ("LEAKY_RELU", "NONE", "NONE", 1.0)], "GD",
                               dict(lr=0.05, momentum=0.9, nesterov=True)),
    "epoch_gd_even_batches": ([10, 8, 8, 4], 48, 12, [("SELU", "BN", "NONE", 1.0), ("ISRLU", "BN", "NONE", 1.0)], "GD",
                              dict(lr=0.1, momentum=0.0, weight_decay=0.02, normalized_wd=False)),
    # iRPROP+ with the epoch driver keeping the two losses; a start step large enough for the loss to get worse
    "epoch_irprop_plus": ([10, 8, 8, 4], 40, 16, [("ELU", "BRN", "NONE", 1.0), ("RELU", "NONE", "NONE", 1.0)], "IRPROP_PLUS",
                          dict(rprop=[1.2, 0.5, 1e-6, 50.0, 0.3])),
}
EPOCHS = 3


def epochs(R):
    """Driver::train three times, then Driver::evalt, on one small data set:
    loss, accuracy, parameters and moving statistics after every epoch."""
    d = {"epoch_cases_json": np.frombuffer(json.dumps(EPOCH_CASES).encode(), dtype=np.uint8)}
    for name, (widths, n, sub, hidden, kind, kw) in EPOCH_CASES.items():
        rng = np.random.default_rng(sum(map(ord, name)))
        L = len(widths)
        X = f32(rng.uniform(0, 1, (n, widths[0])))
        Y = f32(np.eye(widths[-1])[rng.integers(0, widths[-1], n)])
        masks = {l: (rng.uniform(size=widths[l]) < hidden[l - 1][3]).astype(np.uint8) for l in range(1, L - 1)}
        d[name + "_X"], d[name + "_Y"] = X, Y
        for l, mk in masks.items():
            d[f"{name}_mask{l}"] = mk
        params = None
        for nt in THREADS:
            M = R.mlp(widths)
            for l in range(1, L - 1):
                a, nm, dr, keep = hidden[l - 1]
                M.set_layer(l, ACT[a], NORM[nm], DROP[dr], keep, masks[l] if dr != "NONE" else None)
            M.set_layer(L - 1, ACT["SOFTMAX"])
            M.set_norm_hyper(0.9, 1e-5, 3.0, 5.0)
            M.prepare(sub, nt)
            if params is None:
                params = M.get_parameters()
                for l in range(1, L):
                    o = M.layer_offsets(l)
                    K, H = widths[l - 1], widths[l]
                    params[o[0]:o[0] + H * K] = glorot(rng, H, K).ravel()
                d[name + "_params"] = params.copy()
            M.set_parameters(params)
            M.set_optimizer(OPT[kind], **kw)
            q = f"{name}_t{nt}_"
            la = []
            for e in range(EPOCHS):
                la.append(M.train_epoch(X, Y, resample_masks=False))
                d[f"{q}e{e}_params"] = M.get_parameters()
            la.append(M.evalt(X, Y))
            d[q + "loss_accu"] = np.array(la, dtype=np.float64)  # rows: epochs 0..2 (training), evaluation
            mm, ms = M.get_moving()
            d[q + "mov_mean"], d[q + "mov_std"] = mm, ms
    save("epoch.npz", d)
    return len(d)


VARIANT_CASES = {
    # name: (widths, B, hidden (act, norm, drop, keep, normalization before the activation), hyper)
    "var_norm_after": ([9, 7, 12, 5, 4], 11, [("SELU", "BRN", "BERNOULLI_INVERTED", 0.8, False),
                                              ("ELU", "BRN", "NONE", 1.0, True),
                                              ("ISRLU", "BRN", "BERNOULLI", 0.6, False)], (0.3, 1e-3, 1.2, 0.1)),
    "var_norm_after_bn": ([6, 10, 8, 3], 13, [("LEAKY_RELU", "BN", "NONE", 1.0, False),
                                              ("RELU", "BN", "BERNOULLI_INVERTED", 0.7, False)], (0.1, 1e-5, 1.0, 0.0)),
    "var_before_dropout": ([8, 6, 6, 3], 9, [("ELU", "BRN", "BERNOULLI", 0.5, True),
                                             ("SELU", "NONE", "BERNOULLI_INVERTED", 0.5, True)], (0.9, 1e-5, 3.0, 5.0)),
}


def variants(R):
    """Layer orderings and propagation states beyond mlp.npz: normalization after
    the activation (fwp_st.cpp:466-511, bwp_st.cpp:559-606) and the
    PROPAGATION::UPDATE_BATCH_NORM forward (batch statistics, no dropout mask)."""
    d = {"variant_cases_json": np.frombuffer(json.dumps(VARIANT_CASES).encode(), dtype=np.uint8)}
    for name, (widths, B, hidden, hyper) in VARIANT_CASES.items():
        rng = np.random.default_rng(sum(map(ord, name)))
        L = len(widths)
        X = f32(rng.uniform(0, 1, (B, widths[0])))
        Y = f32(np.eye(widths[-1])[rng.integers(0, widths[-1], B)])
        masks = {l: (rng.uniform(size=widths[l]) < hidden[l - 1][3]).astype(np.uint8) for l in range(1, L - 1)}
        d[name + "_X"], d[name + "_Y"] = X, Y
        for l, mk in masks.items():
            d[f"{name}_mask{l}"] = mk
        params = None
        for nt in THREADS:
            M = R.mlp(widths)
            for l in range(1, L - 1):
                a, nm, dr, keep, before = hidden[l - 1]
                M.set_layer(l, ACT[a], NORM[nm], DROP[dr], keep, masks[l] if dr != "NONE" else None, norm_before=before)
            M.set_layer(L - 1, ACT["SOFTMAX"])
            M.set_norm_hyper(*hyper)
            M.prepare(B, nt)
            if params is None:
                params = M.get_parameters()
                for l in range(1, L):
                    o = M.layer_offsets(l)
                    K, H = widths[l - 1], widths[l]
                    params[o[0]:o[0] + H * K] = glorot(rng, H, K).ravel()
                    params[o[1]:o[1] + H] = f32(rng.uniform(-0.2, 0.2, H))
                    params[o[2]:o[2] + H] = f32(rng.uniform(0.8, 1.2, H))
                    params[o[3]:o[3] + H] = f32(rng.uniform(-0.1, 0.1, H))
                d[name + "_params"] = params.copy()
            M.set_parameters(params)
            q = f"{name}_t{nt}_"
            M.step(STATE["TRAINING"], X, Y, backward=True)
            for l in range(1, L):
                d[f"{q}train_L{l}_out"] = M.layer_buffer(l, 6)
                d[f"{q}train_L{l}_dZ"] = M.layer_buffer(l, 4)
            d[q + "dparams"] = M.get_dparams()
            d[q + "train_mov_mean"], d[q + "train_mov_std"] = M.get_moving()
            M.step(STATE["UPDATE_BATCH_NORM"], X, None, backward=False)
            for l in range(1, L):
                d[f"{q}ubn_L{l}_out"] = M.layer_buffer(l, 6)
            d[q + "ubn_mov_mean"], d[q + "ubn_mov_std"] = M.get_moving()
            M.step(STATE["INFERENCE"], X, None, backward=False)
            for l in range(1, L):
                d[f"{q}infer_L{l}_out"] = M.layer_buffer(l, 6)
    save("variants.npz", d)
    return len(d)


SHORTCUT_CASES = [(9, 6, 6, 0), (9, 10, 6, 2), (9, 6, 10, 3), (5, 8, 4, 4), (33, 130, 66, 17), (1, 3, 3, 0)]  # B, HA, HB, padding (0 only with equal widths)


def shortcuts(R):
    """Zero-padded identity shortcut of a residual block and the routing of its
    gradient (fwp_st.cpp:5051-5112, bwp_st.cpp:1047-1068, 1112-1175)."""
    rng = np.random.default_rng(5051)
    d = {"shortcut_cases": np.array(SHORTCUT_CASES)}
    for ci, (B, HA, HB, pad) in enumerate(SHORTCUT_CASES):
        a, b = f32(rng.standard_normal((B, HA))), f32(rng.standard_normal((B, HB)))
        g = f32(rng.standard_normal((B, max(HA, HB))))       # gradient of the block's output
        da0, db0 = f32(rng.standard_normal((B, HA))), f32(rng.standard_normal((B, HB)))
        d[f"sc{ci}_a"], d[f"sc{ci}_b"], d[f"sc{ci}_g"], d[f"sc{ci}_da0"], d[f"sc{ci}_db0"] = a, b, g, da0, db0
        for nt in THREADS:
            d[f"sc{ci}_t{nt}_out"] = R.zero_padded_identity_fwd(a, b, pad, nt)
            d[f"sc{ci}_t{nt}_da"] = R.residual_bwd(g, da0, pad, nt)
            d[f"sc{ci}_t{nt}_db"] = R.residual_bwd(g, db0, pad, nt)
    save("shortcut.npz", d)
    return len(d)


RESNET_CASES = {
    # name: (layer list, batch, {entry: (activation or None, norm, dropout, keep)}, hyper)
    "res_two_blocks": ([("FC", 8), ("FC", 6), ("RES", 2), ("FC", 6), ("FC", 6), ("RES", 2), ("FC", 5), ("FC", 6), ("FC", 3)], 7,
                       {1: ("RELU", "BRN", "NONE", 1.0), 2: (None, "BRN", "NONE", 1.0), 3: ("ELU", "BRN", "NONE", 1.0),
                        4: ("ELU", "BRN", "NONE", 1.0), 5: (None, "NONE", "NONE", 1.0), 6: ("SELU", "BRN", "NONE", 1.0),
                        7: ("SELU", "NONE", "NONE", 1.0)}, (0.5, 1e-5, 2.0, 1.0)),
    "res_padded_narrow_block": ([("FC", 8), ("FC", 6), ("RES", 2), ("FC", 7), ("FC", 4), ("FC", 3)], 9,
                                {1: ("RELU", "BRN", "NONE", 1.0), 2: (None, "BRN", "NONE", 1.0),
                                 3: ("ISRLU", "BRN", "NONE", 1.0), 4: ("LEAKY_RELU", "BRN", "NONE", 1.0)},
                                (0.9, 1e-5, 3.0, 5.0)),
    "res_dropout_wide_block": ([("FC", 8), ("FC", 6), ("RES", 3), ("FC", 7), ("FC", 5), ("FC", 9), ("RES", 2), ("FC", 9),
                                ("FC", 4), ("FC", 3)], 11,
                               {1: ("RELU", "BN", "BERNOULLI_INVERTED", 0.7), 2: (None, "BN", "NONE", 1.0),
                                3: ("ISRLU", "BN", "NONE", 1.0), 4: ("LEAKY_RELU", "NONE", "BERNOULLI", 0.6),
                                5: ("ELU", "BN", "BERNOULLI_INVERTED", 0.8), 7: ("SELU", "BN", "NONE", 1.0),
                                8: ("RELU", "BN", "BERNOULLI_INVERTED", 0.5)}, (0.3, 1e-4, 1.0, 0.0)),
}


RESNET_EPOCH_CASE = "res_dropout_wide_block"


def resnets(R):
    """Layer lists with the reference's residual blocks (fwp_st.cpp:3876-4442,
    bwp_st.cpp:80-185, 345-541): outputs of every entry in the three propagation
    states, the error of every FC layer, parameter gradients, moving statistics."""
    d = {"resnet_cases_json": np.frombuffer(json.dumps({k: [v[0], v[1], {str(a): b for a, b in v[2].items()}, v[3]]
                                                        for k, v in RESNET_CASES.items()}).encode(), dtype=np.uint8)}
    for name, (layers, B, cfg, hyper) in RESNET_CASES.items():
        rng = np.random.default_rng(sum(map(ord, name)))
        n = len(layers)
        X = f32(rng.uniform(0, 1, (B, layers[0][1])))
        Y = f32(np.eye(layers[-1][1])[rng.integers(0, layers[-1][1], B)])
        d[name + "_X"], d[name + "_Y"] = X, Y
        unit_masks = {l: (rng.uniform(size=64) < c[3]).astype(np.uint8) for l, c in cfg.items() if c[2] != "NONE"}
        params = None
        for nt in THREADS:
            M = ReferenceNet(R, layers)
            for l, (a, nm, dr, keep) in cfg.items():
                M.set_layer(l, ACT[a] if a else 0, NORM[nm], DROP[dr], keep)
            M.set_layer(n - 1, ACT["SOFTMAX"])
            M.set_norm_hyper(*hyper)
            # dropout units of a block layer are as many as its inputs: known once the normalization is set up
            for l, mk in unit_masks.items():
                nu = M.info(l)["n_unit"]
                M._masks[l] = mk[:nu].copy()
                d[f"{name}_mask{l}"] = mk[:nu].copy()
            M.prepare(B, nt)
            if params is None:
                d[name + "_info"] = np.array([list(M.info(l).values()) for l in range(n)])
                d[name + "_P"] = np.array([M.P, M.n_units])
                params = M.get_parameters()  # gamma 1, beta 0 from the reference's allocator
                nwb = M.info(0)["gamma"]     # weights and biases come first
                params[:nwb] = f32(rng.uniform(-0.5, 0.5, nwb))
                params[nwb:nwb + M.n_units] = f32(rng.uniform(0.8, 1.2, M.n_units))
                params[nwb + M.n_units:] = f32(rng.uniform(-0.1, 0.1, M.n_units))
                d[name + "_params"] = params.copy()
            M.set_parameters(params)
            q = f"{name}_t{nt}_"
            for st in ("TRAINING", "UPDATE_BATCH_NORM", "INFERENCE"):
                M.step(STATE[st], X, Y, backward=(st == "TRAINING"))
                for l in range(1, n):
                    d[f"{q}{st}_L{l}_out"] = M.layer_output(l)
                if st == "TRAINING":
                    for l in M.fc_layers():
                        d[f"{q}L{l}_dZ"] = M.layer_error(l)
                    d[q + "dparams"] = M.get_dparams()
                    d[q + "mov_mean"], d[q + "mov_std"] = M.get_moving()
    # The whole caller-side chain on the network with dropout inside its blocks: Glorot
    # initialization from a seeded generator, two Driver::train epochs over 30 rows in
    # sub-batches of 11 (one Nesterov-momentum step each), then Driver::evalt.
    name = RESNET_EPOCH_CASE
    layers, B, cfg, hyper = RESNET_CASES[name]
    rng = np.random.default_rng(99)
    X = f32(rng.uniform(0, 1, (30, layers[0][1])))
    Y = f32(np.eye(layers[-1][1])[rng.integers(0, layers[-1][1], 30)])
    d["epoch_X"], d["epoch_Y"] = X, Y
    for nt in THREADS:
        M = ReferenceNet(R, layers)
        for l, (a, nm, dr, keep) in cfg.items():
            M.set_layer(l, ACT[a] if a else 0, NORM[nm], DROP[dr], keep)
        M.set_layer(len(layers) - 1, ACT["SOFTMAX"])
        M.set_norm_hyper(*hyper)
        for l in cfg:
            if f"{name}_mask{l}" in d:
                M._masks[l] = d[f"{name}_mask{l}"]
        M.prepare(B, nt)
        M.glorot_uniform(2024, 0.0)
        d[f"epoch_t{nt}_init"] = M.get_parameters()
        # momentum rather than Adam: the bias of an un-normalized layer that feeds a batch
        # normalization has an analytically zero gradient, and Adam turns the rounding noise
        # computed in its place into full-size steps of random sign
        M.set_optimizer(OPT["GD"], lr=0.01, momentum=0.9, nesterov=True, weight_decay=0.01)
        la = []
        for e in range(2):
            la.append(M.train_epoch(X, Y, resample_masks=False))
            d[f"epoch_t{nt}_e{e}_params"] = M.get_parameters()
        la.append(M.evalt(X, Y))
        d[f"epoch_t{nt}_loss_accu"] = np.array(la, dtype=np.float64)
        d[f"epoch_t{nt}_mov_mean"], d[f"epoch_t{nt}_mov_std"] = M.get_moving()
    save("resnet.npz", d)
    return len(d)


INIT_CASES = {
    # name: (layer list, {entry: activation}, {entry: norm}, seed, bias, None for Glorot or (lower, upper))
    "glorot_plain": ([("FC", 8), ("FC", 20), ("FC", 30), ("FC", 12), ("FC", 5)],
                     {1: "RELU", 2: "ELU", 3: "LEAKY_RELU", 4: "SOFTMAX"}, {2: "BRN"}, 123, 0.0, None),
    "glorot_selu_default": ([("FC", 7), ("FC", 16), ("FC", 9), ("FC", 11), ("FC", 3)],
                            {1: "SELU", 3: "ISRLU", 4: "SOFTMAX"}, {}, 5489, 0.25, None),  # entry 2 keeps the sigmoid default
    "glorot_two_blocks": ([("FC", 6), ("FC", 10), ("RES", 2), ("FC", 14), ("FC", 18), ("RES", 3), ("FC", 22), ("FC", 26),
                           ("FC", 30), ("FC", 34), ("FC", 4)],
                          {1: "ELU", 3: "ELU", 4: "ELU", 6: "ELU", 7: "ELU", 8: "ELU", 9: "ELU", 10: "SOFTMAX"},
                          {1: "BN", 2: "BN", 4: "BN"}, 77, 0.5, None),
    "glorot_block_gains": ([("FC", 6), ("FC", 10), ("RES", 1), ("FC", 14), ("FC", 9), ("RES", 2), ("FC", 5), ("FC", 12),
                            ("FC", 4)],
                           {1: "LINEAR", 3: "RELU", 4: "SELU", 6: "SELU", 7: "RELU", 8: "SOFTMAX"}, {3: "BRN"}, 1, 0.0, None),
    "uniform_plain": ([("FC", 8), ("FC", 20), ("FC", 5)], {1: "RELU", 2: "SOFTMAX"}, {1: "BN"}, 9, 0.1, (-0.3, 0.7)),
    "uniform_block": ([("FC", 6), ("FC", 10), ("RES", 2), ("FC", 14), ("FC", 8), ("FC", 4)],
                      {1: "ELU", 3: "ELU", 4: "RELU", 5: "SOFTMAX"}, {2: "BRN", 3: "BRN"}, 31337, -0.2, (-1.0, 1.0)),
}


def inits(R):
    """Uniform weight initializers (glorot.cpp:225-359, uniform.cpp:26-90) with the
    model's generator seeded: the parameter vector and the moving statistics after
    the call, from a model whose parameters and statistics held other values."""
    d = {"init_cases_json": np.frombuffer(json.dumps({k: [v[0], {str(a): b for a, b in v[1].items()},
                                                         {str(a): b for a, b in v[2].items()}, v[3], v[4], v[5]]
                                                     for k, v in INIT_CASES.items()}).encode(), dtype=np.uint8)}
    for name, (layers, acts, norms, seed, bias, rng_bounds) in INIT_CASES.items():
        M = ReferenceNet(R, layers)
        for l in sorted(set(acts) | set(norms)):
            M.set_layer(l, ACT[acts[l]] if l in acts else 0, NORM[norms.get(l, "NONE")])
        M.prepare(4)
        rng = np.random.default_rng(seed)
        M.set_parameters(f32(rng.uniform(-2, 2, M.P)))
        M.set_moving(f32(rng.uniform(-2, 2, M.n_units)), f32(rng.uniform(1, 3, M.n_units)))
        if rng_bounds is None:
            M.glorot_uniform(seed, bias)
        else:
            M.init_uniform(seed, bias, *rng_bounds)
        d[name + "_info"] = np.array([list(M.info(l).values()) for l in range(len(layers))])
        d[name + "_P"] = np.array([M.P, M.n_units])
        d[name + "_params"] = M.get_parameters()
        d[name + "_mov_mean"], d[name + "_mov_std"] = M.get_moving()
    save("init.npz", d)
    return len(d)


MASK_CASE = dict(widths=[8, 40, 30, 20, 25, 5], seed=42,
                 dropout={1: ("BERNOULLI", 0.6), 2: ("BERNOULLI_INVERTED", 0.7), 3: ("BERNOULLI", 0.0), 4: ("BERNOULLI", 0.3)})


def dropout_masks(R):
    """Model::Dropout_Bernoulli (bernoulli_st.cpp:27-100) twice in a row on a single-thread model
    whose first generator was seeded: the per-unit masks of every layer after each call."""
    c = MASK_CASE
    d = {"mask_case_json": np.frombuffer(json.dumps({"widths": c["widths"], "seed": c["seed"],
                                                     "dropout": {str(k): v for k, v in c["dropout"].items()}}).encode(),
                                         dtype=np.uint8)}
    M = R.mlp(c["widths"])
    for l, (kind, keep) in c["dropout"].items():
        M.set_layer(l, ACT["RELU"], NORM["NONE"], DROP[kind], keep)
    M.set_layer(len(c["widths"]) - 1, ACT["SOFTMAX"])
    M.prepare(4, 0)
    for l in c["dropout"]:
        d[f"mask_initial_L{l}"] = M.dropout_mask(l, c["widths"][l])
    for call in range(2):
        M.dropout_bernoulli(c["seed"] if call == 0 else None)
        for l in c["dropout"]:
            d[f"mask_call{call}_L{l}"] = M.dropout_mask(l, c["widths"][l])
    save("masks.npz", d)
    return len(d)


# name: (widths, B, output activation, loss, accuracy, acc_var, kind of targets)
REGRESS_CASES = {
    "linear_mse_distance": ([7, 12, 5], 19, "LINEAR", "MSE", "DISTANCE", 0.3, "real"),
    "elu_mae_sign": ([6, 9, 4], 13, "ELU", "MAE", "SIGN", 0.49, "signed"),
    "isrlu_l2_directional": ([5, 8, 3], 11, "ISRLU", "L2", "DIRECTIONAL", 0.49, "real"),
    "selu_rmse_distance": ([9, 14, 6], 23, "SELU", "RMSE", "DISTANCE", 0.49, "real"),
    "lrelu_me_sign": ([4, 10, 7], 16, "LEAKY_RELU", "ME", "SIGN", 0.49, "signed"),
    "relu_l1_distance": ([8, 11, 2], 9, "RELU", "L1", "DISTANCE", 0.1, "real"),
    "linear_ce_ce": ([6, 10, 4], 15, "LINEAR", "CROSS_ENTROPY", "CROSS_ENTROPY", 0.49, "onehot"),
    "linear_mse_wide": ([20, 40, 130], 37, "LINEAR", "MSE", "DISTANCE", 0.49, "real"),
    "sigmoid_net_mse_distance": ([8, 13, 9, 5], 21, "SIGMOID", "MSE", "DISTANCE", 0.25, "unit"),
    "tanh_net_mae_sign": ([7, 11, 6], 17, "TANH", "MAE", "SIGN", 0.49, "signed"),
    "sigmoid_ce_ce": ([6, 10, 4], 15, "SIGMOID", "CROSS_ENTROPY", "CROSS_ENTROPY", 0.49, "onehot"),
}
# activation of the hidden layers where it is not ELU
REGRESS_HIDDEN = {"sigmoid_net_mse_distance": "SIGMOID", "tanh_net_mae_sign": "TANH"}


def regressions(R):
    """Output layers with an element-wise activation and the regression losses
    (compute_error_st.cpp:80-123, compute_loss.cpp:25-138, loss.cpp:98-221): one
    training step with its seed gradient, loss and accuracy, then three epochs of
    Nesterov momentum through the epoch driver with the loss it reports."""
    d = {"regress_cases_json": np.frombuffer(json.dumps(REGRESS_CASES).encode(), dtype=np.uint8),
         "regress_hidden_json": np.frombuffer(json.dumps(REGRESS_HIDDEN).encode(), dtype=np.uint8)}
    for name, (widths, B, out_act, loss, accu, acc_var, targets) in REGRESS_CASES.items():
        rng = np.random.default_rng(sum(map(ord, name)))
        L = len(widths)
        X = f32(rng.uniform(-1, 1, (B, widths[0])))
        hidden = ACT[REGRESS_HIDDEN.get(name, "ELU")]
        if targets == "onehot":
            Y = f32(np.eye(widths[-1])[rng.integers(0, widths[-1], B)])
        elif targets == "unit":
            Y = f32(rng.uniform(0, 1, (B, widths[-1])))
        else:
            Y = f32(rng.uniform(-1, 1, (B, widths[-1])))
            if targets == "signed":
                Y[rng.uniform(size=Y.shape) < 0.2] = 0.0
        d[name + "_X"], d[name + "_Y"] = X, Y
        params = None
        for nt in THREADS:
            M = R.mlp(widths)
            for l in range(1, L - 1):
                M.set_layer(l, hidden, NORM["BRN"])
            M.set_layer(L - 1, ACT[out_act])
            M.prepare(B, nt)
            M.set_loss(loss, accu, acc_var)
            if params is None:
                M.glorot_uniform(sum(map(ord, name)))
                params = M.get_parameters()
                d[name + "_params"] = params.copy()
            M.set_parameters(params)
            q = f"{name}_t{nt}_"
            M.reset_loss()
            M.step(STATE["TRAINING"], X, Y, backward=True)
            for l in range(1, L):
                d[f"{q}L{l}_Z"] = M.layer_buffer(l, 0)
                d[f"{q}L{l}_out"] = M.layer_buffer(l, 6)
                d[f"{q}L{l}_dZ"] = M.layer_buffer(l, 4)
            d[q + "dparams"] = M.get_dparams()
            d[q + "loss_accu"] = np.array(M.loss_accu(B))
            if targets == "onehot":  # clipped probabilities give gradients of 1e7: one step is enough
                continue
            # the epoch driver on the same data: sub-batches of 7, one update per epoch
            M2 = R.mlp(widths)
            for l in range(1, L - 1):
                M2.set_layer(l, hidden, NORM["BRN"])
            M2.set_layer(L - 1, ACT[out_act])
            M2.set_norm_hyper(0.5, 1e-5, 3.0, 5.0)
            M2.prepare(7, nt)
            M2.set_loss(loss, accu, acc_var)
            M2.set_parameters(params)
            M2.set_optimizer(OPT["GD"], lr=0.01, momentum=0.9, nesterov=True)
            rep = []
            for _ in range(3):
                rep.append(M2.train_epoch(X, Y))
            rep.append(M2.evalt(X, Y))
            d[q + "epoch_reports"] = np.array(rep)
            d[q + "epoch_params"] = M2.get_parameters()
    save("regress.npz", d)
    return len(d)


if __name__ == "__main__":
    R = Reference()
    only = sys.argv[1:]  # names of the fixtures to write; all of them without arguments
    for label, fn in [("leaves", leaves), ("mlp", mlps), ("optim", optimizers), ("epoch", epochs), ("variants", variants),
                      ("shortcut", shortcuts), ("resnet", resnets), ("init", inits), ("masks", dropout_masks),
                      ("regress", regressions)]:
        if not only or label in only:
            print(label + ":", fn(R), "arrays")
