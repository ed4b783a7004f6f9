"""TEST INFRASTRUCTURE — numpy/ctypes bindings for the two CPU checkers.

* ``Oracle``  → oracle/libdloracle.so, this repository's CPU restatement of the
  reference's FC / batch-(re)norm / activation leaves (oracle/dl_oracle.c).
* ``Reference`` → oracle/_ref/libdlref.so, the real reference sources compiled by
  oracle/Makefile.ref (only present where that build was run; the sources do
  not travel).

Both expose the same leaf interface so a test can be parametrized over them.
Only tests/, ``__graft_entry__.smoke()`` and ``bench.py``'s cpu_baseline leg may
import this module; the product (deep-learning_amd/) never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(_HERE, "libdloracle.so")
REF_SO = os.path.join(_HERE, "_ref", "libdlref.so")

c_sz = ctypes.c_size_t
c_int = ctypes.c_int
c_f = ctypes.c_float
c_d = ctypes.c_double
vp = ctypes.c_void_p

# ACTIVATION / LAYER_NORM / LAYER_DROPOUT / PROPAGATION values of the reference
# (v1/data/enum/activation.hpp:24-53, layer_norm.hpp:24-26,
#  layer_dropout.hpp:24-28, propagation.hpp)
ACT = dict(ELU=3, ISRLU=10, LINEAR=11, LEAKY_RELU=14, RELU=16, SELU=17, SIGMOID=18, SOFTMAX=22, TANH=23)
NORM = dict(NONE=0, BN=1, BRN=2)
DROP = dict(NONE=0, BERNOULLI=2, BERNOULLI_INVERTED=3)
STATE = dict(INFERENCE=0, TRAINING=1, UPDATE_BATCH_NORM=2)
# v1/data/enum/optimizer.hpp:24-42
# v1/data/enum/loss_fn.hpp:22-71
LOSS = dict(CROSS_ENTROPY=2, L1=3, L2=4, MAE=5, MAPE=6, ME=9, MSE=10, RMSE=11, SMAPE=12)
ACCU = dict(CROSS_ENTROPY=1, DIRECTIONAL=2, DISTANCE=3, R=4, SIGN=5)
OPT = dict(NONE=0, ADABOUND=1, ADAM=2, AMSBOUND=4, AMSGRAD=5, GD=6, IRPROP_PLUS=8, NOSADAM=9)
_ADAM_FAMILY = (1, 2, 4, 5, 9)


class HarnessRng:
    """The benchmark harness's input generator (oracle/harness_rng.c): one mt19937_64 stream per
    tensor, seed = base + tensor id; both sides of bench.py are fed the arrays it returns."""

    def __init__(self, base_seed=1234):
        if not os.path.exists(ORACLE_SO):
            build_oracle()
        self.lib = ctypes.CDLL(ORACLE_SO)
        self.base = int(base_seed)

    def raw(self, tensor_id, n):
        out = np.empty(n, np.uint64)
        self.lib.dlo_rng_raw(ctypes.c_uint64(self.base + tensor_id), c_sz(n), _ptr(out))
        return out

    def uniform(self, tensor_id, shape, lo=0.0, hi=1.0):
        out = np.empty(shape, np.float32)
        self.lib.dlo_rng_uniform(ctypes.c_uint64(self.base + tensor_id), c_sz(out.size), c_f(lo), c_f(hi), _ptr(out))
        return out

    def normal(self, tensor_id, shape):
        out = np.empty(shape, np.float32)
        self.lib.dlo_rng_normal(ctypes.c_uint64(self.base + tensor_id), c_sz(out.size), _ptr(out))
        return out

    def bernoulli_u8(self, tensor_id, shape, keep):
        out = np.empty(shape, np.uint8)
        self.lib.dlo_rng_bernoulli_u8(ctypes.c_uint64(self.base + tensor_id), c_sz(out.size), c_f(keep), _ptr(out))
        return out

    def index(self, tensor_id, n, k):
        out = np.empty(n, np.uint32)
        self.lib.dlo_rng_index(ctypes.c_uint64(self.base + tensor_id), c_sz(n), ctypes.c_uint32(k), _ptr(out))
        return out


def build_oracle():
    subprocess.run(["make", "-C", _HERE], check=True, stdout=subprocess.DEVNULL)


def _ptr(a):
    return None if a is None else a.ctypes.data_as(vp)


class OptimizerHost:
    """The host arithmetic around an optimizer leaf, in float like the reference:
    time step, bias-corrected step size (adam.cpp:50-54), normalized weight decay
    (train.cpp:278-283; GD scales wd by lr_scale = 1 without warm restarts,
    gradient_descent.cpp:72-75).  `leaves` is anything with opt_gd /
    opt_gd_momentum / opt_adam updating float32 arrays in place."""

    def __init__(self, leaves, n, kind, lr=0.01, momentum=0.9, nesterov=False, adam_lr=0.001, beta1=0.9,
                 beta2=0.999, eps=1e-8, bias_correction=True, weight_decay=0.0, normalized_wd=True, mask=None,
                 lr_final=0.1, gamma=1e-3, adam_gamma=0.1, clip=None, max_norm=0.0, weight_rows=(),
                 rprop=(1.2, 0.5, 1e-6, 50.0, 0.1), rprop_losses=None, warm_restarts=None):
        f = np.float32
        # warm_restarts: None or (decay of the peak rate, peak rate, floor, first period, period multiplier)
        self.wr = None if warm_restarts is None else dict(zip(("decay", "max", "min", "T", "mult"),
                                                              (f(v) for v in warm_restarts)))
        # iRPROP+: (increase, decrease, delta_min, delta_max, delta_zero), model.hpp:3331-3335.  loss_rprop /
        # loss_rprop_tm1 are the caller's (drivers/driver.cpp:232, 263); rprop_losses, if given, is the
        # [loss, loss_tm1] pair to install before each update (for replaying a recorded sequence).
        self.rprop = tuple(f(v) for v in rprop)
        self.loss_rprop = self.loss_rprop_tm1 = float(np.finfo(np.float32).max)  # train.cpp:167-168
        self.rprop_losses, self.n_updates = rprop_losses, 0
        if kind == OPT["IRPROP_PLUS"]:
            self.prev_g, self.prev_move = np.zeros(n, np.float32), np.zeros(n, np.float32)
            self.steps = np.full(n, self.rprop[4], np.float32)
        else:
            self.prev_g = self.prev_move = self.steps = None
        # Update_Parameter (model.cpp:4797-4866): [gradient clip] -> optimizer -> [max-norm per unit].
        # weight_rows: (first weight index, units, fan-in) of every fully-connected layer.
        self.clip, self.max_norm, self.weight_rows = clip, f(max_norm), tuple(weight_rows)
        self.leaves, self.n, self.kind = leaves, n, kind
        self.lr, self.momentum, self.nesterov = f(lr), f(momentum), bool(nesterov)
        self.adam_lr, self.beta1, self.beta2, self.eps = f(adam_lr), f(beta1), f(beta2), f(eps)
        self.bias_correction, self.weight_decay, self.normalized_wd = bool(bias_correction), f(weight_decay), bool(normalized_wd)
        # AdaBound / AMSBound: learning_rate_final, learning_gamma; NosAdam: adam_gamma (model.hpp:3021-3034)
        self.lr_final, self.gamma, self.adam_gamma, self.previous_beta2 = f(lr_final), f(gamma), f(adam_gamma), f(0)
        self.mask = None if mask is None else np.ascontiguousarray(mask, np.float32)
        self.t = f(0)
        self.epoch_time_step = f(1)
        self.delta = np.zeros(n, np.float32) if kind == OPT["GD"] and self.momentum != 0 else None
        if kind == OPT["IRPROP_PLUS"]:
            self.delta = self.prev_move  # the reference keeps it in the same array (previous delta parameters)
        self.m1 = np.zeros(n, np.float32) if kind in _ADAM_FAMILY else None
        self.m2 = np.zeros(n, np.float32) if kind in _ADAM_FAMILY else None
        self.vhat = np.zeros(n, np.float32) if kind in (OPT["AMSGRAD"], OPT["AMSBOUND"]) else None

    def wd(self, batch, training_size):
        f = np.float32
        if self.normalized_wd:
            return f(self.weight_decay * np.sqrt(f(f(batch) / f(f(training_size) * self.epoch_time_step))))
        return self.weight_decay

    def lr_t(self, lr_scale=np.float32(1)):
        f = np.float32
        lr = f(lr_scale * self.adam_lr)
        if not self.bias_correction:
            return lr
        return f(f(lr * np.sqrt(f(f(1) - np.power(self.beta2, self.t)))) / f(f(1) - np.power(self.beta1, self.t)))

    def clear(self):
        """Clear_Optimizer, train.cpp:136-248."""
        f = np.float32
        for a in (self.delta, self.m1, self.m2, self.vhat, self.prev_g):
            if a is not None:
                a[...] = 0
        if self.steps is not None:
            self.steps[...] = self.rprop[4]
        self.t, self.epoch_time_step, self.previous_beta2 = f(0), f(1), f(0)

    def warm_restarts_decay(self):
        """train.cpp:250-275: cosine annealing of the rate over a period of T_i steps; at the end of the
        period the optimizer restarts, the period stretches and the peak rate decays."""
        f = np.float32
        w = self.wr
        lr = f(w["min"] + f(f(f(0.5) * f(w["max"] - w["min"])) * f(f(1) + np.cos(f(f(self.t / w["T"]) * f(np.pi))))))
        if self.t >= w["T"]:
            self.clear()
            w["T"] = f(w["T"] * w["mult"])
            w["max"] = max(f(w["max"] * w["decay"]), w["min"])
        return lr

    def update(self, p, g, batch, training_size, nthreads=0):
        if self.clip is not None:
            self.leaves.clip_gradient(g, np.float32(self.clip), nthreads)
        self._step(p, g, batch, training_size, nthreads)
        if self.max_norm != 0:
            for w0, rows, cols in self.weight_rows:
                self.leaves.max_norm_rows(p[w0:w0 + rows * cols].reshape(rows, cols), self.max_norm, nthreads)

    def _step(self, p, g, batch, training_size, nthreads):
        if self.kind == OPT["IRPROP_PLUS"]:
            if self.rprop_losses is not None:
                self.loss_rprop, self.loss_rprop_tm1 = (float(v) for v in self.rprop_losses[self.n_updates])
            self.n_updates += 1
            incr, decr, dmin, dmax, _ = self.rprop
            self.leaves.opt_irprop_plus(p, g, self.prev_g, self.prev_move, self.steps, incr, decr, dmin, dmax,
                                        self.loss_rprop > self.loss_rprop_tm1, nthreads)
            return
        # every one of these asks the warm-restart schedule first (it may restart the optimizer, clocks
        # included), then advances the time step and reads the weight decay; gradient descent scales the decay
        # by the same factor, the Adam family does not (gradient_descent.cpp:66-75, adam.cpp:38-49)
        f = np.float32
        gd = self.kind == OPT["GD"]
        scale = f(self.warm_restarts_decay() / (self.lr if gd else self.adam_lr)) if self.wr is not None else f(1)
        self.t = np.float32(self.t + np.float32(1))
        wd = self.wd(batch, training_size)
        if gd:
            lr, wd = f(scale * self.lr), f(scale * wd)
            if self.momentum != 0:
                self.leaves.opt_gd_momentum(p, g, self.delta, self.mask, lr, self.momentum, wd, self.nesterov, nthreads)
            else:
                self.leaves.opt_gd(p, g, self.mask, lr, wd, nthreads)
        elif self.kind in (OPT["ADABOUND"], OPT["AMSBOUND"]):
            # adabound.cpp:49-55: the band closes on learning_rate_final as the time step grows
            f, one = np.float32, np.float32(1)
            lower = f(f(scale * self.lr_final) * f(one - f(one / f(f(self.gamma * self.t) + one))))
            upper = f(f(scale * self.lr_final) * f(one + f(one / f(self.gamma * self.t))))
            self.leaves.opt_adabound(p, g, self.m1, self.m2, self.vhat, self.mask, self.lr_t(scale), self.beta1, self.beta2,
                                     self.eps, wd, lower, upper, nthreads)
        elif self.kind == OPT["NOSADAM"]:
            # nosadam.cpp:49-52, 68: the second-moment decay of step t is B_{t-1} / B_t with
            # B_t = sum_{k<=t} k^-gamma; the bias correction still uses the fixed beta2
            f = np.float32
            term = f(np.power(self.t, f(-self.adam_gamma)))
            beta2_t = f(self.previous_beta2 / f(self.previous_beta2 + term))
            self.previous_beta2 = f(self.previous_beta2 + term)
            self.leaves.opt_adam(p, g, self.m1, self.m2, None, self.mask, self.lr_t(scale), self.beta1, beta2_t, self.eps, wd,
                                 nthreads)
        else:
            self.leaves.opt_adam(p, g, self.m1, self.m2, self.vhat, self.mask, self.lr_t(scale), self.beta1, self.beta2,
                                 self.eps, wd, nthreads)


class _Leaves:
    """Shared leaf-level wrappers.  ``self._f(name)`` resolves a C symbol,
    ``self.dtype`` is the numpy element type the library works in."""

    dtype = np.float32

    def _a(self, x, copy=False):
        if x is None:
            return None
        a = np.ascontiguousarray(x, dtype=self.dtype)
        return a.copy() if copy and a is x else a

    def _real(self, v):
        return c_f(v) if self.dtype == np.float32 else c_d(v)

    def fc_fwd(self, X, W, nthreads=0):
        X, W = self._a(X), self._a(W)
        B, K = X.shape
        H = W.shape[0]
        Z = np.empty((B, H), self.dtype)
        self._f("fc_fwd")(c_int(nthreads), c_sz(B), c_sz(K), c_sz(H), _ptr(X), _ptr(W), _ptr(Z))
        return Z

    def bias_fwd(self, Z, bias, nthreads=0):
        Z = np.array(Z, dtype=self.dtype, order="C", copy=True)
        bias = self._a(bias)
        B, H = Z.shape
        self._f("bias_fwd")(c_int(nthreads), c_sz(B), c_sz(H), _ptr(bias), _ptr(Z))
        return Z

    def norm_fwd_train(self, x, gamma, beta, mov_mean, mov_std, momentum, eps,
                       r_max=1.0, d_max=0.0, renorm=True, nthreads=0):
        """Returns dict(mean, std, mov_mean, mov_std, r, d, xhat, out)."""
        x, gamma, beta = self._a(x), self._a(gamma), self._a(beta)
        B, H = x.shape
        mm = np.array(mov_mean, dtype=self.dtype, copy=True)
        ms = np.array(mov_std, dtype=self.dtype, copy=True)
        mean = np.empty(H, self.dtype)
        std = np.empty(H, self.dtype)
        r = np.ones(H, self.dtype)
        d = np.zeros(H, self.dtype)
        xhat = np.empty((B, H), self.dtype)
        out = np.empty((B, H), self.dtype)
        self._f("norm_fwd_train")(
            c_int(nthreads), c_int(1 if renorm else 0), c_sz(B), c_sz(H),
            self._real(momentum), self._real(eps), self._real(r_max), self._real(d_max),
            _ptr(x), _ptr(gamma), _ptr(beta), _ptr(mean), _ptr(std), _ptr(mm), _ptr(ms),
            _ptr(r), _ptr(d), _ptr(xhat), _ptr(out))
        return dict(mean=mean, std=std, mov_mean=mm, mov_std=ms, r=r, d=d, xhat=xhat, out=out)

    def norm_fwd_infer(self, x, gamma, beta, mov_mean, mov_std, nthreads=0):
        x = self._a(x)
        B, H = x.shape
        out = np.empty((B, H), self.dtype)
        self._f("norm_fwd_infer")(c_int(nthreads), c_sz(B), c_sz(H), _ptr(x), _ptr(self._a(gamma)),
                                  _ptr(self._a(beta)), _ptr(self._a(mov_mean)), _ptr(self._a(mov_std)),
                                  _ptr(out))
        return out

    def act_fwd(self, act, x, nthreads=0):
        x = self._a(x)
        B, H = x.shape
        y = np.empty((B, H), self.dtype)
        self._f("act_fwd")(c_int(nthreads), c_int(act), c_sz(B), c_sz(H), _ptr(x), _ptr(y))
        return y

    def softmax_fwd(self, x, nthreads=0):
        x = self._a(x)
        B, H = x.shape
        y = np.empty((B, H), self.dtype)
        self._f("softmax_fwd")(c_int(nthreads), c_sz(B), c_sz(H), _ptr(x), _ptr(y))
        return y

    def identity_add(self, a, b, nthreads=0):
        a, b = self._a(a), self._a(b)
        B, H = a.shape
        out = np.empty((B, H), self.dtype)
        self._f("identity_add")(c_int(nthreads), c_sz(B), c_sz(H), _ptr(a), _ptr(b), _ptr(out))
        return out

    def zero_padded_identity_fwd(self, a, b, padding, nthreads=0):
        a, b = self._a(a), self._a(b)
        B, HA = a.shape
        HB = b.shape[1]
        out = np.empty((B, max(HA, HB)), self.dtype)
        self._f("zero_padded_identity_fwd")(c_int(nthreads), c_sz(B), c_sz(HA), c_sz(HB), c_sz(padding), _ptr(a),
                                            _ptr(b), _ptr(out))
        return out

    def residual_bwd(self, d_inputs, derivatives, padding, nthreads=0):
        """Returns derivatives + the routed columns of d_inputs."""
        di = self._a(d_inputs)
        dd = np.array(derivatives, dtype=self.dtype, order="C", copy=True)
        self._f("residual_bwd")(c_int(nthreads), c_sz(di.shape[0]), c_sz(di.shape[1]), c_sz(dd.shape[1]),
                                c_sz(padding), _ptr(di), _ptr(dd))
        return dd

    def fc_bwd_dx(self, dZn, Wn, dY_init=None, nthreads=0):
        dZn, Wn = self._a(dZn), self._a(Wn)
        B, Hn = dZn.shape
        H = Wn.shape[1]
        dY = (np.zeros((B, H), self.dtype) if dY_init is None
              else np.array(dY_init, dtype=self.dtype, order="C", copy=True))
        self._f("fc_bwd_dx")(c_int(nthreads), c_sz(B), c_sz(Hn), c_sz(H), _ptr(dZn), _ptr(Wn), _ptr(dY))
        return dY

    def act_bwd(self, act, pre, post, dY, nthreads=0):
        pre, post, dY = self._a(pre), self._a(post), self._a(dY)
        B, H = pre.shape
        dN = np.empty((B, H), self.dtype)
        self._f("act_bwd")(c_int(nthreads), c_int(act), c_sz(B), c_sz(H), _ptr(pre), _ptr(post),
                           _ptr(dY), _ptr(dN))
        return dN

    def norm_bwd(self, mean, std, gamma, r, x, xhat, dN, dgamma_init=None, dbeta_init=None,
                 renorm=True, nthreads=0):
        """Returns dict(dgamma, dbeta, dmean, dstd, dx)."""
        x, xhat, dN = self._a(x), self._a(xhat), self._a(dN)
        B, H = x.shape
        dg = (np.zeros(H, self.dtype) if dgamma_init is None
              else np.array(dgamma_init, dtype=self.dtype, copy=True))
        db = (np.zeros(H, self.dtype) if dbeta_init is None
              else np.array(dbeta_init, dtype=self.dtype, copy=True))
        dmean = np.empty(H, self.dtype)
        dstd = np.empty(H, self.dtype)
        dx = np.empty((B, H), self.dtype)
        r = np.ones(H, self.dtype) if r is None else self._a(r)
        self._f("norm_bwd")(c_int(nthreads), c_int(1 if renorm else 0), c_sz(B), c_sz(H),
                            _ptr(self._a(mean)), _ptr(self._a(std)), _ptr(self._a(gamma)), _ptr(r),
                            _ptr(x), _ptr(xhat), _ptr(dN), _ptr(dg), _ptr(db), _ptr(dmean),
                            _ptr(dstd), _ptr(dx))
        return dict(dgamma=dg, dbeta=db, dmean=dmean, dstd=dstd, dx=dx)

    def fc_bwd_dw(self, Xin, dZ, dW_init=None, db_init=None, with_bias=True, nthreads=0):
        Xin, dZ = self._a(Xin), self._a(dZ)
        B, K = Xin.shape
        H = dZ.shape[1]
        dW = (np.zeros((H, K), self.dtype) if dW_init is None
              else np.array(dW_init, dtype=self.dtype, order="C", copy=True))
        db = None
        if with_bias:
            db = (np.zeros(H, self.dtype) if db_init is None
                  else np.array(db_init, dtype=self.dtype, copy=True))
        self._f("fc_bwd_dw")(c_int(nthreads), c_sz(B), c_sz(K), c_sz(H), _ptr(Xin), _ptr(dZ),
                             _ptr(dW), _ptr(db))
        return dW, db


class Oracle(_Leaves):
    """The restatement; ``Oracle(np.float64)`` selects the double arbiter."""

    def __init__(self, dtype=np.float32):
        if not os.path.exists(ORACLE_SO):
            build_oracle()
        self.lib = ctypes.CDLL(ORACLE_SO)
        self.dtype = np.dtype(dtype).type
        self.suffix = "_f32" if self.dtype == np.float32 else "_f64"
        self.lib.dlo_max_threads.restype = c_int
        self.lib.dlo_mlp_create.restype = vp
        for n in ("parameters", "dparameters", "moving_mean", "moving_std"):
            getattr(self.lib, "dlo_mlp_" + n).restype = ctypes.POINTER(c_f)
        self.lib.dlo_mlp_layer_buffer.restype = ctypes.POINTER(c_f)
        self.lib.dlo_mlp_layer_vector.restype = ctypes.POINTER(c_f)
        self.lib.dlo_mlp_total_parameters.restype = c_sz
        self.lib.dlo_mlp_total_units.restype = c_sz
        self.lib.dlo_mlp_loss_sum.restype = c_d
        self.lib.dlo_mlp_n_correct.restype = c_d

    name = "oracle"

    def max_threads(self):
        return self.lib.dlo_max_threads()

    def _f(self, leaf):
        fn = getattr(self.lib, "dlo_" + leaf + self.suffix)
        fn.restype = None
        return fn

    # ---- optimizer leaves: all update their array arguments IN PLACE ----------
    def opt_gd(self, p, g, mask, lr, wd, nthreads=0):
        self._f("opt_gd")(c_int(nthreads), c_sz(p.size), _ptr(p), _ptr(g), _ptr(mask), self._real(lr),
                          self._real(wd))

    def opt_gd_momentum(self, p, g, delta_prev, mask, lr, mom, wd, nesterov, nthreads=0):
        self._f("opt_gd_momentum")(c_int(nthreads), c_sz(p.size), _ptr(p), _ptr(g), _ptr(delta_prev), _ptr(mask),
                                   self._real(lr), self._real(mom), self._real(wd), c_int(1 if nesterov else 0))

    def opt_adam(self, p, g, m1, m2, vhat, mask, lr_t, beta1, beta2, eps, wd, nthreads=0):
        self._f("opt_adam")(c_int(nthreads), c_sz(p.size), _ptr(p), _ptr(g), _ptr(m1), _ptr(m2), _ptr(vhat),
                            _ptr(mask), self._real(lr_t), self._real(beta1), self._real(beta2), self._real(eps),
                            self._real(wd))

    def opt_irprop_plus(self, p, g, prev_g, prev_move, steps, incr, decr, step_min, step_max, worse, nthreads=0):
        self._f("opt_irprop_plus")(c_int(nthreads), c_sz(p.size), _ptr(p), _ptr(g), _ptr(prev_g), _ptr(prev_move),
                                   _ptr(steps), self._real(incr), self._real(decr), self._real(step_min),
                                   self._real(step_max), c_int(1 if worse else 0))

    def clip_gradient(self, g, max_norm, nthreads=0):
        """euclidean_norm on the whole array, in place."""
        self._f("euclidean_norm")(c_int(nthreads), c_sz(g.size), self._real(max_norm), _ptr(g))

    def max_norm_rows(self, W, max_norm, nthreads=0):
        """euclidean_norm on every row of W [rows, cols], in place."""
        self._f("max_norm_rows")(c_int(nthreads), c_sz(W.shape[0]), c_sz(W.shape[1]), self._real(max_norm), _ptr(W))

    def opt_adabound(self, p, g, m1, m2, vhat, mask, lr_t, beta1, beta2, eps, wd, rate_lower, rate_upper, nthreads=0):
        self._f("opt_adabound")(c_int(nthreads), c_sz(p.size), _ptr(p), _ptr(g), _ptr(m1), _ptr(m2), _ptr(vhat),
                                _ptr(mask), self._real(lr_t), self._real(beta1), self._real(beta2), self._real(eps),
                                self._real(wd), self._real(rate_lower), self._real(rate_upper))

    def dropout_fwd(self, kind, v, mask, scale_or_keep, nthreads=0):
        """kind 0 inverted, 1 plain, 2 inference.  mask [H] (reference semantics,
        one value per unit) or [B,H] (per element) uint8."""
        v = np.array(v, dtype=self.dtype, order="C", copy=True)
        B, H = v.shape
        per_element = 0
        m = None
        if mask is not None:
            m = np.ascontiguousarray(mask, dtype=np.uint8)
            per_element = 1 if m.ndim == 2 else 0
        self._f("dropout_fwd")(c_int(nthreads), c_int(kind), c_int(per_element), c_sz(B), c_sz(H),
                               _ptr(m), self._real(scale_or_keep), _ptr(v))
        return v

    def softmax_ce_seed(self, q, y, nthreads=0):
        """Returns (dZ, loss_sum, n_correct)."""
        q, y = self._a(q), self._a(y)
        B, H = q.shape
        dZ = np.empty((B, H), self.dtype)
        loss = c_d(0.0)
        corr = c_d(0.0)
        self._f("softmax_ce_seed")(c_int(nthreads), c_sz(B), c_sz(H), _ptr(q), _ptr(y), _ptr(dZ),
                                   ctypes.byref(loss), ctypes.byref(corr))
        return dZ, loss.value, corr.value

    def loss_seed(self, loss, accu, acc_var, act, z, q, y, nthreads=0, want_dz=True):
        """Returns (dZ or None, loss_sum, n_accurate) of an element-wise output layer."""
        z, q, y = self._a(z), self._a(q), self._a(y)
        B, H = q.shape
        dZ = np.empty((B, H), self.dtype) if want_dz else None
        loss_sum = c_d(0.0)
        acc = c_d(0.0)
        f = self._f("loss_seed")
        f.restype = c_int
        rc = f(c_int(nthreads), c_int(loss), c_int(accu), self._real(acc_var), c_int(act), c_sz(B), c_sz(H), _ptr(z),
               _ptr(q), _ptr(y), _ptr(dZ) if want_dz else None, ctypes.byref(loss_sum), ctypes.byref(acc))
        if rc != 0:
            raise ValueError("loss / accuracy function not managed")
        return dZ, loss_sum.value, acc.value

    def mlp(self, widths):
        return OracleMLP(self, widths)


class OracleMLP:
    """Whole-model restatement (float only): dispatcher order + packed
    parameter layout of the reference."""

    def __init__(self, oracle, widths):
        self.o = oracle
        self.lib = oracle.lib
        self.widths = [int(w) for w in widths]
        arr = (c_sz * len(widths))(*self.widths)
        self.h = vp(self.lib.dlo_mlp_create(c_sz(len(widths)), arr))
        self.P = self.lib.dlo_mlp_total_parameters(self.h)
        self.n_units = self.lib.dlo_mlp_total_units(self.h)
        self.max_batch = 0

    def __del__(self):
        try:
            self.lib.dlo_mlp_destroy(self.h)
        except Exception:
            pass

    def set_layer(self, l, act, norm=0, drop=0, keep=1.0, mask=None, norm_before=True):
        m = None if mask is None else np.ascontiguousarray(mask, dtype=np.uint8)
        self.lib.dlo_mlp_set_layer(self.h, c_sz(l), c_int(act), c_int(norm), c_int(drop), c_f(keep), _ptr(m))
        self.lib.dlo_mlp_set_norm_order(self.h, c_sz(l), c_int(int(norm_before)))

    def set_norm_hyper(self, momentum, eps, r_max, d_max):
        self.lib.dlo_mlp_set_norm_hyper(self.h, c_f(momentum), c_f(eps), c_f(r_max), c_f(d_max))

    def layer_offsets(self, l):
        out = (c_sz * 6)()
        self.lib.dlo_mlp_layer_offsets(self.h, c_sz(l), out)
        return list(out)

    def prepare(self, max_batch, nthreads=0):
        self.max_batch = max_batch
        self.nthreads = nthreads
        self.lib.dlo_mlp_prepare(self.h, c_sz(max_batch))

    def _view(self, fn, n):
        return np.ctypeslib.as_array(fn(self.h), shape=(n,))

    @property
    def parameters(self):
        return self._view(self.lib.dlo_mlp_parameters, self.P)

    @property
    def dparameters(self):
        return self._view(self.lib.dlo_mlp_dparameters, self.P)

    @property
    def moving_mean(self):
        return self._view(self.lib.dlo_mlp_moving_mean, self.n_units)

    @property
    def moving_std(self):
        return self._view(self.lib.dlo_mlp_moving_std, self.n_units)

    def step(self, state, X, Y=None, backward=True):
        X = np.ascontiguousarray(X, np.float32)
        B = X.shape[0]
        self.B = B
        self.lib.dlo_mlp_forward(self.h, c_int(self.nthreads), c_int(state), c_sz(B), _ptr(X))
        if backward:
            Y = np.ascontiguousarray(Y, np.float32)
            self.lib.dlo_mlp_backward(self.h, c_int(self.nthreads), c_sz(B), _ptr(Y))

    def layer_buffer(self, l, which):
        p = self.lib.dlo_mlp_layer_buffer(self.h, c_sz(l), c_int(which))
        return np.ctypeslib.as_array(p, shape=(self.max_batch, self.widths[l]))[: self.B].copy()

    def layer_vector(self, l, which):
        p = self.lib.dlo_mlp_layer_vector(self.h, c_sz(l), c_int(which))
        return np.ctypeslib.as_array(p, shape=(self.widths[l],)).copy()

    def get_dparams(self):
        return self.dparameters.copy()

    # ---- optimizer and epoch driver (drivers/driver.cpp:60-340) --------------------
    def set_optimizer(self, kind, **kw):
        wd = kw.get("weight_decay", 0.0)
        mask = None
        if wd != 0.0:  # 1 on the weights, 0 on biases / gamma / beta (indexing.cpp:59-85)
            nw = sum(self.widths[l] * self.widths[l - 1] for l in range(1, len(self.widths)))
            mask = np.zeros(self.P, np.float32)
            mask[:nw] = 1
        rows = [(self.layer_offsets(l)[0], self.widths[l], self.widths[l - 1]) for l in range(1, len(self.widths))]
        self.opt = OptimizerHost(self.o, self.P, kind, mask=mask, weight_rows=rows, **kw)

    def update_parameter(self, batch, training_size):
        self.opt.update(self.parameters, self.dparameters, batch, training_size, self.nthreads)

    def _batches(self, n):
        bs = min(self.max_batch, n)
        return [(i, min(bs, n - i)) for i in range(0, n, bs)]

    def set_loss(self, loss, accu, acc_var=0.49):
        """set_loss_fn / set_accu_fn / acc_var for an output layer with an element-wise activation."""
        self.loss_fn, self.accu_fn = LOSS[loss] if isinstance(loss, str) else loss, ACCU[accu] if isinstance(accu, str) else accu
        self.lib.dlo_mlp_set_loss(self.h, c_int(self.loss_fn), c_int(self.accu_fn), c_f(acc_var))

    def reset_loss(self):
        self.lib.dlo_mlp_reset_loss(self.h)

    def loss_accu(self, n_data):
        return self._loss_accu(n_data)

    def _loss_accu(self, n):
        total, hout = self.lib.dlo_mlp_loss_sum(self.h), self.widths[-1]
        loss_fn, accu_fn = getattr(self, "loss_fn", LOSS["CROSS_ENTROPY"]), getattr(self, "accu_fn", ACCU["CROSS_ENTROPY"])
        terms = n * hout  # update_loss counts every output (compute_loss.cpp:50-52)
        if loss_fn == LOSS["CROSS_ENTROPY"]:
            loss = total / n if n else float("inf")                            # get_ace, loss.cpp:212-221
        elif loss_fn in (LOSS["L1"], LOSS["L2"]):
            loss = total                                                       # loss.cpp:146, 158
        elif loss_fn == LOSS["RMSE"]:
            loss = float(np.sqrt(total / terms)) if terms else 1.0             # loss.cpp:170-178
        else:
            loss = total / terms if terms else 1.0                             # get_me / get_mae / get_mse
        trials = n * (1 if accu_fn == ACCU["CROSS_ENTROPY"] else hout)         # drivers/driver.cpp:95-99
        return loss, self.lib.dlo_mlp_n_correct(self.h) / trials * 100.0       # get_accu, metrics.cpp:89-114

    def train_epoch(self, X, Y):
        """Driver::train: gradients accumulate over the sub-batches, ONE parameter
        update with batch = training size = n_data, then epoch_time_step += 1."""
        X, Y = np.ascontiguousarray(X, np.float32), np.ascontiguousarray(Y, np.float32)
        n = X.shape[0]
        self.lib.dlo_mlp_reset_loss(self.h)
        irprop = self.opt.kind == OPT["IRPROP_PLUS"]  # drivers/driver.cpp:228-232, 263
        if irprop:
            self.opt.loss_rprop_tm1 = self.opt.loss_rprop
        for i, b in self._batches(n):
            self.step(STATE["TRAINING"], X[i:i + b], Y[i:i + b], backward=True)
        if irprop:
            self.opt.loss_rprop = abs(self._loss_accu(n)[0])
        self.update_parameter(n, n)
        self.opt.epoch_time_step = np.float32(self.opt.epoch_time_step + np.float32(1))
        return self._loss_accu(n)

    def evalt(self, X, Y):
        X, Y = np.ascontiguousarray(X, np.float32), np.ascontiguousarray(Y, np.float32)
        n = X.shape[0]
        self.lib.dlo_mlp_reset_loss(self.h)
        for i, b in self._batches(n):
            self.step(STATE["INFERENCE"], X[i:i + b], None, backward=False)
            self.lib.dlo_mlp_compute_loss(self.h, c_int(self.nthreads), c_sz(b), _ptr(Y[i:i + b]))
        return self._loss_accu(n)

    def get_moving(self):
        return self.moving_mean.copy(), self.moving_std.copy()

    # ---- LSUV (v1/ops/initializers/lsuv.cpp:53-177) on weights the caller initialized ----------------
    def layer_variance(self, l, batch):
        """get_layer_variance(layer, batch) after the last forward pass (model.cpp:2824-2858)."""
        self.lib.dlo_layer_variance.restype = c_f
        out = np.ascontiguousarray(self.layer_buffer(l, 3)[:batch])
        return float(self.lib.dlo_layer_variance(c_sz(batch), c_sz(self.widths[l]), _ptr(out)))

    def lsuv(self, X, max_n_trials=10, max_batch_size=32, bias=0.0, var_target=1.0, var_tolerance=0.01, state=0):
        """Initialization__LSUV without the orthogonal pre-initialization: constant biases, then layer by layer
        scale the weights until the variance of the layer's output meets the target (Initialization__LSUV__Loop,
        lsuv.cpp:108-177; a multi-batch data set SUMS the mini-batch variances, lsuv.cpp:137), then the
        normalization parameters back to their start values.  Returns the scalings applied per layer.  A pass
        here runs the whole network; the layers behind the one being measured do not change its output."""
        X = np.ascontiguousarray(X, np.float32)
        f32 = np.float32
        eps = f32(1e-7)
        target, tol = max(f32(var_target), eps), f32(var_tolerance)
        n = min(int(max_batch_size), X.shape[0])
        self.prepare(n, self.nthreads)  # update_mem_batch_size(n_data): one mini-batch holds the whole sample
        L = len(self.widths)
        for l in range(1, L):
            b0 = self.layer_offsets(l)[1]
            self.parameters[b0:b0 + self.widths[l]] = f32(bias)
        trials = [0] * L

        def variance(l):
            self.step(state, X[:n], None, backward=False)
            v = f32(self.layer_variance(l, n))
            return eps if v <= 0 else v

        for l in range(1, L):
            w0 = self.layer_offsets(l)[0]
            w1 = w0 + self.widths[l] * self.widths[l - 1]
            v = variance(l)
            while abs(f32(v - target)) >= tol:
                w = np.ascontiguousarray(self.parameters[w0:w1])
                self.lib.dlo_lsuv_scale(_ptr(w), c_sz(w.size), c_f(v), c_f(target))
                self.parameters[w0:w1] = w
                trials[l] += 1
                if trials[l] < max_n_trials:
                    v = variance(l)
                else:
                    break
        self.dparameters[:] = 0
        if self.n_units:  # Clear__Parameter__Normalized_Unit: scales 1, shifts 0, moving mean 0, moving std 1
            g0 = self.P - 2 * self.n_units
            self.parameters[g0:g0 + self.n_units] = 1
            self.parameters[g0 + self.n_units:] = 0
            self.moving_mean[:] = 0
            self.moving_std[:] = 1
        return trials


def reference_available():
    return os.path.exists(REF_SO)


class Reference(_Leaves):
    """The real reference sources, compiled.  The shared object leaves the
    reference's console / file-IO symbols undefined (their translation units
    need Boost / systemd and are not on this path), so it must be opened with
    lazy binding; ctypes.CDLL alone forces RTLD_NOW."""

    name = "reference"

    def __init__(self):
        if not reference_available():
            raise FileNotFoundError(REF_SO)
        dl = ctypes.CDLL(None)
        dl.dlopen.restype = vp
        dl.dlopen.argtypes = [ctypes.c_char_p, c_int]
        handle = dl.dlopen(REF_SO.encode(), os.RTLD_LAZY | os.RTLD_LOCAL)
        if not handle:
            raise OSError("dlopen failed for " + REF_SO)
        self.lib = ctypes.CDLL(REF_SO, handle=handle)
        self.lib.dlref_init()
        self.lib.dlref_max_threads.restype = c_int
        self.lib.dlref_model_create.restype = vp
        for n in ("number_threads", "total_parameters", "total_norm_units"):
            getattr(self.lib, "dlref_model_" + n).restype = c_sz

    def max_threads(self):
        return self.lib.dlref_max_threads()

    def _f(self, leaf):
        fn = getattr(self.lib, "dlref_" + leaf)
        fn.restype = None
        return fn

    def dropout_fwd(self, kind, v, mask, scale_or_keep, nthreads=0):
        v = np.array(v, dtype=np.float32, order="C", copy=True)
        B, H = v.shape
        m = None if mask is None else np.ascontiguousarray(mask, dtype=np.uint8)
        assert m is None or m.ndim == 1, "the reference's mask is per unit"
        self._f("dropout_fwd")(c_int(nthreads), c_int(kind), c_sz(B), c_sz(H), _ptr(m),
                               c_f(scale_or_keep), _ptr(v))
        return v

    def clip_gradient(self, g, max_norm, nthreads=0):
        """euclidean_norm_st (nthreads 0) / euclidean_norm_mp on a float32 array, in place."""
        self._f("euclidean_norm")(c_int(nthreads), c_sz(g.size), c_f(max_norm), _ptr(g))

    def max_norm_rows(self, W, max_norm, nthreads=0):
        # max_norm.cpp:61-78 walks the units and calls euclidean_norm_st on each one's weights
        for r in range(W.shape[0]):
            self._f("euclidean_norm")(c_int(0), c_sz(W.shape[1]), c_f(max_norm), _ptr(W[r]))

    def mlp(self, widths, allowable_bytes=1 << 32):
        return ReferenceMLP(self, widths, allowable_bytes)


class ReferenceMLP:
    """A real DL::v1::Model built through compile() and the public setters."""

    def __init__(self, ref, widths, allowable_bytes):
        self.lib = ref.lib
        self.widths = [int(w) for w in widths]
        arr = (c_sz * len(widths))(*self.widths)
        h = self.lib.dlref_model_create(c_sz(len(widths)), arr, c_sz(allowable_bytes))
        if not h:
            raise RuntimeError("reference Model::compile failed")
        self.h = vp(h)
        self.P = self.lib.dlref_model_total_parameters(self.h)
        self.n_units = self.lib.dlref_model_total_norm_units(self.h)
        self._hyper = None

    def __del__(self):
        try:
            self.lib.dlref_model_destroy(self.h)
        except Exception:
            pass

    def set_layer(self, l, act, norm=0, drop=0, keep=1.0, mask=None, norm_before=True):
        ok = self.lib.dlref_model_set_activation(self.h, c_sz(l), c_int(act))
        assert ok, "set_layer_activation_function refused"
        if norm:
            self.lib.dlref_model_set_norm_order(self.h, c_sz(l), c_int(int(norm_before)))
            ok = self.lib.dlref_model_set_normalization(self.h, c_sz(l), c_int(norm))
            assert ok, "Set__Layer_Normalization refused"
        if drop:
            ok = self.lib.dlref_model_set_dropout(self.h, c_sz(l), c_int(drop), c_f(keep))
            assert ok, "set_dropout refused"
        self._masks = getattr(self, "_masks", {})
        if mask is not None:
            self._masks[l] = np.ascontiguousarray(mask, dtype=np.uint8)

    def set_norm_hyper(self, momentum, eps, r_max, d_max):
        ok = self.lib.dlref_model_set_norm_hyper(self.h, c_f(momentum), c_f(eps), c_f(r_max), c_f(d_max))
        assert ok

    def layer_offsets(self, l):
        out = (c_sz * 6)()
        self.lib.dlref_model_layer_offsets(self.h, c_sz(l), out)
        return list(out)

    def prepare(self, max_batch, nthreads=0):
        self.max_batch = max_batch
        ok = self.lib.dlref_model_prepare(self.h, c_sz(max_batch), c_int(nthreads))
        assert ok, "reference prepare failed"
        for l, m in getattr(self, "_masks", {}).items():
            ok = self.lib.dlref_model_set_dropout_mask(self.h, c_sz(l), c_sz(self.widths[l]), _ptr(m))
            assert ok
        self.lib.dlref_model_zero_dparams(self.h)
        # the normalization parameters are only allocated once a layer asks for them
        self.P = self.lib.dlref_model_total_parameters(self.h)
        self.n_units = self.lib.dlref_model_total_norm_units(self.h)

    def number_threads(self):
        return self.lib.dlref_model_number_threads(self.h)

    def set_parameters(self, p):
        p = np.ascontiguousarray(p, np.float32)
        assert p.size == self.P
        self.lib.dlref_model_set_parameters(self.h, _ptr(p), c_sz(self.P))

    def get_parameters(self):
        p = np.empty(self.P, np.float32)
        self.lib.dlref_model_get_parameters(self.h, _ptr(p), c_sz(self.P))
        return p

    def glorot_uniform(self, seed, bias=0.0):
        """real_gen.seed(seed); initialize_weights_with_glorot_uniform(bias)"""
        self.lib.dlref_model_glorot_uniform(self.h, ctypes.c_uint(seed), c_f(bias))

    def init_uniform(self, seed, bias=0.0, lower=-1.0, upper=1.0):
        """real_gen.seed(seed); Initialization__Uniform(bias, lower, upper)"""
        self.lib.dlref_model_init_uniform(self.h, ctypes.c_uint(seed), c_f(bias), c_f(lower), c_f(upper))

    def init_identity(self, bias=0.0):
        """Initialization__Identity(bias)"""
        self.lib.dlref_model_init_identity(self.h, c_f(bias))

    def glorot_gaussian(self, seed, bias=0.0):
        """gaussian.seed(seed); Initialization__Glorot__Gaussian(bias)"""
        self.lib.dlref_model_glorot_gaussian(self.h, ctypes.c_uint(seed), c_f(bias))

    def gaussian_draws(self, seed, n):
        """gaussian.seed(seed); weights_initialize_gaussian over n values, variance 1 (model.cpp:5401-5409)"""
        out = np.empty(n, np.float32)
        self.lib.dlref_model_gaussian_draws(self.h, ctypes.c_uint(seed), c_sz(n), _ptr(out))
        return out

    def dropout_bernoulli(self, seed=None):
        """[bernoulli[0].seed(seed);] Model::Dropout_Bernoulli() on a single-thread model."""
        ok = self.lib.dlref_model_dropout_bernoulli(self.h, ctypes.c_uint(seed or 0), c_int(int(seed is not None)))
        assert ok, "the reference has no mask generator (no dropout layer set)"

    def dropout_mask(self, l, n):
        out = np.zeros(n, np.uint8)
        return out if self.lib.dlref_model_get_dropout_mask(self.h, c_sz(l), c_sz(n), _ptr(out)) else None

    def set_moving(self, mean, std):
        mean = np.ascontiguousarray(mean, np.float32)
        std = np.ascontiguousarray(std, np.float32)
        self.lib.dlref_model_set_moving(self.h, _ptr(mean), _ptr(std), c_sz(self.n_units))

    def get_moving(self):
        mean = np.empty(self.n_units, np.float32)
        std = np.empty(self.n_units, np.float32)
        self.lib.dlref_model_get_moving(self.h, _ptr(mean), _ptr(std), c_sz(self.n_units))
        return mean, std

    def lsuv(self, X, max_n_trials=10, max_batch_size=32, bias=0.0, var_target=1.0, var_tolerance=0.01):
        """The reference's Initialize__LSUV + Initialization__LSUV__Loop on weights already initialized (its
        orthogonal pre-initialization is not part of the oracle: the facade has its own, tests/test_orthogonal_weights.py)."""
        X = np.ascontiguousarray(X, np.float32)
        ok = self.lib.dlref_model_lsuv(self.h, c_sz(max_n_trials), c_sz(max_batch_size), c_f(bias), c_f(var_target),
                                       c_f(var_tolerance), c_sz(X.shape[0]), _ptr(X), c_sz(X.shape[1]))
        if not ok:
            raise RuntimeError("reference LSUV failed")

    def layer_variance(self, l, batch):
        self.lib.dlref_model_layer_variance.restype = c_f
        return float(self.lib.dlref_model_layer_variance(self.h, c_sz(l), c_sz(batch)))

    def step(self, state, X, Y=None, backward=True):
        X = np.ascontiguousarray(X, np.float32)
        B, K0 = X.shape
        self.B = B
        Yp, Hout = None, self.widths[-1]
        if backward:
            Y = np.ascontiguousarray(Y, np.float32)
            Yp = _ptr(Y)
        self.lib.dlref_model_step(self.h, c_int(state), c_sz(B), _ptr(X), c_sz(K0), Yp, c_sz(Hout),
                                  c_int(1 if backward else 0))

    def layer_buffer(self, l, which):
        out = np.empty((self.max_batch, self.widths[l]), np.float32)
        ok = self.lib.dlref_model_get_layer_buffer(self.h, c_sz(l), c_int(which), c_sz(self.max_batch),
                                                   _ptr(out))
        assert ok
        return out[: self.B].copy()

    def layer_vector(self, l, which):
        out = np.empty(self.widths[l], np.float32)
        ok = self.lib.dlref_model_get_layer_vector(self.h, c_sz(l), c_int(which), _ptr(out))
        assert ok
        return out

    def get_dparams(self):
        p = np.empty(self.P, np.float32)
        self.lib.dlref_model_get_dparams(self.h, _ptr(p), c_sz(self.P))
        return p

    # ---- loss / accuracy function (set_loss_fn, set_accu_fn, acc_var) -----------
    def set_loss(self, loss, accu, acc_var=0.49):
        self.lib.dlref_model_set_loss(self.h, c_int(LOSS[loss] if isinstance(loss, str) else loss),
                                      c_int(ACCU[accu] if isinstance(accu, str) else accu), c_f(acc_var))

    def reset_loss(self):
        self.lib.dlref_model_reset_loss(self.h)

    def loss_accu(self, n_data):
        """(get_loss(NONE), get_accu(NONE)) as Driver reports them after n_data examples."""
        out = (c_d * 2)()
        self.lib.dlref_model_loss_accu(self.h, c_sz(n_data), out)
        return out[0], out[1]

    # ---- optimizer (Model::Update_Parameter) ---------------------------------
    def set_optimizer(self, kind, lr=0.01, momentum=0.9, nesterov=False, adam_lr=0.001, beta1=0.9, beta2=0.999,
                      eps=1e-8, bias_correction=True, weight_decay=0.0, normalized_wd=True, lr_final=0.1, gamma=1e-3,
                      adam_gamma=0.1, clip=None, max_norm=0.0, rprop=(1.2, 0.5, 1e-6, 50.0, 0.1), rprop_losses=None,
                      warm_restarts=None):
        """warm_restarts: None or (decay of the peak rate, peak rate, floor, first period, period multiplier)."""
        wr = warm_restarts or (1.0, 1.0, 1e-7, 1.0, 2.0)
        self.lib.dlref_model_set_warm_restarts(self.h, c_int(int(warm_restarts is not None)), *(c_f(v) for v in wr))
        self.lib.dlref_model_set_bound_hyper(self.h, c_f(lr_final), c_f(gamma), c_f(adam_gamma))
        self.lib.dlref_model_set_rprop(self.h, *(c_f(v) for v in rprop))
        self._rprop_losses, self._n_updates = rprop_losses, 0
        ok = self.lib.dlref_model_set_constraints(self.h, c_int(int(clip is not None)), c_f(1.0 if clip is None else clip),
                                                  c_f(max_norm))
        assert ok, "reference refused the constraint settings"
        ok = self.lib.dlref_model_set_optimizer(self.h, c_int(kind), c_f(lr), c_f(momentum), c_int(int(nesterov)),
                                                c_f(adam_lr), c_f(beta1), c_f(beta2), c_f(eps),
                                                c_int(int(bias_correction)), c_f(weight_decay),
                                                c_int(int(normalized_wd)))
        assert ok, "reference refused the optimizer settings"

    def set_epoch_time_step(self, v):
        self.lib.dlref_model_set_epoch_time_step(self.h, c_f(v))

    def set_dparams(self, g):
        g = np.ascontiguousarray(g, np.float32)
        assert g.size == self.P
        self.lib.dlref_model_set_dparams(self.h, _ptr(g), c_sz(self.P))

    def update_parameter(self, batch, training_size):
        if getattr(self, "_rprop_losses", None) is not None:  # replay of a recorded loss sequence (iRPROP+)
            loss, loss_tm1 = self._rprop_losses[self._n_updates]
            self.lib.dlref_model_set_rprop_loss(self.h, c_d(loss), c_d(loss_tm1))
        self._n_updates = getattr(self, "_n_updates", 0) + 1
        self.lib.dlref_model_update_parameter(self.h, c_sz(batch), c_sz(training_size))

    def opt_state(self, which):
        """which: 0 previous delta, 1 first moment, 2 second moment, 3 second moment hat, 4 regularization mask,
        5 previous gradient, 6 step sizes (iRPROP+); None when the reference has not allocated it."""
        out = np.empty(self.P, np.float32)
        ok = self.lib.dlref_model_get_opt_state(self.h, c_int(which), _ptr(out), c_sz(self.P))
        return out if ok else None

    # ---- epoch driver (Driver::train / Driver::evalt over dense arrays) ---------------
    def train_epoch(self, X, Y, resample_masks=False):
        X, Y = np.ascontiguousarray(X, np.float32), np.ascontiguousarray(Y, np.float32)
        out = (c_d * 2)()
        self.lib.dlref_model_train_epoch(self.h, c_sz(X.shape[0]), _ptr(X), c_sz(X.shape[1]), _ptr(Y),
                                         c_sz(Y.shape[1]), c_int(int(resample_masks)), out)
        return out[0], out[1]

    def evalt(self, X, Y):
        X, Y = np.ascontiguousarray(X, np.float32), np.ascontiguousarray(Y, np.float32)
        out = (c_d * 2)()
        self.lib.dlref_model_evalt(self.h, c_sz(X.shape[0]), _ptr(X), c_sz(X.shape[1]), _ptr(Y), c_sz(Y.shape[1]),
                                   out)
        return out[0], out[1]


# ---- layer lists with residual blocks ---------------------------------------------
LAYER = dict(FULLY_CONNECTED=3, RESIDUAL=9)  # v1/data/enum/layer.hpp


class _NetBase:
    """Driving interface shared by OracleNet and ReferenceNet.  `layers` is a list
    of ("FC", units) and ("RES", depth, padding) entries, entry 0 the input width."""

    def _spec(self, layers):
        self.layers = list(layers)
        n = len(layers)
        types = [LAYER["FULLY_CONNECTED"] if e[0] == "FC" else LAYER["RESIDUAL"] for e in layers]
        units = [int(e[1]) for e in layers]
        pads = [int(e[2]) if len(e) > 2 else 0 for e in layers]
        return n, (c_int * n)(*types), (c_sz * n)(*units), (c_sz * n)(*pads)

    def info(self, l):
        """dict(type, n_out, w0, w1, bias, use_bias, n_unit, gamma, unit, n_af, depth, padding)"""
        out = (c_sz * 12)()
        self._info(l, out)
        keys = ("type", "n_out", "w0", "w1", "bias", "use_bias", "n_unit", "gamma", "unit", "n_af", "depth", "padding")
        return dict(zip(keys, (int(v) for v in out)))

    def fc_layers(self):
        return [l for l, e in enumerate(self.layers) if l > 0 and e[0] == "FC"]


class OracleNet(_NetBase):
    def __init__(self, oracle, layers):
        self.o, self.lib = oracle, oracle.lib
        n, t, u, p = self._spec(layers)
        self.lib.dlo_net_create.restype = vp
        for f in ("parameters", "dparameters", "moving_mean", "moving_std", "layer_output", "layer_error"):
            getattr(self.lib, "dlo_net_" + f).restype = ctypes.POINTER(c_f)
        self.lib.dlo_net_total_parameters.restype = c_sz
        self.lib.dlo_net_total_units.restype = c_sz
        self.lib.dlo_net_loss_sum.restype = c_d
        self.lib.dlo_net_n_correct.restype = c_d
        self.h = vp(self.lib.dlo_net_create(c_sz(n), t, u, p))
        self.P = self.lib.dlo_net_total_parameters(self.h)
        self.n_units = self.lib.dlo_net_total_units(self.h)

    def __del__(self):
        try:
            self.lib.dlo_net_destroy(self.h)
        except Exception:
            pass

    def _info(self, l, out):
        self.lib.dlo_net_layer_info(self.h, c_sz(l), out)

    def set_layer(self, l, act, norm=0, drop=0, keep=1.0, mask=None):
        m = None if mask is None else np.ascontiguousarray(mask, dtype=np.uint8)
        self.lib.dlo_net_set_layer(self.h, c_sz(l), c_int(act), c_int(norm), c_int(drop), c_f(keep), _ptr(m))

    def set_norm_hyper(self, momentum, eps, r_max, d_max):
        self.lib.dlo_net_set_norm_hyper(self.h, c_f(momentum), c_f(eps), c_f(r_max), c_f(d_max))

    def prepare(self, max_batch, nthreads=0):
        self.max_batch, self.nthreads = max_batch, nthreads
        self.lib.dlo_net_prepare(self.h, c_sz(max_batch))

    def _view(self, fn, n):
        return np.ctypeslib.as_array(fn(self.h), shape=(n,))

    def set_parameters(self, p):
        self._view(self.lib.dlo_net_parameters, self.P)[:] = p

    def get_parameters(self):
        return self._view(self.lib.dlo_net_parameters, self.P).copy()

    def get_dparams(self):
        return self._view(self.lib.dlo_net_dparameters, self.P).copy()

    def get_moving(self):
        return (self._view(self.lib.dlo_net_moving_mean, self.n_units).copy(),
                self._view(self.lib.dlo_net_moving_std, self.n_units).copy())

    def step(self, state, X, Y=None, backward=True):
        X = np.ascontiguousarray(X, np.float32)
        self.B = X.shape[0]
        self.lib.dlo_net_forward(self.h, c_int(self.nthreads), c_int(state), c_sz(self.B), _ptr(X))
        if backward:
            Y = np.ascontiguousarray(Y, np.float32)
            self.lib.dlo_net_backward(self.h, c_int(self.nthreads), c_sz(self.B), _ptr(Y))

    def layer_output(self, l):
        w = self.info(l)["n_out"]
        return np.ctypeslib.as_array(self.lib.dlo_net_layer_output(self.h, c_sz(l)), shape=(self.max_batch, w))[: self.B].copy()

    def layer_error(self, l):
        w = self.info(l)["n_out"]
        return np.ctypeslib.as_array(self.lib.dlo_net_layer_error(self.h, c_sz(l)), shape=(self.max_batch, w))[: self.B].copy()


class ReferenceNet(_NetBase, ReferenceMLP):
    """A real DL::v1::Model compiled from a typed layer list."""

    def __init__(self, ref, layers, allowable_bytes=1 << 32):
        self.lib = ref.lib
        n, t, u, p = self._spec(layers)
        self.lib.dlref_model_create_typed.restype = vp
        h = self.lib.dlref_model_create_typed(c_sz(n), t, u, p, c_sz(allowable_bytes))
        if not h:
            raise RuntimeError("reference Model::compile failed")
        self.h = vp(h)
        self.P = self.lib.dlref_model_total_parameters(self.h)
        self.n_units = self.lib.dlref_model_total_norm_units(self.h)
        self.widths = [0] * n  # filled by prepare(): outputs per entry

    def _info(self, l, out):
        self.lib.dlref_model_layer_info(self.h, c_sz(l), out)

    def set_layer(self, l, act, norm=0, drop=0, keep=1.0, mask=None):
        if self.layers[l][0] == "FC":
            ok = self.lib.dlref_model_set_activation(self.h, c_sz(l), c_int(act))
            assert ok, "set_layer_activation_function refused"
        if norm:
            ok = self.lib.dlref_model_set_normalization(self.h, c_sz(l), c_int(norm))
            assert ok, "Set__Layer_Normalization refused"
        if drop:
            ok = self.lib.dlref_model_set_dropout(self.h, c_sz(l), c_int(drop), c_f(keep))
            assert ok, "set_dropout refused"
        self._masks = getattr(self, "_masks", {})
        if mask is not None:
            self._masks[l] = np.ascontiguousarray(mask, dtype=np.uint8)

    def prepare(self, max_batch, nthreads=0):
        self.max_batch = max_batch
        ok = self.lib.dlref_model_prepare(self.h, c_sz(max_batch), c_int(nthreads))
        assert ok, "reference prepare failed"
        for l, m in getattr(self, "_masks", {}).items():
            ok = self.lib.dlref_model_set_dropout_mask(self.h, c_sz(l), c_sz(m.size), _ptr(m))
            assert ok
        self.lib.dlref_model_zero_dparams(self.h)
        self.P = self.lib.dlref_model_total_parameters(self.h)
        self.n_units = self.lib.dlref_model_total_norm_units(self.h)
        self.widths = [self.info(l)["n_out"] for l in range(len(self.layers))]

    def layer_output(self, l):
        return self.layer_buffer(l, 6)

    def layer_error(self, l):
        return self.layer_buffer(l, 4)
