"""deep-learning_amd — MI355X (gfx950) implementation of the fully-connected /
batch-(re)normalization / activation hot path of SebastienKeroack/deep-learning.

The product is ``lib/libdlmi.so`` (hand-written HIP kernels behind the C ABI of
``include/dlmi.h`` plus the C++ ``Model`` facade of ``include/dlmi_model.h``).
This module is only the thin Python binding the tests and the benchmark use:
PyTorch supplies device memory and the stream, every computation goes through
the C ABI.  There is no CPU or PyTorch fallback: if the library is not built, or
no gfx950 device is present, construction raises.

The directory name carries a hyphen, so import it by path::

    spec = importlib.util.spec_from_file_location(
        "deep_learning_amd", ".../deep-learning_amd/__init__.py",
        submodule_search_locations=[".../deep-learning_amd"])
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# DLMI_LIBRARY in the environment names another build of the library (tuning runs); the default is the in-tree one
LIB_PATH = os.environ.get("DLMI_LIBRARY") or os.path.join(_HERE, "lib", "libdlmi.so")

c_sz = ctypes.c_size_t
c_int = ctypes.c_int
c_f = ctypes.c_float
vp = ctypes.c_void_p

# enum values shared with the reference (include/dlmi.h)
ACT = dict(ELU=3, ISRLU=10, LINEAR=11, LEAKY_RELU=14, RELU=16, SELU=17, SOFTMAX=22)
NORM = dict(NONE=0, BN=1, BRN=2)
DROP = dict(NONE=0, BERNOULLI=2, BERNOULLI_INVERTED=3)
DROP_BWD = dict(REFERENCE=0, MASKED=1)
STATE = dict(INFERENCE=0, TRAINING=1, UPDATE_BATCH_NORM=2)

# every symbol include/dlmi.h declares
C_ABI_SYMBOLS = [
    "dlmi_gemm_plan", "dlmi_ctx_create", "dlmi_ctx_destroy", "dlmi_ctx_set_stream", "dlmi_ctx_synchronize", "dlmi_last_error",
    "dlmi_ctx_compute_units", "dlmi_layer_variance", "dlmi_scale", "dlmi_fc_fwd", "dlmi_fc_bwd_dx", "dlmi_fc_bwd_dw", "dlmi_bias_fwd",
    "dlmi_norm_fwd_train", "dlmi_norm_fwd_infer", "dlmi_norm_bwd", "dlmi_act_fwd", "dlmi_act_fwd_units", "dlmi_act_bwd_units", "dlmi_act_bwd",
    "dlmi_softmax_fwd", "dlmi_dropout_fwd", "dlmi_identity_add", "dlmi_softmax_ce_seed",
    "dlmi_fused_norm_act_fwd", "dlmi_fused_norm_act_bwd", "dlmi_fused_norm_act_infer", "dlmi_fc_norm_act_fwd",
    "dlmi_opt_gd", "dlmi_opt_gd_momentum", "dlmi_opt_adam", "dlmi_zero_padded_identity_fwd", "dlmi_residual_bwd",
    "dlmi_opt_adabound", "dlmi_clip_gradient", "dlmi_max_norm_rows", "dlmi_opt_irprop_plus", "dlmi_loss_seed", "dlmi_zero",
    "dlmi_fused_norm_act_fwd_noalloc", "dlmi_fused_norm_act_residual_fwd", "dlmi_fc_norm_act_residual_fwd",
    "dlmi_fc_softmax_fwd", "dlmi_fc_softmax_ce_fwd", "dlmi_fc_bwd_dx_norm_act_bwd",
    "dlmi_ctx_reserve_layer", "dlmi_ctx_scratch_generation", "dlmi_ctx_norm_panel_enabled", "dlmi_ctx_norm_panel_poke",
    "dlmi_fc_bwd_dw_grouped", "dlmi_fused_norm_act_bwd_db", "dlmi_ctx_gemm_clock", "dlmi_ctx_gemm_timeline", "dlmi_probe_strip_stream",
]


class FusedDesc(ctypes.Structure):
    """dlmi_fused_desc of include/dlmi.h."""
    _fields_ = [("norm", c_int), ("act", c_int), ("dropout", c_int), ("mask_per_element", c_int),
                ("dropout_bwd", c_int), ("momentum", c_f), ("eps", c_f), ("r_max", c_f), ("d_max", c_f),
                ("drop_scale", c_f)]


class DwProblem(ctypes.Structure):
    _fields_ = [("B", ctypes.c_size_t), ("K", ctypes.c_size_t), ("H", ctypes.c_size_t), ("Xin", ctypes.c_void_p),
                ("dZ", ctypes.c_void_p), ("dW", ctypes.c_void_p), ("db", ctypes.c_void_p)]


class DlmiError(RuntimeError):
    pass


def load_library():
    if not os.path.exists(LIB_PATH):
        raise DlmiError("%s is missing: build it with `python deep-learning_amd/build.py` "
                        "(there is no fallback path)" % LIB_PATH)
    # A process that also uses torch on the GPU must have torch's HIP runtime loaded before this library's:
    # with the order reversed, torch.cuda.is_available() turns False later on.  Without torch installed the
    # library stands alone (the Model facade needs no torch).
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = ctypes.CDLL(LIB_PATH)
    lib.dlmi_last_error.restype = ctypes.c_char_p
    lib.dlmi_last_error.argtypes = [vp]
    return lib


def _p(t):
    return vp(0) if t is None else vp(t.data_ptr())


class Dlmi:
    """One dlmi context bound to a torch CUDA(HIP) device and its current stream."""

    def __init__(self, device=0):
        import torch
        self.torch = torch
        self.lib = load_library()
        if not torch.cuda.is_available():
            raise DlmiError("no GPU visible: dlmi has no CPU path")
        self.device = torch.device("cuda", device)
        ctx = vp()
        stream = torch.cuda.current_stream(self.device).cuda_stream
        rc = self.lib.dlmi_ctx_create(ctypes.byref(ctx), c_int(device), vp(stream))
        if rc != 0:
            raise DlmiError("dlmi_ctx_create failed with %d" % rc)
        self.ctx = ctx

    def close(self):
        if getattr(self, "ctx", None):
            self.lib.dlmi_ctx_destroy(self.ctx)
            self.ctx = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ------------------------------------------------------------ helpers
    def _ck(self, rc):
        if rc != 0:
            raise DlmiError("dlmi call failed (%d): %s" % (rc, self.lib.dlmi_last_error(self.ctx).decode()))

    def _chk(self, *tensors):
        for t in tensors:
            if t is None:
                continue
            assert t.is_cuda and t.is_contiguous(), "dlmi takes contiguous device tensors"

    def empty(self, *shape, dtype=None):
        return self.torch.empty(*shape, dtype=dtype or self.torch.float32, device=self.device)

    def zeros(self, *shape, dtype=None):
        return self.torch.zeros(*shape, dtype=dtype or self.torch.float32, device=self.device)

    def set_stream(self, stream):
        self._ck(self.lib.dlmi_ctx_set_stream(self.ctx, vp(stream.cuda_stream)))

    def synchronize(self):
        self._ck(self.lib.dlmi_ctx_synchronize(self.ctx))

    def compute_units(self):
        return self.lib.dlmi_ctx_compute_units(self.ctx)

    def gemm_clock(self):
        """(engine clock in MHz, lifetime in us) of the first tile's workgroup of the last product launched; the
        context must have been created with DLMI_GEMM_CLOCK=1 in the environment."""
        mhz, us = ctypes.c_double(0), ctypes.c_double(0)
        self._ck(self.lib.dlmi_ctx_gemm_clock(self.ctx, ctypes.byref(mhz), ctypes.byref(us)))
        return mhz.value, us.value

    def gemm_timeline(self, workgroups):
        """[workgroups, 4] int64: per workgroup of the last product launched the 100 MHz counter at entry, after its
        last store was issued and after it was acknowledged, and XCC_ID << 32 | HW_ID (DLMI_GEMM_CLOCK=1 contexts)."""
        import numpy as np
        buf = (ctypes.c_ulonglong * (4 * workgroups))()
        self._ck(self.lib.dlmi_ctx_gemm_timeline(self.ctx, buf, ctypes.c_size_t(workgroups)))
        return np.frombuffer(buf, dtype=np.uint64).reshape(workgroups, 4).astype(np.int64)

    def norm_panel_enabled(self):
        """Whether this context may still launch the single-launch normalization kernels."""
        return bool(self.lib.dlmi_ctx_norm_panel_enabled(self.ctx))

    def norm_panel_poke(self, xcd, word, value):
        """Test hook: one word of an XCD's barrier state (see dlmi.h)."""
        self._ck(self.lib.dlmi_ctx_norm_panel_poke(self.ctx, ctypes.c_uint(xcd), ctypes.c_uint(word), ctypes.c_uint(value)))

    def probe_strip_stream(self, x, y, x2=None):
        """Measurement aid: y = x (+ x2) streamed in the column panel kernels' access pattern (see dlmi.h)."""
        self._chk(x, y, x2)
        B, H = x.shape
        self._ck(self.lib.dlmi_probe_strip_stream(self.ctx, c_sz(B), c_sz(H), _p(x), _p(x2), _p(y)))
        return y

    # ------------------------------------------------------------ GEMMs
    def fc_fwd(self, X, W, bias=None, out=None):
        self._chk(X, W, bias, out)
        B, K = X.shape
        H = W.shape[0]
        assert W.shape[1] == K
        Z = out if out is not None else self.empty(B, H)
        self._ck(self.lib.dlmi_fc_fwd(self.ctx, c_sz(B), c_sz(K), c_sz(H), _p(X), _p(W), _p(bias), _p(Z)))
        return Z

    def fc_bwd_dx(self, dZn, Wn, out=None, accumulate=False):
        self._chk(dZn, Wn, out)
        B, Hn = dZn.shape
        H = Wn.shape[1]
        assert Wn.shape[0] == Hn
        dY = out if out is not None else self.empty(B, H)
        assert out is not None or not accumulate
        self._ck(self.lib.dlmi_fc_bwd_dx(self.ctx, c_sz(B), c_sz(Hn), c_sz(H), _p(dZn), _p(Wn), _p(dY),
                                         c_int(1 if accumulate else 0)))
        return dY

    def fc_bwd_dw(self, Xin, dZ, dW=None, db=None, with_bias=False, accumulate=False):
        self._chk(Xin, dZ, dW, db)
        B, K = Xin.shape
        H = dZ.shape[1]
        assert dZ.shape[0] == B
        if dW is None:
            assert not accumulate
            dW = self.empty(H, K)
        if db is None and with_bias:
            db = self.empty(H)
        self._ck(self.lib.dlmi_fc_bwd_dw(self.ctx, c_sz(B), c_sz(K), c_sz(H), _p(Xin), _p(dZ), _p(dW), _p(db),
                                         c_int(1 if accumulate else 0)))
        return dW, db

    def fc_bwd_dw_grouped(self, problems, accumulate=False):
        """problems: list of (Xin, dZ, dW, db or None); one launch per kernel variant (dlmi_fc_bwd_dw_grouped)."""
        arr = (DwProblem * len(problems))()
        for a, (Xin, dZ, dW, db) in zip(arr, problems):
            self._chk(Xin, dZ, dW, db)
            a.B, a.K, a.H = Xin.shape[0], Xin.shape[1], dZ.shape[1]
            a.Xin, a.dZ, a.dW, a.db = _p(Xin), _p(dZ), _p(dW), _p(db)
        self._ck(self.lib.dlmi_fc_bwd_dw_grouped(self.ctx, c_sz(len(problems)), arr, c_int(1 if accumulate else 0)))

    def bias_fwd(self, Z, bias):
        self._chk(Z, bias)
        B, H = Z.shape
        self._ck(self.lib.dlmi_bias_fwd(self.ctx, c_sz(B), c_sz(H), _p(bias), _p(Z)))
        return Z

    # ------------------------------------------------------------ normalization (un-fused leaves)
    def norm_fwd_train(self, x, gamma, beta, mov_mean, mov_std, momentum, eps, r_max=1.0, d_max=0.0,
                       renorm=True, want_xhat=True, want_out=True):
        """mov_mean / mov_std are updated in place.  Returns dict(mean,std,r,d,xhat,out)."""
        self._chk(x, gamma, beta, mov_mean, mov_std)
        B, H = x.shape
        o = dict(mean=self.empty(H), std=self.empty(H), r=self.empty(H), d=self.empty(H),
                 xhat=self.empty(B, H) if want_xhat else None, out=self.empty(B, H) if want_out else None)
        self._ck(self.lib.dlmi_norm_fwd_train(
            self.ctx, c_int(NORM["BRN"] if renorm else NORM["BN"]), c_sz(B), c_sz(H), c_f(momentum), c_f(eps),
            c_f(r_max), c_f(d_max), _p(x), _p(gamma), _p(beta), _p(o["mean"]), _p(o["std"]), _p(mov_mean),
            _p(mov_std), _p(o["r"]), _p(o["d"]), _p(o["xhat"]), _p(o["out"])))
        return o

    def norm_fwd_infer(self, x, gamma, beta, mov_mean, mov_std):
        self._chk(x, gamma, beta, mov_mean, mov_std)
        B, H = x.shape
        out = self.empty(B, H)
        self._ck(self.lib.dlmi_norm_fwd_infer(self.ctx, c_sz(B), c_sz(H), _p(x), _p(gamma), _p(beta), _p(mov_mean),
                                              _p(mov_std), _p(out)))
        return out

    def norm_bwd(self, mean, std, gamma, r, x, xhat, dN, dgamma, dbeta, renorm=True):
        """dgamma / dbeta accumulate in place.  Returns dict(dmean,dstd,dx)."""
        self._chk(mean, std, gamma, r, x, xhat, dN, dgamma, dbeta)
        B, H = x.shape
        o = dict(dmean=self.empty(H), dstd=self.empty(H), dx=self.empty(B, H))
        self._ck(self.lib.dlmi_norm_bwd(self.ctx, c_int(NORM["BRN"] if renorm else NORM["BN"]), c_sz(B), c_sz(H),
                                        _p(mean), _p(std), _p(gamma), _p(r), _p(x), _p(xhat), _p(dN), _p(dgamma),
                                        _p(dbeta), _p(o["dmean"]), _p(o["dstd"]), _p(o["dx"])))
        return o

    # ------------------------------------------------------------ element-wise leaves
    def act_fwd(self, act, x, out=None):
        self._chk(x, out)
        B, H = x.shape
        y = out if out is not None else self.empty(B, H)
        self._ck(self.lib.dlmi_act_fwd(self.ctx, c_int(act), c_sz(B), c_sz(H), _p(x), _p(y)))
        return y

    def act_bwd(self, act, pre, post, dY, out=None):
        self._chk(pre, post, dY, out)
        B, H = pre.shape
        dN = out if out is not None else self.empty(B, H)
        self._ck(self.lib.dlmi_act_bwd(self.ctx, c_int(act), c_sz(B), c_sz(H), _p(pre), _p(post), _p(dY), _p(dN)))
        return dN

    def act_fwd_units(self, types, x):
        """types: one activation code per unit (host integers)."""
        self._chk(x)
        B, H = x.shape
        t = (c_int * H)(*[int(v) for v in types])
        y = self.empty(B, H)
        self._ck(self.lib.dlmi_act_fwd_units(self.ctx, t, c_sz(B), c_sz(H), _p(x), _p(y)))
        return y

    def act_bwd_units(self, types, pre, post, dY):
        self._chk(pre, post, dY)
        B, H = pre.shape
        t = (c_int * H)(*[int(v) for v in types])
        dN = self.empty(B, H)
        self._ck(self.lib.dlmi_act_bwd_units(self.ctx, t, c_sz(B), c_sz(H), _p(pre), _p(post), _p(dY), _p(dN)))
        return dN

    def softmax_fwd(self, x):
        self._chk(x)
        B, H = x.shape
        y = self.empty(B, H)
        self._ck(self.lib.dlmi_softmax_fwd(self.ctx, c_sz(B), c_sz(H), _p(x), _p(y)))
        return y

    def dropout_fwd(self, kind, v, mask, scale, training=True):
        """In place on v.  mask [H] or [B,H] uint8."""
        self._chk(v, mask)
        B, H = v.shape
        per_element = 1 if (mask is not None and mask.dim() == 2) else 0
        self._ck(self.lib.dlmi_dropout_fwd(self.ctx, c_int(kind), c_int(1 if training else 0), c_int(per_element),
                                           c_sz(B), c_sz(H), _p(mask), c_f(scale), _p(v)))
        return v

    def identity_add(self, a, b, out=None):
        self._chk(a, b, out)
        o = out if out is not None else self.torch.empty_like(a)
        self._ck(self.lib.dlmi_identity_add(self.ctx, c_sz(a.numel()), _p(a), _p(b), _p(o)))
        return o

    def zero_padded_identity_fwd(self, a, b, padding, out=None):
        self._chk(a, b, out)
        B, HA = a.shape
        HB = b.shape[1]
        o = out if out is not None else self.empty(B, max(HA, HB))
        self._ck(self.lib.dlmi_zero_padded_identity_fwd(self.ctx, c_sz(B), c_sz(HA), c_sz(HB), c_sz(padding), _p(a),
                                                        _p(b), _p(o)))
        return o

    def residual_bwd(self, d_inputs, derivatives, padding):
        """derivatives += the routed columns of d_inputs, in place."""
        self._chk(d_inputs, derivatives)
        self._ck(self.lib.dlmi_residual_bwd(self.ctx, c_sz(d_inputs.shape[0]), c_sz(d_inputs.shape[1]),
                                            c_sz(derivatives.shape[1]), c_sz(padding), _p(d_inputs), _p(derivatives)))
        return derivatives

    # optimizer steps: every tensor argument is updated in place, grads end up zero
    def opt_gd(self, p, g, mask, lr, wd, nthreads=0):
        self._chk(p, g, mask)
        self._ck(self.lib.dlmi_opt_gd(self.ctx, c_sz(p.numel()), _p(p), _p(g), _p(mask), c_f(lr), c_f(wd)))

    def opt_gd_momentum(self, p, g, delta_prev, mask, lr, mom, wd, nesterov, nthreads=0):
        self._chk(p, g, delta_prev, mask)
        self._ck(self.lib.dlmi_opt_gd_momentum(self.ctx, c_sz(p.numel()), _p(p), _p(g), _p(delta_prev), _p(mask),
                                               c_f(lr), c_f(mom), c_f(wd), c_int(1 if nesterov else 0)))

    def opt_adam(self, p, g, m1, m2, vhat, mask, lr_t, beta1, beta2, eps, wd, nthreads=0):
        self._chk(p, g, m1, m2, vhat, mask)
        self._ck(self.lib.dlmi_opt_adam(self.ctx, c_sz(p.numel()), _p(p), _p(g), _p(m1), _p(m2), _p(vhat), _p(mask),
                                        c_f(lr_t), c_f(beta1), c_f(beta2), c_f(eps), c_f(wd)))

    def opt_adabound(self, p, g, m1, m2, vhat, mask, lr_t, beta1, beta2, eps, wd, rate_lower, rate_upper, nthreads=0):
        self._chk(p, g, m1, m2, vhat, mask)
        self._ck(self.lib.dlmi_opt_adabound(self.ctx, c_sz(p.numel()), _p(p), _p(g), _p(m1), _p(m2), _p(vhat), _p(mask),
                                            c_f(lr_t), c_f(beta1), c_f(beta2), c_f(eps), c_f(wd), c_f(rate_lower),
                                            c_f(rate_upper)))

    def opt_irprop_plus(self, p, g, prev_g, prev_move, steps, incr, decr, step_min, step_max, worse, nthreads=0):
        self._chk(p, g, prev_g, prev_move, steps)
        self._ck(self.lib.dlmi_opt_irprop_plus(self.ctx, c_sz(p.numel()), _p(p), _p(g), _p(prev_g), _p(prev_move),
                                               _p(steps), c_f(incr), c_f(decr), c_f(step_min), c_f(step_max),
                                               c_int(1 if worse else 0)))

    def clip_gradient(self, g, max_norm):
        """In place: g *= max_norm / ||g|| when ||g|| >= max_norm."""
        self._chk(g)
        self._ck(self.lib.dlmi_clip_gradient(self.ctx, c_sz(g.numel()), _p(g), c_f(max_norm)))

    def max_norm_rows(self, W, max_norm):
        """In place, per row of W [rows, cols]."""
        self._chk(W)
        rows, cols = W.shape
        self._ck(self.lib.dlmi_max_norm_rows(self.ctx, c_sz(rows), c_sz(cols), _p(W), c_f(max_norm)))

    def softmax_ce_seed(self, q, y, stats=None):
        """stats: optional device tensor of 2 float64 accumulators."""
        self._chk(q, y, stats)
        B, H = q.shape
        dZ = self.empty(B, H)
        self._ck(self.lib.dlmi_softmax_ce_seed(self.ctx, c_sz(B), c_sz(H), _p(q), _p(y), _p(dZ), _p(stats)))
        return dZ

    def layer_variance(self, y):
        """Model::get_layer_variance: population variance of all values of y [B, H] (a float, on the host)."""
        self._chk(y)
        out = ctypes.c_float(0)
        B, H = (y.shape[0], y.numel() // y.shape[0]) if y.dim() > 1 else (1, y.numel())
        self._ck(self.lib.dlmi_layer_variance(self.ctx, c_sz(B), c_sz(H), _p(y), ctypes.byref(out)))
        return out.value

    def scale(self, t, factor, n=None):
        """t[0:n] *= factor (scale_parameters_st)."""
        self._chk(t)
        self._ck(self.lib.dlmi_scale(self.ctx, c_sz(t.numel() if n is None else n), _p(t), ctypes.c_float(factor)))
        return t

    def zero(self, t):
        self._chk(t)
        self._ck(self.lib.dlmi_zero(self.ctx, c_sz(t.numel()), _p(t)))
        return t

    def loss_seed(self, loss, accu, accu_threshold, act, z, q, y, stats=None, want_dz=True):
        """Seed gradient of an element-wise output layer; stats: optional device tensor of 2 float64 accumulators."""
        self._chk(z, q, y, stats)
        B, H = q.shape
        dZ = self.empty(B, H) if want_dz else None
        self._ck(self.lib.dlmi_loss_seed(self.ctx, c_int(loss), c_int(accu), c_f(accu_threshold), c_int(act), c_sz(B),
                                         c_sz(H), _p(z), _p(q), _p(y), _p(dZ), _p(stats)))
        return dZ

    # ------------------------------------------------------------ fused hot path
    @staticmethod
    def desc(act, renorm=True, dropout=0, mask_per_element=False, dropout_bwd=0, momentum=0.99, eps=1e-5,
             r_max=3.0, d_max=5.0, drop_scale=1.0):
        return FusedDesc(NORM["BRN"] if renorm else NORM["BN"], act, dropout, 1 if mask_per_element else 0,
                         dropout_bwd, momentum, eps, r_max, d_max, drop_scale)

    def fused_fwd(self, desc, x, gamma, beta, mov_mean, mov_std, mask=None, out=None, stats=None, noalloc=False,
                  shortcut=None):
        """Returns (y, stats) with stats = dict(mean,std,r,d) kept for the backward.
        noalloc: go through dlmi_fused_norm_act_fwd_noalloc (the library's fixed scratch array; the
        caller then passes `out` and `stats` so that nothing is allocated on the way).
        shortcut: y = shortcut + (activation output after dropout), dlmi_fused_norm_act_residual_fwd."""
        self._chk(x, gamma, beta, mov_mean, mov_std, mask, out, shortcut)
        B, H = x.shape
        y = out if out is not None else self.empty(B, H)
        s = stats or dict(mean=self.empty(H), std=self.empty(H), r=self.empty(H), d=self.empty(H))
        if shortcut is not None:
            assert not noalloc and shortcut.shape == x.shape
            self._ck(self.lib.dlmi_fused_norm_act_residual_fwd(
                self.ctx, ctypes.byref(desc), c_sz(B), c_sz(H), _p(x), _p(gamma), _p(beta), _p(mask), _p(shortcut),
                _p(s["mean"]), _p(s["std"]), _p(mov_mean), _p(mov_std), _p(s["r"]), _p(s["d"]), _p(y)))
            return y, s
        fn = self.lib.dlmi_fused_norm_act_fwd_noalloc if noalloc else self.lib.dlmi_fused_norm_act_fwd
        self._ck(fn(self.ctx, ctypes.byref(desc), c_sz(B), c_sz(H), _p(x), _p(gamma),
                                                  _p(beta), _p(mask), _p(s["mean"]), _p(s["std"]), _p(mov_mean),
                                                  _p(mov_std), _p(s["r"]), _p(s["d"]), _p(y)))
        return y, s

    def fc_norm_act_fwd(self, desc, X, W, gamma, beta, mov_mean, mov_std, mask=None, Z=None, out=None, stats=None,
                        shortcut=None):
        """Z = X W^T with the batch statistics taken in the GEMM epilogue, then
        normalization + activation (+ dropout) (+ shortcut).  Returns (Z, y, stats)."""
        self._chk(X, W, gamma, beta, mov_mean, mov_std, mask, Z, out, shortcut)
        B, K = X.shape
        H = W.shape[0]
        Z = Z if Z is not None else self.empty(B, H)
        y = out if out is not None else self.empty(B, H)
        s = stats or dict(mean=self.empty(H), std=self.empty(H), r=self.empty(H), d=self.empty(H))
        if shortcut is not None:
            self._ck(self.lib.dlmi_fc_norm_act_residual_fwd(
                self.ctx, ctypes.byref(desc), c_sz(B), c_sz(K), c_sz(H), _p(X), _p(W), _p(gamma), _p(beta), _p(mask),
                _p(shortcut), _p(Z), _p(s["mean"]), _p(s["std"]), _p(mov_mean), _p(mov_std), _p(s["r"]), _p(s["d"]),
                _p(y)))
            return Z, y, s
        self._ck(self.lib.dlmi_fc_norm_act_fwd(self.ctx, ctypes.byref(desc), c_sz(B), c_sz(K), c_sz(H), _p(X), _p(W),
                                               _p(gamma), _p(beta), _p(mask), _p(Z), _p(s["mean"]), _p(s["std"]),
                                               _p(mov_mean), _p(mov_std), _p(s["r"]), _p(s["d"]), _p(y)))
        return Z, y, s

    def fused_bwd(self, desc, x, gamma, beta, stats, dY, dgamma, dbeta, mask=None, out=None, db=None, accumulate_db=False):
        """db: also form the bias gradient sum_b dX[b, :] in the pass that writes dX (dlmi_fused_norm_act_bwd_db)."""
        self._chk(x, gamma, beta, dY, dgamma, dbeta, mask, out, db)
        B, H = x.shape
        dX = out if out is not None else self.empty(B, H)
        if db is not None:
            self._ck(self.lib.dlmi_fused_norm_act_bwd_db(
                self.ctx, ctypes.byref(desc), c_sz(B), c_sz(H), _p(x), _p(gamma), _p(beta), _p(mask), _p(stats["mean"]),
                _p(stats["std"]), _p(stats["r"]), _p(stats["d"]), _p(dY), _p(dgamma), _p(dbeta), _p(dX), _p(db),
                c_int(1 if accumulate_db else 0)))
            return dX
        self._ck(self.lib.dlmi_fused_norm_act_bwd(self.ctx, ctypes.byref(desc), c_sz(B), c_sz(H), _p(x), _p(gamma),
                                                  _p(beta), _p(mask), _p(stats["mean"]), _p(stats["std"]),
                                                  _p(stats["r"]), _p(stats["d"]), _p(dY), _p(dgamma), _p(dbeta),
                                                  _p(dX)))
        return dX

    def fc_softmax_fwd(self, X, W, bias=None):
        """Z = X W^T + bias, Q = softmax(Z).  Returns (Z, Q)."""
        self._chk(X, W, bias)
        B, K = X.shape
        H = W.shape[0]
        Z, Q = self.empty(B, H), self.empty(B, H)
        self._ck(self.lib.dlmi_fc_softmax_fwd(self.ctx, c_sz(B), c_sz(K), c_sz(H), _p(X), _p(W), _p(bias), _p(Z), _p(Q)))
        return Z, Q

    def fc_softmax_ce_fwd(self, X, W, Y, bias=None, stats=None):
        """Z = X W^T + bias, Q = softmax(Z), dZ = cross-entropy seed gradient against Y, stats (2 doubles on the
        device, optional) += (loss sum, correct predictions).  Returns (Z, Q, dZ)."""
        self._chk(X, W, Y, bias)
        B, K = X.shape
        H = W.shape[0]
        Z, Q, dZ = self.empty(B, H), self.empty(B, H), self.empty(B, H)
        self._ck(self.lib.dlmi_fc_softmax_ce_fwd(self.ctx, c_sz(B), c_sz(K), c_sz(H), _p(X), _p(W), _p(bias), _p(Y),
                                                 _p(Z), _p(Q), _p(dZ), _p(stats)))
        return Z, Q, dZ

    def fc_bwd_dx_fused_bwd(self, desc, dZn, Wn, x, gamma, beta, stats, dgamma, dbeta, mask=None):
        """dY = dZn Wn, then the fused normalization backward on dY.  Returns dX."""
        self._chk(dZn, Wn, x, gamma, beta, dgamma, dbeta, mask)
        B, Hn = dZn.shape
        H = Wn.shape[1]
        assert Wn.shape[0] == Hn and tuple(x.shape) == (B, H)
        dX = self.empty(B, H)
        self._ck(self.lib.dlmi_fc_bwd_dx_norm_act_bwd(
            self.ctx, ctypes.byref(desc), c_sz(B), c_sz(Hn), c_sz(H), _p(dZn), _p(Wn), _p(x), _p(gamma), _p(beta),
            _p(mask), _p(stats["mean"]), _p(stats["std"]), _p(stats["r"]), _p(stats["d"]), _p(dgamma), _p(dbeta), _p(dX)))
        return dX

    def fused_infer(self, desc, x, gamma, beta, mov_mean, mov_std, out=None):
        self._chk(x, gamma, beta, mov_mean, mov_std, out)
        B, H = x.shape
        y = out if out is not None else self.empty(B, H)
        self._ck(self.lib.dlmi_fused_norm_act_infer(self.ctx, ctypes.byref(desc), c_sz(B), c_sz(H), _p(x), _p(gamma),
                                                    _p(beta), _p(mov_mean), _p(mov_std), _p(y)))
        return y
