"""ctypes binding of the C++ Model facade (include/dlmi_model.h): the
reference's Model API for a stack of fully-connected layers, running on the GPU.
Host numpy arrays go in and out here because that is the boundary the reference
has (`forward_pass(batch, rows of X)`); the copies to HBM happen inside the
facade."""
import ctypes

import numpy as np

c_sz = ctypes.c_size_t
c_int = ctypes.c_int
c_f = ctypes.c_float
vp = ctypes.c_void_p

MODEL_C_ABI_SYMBOLS = [
    "dlmi_model_create", "dlmi_model_destroy", "dlmi_model_context", "dlmi_model_last_error", "dlmi_model_set_layer_activation_function",
    "dlmi_model_set_layer_normalization", "dlmi_model_set_layer_normalization_order", "dlmi_model_set_norm_hyper", "dlmi_model_set_dropout",
    "dlmi_model_set_dropout_mask", "dlmi_model_set_dropout_backward_mode", "dlmi_model_prepare",
    "dlmi_model_total_parameters", "dlmi_model_total_normalized_units", "dlmi_model_layer_offsets",
    "dlmi_model_set_parameters", "dlmi_model_get_parameters", "dlmi_model_set_moving", "dlmi_model_get_moving",
    "dlmi_model_get_derivatives", "dlmi_model_clear_training_arrays", "dlmi_model_step", "dlmi_model_download_layer",
    "dlmi_model_get_out", "dlmi_model_loss_sum", "dlmi_model_accuracy_sum", "dlmi_model_set_optimizer",
    "dlmi_model_set_epoch_time_step", "dlmi_model_set_derivatives", "dlmi_model_update_parameter",
    "dlmi_model_get_optimizer_state", "dlmi_driver_create", "dlmi_driver_destroy", "dlmi_driver_train",
    "dlmi_driver_evalt", "dlmi_model_create_typed", "dlmi_model_layer_info", "dlmi_mnist_create",
    "dlmi_mnist_destroy", "dlmi_mnist_load", "dlmi_mnist_last_error", "dlmi_mnist_copy",
    "dlmi_model_glorot_uniform", "dlmi_model_init_uniform", "dlmi_model_set_bound_hyper", "dlmi_model_set_constraints",
    "dlmi_model_set_rprop", "dlmi_model_set_rprop_loss", "dlmi_model_set_warm_restarts",
    "dlmi_model_dropout_bernoulli", "dlmi_model_get_dropout_mask", "dlmi_model_set_loss", "dlmi_model_reset_loss",
    "dlmi_model_loss_accu", "dlmi_driver_set_record_batches", "dlmi_driver_recorded_batches",
    "dlmi_model_set_allowable_memory", "dlmi_model_memory", "dlmi_model_create_empty", "dlmi_model_save_params",
    "dlmi_model_save_spec_params", "dlmi_model_load_spec_params", "dlmi_model_load", "dlmi_model_total_layers",
    "dlmi_checkpointer_create", "dlmi_checkpointer_destroy", "dlmi_checkpointer_save", "dlmi_checkpointer_load",
    "dlmi_model_forward_to", "dlmi_model_lsuv", "dlmi_model_lsuv_trials", "dlmi_model_layer_variance", "dlmi_model_steps",
]

LAYER_FULLY_CONNECTED, LAYER_RESIDUAL = 3, 9  # v1/data/enum/layer.hpp


def _ptr(a):
    return None if a is None else a.ctypes.data_as(vp)


class Model:
    """Same driving interface as the oracle's and the reference's whole-model
    wrappers in oracle/binding.py, so one test body can run all three."""

    def __init__(self, lib, widths):
        self._bind(lib)
        self.widths = [int(w) for w in widths]
        arr = (c_sz * len(widths))(*self.widths)
        h = lib.dlmi_model_create(c_sz(len(widths)), arr)
        self._created(h)

    def _bind(self, lib):
        self.lib = lib
        lib.dlmi_model_create.restype = vp
        lib.dlmi_model_create_typed.restype = vp
        lib.dlmi_model_last_error.restype = ctypes.c_char_p
        lib.dlmi_model_last_error.argtypes = [vp]
        lib.dlmi_model_total_parameters.restype = c_sz
        lib.dlmi_model_total_normalized_units.restype = c_sz
        lib.dlmi_model_loss_sum.restype = ctypes.c_double
        lib.dlmi_model_accuracy_sum.restype = ctypes.c_double

    def _created(self, h):
        if not h:
            raise RuntimeError("dlmi_model_create failed (no GPU, the library is not built for it, or a layer list "
                               "the path does not take)")
        self.h = vp(h)
        self.P = self.lib.dlmi_model_total_parameters(self.h)
        self.n_units = self.lib.dlmi_model_total_normalized_units(self.h)
        self.max_batch = 0

    def close(self):
        for d, _, _ in self.__dict__.pop("_drivers", {}).values():
            self.lib.dlmi_driver_destroy(d)
        if getattr(self, "h", None):
            self.lib.dlmi_model_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _ok(self, rc, what):
        if not rc:
            raise RuntimeError("%s failed: %s" % (what, self.lib.dlmi_model_last_error(self.h).decode()))

    def set_layer(self, l, act, norm=0, drop=0, keep=1.0, mask=None, norm_before=True):
        self._ok(self.lib.dlmi_model_set_layer_activation_function(self.h, c_sz(l), c_int(act)), "activation")
        if norm:
            self._ok(self.lib.dlmi_model_set_layer_normalization_order(self.h, c_sz(l), c_int(int(norm_before))),
                     "normalization order")
            self._ok(self.lib.dlmi_model_set_layer_normalization(self.h, c_sz(l), c_int(norm)), "normalization")
        if drop:
            self._ok(self.lib.dlmi_model_set_dropout(self.h, c_sz(l), c_int(drop), c_f(keep)), "dropout")
        if mask is not None:
            m = np.ascontiguousarray(mask, dtype=np.uint8)
            self._ok(self.lib.dlmi_model_set_dropout_mask(self.h, c_sz(l), _ptr(m)), "dropout mask")
        self._sizes()

    def set_norm_hyper(self, momentum, eps, r_max, d_max):
        self._ok(self.lib.dlmi_model_set_norm_hyper(self.h, c_f(momentum), c_f(eps), c_f(r_max), c_f(d_max)), "hyper")

    def dropout_bernoulli(self, seed=None):
        """[bernoulli[0].seed(seed);] Model::Dropout_Bernoulli()"""
        self._ok(self.lib.dlmi_model_dropout_bernoulli(self.h, ctypes.c_uint(seed or 0), c_int(int(seed is not None))),
                 "Dropout_Bernoulli")

    def dropout_mask(self, l, n):
        out = np.zeros(n, np.uint8)
        self._ok(self.lib.dlmi_model_get_dropout_mask(self.h, c_sz(l), _ptr(out)), "dropout mask")
        return out

    def set_dropout_backward_mode(self, masked):
        self.lib.dlmi_model_set_dropout_backward_mode(self.h, c_int(1 if masked else 0))

    def layer_offsets(self, l):
        out = (c_sz * 6)()
        self.lib.dlmi_model_layer_offsets(self.h, c_sz(l), out)
        return list(out)

    def prepare(self, max_batch, nthreads=0):
        self.max_batch = max_batch
        self._ok(self.lib.dlmi_model_prepare(self.h, c_sz(max_batch)), "prepare")
        self._sizes()

    def _sizes(self):
        """The scale / shift slots exist only once a layer is normalized: re-read the lengths."""
        self.P = self.lib.dlmi_model_total_parameters(self.h)
        self.n_units = self.lib.dlmi_model_total_normalized_units(self.h)

    def set_parameters(self, p):
        p = np.ascontiguousarray(p, np.float32)
        self._ok(self.lib.dlmi_model_set_parameters(self.h, _ptr(p), c_sz(p.size)), "set_parameters")

    def get_parameters(self):
        p = np.empty(self.P, np.float32)
        self._ok(self.lib.dlmi_model_get_parameters(self.h, _ptr(p), c_sz(self.P)), "get_parameters")
        return p

    def set_moving(self, mean, std):
        mean = np.ascontiguousarray(mean, np.float32)
        std = np.ascontiguousarray(std, np.float32)
        self._ok(self.lib.dlmi_model_set_moving(self.h, _ptr(mean), _ptr(std), c_sz(self.n_units)), "set_moving")

    def get_moving(self):
        mean = np.empty(self.n_units, np.float32)
        std = np.empty(self.n_units, np.float32)
        self._ok(self.lib.dlmi_model_get_moving(self.h, _ptr(mean), _ptr(std), c_sz(self.n_units)), "get_moving")
        return mean, std

    def clear_training_arrays(self):
        self.lib.dlmi_model_clear_training_arrays(self.h)

    def glorot_uniform(self, seed, bias=0.0):
        """real_gen.seed(seed); initialize_weights_with_glorot_uniform(bias)"""
        self.lib.dlmi_model_glorot_uniform(self.h, ctypes.c_uint(seed), c_f(bias))

    def glorot_gaussian(self, seed, bias=0.0):
        """gaussian_gen.seed(seed); Initialization__Glorot__Gaussian(bias)"""
        self.lib.dlmi_model_glorot_gaussian(self.h, ctypes.c_uint(seed), c_f(bias))

    def init_identity(self, bias=0.0):
        """Initialization__Identity(bias)"""
        self.lib.dlmi_model_init_identity(self.h, c_f(bias))

    def init_uniform(self, seed, bias=0.0, lower=-1.0, upper=1.0):
        """real_gen.seed(seed); Initialization__Uniform(bias, lower, upper)"""
        self.lib.dlmi_model_init_uniform(self.h, ctypes.c_uint(seed), c_f(bias), c_f(lower), c_f(upper))

    def step(self, state, X, Y=None, backward=True):
        X = np.ascontiguousarray(X, np.float32)
        self.B = X.shape[0]
        Yp = None
        if backward:
            Y = np.ascontiguousarray(Y, np.float32)
            Yp = _ptr(Y)
        self._ok(self.lib.dlmi_model_step(self.h, c_int(state), c_sz(self.B), _ptr(X), Yp, c_int(1 if backward else 0)),
                 "step")

    def steps(self, state, X, Y, batch, backward=True):
        """len(X) / batch steps on consecutive row blocks, the host waiting only after the last one."""
        X = np.ascontiguousarray(X, np.float32)
        Y = np.ascontiguousarray(Y, np.float32)
        n = X.shape[0] // batch
        self.B = batch
        self._ok(self.lib.dlmi_model_steps(self.h, c_int(state), c_sz(n), c_sz(batch), _ptr(X), _ptr(Y),
                                           c_int(1 if backward else 0)), "steps")

    def forward_to(self, state, X, end_layer):
        """forward_pass(B, X, 0, end_layer): layers [1, end_layer) only."""
        X = np.ascontiguousarray(X, np.float32)
        self.B = X.shape[0]
        self._ok(self.lib.dlmi_model_forward_to(self.h, c_int(state), c_sz(self.B), _ptr(X), c_sz(end_layer)), "forward_to")

    def orthogonal(self, seed, bias=0.0):
        """gaussian_gen.seed(seed); layers_initialize_orthogonal(false, bias)"""
        self.lib.dlmi_model_orthogonal(self.h, ctypes.c_uint(seed), c_f(bias))

    def seed_gaussian(self, seed):
        self.lib.dlmi_model_seed_gaussian(self.h, ctypes.c_uint(seed))

    def gaussian_draws(self, n):
        out = np.empty(n, np.float32)
        self.lib.dlmi_model_gaussian_draws(self.h, c_sz(n), _ptr(out))
        return out

    def lsuv(self, X, max_n_trials=10, max_batch_size=32, bias=0.0, var_target=1.0, var_tolerance=0.01, pre_initialize=True):
        """Initialize__LSUV + Initialization__LSUV on the rows of X; returns the scalings applied per layer.
        pre_initialize=False: the scaling loop alone, on the weights the model holds."""
        X = np.ascontiguousarray(X, np.float32)
        self._ok(self.lib.dlmi_model_lsuv(self.h, c_sz(max_n_trials), c_sz(max_batch_size), c_f(bias), c_f(var_target),
                                          c_f(var_tolerance), c_sz(X.shape[0]), _ptr(X), c_int(1 if pre_initialize else 0)),
                 "Initialization__LSUV")
        self.lib.dlmi_model_lsuv_trials.restype = c_sz
        return [int(self.lib.dlmi_model_lsuv_trials(self.h, c_sz(l))) for l in range(len(self.widths))]

    def layer_variance(self, l, batch):
        self.lib.dlmi_model_layer_variance.restype = c_f
        return float(self.lib.dlmi_model_layer_variance(self.h, c_sz(l), c_sz(batch)))

    def layer_buffer(self, l, which):
        out = np.empty((self.B, self.widths[l]), np.float32)
        self._ok(self.lib.dlmi_model_download_layer(self.h, c_sz(l), c_int(which), c_sz(self.B), _ptr(out)), "download")
        return out

    def layer_vector(self, l, which):
        out = np.empty(self.widths[l], np.float32)
        self._ok(self.lib.dlmi_model_download_layer(self.h, c_sz(l), c_int(10 + which), c_sz(1), _ptr(out)), "download")
        return out

    def get_out(self):
        out = np.empty((self.B, self.widths[-1]), np.float32)
        for i in range(self.B):
            self._ok(self.lib.dlmi_model_get_out(self.h, c_sz(i), _ptr(out[i])), "get_out")
        return out

    def get_dparams(self):
        p = np.empty(self.P, np.float32)
        self._ok(self.lib.dlmi_model_get_derivatives(self.h, _ptr(p), c_sz(self.P)), "get_derivatives")
        return p

    def set_allowable_memory(self, nbytes):
        """maximum_allowable_memory_bytes: the device-memory budget update_mem_batch_size() sizes the batch for."""
        self.lib.dlmi_model_set_allowable_memory(self.h, c_sz(nbytes))

    def memory(self):
        out = (c_sz * 4)()
        self.lib.dlmi_model_memory(self.h, out)
        return dict(zip(("budget", "model_bytes", "bytes_per_example", "batch_size"), (int(v) for v in out)))

    def lanes_enabled(self):
        """Whether the epoch driver runs this model's mini-batches on two sets of per-batch buffers."""
        return bool(self.lib.dlmi_model_lanes_enabled(self.h))

    def set_loss(self, loss, accu, acc_var=0.49):
        """set_loss_fn / set_accu_fn / Set__Accurancy_Variance (after prepare, which selects cross-entropy)."""
        self._ok(self.lib.dlmi_model_set_loss(self.h, c_int(loss), c_int(accu), c_f(acc_var)), "set_loss")

    def reset_loss(self):
        self.lib.dlmi_model_reset_loss(self.h)

    def loss_accu(self, n_data):
        """(get_loss(NONE), get_accu(NONE)) as the epoch driver reports them after n_data examples."""
        out = (ctypes.c_double * 2)()
        self.lib.dlmi_model_loss_accu(self.h, c_sz(n_data), out)
        return out[0], out[1]

    def loss_sum(self):
        return self.lib.dlmi_model_loss_sum(self.h)

    def accuracy_sum(self):
        return self.lib.dlmi_model_accuracy_sum(self.h)

    # ---- optimizer (Model::set_optimizer / set_weight_decay / Update_Parameter) ----
    def set_optimizer(self, kind, lr=0.01, momentum=0.9, nesterov=False, adam_lr=0.001, beta1=0.9, beta2=0.999,
                      eps=1e-8, bias_correction=True, weight_decay=0.0, normalized_wd=True, lr_final=0.1, gamma=1e-3,
                      adam_gamma=0.1, clip=None, max_norm=0.0, rprop=(1.2, 0.5, 1e-6, 50.0, 0.1), rprop_losses=None,
                      warm_restarts=None):
        """rprop: iRPROP+ (increase, decrease, delta_min, delta_max, delta_zero).  rprop_losses: a recorded
        sequence of [loss_rprop, loss_rprop_tm1] to install before each update_parameter() call, for callers
        that drive the updates themselves (train_epoch keeps the two losses on its own).  warm_restarts: None
        or (decay of the peak rate, peak rate, floor, first period in steps, period multiplier)."""
        wr = warm_restarts or (1.0, 1.0, 1e-7, 1.0, 2.0)
        self.lib.dlmi_model_set_warm_restarts(self.h, c_int(int(warm_restarts is not None)), *(c_f(v) for v in wr))
        self.lib.dlmi_model_set_bound_hyper(self.h, c_f(lr_final), c_f(gamma), c_f(adam_gamma))
        self.lib.dlmi_model_set_rprop(self.h, *(c_f(v) for v in rprop))
        self._rprop_losses, self._n_updates = rprop_losses, 0
        self._ok(self.lib.dlmi_model_set_constraints(self.h, c_int(int(clip is not None)),
                                                     c_f(1.0 if clip is None else clip), c_f(max_norm)), "constraints")
        self._ok(self.lib.dlmi_model_set_optimizer(self.h, c_int(kind), c_f(lr), c_f(momentum), c_int(int(nesterov)),
                                                   c_f(adam_lr), c_f(beta1), c_f(beta2), c_f(eps),
                                                   c_int(int(bias_correction)), c_f(weight_decay),
                                                   c_int(int(normalized_wd))), "set_optimizer")

    def set_epoch_time_step(self, v):
        self.lib.dlmi_model_set_epoch_time_step(self.h, c_f(v))

    def set_dparams(self, g):
        g = np.ascontiguousarray(g, np.float32)
        self._ok(self.lib.dlmi_model_set_derivatives(self.h, _ptr(g), c_sz(g.size)), "set_derivatives")

    def update_parameter(self, batch, training_size):
        if getattr(self, "_rprop_losses", None) is not None:
            loss, loss_tm1 = self._rprop_losses[self._n_updates]
            self.lib.dlmi_model_set_rprop_loss(self.h, ctypes.c_double(loss), ctypes.c_double(loss_tm1))
        self._n_updates = getattr(self, "_n_updates", 0) + 1
        self.lib.dlmi_model_update_parameter(self.h, c_sz(batch), c_sz(training_size))

    def opt_state(self, which):
        out = np.empty(self.P, np.float32)
        ok = self.lib.dlmi_model_get_optimizer_state(self.h, c_int(which), _ptr(out))
        return out if ok else None

    # ---- epoch driver (Driver::train / Driver::evalt) -------------------------------
    def _driver(self, X, Y, on_device=True):
        """One driver per data set (identified by the arrays' contents' identity)."""
        X, Y = np.ascontiguousarray(X, np.float32), np.ascontiguousarray(Y, np.float32)
        key = (X.ctypes.data, Y.ctypes.data, X.shape, on_device)
        drivers = self.__dict__.setdefault("_drivers", {})
        if key not in drivers:
            self.lib.dlmi_driver_create.restype = vp
            d = self.lib.dlmi_driver_create(self.h, c_sz(X.shape[0]), _ptr(X), _ptr(Y), c_int(1), c_int(int(on_device)))
            if not d:
                raise RuntimeError("dlmi_driver_create failed")
            drivers[key] = (vp(d), X, Y)  # the arrays stay alive with the key
        return drivers[key][0]

    def train_epoch(self, X, Y, resample_masks=False, on_device=True, record_batches=None):
        """record_batches: None leaves Driver::record_batches as it is (on, unless DLMI_RECORD_BATCHES=0)."""
        out = (ctypes.c_double * 2)()
        d = self._driver(X, Y, on_device)
        if record_batches is not None:
            self.lib.dlmi_driver_set_record_batches(d, c_int(int(record_batches)))
        self._ok(self.lib.dlmi_driver_train(d, c_int(int(resample_masks)), out), "Driver::train")
        return out[0], out[1]

    def set_record_batches(self, X, Y, on, on_device=True):
        self.lib.dlmi_driver_set_record_batches(self._driver(X, Y, on_device), c_int(int(on)))

    def recorded_batches(self, X, Y, on_device=True):
        """Mini-batches of this data set's driver that are held as HIP graphs (training plus evaluation passes)."""
        self.lib.dlmi_driver_recorded_batches.restype = c_sz
        return int(self.lib.dlmi_driver_recorded_batches(self._driver(X, Y, on_device)))

    # ---- text files of the reference (Model::save_params / save_spec_params / load) ----
    def save_params(self, path):
        """`model.net`: dimensions, per-layer settings, weights, biases, scales / shifts, moving statistics."""
        self._ok(self.lib.dlmi_model_save_params(self.h, str(path).encode()), "save_params")

    def save_spec_params(self, path):
        """`model.nn`: the hyper-parameter sections."""
        self._ok(self.lib.dlmi_model_save_spec_params(self.h, str(path).encode()), "save_spec_params")

    def load_spec_params(self, path):
        self._ok(self.lib.dlmi_model_load_spec_params(self.h, str(path).encode()), "load_spec_params")

    def load_files(self, path_params, path_spec_params, allowable_memory=0):
        """Model::load into THIS model (cleared first); False with last_error() set when the files are refused."""
        ok = bool(self.lib.dlmi_model_load(self.h, str(path_params).encode(), str(path_spec_params).encode(),
                                           c_sz(allowable_memory)))
        if ok:
            self.P = self.lib.dlmi_model_total_parameters(self.h)
            self.n_units = self.lib.dlmi_model_total_normalized_units(self.h)
            self.lib.dlmi_model_total_layers.restype = c_sz
            n = int(self.lib.dlmi_model_total_layers(self.h))
            info = (c_sz * 12)()
            self.widths = []
            for l in range(n):
                self.lib.dlmi_model_layer_info(self.h, c_sz(l), info)
                self.widths.append(int(info[1]))
        return ok

    @classmethod
    def load(cls, lib, path_params, path_spec_params, allowable_memory=0):
        """A new model read from the two files."""
        self = cls.__new__(cls)
        self._bind(lib)
        lib.dlmi_model_create_empty.restype = vp
        self.h = vp(lib.dlmi_model_create_empty())
        self.P = self.n_units = self.max_batch = 0
        self.widths = []
        if not self.load_files(path_params, path_spec_params, allowable_memory):
            err = self.last_error()
            self.close()
            raise RuntimeError("Model::load failed: " + err)
        return self

    def last_error(self):
        return self.lib.dlmi_model_last_error(self.h).decode()

    def context(self):
        """The dlmi_ctx handle the model's kernels run on (owned by the model)."""
        self.lib.dlmi_model_context.restype = vp
        return vp(self.lib.dlmi_model_context(self.h))

    def evalt(self, X, Y, on_device=True):
        out = (ctypes.c_double * 2)()
        self._ok(self.lib.dlmi_driver_evalt(self._driver(X, Y, on_device), out), "Driver::evalt")
        return out[0], out[1]


def load_mnist(lib, workdir, train=True):
    """dlmi::MNIST(workdir).load(ENV::TRAIN or ENV::TESTG): (X [n, rows*cols] in [0, 1],
    Y [n, 10] one-hot) from the IDX files in `workdir`.  Host code only (no GPU needed)."""
    lib.dlmi_mnist_create.restype = vp
    lib.dlmi_mnist_last_error.restype = ctypes.c_char_p
    lib.dlmi_mnist_last_error.argtypes = [vp]
    h = vp(lib.dlmi_mnist_create(str(workdir).encode()))
    try:
        shape = (c_sz * 3)()
        if not lib.dlmi_mnist_load(h, c_int(1 if train else 3), shape):
            raise RuntimeError("MNIST::load failed: " + lib.dlmi_mnist_last_error(h).decode())
        X = np.empty((shape[0], shape[1]), np.float32)
        Y = np.empty((shape[0], shape[2]), np.float32)
        if not lib.dlmi_mnist_copy(h, _ptr(X), _ptr(Y)):
            raise RuntimeError("dlmi_mnist_copy failed")
        return X, Y
    finally:
        lib.dlmi_mnist_destroy(h)


class Net(Model):
    """A Model compiled from a typed layer list: ("FC", units) entries and
    ("RES", depth) entries, each of the latter followed by the `depth` layers of its
    residual block.  Entry 0 is the input width.  Same driving interface as
    OracleNet / ReferenceNet in oracle/binding.py."""

    INFO_KEYS = ("type", "n_out", "w0", "w1", "bias", "use_bias", "n_unit", "gamma", "unit", "n_af", "depth", "padding")

    def __init__(self, lib, layers):
        self._bind(lib)
        self.layers = list(layers)
        n = len(self.layers)
        types = (c_int * n)(*[LAYER_FULLY_CONNECTED if e[0] == "FC" else LAYER_RESIDUAL for e in self.layers])
        units = (c_sz * n)(*[int(e[1]) for e in self.layers])
        self._created(lib.dlmi_model_create_typed(c_sz(n), types, units))
        self.widths = [self.info(l)["n_out"] for l in range(n)]

    def info(self, l):
        out = (c_sz * 12)()
        self.lib.dlmi_model_layer_info(self.h, c_sz(l), out)
        return dict(zip(self.INFO_KEYS, (int(v) for v in out)))

    def fc_layers(self):
        return [l for l, e in enumerate(self.layers) if l > 0 and e[0] == "FC"]

    def set_layer(self, l, act, norm=0, drop=0, keep=1.0, mask=None, norm_before=True):
        if self.layers[l][0] == "FC":
            self._ok(self.lib.dlmi_model_set_layer_activation_function(self.h, c_sz(l), c_int(act)), "activation")
        if norm:
            self._ok(self.lib.dlmi_model_set_layer_normalization(self.h, c_sz(l), c_int(norm)), "normalization")
        if drop:
            self._ok(self.lib.dlmi_model_set_dropout(self.h, c_sz(l), c_int(drop), c_f(keep)), "dropout")
        if mask is not None:
            m = np.ascontiguousarray(mask, dtype=np.uint8)
            assert m.size == self.info(l)["n_unit"], "one mask entry per dropout unit of the entry"
            self._ok(self.lib.dlmi_model_set_dropout_mask(self.h, c_sz(l), _ptr(m)), "dropout mask")
        self._sizes()

    def layer_output(self, l):
        return self.layer_buffer(l, 3)

    def layer_error(self, l):
        return self.layer_buffer(l, 4)


class Checkpointer:
    """nn/checkpointer.cpp: `<dir>/ckpt-<step>/{model.net, model.nn}` plus the `<dir>/checkpoint` pointer file,
    the `max_to_keep` newest directories kept."""

    def __init__(self, model, directory, max_to_keep=5):
        self.model, self.lib = model, model.lib
        self.lib.dlmi_checkpointer_create.restype = vp
        self.h = vp(self.lib.dlmi_checkpointer_create(str(directory).encode(), model.h, c_int(max_to_keep)))
        if not self.h:
            raise RuntimeError("dlmi_checkpointer_create failed")

    def save(self, step):
        return bool(self.lib.dlmi_checkpointer_save(self.h, c_int(int(step))))

    def load(self):
        ok = bool(self.lib.dlmi_checkpointer_load(self.h))
        if ok:
            self.model.P = self.lib.dlmi_model_total_parameters(self.model.h)
            self.model.n_units = self.lib.dlmi_model_total_normalized_units(self.model.h)
        return ok

    def close(self):
        if getattr(self, "h", None):
            self.lib.dlmi_checkpointer_destroy(self.h)
            self.h = None
