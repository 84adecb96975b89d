"""ctypes binding of libglades_hip.so (the C ABI in include/glades_hip.h).

No CPU fallback: if the library is missing or no gfx950 device is usable, calls raise.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
LIB_PATH = os.path.join(PKG, "libglades_hip.so")
MAX_LAYERS = 16

TANH, TANHP, SIGMOID, SIGMOIDP, LINEAR, RELU, LEAKY, STEP, SOFTMAX = range(9)
REGRESSION, CLASSIFICATION, KL = range(3)
MODE_EXACT, MODE_CANONICAL = 0, 1
F32, BF16, FP8_INFER = 0, 1, 2
BIAS_SEQUENTIAL, BIAS_CLOSED_FORM = 0, 1
FP8_ACT_PER_TOKEN, FP8_ACT_BLOCK32 = 0, 1
CANON_PATH_AUTO, CANON_PATH_LAUNCHES, CANON_PATH_ONE_WORKGROUP = 0, 1, 2

EXPORTS = [
    "ghip_init", "ghip_gmath_eval", "ghip_net_create", "ghip_net_destroy", "ghip_net_set_params", "ghip_net_get_params",
    "ghip_net_get_state", "ghip_net_set_state",
    "ghip_net_set_dropout_masks", "ghip_net_get_dropout_state", "ghip_net_set_dropout_state",
    "ghip_net_set_dataset", "ghip_net_set_dataset_device", "ghip_net_run_epochs_exact", "ghip_net_run_epochs_exact_multi",
    "ghip_net_run_epoch_canonical", "ghip_net_run_epochs_canonical", "ghip_net_set_canonical_path", "ghip_net_train_step", "ghip_net_last_metrics", "ghip_net_forward", "ghip_net_forward_resident", "ghip_forward_noalloc", "ghip_net_eval_resident",
    "ghip_net_confusion_enable", "ghip_net_confusion_reset", "ghip_net_confusion_get", "ghip_net_class_metrics",
    "ghip_net_quantize_fp8", "ghip_net_set_fp8_activation_scaling", "ghip_quantize_rows_e4m3_block32", "ghip_net_sync", "ghip_net_profile", "ghip_net_profile_count",
    "ghip_net_profile_entry", "ghip_net_profile_reset", "ghip_last_error", "ghip_version",
]


class Spec(C.Structure):
    _fields_ = [
        ("n_layers", C.c_int),
        ("sizes", C.c_int * (MAX_LAYERS + 1)),
        ("lr", C.c_float * MAX_LAYERS),
        ("mom", C.c_float * MAX_LAYERS),
        ("wd1", C.c_float * MAX_LAYERS),
        ("wd2", C.c_float * MAX_LAYERS),
        ("act", C.c_int * MAX_LAYERS),
        ("act_param", C.c_float * MAX_LAYERS),
        ("batch", C.c_int),
        ("cost", C.c_int),
        ("mode", C.c_int),
        ("dtype", C.c_int),
        ("bias_mode", C.c_int),
    ]


class Metrics(C.Structure):
    _fields_ = [("loss", C.c_float), ("accuracy", C.c_float), ("correct", C.c_int64)]


METRICS_DTYPE = np.dtype([("loss", "<f4"), ("accuracy", "<f4"), ("correct", "<i8")])  # Metrics as a numpy record
assert METRICS_DTYPE.itemsize == C.sizeof(Metrics)


class ClassMetrics(C.Structure):
    _fields_ = [("accuracy", C.c_float), ("precision", C.c_float), ("recall", C.c_float),
                ("specificity", C.c_float), ("f1", C.c_float)]


class GladesHipError(RuntimeError):
    pass


_lib = None


def load():
    """Loads the built library (raises if it was not built: there is no fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise GladesHipError(f"{LIB_PATH} is missing: build it with `python glades-ml_amd/build.py`")
        L = C.CDLL(LIB_PATH)
        vp, i, f, i64 = C.c_void_p, C.c_int, C.c_float, C.c_int64
        sig = {
            "ghip_init": (i, [i]),
            "ghip_gmath_eval": (i, [i, i, f, vp, vp, vp, i64]),
            "ghip_net_create": (i, [C.POINTER(Spec), C.POINTER(vp)]),
            "ghip_net_destroy": (i, [vp]),
            "ghip_net_set_params": (i, [vp, i, vp, vp, i]),
            "ghip_net_get_params": (i, [vp, i, vp, vp, i]),
            "ghip_net_get_state": (i, [vp, i, vp, vp]),
            "ghip_net_set_state": (i, [vp, i, vp, vp]),
            "ghip_net_set_dropout_masks": (i, [vp, vp, i]),
            "ghip_net_get_dropout_state": (i, [vp, i, vp, vp]),
            "ghip_net_set_dropout_state": (i, [vp, i, vp, vp]),
            "ghip_net_set_dataset": (i, [vp, vp, vp, i64]),
            "ghip_net_set_dataset_device": (i, [vp, vp, vp, i64]),
            "ghip_net_run_epochs_exact": (i, [vp, i, i, f, vp, C.POINTER(i), vp]),
            "ghip_net_run_epochs_exact_multi": (i, [vp, i, i, i, f, vp, vp]),
            "ghip_net_run_epoch_canonical": (i, [vp, i, i, C.POINTER(Metrics)]),
            "ghip_net_run_epochs_canonical": (i, [vp, i, i, i, f, vp, C.POINTER(i)]),
            "ghip_net_set_canonical_path": (i, [vp, i]),
            "ghip_net_train_step": (i, [vp, i64, i, vp]),
            "ghip_net_last_metrics": (i, [vp, C.POINTER(Metrics)]),
            "ghip_net_forward": (i, [vp, vp, i, vp]),
            "ghip_net_forward_resident": (i, [vp, i64, i, vp]),
            "ghip_forward_noalloc": (i, [C.POINTER(Spec), C.POINTER(vp), C.POINTER(vp), vp, i, vp, vp]),
            "ghip_net_eval_resident": (i, [vp, i64, i, C.POINTER(Metrics)]),
            "ghip_net_confusion_enable": (i, [vp, i]),
            "ghip_net_confusion_reset": (i, [vp]),
            "ghip_net_confusion_get": (i, [vp, vp, i64]),
            "ghip_net_class_metrics": (i, [vp, i, C.POINTER(ClassMetrics)]),
            "ghip_net_quantize_fp8": (i, [vp, vp, vp]),
            "ghip_net_set_fp8_activation_scaling": (i, [vp, i]),
            "ghip_quantize_rows_e4m3_block32": (i, [vp, i64, i, vp, vp]),
            "ghip_net_sync": (i, [vp]),
            "ghip_net_profile": (i, [vp, i]),
            "ghip_net_profile_count": (i, [vp]),
            "ghip_net_profile_entry": (i, [vp, i, C.c_char_p, i, C.POINTER(C.c_double), C.POINTER(i64)]),
            "ghip_net_profile_reset": (i, [vp]),
            "ghip_last_error": (C.c_char_p, []),
            "ghip_version": (C.c_char_p, []),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def _check(rc):
    if rc != 0:
        raise GladesHipError(f"[{rc}] {load().ghip_last_error().decode()}")


def make_spec(sizes, acts, lr=0.01, mom=0.0, wd1=0.0, wd2=0.0, act_params=0.0, batch=1, cost=REGRESSION,
              mode=MODE_EXACT, dtype=F32, bias_mode=BIAS_SEQUENTIAL):
    nl = len(sizes) - 1

    def per(v):
        return list(v) if isinstance(v, (list, tuple, np.ndarray)) else [v] * nl

    s = Spec()
    s.n_layers = nl
    for k, v in enumerate(sizes):
        s.sizes[k] = int(v)
    for name, v in (("lr", lr), ("mom", mom), ("wd1", wd1), ("wd2", wd2), ("act_param", act_params)):
        arr = getattr(s, name)
        for k, x in enumerate(per(v)):
            arr[k] = float(x)
    for k, a in enumerate(per(acts)):
        s.act[k] = int(a)
    s.batch, s.cost, s.mode, s.dtype, s.bias_mode = int(batch), int(cost), int(mode), int(dtype), int(bias_mode)
    return s


def _ptr(a):
    return None if a is None else C.c_void_p(a.ctypes.data)


def quantize_rows_e4m3_block32(x):
    """The block-scaled e4m3 quantiser on its own: (codes [rows][cols], E8M0 bytes [rows][ceil(cols / 32)])."""
    x = np.ascontiguousarray(x, np.float32)
    codes = np.empty(x.shape, np.uint8)
    scales = np.empty((x.shape[0], (x.shape[1] + 31) // 32), np.uint8)
    _check(load().ghip_quantize_rows_e4m3_block32(_ptr(x), x.shape[0], x.shape[1], _ptr(codes), _ptr(scales)))
    return codes, scales


def gmath_eval(fn, kind, a, b=None, param=0.0):
    """fn 0 squash, 1 activationErrDer, 2 outputNodeCost(expected a, predicted b, dataSize param),
    3 costErrDer(expected a, predicted b), element by element on the device with exact mode's arithmetic;
    4 the layer bias after one row's chain of subtractions (a: bias before, b: [cases][64] lr*d, param:
    rounds; kind 0 walked, 1 as the kernel does it, 2 whether the integer shortcut applies)."""
    a = np.ascontiguousarray(a, np.float32)
    b = None if b is None else np.ascontiguousarray(b, np.float32)
    if b is not None and b.size != a.size * (64 if fn == 4 else 1):
        raise ValueError("b has %d elements for %d cases" % (b.size, a.size))
    out = np.empty_like(a)
    _check(load().ghip_gmath_eval(int(fn), int(kind), float(param), _ptr(a), _ptr(b), _ptr(out), a.size))
    return out


class Net:
    """One device-side network (owns a stream).  Host arrays are numpy float32."""

    def __init__(self, spec, device=0):
        self.lib = load()
        _check(self.lib.ghip_init(device))
        self.spec = spec
        self.sizes = [spec.sizes[k] for k in range(spec.n_layers + 1)]
        self.nl = spec.n_layers
        h = C.c_void_p()
        _check(self.lib.ghip_net_create(C.byref(spec), C.byref(h)))
        self.h = h
        self.n_rows = 0

    def close(self):
        if getattr(self, "h", None):
            self.lib.ghip_net_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---- parameters
    def set_params(self, l, W, bias=None):
        W = np.ascontiguousarray(W, np.float32)
        assert W.shape == (self.sizes[l + 1], self.sizes[l])
        if bias is None:
            _check(self.lib.ghip_net_set_params(self.h, l, _ptr(W), None, 0))
        else:
            b = np.ascontiguousarray(np.atleast_1d(bias), np.float32)
            _check(self.lib.ghip_net_set_params(self.h, l, _ptr(W), _ptr(b), b.size))

    def get_params(self, l):
        W = np.empty((self.sizes[l + 1], self.sizes[l]), np.float32)
        blen = 1 if self.spec.mode == MODE_EXACT else self.sizes[l + 1]
        b = np.zeros((blen,), np.float32)
        _check(self.lib.ghip_net_get_params(self.h, l, _ptr(W), _ptr(b), blen))
        return W, b

    def get_state(self, l):
        """exact: (pending-delta sums, last pending delta); canonical: (weight momentum, bias momentum)."""
        a = np.empty((self.sizes[l + 1], self.sizes[l]), np.float32)
        b = np.empty((self.sizes[l + 1], self.sizes[l]) if self.spec.mode == MODE_EXACT else (self.sizes[l + 1],), np.float32)
        _check(self.lib.ghip_net_get_state(self.h, l, _ptr(a), _ptr(b)))
        return a, b

    def set_state(self, l, a, b):
        a = np.ascontiguousarray(a, np.float32)
        b = np.ascontiguousarray(b, np.float32)
        _check(self.lib.ghip_net_set_state(self.h, l, _ptr(a), _ptr(b)))

    def set_dropout_masks(self, masks):
        """masks: epochs x n_rows x sum(sizes[:-1]) uint8 (1 = dropped) for the next exact run, or None."""
        if masks is None:
            _check(self.lib.ghip_net_set_dropout_masks(self.h, None, 0))
            return
        masks = np.ascontiguousarray(masks, np.uint8)
        assert masks.ndim == 3 and masks.shape[1:] == (self.n_rows, sum(self.sizes[:-1])), masks.shape
        _check(self.lib.ghip_net_set_dropout_masks(self.h, _ptr(masks), masks.shape[0]))

    def get_dropout_state(self, l):
        """(pending-delta counts of weight layer l, error accumulators of the nodes of layer l+1)."""
        c = np.empty((self.sizes[l + 1], self.sizes[l]), np.int32)
        e = np.empty(self.sizes[l + 1], np.float32)
        _check(self.lib.ghip_net_get_dropout_state(self.h, l, _ptr(c), _ptr(e)))
        return c, e

    def set_dropout_state(self, l, counts, errder):
        c = None if counts is None else np.ascontiguousarray(counts, np.int32)
        e = None if errder is None else np.ascontiguousarray(errder, np.float32)
        _check(self.lib.ghip_net_set_dropout_state(self.h, l, _ptr(c), _ptr(e)))

    # ---- data
    def set_dataset(self, X, Y):
        X = np.ascontiguousarray(X, np.float32)
        Y = None if Y is None else np.ascontiguousarray(Y, np.float32)
        assert X.shape[1] == self.sizes[0]
        _check(self.lib.ghip_net_set_dataset(self.h, _ptr(X), _ptr(Y), X.shape[0]))
        self.n_rows = X.shape[0]

    def set_dataset_device(self, x_ptr, y_ptr, n_rows):
        """x_ptr / y_ptr: integer device addresses of fp32 tables the caller keeps alive."""
        _check(self.lib.ghip_net_set_dataset_device(self.h, C.c_void_p(x_ptr), C.c_void_p(y_ptr) if y_ptr else None, n_rows))
        self.n_rows = n_rows

    # ---- exact mode
    def run_epochs_exact(self, n_epochs, train=True, stop_accuracy=0.0, want_preds=False):
        ms = (Metrics * n_epochs)()
        ran = C.c_int(0)
        preds = np.empty((self.n_rows, self.sizes[-1]), np.float32) if want_preds else None
        _check(self.lib.ghip_net_run_epochs_exact(self.h, n_epochs, 1 if train else 0, float(stop_accuracy),
                                                  C.cast(ms, C.c_void_p), C.byref(ran), _ptr(preds)))
        out = [(ms[k].loss, ms[k].accuracy, ms[k].correct) for k in range(ran.value)]
        return out, preds

    # ---- confusion matrix
    def confusion_enable(self, enable=True):
        _check(self.lib.ghip_net_confusion_enable(self.h, 1 if enable else 0))

    def confusion_reset(self):
        _check(self.lib.ghip_net_confusion_reset(self.h))

    def confusion(self):
        n = self.sizes[-1]
        M = np.zeros((n, n), np.int32)
        _check(self.lib.ghip_net_confusion_get(self.h, _ptr(M), n * n))
        return M

    def class_metrics(self, epoch):
        m = ClassMetrics()
        _check(self.lib.ghip_net_class_metrics(self.h, epoch, C.byref(m)))
        return np.array([m.accuracy, m.precision, m.recall, m.specificity, m.f1], np.float32)

    # ---- canonical mode
    def train_step(self, row0, batch, want_metrics=True):
        if want_metrics:
            m = Metrics()
            _check(self.lib.ghip_net_train_step(self.h, row0, batch, C.cast(C.byref(m), C.c_void_p)))
            return m
        _check(self.lib.ghip_net_train_step(self.h, row0, batch, None))
        return None

    def run_epoch_canonical(self, batch, train=True):
        """One pass over the resident table in batches of `batch`; one synchronisation at the end."""
        m = Metrics()
        _check(self.lib.ghip_net_run_epoch_canonical(self.h, int(batch), 1 if train else 0, C.byref(m)))
        return m

    def run_epochs_canonical(self, batch, n_epochs, train=True, stop_accuracy=0.0):
        """Up to n_epochs passes (one launch for a narrow fp32 network): list of (loss, accuracy, correct) per epoch run."""
        ms = (Metrics * n_epochs)()
        ran = C.c_int(0)
        _check(self.lib.ghip_net_run_epochs_canonical(self.h, int(batch), int(n_epochs), 1 if train else 0, float(stop_accuracy),
                                                      C.cast(ms, C.c_void_p), C.byref(ran)))
        return [(ms[e].loss, ms[e].accuracy, ms[e].correct) for e in range(ran.value)]

    def set_canonical_path(self, path):
        _check(self.lib.ghip_net_set_canonical_path(self.h, int(path)))

    def last_metrics(self):
        m = Metrics()
        _check(self.lib.ghip_net_last_metrics(self.h, C.byref(m)))
        return m

    def forward(self, X):
        X = np.ascontiguousarray(X, np.float32)
        out = np.empty((X.shape[0], self.sizes[-1]), np.float32)
        _check(self.lib.ghip_net_forward(self.h, _ptr(X), X.shape[0], _ptr(out)))
        return out

    def forward_resident(self, row0, batch, out_ptr=None):
        _check(self.lib.ghip_net_forward_resident(self.h, row0, batch, C.c_void_p(out_ptr) if out_ptr else None))

    def eval_resident(self, row0, batch):
        m = Metrics()
        _check(self.lib.ghip_net_eval_resident(self.h, row0, batch, C.byref(m)))
        return m

    def quantize_fp8(self, want=True):
        if not want:
            _check(self.lib.ghip_net_quantize_fp8(self.h, None, None))
            return None, None
        scales = [np.empty((self.sizes[l + 1],), np.float32) for l in range(self.nl)]
        codes = [np.empty((self.sizes[l + 1], self.sizes[l]), np.uint8) for l in range(self.nl)]
        sp = (C.c_void_p * self.nl)(*[s.ctypes.data for s in scales])
        cp = (C.c_void_p * self.nl)(*[c.ctypes.data for c in codes])
        _check(self.lib.ghip_net_quantize_fp8(self.h, C.cast(sp, C.c_void_p), C.cast(cp, C.c_void_p)))
        return codes, scales

    def set_fp8_activation_scaling(self, mode):
        _check(self.lib.ghip_net_set_fp8_activation_scaling(self.h, mode))

    def sync(self):
        _check(self.lib.ghip_net_sync(self.h))

    # ---- profiling
    def profile(self, enable=True):
        _check(self.lib.ghip_net_profile(self.h, 1 if enable else 0))

    def profile_reset(self):
        _check(self.lib.ghip_net_profile_reset(self.h))

    def profile_table(self):
        n = self.lib.ghip_net_profile_count(self.h)
        out = {}
        for k in range(n):
            name = C.create_string_buffer(96)
            ms = C.c_double()
            cnt = C.c_int64()
            _check(self.lib.ghip_net_profile_entry(self.h, k, name, 96, C.byref(ms), C.byref(cnt)))
            out[name.value.decode()] = (ms.value, cnt.value)
        return out


def run_epochs_exact_multi(nets, n_epochs, train=True, stop_accuracy=0.0):
    """One launch for several exact-mode networks of one specification.  Returns per network the list
    of (loss, accuracy, correct) per epoch run."""
    lib = load()
    k = len(nets)
    handles = (C.c_void_p * k)(*[n.h for n in nets])
    ms = np.zeros((k, n_epochs), dtype=METRICS_DTYPE)
    ran = np.zeros(k, dtype=np.int32)
    _check(lib.ghip_net_run_epochs_exact_multi(C.cast(handles, C.c_void_p), k, n_epochs, 1 if train else 0, float(stop_accuracy),
                                               _ptr(ms), _ptr(ran)))
    return [ms[j, :ran[j]].tolist() for j in range(k)]
