"""ctypes view of oracle/libglades_oracle.so (the CPU restatement).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the CPU-baseline
leg of bench.py -- never by the product package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libglades_oracle.so")
REF_HARNESS = os.path.join(HERE, "_ref", "ref_harness")
MAX_LAYERS = 16

TANH, TANHP, SIGMOID, SIGMOIDP, LINEAR, RELU, LEAKY, STEP, SOFTMAX = range(9)
REGRESSION, CLASSIFICATION, KL = range(3)


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
    ]


class Metrics(C.Structure):
    _fields_ = [("loss", C.c_float), ("accuracy", C.c_float), ("correct", C.c_int64)]


def build(force=False):
    """Compile the C restatement (and the reference harness when the reference tree exists)."""
    if force or not os.path.exists(LIB_PATH):
        subprocess.check_call(["make", "-C", HERE, "-B", "libglades_oracle.so"])
    if os.path.isdir("/root/reference") and (force or not os.path.exists(REF_HARNESS)):
        subprocess.check_call(["make", "-C", HERE, "-B", "ref"])


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
        u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
        i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
        vp = C.c_void_p
        sig = {
            "go_squash": (C.c_float, [C.c_float, C.c_int, C.c_float]),
            "go_act_der": (C.c_float, [C.c_float, C.c_int, C.c_float]),
            "go_cost": (C.c_float, [C.c_float, C.c_float, C.c_float, C.c_int]),
            "go_cost_der": (C.c_float, [C.c_float, C.c_float, C.c_int]),
            "go_percent_error": (C.c_float, [C.c_float, C.c_float]),
            "go_argmax_ref": (C.c_int, [f32p, C.c_int]),
            "go_eval": (None, [C.c_int, C.c_int, C.c_float, f32p, vp, f32p, C.c_int64]),
            "go_cmatrix_add": (None, [C.c_int, i32p, f32p, f32p]),
            "go_cmatrix_params": (None, [C.c_int, i32p, i32p, i32p, i32p, i32p]),
            "go_cmatrix_overall": (None, [C.c_int, i32p, i32p, i32p, i32p, f32p]),
            "go_ref_xavier_layer": (None, [C.c_int, C.c_int, C.c_int, f32p]),
            "go_exact_create": (vp, [C.POINTER(Spec)]),
            "go_exact_destroy": (None, [vp]),
            "go_exact_set_weights": (None, [vp, C.c_int, f32p]),
            "go_exact_get_weights": (None, [vp, C.c_int, f32p]),
            "go_exact_set_bias": (None, [vp, C.c_int, C.c_float]),
            "go_exact_get_bias": (C.c_float, [vp, C.c_int]),
            "go_exact_get_window": (None, [vp, C.c_int, f32p, f32p]),
            "go_exact_epoch": (None, [vp, f32p, f32p, C.c_int64, C.c_int, C.POINTER(Metrics), vp]),
            "go_exact_mask_len": (C.c_int, [vp]),
            "go_exact_set_dropout": (None, [vp, vp]),
            "go_dropout_draw": (None, [C.POINTER(Spec), f32p, C.c_int64, u8p]),
            "go_exact_get_pending": (None, [vp, C.c_int, i32p]),
            "go_exact_get_errder": (None, [vp, C.c_int, f32p]),
            "srand": (None, [C.c_uint]),
            "rand": (C.c_int, []),
            "go_canon_create": (vp, [C.POINTER(Spec)]),
            "go_canon_destroy": (None, [vp]),
            "go_canon_set_params": (None, [vp, C.c_int, f32p, vp]),
            "go_canon_get_params": (None, [vp, C.c_int, vp, vp]),
            "go_canon_get_momentum": (None, [vp, C.c_int, vp, vp]),
            "go_canon_get_grads": (None, [vp, C.c_int, vp, vp]),
            "go_canon_forward": (None, [vp, f32p, C.c_int64, f32p]),
            "go_canon_step": (None, [vp, f32p, f32p, C.c_int64, C.POINTER(Metrics)]),
            "go_canon_loss": (C.c_double, [vp, f32p, f32p, C.c_int64]),
            "go_canon_set_drop": (None, [vp, vp]),
            "go_set_threads": (None, [C.c_int]),
            "go_set_sum_order": (None, [C.c_int]),
            "go_bf16_from_f32": (C.c_uint16, [C.c_float]),
            "go_bf16_to_f32": (C.c_float, [C.c_uint16]),
            "go_e4m3_from_f32": (C.c_uint8, [C.c_float]),
            "go_e4m3_to_f32": (C.c_float, [C.c_uint8]),
            "go_e4m3_quant_rows": (None, [f32p, C.c_int64, C.c_int64, u8p, f32p]),
            "go_fp8_forward": (None, [C.POINTER(Spec), C.POINTER(vp), C.POINTER(vp), f32p, C.c_int64, f32p]),
            "go_e4m3_quant_rows_block32": (None, [f32p, C.c_int64, C.c_int64, u8p, u8p]),
            "go_fp8_forward_block32": (None, [C.POINTER(Spec), C.POINTER(vp), C.POINTER(vp), f32p, C.c_int64, f32p]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def make_spec(sizes, acts, lr=0.01, mom=0.0, wd1=0.0, wd2=0.0, act_params=0.0, batch=1,
              cost=REGRESSION):
    """sizes: n_layers+1 ints; the per-layer arguments are scalars or lists of n_layers."""
    nl = len(sizes) - 1
    assert 1 <= nl <= MAX_LAYERS

    def per(v):
        return list(v) if isinstance(v, (list, tuple, np.ndarray)) else [v] * nl

    s = Spec()
    s.n_layers = nl
    for i, v in enumerate(sizes):
        s.sizes[i] = int(v)
    for name, v in (("lr", lr), ("mom", mom), ("wd1", wd1), ("wd2", wd2), ("act_param", act_params)):
        arr = getattr(s, name)
        for i, x in enumerate(per(v)):
            arr[i] = float(x)
    for i, a in enumerate(per(acts)):
        s.act[i] = int(a)
    s.batch = int(batch)
    s.cost = int(cost)
    return s


def _vp(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


class ExactNet:
    """Reference semantics: sequential rows, scalar layer bias, delta windows."""

    def __init__(self, spec):
        self.spec = spec
        self.sizes = [spec.sizes[i] for i in range(spec.n_layers + 1)]
        self.h = lib().go_exact_create(C.byref(spec))

    def __del__(self):
        if getattr(self, "h", None):
            lib().go_exact_destroy(self.h)
            self.h = None

    def set_weights(self, l, W):
        W = np.ascontiguousarray(W, np.float32)
        assert W.shape == (self.sizes[l + 1], self.sizes[l])
        lib().go_exact_set_weights(self.h, l, W)

    def get_weights(self, l):
        W = np.empty((self.sizes[l + 1], self.sizes[l]), np.float32)
        lib().go_exact_get_weights(self.h, l, W)
        return W

    def set_bias(self, l, b):
        lib().go_exact_set_bias(self.h, l, float(b))

    def get_bias(self, l):
        return np.float32(lib().go_exact_get_bias(self.h, l))

    def get_window(self, l):
        s = np.empty((self.sizes[l + 1], self.sizes[l]), np.float32)
        t = np.empty_like(s)
        lib().go_exact_get_window(self.h, l, s, t)
        return s, t

    def get_pending(self, l):
        c = np.empty((self.sizes[l + 1], self.sizes[l]), np.int32)
        lib().go_exact_get_pending(self.h, l, c)
        return c

    def get_errder(self, layer):
        e = np.empty(self.sizes[layer], np.float32)
        lib().go_exact_get_errder(self.h, layer, e)
        return e

    def epoch(self, X, Y, train=True, want_preds=True, masks=None):
        """masks: N x sum(sizes[:-1]) uint8 dropout flags of this epoch (1 = dropped) or None."""
        X = np.ascontiguousarray(X, np.float32)
        Y = np.ascontiguousarray(Y, np.float32)
        N = X.shape[0]
        assert X.shape == (N, self.sizes[0]) and Y.shape == (N, self.sizes[-1])
        if masks is not None:
            masks = np.ascontiguousarray(masks, np.uint8)
            assert masks.shape == (N, sum(self.sizes[:-1]))
        lib().go_exact_set_dropout(self.h, _vp(masks))
        preds = np.empty((N, self.sizes[-1]), np.float32) if want_preds else None
        m = Metrics()
        lib().go_exact_epoch(self.h, X, Y, N, 1 if train else 0, C.byref(m), _vp(preds))
        return m, preds


class CanonNet:
    """Batched textbook training; forward identical to the reference forward."""

    def __init__(self, spec):
        self.spec = spec
        self.sizes = [spec.sizes[i] for i in range(spec.n_layers + 1)]
        self.h = lib().go_canon_create(C.byref(spec))

    def __del__(self):
        if getattr(self, "h", None):
            lib().go_canon_destroy(self.h)
            self.h = None

    def set_params(self, l, W, b=None):
        W = np.ascontiguousarray(W, np.float32)
        assert W.shape == (self.sizes[l + 1], self.sizes[l])
        if b is not None:
            b = np.ascontiguousarray(b, np.float32)
            assert b.shape == (self.sizes[l + 1],)
        lib().go_canon_set_params(self.h, l, W, _vp(b))

    def _pair(self, fn, l):
        W = np.empty((self.sizes[l + 1], self.sizes[l]), np.float32)
        b = np.empty((self.sizes[l + 1],), np.float32)
        fn(self.h, l, _vp(W), _vp(b))
        return W, b

    def get_params(self, l):
        return self._pair(lib().go_canon_get_params, l)

    def get_momentum(self, l):
        return self._pair(lib().go_canon_get_momentum, l)

    def get_grads(self, l):
        return self._pair(lib().go_canon_get_grads, l)

    def _drop(self, drop, B):
        """dropout flags [B][sum of sizes[:-1]] (1 = dropped) for the call that follows, or None"""
        if drop is None:
            lib().go_canon_set_drop(self.h, None)
            return None
        drop = np.ascontiguousarray(drop, np.uint8)
        assert drop.shape == (B, sum(self.sizes[:-1]))
        lib().go_canon_set_drop(self.h, drop.ctypes.data_as(C.c_void_p))
        return drop

    def forward(self, X, drop=None):
        X = np.ascontiguousarray(X, np.float32)
        out = np.empty((X.shape[0], self.sizes[-1]), np.float32)
        keep = self._drop(drop, X.shape[0])
        lib().go_canon_forward(self.h, X, X.shape[0], out)
        lib().go_canon_set_drop(self.h, None)
        del keep
        return out

    def step(self, X, Y, drop=None):
        X = np.ascontiguousarray(X, np.float32)
        Y = np.ascontiguousarray(Y, np.float32)
        m = Metrics()
        keep = self._drop(drop, X.shape[0])
        lib().go_canon_step(self.h, X, Y, X.shape[0], C.byref(m))
        lib().go_canon_set_drop(self.h, None)
        del keep
        return m

    def loss(self, X, Y):
        X = np.ascontiguousarray(X, np.float32)
        Y = np.ascontiguousarray(Y, np.float32)
        return lib().go_canon_loss(self.h, X, Y, X.shape[0])


def bf16_round(x):
    """fp32 array -> fp32 array holding the bf16-rounded values (RNE)."""
    x = np.ascontiguousarray(x, np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return r.astype(np.uint32).view(np.float32).reshape(x.shape)


def e4m3_quant_rows(x):
    x = np.ascontiguousarray(x, np.float32)
    q = np.empty(x.shape, np.uint8)
    s = np.empty((x.shape[0],), np.float32)
    lib().go_e4m3_quant_rows(x, x.shape[0], x.shape[1], q, s)
    return q, s


def e4m3_table():
    return np.array([lib().go_e4m3_to_f32(i) for i in range(256)], np.float32)


def e4m3_quant_rows_block32(x):
    """Block-scaled quantiser: (codes [rows][cols], E8M0 bytes [rows][ceil(cols / 32)])."""
    x = np.ascontiguousarray(x, np.float32)
    q = np.empty(x.shape, np.uint8)
    s = np.empty((x.shape[0], (x.shape[1] + 31) // 32), np.uint8)
    lib().go_e4m3_quant_rows_block32(x, x.shape[0], x.shape[1], q, s)
    return q, s


def fp8_forward(spec, Wq, wscale, X, block32=False):
    nl = spec.n_layers
    X = np.ascontiguousarray(X, np.float32)
    Wq = [np.ascontiguousarray(w, np.uint8) for w in Wq]
    wscale = [np.ascontiguousarray(s, np.float32) for s in wscale]
    wp = (C.c_void_p * nl)(*[w.ctypes.data for w in Wq])
    sp = (C.c_void_p * nl)(*[s.ctypes.data for s in wscale])
    out = np.empty((X.shape[0], spec.sizes[nl]), np.float32)
    (lib().go_fp8_forward_block32 if block32 else lib().go_fp8_forward)(C.byref(spec), wp, sp, X, X.shape[0], out)
    return out


# ---------------------------------------------------------------- reference harness


def have_ref():
    return os.path.exists(REF_HARNESS)


def gmath_eval(fn, kind, a, b=None, param=0.0):
    """fn 0 squash, 1 act_der, 2 cost(expected a, predicted b, data_size param), 3 cost_der, per element."""
    a = np.ascontiguousarray(a, np.float32)
    b = None if b is None else np.ascontiguousarray(b, np.float32)
    out = np.empty_like(a)
    lib().go_eval(int(fn), int(kind), float(param), a, _vp(b), out, a.size)
    return out


def libc_srand(seed):
    """Seeds the libc rand() stream that go_dropout_draw and go_ref_xavier_layer consume."""
    lib().srand(int(seed))


def libc_rand():
    return lib().rand()


def dropout_draw(spec, p, N):
    """One epoch's dropout flags drawn from libc rand() in the reference's order: N x sum(sizes[:-1])."""
    nl = spec.n_layers
    p = np.ascontiguousarray(p, np.float32)
    assert p.shape == (nl,)
    m = np.zeros((N, sum(spec.sizes[i] for i in range(nl))), np.uint8)
    lib().go_dropout_draw(C.byref(spec), p, N, m)
    return m


def ref_train(spec, weights, biases, X, Y, epochs, tmpdir, dropout=None):
    """Run the harness built from the reference's compiled objects.  Returns a dict with
    per-epoch (loss, accuracy), final weights, biases, last-epoch predictions and windows.
    dropout = (seed, [p per non-output layer]) also returns the flags the reference drew
    ("masks": epochs x N x sum(sizes[:-1])), the window lengths ("wcnt"), the hidden nodes'
    error accumulators ("errder") and the next rand() % 65536 ("rand_after")."""
    nl = spec.n_layers
    sizes = [spec.sizes[i] for i in range(nl + 1)]
    X = np.ascontiguousarray(X, np.float32)
    Y = np.ascontiguousarray(Y, np.float32)
    N = X.shape[0]
    cin = os.path.join(tmpdir, "case.bin")
    cout = os.path.join(tmpdir, "out.bin")
    with open(cin, "wb") as f:
        f.write(np.array([0x474C4144, nl] + sizes + [spec.batch, spec.cost, N, epochs], np.int32).tobytes())
        for l in range(nl):
            f.write(np.array([spec.lr[l], spec.mom[l], spec.wd1[l], spec.wd2[l]], np.float32).tobytes())
            f.write(np.array([spec.act[l]], np.int32).tobytes())
            f.write(np.array([spec.act_param[l]], np.float32).tobytes())
        for l in range(nl):
            f.write(np.ascontiguousarray(weights[l], np.float32).tobytes())
        f.write(np.array([biases[l] for l in range(nl)], np.float32).tobytes())
        f.write(X.tobytes())
        f.write(Y.tobytes())
        if dropout is not None:
            f.write(np.array([dropout[0]], np.int32).tobytes())
            f.write(np.asarray(dropout[1], np.float32).tobytes())
    with open(os.devnull, "w") as dn:
        subprocess.check_call([REF_HARNESS, "train", cin, cout], stdout=dn)
    raw = np.fromfile(cout, np.float32)
    pos = 0
    out = {"epochs": raw[: 2 * epochs].reshape(epochs, 2).copy()}
    pos = 2 * epochs
    out["W"] = []
    for l in range(nl):
        cnt = sizes[l] * sizes[l + 1]
        out["W"].append(raw[pos : pos + cnt].reshape(sizes[l + 1], sizes[l]).copy())
        pos += cnt
    out["bias"] = raw[pos : pos + nl].copy()
    pos += nl
    out["preds"] = raw[pos : pos + N * sizes[-1]].reshape(N, sizes[-1]).copy()
    pos += N * sizes[-1]
    out["wsum"], out["wlast"] = [], []
    for l in range(nl):
        cnt = sizes[l] * sizes[l + 1]
        w = raw[pos : pos + 2 * cnt].reshape(sizes[l + 1], sizes[l], 2)
        out["wsum"].append(w[..., 0].copy())
        out["wlast"].append(w[..., 1].copy())
        pos += 2 * cnt
    if dropout is not None:
        ml = sum(sizes[:-1])
        out["masks"] = raw[pos : pos + epochs * N * ml].reshape(epochs, N, ml).astype(np.uint8)
        pos += epochs * N * ml
        out["wcnt"] = []
        for l in range(nl):
            cnt = sizes[l] * sizes[l + 1]
            out["wcnt"].append(raw[pos : pos + cnt].reshape(sizes[l + 1], sizes[l]).astype(np.int32))
            pos += cnt
        out["errder"] = []
        for l in range(1, nl):
            out["errder"].append(raw[pos : pos + sizes[l]].copy())
            pos += sizes[l]
        out["rand_after"] = int(raw[pos])
        pos += 1
    assert pos == raw.size
    return out


def cmatrix(expected, predicted):
    """Confusion matrix of the reference (row expected, column predicted) over the rows of two [N][n] arrays."""
    expected = np.ascontiguousarray(expected, np.float32)
    predicted = np.ascontiguousarray(predicted, np.float32)
    n = expected.shape[1]
    M = np.zeros((n, n), np.int32)
    for e, p in zip(expected, predicted):
        lib().go_cmatrix_add(n, M, np.ascontiguousarray(e), np.ascontiguousarray(p))
    return M


def cmatrix_metrics(M):
    """(tp, tn, fp, fn, overall[6]) of cmatrix.cpp for an n x n int32 matrix."""
    M = np.ascontiguousarray(M, np.int32)
    n = M.shape[0]
    tp, tn, fp, fn = (np.zeros(n, np.int32) for _ in range(4))
    lib().go_cmatrix_params(n, M, tp, tn, fp, fn)
    out = np.zeros(6, np.float32)
    with np.errstate(all="ignore"):
        lib().go_cmatrix_overall(n, tp, tn, fp, fn, out)
    return tp, tn, fp, fn, out
