"""Writes the golden fixtures in this directory.

Runs ONLY where oracle/_ref/ref_harness exists (the build container: it is compiled from the
reference's own node/edge/layer/Terminator/gmath sources by `make -C oracle ref`).  Every
number stored here was produced by that reference code; the inputs are seeded numpy draws,
the reference's unit-test data (xor gate table, iris measurements) and its NNInfo fixture
hyper-parameters (xornet: 2-2-1 TANH lr .003 mb 1 REGRESSION; iris: 4-5-3 SIGMOID lr .01
mb 1 CLASSIFICATION).

    python tests/golden/make_golden.py            # everything
    python tests/golden/make_golden.py full       # only the full-schedule runs (about 5 minutes)
    python tests/golden/make_golden.py init       # only the whole-network initialisations
"""
import os
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import pyoracle as po  # noqa: E402

# (name, sizes, acts, cost, N, mb, epochs, lr, mom, wd1, wd2, act_params, seed, kind)
CASES = [
    ("one_sample_2_3_2", [2, 3, 2], [po.TANH, po.TANH], po.REGRESSION, 1, 1, 1, 0.1, 0, 0, 0, 0, 1, "rand"),
    ("window_4_5_3_1", [4, 5, 3, 1], [po.TANH] * 3, po.REGRESSION, 11, 3, 4, 0.05, 0.5, 0, 0, 0, 2, "rand"),
    ("decay_3_4_2", [3, 4, 2], [po.SIGMOID] * 2, po.CLASSIFICATION, 10, 4, 3, 0.05, 0.9, 0.01, 0.01, 0, 3, "rand"),
    ("cfg1_shape_4_16_3", [4, 16, 3], [po.SIGMOID] * 2, po.CLASSIFICATION, 150, 150, 25, 0.01, 0.9, 0, 0, 0, 4, "rand"),
    ("cfg2_shape_32_64_64_1", [32, 64, 64, 1], [po.TANH, po.TANH, po.LINEAR], po.REGRESSION, 300, 256, 2,
     0.01, 0.9, 0, 0, [0, 0, 1.0], 5, "rand"),
    ("mixed_5_7_6_4", [5, 7, 6, 4], [po.RELU, po.LEAKY, po.SIGMOIDP], po.CLASSIFICATION, 23, 5, 3, 0.01, 0.3,
     0.001, 0.002, [0, 0.05, 0.1], 6, "rand"),
    ("kl_3_5_4_2", [3, 5, 4, 2], [po.TANHP, po.STEP, po.LINEAR], po.KL, 9, 2, 2, 0.01, 0.2, 0, 0,
     [0.1, 0.2, 0.5], 7, "rand"),
    ("xornet", [2, 2, 1], [po.TANH, po.TANH], po.REGRESSION, 4, 1, 200, 0.003, 0, 0, 0, 0, 11, "xor"),
    ("iris", [4, 5, 3], [po.SIGMOID, po.SIGMOID], po.CLASSIFICATION, 150, 1, 30, 0.01, 0, 0, 0, 0, 12, "iris"),
]

# dropout runs: (name, sizes, acts, cost, N, mb, epochs, lr, mom, wd1, wd2, act_params, seed, p per non-output layer)
# The reference's error accumulators are not cleared for rows whose last input node is dropped
# (network.cpp:621-631), so wide upper layers overflow within a few rows: the cases keep the upper
# layers narrow and the numbers finite (if wild), which is the harsher bit-for-bit test.
DROPOUT_CASES = [
    ("window_4_5_3_1", [4, 5, 3, 1], [po.TANH] * 3, po.REGRESSION, 11, 3, 4, 0.05, 0.5, 0, 0, 0, 2, [0.2, 0.5, 0.3]),
    ("decay_3_4_2", [3, 4, 2], [po.SIGMOID] * 2, po.CLASSIFICATION, 10, 4, 3, 0.05, 0.9, 0.01, 0.01, 0, 3, [0.0, 0.5]),
    ("out_of_range_6_8_2", [6, 8, 2], [po.TANH, po.TANH], po.REGRESSION, 40, 7, 5, 0.02, 0.8, 0, 0, 0, 9, [-0.5, 1.0]),
    ("heavy_6_8_2", [6, 8, 2], [po.TANH, po.TANH], po.REGRESSION, 40, 7, 5, 0.02, 0.8, 0, 0, 0, 9, [0.5, 0.9]),
    ("batch1_5_7_6_4", [5, 7, 6, 4], [po.TANH, po.SIGMOID, po.SIGMOID], po.CLASSIFICATION, 23, 1, 3, 0.001, 0.3,
     0.001, 0.002, 0, 6, [0.1, 0.25, 0.4]),
    ("deep_64_48_6_2", [64, 48, 6, 2], [po.TANH, po.TANH, po.SIGMOID], po.CLASSIFICATION, 40, 8, 3, 0.001, 0.5, 0, 0, 0,
     8, [0.3, 0.3, 0.2]),
    ("wide_1100_12_2", [1100, 12, 2], [po.RELU, po.LINEAR], po.REGRESSION, 12, 4, 2, 0.0005, 0.5, 0, 0, [0, 1.0], 8,
     [0.5, 0.25]),
]

# The two CPU-sized benchmark configurations on their own data and over their whole schedule:
# (name, sizes, acts, cost, mb, epochs, lr, mom, act_params, seed, data)
FULL_CASES = [
    # 150 rows from 3 Gaussian clusters, 4-16-3 sigmoid, BCE, full batch (mb = N), 500 epochs.  lr 0.01
    # trains; lr 0.1 (the configuration as written) turns to NaN in the reference within the first
    # epochs, and the NaNs have to sit in the same places
    ("cfg1_full_lr001", [4, 16, 3], [po.SIGMOID] * 2, po.CLASSIFICATION, 150, 500, 0.01, 0.9, 0, 101, "clusters"),
    ("cfg1_full_lr01", [4, 16, 3], [po.SIGMOID] * 2, po.CLASSIFICATION, 150, 500, 0.1, 0.9, 0, 101, "clusters"),
    # 10 000 windows of 32 lagged values of a sum of three sines plus noise, 32-64-64-1 tanh / tanh /
    # linear, MSE, mb 256, 50 epochs = 500 000 rows through the reference's objects
    ("cfg2_full", [32, 64, 64, 1], [po.TANH, po.TANH, po.LINEAR], po.REGRESSION, 256, 50, 0.01, 0.9, [0, 0, 1.0], 102, "sines"),
]

IRIS = os.path.join(HERE, "iris_measurements.csv")


def scale_classification_columns(feats):
    """NumberInput.cpp:68-212 on a classification table: min/max start from 0 for every column but
    the first; x -> (x-min)/range*0.98+0.01."""
    X = np.empty_like(feats)
    for c in range(feats.shape[1]):
        col = feats[:, c]
        fmin = np.float32(min(col.min(), col[0] if c == 0 else np.float32(0)))
        fmax = np.float32(max(col.max(), col[0] if c == 0 else np.float32(0)))
        X[:, c] = ((col - fmin) / np.float32(fmax - fmin)) * np.float32(0.98) + np.float32(0.01)
    return X


def cluster_table(seed, n_rows=150, n_feat=4, n_cls=3, sigma=0.5):
    """Rows from n_cls isotropic Gaussian clusters (centres uniform in [0,8]^n_feat), classes
    interleaved, scaled and labelled (0.99 / 0.01) the way the reference's CSV path would."""
    rng = np.random.default_rng(seed)
    centres = rng.uniform(0.0, 8.0, (n_cls, n_feat))
    cls = np.arange(n_rows) % n_cls
    feats = (centres[cls] + sigma * rng.standard_normal((n_rows, n_feat))).astype(np.float32)
    Y = np.where(np.eye(n_cls)[cls] > 0, np.float32(0.99), np.float32(0.01)).astype(np.float32)
    return scale_classification_columns(feats), Y


def sine_series(seed, n_rows=10000, lags=32):
    """n_rows + lags values of a sum of three sines (random frequency and phase) plus N(0, 0.05)
    noise, scaled to [0, 1]: row i of the table is series[i : i+lags], its target series[i+lags]."""
    rng = np.random.default_rng(seed)
    t = np.arange(n_rows + lags, dtype=np.float64)
    f = rng.uniform(0.005, 0.05, 3)
    ph = rng.uniform(0.0, 2 * np.pi, 3)
    v = sum(np.sin(2 * np.pi * f[k] * t + ph[k]) for k in range(3)) + 0.05 * rng.standard_normal(t.size)
    v = (v - v.min()) / (v.max() - v.min())
    return v.astype(np.float32)


def windows(series, lags=32):
    n = series.size - lags
    X = np.lib.stride_tricks.sliding_window_view(series, lags)[:n].copy()
    return X, series[lags:].reshape(n, 1).copy()


# Whole-network initialisations: (name, seed, n_feat, hidden sizes, acts as NNInfo::getActivationType(i)
# returns them for i = 0 .. H-1 (the input row, then the hidden rows but the last), n_out, output type)
INIT_CASES = [
    ("plain_tanh", 21, 4, [5, 3], [po.TANH, po.TANH], 2, po.REGRESSION),             # no restart
    ("restart_row0", 22, 4, [5], [po.SIGMOID], 3, po.CLASSIFICATION),                 # restart at row 0: nothing thrown away
    ("restart_row1_wider", 23, 3, [6, 4], [po.TANH, po.SIGMOID], 2, po.REGRESSION),   # row 1: layer 0 again, with fan-in 6
    ("restart_row2_equal", 24, 5, [3, 5, 4], [po.TANH, po.TANH, po.RELU], 2, po.REGRESSION),   # row 2: layer 0 with fan-in 5 = features
]


def init_call_sequence(n_feat, hidden, acts, n_out, out_type):
    """The Layer::initWeights calls of LayerBuilder::buildHiddenLayers + buildOutputLayer
    (LayerBuilder.cpp:192-265) in order: (fan_in, n_out, act, kept layer index or -1).  A restart
    (the first row whose activation is SIGMOID / RELU / LEAKY, any row for CLASSIFICATION) throws away
    what was built and starts over without resetting prevLayerSize."""
    calls, positive, prev, i = [], False, n_feat, 0
    while i < len(hidden):
        at = acts[i]
        if not positive and (at in (po.SIGMOID, po.RELU, po.LEAKY) or out_type == po.CLASSIFICATION):
            positive = True
            calls = [(f, n, a, -1) for (f, n, a, _) in calls]
            i = 0
            continue
        calls.append((prev, hidden[i], at, i))
        prev = hidden[i]
        i += 1
    last = hidden[-1] if hidden else n_feat
    calls.append((last, n_out, acts[len(hidden) - 1] if hidden else acts[0], len(hidden)))
    return calls


def init_sequences(td):
    d = {}
    for (name, seed, n_feat, hidden, acts, n_out, out_type) in INIT_CASES:
        calls = init_call_sequence(n_feat, hidden, acts, n_out, out_type)
        out = os.path.join(td, "seq.bin")
        args = [str(v) for c in calls for v in c[:3]]
        subprocess.check_call([po.REF_HARNESS, "xavierseq", str(seed), out] + args)
        raw = np.fromfile(out, np.float32)
        pos = 0
        sizes = [n_feat] + hidden + [n_out]
        for (fan, n, a, keep) in calls:
            w = raw[pos:pos + fan * n].reshape(n, fan)
            pos += fan * n
            if keep >= 0:
                assert fan >= sizes[keep]
                d[f"{name}_W{keep}"] = w[:, :sizes[keep]].copy()   # surplus edges exist in the reference but are never visited
        d[f"{name}_next"] = raw[pos:pos + 1].copy()
        d[f"{name}_spec"] = np.array([seed, n_feat, n_out, out_type, len(hidden)] + hidden + acts, np.int32)
        print("init", name, "calls", [(c[0], c[1], c[3]) for c in calls])
    np.savez_compressed(os.path.join(HERE, "init_sequences.npz"), **d)


def full_schedule_runs(td):
    for (name, sizes, acts, cost, mb, epochs, lr, mom, params, seed, data) in FULL_CASES:
        nl = len(sizes) - 1
        spec = po.make_spec(sizes, acts, lr=lr, mom=mom, act_params=params, batch=mb, cost=cost)
        # the reference's own sampler (Layer::initWeights, layer.cpp:196-217) under srand(seed + layer)
        Ws = [ref_xavier(seed + l, sizes[l], sizes[l + 1], acts[max(l - 1, 0)] if l == nl - 1 else acts[l], td)
              for l in range(nl)]
        bs = [0.0] * nl
        extra = {}
        if data == "clusters":
            X, Y = cluster_table(seed)
            extra = dict(X=X, Y=Y)
        else:
            series = sine_series(seed)
            X, Y = windows(series)
            extra = dict(series=series)        # the table is rebuilt from it (40 KB instead of 1.3 MB)
        ref = po.ref_train(spec, Ws, bs, X, Y, epochs, td)
        d = dict(sizes=np.array(sizes, np.int32), acts=np.array(acts, np.int32),
                 hyper=np.array([lr, mom, 0, 0], np.float32),
                 act_params=np.array(params if isinstance(params, list) else [params] * nl, np.float32),
                 ints=np.array([cost, X.shape[0], mb, epochs], np.int32),
                 bias0=np.array(bs, np.float32), epochs=ref["epochs"], bias=ref["bias"], preds=ref["preds"], **extra)
        for l in range(nl):
            d[f"W0_{l}"] = Ws[l]
            d[f"W_{l}"] = ref["W"][l]
            d[f"wsum_{l}"] = ref["wsum"][l]
            d[f"wlast_{l}"] = ref["wlast"][l]
        np.savez_compressed(os.path.join(HERE, f"train_{name}.npz"), **d)
        ep = ref["epochs"]
        print(name, "epochs", epochs, "first", ep[0], "last", ep[-1], "non-finite epochs", int((~np.isfinite(ep[:, 0])).sum()),
              "max|W0|", float(np.nanmax(np.abs(ref["W"][0]))), flush=True)


def ref_xavier(seed, fan_in, n_out, act, td):
    out = os.path.join(td, "xav.bin")
    subprocess.check_call([po.REF_HARNESS, "xavier", str(seed), str(fan_in), str(n_out), str(act), out])
    return np.fromfile(out, np.float32).reshape(n_out, fan_in)


def iris_tables():
    """Measurements scaled the way NumberInput.cpp:68-212 scales a classification table
    (min/max start from 0 for every column but the first; x -> (x-min)/range*0.98+0.01) and
    labels one-hot at 0.99/0.01 in order of first appearance (OHE.cpp:159-198)."""
    rows = [ln.strip().split(",") for ln in open(IRIS) if ln.strip()]
    feats = np.array([[np.float32(v) for v in r[:4]] for r in rows], np.float32)
    names = []
    for r in rows:
        if r[4] not in names:
            names.append(r[4])
    X = np.empty_like(feats)
    for c in range(4):
        col = feats[:, c]
        fmin = np.float32(min(col.min(), col[0] if c == 0 else np.float32(0)))
        fmax = np.float32(max(col.max(), col[0] if c == 0 else np.float32(0)))
        rng = np.float32(fmax - fmin)
        X[:, c] = ((col - fmin) / rng) * np.float32(0.98) + np.float32(0.01)
    Y = np.full((len(rows), 3), 0.01, np.float32)
    for i, r in enumerate(rows):
        Y[i, names.index(r[4])] = 0.99
    return X, Y


def main():
    if not po.have_ref():
        raise SystemExit("oracle/_ref/ref_harness missing: run `make -C oracle ref` where /root/reference exists")
    with tempfile.TemporaryDirectory() as td:
        if sys.argv[1:] == ["init"]:
            return init_sequences(td)
        init_sequences(td)
        full_schedule_runs(td)
        if sys.argv[1:] == ["full"]:
            return
        # element-wise grid
        g = os.path.join(td, "g.bin")
        subprocess.check_call([po.REF_HARNESS, "gmath", g])
        raw = open(g, "rb").read()
        nz, npar = np.frombuffer(raw[:8], np.int32)
        body = np.frombuffer(raw[8:], np.float32)
        n_act = 8 * npar * nz * 3
        np.savez_compressed(os.path.join(HERE, "gmath_grid.npz"), nz=nz, npar=npar,
                            act=body[:n_act].reshape(8, npar, nz, 3), cost=body[n_act:].reshape(3, 6, -1, 5))
        # Terminator truth table
        t = os.path.join(td, "t.bin")
        subprocess.check_call([po.REF_HARNESS, "term", t])
        np.savez_compressed(os.path.join(HERE, "terminator_table.npz"),
                            rec=np.fromfile(t, np.int32).reshape(-1, 7))
        # sampler
        xav = {}
        for seed, fi, no, act in [(1, 4, 5, po.SIGMOID), (7, 2, 2, po.TANH), (42, 16, 3, po.RELU), (3, 64, 8, po.TANH)]:
            xav[f"s{seed}_{fi}_{no}_{act}"] = ref_xavier(seed, fi, no, act, td)
        np.savez_compressed(os.path.join(HERE, "xavier_samples.npz"), **xav)
        # training runs
        for (name, sizes, acts, cost, N, mb, epochs, lr, mom, wd1, wd2, params, seed, kind) in CASES:
            rng = np.random.default_rng(seed)
            nl = len(sizes) - 1
            spec = po.make_spec(sizes, acts, lr=lr, mom=mom, wd1=wd1, wd2=wd2, act_params=params, batch=mb, cost=cost)
            if kind == "rand":
                Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * 0.5).astype(np.float32) for l in range(nl)]
                bs = [0.0] + [float(np.float32(rng.standard_normal() * 0.1)) for _ in range(nl - 1)]
                X = rng.random((N, sizes[0])).astype(np.float32)
                if cost == po.CLASSIFICATION:
                    Y = (np.eye(sizes[-1], dtype=np.float32)[rng.integers(0, sizes[-1], N)] * 0.98 + 0.01).astype(np.float32)
                else:
                    Y = rng.random((N, sizes[-1])).astype(np.float32)
            else:
                Ws = [ref_xavier(seed + l, sizes[l], sizes[l + 1], acts[max(l - 1, 0)] if l == nl - 1 else acts[l], td)
                      for l in range(nl)]
                bs = [0.0] * nl
                if kind == "xor":
                    X = np.array([[0, 0], [0, 1], [1, 0], [1, 1]], np.float32)
                    Y = np.array([[0], [1], [1], [0]], np.float32)
                else:
                    X, Y = iris_tables()
            ref = po.ref_train(spec, Ws, bs, X, Y, epochs, td)
            d = dict(sizes=np.array(sizes, np.int32), acts=np.array(acts, np.int32),
                     hyper=np.array([lr, mom, wd1, wd2], np.float32),
                     act_params=np.array(params if isinstance(params, list) else [params] * nl, np.float32),
                     ints=np.array([cost, N, mb, epochs], np.int32), X=X, Y=Y,
                     bias0=np.array(bs, np.float32), epochs=ref["epochs"], bias=ref["bias"], preds=ref["preds"])
            for l in range(nl):
                d[f"W0_{l}"] = Ws[l]
                d[f"W_{l}"] = ref["W"][l]
                d[f"wsum_{l}"] = ref["wsum"][l]
                d[f"wlast_{l}"] = ref["wlast"][l]
            np.savez_compressed(os.path.join(HERE, f"train_{name}.npz"), **d)
            print(name, "epochs", epochs, "last", ref["epochs"][-1])
        # dropout runs: the flags come from the reference's compiled Layer::generateDropout under srand(seed)
        for (name, sizes, acts, cost, N, mb, epochs, lr, mom, wd1, wd2, params, seed, pd) in DROPOUT_CASES:
            rng = np.random.default_rng(seed)
            nl = len(sizes) - 1
            spec = po.make_spec(sizes, acts, lr=lr, mom=mom, wd1=wd1, wd2=wd2, act_params=params, batch=mb, cost=cost)
            Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * 0.5).astype(np.float32) for l in range(nl)]
            bs = [0.0] + [float(np.float32(rng.standard_normal() * 0.1)) for _ in range(nl - 1)]
            X = rng.random((N, sizes[0])).astype(np.float32)
            Y = rng.random((N, sizes[-1])).astype(np.float32)
            ref = po.ref_train(spec, Ws, bs, X, Y, epochs, td, dropout=(seed, pd))
            assert all(np.isfinite(w).all() for w in ref["W"]), name
            d = dict(sizes=np.array(sizes, np.int32), acts=np.array(acts, np.int32),
                     hyper=np.array([lr, mom, wd1, wd2], np.float32),
                     act_params=np.array(params if isinstance(params, list) else [params] * nl, np.float32),
                     ints=np.array([cost, N, mb, epochs], np.int32), X=X, Y=Y, seed=np.int32(seed),
                     p=np.array(pd, np.float32), masks=ref["masks"], rand_after=np.int32(ref["rand_after"]),
                     bias0=np.array(bs, np.float32), epochs=ref["epochs"], bias=ref["bias"], preds=ref["preds"])
            for l in range(nl):
                d[f"W0_{l}"] = Ws[l]
                d[f"W_{l}"] = ref["W"][l]
                d[f"wsum_{l}"] = ref["wsum"][l]
                d[f"wlast_{l}"] = ref["wlast"][l]
                d[f"wcnt_{l}"] = ref["wcnt"][l]
            for l in range(1, nl):
                d[f"errder_{l}"] = ref["errder"][l - 1]
            np.savez_compressed(os.path.join(HERE, f"dropout_{name}.npz"), **d)
            print("dropout", name, "dropped %.2f" % ref["masks"].mean(), "last", ref["epochs"][-1])


if __name__ == "__main__":
    main()
