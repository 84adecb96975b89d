"""Shared helpers for the parity tests."""
import os

import numpy as np

import pyoracle as po

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TRAIN_CASES = ["one_sample_2_3_2", "window_4_5_3_1", "decay_3_4_2", "cfg1_shape_4_16_3",
               "cfg2_shape_32_64_64_1", "mixed_5_7_6_4", "kl_3_5_4_2", "xornet", "iris"]


# the two CPU-sized benchmark configurations on their own data over their whole schedule: 500 epochs of
# 150 rows from 3 Gaussian clusters at lr 0.01 and at lr 0.1 (where the reference turns to NaN), and
# 50 epochs of 10 000 sine windows (500 000 rows), all through the reference's compiled objects
FULL_CASES = ["cfg1_full_lr001", "cfg1_full_lr01", "cfg2_full"]

DROPOUT_CASES = ["window_4_5_3_1", "decay_3_4_2", "out_of_range_6_8_2", "heavy_6_8_2", "batch1_5_7_6_4",
                 "deep_64_48_6_2", "wide_1100_12_2"]


def load_case(name, kind="train"):
    """kind "train": runs without dropout; "dropout": runs whose flags the reference's compiled
    Layer::generateDropout drew (d["masks"]: epochs x N x sum(sizes[:-1]), d["seed"], d["p"])."""
    d = np.load(os.path.join(GOLDEN, f"{kind}_{name}.npz"), allow_pickle=False)
    sizes = [int(v) for v in d["sizes"]]
    nl = len(sizes) - 1
    cost, N, mb, epochs = [int(v) for v in d["ints"]]
    lr, mom, wd1, wd2 = [float(v) for v in d["hyper"]]
    spec = po.make_spec(sizes, [int(a) for a in d["acts"]], lr=lr, mom=mom, wd1=wd1, wd2=wd2,
                        act_params=[float(v) for v in d["act_params"]], batch=mb, cost=cost)
    if "series" in d.files:   # lagged windows of one series: row i = series[i : i+lags], target series[i+lags]
        series = d["series"]
        X = np.lib.stride_tricks.sliding_window_view(series, sizes[0])[:N].copy()
        Y = series[sizes[0]:].reshape(N, 1).copy()
    else:
        X, Y = d["X"], d["Y"]
    return dict(d=d, sizes=sizes, nl=nl, cost=cost, N=N, mb=mb, epochs=epochs, spec=spec,
                W0=[d[f"W0_{l}"] for l in range(nl)], bias0=d["bias0"], X=X, Y=Y)


def bits_equal(a, b):
    """Bit equality of two fp32 arrays, NaNs compared by position."""
    a = np.ascontiguousarray(a, np.float32).ravel()
    b = np.ascontiguousarray(b, np.float32).ravel()
    if a.shape != b.shape:
        return False
    na, nb = np.isnan(a), np.isnan(b)
    if not np.array_equal(na, nb):
        return False
    return np.array_equal(a[~na].view(np.uint32), b[~nb].view(np.uint32))


def rel_err(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.max(np.abs(a - b) / (np.abs(b) + 1e-6))) if a.size else 0.0


def cluster_centres(rng, n_cls, dim):
    return rng.standard_normal((n_cls, dim), dtype=np.float32)


def cluster_rows(rng, centres, n_rows, sigma=1.0, n_out=None):
    """Rows from isotropic Gaussian clusters around `centres` (class = cluster), scaled so that every
    feature is N(0,1) overall, with one-hot labels n_out wide: classes that a trained network separates
    with a margin, so that "which class wins" is a question with an answer for every row."""
    n_cls, dim = centres.shape
    cls = rng.integers(0, n_cls, n_rows)
    X = centres[cls] + np.float32(sigma) * rng.standard_normal((n_rows, dim), dtype=np.float32)
    X *= np.float32(1.0 / np.sqrt(1.0 + sigma * sigma))
    Y = np.zeros((n_rows, n_out or n_cls), np.float32)
    Y[np.arange(n_rows), cls] = 1.0
    return X, Y, cls


def he_init(rng, sizes):
    return [rng.standard_normal((sizes[l + 1], sizes[l]), dtype=np.float32) * np.float32(np.sqrt(2.0 / sizes[l]))
            for l in range(len(sizes) - 1)]


def rel_rms(a, b):
    return float(np.sqrt(np.mean((np.asarray(a, np.float64) - b) ** 2)) / np.sqrt(np.mean(np.asarray(b, np.float64) ** 2)))


def bf16_pipeline_steps(sizes, acts, Ws, bs, X, Y, B, steps, lr, mom, wd2, wide=True):
    """numpy statement of the bf16 training pipeline: bf16 weights (rounded from the fp32 master),
    bf16 activations and deltas, products exact and summed in float64, fp32 logits/softmax,
    fp32 master + momentum update.  Hidden activations: TANH / RELU (0.046 knee) / SIGMOID;
    output: SOFTMAX with cross-entropy.  Returns final master weights, biases and losses."""
    q = po.bf16_round
    mm = np.float64 if wide else np.float32   # accumulation type of the matrix products
    Wm = [w.astype(np.float32).copy() for w in Ws]
    bm = [b.astype(np.float32).copy() for b in bs]
    vW = [np.zeros_like(w) for w in Wm]
    vb = [np.zeros_like(b) for b in bm]
    L = len(Wm)
    losses = []
    for s in range(steps):
        x, y = X[s * B:(s + 1) * B], Y[s * B:(s + 1) * B]
        Wh = [q(w) for w in Wm]
        H = [q(x)]
        for l in range(L):
            Z = (H[l].astype(mm) @ Wh[l].T.astype(mm)).astype(np.float32) + bm[l]
            if l == L - 1:
                break
            if acts[l] == po.TANH:
                A = np.tanh(Z)
            elif acts[l] == po.RELU:
                A = np.where(Z < np.float32(0.046), np.float32(0), Z)
            else:
                A = 1.0 / (1.0 + np.exp(-Z))
            H.append(q(A.astype(np.float32)))
        E = np.exp(Z - Z.max(1, keepdims=True))
        P = (E / E.sum(1, keepdims=True)).astype(np.float32)
        losses.append(float(-(y * np.log(np.maximum(P, 1e-30))).sum(1).mean()))
        D = q(P - y)
        for l in range(L - 1, -1, -1):
            g = (D.T.astype(mm) @ H[l].astype(mm) / B).astype(np.float32)
            gb = D.astype(np.float64).mean(0).astype(np.float32)
            if l > 0:
                Eb = (D.astype(mm) @ Wh[l].astype(mm)).astype(np.float32)
                h = H[l]
                der = (1 - h * h) if acts[l - 1] == po.TANH else ((h > 0).astype(np.float32) if acts[l - 1] == po.RELU else h * (1 - h))
                D = q(Eb * der)
            d = lr * (g + wd2 * Wm[l]) + mom * vW[l]
            vW[l] = d
            Wm[l] = Wm[l] - d
            db = lr * gb + mom * vb[l]
            vb[l] = db
            bm[l] = bm[l] - db
    return Wm, bm, losses
