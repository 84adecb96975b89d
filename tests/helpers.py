"""Shared helpers for the parity tests."""
import os

import numpy as np

import pyoracle as po

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TRAIN_CASES = ["one_sample_2_3_2", "window_4_5_3_1", "decay_3_4_2", "cfg1_shape_4_16_3",
               "cfg2_shape_32_64_64_1", "mixed_5_7_6_4", "kl_3_5_4_2", "xornet", "iris"]


def load_case(name):
    d = np.load(os.path.join(GOLDEN, f"train_{name}.npz"), allow_pickle=False)
    sizes = [int(v) for v in d["sizes"]]
    nl = len(sizes) - 1
    cost, N, mb, epochs = [int(v) for v in d["ints"]]
    lr, mom, wd1, wd2 = [float(v) for v in d["hyper"]]
    spec = po.make_spec(sizes, [int(a) for a in d["acts"]], lr=lr, mom=mom, wd1=wd1, wd2=wd2,
                        act_params=[float(v) for v in d["act_params"]], batch=mb, cost=cost)
    return dict(d=d, sizes=sizes, nl=nl, cost=cost, N=N, mb=mb, epochs=epochs, spec=spec,
                W0=[d[f"W0_{l}"] for l in range(nl)], bias0=d["bias0"], X=d["X"], Y=d["Y"])


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
