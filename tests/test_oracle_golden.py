"""The C restatement against numbers produced by the reference's own compiled
node/edge/layer/Terminator/gmath code (fixtures written by tests/golden/make_golden.py)."""
import os
import tempfile

import numpy as np
import pytest

import pyoracle as po
from helpers import GOLDEN, TRAIN_CASES, bits_equal, load_case


def test_elementwise_grid_bit_exact():
    g = np.load(os.path.join(GOLDEN, "gmath_grid.npz"), allow_pickle=False)
    act = g["act"]
    params = [0.0, 0.01, 0.1]
    L = po.lib()
    for a in range(8):
        for p in range(3):
            for z, sq, der in act[a, p]:
                s = np.float32(L.go_squash(float(z), a, params[p]))
                assert bits_equal(s, sq), (a, p, z)
                assert bits_equal(np.float32(L.go_act_der(float(s), a, params[p])), der), (a, p, z)
    for c in range(3):
        for row in g["cost"][c].reshape(-1, 5):
            e, p, cost, cder, pe = [float(v) for v in row]
            with np.errstate(all="ignore"):
                assert bits_equal(np.float32(L.go_cost(e, p, 12.0, c)), np.float32(cost)), (c, e, p)
                assert bits_equal(np.float32(L.go_cost_der(e, p, c)), np.float32(cder)), (c, e, p)
            assert bits_equal(np.float32(L.go_percent_error(np.float32(p * 3.0 - 1.0), e)), np.float32(pe))


def test_xavier_sampler_bit_exact():
    """Same libc rand() stream as the reference sampler (glibc: srand(seed) is reproducible)."""
    import ctypes
    libc = ctypes.CDLL(None)
    g = np.load(os.path.join(GOLDEN, "xavier_samples.npz"), allow_pickle=False)
    for key in g.files:
        seed, fi, no, act = [int(v) for v in key[1:].split("_")]
        libc.srand(seed)
        W = np.empty((no, fi), np.float32)
        po.lib().go_ref_xavier_layer(fi, no, act, W)
        assert bits_equal(W, g[key]), key
        assert (W >= 0).all()  # the sampler only ever returns the positive half


@pytest.mark.parametrize("name", TRAIN_CASES)
def test_exact_training_bit_exact(name):
    c = load_case(name)
    net = po.ExactNet(c["spec"])
    for l in range(c["nl"]):
        net.set_weights(l, c["W0"][l])
        net.set_bias(l, c["bias0"][l])
    eps = []
    for _ in range(c["epochs"]):
        m, preds = net.epoch(c["X"], c["Y"])
        eps.append((m.loss, m.accuracy))
    d = c["d"]
    assert bits_equal(np.array(eps, np.float32), d["epochs"])
    assert bits_equal(preds, d["preds"])
    for l in range(c["nl"]):
        assert bits_equal(net.get_weights(l), d[f"W_{l}"]), l
        s, t = net.get_window(l)
        assert bits_equal(s, d[f"wsum_{l}"]) and bits_equal(t, d[f"wlast_{l}"]), l
        if l >= 1:
            assert bits_equal(net.get_bias(l), d["bias"][l]), l


@pytest.mark.skipif(not po.have_ref(), reason="reference harness only exists in the build container")
def test_exact_against_live_reference_objects():
    """Fresh seeds every call site the fixtures do not cover: odd sizes, N < mb, mb not dividing N."""
    rng = np.random.default_rng(2024)
    for trial in range(6):
        nl = int(rng.integers(1, 4))
        sizes = [int(rng.integers(1, 9)) for _ in range(nl + 1)]
        acts = [int(rng.integers(0, 7)) for _ in range(nl)]
        N = int(rng.integers(1, 14))
        mb = int(rng.integers(1, 17))
        spec = po.make_spec(sizes, acts, lr=0.02, mom=float(rng.random()), wd1=0.003, wd2=0.004,
                            act_params=[float(rng.random() * 0.1) for _ in range(nl)], batch=mb,
                            cost=int(rng.integers(0, 2)))
        Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * 0.4).astype(np.float32) for l in range(nl)]
        bs = [0.0] + [0.05] * (nl - 1)
        X = rng.random((N, sizes[0])).astype(np.float32)
        Y = (rng.random((N, sizes[-1])) * 0.9 + 0.05).astype(np.float32)
        net = po.ExactNet(spec)
        for l in range(nl):
            net.set_weights(l, Ws[l])
            net.set_bias(l, bs[l])
        eps = []
        with np.errstate(all="ignore"):
            for _ in range(3):
                m, preds = net.epoch(X, Y)
                eps.append((m.loss, m.accuracy))
        with tempfile.TemporaryDirectory() as td:
            ref = po.ref_train(spec, Ws, bs, X, Y, 3, td)
        assert bits_equal(np.array(eps, np.float32), ref["epochs"]), (trial, sizes)
        for l in range(nl):
            assert bits_equal(net.get_weights(l), ref["W"][l]), (trial, sizes, l)


def test_terminator_table_matches_rule():
    """Terminator.cpp:63-78 as a predicate; the table was produced by the reference's object."""
    rec = np.load(os.path.join(GOLDEN, "terminator_table.npz"), allow_pickle=False)["rec"]
    for ts, ep, acc2, now, cep, cacc4, trig in rec:
        acc, cacc = acc2 / 2.0, cacc4 / 4.0
        want = (ts > 0 and now % ts == 0) or (ep > 0 and cep % ep == 0) or (acc > 0 and cacc >= acc)
        assert bool(trig) == bool(want)
