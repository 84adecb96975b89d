"""The C restatement against numbers produced by the reference's own compiled
node/edge/layer/Terminator/gmath code (fixtures written by tests/golden/make_golden.py)."""
import os
import tempfile

import numpy as np
import pytest

import pyoracle as po
from helpers import DROPOUT_CASES, FULL_CASES, GOLDEN, TRAIN_CASES, bits_equal, load_case


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


@pytest.mark.parametrize("name", TRAIN_CASES + FULL_CASES)
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


@pytest.mark.parametrize("name", DROPOUT_CASES)
def test_dropout_draw_and_training_bit_exact(name):
    """Flags, rand() stream position and trained state against the reference's compiled
    Layer::generateDropout / possiblePath / lastValidPath and Node/Edge objects."""
    c = load_case(name, "dropout")
    d = c["d"]
    net = po.ExactNet(c["spec"])
    for l in range(c["nl"]):
        net.set_weights(l, c["W0"][l])
        net.set_bias(l, c["bias0"][l])
    po.libc_srand(int(d["seed"]))
    eps = []
    for ep in range(c["epochs"]):
        masks = po.dropout_draw(c["spec"], d["p"], c["N"])
        assert np.array_equal(masks, d["masks"][ep]), ep
        m, preds = net.epoch(c["X"], c["Y"], masks=masks)
        eps.append((m.loss, m.accuracy))
    assert po.libc_rand() % 65536 == int(d["rand_after"])
    assert bits_equal(np.array(eps, np.float32), d["epochs"])
    assert bits_equal(preds, d["preds"])
    for l in range(c["nl"]):
        assert bits_equal(net.get_weights(l), d[f"W_{l}"]), l
        s, t = net.get_window(l)
        assert bits_equal(s, d[f"wsum_{l}"]) and bits_equal(t, d[f"wlast_{l}"]), l
        assert np.array_equal(net.get_pending(l), d[f"wcnt_{l}"]), l
        if l:
            assert bits_equal(net.get_bias(l), d["bias"][l]), l
            assert bits_equal(net.get_errder(l), d[f"errder_{l}"]), l


def test_dropout_flags_change_the_result_and_zero_flags_do_not():
    """All-zero flags reproduce the run without dropout; the fixture's flags do not (the test
    above would pass vacuously if the flags were ignored)."""
    c = load_case("window_4_5_3_1", "dropout")
    outs = []
    for masks in (None, np.zeros_like(c["d"]["masks"][0]), c["d"]["masks"][0]):
        net = po.ExactNet(c["spec"])
        for l in range(c["nl"]):
            net.set_weights(l, c["W0"][l])
            net.set_bias(l, c["bias0"][l])
        net.epoch(c["X"], c["Y"], masks=masks)
        outs.append([net.get_weights(l) for l in range(c["nl"])])
    assert all(bits_equal(a, b) for a, b in zip(outs[0], outs[1]))
    assert not all(bits_equal(a, b) for a, b in zip(outs[0], outs[2]))


def test_dropped_hidden_node_outputs_squash_of_bias():
    """network.cpp:491-516 finalises every output node at the last valid input: a dropped hidden
    node still takes squash(0 + bias) (squash(0) in the first hidden layer), and feeds nothing on."""
    spec = po.make_spec([2, 3, 1], [po.SIGMOID, po.LINEAR], act_params=[0, 1.0], lr=0.0)
    net = po.ExactNet(spec)
    net.set_weights(0, np.array([[1, 2], [3, 4], [5, 6]], np.float32))
    net.set_weights(1, np.array([[1, 10, 100]], np.float32))
    net.set_bias(1, 0.5)
    X = np.array([[1.0, 1.0]], np.float32)
    Y = np.zeros((1, 1), np.float32)
    sig = lambda z: np.float32(po.lib().go_squash(float(z), po.SIGMOID, 0.0))
    # drop input 1 and hidden node 1
    _, p = net.epoch(X, Y, train=False, masks=np.array([[0, 1, 0, 1, 0]], np.uint8))
    want = np.float32(np.float32(sig(1.0) * np.float32(1)) + np.float32(sig(5.0) * np.float32(100))) + np.float32(0.5)
    assert bits_equal(p, np.array([[want]], np.float32))


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
