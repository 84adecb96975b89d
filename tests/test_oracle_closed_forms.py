"""Pins for the exact-mode restatement that do not come from running reference code:
closed forms the reference's loop nest implies, written in matrix form in float64."""
import numpy as np
import pytest

import pyoracle as po
from helpers import bits_equal


def _act(z, a, p):
    if a == po.TANH:
        return np.tanh(z)
    if a == po.SIGMOID:
        return 1.0 / (1.0 + np.exp(-z))
    if a == po.LINEAR:
        return p * z
    raise AssertionError


def _der(y, a):
    # the reference always passes 0.01 as the parameter of the derivative (network.cpp:617-618)
    if a == po.TANH:
        return 1.0 - y * y
    if a == po.SIGMOID:
        return y * (1.0 - y)
    if a == po.LINEAR:
        return np.full_like(y, 0.01)
    raise AssertionError


def matrix_form_online(sizes, acts, params, cost, lr, Ws, bs, X, Y, epochs):
    """mb = 1, momentum 0, decay 0: every row applies its own delta immediately, so the
    reference reduces to: delta_out = dC/dp (no output derivative); W -= lr*delta (x) a;
    scalar bias -= n_in*lr*sum(delta); e_in = sum_o 2^(n_out-1-o) * delta_o * W'[o,:] with W'
    the already updated weights; delta_in = e_in * f'(a_in)."""
    Ws = [w.astype(np.float64) for w in Ws]
    bs = [float(b) for b in bs]
    nl = len(sizes) - 1
    for _ in range(epochs):
        for x, y in zip(X.astype(np.float64), Y.astype(np.float64)):
            a = [x]
            for l in range(nl):
                z = Ws[l] @ a[l] + (bs[l] if l >= 1 else 0.0)
                a.append(_act(z, acts[l], params[l]))
            p = a[-1]
            if cost == po.REGRESSION:
                delta = 2.0 * (p - y)
            else:
                delta = (p - y) / ((1.0 - p) * p)
            for l in range(nl - 1, -1, -1):
                n_in, n_out = sizes[l], sizes[l + 1]
                Ws[l] = Ws[l] - lr * np.outer(delta, a[l])
                if l >= 1:
                    bs[l] -= n_in * lr * delta.sum()
                pw = 2.0 ** (n_out - 1 - np.arange(n_out))
                e_in = (pw * delta) @ Ws[l]
                if l >= 1:
                    delta = e_in * _der(a[l], acts[l - 1])
    return Ws, bs


@pytest.mark.parametrize("sizes,acts,params,cost", [
    ([2, 2, 1], [po.TANH, po.TANH], [0, 0], po.REGRESSION),           # the xornet fixture's shape
    ([3, 4, 3], [po.TANH, po.LINEAR], [0, 1.0], po.REGRESSION),       # 3 outputs: weights 4,2,1
    ([4, 5, 3], [po.SIGMOID, po.SIGMOID], [0, 0], po.CLASSIFICATION), # the iris fixture's shape
    ([3, 4, 5, 2], [po.TANH, po.SIGMOID, po.LINEAR], [0, 0, 0.5], po.REGRESSION),
])
def test_online_reduction_matches_matrix_form(sizes, acts, params, cost):
    rng = np.random.default_rng(5)
    nl = len(sizes) - 1
    lr = 0.01
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * 0.4).astype(np.float32) for l in range(nl)]
    bs = [0.0] + [0.1] * (nl - 1)
    X = rng.random((9, sizes[0])).astype(np.float32)
    Y = (rng.random((9, sizes[-1])) * 0.8 + 0.1).astype(np.float32)
    spec = po.make_spec(sizes, acts, lr=lr, act_params=params, batch=1, cost=cost)
    net = po.ExactNet(spec)
    for l in range(nl):
        net.set_weights(l, Ws[l])
        net.set_bias(l, bs[l])
    for _ in range(3):
        net.epoch(X, Y)
    Wm, bm = matrix_form_online(sizes, acts, params, cost, lr, Ws, bs, X, Y, 3)
    for l in range(nl):
        np.testing.assert_allclose(net.get_weights(l), Wm[l], rtol=2e-4, atol=2e-6)
        if l >= 1:
            np.testing.assert_allclose(net.get_bias(l), bm[l], rtol=2e-4, atol=2e-6)


def test_doubling_accumulator_is_not_the_textbook_sum():
    """With two or more output nodes the hidden error is sum_o 2^(n_out-1-o) delta_o w_oi:
    dropping the doubling (textbook) must NOT reproduce the oracle."""
    sizes, acts = [2, 3, 2], [po.TANH, po.TANH]
    rng = np.random.default_rng(0)
    Ws = [(rng.standard_normal((3, 2)) * 0.5).astype(np.float32), (rng.standard_normal((2, 3)) * 0.5).astype(np.float32)]
    x = rng.random((1, 2)).astype(np.float32)
    y = rng.random((1, 2)).astype(np.float32)
    spec = po.make_spec(sizes, acts, lr=0.1, batch=1, cost=po.REGRESSION)
    net = po.ExactNet(spec)
    net.set_weights(0, Ws[0]); net.set_weights(1, Ws[1])
    net.epoch(x, y)
    Wm, _ = matrix_form_online(sizes, acts, [0, 0], po.REGRESSION, 0.1, Ws, [0, 0], x, y, 1)
    np.testing.assert_allclose(net.get_weights(0), Wm[0], rtol=1e-5, atol=1e-7)
    # textbook: e = W'^T delta
    a1 = np.tanh(Ws[0].astype(np.float64) @ x[0])
    p = np.tanh(Ws[1].astype(np.float64) @ a1)
    delta = 2 * (p - y[0])
    W1n = Ws[1] - 0.1 * np.outer(delta, a1)
    e = delta @ W1n
    W0_textbook = Ws[0] - 0.1 * np.outer(e * (1 - a1 * a1), x[0])
    assert np.abs(net.get_weights(0) - W0_textbook).max() > 1e-4


def test_window_schedule():
    """Applies happen at rows 0, mb, 2mb, ... of every epoch (network.cpp:647-651): the window is
    empty after an epoch exactly when (N-1) % mb == 0, and the very first apply divides a single
    delta by mb."""
    rng = np.random.default_rng(1)
    sizes, acts = [3, 4, 1], [po.TANH, po.TANH]
    Ws = [(rng.standard_normal((4, 3)) * 0.3).astype(np.float32), (rng.standard_normal((1, 4)) * 0.3).astype(np.float32)]

    def run(N, mb, epochs=1, mom=0.0):
        X = np.random.default_rng(2).random((N, 3)).astype(np.float32)
        Y = np.random.default_rng(3).random((N, 1)).astype(np.float32)
        net = po.ExactNet(po.make_spec(sizes, acts, lr=0.05, mom=mom, batch=mb, cost=po.REGRESSION))
        net.set_weights(0, Ws[0]); net.set_weights(1, Ws[1])
        for _ in range(epochs):
            net.epoch(X, Y)
        return net

    for N, mb in [(7, 3), (1, 5), (9, 4), (4, 1)]:
        s, t = run(N, mb).get_window(1)
        assert not s.any() and not t.any(), (N, mb)
    for N, mb in [(8, 3), (2, 5), (3, 4)]:
        s, t = run(N, mb).get_window(1)
        assert s.any() and t.any(), (N, mb)
    # first apply: one delta / mb  => (W0 - W) scales as 1/mb (output layer, same forward)
    d1 = Ws[1] - run(1, 1).get_weights(1)
    d4 = Ws[1] - run(1, 4).get_weights(1)
    np.testing.assert_allclose(d4 * 4, d1, rtol=1e-3)  # W0-W cancels ~4 digits in fp32
    # rows after the last multiple of mb stay pending and are carried into the next epoch's
    # row-0 apply: N=6, mb=4 -> applies at rows 0 and 4, row 5 pending (one entry: sum == last)
    s1, t1 = run(6, 4, epochs=1).get_window(0)
    assert s1.any() and bits_equal(s1, t1)
    s2, t2 = run(6, 4, epochs=2, mom=0.9).get_window(0)
    assert s2.any() and bits_equal(s2, t2)
    # N=7: rows 5 and 6 pending; sum = d5 + d6 differs from last = d6
    s3, t3 = run(7, 4, epochs=1, mom=0.9).get_window(0)
    assert not bits_equal(s3, t3)
    # momentum chains inside the window (node.cpp:285-291): N=3, mb=4 -> only row 0 applies (its
    # window holds one delta whose momentum term is 0), rows 1,2 stay pending and see identical
    # weights with or without momentum, so d2(mom) - d2(no mom) = mom * d1
    s5, t5 = run(3, 4, mom=0.9).get_window(0)
    s6, t6 = run(3, 4, mom=0.0).get_window(0)
    np.testing.assert_allclose(t5 - t6, 0.9 * (s6 - t6), rtol=1e-3, atol=1e-9)


def test_forward_is_gemv_plus_scalar_bias():
    rng = np.random.default_rng(9)
    sizes, acts = [6, 5, 4, 3], [po.SIGMOID, po.TANH, po.LINEAR]
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * 0.5).astype(np.float32) for l in range(3)]
    bs = [0.0, 0.3, -0.2]
    X = rng.standard_normal((17, 6)).astype(np.float32)
    Y = rng.random((17, 3)).astype(np.float32)
    net = po.ExactNet(po.make_spec(sizes, acts, act_params=[0, 0, 0.7], batch=4, cost=po.REGRESSION))
    for l in range(3):
        net.set_weights(l, Ws[l]); net.set_bias(l, bs[l])
    m, preds = net.epoch(X, Y, train=False)
    a = X.astype(np.float64)
    a = 1 / (1 + np.exp(-(a @ Ws[0].T.astype(np.float64))))
    a = np.tanh(a @ Ws[1].T.astype(np.float64) + 0.3)
    a = 0.7 * (a @ Ws[2].T.astype(np.float64) - 0.2)
    np.testing.assert_allclose(preds, a, rtol=1e-5, atol=1e-6)
    # loss = mean squared error over N*n_out, accuracy = mean (1-min(|p-y|,1))*100
    np.testing.assert_allclose(m.loss, np.mean((a - Y) ** 2), rtol=1e-5)
    np.testing.assert_allclose(m.accuracy, np.mean((1 - np.minimum(np.abs(a - Y), 1)) * 100), rtol=1e-5)
    # test mode leaves the parameters untouched
    for l in range(3):
        assert bits_equal(net.get_weights(l), Ws[l])


def test_argmax_rule():
    L = po.lib()
    assert L.go_argmax_ref(np.array([0.1, 0.7, 0.7], np.float32), 3) == 1  # strict >: first maximum wins
    assert L.go_argmax_ref(np.array([-1.0, 0.0, -0.5], np.float32), 3) == -1  # nothing above 0
    assert L.go_argmax_ref(np.array([0.01, 0.99, 0.01], np.float32), 3) == 1
