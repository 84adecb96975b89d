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


def matrix_form_dropout(sizes, acts, params, cost, lr, mom, mb, Ws, bs, X, Y, masks, epochs,
                        derivative_on_dropped=False, clear_on="last_node", apply_all=False):
    """float64 statement of the reference's rows WITH dropout flags, written from the loop nests of
    network.cpp:457-575 (forward) and :577-668 (back-propagation) a layer at a time over the
    (input node, output node) grid.  masks[e][r] holds one 0/1 flag per node of layers 0..L-1
    (1 = dropped); the output layer never drops (layer.cpp:136-149).

    forward, weight layer l:  a pair contributes w*a only if both its nodes are kept (:479-487); the
      node is finalised at the last KEPT input node whatever its own flag (:489-511), so a dropped
      node ends up as squash(0 + bias).
    back-propagation, weight layer l, pair (i, o), i outer, o inner:
      E_out[o] is the output node's accumulator: the cost derivative at the output layer (rewritten
      on every visit, :599-612), else what the layer above left in it.
      c = E_out[o] * f'(a_out[o]) for a kept pair, and c = E_out[o] WITHOUT the derivative for a
      dropped one (:621-626: the product sits inside `if (!dropout)`).
      kept pair: push d = lr*c*a_in[i] + mom*last(window) (+ decay terms, 0 here) on the edge's
      window (:641-644); at rows with r % mb == 0 subtract (sum of the window's first mb entries)/mb
      and empty the window (:647-651, node.cpp:294-307); bias_l -= lr*c for l >= 1 (:654-656).
      E_out[o] is cleared only by a KEPT pair whose input node is the layer's LAST node, kept or not
      (:628-631: `cInputNodeCounter == cInputLayer->size() - 1` inside `if (!dropout)`), so it can
      outlive the row.
      every pair, kept or not: E_in[i] <- E_in[i] + (E_in[i] + c * W[o,i]) with the weight as it is
      after this pair's update (:659-662), i.e. over o:
      E_in[i] = 2^n_out * E_in[i] + sum_o 2^(n_out-1-o) * c[i,o] * W'[o,i].
    The keyword switches state the rules the other way round (apply_all: an apply sums the whole
    window instead of its first mb entries); the test shows that they then do NOT reproduce the
    restatement.  Also returns the longest window an apply met."""
    nl = len(sizes) - 1
    W = [w.astype(np.float64) for w in Ws]
    b = [float(v) for v in bs]
    cap = 4 * mb + 8 * len(X)
    win = [np.zeros((sizes[l + 1], sizes[l], cap)) for l in range(nl)]
    cnt = [np.zeros((sizes[l + 1], sizes[l]), np.int64) for l in range(nl)]
    E = [np.zeros(sizes[l]) for l in range(nl + 1)]   # accumulators of the nodes of layers 1..L (index 0 unused)
    offs = np.concatenate([[0], np.cumsum(sizes[:-1])])
    peak = 0
    for ep in range(epochs):
        for r, (x, y) in enumerate(zip(X.astype(np.float64), Y.astype(np.float64))):
            keep = [masks[ep][r][offs[l]:offs[l + 1]] == 0 for l in range(nl)] + [np.ones(sizes[-1], bool)]
            a = [x]
            for l in range(nl):
                valid = keep[l + 1][:, None] & keep[l][None, :]            # [o, i]
                z = (W[l] * valid) @ a[l] + (b[l] if l >= 1 else 0.0)
                a.append(_act(z, acts[l], params[l]))
            p = a[-1]
            cder = 2.0 * (p - y) if cost == po.REGRESSION else (p - y) / ((1.0 - p) * p)
            for l in range(nl - 1, -1, -1):
                n_in, n_out = sizes[l], sizes[l + 1]
                valid = keep[l][:, None] & keep[l + 1][None, :]            # [i, o]
                if l == nl - 1:
                    e_out, der = cder, np.ones(n_out)
                else:
                    e_out, der = E[l + 1], _der(a[l + 1], acts[l])
                factor = np.broadcast_to(der[None, :], (n_in, n_out)) if derivative_on_dropped else np.where(valid, der[None, :], 1.0)
                c = e_out[None, :] * factor                                # [i, o]
                # kept pairs: push on the window, maybe apply, bias
                last = np.take_along_axis(win[l], np.maximum(cnt[l] - 1, 0)[..., None], 2)[..., 0] * (cnt[l] > 0)
                d = lr * c.T * a[l][None, :] + mom * last                  # [o, i]
                vt = valid.T
                oi = np.nonzero(vt)
                win[l][oi[0], oi[1], cnt[l][oi]] = d[oi]
                cnt[l][oi] += 1
                if r % mb == 0:
                    peak = max(peak, int(cnt[l][oi].max()) if oi[0].size else 0)
                    upd = (win[l] if apply_all else win[l][:, :, :mb]).sum(2) / mb
                    W[l] = np.where(vt, W[l] - upd, W[l])
                    win[l][oi[0], oi[1], :] = 0.0
                    cnt[l][oi] = 0
                if l >= 1:
                    b[l] -= lr * c[valid].sum()
                # output nodes' accumulators after the layer
                if l < nl - 1:
                    if clear_on == "last_node":
                        cleared = valid[n_in - 1, :]
                    elif clear_on == "last_kept":
                        cleared = valid[np.nonzero(keep[l])[0].max(), :]
                    else:
                        cleared = np.ones(n_out, bool)
                    E[l + 1] = np.where(cleared, 0.0, E[l + 1])
                # every pair hands its share down
                if l >= 1:
                    pw = 2.0 ** (n_out - 1 - np.arange(n_out))
                    E[l] = 2.0 ** n_out * E[l] + (c * W[l].T * pw[None, :]).sum(1)
    return W, b, E, cnt, peak


def _dropout_case(sizes, acts, params, cost, mb, mom, rows, epochs, seed, hand_masks=None):
    rng = np.random.default_rng(seed)
    nl = len(sizes) - 1
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * 0.4).astype(np.float32) for l in range(nl)]
    bs = [0.0] + [0.1] * (nl - 1)
    X = rng.random((rows, sizes[0])).astype(np.float32)
    Y = (rng.random((rows, sizes[-1])) * 0.8 + 0.1).astype(np.float32)
    ml = sum(sizes[:-1])
    if hand_masks is not None:
        masks = np.array(hand_masks, np.uint8).reshape(epochs, rows, ml)
    else:
        masks = (rng.random((epochs, rows, ml)) < 0.35).astype(np.uint8)
        offs = np.concatenate([[0], np.cumsum(sizes[:-1])])
        for l in range(nl):   # no layer may lose every node (the reference redraws such a layer, layer.cpp:116-133)
            blk = masks[:, :, offs[l]:offs[l + 1]]
            blk[blk.all(2), 0] = 0
    return Ws, bs, X, Y, masks


def _run_oracle_with_masks(sizes, acts, params, cost, lr, mom, mb, Ws, bs, X, Y, masks):
    net = po.ExactNet(po.make_spec(sizes, acts, lr=lr, mom=mom, act_params=params, batch=mb, cost=cost))
    for l in range(len(sizes) - 1):
        net.set_weights(l, Ws[l])
        net.set_bias(l, bs[l])
    for ep in range(masks.shape[0]):
        net.epoch(X, Y, masks=masks[ep])
    return net


# flags per row: layer 0 nodes, then layer 1 nodes (1 = dropped); two epochs of three rows each
HAND_2_3_2 = [
    # epoch 0
    [0, 0, 0, 1, 0],     # hidden node 1 dropped: its pairs hand E down without f' in the layer below
    [0, 1, 0, 0, 0],     # LAST input node dropped: no pair clears the hidden accumulators, they survive the row
    [1, 0, 0, 0, 1],     # first input and last hidden node dropped
    # epoch 1
    [0, 0, 1, 0, 0],
    [0, 1, 1, 0, 0],
    [0, 0, 0, 0, 0],     # a clean row that inherits what the rows before left behind
]
# mb 2, five rows: input node 1 sits out row 2, an applying row, so its edges meet row 4's apply with
# three entries (rows 1, 3, 4) of which applyDeltas reads two
HAND_3_4_2_WINDOW = [
    [0, 0, 0, 0, 0, 0, 0],
    [0, 0, 0, 0, 0, 0, 0],
    [0, 1, 0, 0, 0, 1, 0],
    [0, 0, 0, 0, 0, 0, 0],
    [0, 0, 0, 0, 0, 0, 0],
]
HAND_2_3_3_2 = [
    [0, 0, 0, 1, 0, 0, 0, 1],   # a dropped node in each hidden layer: the pair between them hands E down without f'
    [0, 1, 1, 0, 0, 0, 1, 0],
    [0, 0, 0, 0, 1, 1, 0, 0],
    [1, 0, 0, 1, 0, 0, 0, 0],
]
HAND_3_4_2 = [
    [0, 0, 1, 0, 0, 0, 1],
    [0, 1, 0, 1, 0, 0, 0],
    [0, 0, 1, 0, 1, 1, 0],
    [1, 0, 0, 0, 0, 0, 0],
    [0, 0, 0, 0, 0, 1, 0],
    [0, 0, 1, 1, 0, 0, 0],
]


@pytest.mark.parametrize("sizes,acts,params,cost,mb,mom,rows,epochs,hand", [
    ([2, 3, 2], [po.TANH, po.TANH], [0, 0], po.REGRESSION, 1, 0.0, 3, 2, HAND_2_3_2),
    ([3, 4, 2], [po.SIGMOID, po.SIGMOID], [0, 0], po.CLASSIFICATION, 1, 0.0, 3, 2, HAND_3_4_2),
    ([3, 4, 2], [po.TANH, po.LINEAR], [0, 1.0], po.REGRESSION, 2, 0.6, 5, 1, HAND_3_4_2_WINDOW),   # a window outgrows mb
    ([2, 3, 3, 2], [po.TANH, po.SIGMOID, po.TANH], [0, 0, 0], po.REGRESSION, 1, 0.0, 4, 1, HAND_2_3_3_2),
    ([4, 5, 3, 2], [po.TANH, po.SIGMOID, po.TANH], [0, 0, 0], po.REGRESSION, 3, 0.5, 7, 3, None),
    ([5, 3, 4, 1], [po.SIGMOID, po.TANH, po.LINEAR], [0, 0, 0.5], po.REGRESSION, 1, 0.0, 6, 2, None),
])
def test_dropout_rows_match_matrix_form(sizes, acts, params, cost, mb, mom, rows, epochs, hand):
    """The restatement's dropout branches against the float64 statement above: weights, scalar
    biases, the accumulators that survive rows and the windows' lengths (which exceed mb when an
    edge sits out an applying row)."""
    lr = 0.02
    Ws, bs, X, Y, masks = _dropout_case(sizes, acts, params, cost, mb, mom, rows, epochs, seed=sum(sizes) + mb, hand_masks=hand)
    net = _run_oracle_with_masks(sizes, acts, params, cost, lr, mom, mb, Ws, bs, X, Y, masks)
    Wm, bm, Em, cm, peak = matrix_form_dropout(sizes, acts, params, cost, lr, mom, mb, Ws, bs, X, Y, masks, epochs)
    nl = len(sizes) - 1
    for l in range(nl):
        np.testing.assert_allclose(net.get_weights(l), Wm[l], rtol=5e-4, atol=5e-6)
        assert np.array_equal(net.get_pending(l), cm[l]), l
        if l >= 1:
            np.testing.assert_allclose(net.get_bias(l), bm[l], rtol=5e-4, atol=5e-6)
            np.testing.assert_allclose(net.get_errder(l), Em[l], rtol=5e-4, atol=1e-6 * max(1.0, np.abs(Em[l]).max()))
    if hand is HAND_3_4_2_WINDOW:
        assert peak > mb      # the case does meet an apply with a window longer than mb


@pytest.mark.parametrize("flip", [dict(derivative_on_dropped=True), dict(clear_on="last_kept"), dict(clear_on="always"),
                                  dict(apply_all=True)])
def test_dropout_rules_the_other_way_round_do_not_match(flip):
    """Each dropout rule of back-propagation stated the other way round -- the derivative factor also
    on dropped pairs; the accumulator cleared at the last KEPT input node, or after every row; an
    apply that sums a whole over-long window -- must move the result away from the restatement (so
    the test above does pin them).  The derivative rule only shows between two hidden layers (what
    the first weight layer hands down lands on input nodes, which nobody reads)."""
    lr = 0.02
    if "apply_all" in flip:
        sizes, acts, params, mb, mom, rows, epochs, hand = [3, 4, 2], [po.TANH, po.LINEAR], [0, 1.0], 2, 0.6, 5, 1, HAND_3_4_2_WINDOW
    else:
        sizes, acts, params, mb, mom, rows, epochs, hand = [2, 3, 3, 2], [po.TANH, po.SIGMOID, po.TANH], [0, 0, 0], 1, 0.0, 4, 1, HAND_2_3_3_2
    Ws, bs, X, Y, masks = _dropout_case(sizes, acts, params, po.REGRESSION, mb, mom, rows, epochs, seed=8, hand_masks=hand)
    net = _run_oracle_with_masks(sizes, acts, params, po.REGRESSION, lr, mom, mb, Ws, bs, X, Y, masks)
    good = matrix_form_dropout(sizes, acts, params, po.REGRESSION, lr, mom, mb, Ws, bs, X, Y, masks, epochs)
    bad = matrix_form_dropout(sizes, acts, params, po.REGRESSION, lr, mom, mb, Ws, bs, X, Y, masks, epochs, **flip)
    got = np.concatenate([net.get_weights(l).ravel() for l in range(len(sizes) - 1)])
    start = np.concatenate([w.ravel() for w in Ws])
    step = np.abs(got - start).max()
    assert np.abs(got - np.concatenate([w.ravel() for w in good[0]])).max() < 1e-4 * step
    assert np.abs(got - np.concatenate([w.ravel() for w in bad[0]])).max() > 1e-2 * step
