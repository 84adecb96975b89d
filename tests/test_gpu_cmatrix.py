"""Device confusion matrix (through the C ABI) against the restated CMatrix: counts bit-exact,
class metrics of every epoch equal to the restatement's float arithmetic on the same counts."""
import numpy as np
import pytest

import pyoracle as po
from helpers import load_case
from test_gpu_exact import gpu_net

pytestmark = pytest.mark.gpu


def oracle_epochs(c, epochs):
    net = po.ExactNet(c["spec"])
    for l in range(c["nl"]):
        net.set_weights(l, c["W0"][l])
        net.set_bias(l, float(c["bias0"][l]))
    out = []
    for _ in range(epochs):
        _, preds = net.epoch(c["X"], c["Y"], train=True, want_preds=True)
        out.append(preds.copy())
    return out


@pytest.mark.parametrize("name", ["iris", "cfg1_shape_4_16_3", "kl_3_5_4_2"])
def test_exact_mode_matrix_and_class_metrics_per_epoch(name):
    print("case", name, flush=True)
    c = load_case(name)
    E = min(c["epochs"], 6)
    ref_preds = oracle_epochs(c, E)
    net = gpu_net(c)
    net.confusion_enable()
    ms, preds = net.run_epochs_exact(E, train=True, want_preds=True)
    assert len(ms) == E
    M = net.confusion()
    # the counters hold the last epoch; rows are counted under the reference's argmax rule
    assert np.array_equal(M, po.cmatrix(c["Y"], preds))
    assert np.array_equal(M, po.cmatrix(c["Y"], ref_preds[-1]))
    for e in range(E):
        want = po.cmatrix_metrics(po.cmatrix(c["Y"], ref_preds[e]))[4][:5]
        got = net.class_metrics(e)
        assert np.array_equal(np.isnan(got), np.isnan(want))
        ok = ~np.isnan(want)
        assert np.array_equal(got[ok], want[ok]), (e, got, want)
    with pytest.raises(Exception):
        net.class_metrics(E)
    # a test pass restarts the counters too
    net.run_epochs_exact(1, train=False, want_preds=False)
    assert net.confusion().sum() <= c["N"]
    net.close()


def test_canonical_mode_accumulates_until_reset():
    import pyglades as pg
    rng = np.random.default_rng(5)
    sizes, B, N = [12, 16, 5], 64, 192
    acts = [pg.TANH, pg.SOFTMAX]
    spec = pg.make_spec(sizes, acts, lr=0.05, mom=0.9, batch=B, cost=pg.CLASSIFICATION, mode=pg.MODE_CANONICAL)
    ospec = po.make_spec(sizes, [po.TANH, po.SOFTMAX], lr=0.05, mom=0.9, batch=B, cost=po.CLASSIFICATION)
    Ws = [rng.normal(0, 0.4, (sizes[l + 1], sizes[l])).astype(np.float32) for l in range(2)]
    bs = [rng.normal(0, 0.1, sizes[l + 1]).astype(np.float32) for l in range(2)]
    X = rng.normal(0, 1, (N, sizes[0])).astype(np.float32)
    Y = np.eye(5, dtype=np.float32)[rng.integers(0, 5, N)]
    Y[7] = 0.0   # a row without a class counts nowhere
    g = pg.Net(spec)
    o = po.CanonNet(ospec)
    for l in range(2):
        g.set_params(l, Ws[l], bs[l])
        o.set_params(l, Ws[l], bs[l])
    g.set_dataset(X, Y)
    g.confusion_enable()
    want = np.zeros((5, 5), np.int32)
    for k in range(N // B):
        P = o.forward(X[k * B:(k + 1) * B])          # predictions the step's metrics are taken on
        want += po.cmatrix(Y[k * B:(k + 1) * B], P)
        o.step(X[k * B:(k + 1) * B], Y[k * B:(k + 1) * B])
        g.train_step(k * B, B)
    got = g.confusion()
    assert got.sum() == N - 1
    assert np.array_equal(got, want)
    g.confusion_reset()
    assert g.confusion().sum() == 0
    g.close()
