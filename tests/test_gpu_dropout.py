"""Dropout in exact mode on the GPU (through the C ABI) against the fixtures made by the reference's
own compiled Layer / Node / Edge objects and against the CPU restatement.  Bar as for the other
exact-mode tests: bit for bit after the full schedule, window lengths and error accumulators
included."""
import numpy as np
import pytest

import pyoracle as po
from helpers import DROPOUT_CASES, bits_equal, load_case
from test_gpu_exact import gpu_net

pytestmark = pytest.mark.gpu


def oracle_net(c):
    o = po.ExactNet(c["spec"])
    for l in range(c["nl"]):
        o.set_weights(l, c["W0"][l])
        o.set_bias(l, c["bias0"][l])
    return o


@pytest.mark.parametrize("name", DROPOUT_CASES)
def test_fixture_schedule_with_reference_flags(name):
    print("case", name, flush=True)
    c = load_case(name, "dropout")
    d = c["d"]
    net = gpu_net(c)
    net.set_dropout_masks(d["masks"])
    ms, preds = net.run_epochs_exact(c["epochs"], train=True, want_preds=True)
    assert len(ms) == c["epochs"]
    assert bits_equal([m[0] for m in ms], d["epochs"][:, 0])
    assert bits_equal([m[1] for m in ms], d["epochs"][:, 1])
    assert bits_equal(preds, d["preds"])
    for l in range(c["nl"]):
        W, b = net.get_params(l)
        assert bits_equal(W, d[f"W_{l}"]), l
        s, t = net.get_state(l)
        assert bits_equal(s, d[f"wsum_{l}"]) and bits_equal(t, d[f"wlast_{l}"]), l
        cnt, err = net.get_dropout_state(l)
        assert np.array_equal(cnt, d[f"wcnt_{l}"]), l
        if l >= 1:
            assert bits_equal(b[0], d["bias"][l]), l
        if l + 1 < c["nl"]:
            assert bits_equal(err, d[f"errder_{l + 1}"]), l
    net.close()


def test_wider_network_with_windows_longer_than_the_minibatch():
    """A hidden layer wider than a wavefront, decays, momentum, minibatch 4 with edges that sit out
    applying rows: flags, windows, their lengths, accumulators and weights bit for bit as the CPU
    restatement's."""
    import pyglades as pg
    rng = np.random.default_rng(31)
    sizes, N, mb, E = [9, 70, 5, 3], 17, 4, 3
    acts = [po.RELU, po.LEAKY, po.LINEAR]
    ospec = po.make_spec(sizes, acts, lr=0.002, mom=0.4, wd1=0.001, wd2=0.002, act_params=[0, 0.05, 1.0], batch=mb,
                         cost=po.REGRESSION)
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * (0.7 / np.sqrt(sizes[l]))).astype(np.float32) for l in range(3)]
    bs = [0.0, 0.05, -0.02]
    X = rng.random((N, sizes[0])).astype(np.float32)
    Y = rng.random((N, sizes[-1])).astype(np.float32)
    po.libc_srand(5)
    masks = np.stack([po.dropout_draw(ospec, [0.3, 0.4, 0.3], N) for _ in range(E)])
    o = po.ExactNet(ospec)
    net = pg.Net(pg.make_spec(sizes, acts, lr=0.002, mom=0.4, wd1=0.001, wd2=0.002, act_params=[0, 0.05, 1.0], batch=mb,
                              cost=pg.REGRESSION, mode=pg.MODE_EXACT))
    for l in range(3):
        o.set_weights(l, Ws[l]); o.set_bias(l, bs[l])
        net.set_params(l, Ws[l], bs[l])
    net.set_dataset(X, Y)
    net.set_dropout_masks(masks)
    ms, preds = net.run_epochs_exact(E, want_preds=True)
    oms = []
    for ep in range(E):
        m, opreds = o.epoch(X, Y, masks=masks[ep])
        oms.append(m)
    assert bits_equal(preds, opreds)
    assert bits_equal([m[0] for m in ms], [m.loss for m in oms])
    for l in range(3):
        W, b = net.get_params(l)
        assert bits_equal(W, o.get_weights(l)), l
        if l:
            assert bits_equal(b[0], o.get_bias(l)), l
        s, t = net.get_state(l)
        os_, ot = o.get_window(l)
        assert bits_equal(s, os_) and bits_equal(t, ot), l
        cnt, err = net.get_dropout_state(l)
        assert np.array_equal(cnt, o.get_pending(l)), l
        if l + 1 < 3:
            assert bits_equal(err, o.get_errder(l + 1)), l
    assert max(int(net.get_dropout_state(l)[0].max()) for l in range(3)) > mb  # windows longer than mb occurred
    net.close()


def test_epoch_by_epoch_equals_one_launch_and_state_round_trips():
    """The accumulators and window lengths survive between launches, and a network rebuilt from
    get_params / get_state / get_dropout_state continues exactly as the original."""
    c = load_case("deep_64_48_6_2", "dropout")
    masks = c["d"]["masks"]
    a, b, r = gpu_net(c), gpu_net(c), gpu_net(c)
    a.set_dropout_masks(masks)
    ms_a, _ = a.run_epochs_exact(3)
    ms_b = []
    for ep in range(3):
        b.set_dropout_masks(masks[ep:ep + 1])
        ms_b += b.run_epochs_exact(1)[0]
        if ep == 0:  # move everything into a fresh handle after the first epoch
            for l in range(c["nl"]):
                W, bias = b.get_params(l)
                r.set_params(l, W, bias)
                r.set_state(l, *b.get_state(l))
                r.set_dropout_state(l, *b.get_dropout_state(l))
    assert ms_a == ms_b
    ms_r = []
    for ep in (1, 2):
        r.set_dropout_masks(masks[ep:ep + 1])
        ms_r += r.run_epochs_exact(1)[0]
    assert ms_r == ms_a[1:]
    for l in range(c["nl"]):
        for other in (b, r):
            assert np.array_equal(a.get_params(l)[0], other.get_params(l)[0])
            assert np.array_equal(a.get_dropout_state(l)[0], other.get_dropout_state(l)[0])
            assert bits_equal(a.get_dropout_state(l)[1], other.get_dropout_state(l)[1])
    for n in (a, b, r):
        n.close()


def test_flags_are_used_once_and_later_runs_keep_the_leftovers():
    """After a run with flags the next run drops nothing, but starts from the accumulators and
    windows the dropout rows left behind -- as the reference's Node / Edge objects would."""
    c = load_case("window_4_5_3_1", "dropout")
    masks = c["d"]["masks"]
    net = gpu_net(c)
    o = oracle_net(c)
    net.set_dropout_masks(masks[:2])
    net.run_epochs_exact(2)
    for ep in range(2):
        o.epoch(c["X"], c["Y"], masks=masks[ep])
    assert any(np.any(o.get_errder(l) != 0) for l in range(1, c["nl"]))  # there are leftovers
    ms, preds = net.run_epochs_exact(2, want_preds=True)
    for ep in range(2):
        m, opreds = o.epoch(c["X"], c["Y"])
    assert bits_equal(preds, opreds)
    assert bits_equal(ms[-1][0], m.loss)
    for l in range(c["nl"]):
        assert bits_equal(net.get_params(l)[0], o.get_weights(l)), l
        assert np.array_equal(net.get_dropout_state(l)[0], o.get_pending(l))
    net.close()


def test_test_pass_drops_too_and_changes_nothing():
    """SGDHelper scrambles before every row whatever the run type (network.cpp:407-411)."""
    c = load_case("batch1_5_7_6_4", "dropout")
    masks = c["d"]["masks"]
    net = gpu_net(c)
    o = oracle_net(c)
    net.set_dropout_masks(masks[:1])
    ms, preds = net.run_epochs_exact(1, train=False, want_preds=True)
    m, opreds = o.epoch(c["X"], c["Y"], train=False, masks=masks[0])
    _, plain = oracle_net(c).epoch(c["X"], c["Y"], train=False)
    assert bits_equal(preds, opreds)
    assert not np.allclose(opreds, plain)
    assert bits_equal(ms[0][0], m.loss)
    for l in range(c["nl"]):
        assert np.array_equal(net.get_params(l)[0], c["W0"][l])
    net.close()


def test_many_networks_with_their_own_flags_equal_their_solo_runs():
    import pyglades as pg
    c = load_case("decay_3_4_2", "dropout")
    po.libc_srand(77)
    K, E = 5, 3
    solo, group, flags = [], [], []
    for k in range(K):
        flags.append(np.stack([po.dropout_draw(c["spec"], c["d"]["p"], c["N"]) for _ in range(E)]))
        solo.append(gpu_net(c))
        group.append(gpu_net(c))
    flags[2] = None  # one of them drops nothing
    want = []
    for n, f in zip(solo, flags):
        n.set_dropout_masks(f)
        want.append(n.run_epochs_exact(E)[0])
    for n, f in zip(group, flags):
        n.set_dropout_masks(f)
    got = pg.run_epochs_exact_multi(group, E)
    assert got == want
    assert len({tuple(ms[-1]) for ms in got}) == K  # different flags, different results
    for a, b in zip(solo, group):
        for l in range(c["nl"]):
            assert np.array_equal(a.get_params(l)[0], b.get_params(l)[0])
            assert np.array_equal(a.get_dropout_state(l)[0], b.get_dropout_state(l)[0])
    for n in solo + group:
        n.close()


def test_error_paths():
    import pyglades as pg
    c = load_case("decay_3_4_2", "dropout")
    masks = c["d"]["masks"]
    net = gpu_net(c)
    net.set_dropout_masks(masks[:1])
    with pytest.raises(pg.GladesHipError):   # more epochs than flags
        net.run_epochs_exact(2)
    bad = masks[:1].copy()
    bad[0, 3, :3] = 1                        # the whole input layer of row 3
    with pytest.raises(pg.GladesHipError):
        net.set_dropout_masks(bad)
    bad = masks[:1].copy()
    bad[0, 0, 0] = 2
    with pytest.raises(pg.GladesHipError):
        net.set_dropout_masks(bad)
    net.set_dropout_masks(None)
    net.run_epochs_exact(2)                  # no flags: runs as before
    net.close()
    fresh = pg.Net(pg.make_spec([3, 4, 2], [2, 2], batch=4, mode=pg.MODE_EXACT))
    with pytest.raises(pg.GladesHipError):   # no table yet
        fresh.lib.ghip_net_set_dropout_masks and pg._check(
            fresh.lib.ghip_net_set_dropout_masks(fresh.h, pg._ptr(masks[:1].copy()), 1))
    fresh.close()
