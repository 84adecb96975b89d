"""Exact mode on the GPU (through the C ABI) against the CPU restatement and the fixtures made
by the reference's own compiled objects.  Bar: bit for bit -- losses, accuracies, predictions,
weights, biases and delta windows after the full schedule (the kernel repeats the reference's fp32
operations one by one, without fused multiply-adds, and its tanh / exp / log return the C library's
floats).  The tolerance helper below only serves the closed-form bias mode, which is a different
summation order on purpose."""
import numpy as np
import pytest

import pyoracle as po
from helpers import FULL_CASES, TRAIN_CASES, bits_equal, load_case

pytestmark = pytest.mark.gpu

RTOL = 1e-4


def close(a, b, rtol=RTOL, atol=None):
    """|a-b| <= rtol*|b| + atol, with atol = rtol * (largest magnitude in b) unless given: an
    entry that is tiny next to its neighbours is held to the array's scale, not its own."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    fin = np.isfinite(b)
    assert np.array_equal(np.isfinite(a), fin)
    if atol is None:
        atol = rtol * (np.abs(b[fin]).max() if fin.any() else 0.0) + 1e-7
    np.testing.assert_allclose(a[fin], b[fin], rtol=rtol, atol=atol)


def gpu_net(c, bias_mode=0):
    import pyglades as pg
    spec = pg.make_spec(c["sizes"], [c["spec"].act[l] for l in range(c["nl"])],
                        lr=[c["spec"].lr[l] for l in range(c["nl"])], mom=[c["spec"].mom[l] for l in range(c["nl"])],
                        wd1=[c["spec"].wd1[l] for l in range(c["nl"])], wd2=[c["spec"].wd2[l] for l in range(c["nl"])],
                        act_params=[c["spec"].act_param[l] for l in range(c["nl"])], batch=c["mb"], cost=c["cost"],
                        mode=pg.MODE_EXACT, bias_mode=bias_mode)
    net = pg.Net(spec)
    for l in range(c["nl"]):
        net.set_params(l, c["W0"][l], c["bias0"][l])
    net.set_dataset(c["X"], c["Y"])
    return net


@pytest.mark.parametrize("name", TRAIN_CASES + FULL_CASES)
def test_fixture_schedule(name):
    print("case", name, flush=True)
    c = load_case(name)
    net = gpu_net(c)
    ms, preds = net.run_epochs_exact(c["epochs"], train=True, want_preds=True)
    d = c["d"]
    assert len(ms) == c["epochs"]
    assert bits_equal([m[0] for m in ms], d["epochs"][:, 0])
    assert bits_equal([m[1] for m in ms], d["epochs"][:, 1])
    assert bits_equal(preds, d["preds"])
    for l in range(c["nl"]):
        W, b = net.get_params(l)
        assert bits_equal(W, d[f"W_{l}"]), l
        s, t = net.get_state(l)
        assert bits_equal(s, d[f"wsum_{l}"]) and bits_equal(t, d[f"wlast_{l}"]), l
        if l >= 1:
            assert bits_equal(b[0], d["bias"][l]), l
    net.close()


def test_epoch_by_epoch_equals_one_launch():
    """Resuming (one launch per epoch) must equal a single multi-epoch launch: all state,
    including pending delta windows, survives between launches."""
    c = load_case("window_4_5_3_1")
    a = gpu_net(c)
    b = gpu_net(c)
    ms_a, _ = a.run_epochs_exact(4)
    ms_b = []
    for _ in range(4):
        m, _ = b.run_epochs_exact(1)
        ms_b += m
    assert ms_a == ms_b
    for l in range(c["nl"]):
        assert np.array_equal(a.get_params(l)[0], b.get_params(l)[0])
    a.close(); b.close()


def test_test_pass_changes_nothing_and_matches_oracle():
    c = load_case("mixed_5_7_6_4")
    net = gpu_net(c)
    ms, preds = net.run_epochs_exact(1, train=False, want_preds=True)
    o = po.ExactNet(c["spec"])
    for l in range(c["nl"]):
        o.set_weights(l, c["W0"][l]); o.set_bias(l, c["bias0"][l])
    m, opreds = o.epoch(c["X"], c["Y"], train=False)
    assert bits_equal(preds, opreds)
    assert bits_equal(ms[0][0], m.loss) and bits_equal(ms[0][1], m.accuracy)
    assert ms[0][2] == m.correct
    for l in range(c["nl"]):
        assert np.array_equal(net.get_params(l)[0], c["W0"][l])
    net.close()


def test_stop_accuracy_ends_early():
    c = load_case("iris")
    net = gpu_net(c)
    target = float(c["d"]["epochs"][9, 1]) - 1e-3   # reached for the first time in some epoch <= 10
    first = int(np.argmax(c["d"]["epochs"][:, 1] >= target)) + 1
    ms, _ = net.run_epochs_exact(c["epochs"], stop_accuracy=target)
    assert len(ms) == first
    net.close()


def test_closed_form_bias_is_close_but_sequential_is_default():
    c = load_case("cfg1_shape_4_16_3")
    seq = gpu_net(c, bias_mode=0)
    fast = gpu_net(c, bias_mode=1)
    ms_s, _ = seq.run_epochs_exact(5)
    ms_f, _ = fast.run_epochs_exact(5)
    close([m[0] for m in ms_f], [m[0] for m in ms_s], rtol=1e-3)
    seq.close(); fast.close()


@pytest.mark.parametrize("sizes,N,mb", [([1, 1], 1, 1), ([3, 300, 2], 5, 2), ([70, 3, 65, 1], 6, 4), ([2, 2, 2, 2, 2, 2], 9, 20)])
def test_edge_shapes_against_oracle(sizes, N, mb):
    """Single node, a layer wider than a wavefront, odd sizes, mb > N, deep narrow."""
    import pyglades as pg
    print("shape", sizes, N, mb, flush=True)
    rng = np.random.default_rng(7)
    nl = len(sizes) - 1
    acts = [po.TANH] * nl
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * (0.5 / np.sqrt(sizes[l]))).astype(np.float32) for l in range(nl)]
    X = rng.random((N, sizes[0])).astype(np.float32)
    Y = rng.random((N, sizes[-1])).astype(np.float32)
    ospec = po.make_spec(sizes, acts, lr=0.01, mom=0.5, batch=mb, cost=po.REGRESSION)
    o = po.ExactNet(ospec)
    net = pg.Net(pg.make_spec(sizes, acts, lr=0.01, mom=0.5, batch=mb, cost=pg.REGRESSION, mode=pg.MODE_EXACT))
    for l in range(nl):
        o.set_weights(l, Ws[l]); net.set_params(l, Ws[l], 0.0)
    net.set_dataset(X, Y)
    oms = [o.epoch(X, Y)[0] for _ in range(3)]
    ms, _ = net.run_epochs_exact(3)
    assert bits_equal([m[0] for m in ms], [m.loss for m in oms])
    assert [m[2] for m in ms] == [m.correct for m in oms]
    for l in range(nl):
        assert bits_equal(net.get_params(l)[0], o.get_weights(l)), l
    net.close()


@pytest.mark.parametrize("seed", range(10))
def test_random_small_networks_against_oracle(seed):
    """Two- and three-layer networks of at most 64 nodes per layer (the shapes the single-wavefront kernel
    serves) with activations, cost, batch size, momentum and both decays drawn at random: losses, accuracies,
    class counts, predictions, weights, biases and delta windows of three epochs bit for bit against the CPU
    restatement.  Widths around the power-of-two lane groups (1, 2, 3, 17, 33, 64) are in the draw."""
    import pyglades as pg
    rng = np.random.default_rng(1000 + seed)
    widths = [1, 2, 3, 4, 5, 7, 8, 9, 16, 17, 31, 33, 48, 64]
    nl = int(rng.integers(2, 4))
    sizes = [int(rng.choice(widths)) for _ in range(nl + 1)]
    hidden = [po.TANH, po.SIGMOID, po.RELU, po.LEAKY, po.TANHP, po.SIGMOIDP, po.LINEAR]
    cost = int(rng.choice([po.REGRESSION, po.CLASSIFICATION, po.KL]))
    acts = [int(rng.choice(hidden)) for _ in range(nl - 1)] + [po.SIGMOID if cost != po.REGRESSION else int(rng.choice(hidden))]
    params = [float(rng.choice([0.0, 0.01, 0.3, 1.0])) for _ in range(nl)]
    N = int(rng.integers(5, 40))
    mb = int(rng.choice([1, 2, 3, N, N + 5]))
    kw = dict(lr=[float(rng.choice([0.01, 0.05])) for _ in range(nl)], mom=[float(rng.choice([0.0, 0.5, 0.9])) for _ in range(nl)],
              wd1=float(rng.choice([0.0, 1e-3])), wd2=float(rng.choice([0.0, 1e-3])), act_params=params, batch=mb, cost=cost)
    print("random net", seed, sizes, acts, cost, N, mb, flush=True)
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * (0.5 / np.sqrt(sizes[l]))).astype(np.float32) for l in range(nl)]
    bs = [float(np.float32(rng.normal(0, 0.1))) for _ in range(nl)]
    X = rng.random((N, sizes[0])).astype(np.float32)
    Y = (rng.random((N, sizes[-1])) * 0.98 + 0.01).astype(np.float32)
    o = po.ExactNet(po.make_spec(sizes, acts, **kw))
    net = pg.Net(pg.make_spec(sizes, acts, mode=pg.MODE_EXACT, **kw))
    for l in range(nl):
        o.set_weights(l, Ws[l]); o.set_bias(l, bs[l]); net.set_params(l, Ws[l], bs[l])
    net.set_dataset(X, Y)
    E = 3
    om = [o.epoch(X, Y) for _ in range(E)]
    ms, preds = net.run_epochs_exact(E, want_preds=True)
    assert bits_equal([m[0] for m in ms], [m.loss for m, _ in om])
    assert bits_equal([m[1] for m in ms], [m.accuracy for m, _ in om])
    assert [m[2] for m in ms] == [m.correct for m, _ in om]
    assert bits_equal(preds, om[-1][1])
    for l in range(nl):
        W, b = net.get_params(l)
        assert bits_equal(W, o.get_weights(l)), l
        assert bits_equal(np.float32(b), o.get_bias(l)), l
        sa, sb = net.get_state(l)
        wa, wb = o.get_window(l)
        assert bits_equal(sa, wa) and bits_equal(sb, wb), l
    # a test pass over the same rows leaves everything as it is and reports the same figures as the restatement's
    mt, _ = net.run_epochs_exact(1, train=False)
    ot, _ = o.epoch(X, Y, train=False)
    assert bits_equal([mt[0][0]], [ot.loss]) and mt[0][2] == ot.correct
    net.close()


def test_network_too_large_for_lds_keeps_its_state_in_global_memory():
    """1100-40-3: three floats per edge are 529 KB, more than a compute unit's LDS, so weights and
    delta windows stay in global memory (L2) and every phase ends with a full barrier; alone and as
    three networks in one launch, bit for bit against the CPU restatement."""
    import pyglades as pg
    rng = np.random.default_rng(17)
    sizes, N, mb, E = [1100, 40, 3], 9, 4, 3
    acts = [po.TANH, po.SIGMOID]
    ospec = po.make_spec(sizes, acts, lr=0.001, mom=0.5, wd2=0.001, batch=mb, cost=po.CLASSIFICATION)
    gspec = pg.make_spec(sizes, acts, lr=0.001, mom=0.5, wd2=0.001, batch=mb, cost=pg.CLASSIFICATION, mode=pg.MODE_EXACT)
    X = rng.random((N, sizes[0])).astype(np.float32)
    Y = (np.eye(3, dtype=np.float32)[rng.integers(0, 3, N)] * 0.98 + 0.01).astype(np.float32)
    nets, want = [], []
    for k in range(4):
        Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * (0.5 / np.sqrt(sizes[l]))).astype(np.float32) for l in range(2)]
        o = po.ExactNet(ospec)
        g = pg.Net(gspec)
        for l in range(2):
            o.set_weights(l, Ws[l]); o.set_bias(l, 0.01 * l)
            g.set_params(l, Ws[l], 0.01 * l)
        g.set_dataset(X, Y)
        oms = [o.epoch(X, Y)[0] for _ in range(E)]
        nets.append(g)
        want.append((o, oms))
    got = [nets[0].run_epochs_exact(E)[0]] + pg.run_epochs_exact_multi(nets[1:], E)
    for g, (o, oms), ms in zip(nets, want, got):
        assert bits_equal([m[0] for m in ms], [m.loss for m in oms])
        assert [m[2] for m in ms] == [m.correct for m in oms]
        for l in range(2):
            W, b = g.get_params(l)
            assert bits_equal(W, o.get_weights(l)), l
            s, t = g.get_state(l)
            os_, ot = o.get_window(l)
            assert bits_equal(s, os_) and bits_equal(t, ot), l
        assert bits_equal(g.get_params(1)[1][0], o.get_bias(1))
        g.close()


def test_error_paths():
    import pyglades as pg
    with pytest.raises(pg.GladesHipError):   # BATCH_FULL = 0 is "row % 0" in the reference
        pg.Net(pg.make_spec([2, 2, 1], [0, 0], batch=0, mode=pg.MODE_EXACT))
    with pytest.raises(pg.GladesHipError):
        pg.Net(pg.make_spec([2, 0, 1], [0, 0], batch=1, mode=pg.MODE_EXACT))
    net = pg.Net(pg.make_spec([2, 2, 1], [0, 0], batch=1, mode=pg.MODE_EXACT))
    with pytest.raises(pg.GladesHipError):   # no dataset yet
        net.run_epochs_exact(1)
    with pytest.raises(pg.GladesHipError):   # wrong mode
        net.train_step(0, 1)
    net.close()


def test_a_crowded_launch_equals_the_solo_runs():
    """More than 2048 small networks in one launch run the instantiation with the smaller register budget
    (four wavefronts per SIMD): 2100 copies of four differently initialised networks, every one of which
    must end bit for bit where its solo run (the other instantiation) ends."""
    import pyglades as pg
    c = load_case("window_4_5_3_1")
    rng = np.random.default_rng(22)
    K, E, V = 2100, 3, 4
    variants = [[(c["W0"][l] + rng.normal(0, 0.05, c["W0"][l].shape)).astype(np.float32) for l in range(c["nl"])] for _ in range(V)]
    want, want_W = [], []
    for Ws in variants:
        n = gpu_net(c)
        for l in range(c["nl"]):
            n.set_params(l, Ws[l], c["bias0"][l])
        want.append(n.run_epochs_exact(E)[0])
        want_W.append([n.get_params(l) for l in range(c["nl"])])
        n.close()
    group = []
    for k in range(K):
        n = gpu_net(c)
        for l in range(c["nl"]):
            n.set_params(l, variants[k % V][l], c["bias0"][l])
        group.append(n)
    got = pg.run_epochs_exact_multi(group, E)
    assert all(got[k] == want[k % V] for k in range(K))
    for k in list(range(0, K, 97)) + [K - 1]:
        for l in range(c["nl"]):
            W, b = group[k].get_params(l)
            assert np.array_equal(W, want_W[k % V][l][0]) and np.array_equal(b, want_W[k % V][l][1]), (k, l)
    for n in group:
        n.close()


def test_many_networks_in_one_launch_equal_their_solo_runs():
    """ghip_net_run_epochs_exact_multi: one workgroup per network; every network ends exactly where
    it ends when it runs alone (metrics of every epoch, weights, biases, delta windows)."""
    import pyglades as pg
    c = load_case("window_4_5_3_1")
    rng = np.random.default_rng(21)
    K, E = 7, 5
    solo, group = [], []
    for k in range(K):
        Ws = [(c["W0"][l] + rng.normal(0, 0.05, c["W0"][l].shape)).astype(np.float32) for l in range(c["nl"])]
        for dst in (solo, group):
            n = gpu_net(c)
            for l in range(c["nl"]):
                n.set_params(l, Ws[l], c["bias0"][l])
            dst.append(n)
    want = [n.run_epochs_exact(E)[0] for n in solo]
    got = pg.run_epochs_exact_multi(group, E)
    assert got == want
    assert len({tuple(m) for ms in got for m in ms}) > K      # the networks really differ
    for a, b in zip(solo, group):
        for l in range(c["nl"]):
            Wa, ba = a.get_params(l); Wb, bb = b.get_params(l)
            assert np.array_equal(Wa, Wb) and np.array_equal(ba, bb)
            sa, sb = a.get_state(l), b.get_state(l)
            assert np.array_equal(sa[0], sb[0]) and np.array_equal(sa[1], sb[1])
    # every network stops on its own: in a test pass (weights fixed) those at or above the target
    # leave after one epoch, the others use all three
    fresh = []
    for k in range(K):
        n = gpu_net(c)
        for l in range(c["nl"]):
            W, b = solo[k].get_params(l)
            n.set_params(l, W, b)
        fresh.append(n)
    alone = [n.run_epochs_exact(1, train=False)[0][0][1] for n in fresh]
    target = float(np.sort(alone)[K // 2])
    test_pass = pg.run_epochs_exact_multi(fresh, 3, train=False, stop_accuracy=target)
    assert [len(ms) for ms in test_pass] == [1 if a >= target else 3 for a in alone]
    assert 1 in [len(ms) for ms in test_pass] and 3 in [len(ms) for ms in test_pass]
    with pytest.raises(pg.GladesHipError):
        pg.run_epochs_exact_multi([group[0], group[0]], 1)
    for n in solo + group + fresh:
        n.close()


# Which kernel a launch runs follows from the network and the launch (ghip_launch_exact): one case per
# instantiation, named for it, each bit for bit against the CPU restatement.
#   exact_wave_kernel<layers 2|3, wavefronts per SIMD 2|4>: two or three weight layers, no layer wider than 64, no
#       dropout state; the 4-per-SIMD build when one launch carries more than 2048 networks
#   exact_kernel<state in LDS, dropout, layers 2|3|any, at most 64|1024 threads>: everything else
INSTANTIATIONS = [
    # name,                                sizes,              mb, dropout, networks in the launch
    ("wave_2_layers",                      [5, 7, 3],           3, False, 1),
    ("wave_3_layers",                      [6, 9, 5, 2],        1, False, 1),
    ("wave_2_layers_crowded",              [3, 4, 2],           2, False, 2060),
    ("wave_3_layers_crowded",              [3, 4, 3, 2],        4, False, 2060),
    ("general_2_layers_64_threads_drop",   [6, 8, 2],           3, True, 1),
    ("general_3_layers_64_threads_drop",   [5, 7, 6, 4],        2, True, 1),
    ("general_2_layers_wide",              [70, 100, 3],        4, False, 1),
    ("general_3_layers_wide",              [20, 80, 66, 2],     1, False, 1),
    ("general_3_layers_wide_drop",         [20, 80, 66, 2],     3, True, 1),
    ("general_1_layer",                    [9, 4],              2, False, 1),
    ("general_4_layers",                   [8, 7, 6, 5, 3],     3, False, 1),
    ("general_4_layers_drop",              [8, 7, 6, 5, 3],     1, True, 1),
]


@pytest.mark.parametrize("name,sizes,mb,drop,count", INSTANTIATIONS, ids=[c[0] for c in INSTANTIATIONS])
def test_each_kernel_instantiation(name, sizes, mb, drop, count):
    import pyglades as pg
    print("instantiation", name, flush=True)
    rng = np.random.default_rng(sum(map(ord, name)))
    nl, N, E = len(sizes) - 1, 11, 3
    acts = [po.TANH, po.SIGMOID, po.RELU, po.LEAKY][:nl - 1] + [po.SIGMOID]
    kw = dict(lr=0.01, mom=0.5, wd1=1e-3, wd2=1e-3, act_params=[0.0, 0.0, 0.0, 0.05][:nl - 1] + [0.0], batch=mb, cost=po.CLASSIFICATION)
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * (0.6 / np.sqrt(sizes[l]))).astype(np.float32) for l in range(nl)]
    bs = [float(np.float32(rng.normal(0, 0.1))) for _ in range(nl)]
    X = rng.random((N, sizes[0])).astype(np.float32)
    Y = (rng.random((N, sizes[-1])) * 0.98 + 0.01).astype(np.float32)
    masks = None
    if drop:   # a third of the nodes of every input and hidden layer, never a whole layer of a row
        masks = (rng.random((E, N, sum(sizes[:-1]))) < 0.33).astype(np.uint8)
        off = 0
        for l in range(nl):
            masks[:, :, off] = 0
            off += sizes[l]
    o = po.ExactNet(po.make_spec(sizes, acts, **kw))
    for l in range(nl):
        o.set_weights(l, Ws[l]); o.set_bias(l, bs[l])
    om = [o.epoch(X, Y, masks=None if masks is None else masks[e]) for e in range(E)]
    nets = []
    for _ in range(min(count, 3) if count > 1 else 1):   # of a crowded launch the first three are compared ...
        n = pg.Net(pg.make_spec(sizes, acts, mode=pg.MODE_EXACT, **kw))
        for l in range(nl):
            n.set_params(l, Ws[l], bs[l])
        n.set_dataset(X, Y)
        nets.append(n)
    if count > 1:
        fill = []
        for _ in range(count - len(nets)):                # ... the others only fill the launch
            n = pg.Net(pg.make_spec(sizes, acts, mode=pg.MODE_EXACT, **kw))
            for l in range(nl):
                n.set_params(l, Ws[l], bs[l])
            n.set_dataset(X, Y)
            fill.append(n)
        got = pg.run_epochs_exact_multi(nets + fill, E)
        ms_all = got[:len(nets)]
        preds = None
    else:
        fill = []
        if drop:
            nets[0].set_dropout_masks(masks)
        ms, preds = nets[0].run_epochs_exact(E, want_preds=True)
        ms_all = [ms]
    for ms in ms_all:
        assert bits_equal([m[0] for m in ms], [m.loss for m, _ in om])
        assert bits_equal([m[1] for m in ms], [m.accuracy for m, _ in om])
        assert [m[2] for m in ms] == [m.correct for m, _ in om]
    if preds is not None:
        assert bits_equal(preds, om[-1][1])
    for n in nets:
        for l in range(nl):
            W, b = n.get_params(l)
            assert bits_equal(W, o.get_weights(l)), l
            assert bits_equal(np.float32(b), o.get_bias(l)), l
            if not drop:
                sa, sb = n.get_state(l)
                wa, wb = o.get_window(l)
                assert bits_equal(sa, wa) and bits_equal(sb, wb), l
    # the accuracy stop inside the launch: the first epoch at or above the bar is the last one run
    # (wide layers overflow the reference's doubling accumulator to NaN within an epoch, bit for bit here too: no bar to reach)
    if count == 1 and not drop and np.isfinite([m[1] for m in ms_all[0]]).all():
        acc = [m[1] for m in ms_all[0]]
        n2 = pg.Net(pg.make_spec(sizes, acts, mode=pg.MODE_EXACT, **kw))
        for l in range(nl):
            n2.set_params(l, Ws[l], bs[l])
        n2.set_dataset(X, Y)
        bar = float(acc[1])
        stopped, _ = n2.run_epochs_exact(E, stop_accuracy=bar)
        assert len(stopped) == next(e for e in range(E) if acc[e] >= bar) + 1
        n2.close()
    for n in nets + fill:
        n.close()
