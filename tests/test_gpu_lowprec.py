"""bf16 training and e4m3 inference paths on the GPU against fp32.

Tolerances (stated where used):
* bf16 training against the fp32 canonical run on the same arrays: loss within 2e-2 relative at every
  step; top-1 agreement of the two trained networks >= 99.5 % over ALL held-out rows.
* bf16 / e4m3 inference against the fp32 forward on the same (for e4m3: the dequantised) weights:
  top-1 agreement >= 99.5 % over ALL rows, on networks trained on separable classes (Gaussian
  clusters), where every row has a class to agree on.  No row is filtered out anywhere.
* e4m3 logits: <= 6e-2 relative RMS against the fp32 forward on the dequantised weights for the
  4-layer network (every e4m3 rounding of an activation has a relative RMS error of 2^-4/sqrt(3) =
  3.6 % at the bottom of a binade and 1.8 % at its top, about 2.7 % on average, and the four
  quantisation points of such a pass add up to sqrt(4) x 2.7 % = 5.4 %: what the format costs, which
  the restated quantised pipeline shows as well), <= 5e-2 for 3 layers; against the restated
  quantised pipeline itself <= 2e-2 (typically 1e-3).  e4m3 codes and scales are bit-exact against
  the restated quantiser.
* on networks with random weights and hundreds of near-flat classes (the benchmark's literal inputs)
  top-1 agreement is limited by the classes' margins, not by the arithmetic: those figures are
  printed, and bounded from below where the bound can fail, never filtered."""
import numpy as np
import pytest

import pyoracle as po

pytestmark = pytest.mark.gpu


def teacher_labels(rng, X, n_cls):
    T = rng.standard_normal((X.shape[1], n_cls)).astype(np.float32)
    return np.eye(n_cls, dtype=np.float32)[(X @ T).argmax(1)]


def test_bf16_training_tracks_fp32():
    """Loss within 2e-2 relative of the fp32 CPU run at every step.  After 6 steps on 256 near-flat
    classes most rows have no clear winner, so top-1 agreement is only bounded by 97 % here (over all
    rows); the 99.5 % bar is held on trained networks below."""
    import pyglades as pg
    print("bf16 training vs fp32", flush=True)
    rng = np.random.default_rng(21)
    sizes, acts = [256, 512, 256, 256], [po.RELU, po.RELU, po.SOFTMAX]
    B, steps = 256, 6
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * np.sqrt(2.0 / sizes[l])).astype(np.float32) for l in range(3)]
    X = rng.standard_normal((B * steps, 256)).astype(np.float32)
    Y = teacher_labels(rng, X, 256)
    kw = dict(lr=0.02, mom=0.9, wd2=1e-4, cost=po.CLASSIFICATION)
    o = po.CanonNet(po.make_spec(sizes, acts, **kw))
    g = pg.Net(pg.make_spec(sizes, acts, mode=pg.MODE_CANONICAL, dtype=pg.BF16, **kw))
    for l in range(3):
        o.set_params(l, Ws[l]); g.set_params(l, Ws[l])
    g.set_dataset(X, Y)
    po.lib().go_set_threads(8)
    for s in range(steps):
        mo = o.step(X[s * B:(s + 1) * B], Y[s * B:(s + 1) * B])
        mg = g.train_step(s * B, B)
        assert abs(mg.loss - mo.loss) <= 2e-2 * abs(mo.loss), (s, mg.loss, mo.loss)
    lo, lg = o.forward(X[:256]), g.forward(X[:256])
    print("top-1 agreement, all rows", (lo.argmax(1) == lg.argmax(1)).mean(), flush=True)
    assert (lo.argmax(1) == lg.argmax(1)).mean() >= 0.97
    g.close()


@pytest.mark.parametrize("acts,steps,mom", [([po.TANH, po.RELU, po.SOFTMAX], 1, 0.0), ([po.RELU, po.SIGMOID, po.SOFTMAX], 3, 0.9)])
def test_bf16_steps_match_the_bf16_pipeline_statement(acts, steps, mom):
    """Against a numpy statement of the same pipeline (same rounding points, exact products, wide
    sums) the kernels may differ only by fp32 accumulation order and the rare bf16 rounding flip
    that causes: accumulated update within 1e-2 of its Frobenius norm (measured 2e-3..4e-3; bf16 against fp32 is 5e-2), losses within 1e-4.
    A wrong tile index, a wrong transposed shadow (W^T, H^T, D^T) or a missing term fails this by
    orders of magnitude."""
    import pyglades as pg
    from helpers import bf16_pipeline_steps
    print("bf16 pipeline", acts, steps, flush=True)
    rng = np.random.default_rng(5)
    sizes = [512, 256, 512, 256]
    B = 512
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * np.sqrt(1.0 / sizes[l])).astype(np.float32) for l in range(3)]
    bs = [(rng.standard_normal(sizes[l + 1]) * 0.05).astype(np.float32) for l in range(3)]
    X = rng.standard_normal((B * steps, 512)).astype(np.float32)
    Y = teacher_labels(rng, X, 256)
    lr, wd2 = 0.5, 1e-3
    g = pg.Net(pg.make_spec(sizes, acts, lr=lr, mom=mom, wd2=wd2, cost=pg.CLASSIFICATION, mode=pg.MODE_CANONICAL, dtype=pg.BF16))
    for l in range(3):
        g.set_params(l, Ws[l], bs[l])
    g.set_dataset(X, Y)
    losses = [g.train_step(s * B, B).loss for s in range(steps)]
    Wm, bm, ref_losses = bf16_pipeline_steps(sizes, acts, Ws, bs, X, Y, B, steps, lr, mom, wd2)
    np.testing.assert_allclose(losses, ref_losses, rtol=1e-4)
    for l in range(3):
        Wg, bg = g.get_params(l)
        fro = np.linalg.norm(Wg - Wm[l]) / np.linalg.norm(Wm[l] - Ws[l])
        frob = np.linalg.norm(bg - bm[l]) / np.linalg.norm(bm[l] - bs[l])
        print("layer", l, "update error vs pipeline statement", fro, frob, flush=True)
        assert fro <= 1e-2 and frob <= 1e-2, (l, fro, frob)
    g.close()


def test_fp8_quantiser_bit_exact_and_forward():
    import pyglades as pg
    print("fp8 inference", flush=True)
    rng = np.random.default_rng(9)
    sizes, acts = [512, 256, 512, 256], [po.RELU, po.RELU, po.RELU]
    B = 256
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) / np.sqrt(sizes[l])).astype(np.float32) for l in range(3)]
    X = po.bf16_round(rng.standard_normal((B, 512)).astype(np.float32))
    g = pg.Net(pg.make_spec(sizes, acts, mode=pg.MODE_CANONICAL, dtype=pg.FP8_INFER))
    for l in range(3):
        g.set_params(l, Ws[l])
    codes, scales = g.quantize_fp8()
    for l in range(3):
        q, s = po.e4m3_quant_rows(Ws[l])
        assert np.array_equal(codes[l], q), l          # byte work: bit exact
        assert np.array_equal(scales[l].view(np.uint32), s.view(np.uint32)), l
    spec = po.make_spec(sizes, acts)
    ca = po.CanonNet(spec)
    for l in range(3):
        ca.set_params(l, po.e4m3_table()[codes[l]] * scales[l][:, None])
    ref = ca.forward(X)
    # both ways of re-quantising the activations between layers: a power-of-two scale per token and 32 units
    # (made in the products' epilogues), one fp32 scale per token (a kernel of its own)
    for mode in (pg.FP8_ACT_BLOCK32, pg.FP8_ACT_PER_TOKEN):
        g.set_fp8_activation_scaling(mode)
        out = g.forward(X)
        emu = po.fp8_forward(spec, codes, scales, X, block32=(mode == pg.FP8_ACT_BLOCK32))
        # same quantised pipeline, only the fp32 accumulation order differs (plus re-quantisation
        # flips it can cause): 2e-2 relative RMS, typically ~1e-3
        err = np.sqrt(np.mean((out - emu) ** 2)) / np.sqrt(np.mean(emu ** 2))
        print("activation scaling", mode, "vs restated pipeline", err, flush=True)
        assert err < 2e-2, (mode, err)
        err = np.sqrt(np.mean((out - ref) ** 2)) / np.sqrt(np.mean(ref ** 2))
        print("activation scaling", mode, "vs fp32 forward on the dequantised weights", err, flush=True)
        assert err < 5e-2, (mode, err)
        # random weights, 256 near-flat classes: printed, not a tolerance (see the trained networks below)
        print("e4m3 top-1 agreement on random weights, all rows", (out.argmax(1) == ref.argmax(1)).mean(), flush=True)
    g.close()


def test_block32_quantiser_bit_exact():
    """The block-scaled activation quantiser on its own (the device function the products' epilogues apply):
    codes and E8M0 bytes bit for bit against the restatement, on blocks of very different magnitudes, an
    all-zero block, a ragged last block and the rule's edge (largest magnitude exactly 448 2^k, and one
    bf16 step above)."""
    import pyglades as pg
    rng = np.random.default_rng(77)
    rows, cols = 129, 32 * 11 + 5
    mag = 10.0 ** rng.uniform(-8, 8, (rows, (cols + 31) // 32))
    x = po.bf16_round((rng.standard_normal((rows, cols)) * np.repeat(mag, 32, axis=1)[:, :cols]).astype(np.float32))
    x[3, 32:64] = 0.0
    x[4, :] = 0.0
    x[5, 0:32] = 0.0; x[5, 7] = 448.0 * 2.0 ** -5
    x[6, 0:32] = 0.0; x[6, 7] = -450.0 * 2.0 ** -5
    codes, scales = pg.quantize_rows_e4m3_block32(x)
    rq, rs = po.e4m3_quant_rows_block32(x)
    assert np.array_equal(scales, rs)
    assert np.array_equal(codes, rq)


def test_lowprec_state_rules():
    import pyglades as pg
    g = pg.Net(pg.make_spec([256, 256, 256], [po.RELU, po.RELU], mode=pg.MODE_CANONICAL, dtype=pg.FP8_INFER))
    with pytest.raises(pg.GladesHipError):   # inference only
        g.train_step(0, 256)
    with pytest.raises(pg.GladesHipError):   # not quantised yet
        g.forward(np.zeros((256, 256), np.float32))
    g.close()


@pytest.mark.parametrize("B", [200, 192])
def test_bf16_steps_off_the_tile_grid(B):
    """Layer widths and batches that are no multiples of the 256-wide tiles: the library rounds them up
    on the device and keeps what it adds at zero, so the steps are those of the network as given.
    Same statement and tolerances as for the shapes on the grid above.  Sigmoid and tanh hidden layers:
    sigmoid(0) = 0.5, so a padded unit that were not held at zero would show at once.  Rows start at
    0, B, 2B: with B = 192 the first layer's gradient reads the transposed table in place, with 200 a
    copy made per step."""
    import pyglades as pg
    from helpers import bf16_pipeline_steps
    print("bf16 off-grid", B, flush=True)
    rng = np.random.default_rng(17)
    sizes, acts = [100, 300, 130, 70], [po.SIGMOID, po.TANH, po.SOFTMAX]
    steps = 3
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * np.sqrt(1.0 / sizes[l])).astype(np.float32) for l in range(3)]
    bs = [(rng.standard_normal(sizes[l + 1]) * 0.05).astype(np.float32) for l in range(3)]
    X = rng.standard_normal((B * steps, sizes[0])).astype(np.float32)
    Y = teacher_labels(rng, X, sizes[-1])
    lr, mom, wd2 = 0.5, 0.9, 1e-3
    g = pg.Net(pg.make_spec(sizes, acts, lr=lr, mom=mom, wd2=wd2, cost=pg.CLASSIFICATION, mode=pg.MODE_CANONICAL, dtype=pg.BF16))
    for l in range(3):
        g.set_params(l, Ws[l], bs[l])
        Wb, bb = g.get_params(l)
        assert np.array_equal(Wb, Ws[l]) and np.array_equal(bb, bs[l])   # through the padded copy and back
    g.set_dataset(X, Y)
    losses = [g.train_step(s * B, B).loss for s in range(steps)]
    Wm, bm, ref_losses = bf16_pipeline_steps(sizes, acts, Ws, bs, X, Y, B, steps, lr, mom, wd2)
    np.testing.assert_allclose(losses, ref_losses, rtol=1e-4)
    for l in range(3):
        Wg, bg = g.get_params(l)
        assert Wg.shape == Ws[l].shape and bg.shape == bs[l].shape
        fro = np.linalg.norm(Wg - Wm[l]) / np.linalg.norm(Wm[l] - Ws[l])
        frob = np.linalg.norm(bg - bm[l]) / np.linalg.norm(bm[l] - bs[l])
        print("layer", l, "update error vs pipeline statement", fro, frob, flush=True)
        assert fro <= 1e-2 and frob <= 1e-2, (l, fro, frob)
    # forward of rows handed over from the host and of rows of the table: the same outputs, of the net's own width
    out_h = g.forward(X[:B])
    assert out_h.shape == (B, sizes[-1])
    np.testing.assert_allclose(out_h.sum(1), 1.0, rtol=1e-5)   # softmax over the 70 real classes only
    m = g.eval_resident(0, B)
    loss_h = float(-np.log(np.maximum((out_h * Y[:B]).sum(1), 1e-30)).mean())
    assert abs(m.loss - loss_h) <= 1e-5 * loss_h, (m.loss, loss_h)
    assert m.correct == int((out_h.argmax(1) == Y[:B].argmax(1)).sum())
    g.close()


@pytest.mark.parametrize("seed", range(5))
def test_low_precision_random_shapes(seed):
    """Widths from 1 to 700 and batches from 1 to 600 drawn at random, two or three layers, random hidden
    activations: two bf16 training steps against the pipeline statement (losses 1e-4, updates 1e-2 of their
    norm) and an e4m3 forward pass of the same shape against the restated quantised pipeline (2e-2 relative
    RMS; codes and scales bit for bit)."""
    import pyglades as pg
    from helpers import bf16_pipeline_steps
    rng = np.random.default_rng(500 + seed)
    nl = int(rng.integers(2, 4))
    sizes = [int(rng.integers(1, 701)) for _ in range(nl)] + [int(rng.integers(2, 300))]
    acts = [int(rng.choice([po.TANH, po.RELU, po.SIGMOID])) for _ in range(nl - 1)] + [po.SOFTMAX]
    B = int(rng.integers(1, 601))
    print("random low-precision shape", seed, sizes, acts, B, flush=True)
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * np.sqrt(1.0 / sizes[l])).astype(np.float32) for l in range(nl)]
    bs = [(rng.standard_normal(sizes[l + 1]) * 0.05).astype(np.float32) for l in range(nl)]
    X = rng.standard_normal((2 * B, sizes[0])).astype(np.float32)
    Y = teacher_labels(rng, X, sizes[-1])
    lr, mom, wd2 = 0.3, 0.9, 1e-3
    g = pg.Net(pg.make_spec(sizes, acts, lr=lr, mom=mom, wd2=wd2, cost=pg.CLASSIFICATION, mode=pg.MODE_CANONICAL, dtype=pg.BF16))
    for l in range(nl):
        g.set_params(l, Ws[l], bs[l])
    g.set_dataset(X, Y)
    losses = [g.train_step(s_ * B, B).loss for s_ in range(2)]
    Wm, bm, ref_losses = bf16_pipeline_steps(sizes, acts, Ws, bs, X, Y, B, 2, lr, mom, wd2)
    np.testing.assert_allclose(losses, ref_losses, rtol=1e-4)
    for l in range(nl):
        Wg, bg = g.get_params(l)
        fro = np.linalg.norm(Wg - Wm[l]) / np.linalg.norm(Wm[l] - Ws[l])
        frob = np.linalg.norm(bg - bm[l]) / np.linalg.norm(bm[l] - bs[l])
        assert fro <= 1e-2 and frob <= 1e-2, (l, fro, frob)
    g.close()
    # the same shape as an e4m3 inference network (ReLU / sigmoid hidden layers, linear output)
    facts = [po.RELU if a == po.TANH else a for a in acts[:-1]] + [po.LINEAR]
    q = pg.Net(pg.make_spec(sizes, facts, act_params=1.0, mode=pg.MODE_CANONICAL, dtype=pg.FP8_INFER))
    for l in range(nl):
        q.set_params(l, Ws[l])
    codes, scales = q.quantize_fp8()
    for l in range(nl):
        c, sc = po.e4m3_quant_rows(Ws[l])
        assert np.array_equal(codes[l], c) and np.array_equal(scales[l].view(np.uint32), sc.view(np.uint32)), l
    Xq = po.bf16_round(X[:B])
    for mode in (pg.FP8_ACT_BLOCK32, pg.FP8_ACT_PER_TOKEN):
        q.set_fp8_activation_scaling(mode)
        out = q.forward(Xq)
        emu = po.fp8_forward(po.make_spec(sizes, facts, act_params=1.0), codes, scales, Xq, block32=(mode == pg.FP8_ACT_BLOCK32))
        err = np.sqrt(np.mean((out - emu) ** 2)) / max(np.sqrt(np.mean(emu ** 2)), 1e-30)
        assert err < 2e-2, (mode, err)
    q.close()


def test_bf16_off_grid_state_round_trip():
    """Momentum of a padded network out and in again (what a checkpoint does): two copies of a network off the
    tile grid take two steps; one hands its parameters and optimiser state to the host and takes them
    back (setting parameters clears the momentum, so the state has to arrive for the next step to agree);
    after a third step both hold the same bits."""
    import pyglades as pg
    print("bf16 off-grid state", flush=True)
    rng = np.random.default_rng(31)
    sizes, acts, B = [100, 300, 70], [po.RELU, po.SOFTMAX], 200
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * np.sqrt(2.0 / sizes[l])).astype(np.float32) for l in range(2)]
    X = rng.standard_normal((3 * B, sizes[0])).astype(np.float32)
    Y = teacher_labels(rng, X, sizes[-1])
    nets = []
    for _ in range(2):
        g = pg.Net(pg.make_spec(sizes, acts, lr=0.1, mom=0.9, wd2=1e-4, cost=pg.CLASSIFICATION, mode=pg.MODE_CANONICAL, dtype=pg.BF16))
        for l in range(2):
            g.set_params(l, Ws[l])
        g.set_dataset(X, Y)
        for s_ in range(2):
            g.train_step(s_ * B, B)
        nets.append(g)
    a, b = nets
    for l in range(2):
        W, bias = b.get_params(l)
        vW, vb = b.get_state(l)
        assert vW.shape == Ws[l].shape and vb.shape == (sizes[l + 1],) and np.any(vW != 0) and np.any(vb != 0)
        b.set_params(l, W, bias)
        b.set_state(l, vW, vb)
    la, lb = a.train_step(2 * B, B).loss, b.train_step(2 * B, B).loss
    assert la == lb
    for l in range(2):
        (Wa, ba), (Wb, bb) = a.get_params(l), b.get_params(l)
        assert np.array_equal(Wa, Wb) and np.array_equal(ba, bb), l
        (va, vba), (vb_, vbb) = a.get_state(l), b.get_state(l)
        assert np.array_equal(va, vb_) and np.array_equal(vba, vbb), l
    a.close(); b.close()


def test_bf16_pass_with_a_short_last_batch():
    """One training pass over 700 rows in batches of 256: 256, 256 and 188 rows.  The short batch follows
    two full ones in the same buffers, whose rows past 188 then hold the earlier batches' deltas unless
    the step clears them.  Against the pipeline statement run as 2 + 1 steps (no momentum, so the
    statement can be restarted from the weights), and the pass's loss against the three batches' own."""
    import pyglades as pg
    from helpers import bf16_pipeline_steps
    print("bf16 ragged pass", flush=True)
    rng = np.random.default_rng(23)
    sizes, acts = [256, 512, 256], [po.RELU, po.SOFTMAX]
    N, B = 700, 256
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * np.sqrt(1.0 / sizes[l])).astype(np.float32) for l in range(2)]
    bs = [(rng.standard_normal(sizes[l + 1]) * 0.05).astype(np.float32) for l in range(2)]
    X = rng.standard_normal((N, sizes[0])).astype(np.float32)
    Y = teacher_labels(rng, X, sizes[-1])
    lr, wd2 = 0.5, 1e-3
    g = pg.Net(pg.make_spec(sizes, acts, lr=lr, wd2=wd2, cost=pg.CLASSIFICATION, mode=pg.MODE_CANONICAL, dtype=pg.BF16))
    for l in range(2):
        g.set_params(l, Ws[l], bs[l])
    g.set_dataset(X, Y)
    m = g.run_epoch_canonical(B, train=True)
    W1, b1, l1 = bf16_pipeline_steps(sizes, acts, Ws, bs, X[:512], Y[:512], B, 2, lr, 0.0, wd2)
    W2, b2, l2 = bf16_pipeline_steps(sizes, acts, W1, b1, X[512:], Y[512:], N - 512, 1, lr, 0.0, wd2)
    ref_loss = (l1[0] * 256 + l1[1] * 256 + l2[0] * (N - 512)) / N
    assert abs(m.loss - ref_loss) <= 1e-4 * ref_loss, (m.loss, ref_loss)
    for l in range(2):
        Wg, bg = g.get_params(l)
        fro = np.linalg.norm(Wg - W2[l]) / np.linalg.norm(W2[l] - Ws[l])
        frob = np.linalg.norm(bg - b2[l]) / np.linalg.norm(b2[l] - bs[l])
        print("layer", l, "update error vs pipeline statement", fro, frob, flush=True)
        assert fro <= 1e-2 and frob <= 1e-2, (l, fro, frob)
    g.close()


def test_fp8_forward_off_the_tile_grid():
    """e4m3 inference on widths and a batch off the 256 grid: codes and scales of the weights as given
    (bit exact against the restated quantiser), outputs against the restated quantised pipeline on the
    network as given (<= 2e-2 relative RMS, as on the grid).  Sigmoid hidden layers: a padded unit left
    at sigmoid(0) = 0.5 could set a row's scale."""
    import pyglades as pg
    print("fp8 off-grid", flush=True)
    rng = np.random.default_rng(29)
    sizes, acts = [300, 500, 200, 70], [po.SIGMOID, po.RELU, po.LINEAR]
    B = 100
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) / np.sqrt(sizes[l])).astype(np.float32) for l in range(3)]
    X = po.bf16_round(rng.standard_normal((B, sizes[0])).astype(np.float32) * np.float32(0.05))
    g = pg.Net(pg.make_spec(sizes, acts, act_params=1.0, mode=pg.MODE_CANONICAL, dtype=pg.FP8_INFER))
    for l in range(3):
        g.set_params(l, Ws[l])
    codes, scales = g.quantize_fp8()
    for l in range(3):
        q, s = po.e4m3_quant_rows(Ws[l])
        assert np.array_equal(codes[l], q), l
        assert np.array_equal(scales[l].view(np.uint32), s.view(np.uint32)), l
    spec = po.make_spec(sizes, acts, act_params=1.0)
    for mode in (pg.FP8_ACT_PER_TOKEN, pg.FP8_ACT_BLOCK32):
        g.set_fp8_activation_scaling(mode)
        out = g.forward(X)
        assert out.shape == (B, sizes[-1])
        emu = po.fp8_forward(spec, codes, scales, X, block32=(mode == pg.FP8_ACT_BLOCK32))
        err = np.sqrt(np.mean((out - emu) ** 2)) / np.sqrt(np.mean(emu ** 2))
        print("off-grid e4m3 vs restated pipeline, activation scaling", mode, err, flush=True)
        assert err < 2e-2, (mode, err)
    # the same rows as a table on the device, and its metrics pass
    Y = np.eye(sizes[-1], dtype=np.float32)[emu.argmax(1)]
    g.set_dataset(X, Y)
    m = g.run_epoch_canonical(64, train=False)   # batches of 64, 36
    assert m.correct >= 0.97 * B, m.correct
    g.close()


def test_bf16_step_at_full_tile_size():
    """Layers of 4096 with a batch of 4096 give 256 tiles of 256 x 256 per product, which is where
    the library switches from its 128 x 128 to its 256 x 256 tile (every smaller case above runs
    the small one).  One training step against the numpy statement of the bf16 pipeline (float32
    matmuls here: 137 GFLOP each): loss 1e-3, update within 1e-2 of its Frobenius norm."""
    import pyglades as pg
    from helpers import bf16_pipeline_steps
    print("bf16 full-size tile", flush=True)
    rng = np.random.default_rng(11)
    sizes, acts = [4096, 4096, 4096], [po.RELU, po.SOFTMAX]
    B = 4096
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l]), dtype=np.float32) * np.float32(np.sqrt(2.0 / sizes[l]))) for l in range(2)]
    bs = [np.zeros(sizes[l + 1], np.float32) for l in range(2)]
    X = rng.standard_normal((B, 4096), dtype=np.float32)
    Y = np.eye(4096, dtype=np.float32)[rng.integers(0, 4096, B)]
    lr = 0.5
    g = pg.Net(pg.make_spec(sizes, acts, lr=lr, cost=pg.CLASSIFICATION, mode=pg.MODE_CANONICAL, dtype=pg.BF16))
    for l in range(2):
        g.set_params(l, Ws[l], bs[l])
    g.set_dataset(X, Y)
    loss = g.train_step(0, B).loss
    Wm, bm, ref_losses = bf16_pipeline_steps(sizes, acts, Ws, bs, X, Y, B, 1, lr, 0.0, 0.0, wide=False)
    assert abs(loss - ref_losses[0]) <= 1e-3 * abs(ref_losses[0]), (loss, ref_losses)
    for l in range(2):
        Wg, bg = g.get_params(l)
        fro = np.linalg.norm(Wg - Wm[l]) / np.linalg.norm(Wm[l] - Ws[l])
        print("layer", l, "update error vs pipeline statement", fro, flush=True)
        assert fro <= 1e-2, (l, fro)
    g.close()


@pytest.mark.parametrize("kind", ["bf16", "e4m3"])
def test_full_size_forward_is_row_wise(kind):
    """At the benchmark's full shapes (bf16: 4096-4096-4096-4096-4096-1024, batch 8192; e4m3: 8192 wide,
    batch 4096) no CPU statement finishes in seconds, but the forward pass has properties that hold at
    any size: every row's outputs depend on that row alone (a row-permuted batch gives the permuted
    outputs, duplicated rows give duplicated outputs), bit for bit -- whatever tile a row lands in,
    its dot products run over K in the same order (for e4m3 the scale is per row as well) -- and a
    batch of zeros gives the activation of the bias, zero here."""
    import pyglades as pg
    print("full size", kind, flush=True)
    rng = np.random.default_rng(5)
    if kind == "bf16":
        sizes, B, dt = [4096, 4096, 4096, 4096, 4096, 1024], 8192, pg.BF16
    else:
        sizes, B, dt = [8192, 8192, 8192, 8192, 1024], 4096, pg.FP8_INFER
    nl = len(sizes) - 1
    g = pg.Net(pg.make_spec(sizes, [po.RELU] * nl, cost=pg.CLASSIFICATION, mode=pg.MODE_CANONICAL, dtype=dt))
    for l in range(nl):
        g.set_params(l, rng.standard_normal((sizes[l + 1], sizes[l]), dtype=np.float32) * np.float32(np.sqrt(2.0 / sizes[l])))
    if kind == "e4m3":
        g.quantize_fp8(want=False)
    X = rng.standard_normal((B, sizes[0]), dtype=np.float32)
    X[B // 2:B // 2 + 256] = X[:256]          # duplicated rows, a tile apart
    out = g.forward(X)
    assert np.isfinite(out).all() and (out > 0).any() and (out == 0).any()   # ReLU outputs of a live network
    assert np.array_equal(out[B // 2:B // 2 + 256], out[:256])
    perm = rng.permutation(B)
    assert np.array_equal(g.forward(X[perm]), out[perm])
    assert not np.any(g.forward(np.zeros((256, sizes[0]), np.float32)))
    g.close()


def test_bf16_and_e4m3_passes_over_the_table():
    """ghip_net_run_epoch_canonical on the low-precision paths: a bf16 training pass leaves the
    parameters of the same steps taken one by one, and an e4m3 pass only evaluates (a short last batch
    has its own test above)."""
    import pyglades as pg
    rng = np.random.default_rng(8)
    sizes, acts = [256, 512, 256], [po.RELU, po.SOFTMAX]
    B, N = 256, 768
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * np.sqrt(2.0 / sizes[l])).astype(np.float32) for l in range(2)]
    X = rng.standard_normal((N, 256)).astype(np.float32)
    Y = teacher_labels(rng, X, 256)
    kw = dict(lr=0.02, mom=0.9, wd2=1e-4, cost=po.CLASSIFICATION, mode=pg.MODE_CANONICAL)
    a = pg.Net(pg.make_spec(sizes, acts, dtype=pg.BF16, **kw))
    b = pg.Net(pg.make_spec(sizes, acts, dtype=pg.BF16, **kw))
    for n in (a, b):
        for l in range(2):
            n.set_params(l, Ws[l])
        n.set_dataset(X, Y)
    loss = correct = 0
    for r0 in range(0, N, B):
        m = a.train_step(r0, B)
        loss += m.loss * B; correct += m.correct
    mp = b.run_epoch_canonical(B)
    assert abs(mp.loss - loss / N) <= 1e-5 * abs(loss / N) and mp.correct == correct
    for l in range(2):
        assert np.array_equal(a.get_params(l)[0], b.get_params(l)[0]), l
    q = pg.Net(pg.make_spec(sizes, acts, dtype=pg.FP8_INFER, **kw))
    for l in range(2):
        q.set_params(l, Ws[l])
    q.set_dataset(X, Y)
    q.quantize_fp8(want=False)
    ev = q.run_epoch_canonical(B, train=False)
    assert 0 <= ev.correct <= N and np.isfinite(ev.loss)
    with pytest.raises(pg.GladesHipError):
        q.run_epoch_canonical(B, train=True)        # inference only
    with pytest.raises(pg.GladesHipError):
        a.run_epoch_canonical(0)
    for n in (a, b, q):
        n.close()


def test_bf16_step_reads_the_batch_from_the_transposed_table_or_transposes_it():
    """The first layer's weight gradient takes the batch transposed: as columns of the table's
    transposed copy when the batch starts on a multiple of 64 rows, from a copy made for the step
    otherwise.  The same rows at offset 0 of one table, at offset 192 and at offset 40 of another
    (488 rows, so the transposed copy's pitch is not a multiple of the batch) give bit-identical
    parameters: the products are the same, only the operand's place and pitch differ."""
    import pyglades as pg
    print("bf16 step: batch at row 0 / 192 / 40 of the table", flush=True)
    rng = np.random.default_rng(33)
    sizes, acts = [256, 256, 256], [po.RELU, po.SOFTMAX]
    B = 256
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) * np.sqrt(2.0 / sizes[l])).astype(np.float32) for l in range(2)]
    Xb = rng.standard_normal((B, 256)).astype(np.float32)
    Yb = teacher_labels(rng, Xb, 256)
    other = rng.standard_normal((488, 256)).astype(np.float32)
    results = []
    for off in (0, 192, 40):
        if off == 0:
            X, Y = Xb, Yb
        else:
            X = other.copy(); Y = teacher_labels(rng, X, 256)
            X[off:off + B] = Xb; Y[off:off + B] = Yb
        g = pg.Net(pg.make_spec(sizes, acts, mode=pg.MODE_CANONICAL, dtype=pg.BF16, lr=0.05, mom=0.9, cost=po.CLASSIFICATION))
        for l in range(2):
            g.set_params(l, Ws[l])
        g.set_dataset(X, Y)
        losses = [g.train_step(off, B).loss for _ in range(3)]
        results.append((losses, [g.get_params(l) for l in range(2)]))
        g.close()
    for losses, params in results[1:]:
        assert losses == results[0][0]
        for l in range(2):
            assert np.array_equal(params[l][0], results[0][1][l][0]), l
            assert np.array_equal(params[l][1], results[0][1][l][1]), l
    assert any(np.any(results[0][1][0][0] != Ws[0]) for _ in [0])  # the first layer did move


def _trained_pair(sizes, B, n_batches, steps, lr, seed, dtypes):
    """Networks of one shape and one initialisation trained side by side on the same Gaussian-cluster
    rows (softmax cross-entropy, momentum 0.9), one per dtype.  Returns them, the per-step metrics and
    a way to draw further rows of the same classes."""
    import pyglades as pg
    from helpers import cluster_centres, cluster_rows, he_init
    rng = np.random.default_rng(seed)
    nl = len(sizes) - 1
    acts = [pg.RELU] * (nl - 1) + [pg.SOFTMAX]
    cen = cluster_centres(rng, sizes[-1], sizes[0])
    X, Y, _ = cluster_rows(rng, cen, B * n_batches)
    Ws = he_init(rng, sizes)
    nets = []
    for dt in dtypes:
        n = pg.Net(pg.make_spec(sizes, acts, lr=lr, mom=0.9, cost=pg.CLASSIFICATION, mode=pg.MODE_CANONICAL, dtype=dt))
        for l in range(nl):
            n.set_params(l, Ws[l])
        n.set_dataset(X, Y)
        nets.append(n)
    del X, Y, Ws
    hist = []
    for s in range(steps):
        hist.append([n.train_step((s % n_batches) * B, B) for n in nets])
    return nets, hist, (lambda r, rows: cluster_rows(r, cen, rows))


def test_lowprec_inference_top1_on_a_trained_network():
    """north_star's inference criterion, all rows counted: a 512-1024-1024-256 network trained 200
    steps in fp32 on the GPU (the path that is pinned to the CPU restatement) on 256 separable
    classes; its bf16 forward, and its e4m3 forward against the fp32 forward on the dequantised
    weights, pick the same class on >= 99.5 % of 2048 held-out rows.  The fp32 side is the CPU
    restatement's forward (the reference forward)."""
    import pyglades as pg
    from helpers import rel_rms
    print("low-precision inference on a trained network", flush=True)
    sizes = [512, 1024, 1024, 256]
    (f,), hist, draw = _trained_pair(sizes, 512, 8, 200, 0.05, 17, [pg.F32])
    assert hist[-1][0].correct == 512 and hist[-1][0].loss < 0.01       # it did learn the classes
    Xt, _, cls = draw(np.random.default_rng(18), 2048)
    Xt = po.bf16_round(Xt)
    Wt = [f.get_params(l) for l in range(3)]
    f.close()
    po.lib().go_set_threads(8)
    ref = po.CanonNet(po.make_spec(sizes, [po.RELU, po.RELU, po.LINEAR], act_params=[0, 0, 1.0]))
    for l in range(3):
        ref.set_params(l, Wt[l][0], Wt[l][1])
    want = ref.forward(Xt)
    assert (want.argmax(1) == cls).mean() >= 0.995
    kw = dict(act_params=[0, 0, 1.0], cost=pg.CLASSIFICATION, mode=pg.MODE_CANONICAL)
    b = pg.Net(pg.make_spec(sizes, [pg.RELU, pg.RELU, pg.LINEAR], dtype=pg.BF16, **kw))
    for l in range(3):
        b.set_params(l, Wt[l][0], Wt[l][1])
    got = b.forward(Xt)
    b.close()
    agree = (got.argmax(1) == want.argmax(1)).mean()
    print("bf16 forward: top-1 agreement %.4f over all rows, logits rel RMS %.2e" % (agree, rel_rms(got, want)), flush=True)
    assert agree >= 0.995
    assert rel_rms(got, want) <= 1e-2        # bf16 weights and activations, fp32 sums
    q = pg.Net(pg.make_spec(sizes, [pg.RELU, pg.RELU, pg.LINEAR], dtype=pg.FP8_INFER, **kw))
    for l in range(3):
        q.set_params(l, Wt[l][0], Wt[l][1])
    codes, scales = q.quantize_fp8()
    for l in range(3):
        ref.set_params(l, po.e4m3_table()[codes[l]] * scales[l][:, None], Wt[l][1])
    want8 = ref.forward(Xt)
    for mode in (pg.FP8_ACT_BLOCK32, pg.FP8_ACT_PER_TOKEN):
        q.set_fp8_activation_scaling(mode)
        got8 = q.forward(Xt)
        agree8 = (got8.argmax(1) == want8.argmax(1)).mean()
        print("e4m3 forward, activation scaling %d: top-1 agreement %.4f over all rows, logits rel RMS %.2e" % (mode, agree8, rel_rms(got8, want8)), flush=True)
        assert agree8 >= 0.995
        assert rel_rms(got8, want8) <= 5e-2      # three quantisation points
    q.close()


def test_bf16_training_top1_on_separable_classes():
    """bf16 training against fp32 training on the GPU, same rows, same initialisation, 200 steps:
    loss within 2e-2 relative at every step and the two trained networks agree on the class of
    >= 99.5 % of 2048 held-out rows (all rows counted)."""
    import pyglades as pg
    print("bf16 vs fp32 training on separable classes", flush=True)
    (f, b), hist, draw = _trained_pair([512, 1024, 1024, 256], 512, 8, 200, 0.05, 19, [pg.F32, pg.BF16])
    for s, (mf, mb) in enumerate(hist):
        assert abs(mb.loss - mf.loss) <= 2e-2 * abs(mf.loss), (s, mb.loss, mf.loss)
    Xt, _, cls = draw(np.random.default_rng(20), 2048)
    of, ob = f.forward(Xt), b.forward(Xt)
    f.close(); b.close()
    print("fp32 accuracy %.4f, bf16 accuracy %.4f, agreement %.4f" % ((of.argmax(1) == cls).mean(), (ob.argmax(1) == cls).mean(),
                                                                    (of.argmax(1) == ob.argmax(1)).mean()), flush=True)
    assert (of.argmax(1) == cls).mean() >= 0.995
    assert (of.argmax(1) == ob.argmax(1)).mean() >= 0.995


def test_cfg4_full_size_training_bf16_against_fp32():
    """The wide benchmark network at its full size -- 4096-4096-4096-4096-4096-1024, batch 8192, both
    tile sizes and the transposed-table operand in every step -- trained its whole schedule of 200 steps in
    bf16 and, side by side, in fp32 on the GPU (the fp32 path is pinned to the CPU restatement in
    test_gpu_canonical.py): loss within 2e-2 relative at every step (measured: 1e-3 at worst, while the loss
    falls from 8.0 to 0.05), and the trained networks agree on the class of >= 99.5 % of 8192 held-out rows, all
    rows counted.  1024 separable classes (Gaussian clusters), 8 batches of 8192 rows walked 25 times, learning
    rate 0.002 with momentum 0.9 (at 0.02 the loss is below 0.03 after 30 steps and two runs' losses, both next
    to nothing, are several per cent of each other apart: a comparison of noise)."""
    import pyglades as pg
    print("cfg4 at full size: bf16 vs fp32 training", flush=True)
    sizes = [4096, 4096, 4096, 4096, 4096, 1024]
    (f, b), hist, draw = _trained_pair(sizes, 8192, 8, 200, 0.002, 23, [pg.F32, pg.BF16])
    worst = 0.0
    for s, (mf, mb) in enumerate(hist):
        if s % 20 == 0 or s == len(hist) - 1:
            print("step %d loss fp32 %.6f bf16 %.6f" % (s, mf.loss, mb.loss), flush=True)
        worst = max(worst, abs(mb.loss - mf.loss) / abs(mf.loss))
        assert abs(mb.loss - mf.loss) <= 2e-2 * abs(mf.loss), (s, mb.loss, mf.loss)
    assert hist[-1][0].loss < 0.2 * hist[0][0].loss                     # the schedule does train
    Xt, _, cls = draw(np.random.default_rng(24), 8192)
    of, ob = f.forward(Xt), b.forward(Xt)
    f.close(); b.close()
    agree = (of.argmax(1) == ob.argmax(1)).mean()
    print("first loss %.4f, last loss fp32 %.5f bf16 %.5f, worst relative loss gap %.2e; held-out accuracy fp32 %.4f bf16 %.4f, "
          "agreement %.4f" % (hist[0][0].loss, hist[-1][0].loss, hist[-1][1].loss, worst, (of.argmax(1) == cls).mean(),
                              (ob.argmax(1) == cls).mean(), agree), flush=True)
    assert (of.argmax(1) == cls).mean() >= 0.99
    assert agree >= 0.995


def test_cfg5_full_size_e4m3_against_fp32():
    """The inference benchmark at its full size -- 8192-8192-8192-8192-1024, batch 16 384 -- against the
    fp32 GPU forward on the dequantised weights: (1) a network trained 28 steps (bf16 path, 1024
    separable classes): top-1 agreement >= 99.5 % over all 16 384 rows, logits within 6e-2 relative
    RMS; (2) the benchmark's literal inputs, N(0, 1/fan_in) weights and N(0,1) rows: logits within
    6.5e-2 relative RMS; their top-1 agreement is printed (1024 near-flat classes: the margin of most
    rows is below what e4m3 activations resolve) and only bounded from below by 80 %."""
    import pyglades as pg
    from helpers import rel_rms
    print("cfg5 at full size: e4m3 vs fp32 forward", flush=True)
    sizes = [8192, 8192, 8192, 8192, 1024]
    (t,), hist, draw = _trained_pair(sizes, 8192, 4, 28, 0.02, 29, [pg.BF16])
    assert hist[-1][0].correct >= 0.99 * 8192
    Wt = [t.get_params(l) for l in range(4)]
    t.close()
    B = 16384
    Xt, _, cls = draw(np.random.default_rng(30), B)
    Xt = po.bf16_round(Xt)
    kw = dict(act_params=[0, 0, 0, 1.0], cost=pg.CLASSIFICATION, mode=pg.MODE_CANONICAL)
    acts = [pg.RELU] * 3 + [pg.LINEAR]
    q = pg.Net(pg.make_spec(sizes, acts, dtype=pg.FP8_INFER, **kw))
    r = pg.Net(pg.make_spec(sizes, acts, dtype=pg.F32, **kw))
    tab = po.e4m3_table()

    def both(Ws, bs, X):
        for l in range(4):
            q.set_params(l, Ws[l], bs[l])
        codes, scales = q.quantize_fp8()
        for l in range(4):
            r.set_params(l, tab[codes[l]] * scales[l][:, None], bs[l])
        q.set_fp8_activation_scaling(pg.FP8_ACT_BLOCK32)
        return q.forward(X), r.forward(X)

    got, want = both([w for w, _ in Wt], [b_ for _, b_ in Wt], Xt)
    agree, err = (got.argmax(1) == want.argmax(1)).mean(), rel_rms(got, want)
    print("trained network: top-1 agreement %.5f over all rows (fp32 accuracy %.4f), logits rel RMS %.3e" % (
        agree, (want.argmax(1) == cls).mean(), err), flush=True)
    assert (want.argmax(1) == cls).mean() >= 0.995
    assert agree >= 0.995
    assert err <= 6e-2
    # the same network with one fp32 scale per token: the same bars
    q.set_fp8_activation_scaling(pg.FP8_ACT_PER_TOKEN)
    got_t = q.forward(Xt)
    agree_t, err_t = (got_t.argmax(1) == want.argmax(1)).mean(), rel_rms(got_t, want)
    print("trained network, one scale per token: top-1 agreement %.5f, logits rel RMS %.3e" % (agree_t, err_t), flush=True)
    assert agree_t >= 0.995 and err_t <= 6e-2
    del Wt
    rng = np.random.default_rng(31)
    Wr = [rng.standard_normal((sizes[l + 1], sizes[l]), dtype=np.float32) * np.float32(np.sqrt(1.0 / sizes[l])) for l in range(4)]
    Xr = po.bf16_round(rng.standard_normal((B, sizes[0]), dtype=np.float32))
    got, want = both(Wr, [np.zeros(sizes[l + 1], np.float32) for l in range(4)], Xr)
    agree, err = (got.argmax(1) == want.argmax(1)).mean(), rel_rms(got, want)
    print("random weights (the benchmark's inputs): top-1 agreement %.5f over all rows, logits rel RMS %.3e" % (agree, err), flush=True)
    assert err <= 6.5e-2     # measured 5.5e-2 .. 5.7e-2: the four e4m3 roundings of the activations
    assert agree >= 0.80
    q.close(); r.close()
