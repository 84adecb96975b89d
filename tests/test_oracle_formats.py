"""bf16 / e4m3 conversions of the restatement against torch's casts."""
import numpy as np
import pytest
import torch

import pyoracle as po


def test_e4m3_decode_all_codes():
    tab = po.e4m3_table()
    ref = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    assert np.array_equal(np.isnan(tab), np.isnan(ref))
    assert np.array_equal(tab[~np.isnan(tab)], ref[~np.isnan(ref)])
    assert tab[0x7E] == 448.0 and tab[0x08] == 2.0 ** -6 and tab[0x01] == 2.0 ** -9


def test_e4m3_encode_matches_torch_in_range():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(20000) * 100, rng.standard_normal(20000) * 0.01,
                        np.linspace(-448, 448, 4001), po.e4m3_table()[:0x7F],
                        (po.e4m3_table()[:0x7E] + po.e4m3_table()[1:0x7F]) / 2]).astype(np.float32)  # exact ties
    x = x[np.abs(x) <= 448]
    L = po.lib()
    mine = np.array([L.go_e4m3_from_f32(float(v)) for v in x], np.uint8)
    ref = torch.tensor(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(mine, ref)
    assert L.go_e4m3_from_f32(1e9) == 0x7E and L.go_e4m3_from_f32(-500.0) == 0xFE  # saturating


def test_bf16_round_matches_torch():
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(50000) * 10.0 ** rng.integers(-20, 20, 50000), [0.0, -0.0, 1.0, 65504.0]]).astype(np.float32)
    ref = torch.tensor(x).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(po.bf16_round(x).view(np.uint32), ref.view(np.uint32))
    L = po.lib()
    for v in x[:2000]:
        assert L.go_bf16_to_f32(L.go_bf16_from_f32(float(v))) == np.float32(torch.tensor(np.float32(v)).to(torch.bfloat16).float().item())


def test_row_quantisation():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((9, 33)).astype(np.float32)
    x[4] = 0.0
    q, s = po.e4m3_quant_rows(x)
    assert s[4] == 1.0 and not q[4].any()
    amax = np.abs(x).max(1)
    np.testing.assert_array_equal(s[amax > 0], (amax / np.float32(448.0))[amax > 0])
    deq = po.e4m3_table()[q] * s[:, None]
    assert np.abs(deq - x).max() <= np.abs(x).max() / 16 + 1e-6  # 3 mantissa bits: rel. step 1/8, half of it
    assert (np.abs(po.e4m3_table()[q]).max(1)[amax > 0] == 448.0).all()


def test_fp8_forward_close_to_fp32_forward_on_dequantised_weights():
    rng = np.random.default_rng(3)
    sizes, acts = [64, 48, 40, 10], [po.RELU, po.RELU, po.RELU]
    spec = po.make_spec(sizes, acts)
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) / np.sqrt(sizes[l])).astype(np.float32) for l in range(3)]
    qs = [po.e4m3_quant_rows(w) for w in Ws]
    X = po.bf16_round(rng.standard_normal((50, 64)).astype(np.float32))
    out = po.fp8_forward(spec, [q for q, _ in qs], [s for _, s in qs], X)
    ca = po.CanonNet(spec)
    for l in range(3):
        ca.set_params(l, po.e4m3_table()[qs[l][0]] * qs[l][1][:, None])
    ref = ca.forward(X)
    err = np.sqrt(np.mean((out - ref) ** 2)) / np.sqrt(np.mean(ref ** 2))
    assert err < 5e-2


def _torch_e4m3(x):
    """float32 array -> (codes, decoded values) through torch's float8_e4m3fn cast: a conversion written by others."""
    t = torch.tensor(np.ascontiguousarray(x, np.float32)).to(torch.float8_e4m3fn)
    return t.view(torch.uint8).numpy(), t.to(torch.float32).numpy()


def test_block32_quantiser_rule_and_codes():
    """Block-scaled quantiser: the scale of every block is THE power of two that puts the block's largest
    magnitude into (224, 448] (one inequality pair fixes it), blocks are runs of 32 columns (each block of the
    input has its own magnitude, so a shifted or widened partition breaks the inequality), codes are torch's
    e4m3 cast of x / scale."""
    rng = np.random.default_rng(11)
    rows, cols = 37, 32 * 7 + 13   # a ragged last block
    mag = 10.0 ** rng.uniform(-6, 6, (rows, (cols + 31) // 32))
    x = (rng.standard_normal((rows, cols)) * np.repeat(mag, 32, axis=1)[:, :cols]).astype(np.float32)
    x = po.bf16_round(x)
    x[5, 64:96] = 0.0           # an all-zero block
    q, s = po.e4m3_quant_rows_block32(x)
    nblk = (cols + 31) // 32
    assert s.shape == (rows, nblk)
    for b in range(nblk):
        blk = x[:, b * 32:(b + 1) * 32]
        amax = np.abs(blk).max(1).astype(np.float64)
        sc = 2.0 ** (s[:, b].astype(np.float64) - 127)
        nz = amax > 0
        assert ((amax[nz] / sc[nz] > 224) & (amax[nz] / sc[nz] <= 448)).all(), b
        ref_codes, _ = _torch_e4m3((blk / sc[:, None]).astype(np.float32))
        assert np.array_equal(q[:, b * 32:(b + 1) * 32], ref_codes), b
    assert not q[5, 64:96].any()
    # the edge of the rule: 448 * 2^k stays (ratio exactly 448), the next bf16 value up moves to the next power of two
    edge = np.zeros((2, 32), np.float32)
    edge[0, 3] = 448.0 * 2.0 ** -5
    edge[1, 3] = 450.0 * 2.0 ** -5      # 1.7578125 * 2^3: bf16-exact, mantissa just above 1.75
    _, se = po.e4m3_quant_rows_block32(edge)
    assert se[0, 0] == 127 - 5 and se[1, 0] == 127 - 4
    # dequantised values are within half an e4m3 step (2^-4 relative) of the input, block by block
    deq = po.e4m3_table()[q] * np.repeat(2.0 ** (s.astype(np.float64) - 127), 32, axis=1)[:, :cols]
    bound = np.repeat(np.stack([np.abs(x[:, b * 32:(b + 1) * 32]).max(1) for b in range(nblk)], 1), 32, axis=1)[:, :cols]
    assert (np.abs(deq - x) <= bound / 16 + 1e-30).all()


def _torch_pipeline(sizes, Wq, wscale, X, block32):
    """The quantised inference pipeline stated with torch's casts and float64 products: quantise the
    (bf16-rounded) activations per row or per 32-column block, multiply code values exactly, scale, ReLU,
    round to bf16 between layers."""
    tab = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float64).numpy()
    cur = X.astype(np.float64)
    nl = len(sizes) - 1
    for l in range(nl):
        if block32:
            ni = sizes[l]
            pad = (-ni) % 32
            blk = np.pad(np.abs(cur), ((0, 0), (0, pad))).reshape(cur.shape[0], -1, 32).max(2)
            # smallest power of two with amax / scale <= 448
            e = np.ceil(np.log2(np.where(blk > 0, blk, 1.0) / 448.0))
            e = np.maximum(e, -127)
            sc = np.repeat(2.0 ** e, 32, axis=1)[:, :ni]
        else:
            amax = np.abs(cur).max(1)
            sc = np.where(amax > 0, (amax.astype(np.float32) / np.float32(448.0)).astype(np.float64), 1.0)[:, None]
        _, xq = _torch_e4m3((cur.astype(np.float32) / sc.astype(np.float32)).astype(np.float32))
        z = (xq.astype(np.float64) * sc) @ tab[Wq[l]].T * wscale[l].astype(np.float64)[None, :]
        cur = np.maximum(z, 0.0) * (z >= 0.046)     # the reference's ReLU: 0 below its knee
        if l + 1 < nl:
            cur = torch.tensor(cur.astype(np.float32)).to(torch.bfloat16).to(torch.float64).numpy()
    return cur


@pytest.mark.parametrize("block32", [False, True])
def test_fp8_forward_equals_an_independent_statement_of_the_pipeline(block32):
    """go_fp8_forward / go_fp8_forward_block32 against the same pipeline written with torch's conversions and
    float64 products: they differ by fp32 accumulation only (1e-5; a quantisation point moved, a scale applied
    to the wrong block or row, or a missing bf16 rounding shows at 1e-2)."""
    rng = np.random.default_rng(12)
    sizes, acts = [96, 80, 72, 10], [po.RELU, po.RELU, po.RELU]
    spec = po.make_spec(sizes, acts)
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) / np.sqrt(sizes[l])).astype(np.float32) for l in range(3)]
    qs = [po.e4m3_quant_rows(w) for w in Ws]
    X = po.bf16_round((rng.standard_normal((40, 96)) * 10.0 ** rng.uniform(-2, 2, (40, 1))).astype(np.float32))
    out = po.fp8_forward(spec, [q for q, _ in qs], [s for _, s in qs], X, block32=block32)
    ref = _torch_pipeline(sizes, [q for q, _ in qs], [s for _, s in qs], X, block32)
    err = np.sqrt(np.mean((out - ref) ** 2)) / np.sqrt(np.mean(ref ** 2))
    # a value that sits on a rounding boundary of bf16 or e4m3 can fall to the other side in fp32: a handful of
    # outputs may then differ at 1e-2 while the rest agree to 1e-6
    close = np.isclose(out, ref, rtol=2e-5, atol=1e-6 * np.abs(ref).max())
    assert close.mean() > 0.97 and err < 5e-3, (close.mean(), err)
