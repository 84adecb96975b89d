"""bf16 / e4m3 conversions of the restatement against torch's casts."""
import numpy as np
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
