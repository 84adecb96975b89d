"""The device's element-wise functions (exact mode's arithmetic, through ghip_gmath_eval) against the
CPU restatement, which calls this machine's C library and is itself bit-compared with the reference's
compiled gmath.cpp: every activation, derivative, cost and cost derivative, bit for bit, NaNs by
position."""
import numpy as np
import pytest

import pyoracle as po
from helpers import bits_equal

pytestmark = pytest.mark.gpu


def inputs():
    """every 509th float (8.4 M patterns: all exponents, both signs, NaNs, infinities, denormals) and
    a dense sweep of the range activations actually see"""
    strided = np.arange(0, 1 << 32, 509, dtype=np.uint64).astype(np.uint32).view(np.float32)
    dense = np.linspace(-30.0, 30.0, 2_000_001, dtype=np.float32)
    return np.concatenate([strided, dense])


@pytest.mark.parametrize("act", list(range(8)))
def test_squash_and_derivative_bit_exact(act):
    import pyglades as pg
    print("activation", act, flush=True)
    z = inputs()
    for param in (0.0, 0.01, 0.3):
        with np.errstate(all="ignore"):
            want = po.gmath_eval(0, act, z, param=param)
        got = pg.gmath_eval(0, act, z, param=param)
        assert bits_equal(got, want), (act, param)
        assert bits_equal(pg.gmath_eval(1, act, want, param=param), po.gmath_eval(1, act, want, param=param)), (act, param)


@pytest.mark.parametrize("cost", [0, 1, 2])
def test_cost_and_derivative_bit_exact(cost):
    import pyglades as pg
    print("cost", cost, flush=True)
    rng = np.random.default_rng(cost)
    n = 4_000_000
    pred = rng.random(n, dtype=np.float32)
    expect = np.where(rng.random(n) < 0.5, rng.random(n, dtype=np.float32), rng.choice(np.array([0.01, 0.99, 0.0, 1.0], np.float32), n))
    # a share of predictions outside (0, 1) and at its ends: logs of zero and of negatives
    pred[::97] = rng.normal(0, 2, pred[::97].shape).astype(np.float32)
    pred[5::1013] = 0.0
    pred[7::1013] = 1.0
    with np.errstate(all="ignore"):
        want = po.gmath_eval(2, cost, expect, pred, param=450.0)
        wder = po.gmath_eval(3, cost, expect, pred)
    assert bits_equal(pg.gmath_eval(2, cost, expect, pred, param=450.0), want)
    assert bits_equal(pg.gmath_eval(3, cost, expect, pred), wder)
