"""The scalar layer bias of exact mode: the reference subtracts lr*d[o] once per (input, output) pair
(network.cpp:654-656), a chain of n_in * n_out dependent fp32 subtractions per row.  The kernel
replaces the walk by integer arithmetic on the bias's binade where that is provably the same float.
Here the shortcut is compared, bit for bit, with the walk on the device and with a float32 walk on
the host, on cases made to hit every way out of it."""
import numpy as np
import pytest

from helpers import bits_equal

pytestmark = pytest.mark.gpu


def host_walk(b, x, rounds):
    b = np.float32(b)
    for _ in range(rounds):
        for v in x:
            b = np.float32(b - v)
    return b


def run(b0, X, rounds):
    import pyglades as pg
    walked = pg.gmath_eval(4, 0, b0, X, rounds)
    kernel = pg.gmath_eval(4, 1, b0, X, rounds)
    took = pg.gmath_eval(4, 2, b0, X, rounds)
    return walked, kernel, took


def ulp_of(b):
    return np.float32(2.0) ** (np.floor(np.log2(np.abs(b.astype(np.float64)))) - 23)


def test_shortcut_equals_the_walk_on_ordinary_rows():
    rng = np.random.default_rng(3)
    n, rounds = 4096, 64
    b0 = (rng.standard_normal(n) * np.float32(2.0) ** rng.integers(-20, 10, n)).astype(np.float32)
    rel = np.float32(2.0) ** rng.integers(-22, -8, n)                    # |lr*d| relative to the bias
    X = (rng.standard_normal((n, 64)) * (np.abs(b0) * rel)[:, None]).astype(np.float32)
    X[:, 48:] = 0                                                         # 48 outputs, padded
    walked, kernel, took = run(b0, X, rounds)
    assert bits_equal(kernel, walked)
    assert took.mean() > 0.8                                              # the shortcut is what ran
    for k in rng.integers(0, n, 24):                                      # and the device's walk is a float32 walk
        assert bits_equal(walked[k], host_walk(b0[k], X[k], rounds)), k


@pytest.mark.parametrize("rounds", [1, 9, 64, 1100])
def test_large_steps_cross_binades_and_fall_back(rounds):
    rng = np.random.default_rng(rounds)
    n = 2048
    b0 = (rng.standard_normal(n) * np.float32(2.0) ** rng.integers(-12, 6, n)).astype(np.float32)
    rel = np.float32(2.0) ** rng.integers(-14, 1, n)                      # up to the size of the bias itself
    X = (rng.standard_normal((n, 64)) * (np.abs(b0) * rel)[:, None] / np.float32(rounds)).astype(np.float32)
    walked, kernel, took = run(b0, X, rounds)
    assert bits_equal(kernel, walked)
    assert 0.02 < took.mean() < 0.98                                      # both ways out were taken


def test_ties_zeros_and_special_values_take_the_walk():
    rng = np.random.default_rng(11)
    n, rounds = 512, 16
    b0 = (rng.standard_normal(n) * 3).astype(np.float32)
    u = ulp_of(b0)
    X = (rng.integers(-40, 40, (n, 64)) * u[:, None]).astype(np.float32)  # whole units: exact, no tie
    walked, kernel, took = run(b0, X, rounds)
    assert bits_equal(kernel, walked)
    Xt = X.copy()
    Xt[:, 5] = (np.float32(7.5) * u).astype(np.float32)                   # exactly half-way: the rounding depends on parity
    walked_t, kernel_t, took_t = run(b0, Xt, rounds)
    assert bits_equal(kernel_t, walked_t)
    assert took_t.max() == 0.0
    special = np.array([0.0, -0.0, 1e-45, -3e-42, np.inf, -np.inf, np.nan, 1.17549435e-38, 3.4e38, -3.4e38], np.float32)
    Xs = (rng.standard_normal((special.size, 64)) * 1e-3).astype(np.float32)
    w, k, t = run(special, Xs, rounds)
    assert bits_equal(k, w)
    bad = X[:4].copy()
    bad[0, 3] = np.nan; bad[1, 9] = np.inf; bad[2, 0] = -np.inf; bad[3, 63] = 1e30
    w, k, t = run(b0[:4], bad, rounds)
    assert bits_equal(k, w)
    assert t.max() == 0.0


def test_power_of_two_boundaries():
    """A bias sitting on or next to a power of two: one unit below it the grid is twice as fine."""
    rounds = 4
    cases, rows = [], []
    for e in (-3, 0, 5):
        p = np.float32(2.0 ** e)
        u = np.float32(2.0 ** (e - 23))
        for b in (p, np.nextafter(p, np.float32(4 * p)), np.nextafter(p, np.float32(0)), -p,
                  np.float32(2 * p) - u, np.float32(p + 3 * u)):
            for step in (u, -u, u / 2, -u / 2, u / 4, 3 * u, 0.75 * u):
                x = np.zeros(64, np.float32)
                x[:8] = np.float32(step)
                cases.append(b); rows.append(x)
    b0 = np.array(cases, np.float32)
    X = np.stack(rows)
    walked, kernel, took = run(b0, X, rounds)
    assert bits_equal(kernel, walked)
    for k in range(0, b0.size, 5):
        assert bits_equal(walked[k], host_walk(b0[k], X[k], rounds)), k
