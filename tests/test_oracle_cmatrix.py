"""The restated confusion matrix (ML/GMath/cmatrix.cpp) pinned without the reference's containers:
a hand-computed matrix, the perfect-classifier closed form, the no-class rule of the argmax scan,
and brute force over random small matrices."""
import numpy as np

import pyoracle as po


def test_hand_computed_three_classes():
    # expected classes 0 1 2 0 1 2 0, predicted 0 1 1 0 2 2 1
    E = np.eye(3, dtype=np.float32)[[0, 1, 2, 0, 1, 2, 0]]
    P = np.eye(3, dtype=np.float32)[[0, 1, 1, 0, 2, 2, 1]] * 0.9
    M = po.cmatrix(E, P)
    assert M.tolist() == [[2, 1, 0], [0, 1, 1], [0, 1, 1]]   # row expected, column predicted
    tp, tn, fp, fn, ov = po.cmatrix_metrics(M)
    assert tp.tolist() == [2, 1, 1]
    assert tn.tolist() == [2, 3, 3]          # other classes' diagonal cells only
    assert fp.tolist() == [0, 2, 1]          # off-diagonal column sums
    assert fn.tolist() == [1, 1, 1]          # off-diagonal row sums
    acc = np.mean([4 / 5, 4 / 7, 4 / 6])
    pre = np.mean([2 / 2, 1 / 3, 1 / 2])
    rec = np.mean([2 / 3, 1 / 2, 1 / 2])
    spe = np.mean([2 / 2, 3 / 5, 3 / 4])
    f1 = np.mean([2 * (2 / 3) * 1 / (2 / 3 + 1), 2 * (1 / 2) * (1 / 3) / (1 / 2 + 1 / 3), 2 * 0.5 * 0.5 / 1.0])
    fa = np.mean([0 / 2, 2 / 5, 1 / 4])
    np.testing.assert_allclose(ov, [acc, pre, rec, spe, f1, fa], rtol=1e-6)


def test_rows_without_a_positive_entry_have_no_class():
    E = np.array([[0, 0, 0], [0, 1, 0], [-1, -2, 0], [0, 0, 0.99]], np.float32)
    P = np.array([[0.9, 0, 0], [0, 0, 0], [0.5, 0.2, 0.1], [0.01, 0.01, 0.02]], np.float32)
    M = po.cmatrix(E, P)
    # row 0: no expected class; row 1: no predicted class; row 2: no expected class; row 3: (2, 2)
    assert M.sum() == 1 and M[2, 2] == 1


def test_perfect_classifier_closed_form():
    rng = np.random.default_rng(3)
    lab = rng.integers(0, 5, 200)
    lab[:5] = np.arange(5)
    E = np.eye(5, dtype=np.float32)[lab] * 0.98 + 0.01
    M = po.cmatrix(E, E)
    assert np.array_equal(M, np.diag(np.bincount(lab, minlength=5)).astype(np.int32))
    _, _, _, _, ov = po.cmatrix_metrics(M)
    np.testing.assert_allclose(ov, [1, 1, 1, 1, 1, 0], atol=1e-7)


def test_ties_and_order_follow_the_strict_scan():
    # equal maxima: the first one wins (strict >)
    M = po.cmatrix(np.array([[0.5, 0.5]], np.float32), np.array([[0.2, 0.2]], np.float32))
    assert M.tolist() == [[1, 0], [0, 0]]


def test_brute_force_counts_on_random_matrices():
    rng = np.random.default_rng(11)
    for n in (2, 3, 7):
        M = rng.integers(0, 9, (n, n)).astype(np.int32)
        tp, tn, fp, fn, ov = po.cmatrix_metrics(M)
        for i in range(n):
            assert tp[i] == M[i, i]
            assert tn[i] == sum(M[k, k] for k in range(n) if k != i)
            assert fp[i] == sum(M[k, i] for k in range(n) if k != i)
            assert fn[i] == sum(M[i, k] for k in range(n) if k != i)
        # a class nobody predicted and nobody expected gives 0/0: NaN poisons the means, as in the reference
        Z = M.copy(); Z[0, :] = 0; Z[:, 0] = 0
        ov = po.cmatrix_metrics(Z)[4]
        assert np.isnan(ov[1]) and np.isnan(ov[2]) and np.isnan(ov[4])
