"""Pins the oracle's restatement of the reference's sparseness projection
(dense_factor_sparsity_constraints.h:205-237) against what its iteration fixes by itself.  The
reference never runs that code and holds no vector for it, so these are the only pins: sums,
signs, order, the closed form of a column that needs one pass, a two-entry column worked by hand,
and the squared norm that the reference's step length (not Hoyer's) leaves.  No GPU."""

import numpy as np
import pytest

from oracle import oracle as orc


@pytest.mark.parametrize("seed,n,r,l1", [(0, 500, 8, 5.0), (1, 64, 3, 2.0), (2, 2000, 16, 20.0), (3, 7, 5, 1.5)])
def test_columns_end_non_negative_with_the_prescribed_sum_and_order(seed, n, r, l1):
    rng = np.random.default_rng(seed)
    W = (rng.random((n, r)) ** 3).astype(np.float32)
    out, passes = orc.sparsify_columns(W, l1, 1.0)
    assert passes >= 1
    assert out.min() >= 0.0
    np.testing.assert_allclose(out.sum(axis=0, dtype=np.float64), l1, rtol=2e-6)
    for c in range(r):
        kept = out[:, c] > 0
        assert kept.any()
        # the entries fixed at zero are the smallest of the input, the others keep their order
        if (~kept).any():
            assert W[~kept, c].max() <= W[kept, c].min()
        order = np.argsort(W[kept, c], kind="stable")
        assert np.all(np.diff(out[kept, c][order]) >= -1e-6 * out[:, c].max())
        # the reference's step length: ||s - m||^2 = l2^2 on the entries left, m = l1 / |Y| there,
        # hence ||s||^2 = l2^2 + l1^2 / |Y| (Hoyer's own projection would end at l2^2)
        y = int(kept.sum())
        np.testing.assert_allclose(np.sum(out[:, c].astype(np.float64) ** 2), 1.0 + l1 * l1 / y, rtol=2e-5)


def test_a_column_that_needs_one_pass_is_an_affine_image_of_its_input():
    """No entry turns negative when l1 / n exceeds l2 max|x - mean x| / ||x - mean x||: the result
    is l1 / n + l2 (x - mean x) / ||x - mean x|| (the reference's step gives the deviation from the
    mean the norm l2 itself), whatever sum and scale x came with."""
    rng = np.random.default_rng(4)
    n, r, l2 = 400, 6, 1.0
    W = (0.5 + 0.1 * rng.random((n, r))).astype(np.float32)
    l1 = 50.0
    out, passes = orc.sparsify_columns(W, l1, l2)
    assert passes == 1
    x = W.astype(np.float64)
    d = x - x.mean(axis=0)
    want = l1 / n + l2 * d / np.linalg.norm(d, axis=0)
    assert want.min() > 0
    np.testing.assert_allclose(out, want, rtol=0, atol=3e-6)
    # scale and offset of the input do not matter
    out2, _ = orc.sparsify_columns((3.0 * W + 0.25).astype(np.float32), l1, l2)
    np.testing.assert_allclose(out2, want, rtol=0, atol=3e-6)


def test_two_entries_by_hand():
    """x = (0.8, 0.2), l1 = l2 = 1: s = (0.5, 0.5) +- 0.3, alpha = 1 / (sqrt 2 * 0.3), so the step
    lands at 0.5 +- 1 / sqrt 2 = (1.2071, -0.2071); the negative entry is fixed at zero and the
    other one shifted to the sum: (1, 0).  The second pass finds nothing negative."""
    W = np.array([[0.8], [0.2]], dtype=np.float32)
    out, passes = orc.sparsify_columns(W, 1.0, 1.0)
    assert passes == 2
    np.testing.assert_allclose(out[:, 0], [1.0, 0.0], atol=1e-6)
    # the larger entry wins whichever comes first
    out, _ = orc.sparsify_columns(W[::-1].copy(), 1.0, 1.0)
    np.testing.assert_allclose(out[:, 0], [0.0, 1.0], atol=1e-6)


def test_l2_norm_scales_the_step():
    """With l1 and l2 scaled together the result scales with them (the iteration is homogeneous)."""
    rng = np.random.default_rng(5)
    W = rng.random((300, 4)).astype(np.float32)
    a, _ = orc.sparsify_columns(W, 4.0, 1.0)
    b, _ = orc.sparsify_columns(W, 8.0, 2.0)
    np.testing.assert_allclose(b, 2.0 * a, rtol=1e-5, atol=3e-5)  # fp32 steps, up to 15 passes
