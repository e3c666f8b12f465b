"""The sparseness projection of the columns of W through the C ABI against the oracle's
restatement of the reference's iteration (dense_factor_sparsity_constraints.h:205-237).

Tolerance: the element arithmetic is the same fp32 sequence on both sides and the column sums are
fp64 on both sides, in different orders; a step multiplies the deviation from the column mean by a
factor that grows as entries are fixed at zero, so last-place differences of the sums grow over
the passes: 1e-5 of a column's largest entry, and the same count of non-zero entries up to entries
that one side leaves within that distance of zero."""

import numpy as np
import pytest

import npeff_ref_amd as d
from oracle import oracle as orc

pytestmark = pytest.mark.gpu


def _compare(got, want, l1):
    scale = np.abs(want).max(axis=0)
    assert np.all(np.abs(got - want) <= 1e-5 * scale + 1e-7)
    assert got.min() >= 0.0
    np.testing.assert_allclose(got.sum(axis=0, dtype=np.float64), l1, rtol=3e-6)
    flips = (got > 0) != (want > 0)
    assert np.all(np.maximum(got, want)[flips] <= 1e-5 * np.broadcast_to(scale, got.shape)[flips] + 1e-7)


@pytest.mark.parametrize("n,r,l1", [(1, 1, 1.0), (2, 1, 1.0), (37, 5, 2.0), (500, 8, 5.0), (2000, 256, 12.0),
                                    (4099, 100, 30.0), (300, 1000, 4.0), (20000, 256, 40.0), (300001, 3, 60.0)])
def test_columns_match_the_oracle(n, r, l1):
    rng = np.random.default_rng(n + r)
    W = (rng.random((n, r)) ** 2).astype(np.float32)
    want, passes = orc.sparsify_columns(W, l1, 1.0)
    dW = d.DeviceArray.from_numpy(W)
    rounds = d.op_sparsify_columns(dW, l1, 1.0)
    d.sync()
    got = dW.numpy()
    _compare(got, want, l1)
    assert abs(rounds - passes) <= 1  # an entry within rounding of zero can cost one more pass
    # the same bits from a second run
    dW2 = d.DeviceArray.from_numpy(W)
    d.op_sparsify_columns(dW2, l1, 1.0)
    d.sync()
    assert np.array_equal(dW2.numpy(), got)


def test_one_pass_column_and_other_l2():
    rng = np.random.default_rng(9)
    n, r = 400, 6
    W = (0.5 + 0.1 * rng.random((n, r))).astype(np.float32)
    dW = d.DeviceArray.from_numpy(W)
    assert d.op_sparsify_columns(dW, 50.0, 1.0) == 1
    d.sync()
    x = W.astype(np.float64)
    dev = x - x.mean(axis=0)
    np.testing.assert_allclose(dW.numpy(), 50.0 / n + dev / np.linalg.norm(dev, axis=0), rtol=0, atol=3e-6)
    W2 = rng.random((900, 7)).astype(np.float32)
    want, _ = orc.sparsify_columns(W2, 9.0, 2.5)
    dW2 = d.DeviceArray.from_numpy(W2)
    d.op_sparsify_columns(dW2, 9.0, 2.5)
    d.sync()
    _compare(dW2.numpy(), want, 9.0)


def test_null_constraint_is_refused():
    dW = d.DeviceArray.from_numpy(np.ones((4, 2), dtype=np.float32))
    with pytest.raises(d.DnpeffError, match="null constraint"):
        d.op_sparsify_columns(dW, -1.0, 1.0)


def test_context_method_projects_W_and_the_loop_goes_on():
    """sparsify_W on a context: W's columns get the prescribed sum, H stays, and the updates that
    follow run as after set_factors with the projected W."""
    n, m_full, k, r, seed = 300, 20000, 400, 16, 3
    A, norms = d.Csr.synth(n, m_full, k_fixed=k, zipf_s=1.1, seed=seed)
    A.normalize_rows(norms)
    A.compact_columns(1)
    nmf = d.MuNmf(A, d.MuNmfParams(rank=r, max_iters=3, eps=1e-12, seed=seed, log_every=10))
    nmf.initialize()
    W0, H0 = nmf.loadWToHostSync(), nmf.loadHToHostSync()
    passes = nmf.sparsify_W(3.0)
    W1 = nmf.loadWToHostSync()
    want, want_passes = orc.sparsify_columns(W0, 3.0, 1.0)
    _compare(W1, want, 3.0)
    assert abs(passes - want_passes) <= 1
    assert np.array_equal(nmf.loadHToHostSync(), H0)
    nmf.step(2)
    Wa, Ha = nmf.loadWToHostSync(), nmf.loadHToHostSync()
    other = d.MuNmf(A, d.MuNmfParams(rank=r, max_iters=3, eps=1e-12, seed=seed, log_every=10))
    other.set_factors(W1, H0)
    other.step(2)
    assert np.array_equal(other.loadWToHostSync(), Wa) and np.array_equal(other.loadHToHostSync(), Ha)
    other.close()
    nmf.close()
    A.close()
