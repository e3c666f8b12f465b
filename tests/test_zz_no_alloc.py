"""The entry point that allocates nothing (dnpeff_op_gram_static) against dnpeff_op_gram, through
the C ABI: same kernels and summation order, so the bits must agree; two calls in a row share
the static scratch array, the second with a smaller input."""

import numpy as np
import pytest

import npeff_ref_amd as d

pytestmark = pytest.mark.gpu


def _both(X, rows, r):
    dX = d.DeviceArray.from_numpy(X)
    G_ref, G_new = d.DeviceArray((r, r)), d.DeviceArray((r, r))
    d.binding._check(d.lib.dnpeff_op_gram(rows, r, dX.ptr, G_ref.ptr))
    d.sync()
    d.op_gram_static(dX, G_new, rows=rows)
    d.sync()
    return G_ref.numpy(), G_new.numpy()


@pytest.mark.parametrize("r", [128, 100, 16])
def test_static_gram_matches_the_allocating_entry_point_twice_in_a_row(r):
    rng = np.random.default_rng(5 + r)
    X = rng.lognormal(-2.0, 1.5, size=(40_000, r)).astype(np.float32)
    # first call: large input (partial sums fill most of the scratch array at ranks above 32)
    ref, got = _both(X, 40_000, r)
    assert np.array_equal(ref, got)
    want = X.astype(np.float64).T @ X.astype(np.float64)
    assert np.max(np.abs(got - want) / np.abs(want)) < 2e-6
    # second call right after it: smaller input, the array still holds the first call's partials
    ref2, got2 = _both(X[:5_001].copy(), 5_001, r)
    assert np.array_equal(ref2, got2)
    want2 = X[:5_001].astype(np.float64).T @ X[:5_001].astype(np.float64)
    assert np.max(np.abs(got2 - want2) / np.abs(want2)) < 2e-6
    assert not np.array_equal(got, got2)


def test_static_gram_back_to_back_without_a_sync_between():
    rng = np.random.default_rng(11)
    r = 128
    Xa = rng.random((30_000, r), dtype=np.float32)
    Xb = rng.random((1_000, r), dtype=np.float32)
    dXa, dXb = d.DeviceArray.from_numpy(Xa), d.DeviceArray.from_numpy(Xb)
    Ga, Gb = d.DeviceArray((r, r)), d.DeviceArray((r, r))
    d.op_gram_static(dXa, Ga)
    d.op_gram_static(dXb, Gb)  # queued behind the first on the library stream
    d.sync()
    Ra, Rb = d.DeviceArray((r, r)), d.DeviceArray((r, r))
    d.op_gram(dXa, Ra)
    d.op_gram(dXb, Rb)
    d.sync()
    assert np.array_equal(Ga.numpy(), Ra.numpy())
    assert np.array_equal(Gb.numpy(), Rb.numpy())


def test_static_gram_refuses_what_does_not_fit():
    X = d.DeviceArray((64, 128))
    G = d.DeviceArray((128, 128))
    with pytest.raises(d.DnpeffError, match="static"):
        d.binding._check(d.lib.dnpeff_op_gram_static(52_225, 128, X.ptr, G.ptr))  # too many rows
    with pytest.raises(d.DnpeffError, match="ranks 1..128"):
        d.binding._check(d.lib.dnpeff_op_gram_static(64, 256, X.ptr, G.ptr))
    with pytest.raises(d.DnpeffError):
        d.binding._check(d.lib.dnpeff_op_gram_static(0, 128, X.ptr, G.ptr))


def test_static_gram_takes_any_row_count_at_small_ranks():
    """At ranks up to 32 the partial sums are one 32 x 32 block per workgroup, at most 512 of them:
    row counts far past the limit of the larger ranks fit the scratch array."""
    rng = np.random.default_rng(3)
    X = rng.random((150_000, 16), dtype=np.float32)
    ref, got = _both(X, 150_000, 16)
    assert np.array_equal(ref, got)
    want = X.astype(np.float64).T @ X.astype(np.float64)
    assert np.max(np.abs(got - want) / np.abs(want)) < 2e-6
