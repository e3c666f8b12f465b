"""Pins the floating-point part of the CPU oracle against what the mathematics fixes: dense
numpy evaluation of the update rules on tiny inputs, the explicit residual for the loss, MU
monotonicity, and the fit path's stale-WHH loss.  No GPU."""

import numpy as np
import pytest

from conftest import csr_to_dense, random_csr
from oracle import oracle as orc


def _dense_mu(A, W, H, eps, iters):
    """Textbook Lee-Seung updates in the reference's order, dense fp64."""
    W, H = W.copy(), H.copy()
    for _ in range(iters):
        W *= (A @ H.T) / (W @ (H @ H.T) + eps)
        H *= (W.T @ A) / ((W.T @ W) @ H + eps)
    return W, H


@pytest.mark.parametrize("seed,r", [(0, 3), (1, 5), (2, 8)])
def test_nmf_f64_matches_dense_numpy(seed, r):
    rng = np.random.default_rng(seed)
    n, m = 12, 30
    rp, ci, va = random_csr(rng, n, m, 10, empty_rows={4})
    A = csr_to_dense(rp, ci, va, m)
    W0, H0 = rng.random((n, r)), rng.random((r, m))
    eps = np.float32(1e-8)
    W, H, losses = orc.nmf_f64(rp, ci, va, m, W0, H0, eps, iters=20, log_every=10)
    Wd, Hd = _dense_mu(A, W0, H0, float(eps), 20)
    np.testing.assert_allclose(W, Wd, rtol=1e-10, atol=1e-14)
    np.testing.assert_allclose(H, Hd, rtol=1e-10, atol=1e-14)
    # the logged loss is the explicit residual (a wrong sign or a dropped term fails here)
    assert len(losses) == 2
    np.testing.assert_allclose(losses[-1], np.linalg.norm(A - Wd @ Hd), rtol=1e-9)
    W10, H10 = _dense_mu(A, W0, H0, float(eps), 10)
    np.testing.assert_allclose(losses[0], np.linalg.norm(A - W10 @ H10), rtol=1e-9)


def test_update_order_matters_and_is_w_first():
    rng = np.random.default_rng(5)
    n, m, r = 8, 15, 3
    rp, ci, va = random_csr(rng, n, m, 7)
    A = csr_to_dense(rp, ci, va, m)
    W0, H0 = rng.random((n, r)), rng.random((r, m))
    W, H, _ = orc.nmf_f64(rp, ci, va, m, W0, H0, np.float32(1e-8), iters=1, log_every=0)
    # H-first would give a different W
    H_first = H0 * (W0.T @ A) / ((W0.T @ W0) @ H0 + 1e-8)
    W_hfirst = W0 * (A @ H_first.T) / (W0 @ (H_first @ H_first.T) + 1e-8)
    assert not np.allclose(W, W_hfirst)
    np.testing.assert_allclose(W, W0 * (A @ H0.T) / (W0 @ (H0 @ H0.T) + np.float32(1e-8)), rtol=1e-12)


def test_loss_terms_and_trace_identity():
    rng = np.random.default_rng(9)
    n, m, r = 10, 22, 4
    rp, ci, va = random_csr(rng, n, m, 9)
    A = csr_to_dense(rp, ci, va, m)
    W, H = rng.random((n, r)), rng.random((r, m))
    loss, terms = orc.loss_f64(rp, ci, va, m, W, H)
    np.testing.assert_allclose(terms[0], (A**2).sum(), rtol=1e-12)
    np.testing.assert_allclose(terms[1], (H * ((W.T @ W) @ H)).sum(), rtol=1e-12)
    np.testing.assert_allclose(terms[2], ((W.T @ A) * H).sum(), rtol=1e-12)
    np.testing.assert_allclose(loss, np.linalg.norm(A - W @ H), rtol=1e-10)


def test_mu_loss_is_non_increasing_and_factors_stay_non_negative():
    rng = np.random.default_rng(21)
    n, m, r = 15, 40, 4
    rp, ci, va = random_csr(rng, n, m, 12)
    W0, H0 = rng.random((n, r)), rng.random((r, m))
    W, H, losses = orc.nmf_f64(rp, ci, va, m, W0, H0, np.float32(1e-12), iters=40, log_every=1)
    assert np.all(np.diff(losses) <= 1e-12)
    assert W.min() >= 0 and H.min() >= 0


def test_single_products_match_numpy():
    rng = np.random.default_rng(4)
    n, m, r = 9, 17, 6
    rp, ci, va = random_csr(rng, n, m, 8)
    A = csr_to_dense(rp, ci, va, m)
    Ht, W = rng.random((m, r)), rng.random((n, r))
    np.testing.assert_allclose(orc.spmm_n_f64(rp, ci, va, Ht), A @ Ht, rtol=1e-12)
    np.testing.assert_allclose(orc.spmm_t_f64(rp, ci, va, m, W), A.T @ W, rtol=1e-12)
    np.testing.assert_allclose(orc.gram_f64(Ht), Ht.T @ Ht, rtol=1e-12)
    G, num = rng.random((r, r)), rng.random((m, r))  # not symmetric on purpose: X G, not X G^T
    out, D = orc.xg_mu_f64(Ht, G, num, np.float32(1e-8))
    np.testing.assert_allclose(D, Ht @ G, rtol=1e-12)
    np.testing.assert_allclose(out, Ht * (num / (Ht @ G + np.float32(1e-8))), rtol=1e-12)


def test_spsp_dense_matches_numpy():
    rng = np.random.default_rng(6)
    n, m, r = 11, 25, 5
    a = random_csr(rng, n, m, 9)
    b = random_csr(rng, r, m, 14, sort_cols=True)
    A, B = csr_to_dense(*a, m), csr_to_dense(*b, m)
    np.testing.assert_allclose(orc.spsp_dense_f64(a, m, b, r), A @ B.T, rtol=1e-12)
    np.testing.assert_allclose(orc.spsp_dense_f64(b, m, b, r), B @ B.T, rtol=1e-12)


def test_fit_reference_loss_uses_stale_whh():
    rng = np.random.default_rng(8)
    n, m, r = 10, 30, 4
    a = random_csr(rng, n, m, 10)
    b = random_csr(rng, r, m, 12, sort_cols=True)
    A, B = csr_to_dense(*a, m), csr_to_dense(*b, m)
    AH, HH, sq = A @ B.T, B @ B.T, (A**2).sum()
    W0 = rng.random((n, r))
    eps = np.float32(1e-7)
    W, ref, tru = orc.fit_f64(AH, HH, sq, W0, eps, iters=6, log_every=3)
    Wd, prev = W0.copy(), None
    want_ref, want_true = [], []
    for i in range(6):
        whh = Wd @ HH
        Wd = Wd * (AH / (whh + eps))
        if (i + 1) % 3 == 0:
            neg = (AH * Wd).sum()
            want_ref.append(np.sqrt(sq + (whh * Wd).sum() - 2 * neg))  # WHH from before the update
            want_true.append(np.linalg.norm(A - Wd @ B))
    np.testing.assert_allclose(W, Wd, rtol=1e-12)
    np.testing.assert_allclose(ref, want_ref, rtol=1e-10)
    np.testing.assert_allclose(tru, want_true, rtol=1e-9)
    assert not np.allclose(ref, tru)


def test_f32_baseline_tracks_f64_oracle():
    rng = np.random.default_rng(31)
    n, m, r = 20, 64, 6
    rp, ci, va = random_csr(rng, n, m, 20)
    W0, H0 = rng.random((n, r)).astype(np.float32), rng.random((r, m)).astype(np.float32)
    eps = np.float32(1e-8)
    W64, H64, _ = orc.nmf_f64(rp, ci, va, m, W0, H0, eps, iters=10, log_every=0)
    b = orc.F32Baseline(rp, ci, va, m, W0, H0, eps)
    b.step(10)
    W32, H32 = b.get()
    b.close()
    assert np.linalg.norm(W32 - W64) / np.linalg.norm(W64) < 1e-5
    assert np.linalg.norm(H32 - H64) / np.linalg.norm(H64) < 1e-5


def test_f32_timed_parts_run_the_same_iteration_and_fit_parts_match_f64():
    """The timed variants used by bench.py's cpu_baseline compute what the untimed ones do (the
    timing must not be of a different loop), the fp32 first-stage product and W update of the
    learner agree with the fp64 restatement."""
    rng = np.random.default_rng(23)
    n, m, r = 37, 411, 19  # neither a multiple of the 8-row blocks
    rp, ci, va = random_csr(rng, n, m, 90)
    W0, H0 = rng.random((n, r)).astype(np.float32), rng.random((r, m)).astype(np.float32)
    a = orc.F32Baseline(rp, ci, va, m, W0, H0, np.float32(1e-8))
    b = orc.F32Baseline(rp, ci, va, m, W0, H0, np.float32(1e-8))
    a.step(3)
    parts = b.step_timed(3)
    assert set(parts) == set(orc.F32Baseline.PARTS) and all(v >= 0 for v in parts.values())
    for x, y in zip(a.get(), b.get()):
        assert np.array_equal(x, y)
    a.close()
    b.close()
    # learner: A B^T with sparse B, then W updates
    brp, bci, bva = random_csr(rng, r, m, 60, sort_cols=True)
    bt = orc.transpose(brp, bci, bva, m)
    out32, secs = orc.spsp_f32_timed((rp, ci, va), bt, r)
    out64 = orc.spsp_dense_f64((rp, ci, va), m, (brp, bci, bva), r)
    assert secs >= 0 and np.allclose(out32, out64, rtol=1e-5, atol=1e-7)
    HH = orc.spsp_dense_f64((brp, bci, bva), m, (brp, bci, bva), r)
    W32, secs = orc.fit_steps_f32_timed(out64, HH, W0, np.float32(1e-7), 4)
    W64, _, _ = orc.fit_f64(out64, HH, 1.0, W0, np.float32(1e-7), 4, log_every=0)
    assert np.linalg.norm(W32 - W64) / np.linalg.norm(W64) < 1e-5


def test_sparsify_H_keeps_the_product_and_thresholds_unit_norm_rows():
    """The product W H is unchanged by the normalisation, kept rows have unit norm, threshold 0
    on non-negative H keeps every entry, and a dense rebuild of the CSR equals the thresholded
    unit-norm H (to_csr of scripts/sparsify_d_npeff.py:27-49 written out densely)."""
    rng = np.random.default_rng(9)
    r, m, n = 5, 300, 7
    H = (rng.random((r, m)) * (rng.random((r, m)) < 0.3)).astype(np.float32)
    H[3] = 0.0  # a dead component stays as it is
    W = rng.random((n, r)).astype(np.float32)
    W2, vals, offs, cols = orc.sparsify_H(W, H, 0.0)
    assert offs[-1] == r * m and np.array_equal(cols[:m], np.arange(m))
    Hn = vals.reshape(r, m)
    assert np.allclose(W2.astype(np.float64) @ Hn, W.astype(np.float64) @ H, rtol=1e-5, atol=1e-7)
    norms = np.linalg.norm(Hn.astype(np.float64), axis=1)
    assert np.allclose(norms[[0, 1, 2, 4]], 1.0, atol=1e-6) and norms[3] == 0
    thr = 0.08
    W3, vals, offs, cols = orc.sparsify_H(W, H, thr)
    dense = np.zeros((r, m), np.float32)
    for k in range(r):
        c = cols[offs[k]:offs[k + 1]]
        assert np.all(np.diff(c) > 0)
        dense[k, c] = vals[offs[k]:offs[k + 1]]
    assert np.array_equal(dense, np.where(Hn >= np.float32(thr), Hn, 0).astype(np.float32))
    assert np.array_equal(W3, W2)


def test_topk_rows_against_a_full_sort_and_known_cases():
    """Known answer with ties (lower index first), and the defining property on random rows:
    the kept values are the k largest of a full sort, every dropped entry is <= the smallest
    kept one, and the indices point at the values."""
    x = np.array([[1.0, 5.0, 5.0, 0.0, 7.0, 5.0]], dtype=np.float32)
    v, i, nrm = orc.topk_rows(x, 4)
    assert v.tolist() == [[7.0, 5.0, 5.0, 5.0]] and i.tolist() == [[4, 1, 2, 5]]
    assert np.isclose(nrm[0], np.sqrt(1 + 75 + 49))
    rng = np.random.default_rng(2)
    x = rng.lognormal(-8, 2, size=(3, 5000)).astype(np.float32)
    x[1, ::7] = 0.25  # many ties
    k = 700
    v, i, _ = orc.topk_rows(x, k)
    for r in range(3):
        assert np.array_equal(v[r], np.sort(x[r])[::-1][:k])
        assert np.array_equal(x[r, i[r]], v[r]) and len(set(i[r].tolist())) == k
        rest = np.delete(x[r], i[r])
        assert rest.max() <= v[r, -1]
        same = np.flatnonzero(np.diff(v[r]) == 0)
        assert np.all(i[r, same] < i[r, same + 1])
