"""The configurations that bench.py times, at their full size: BASELINE configs[1] (10,000 x
110M, 65,536 entries per row, r = 128) and configs[3] (20,000 x 350M, 262,144 entries per row,
Zipf 1.3, r = 256: 5.24e9 entries, past 2^31).  No CPU run of the whole matrix is possible at
these sizes; instead
  * sampled rows are made again on the host by the generator's host twin, pushed through the
    loader's rules (fp32 division by norm + 1e-9, ascending renumbering of the kept columns) and
    compared bit for bit with what the device holds for the products (dense head + sparse part);
  * A H^T on those rows and A^T W on sampled columns (head, dense, middle and far-tail columns,
    the last columns of the matrix) are compared with fp64 sums on the host, 2e-5;
  * sampled entries of the rows are looked up in the transposed copy, whose columns must list
    their rows in ascending order;
  * <A H^T, W> = <A^T W, H> ties the two copies together over every entry;
  * W and sampled H stay non-negative and finite, the logged loss decreases, and a second run of
    a step from the same seeded factors gives the same bits."""

import ctypes as C

import numpy as np
import pytest

import npeff_ref_amd as d

pytestmark = pytest.mark.gpu

TOL = 2e-5


def _full_size_checks(n, m_full, k, zipf_s, r, seed, n_rows_sampled, tiled_expected, k_min=0, k_max=0, tail_lists_expected=False):
    A, norms = d.Csr.synth(n, m_full, k_fixed=k, k_min=k_min, k_max=k_max, zipf_s=zipf_s, seed=seed)
    A.normalize_rows(norms)
    A.compact_columns(1)
    m, z = A.n_cols, A.nnz
    assert (z == n * k if k else n * k_min <= z <= n * k_max) and A.full_dense_size == m_full
    kept = A.kept_indices()
    assert np.all(np.diff(kept.astype(np.int64)) > 0)  # newToOgIndex ascends
    nmf = d.MuNmf(A, d.MuNmfParams(rank=r, max_iters=0, eps=1e-12, seed=seed), consume_matrix=True)
    assert nmf.info()[0] == tiled_expected
    n_dense, z_sparse = A.head_info()
    assert n_dense > 0 and 0 < z_sparse < z

    # one step twice from the same seeded factors: same bits
    probe_cols = np.unique(np.concatenate([np.arange(0, 64), np.linspace(0, m - 1, 4096).astype(np.int64)]))
    def one_step():
        nmf.initialize()
        nmf.step(1)
        w_dev, h_dev = nmf.device_factors()
        return nmf.loadWToHostSync(), d.gather_rows(h_dev, r, probe_cols), nmf.computeUncachedLoss()
    W1, Hs1, loss1 = one_step()
    W1b, Hs1b, loss1b = one_step()
    assert np.array_equal(W1, W1b) and np.array_equal(Hs1, Hs1b) and loss1 == loss1b
    assert np.isfinite(W1).all() and W1.min() >= 0 and np.isfinite(Hs1).all() and Hs1.min() >= 0

    # the loss decreases over further steps
    losses = [loss1]
    for _ in range(2):
        nmf.step(1)
        losses.append(nmf.computeUncachedLoss())
    assert np.all(np.isfinite(losses)) and losses[0] > losses[1] > losses[2]

    # both sparse products see the same matrix
    via_rows, via_cols = nmf.check_products()
    assert abs(via_rows - via_cols) <= 5e-6 * abs(via_rows)

    W = nmf.loadWToHostSync()
    w_dev, h_dev = nmf.device_factors()
    assert np.isfinite(W).all() and W.min() >= 0
    Hs = d.gather_rows(h_dev, r, probe_cols)
    assert np.isfinite(Hs).all() and Hs.min() >= 0

    # A H^T on the device (the kernels of the W update)
    N_dev = d.DeviceArray((n, r))
    d.binding._check(d.lib.dnpeff_op_spmm_n(A._h, r, C.c_void_p(h_dev), N_dev.ptr))
    d.sync()
    N = N_dev.numpy()
    # how the sparse part ran: at ranks from 256 with rows enough, the far tail from slot lists
    info = A.products_info()
    assert (info["tail_floor"] > 0 and info["list_entries"] > 0) == tail_lists_expected, info

    rng = np.random.default_rng(seed % 1000)
    rows = np.unique(np.concatenate([[0, n // 3, n - 1], rng.integers(0, n, n_rows_sampled)]))[:n_rows_sampled]
    lookups = []
    for i in rows:
        rp, ci, va, nr = d.synth_pef_host_rows(int(i), 1, m_full, k_fixed=k, k_min=k_min, k_max=k_max,
                                               zipf_s=zipf_s, seed=seed)
        k_row = len(ci)
        assert nr[0] == norms[i]  # host twin and device generator agree on the row
        want_cols = np.searchsorted(kept, ci).astype(np.int32)
        assert np.array_equal(kept[want_cols], ci)
        want_vals = (va / np.float32(nr[0] + np.float32(1e-9))).astype(np.float32)
        got_cols, got_vals = A.get_row(int(i))
        assert len(got_cols) == k_row
        o_w, o_g = np.argsort(want_cols, kind="stable"), np.argsort(got_cols, kind="stable")
        assert np.array_equal(want_cols[o_w], got_cols[o_g])
        assert np.array_equal(want_vals[o_w], got_vals[o_g])  # bit-exact loader at this size
        Hrows = d.gather_rows(h_dev, r, want_cols).astype(np.float64)
        N64 = want_vals.astype(np.float64) @ Hrows
        assert np.max(np.abs(N[i] - N64)) <= TOL * np.max(np.abs(N64))
        pick = rng.integers(0, k_row, 6)
        lookups += [(int(i), int(want_cols[p]), want_vals[p]) for p in pick]

    # the transposed copy lists these entries too
    for i, j, v in lookups:
        rws, vls = A.get_column(j)
        at = np.searchsorted(rws, i)
        assert at < len(rws) and rws[at] == i and vls[at] == v

    # A^T W on windows of columns: head, the densest sparse columns, middle, far tail, the end
    win = 4096
    starts = sorted({0, max(0, min(m - win, n_dense - win // 2)), (m // 7) // 128 * 128, (m // 2) // 128 * 128,
                     (m - win) // 128 * 128, max(0, m - win)})
    T_dev = d.DeviceArray((win, r))
    for c0 in starts:
        c1 = min(m, c0 + win)
        d.binding._check(d.lib.dnpeff_op_spmm_t_tile(A._h, r, C.c_void_p(w_dev), c0, c1, T_dev.ptr))
        d.sync()
        T = T_dev.numpy()
        for j in np.unique(np.concatenate([[c0, c1 - 1], rng.integers(c0, c1, 40)])):
            rws, vls = A.get_column(int(j))
            assert np.all(np.diff(rws) > 0)  # ascending rows, none twice
            T64 = vls.astype(np.float64) @ W[rws].astype(np.float64) if len(rws) else np.zeros(r)
            scale = np.max(np.abs(T64)) if len(rws) else 0.0
            assert np.max(np.abs(T[j - c0] - T64)) <= TOL * scale
    nmf.close()
    A.close()


def test_configs1_at_full_size():
    _full_size_checks(10_000, 110_000_000, 65_536, 1.1, 128, 43190432042, n_rows_sampled=24,
                      tiled_expected=False)


@pytest.mark.timeout(600)
def test_configs3_at_full_size():
    free, total = d.device_memory()
    if total < 280e9:
        pytest.skip("configs[3] needs the 288 GB of an MI355X")
    _full_size_checks(20_000, 350_000_000, 262_144, 1.3, 256, 43190432042, n_rows_sampled=8,
                      tiled_expected=True, tail_lists_expected=True)


@pytest.mark.timeout(600)
def test_configs4_ragged_rows_at_full_size():
    """configs[4]: 40,000 rows of 1,024 ... 524,288 entries (3.34e9 in all) x 110M, r = 512."""
    free, total = d.device_memory()
    if total < 280e9:
        pytest.skip("configs[4] needs the 288 GB of an MI355X")
    _full_size_checks(40_000, 110_000_000, 0, 1.1, 512, 43190432042, n_rows_sampled=6, tiled_expected=True,
                      k_min=1_024, k_max=524_288, tail_lists_expected=True)


def test_configs2_fit_path_at_full_size():
    """configs[2]: 50,000 new examples x 65,536 entries (3.28e9, past 2^31) against a fixed sparse
    H of rank 256 over 110M features at 1 % density.  First stage: sampled rows of A H^T and the
    whole of H H^T against fp64 sums on the host; second stage: the W update works row by row, so
    the sampled rows are followed on the host in fp64 from the same seeded start, and the logged
    loss is the reference's (stale W H H^T) formula on the device's own products."""
    from oracle import oracle as orc

    n, m, k, r, seed = 50_000, 110_000_000, 65_536, 256, 43190432042
    rng = np.random.default_rng(3)
    rp, cols = [0], []
    for _ in range(r):  # every entry present with probability 0.01: geometric gaps
        idx = np.cumsum(rng.geometric(0.01, size=int(m * 0.0105) + 64)) - 1
        idx = idx[idx < m].astype(np.int32)
        cols.append(idx)
        rp.append(rp[-1] + len(idx))
    hci = np.concatenate(cols)
    hva = np.exp(rng.normal(-8.0, 2.0, size=len(hci))).astype(np.float32)
    hrp = np.array(rp, dtype=np.int64)
    H = d.Csr.from_host(hrp, hci, hva, m)
    A, norms = d.Csr.synth(n, m, k_fixed=k, zipf_s=1.1, seed=seed)
    A.normalize_rows(norms)
    assert A.nnz == n * k > 2**31
    L = d.Learner(A, H, d.LearnerParams(max_iters=0, eps=1e-7, seed=seed))
    AH, HH, sq = L.products()
    assert abs(sq - n) < 1e-3 * n  # rows are L2-normalised
    # H H^T in fp64 from H's rows (sorted columns: intersections by searchsorted)
    for a, b in [(0, 0), (3, 200), (255, 17), (100, 100)]:
        ca, va_ = hci[hrp[a]:hrp[a + 1]], hva[hrp[a]:hrp[a + 1]].astype(np.float64)
        cb, vb_ = hci[hrp[b]:hrp[b + 1]], hva[hrp[b]:hrp[b + 1]].astype(np.float64)
        pos = np.searchsorted(cb, ca)
        hit = (pos < len(cb)) & (cb[np.minimum(pos, len(cb) - 1)] == ca)
        want = float(np.sum(va_[hit] * vb_[pos[hit]]))
        assert abs(HH[a, b] - want) <= 2e-5 * max(abs(want), 1e-30)
        assert abs(HH[a, b] - HH[b, a]) <= 1e-6 * abs(want)  # (two sums of the same terms in another order)
    # sampled rows of A H^T: the row made again on the host, H's columns looked up in its CSC
    colptr, comp, tv = orc.transpose(hrp, hci, hva, m)
    rows = [0, 1, n // 2, n - 1] + list(rng.integers(0, n, 12))
    for i in rows:
        rpi, ci, va, nr = d.synth_pef_host_rows(int(i), 1, m, k_fixed=k, zipf_s=1.1, seed=seed)
        v = (va / np.float32(nr[0] + np.float32(1e-9))).astype(np.float64)
        want = np.zeros(r)
        lens = colptr[ci.astype(np.int64) + 1] - colptr[ci]
        for e in np.nonzero(lens)[0]:
            p0, p1 = colptr[ci[e]], colptr[ci[e] + 1]
            np.add.at(want, comp[p0:p1], v[e] * tv[p0:p1].astype(np.float64))
        assert np.max(np.abs(AH[i] - want)) <= 2e-5 * np.max(np.abs(want))
    # second stage on the sampled rows
    L.initialize()
    L.step(25)
    W = L.GetOnHost_W()
    ref_loss, true_loss = L.losses()
    sel = np.array(sorted(set(int(x) for x in rows)))
    W0 = np.array([[d.uniform_at(seed, 0, i, c, r) for c in range(r)] for i in sel], dtype=np.float32)
    W64, _, _ = orc.fit_f64(AH[sel], HH, 1.0, W0, np.float32(1e-7), 25, log_every=0)
    assert np.linalg.norm(W[sel] - W64) / np.linalg.norm(W64) < 1e-4
    assert np.isfinite(W).all() and W.min() >= 0 and np.isfinite([ref_loss, true_loss]).all()
    L.close()
    A.close()
    H.close()
