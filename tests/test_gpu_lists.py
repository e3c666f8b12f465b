"""The sparse products on component slices (slot lists of A H^T, column blocks of A^T W) through
the C ABI, forced on with the n_lists / t_lists switches, against fp64 sums of the oracle.

Tolerance: fp32 sums in an order fixed by the matrix structure, 2e-5 of the largest magnitude of
each output row against fp64.  Shapes cover several pieces per slot (small nl_piece_cols), empty
rows and columns, columns longer than a block, fewer slices than XCDs (row parts) and more
(several launches), and the inspection calls on a consumed matrix."""

import numpy as np
import pytest

import npeff_ref_amd as d
from conftest import csr_to_dense, random_csr
from oracle import oracle as orc

pytestmark = pytest.mark.gpu

TOL = 2e-5


def _row_rel(a, b):
    return (np.abs(a - b).max(axis=1) / np.maximum(np.abs(b).max(axis=1), 1e-30)).max()


@pytest.mark.parametrize("r", [32, 64, 128, 256, 512])
@pytest.mark.parametrize("shape,piece_cols", [((37, 900, 60), 64), ((130, 5000, 3000), 512), ((1500, 70000, 900), 4096)])
def test_spmm_n_from_slot_lists(r, shape, piece_cols, tune):
    n, m, maxk = shape
    tune("n_lists", 1)
    tune("nl_piece_cols", piece_cols)
    rng = np.random.default_rng(r + n)
    rp, ci, va = random_csr(rng, n, m, maxk, empty_rows={1, n - 1})
    A = d.Csr.from_host(rp, ci, va, m)
    H = rng.random((m, r)).astype(np.float32)
    dH, dN = d.DeviceArray.from_numpy(H), d.DeviceArray((n, r))
    d.op_spmm_n(A, r, dH, dN)
    N = dN.numpy()
    assert _row_rel(N.astype(np.float64), orc.spmm_n_f64(rp, ci, va, H)) < TOL
    assert np.all(N[1] == 0) and np.all(N[n - 1] == 0)  # empty rows
    # same bits again, and whatever the lock step of the workgroups does
    d.op_spmm_n(A, r, dH, dN)
    assert np.array_equal(dN.numpy(), N)
    tune("nl_lag", 3)
    tune("nl_spin", 1)
    d.op_spmm_n(A, r, dH, dN)
    assert np.array_equal(dN.numpy(), N)
    A.close()


@pytest.mark.parametrize("r", [32, 64, 128, 256, 512])
@pytest.mark.parametrize("shape", [(37, 900, 60), (130, 5000, 3000), (1500, 70000, 900)])
def test_spmm_t_in_column_blocks(r, shape, tune):
    n, m, maxk = shape
    tune("t_lists", 1)
    rng = np.random.default_rng(r + n + 1)
    rp, ci, va = random_csr(rng, n, m, maxk, empty_rows={1, n - 1})
    A = d.Csr.from_host(rp, ci, va, m)
    W = rng.random((n, r)).astype(np.float32)
    dW, dT = d.DeviceArray.from_numpy(W), d.DeviceArray((m, r))
    d.op_spmm_t(A, r, dW, dT)
    T = dT.numpy()
    want = orc.spmm_t_f64(rp, ci, va, m, W)
    assert np.abs(T - want).max() <= TOL * np.abs(want).max()
    assert _row_rel(T.astype(np.float64), want) < TOL
    d.op_spmm_t(A, r, dW, dT)
    assert np.array_equal(dT.numpy(), T)
    # a tile of columns is the same launch on a range of blocks
    c0, c1 = 128, min(m, 128 + 64 * 9)
    dTt = d.DeviceArray((c1 - c0, r))
    d.binding._check(d.lib.dnpeff_op_spmm_t_tile(A._h, r, dW.ptr, c0, c1, dTt.ptr))
    d.sync()
    assert np.array_equal(dTt.numpy(), T[c0:c1])
    A.close()


def test_long_columns_and_long_rows_on_slices(tune):
    """Zipf columns: the first columns hold most rows (several blocks of one column each in A^T W),
    rows of 5,000 entries span many pieces."""
    tune("n_lists", 1)
    tune("t_lists", 1)
    tune("nl_piece_cols", 1024)
    rng = np.random.default_rng(5)
    n, m, r = 3000, 20000, 128
    rowptr, colind, vals, _ = d.synth_pef_host(n, m, k_fixed=5000, zipf_s=1.1, seed=2)
    A = d.Csr.from_host(rowptr, colind, vals, m)
    H = rng.random((m, r)).astype(np.float32)
    W = rng.random((n, r)).astype(np.float32)
    dN, dT = d.DeviceArray((n, r)), d.DeviceArray((m, r))
    d.op_spmm_n(A, r, d.DeviceArray.from_numpy(H), dN)
    d.op_spmm_t(A, r, d.DeviceArray.from_numpy(W), dT)
    assert _row_rel(dN.numpy().astype(np.float64), orc.spmm_n_f64(rowptr, colind, vals, H)) < TOL
    assert _row_rel(dT.numpy().astype(np.float64), orc.spmm_t_f64(rowptr, colind, vals, m, W)) < TOL
    A.close()


@pytest.mark.parametrize("r,n", [(256, 2100), (128, 1300)])
def test_nmf_on_slices_matches_oracle_and_inspection_after_consume(r, n, tune):
    """A factorisation whose sparse products both run on component slices, with a dense head and a
    consumed matrix: 20 iterations against the fp64 oracle from the same seeded factors (1e-4), the
    rows of the matrix read back from the slot lists, and the same bits from a second run."""
    tune("n_lists", 1)
    tune("t_lists", 1)
    tune("nl_piece_cols", 2048)
    m_full, k, iters, eps, seed = 100000, 2000, 20, 1e-12, 77
    A, norms = d.Csr.synth(n, m_full, k_fixed=k, zipf_s=1.3, seed=seed)
    A.normalize_rows(norms)
    A.compact_columns(1)
    rp, ci, va = A.download()
    m = A.n_cols
    nmf = d.MuNmf(A, d.MuNmfParams(rank=r, max_iters=iters, eps=eps, seed=seed, log_every=10), consume_matrix=True)
    assert A.head_info()[0] > 0
    for i in (0, 7, n // 2, n - 1):
        cols, vals = A.get_row(i)
        o = np.argsort(cols, kind="stable")
        want_c, want_v = ci[rp[i]:rp[i + 1]], va[rp[i]:rp[i + 1]]
        ow = np.argsort(want_c, kind="stable")
        assert np.array_equal(cols[o], want_c[ow]) and np.array_equal(vals[o], want_v[ow])
    nmf.initialize()
    W0, H0 = nmf.loadWToHostSync(), nmf.loadHToHostSync()
    hist = nmf.run(log=lambda s: None)
    W, H = nmf.loadWToHostSync(), nmf.loadHToHostSync()
    W64, H64, losses = orc.nmf_f64(rp, ci, va, m, W0, H0, np.float32(eps), iters, 10)
    assert np.linalg.norm(W - W64) / np.linalg.norm(W64) < 1e-4
    assert np.linalg.norm(H - H64) / np.linalg.norm(H64) < 1e-4
    assert abs(hist[-1][1] - losses[-1]) / losses[-1] < 1e-4
    via_rows, via_cols = nmf.check_products()
    assert abs(via_rows - via_cols) <= 5e-6 * abs(via_rows)
    nmf.initialize()
    nmf.run(log=lambda s: None)
    assert np.array_equal(nmf.loadWToHostSync(), W) and np.array_equal(nmf.loadHToHostSync(), H)
    nmf.close()
    A.close()


def _tail_plan(tune, r, piece_cols=2000, sweep_min=50):
    """Six coarse panels of which the widest (the last) holds too few entries per row and piece to
    be swept: with n_lists = 2 its entries go to slot lists, the others stay panels and pieces."""
    tune("n_lists", 2)
    tune("panels", 6)
    tune("sweep_bytes", piece_cols * 4 * min(r, 256))  # (ranks above 256 are swept in slices of 256)
    tune("sweep_min", sweep_min)
    tune("nl_piece_cols", 1024)


@pytest.mark.parametrize("r", [64, 128, 256, 512])
def test_far_tail_from_slot_lists_beside_panels_and_pieces(r, tune):
    _tail_plan(tune, r)
    rng = np.random.default_rng(r)
    n, m_full = 300, 40000
    rowptr, colind, vals, _ = d.synth_pef_host(n, m_full, k_fixed=2048, zipf_s=1.1, seed=9)
    A = d.Csr.from_host(rowptr, colind, vals, m_full)
    H = rng.random((m_full, r)).astype(np.float32)
    dH, dN = d.DeviceArray.from_numpy(H), d.DeviceArray((n, r))
    d.op_spmm_n(A, r, dH, dN)
    info = A.products_info()
    assert info["tail_floor"] > 0 and info["swept_pieces"] > 0
    want_tail = int((colind >= info["tail_floor"]).sum())
    assert info["list_entries"] == want_tail and 0 < want_tail < len(colind)
    N = dN.numpy()
    assert _row_rel(N.astype(np.float64), orc.spmm_n_f64(rowptr, colind, vals, H)) < TOL
    d.op_spmm_n(A, r, dH, dN)
    assert np.array_equal(dN.numpy(), N)
    # the same product without the lists: same sums up to the order of the tail's entries
    tune("n_lists", 0)
    d.op_spmm_n(A, r, dH, dN)
    assert A.products_info()["tail_floor"] == 0
    assert _row_rel(dN.numpy().astype(np.float64), N.astype(np.float64)) < TOL
    A.close()


def test_nmf_with_the_far_tail_on_slot_lists(tune):
    """A factorisation (dense head, consumed matrix) whose far tail runs from slot lists: 20
    iterations against the fp64 oracle, rows read back from panels + lists, same bits again."""
    r, n = 256, 2100
    tune("n_lists", 2)
    tune("panels", 8)
    tune("sweep_bytes", 3000 * 4 * r)
    tune("sweep_min", 40)
    tune("nl_piece_cols", 2048)
    m_full, k, iters, eps, seed = 100000, 2000, 20, 1e-12, 78
    A, norms = d.Csr.synth(n, m_full, k_fixed=k, zipf_s=1.3, seed=seed)
    A.normalize_rows(norms)
    A.compact_columns(1)
    rp, ci, va = A.download()
    m = A.n_cols
    nmf = d.MuNmf(A, d.MuNmfParams(rank=r, max_iters=iters, eps=eps, seed=seed, log_every=10), consume_matrix=True)
    info = A.products_info()
    assert info["tail_floor"] > 0 and info["list_entries"] > 0 and info["swept_pieces"] > 0, info
    for i in (0, 7, n // 2, n - 1):
        cols, vals = A.get_row(i)
        o = np.argsort(cols, kind="stable")
        want_c, want_v = ci[rp[i]:rp[i + 1]], va[rp[i]:rp[i + 1]]
        ow = np.argsort(want_c, kind="stable")
        assert np.array_equal(cols[o], want_c[ow]) and np.array_equal(vals[o], want_v[ow])
    nmf.initialize()
    W0, H0 = nmf.loadWToHostSync(), nmf.loadHToHostSync()
    hist = nmf.run(log=lambda s: None)
    W, H = nmf.loadWToHostSync(), nmf.loadHToHostSync()
    W64, H64, losses = orc.nmf_f64(rp, ci, va, m, W0, H0, np.float32(eps), iters, 10)
    assert np.linalg.norm(W - W64) / np.linalg.norm(W64) < 1e-4
    assert np.linalg.norm(H - H64) / np.linalg.norm(H64) < 1e-4
    assert abs(hist[-1][1] - losses[-1]) / losses[-1] < 1e-4
    via_rows, via_cols = nmf.check_products()
    assert abs(via_rows - via_cols) <= 5e-6 * abs(via_rows)
    nmf.initialize()
    nmf.run(log=lambda s: None)
    assert np.array_equal(nmf.loadWToHostSync(), W) and np.array_equal(nmf.loadHToHostSync(), H)
    nmf.close()
    A.close()


def test_far_tail_stays_panels_when_its_lists_would_not_fit(tune):
    """With no memory allowed beyond the panel copy the lists are declined, the tail stays plain
    panels, and later plans of the same (by then consumed) matrix come to the same answer."""
    r, n = 256, 2100
    tune("n_lists", 2)
    tune("nl_extra_mb", 0)
    tune("panels", 8)
    tune("sweep_bytes", 3000 * 4 * r)
    tune("sweep_min", 40)
    m_full, k, iters, eps, seed = 100000, 2000, 5, 1e-12, 79
    A, norms = d.Csr.synth(n, m_full, k_fixed=k, zipf_s=1.3, seed=seed)
    A.normalize_rows(norms)
    A.compact_columns(1)
    rp, ci, va = A.download()
    nmf = d.MuNmf(A, d.MuNmfParams(rank=r, max_iters=iters, eps=eps, seed=seed, log_every=5), consume_matrix=True)
    info = A.products_info()
    assert info["tail_floor"] == 0 and info["list_entries"] == 0 and info["swept_pieces"] > 0 and info["plain"] > 1, info
    nmf.initialize()
    W0, H0 = nmf.loadWToHostSync(), nmf.loadHToHostSync()
    nmf.run(log=lambda s: None)
    W64, H64, _ = orc.nmf_f64(rp, ci, va, A.n_cols, W0, H0, np.float32(eps), iters, 5)
    assert np.linalg.norm(nmf.loadWToHostSync() - W64) / np.linalg.norm(W64) < 1e-4
    assert A.products_info() == info
    nmf.close()
    A.close()


def test_far_tail_lists_with_ragged_empty_and_tail_only_rows(tune):
    """Rows of 16 ... 4,096 entries, two empty rows, one row with entries in the far tail only and
    one with none there: the panel copy without the tail and the lists must split every row where
    its entries say, wherever they stand in the row."""
    r = 256
    _tail_plan(tune, r, piece_cols=1500, sweep_min=12)
    rng = np.random.default_rng(11)
    n, m_full = 420, 60000
    rowptr, colind, vals, _ = d.synth_pef_host(n, m_full, k_fixed=0, k_min=16, k_max=4096, zipf_s=1.1, seed=21)
    keep = np.ones(len(colind), dtype=bool)
    row_of = np.repeat(np.arange(n), np.diff(rowptr))
    keep[(row_of == 1) | (row_of == n - 1)] = False                 # empty rows
    keep[(row_of == 5) & (colind < 30000)] = False                  # far columns only
    keep[(row_of == 6) & (colind >= 2000)] = False                  # near columns only
    colind, vals = colind[keep], vals[keep]
    rowptr = np.concatenate([[0], np.cumsum(np.bincount(row_of[keep], minlength=n))]).astype(np.int64)
    A = d.Csr.from_host(rowptr, colind, vals, m_full)
    H = rng.random((m_full, r)).astype(np.float32)
    dH, dN = d.DeviceArray.from_numpy(H), d.DeviceArray((n, r))
    d.op_spmm_n(A, r, dH, dN)
    info = A.products_info()
    assert info["tail_floor"] > 0 and info["swept_pieces"] > 0, info
    assert info["list_entries"] == int((colind >= info["tail_floor"]).sum())
    assert 2000 < info["tail_floor"] <= 30000  # rows 5 and 6 lie on one side each
    N = dN.numpy()
    want = orc.spmm_n_f64(rowptr, colind, vals, H)
    assert _row_rel(N[[i for i in range(n) if i not in (1, n - 1)]].astype(np.float64),
                    want[[i for i in range(n) if i not in (1, n - 1)]]) < TOL
    assert np.all(N[1] == 0) and np.all(N[n - 1] == 0)
    for i in (0, 1, 5, 6, n - 1):
        cols, got = A.get_row(i)
        o, ow = np.argsort(cols, kind="stable"), np.argsort(colind[rowptr[i]:rowptr[i + 1]], kind="stable")
        assert np.array_equal(cols[o], colind[rowptr[i]:rowptr[i + 1]][ow])
        assert np.array_equal(got[o], vals[rowptr[i]:rowptr[i + 1]][ow])
    A.close()
