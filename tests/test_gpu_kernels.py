"""Each HIP kernel through its own C-ABI entry point vs the fp64 CPU oracle.

Tolerances: the kernels compute in fp32 with fp32 (MFMA / FMA) accumulation over blocked
partial sums; against fp64 the bound used is 2e-5 relative to the largest magnitude of the
output (norm-wise), far inside the 1e-4 the full 50-iteration run has to meet."""

import numpy as np
import pytest

import npeff_ref_amd as d
from conftest import csr_to_dense, random_csr
from oracle import oracle as orc

pytestmark = pytest.mark.gpu

TOL = 2e-5


def _rel(a, b):
    return np.abs(a.astype(np.float64) - b).max() / max(np.abs(b).max(), 1e-300)


def test_mu_bit_exact():
    rng = np.random.default_rng(0)
    n = 100003
    F, num, den = (rng.random(n).astype(np.float32) for _ in range(3))
    eps = np.float32(1e-8)
    dF, dn, dd = d.DeviceArray.from_numpy(F), d.DeviceArray.from_numpy(num), d.DeviceArray.from_numpy(den)
    d.op_mu(dF, dn, dd, eps)
    want = (F * (num / (den + eps))).astype(np.float32)  # divide first, then multiply
    assert np.array_equal(dF.numpy(), want)


@pytest.mark.parametrize("r", [16, 50, 64, 128, 256, 512])
@pytest.mark.parametrize("shape", [(37, 900, 60), (130, 5000, 3000)])
def test_spmm_n_and_t(r, shape):
    n, m, maxk = shape
    rng = np.random.default_rng(r + n)
    rp, ci, va = random_csr(rng, n, m, maxk, empty_rows={1, n - 1})
    A = d.Csr.from_host(rp, ci, va, m)
    H = rng.random((m, r)).astype(np.float32)
    W = rng.random((n, r)).astype(np.float32)
    dH, dW = d.DeviceArray.from_numpy(H), d.DeviceArray.from_numpy(W)
    dN, dT = d.DeviceArray((n, r)), d.DeviceArray((m, r))
    d.op_spmm_n(A, r, dH, dN)
    d.op_spmm_t(A, r, dW, dT)
    N, T = dN.numpy(), dT.numpy()
    assert _rel(N, orc.spmm_n_f64(rp, ci, va, H)) < TOL
    assert _rel(T, orc.spmm_t_f64(rp, ci, va, m, W)) < TOL
    assert np.all(N[1] == 0) and np.all(N[n - 1] == 0)  # empty rows
    # reproducible bit for bit
    d.op_spmm_n(A, r, dH, dN)
    d.op_spmm_t(A, r, dW, dT)
    assert np.array_equal(dN.numpy(), N) and np.array_equal(dT.numpy(), T)
    A.close()


def test_spmm_long_rows_and_long_columns():
    """Rows spanning several work chunks and columns long enough for the workgroup path."""
    rng = np.random.default_rng(5)
    n, m, r = 700, 20000, 128
    rowptr, colind, vals, _ = d.synth_pef_host(n, m, k_fixed=5000, zipf_s=1.1, seed=2)
    A = d.Csr.from_host(rowptr, colind, vals, m)
    H = rng.random((m, r)).astype(np.float32)
    W = rng.random((n, r)).astype(np.float32)
    dN, dT = d.DeviceArray((n, r)), d.DeviceArray((m, r))
    d.op_spmm_n(A, r, d.DeviceArray.from_numpy(H), dN)
    d.op_spmm_t(A, r, d.DeviceArray.from_numpy(W), dT)
    assert _rel(dN.numpy(), orc.spmm_n_f64(rowptr, colind, vals, H)) < TOL
    assert _rel(dT.numpy(), orc.spmm_t_f64(rowptr, colind, vals, m, W)) < TOL
    A.close()


@pytest.mark.parametrize("rows,r", [(1, 16), (31, 16), (2, 1), (100001, 7), (70000, 32), (333333, 24), (1000, 50), (4097, 128), (20000, 256), (9000, 512), (300, 130),
                                     (1025, 1024), (5000, 384), (1023, 256)])
def test_gram(rows, r):
    rng = np.random.default_rng(rows + r)
    X = rng.random((rows, r)).astype(np.float32)
    dG = d.DeviceArray((r, r))
    d.op_gram(d.DeviceArray.from_numpy(X), dG)
    G = dG.numpy()
    want = orc.gram_f64(X)
    assert _rel(G, want) < TOL
    assert np.array_equal(G, G.T) or _rel(G, G.T.astype(np.float64)) < 1e-6


@pytest.mark.parametrize("fold", [2, 1, 0])
@pytest.mark.parametrize("rows,r", [(4096, 256), (20011, 256), (3000, 384), (2500, 1024), (9000, 512), (1500, 768), (31, 256),
                                    (64, 512)])
def test_gram_diagonal_tiles_with_and_without_their_symmetry(rows, r, fold, tune):
    """X^T X at the ranks that run on tiles, with signed entries over eight decades (a partial
    product taken from the wrong side of the diagonal, or left out, shows at 2^-8 or 2^-16 of the
    element): the diagonal tiles two and two as squares of 256 columns in one workgroup (36 of 64
    blocks, a block in two halves; at ranks that are multiples of 256), each by itself with its
    symmetry used (ten blocks, four products on the diagonal ones), and plain."""
    tune("gram_fold", fold)
    rng = np.random.default_rng(rows + r + fold)
    X = (rng.standard_normal((rows, r)) * 10.0 ** rng.uniform(-4, 4, size=(1, r))).astype(np.float32)
    dG = d.DeviceArray((r, r))
    d.op_gram(d.DeviceArray.from_numpy(X), dG)
    G = dG.numpy()
    want = orc.gram_f64(X)
    scale = np.sqrt(np.outer(np.diag(want), np.diag(want)))  # |G_ab| <= sqrt(G_aa G_bb)
    assert np.all(np.abs(G - want) <= 2e-6 * scale)
    assert np.array_equal(G, G.T)
    d.op_gram(d.DeviceArray.from_numpy(X), dG)
    assert np.array_equal(dG.numpy(), G)


@pytest.mark.parametrize("rows,r", [(1, 16), (33, 16), (1000, 50), (4100, 128), (5000, 256), (3000, 512), (300, 130),
                                    (700, 64), (1000, 100), (513, 36), (300, 20), (257, 32), (70001, 128),
                                    (140000, 64), (256, 128), (255, 128), (1001, 384), (40000, 256), (257, 1024)])
def test_xg_mu(rows, r):
    rng = np.random.default_rng(rows * 3 + r)
    X = rng.random((rows, r)).astype(np.float32)
    G = rng.random((r, r)).astype(np.float32)  # deliberately not symmetric
    num = rng.random((rows, r)).astype(np.float32)
    eps = np.float32(1e-8)
    dX, dG, dnum = d.DeviceArray.from_numpy(X), d.DeviceArray.from_numpy(G), d.DeviceArray.from_numpy(num)
    dout, dD = d.DeviceArray((rows, r)), d.DeviceArray((rows, r))
    d.op_xg_mu(dX, dG, dnum, eps, dout, dD)
    want, wantD = orc.xg_mu_f64(X, G, num, eps)
    assert _rel(dD.numpy(), wantD) < TOL
    assert _rel(dout.numpy(), want) < TOL
    # in place on the numerator buffer gives the same bits
    out1 = dout.numpy()
    d.op_xg_mu(dX, dG, dnum, eps, dnum, None)
    assert np.array_equal(dnum.numpy(), out1)


@pytest.mark.parametrize("rows,r", [(128, 256), (4100, 256), (40000, 256), (3000, 512), (700, 1024), (1001, 384),
                                    (400000, 256)])
def test_xg_mu_tiles_with_two_and_three_workgroups_per_cu(rows, r, tune):
    """The update at ranks from 256 on planes without padding (three workgroups per CU, one
    operand stage, the default) and on padded planes (two, two stages): the same products in the
    same order, so the same bits, and both within the fp32 bar of the fp64 result."""
    rng = np.random.default_rng(rows + r)
    X = (rng.random((rows, r)) * 10.0 ** rng.uniform(-3, 3, size=(1, r))).astype(np.float32)
    G = rng.random((r, r)).astype(np.float32)
    num = rng.random((rows, r)).astype(np.float32)
    eps = np.float32(1e-8)
    dX, dG, dnum = d.DeviceArray.from_numpy(X), d.DeviceArray.from_numpy(G), d.DeviceArray.from_numpy(num)
    outs = []
    for wgs in (4, 2):  # (4: three per CU whatever the size; 3, the default, only for launches that fill the CUs eight times)
        tune("xg_wgs", wgs)
        dout, dD = d.DeviceArray((rows, r)), d.DeviceArray((rows, r))
        d.op_xg_mu(dX, dG, dnum, eps, dout, dD)
        outs.append((dout.numpy(), dD.numpy()))
        dout2 = d.DeviceArray((rows, r))
        d.op_xg_mu(dX, dG, dnum, eps, dout2, None)
        assert np.array_equal(dout2.numpy(), outs[-1][0])
    want, wantD = orc.xg_mu_f64(X, G, num, eps)
    assert _rel(outs[0][1], wantD) < TOL and _rel(outs[0][0], want) < TOL
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])
    tune("xg_wgs", 3)
    dout = d.DeviceArray((rows, r))
    d.op_xg_mu(dX, dG, dnum, eps, dout, None)
    assert np.array_equal(dout.numpy(), outs[0][0])


@pytest.mark.parametrize("split", ["1", "0"])
@pytest.mark.parametrize("rows", [64, 95, 4100, 70001, 300033])
def test_xg_mu_gram_fused(rows, split, tune):
    """Rank 128, update and Gram matrix of the result in one pass: on the bf16 matrix cores with
    every operand split in three (default) and on the fp32 ones.  Both must meet the fp32 bar;
    the operands span 12 decades and hold zeros, so the split's low parts matter."""
    tune("split_bf16", float(split))
    r = 128
    rng = np.random.default_rng(rows)
    X = (rng.random((rows, r)) * 10.0 ** rng.uniform(-6, 0, (rows, r))).astype(np.float32)
    X[rng.random((rows, r)) < 0.05] = 0.0
    G = (rng.random((r, r)) * 10.0 ** rng.uniform(-3, 3, (r, r))).astype(np.float32)
    num = (rng.random((rows, r)) * 10.0 ** rng.uniform(-3, 3, (rows, r))).astype(np.float32)
    eps = np.float32(1e-12)
    dX, dG, dnum = d.DeviceArray.from_numpy(X), d.DeviceArray.from_numpy(G), d.DeviceArray.from_numpy(num)
    dout, dGo = d.DeviceArray((rows, r)), d.DeviceArray((r, r))
    d.op_xg_mu_gram(dX, dG, dnum, eps, dout, dGo)
    want, _ = orc.xg_mu_f64(X, G, num, eps)
    out = dout.numpy()
    # element-wise: every entry to a few fp32 ulps, not only the norm
    ok = np.abs(out - want) <= 2e-6 * np.abs(want) + 1e-30
    assert ok.all(), float(np.max(np.abs(out - want) / (np.abs(want) + 1e-30)))
    Go = dGo.numpy()
    wantG = orc.gram_f64(out)
    assert _rel(Go, wantG) < 2e-6
    assert np.array_equal(Go, Go.T)
    # in place on the numerator buffer gives the same bits
    d.op_xg_mu_gram(dX, dG, dnum, eps, dnum, dGo)
    assert np.array_equal(dnum.numpy(), out)
    assert np.array_equal(dGo.numpy(), Go)


def test_dot_fp64_accumulation():
    rng = np.random.default_rng(1)
    n = 3_000_001
    x, y = rng.random(n).astype(np.float32), rng.random(n).astype(np.float32)
    got = d.op_dot(d.DeviceArray.from_numpy(x), d.DeviceArray.from_numpy(y))
    want = np.dot(x.astype(np.float64), y.astype(np.float64))
    assert abs(got - want) / want < 1e-13


def test_init_uniform_matches_host_rule():
    seed, n, r, m = 43190432042, 37, 16, 211
    dW, dH = d.DeviceArray((n, r)), d.DeviceArray((m, r))
    d.op_init_uniform(0, n, r, seed, dW)
    d.op_init_uniform(1, r, m, seed, dH)
    W, Ht = dW.numpy(), dH.numpy()
    for i, c in [(0, 0), (5, 3), (36, 15)]:
        assert W[i, c] == np.float32(d.uniform_at(seed, 0, i, c, r))
    for c, j in [(0, 0), (7, 100), (15, 210)]:
        assert Ht[j, c] == np.float32(d.uniform_at(seed, 1, c, j, m))


@pytest.mark.parametrize("r", [16, 100, 256])
def test_spsp_dense(r):
    rng = np.random.default_rng(40 + r)
    n, m = 150, 6000
    a = random_csr(rng, n, m, 3000, empty_rows={2})
    b = random_csr(rng, r, m, 400, sort_cols=True)
    A, B = d.Csr.from_host(*a, m), d.Csr.from_host(*b, m)
    out = d.DeviceArray((n, r))
    d.op_spsp_dense(A, B, out)
    first = out.numpy()
    assert _rel(first, orc.spsp_dense_f64(a, m, b, r)) < TOL
    for _ in range(3):  # lanes that meet in a component are added in a fixed order
        d.op_spsp_dense(A, B, out)
        assert np.array_equal(out.numpy(), first)
    hh = d.DeviceArray((r, r))
    d.op_spsp_dense(B, B, hh)
    assert _rel(hh.numpy(), orc.spsp_dense_f64(b, m, b, r)) < TOL
    A.close()
    B.close()


@pytest.mark.parametrize("slices,r", [(2, 128), (4, 256), (8, 512), (4, 64)])
def test_spmm_t_component_slices(slices, r, tune):
    """The sliced launch of A^T W (one slice of the components per workgroup)."""
    tune("spmm_t_slices", slices)
    rng = np.random.default_rng(slices + r)
    n, m = 3000, 30000
    rowptr, colind, vals, _ = d.synth_pef_host(n, m, k_fixed=300, zipf_s=1.1, seed=7)
    A = d.Csr.from_host(rowptr, colind, vals, m)
    W = rng.random((n, r)).astype(np.float32)
    dT = d.DeviceArray((m, r))
    d.op_spmm_t(A, r, d.DeviceArray.from_numpy(W), dT)
    T = dT.numpy()
    want = orc.spmm_t_f64(rowptr, colind, vals, m, W)
    # row-wise: short columns have small sums that a max-normalised check would hide
    err = np.abs(T - want).max(axis=1) / (np.abs(want).max(axis=1) + 1e-300)
    assert err.max() < TOL
    A.close()


def test_spmm_t_more_columns_than_one_pass_of_the_grid():
    """36M columns: more (column, slice) work items than workgroups in the capped grid, so every
    workgroup walks several column groups; columns without entries must come out as zeros."""
    n, m, r = 64, 36_000_000, 16
    rng = np.random.default_rng(3)
    rp, ci, va = random_csr(rng, n, m, 500)
    A = d.Csr.from_host(rp, ci, va, m)
    W = rng.random((n, r)).astype(np.float32)
    dT = d.DeviceArray((m, r))
    d.op_init_uniform(0, m, r, 5, dT)  # stale contents that must all be overwritten
    d.op_spmm_t(A, r, d.DeviceArray.from_numpy(W), dT)
    T = dT.numpy()
    used = np.unique(ci)
    want = orc.spmm_t_f64(rp, ci, va, m, W)[used]
    assert _rel(T[used], want) < TOL
    mask = np.ones(m, dtype=bool)
    mask[used] = False
    assert not T[mask].any()
    A.close()


def _hot_column_matrix(rng, n, m, hot, k_tail, dup=False):
    """Rows holding most of `hot` columns (each kept with probability 0.8) plus random others."""
    hot_cols = rng.choice(m, size=hot, replace=False)
    others = np.setdiff1d(np.arange(m), hot_cols)
    rowptr, cols, vals = [0], [], []
    for i in range(n):
        c = np.concatenate([hot_cols[rng.random(hot) < 0.8],
                            rng.choice(others, size=int(rng.integers(0, k_tail + 1)), replace=False)])
        if dup and i % 7 == 0 and len(c):
            c = np.concatenate([c, c[:3]])  # repeated (row, column) pairs add up
        rng.shuffle(c)
        cols.append(c.astype(np.int32))
        vals.append(rng.lognormal(-2.0, 1.0, size=len(c)).astype(np.float32))
        rowptr.append(rowptr[-1] + len(c))
    return (np.array(rowptr, dtype=np.int64), np.concatenate(cols).astype(np.int32),
            np.concatenate(vals).astype(np.float32), np.sort(hot_cols))


@pytest.mark.parametrize("n,m,hot,r", [(300, 4000, 70, 128), (1030, 9000, 300, 64), (257, 3000, 129, 256),
                                       (140, 2000, 40, 36), (500, 2500, 33, 512)])
def test_dense_head_products(n, m, hot, r):
    """Columns held by many rows move to a dense block; A H^T and A^T W stay the same sums."""
    rng = np.random.default_rng(n + r)
    rp, ci, va, hot_cols = _hot_column_matrix(rng, n, m, hot, 40)
    A = d.Csr.from_host(rp, ci, va, m)
    H = rng.random((m, r)).astype(np.float32)
    W = rng.random((n, r)).astype(np.float32)
    dH, dW = d.DeviceArray.from_numpy(H), d.DeviceArray.from_numpy(W)
    dN, dT = d.DeviceArray((n, r)), d.DeviceArray((m, r))
    n_dense = A.split_dense_head(0.5)
    assert n_dense == hot
    nd, z_sparse = A.head_info()
    in_head = np.isin(ci, hot_cols)
    assert nd == hot and z_sparse == int((~in_head).sum())
    d.op_spmm_n(A, r, dH, dN)
    d.op_spmm_t(A, r, dW, dT)
    N, T = dN.numpy(), dT.numpy()
    N64, T64 = orc.spmm_n_f64(rp, ci, va, H), orc.spmm_t_f64(rp, ci, va, m, W)
    # row-wise: a wrong head row must not hide behind a large one
    assert (np.abs(N - N64).max(axis=1) / np.maximum(np.abs(N64).max(axis=1), 1e-30)).max() < TOL
    scale = np.maximum(np.abs(T64).max(axis=1), 1e-30)
    assert (np.abs(T - T64).max(axis=1) / scale)[np.abs(T64).max(axis=1) > 0].max() < TOL
    assert np.all(T[np.abs(T64).max(axis=1) == 0] == 0)
    # the loader still sees the whole matrix, and the split can be undone
    rp2, ci2, va2 = A.download()
    assert np.array_equal(ci2, ci) and np.array_equal(va2, va)
    d.op_spmm_n(A, r, dH, dN)
    assert np.array_equal(dN.numpy(), N)
    assert A.split_dense_head(0.0) == 0 and A.head_info() == (0, len(ci))
    d.op_spmm_n(A, r, dH, dN)
    assert _rel(dN.numpy(), N64) < TOL
    A.close()


def test_duplicate_entries_are_refused_by_the_products():
    """A row that holds a column twice has no deterministic transposed copy: the loader still
    takes the matrix (the reference's loader does not look either), the products refuse it."""
    rng = np.random.default_rng(8)
    rp, ci, va, _ = _hot_column_matrix(rng, 200, 3000, 30, 40, dup=True)
    A = d.Csr.from_host(rp, ci, va, 3000)
    assert np.array_equal(A.download()[1], ci)
    with pytest.raises(d.DnpeffError, match="duplicate"):
        A.build_transpose()
    H = d.DeviceArray.from_numpy(rng.random((3000, 64)).astype(np.float32))
    with pytest.raises(d.DnpeffError, match="duplicate"):
        d.op_spmm_n(A, 64, H, d.DeviceArray((200, 64)))
    # the repeated pairs sit in columns that most rows hold: moving those to the dense head (which
    # would otherwise add them up, in an order of the hardware's choosing) finds them too
    with pytest.raises(d.DnpeffError, match="duplicate"):
        A.split_dense_head(0.5)
    A.close()


def test_spmm_t_is_bit_identical_on_a_rerun():
    rng = np.random.default_rng(21)
    n, m, r = 2000, 20000, 128
    rowptr, colind, vals, _ = d.synth_pef_host(n, m, k_fixed=400, zipf_s=1.1, seed=5)
    A = d.Csr.from_host(rowptr, colind, vals, m)
    dW = d.DeviceArray.from_numpy(rng.random((n, r)).astype(np.float32))
    T1, T2 = d.DeviceArray((m, r)), d.DeviceArray((m, r))
    d.op_spmm_t(A, r, dW, T1)
    d.op_spmm_t(A, r, dW, T2)
    d.sync()
    assert np.array_equal(T1.numpy(), T2.numpy())
    A.close()
    # a second build of the transposed copy gives the same arrays
    B = d.Csr.from_host(rowptr, colind, vals, m)
    A2 = d.Csr.from_host(rowptr, colind, vals, m)
    for x, y in zip(B.download_transpose(), A2.download_transpose()):
        assert np.array_equal(x, y)
    B.close()
    A2.close()


def test_dense_head_needs_rank_multiple_of_4():
    rng = np.random.default_rng(3)
    rp, ci, va, _ = _hot_column_matrix(rng, 100, 1000, 20, 10)
    A = d.Csr.from_host(rp, ci, va, 1000)
    assert A.split_dense_head(0.5) == 20
    H = d.DeviceArray.from_numpy(rng.random((1000, 50)).astype(np.float32))
    with pytest.raises(RuntimeError, match="multiple of 4"):
        d.op_spmm_n(A, 50, H, d.DeviceArray((100, 50)))
    A.close()


@pytest.mark.parametrize("panels,r,n,m,maxk", [(8, 128, 130, 5000, 3000), (37, 64, 61, 900, 400), (256, 50, 300, 20000, 700), (512, 32, 40, 30000, 2000),
                                               (2, 16, 5, 40, 30)])
def test_spmm_n_column_panels(panels, r, n, m, maxk, tune):
    """Entries regrouped by column panel, one wave per (row, panel) segment: same sums, same bits
    on every run, empty rows and empty segments included."""
    tune("panels", panels)
    rng = np.random.default_rng(panels + r)
    rp, ci, va = random_csr(rng, n, m, maxk, empty_rows={1, n - 1})
    A = d.Csr.from_host(rp, ci, va, m)
    H = rng.random((m, r)).astype(np.float32)
    dH, dN = d.DeviceArray.from_numpy(H), d.DeviceArray((n, r))
    d.op_spmm_n(A, r, dH, dN)
    N = dN.numpy()
    N64 = orc.spmm_n_f64(rp, ci, va, H)
    assert (np.abs(N - N64).max(axis=1) / np.maximum(np.abs(N64).max(axis=1), 1e-30)).max() < TOL
    assert np.all(N[1] == 0) and np.all(N[n - 1] == 0)
    d.op_spmm_n(A, r, dH, dN)
    assert np.array_equal(dN.numpy(), N)
    # the other product and the loader are untouched by the regrouping
    W = rng.random((n, r)).astype(np.float32)
    dT = d.DeviceArray((m, r))
    d.op_spmm_t(A, r, d.DeviceArray.from_numpy(W), dT)
    assert _rel(dT.numpy(), orc.spmm_t_f64(rp, ci, va, m, W)) < TOL
    assert np.array_equal(A.download()[1], ci)
    # without panels: the chunked path again
    tune("panels", 0)
    d.op_spmm_n(A, r, dH, dN)
    assert _rel(dN.numpy(), N64) < TOL
    A.close()


@pytest.mark.parametrize("r,n,m,maxk,panels,sweep_bytes,waves", [
    (128, 2700, 6000, 900, 4, 64 * 512, 1),      # two passes, 64-column pieces
    (128, 130, 3000, 2500, 3, 300 * 512, 8),     # the 5 segments of a wave hold several batches of 64
    (64, 1500, 9000, 60, 8, 500 * 256, 1),       # short segments, many empty; 3 lane groups idle
    (32, 333, 5000, 300, 5, 200 * 128, 2),
    (256, 90, 2000, 700, 2, 400 * 1024, 8),      # 6 pieces: two XCDs have none
    (128, 40, 50000, 300, 16, 1000 * 512, 8),
    (128, 40, 50000, 300, 16, 4 * 512, 8),       # more pieces than the split handles: fewer panels get cut
    (64, 200, 4000, 3000, 2, 300 * 256, 8),      # long segments at 4 lane groups (several batches of 64)
    (32, 150, 3000, 2500, 2, 400 * 128, 4),      # long segments at 8 lane groups (shuffles, no row broadcasts)
    (256, 120, 3000, 2800, 2, 500 * 1024, 6),    # long segments at one lane group (4 rows of 16 lanes)
    (512, 90, 2000, 700, 2, 400 * 1024, 8),      # rank above 256: two slices of 256 components
    (384, 70, 1500, 500, 3, 300 * 512, 4),       # three slices of 128
    (1024, 40, 900, 400, 2, 200 * 1024, 2),      # four slices of 256
])
def test_spmm_n_swept_panels(r, n, m, maxk, panels, sweep_bytes, waves, tune):
    """Coarse panels cut into L2-sized pieces that one XCD sweeps for all rows, running sums in
    registers: same sums as the fp64 restatement, same bits on every run, empty rows included; a
    factor that is not 16-byte aligned takes the 4-byte loads."""
    tune("panels", panels)
    tune("sweep_bytes", sweep_bytes)
    tune("sweep_min", 0)
    tune("sweep_waves", waves)
    rng = np.random.default_rng(r + n)
    rp, ci, va = random_csr(rng, n, m, maxk, empty_rows={0, n // 2})
    A = d.Csr.from_host(rp, ci, va, m)
    H = rng.random((m, r)).astype(np.float32)
    dH, dN = d.DeviceArray.from_numpy(H), d.DeviceArray((n, r))
    d.op_spmm_n(A, r, dH, dN)
    N = dN.numpy()
    N64 = orc.spmm_n_f64(rp, ci, va, H)
    assert (np.abs(N - N64).max(axis=1) / np.maximum(np.abs(N64).max(axis=1), 1e-30)).max() < TOL
    assert np.all(N[0] == 0) and np.all(N[n // 2] == 0)
    d.op_spmm_n(A, r, dH, dN)
    assert np.array_equal(dN.numpy(), N)
    # the same factor one float further on: not 16-byte aligned
    import ctypes, types
    shifted = d.DeviceArray.from_numpy(np.concatenate([np.zeros(1, np.float32), H.ravel()]))
    view = types.SimpleNamespace(ptr=ctypes.c_void_p(shifted.ptr.value + 4))
    d.op_spmm_n(A, r, view, dN)
    assert (np.abs(dN.numpy() - N64).max(axis=1) / np.maximum(np.abs(N64).max(axis=1), 1e-30)).max() < TOL
    # workgroups that stop waiting for each other after one poll: same bits
    tune("sweep_spin", 1)
    d.op_spmm_n(A, r, dH, dN)
    assert np.array_equal(dN.numpy(), N)
    tune("sweep_spin", 400)
    # without sweeps: every panel one wave per (row, panel) segment
    tune("sweep_bytes", 0)
    d.op_spmm_n(A, r, dH, dN)
    assert _rel(dN.numpy(), N64) < TOL
    A.close()


def test_column_panels_with_dense_head(tune):
    tune("panels", 16)
    rng = np.random.default_rng(11)
    n, m, r = 400, 6000, 128
    rp, ci, va, hot_cols = _hot_column_matrix(rng, n, m, 50, 200)
    A = d.Csr.from_host(rp, ci, va, m)
    assert A.split_dense_head(0.5) == 50
    H = rng.random((m, r)).astype(np.float32)
    dN = d.DeviceArray((n, r))
    d.op_spmm_n(A, r, d.DeviceArray.from_numpy(H), dN)
    N64 = orc.spmm_n_f64(rp, ci, va, H)
    assert (np.abs(dN.numpy() - N64).max(axis=1) / np.abs(N64).max(axis=1)).max() < TOL
    A.close()


@pytest.mark.parametrize("n,div,thr", [(100003, 3.7, 0.1), (5, 1.0, 0.0), (4096, 0.5, 5.0), (70000, 2.0, -1.0)])
def test_threshold_compact_bit_exact(n, div, thr):
    rng = np.random.default_rng(n)
    x = rng.random(n).astype(np.float32)
    idx, val = d.op_threshold_compact(d.DeviceArray.from_numpy(x), div, thr)
    q = (x / np.float32(div)).astype(np.float32)
    keep = q >= np.float32(thr)
    assert np.array_equal(idx, np.nonzero(keep)[0].astype(np.int32))
    assert np.array_equal(val, q[keep])


@pytest.mark.parametrize("n,count,k", [(3, 100000, 4096), (2, 5000, 1), (1, 70001, 70001), (4, 30000, 5000),
                                       (1, 3_000_000, 65536)])
@pytest.mark.parametrize("cap", [None, 0, 9000])
def test_topk_rows_bit_exact(n, count, k, cap, tune):
    """Device top-k sparsifier vs the full-sort restatement: same values, same indices (ties by
    ascending index), zeros and repeated values included; both the two-read path and the
    exact-threshold path for crowded bins (forced with a zero cap)."""
    if cap is not None:
        tune("topk_fast_cap", cap)
    rng = np.random.default_rng(count + k)
    x = rng.lognormal(-8, 2, size=(n, count)).astype(np.float32)
    x[0, ::5] = 0.0
    x[-1, 1::3] = np.float32(0.125)  # far more ties than k when k is small
    if count > 1000:
        x[0, 17] = np.float32(-1.0)  # a negative entry sorts below the zeros
    v, i, nrm = d.topk_rows(d.DeviceArray.from_numpy(x), k)
    wv, wi, wn = orc.topk_rows(x, k)
    assert np.array_equal(v, wv) and np.array_equal(i, wi)
    assert np.all(np.abs(nrm - wn) <= 1e-6 * wn)


def test_row_and_column_inspection_and_gathered_rows():
    """dnpeff_csr_get_row / get_column return the matrix as the products hold it (dense head +
    sparse part), before and after a consuming create; dnpeff_op_gather_rows picks rows of a factor;
    the host generator's row range equals the rows of the whole matrix."""
    rng = np.random.default_rng(17)
    n, m, r = 1100, 9000, 64
    rp, ci, va, hot = _hot_column_matrix(rng, n, m, 120, 60)
    A = d.Csr.from_host(rp, ci, va, m)
    assert A.split_dense_head(0.5) == 120
    nmf = d.MuNmf(A, d.MuNmfParams(rank=r, max_iters=0), consume_matrix=True)
    dense = csr_to_dense(rp, ci, va, m, dtype=np.float32)
    for i in (0, 1, n // 2, n - 1):
        cols, vals = A.get_row(i)
        o = np.argsort(cols, kind="stable")
        want = np.nonzero(dense[i])[0]
        assert np.array_equal(cols[o], want) and np.array_equal(vals[o], dense[i, want])
    for j in list(hot[:3]) + [0, 5, m - 1] + list(rng.integers(0, m, 20)):
        rows, vals = A.get_column(int(j))
        want = np.nonzero(dense[:, j])[0]
        assert np.array_equal(rows, want) and np.array_equal(vals, dense[want, j])
    nmf.initialize()
    w_dev, h_dev = nmf.device_factors()
    H = nmf.loadHToHostSync()
    pick = np.array([5, 0, m - 1, 5, 77], dtype=np.int32)
    assert np.array_equal(d.gather_rows(h_dev, r, pick), H[:, pick].T)
    nmf.close()
    A.close()
    rowptr, colind, vals, norms = d.synth_pef_host(40, 50000, k_min=16, k_max=600, seed=4)
    rp2, ci2, va2, nr2 = d.synth_pef_host_rows(7, 9, 50000, k_min=16, k_max=600, seed=4)
    assert np.array_equal(rp2, rowptr[7:17] - rowptr[7])
    assert np.array_equal(ci2, colind[rowptr[7]:rowptr[16]]) and np.array_equal(va2, vals[rowptr[7]:rowptr[16]])
    assert np.array_equal(nr2, norms[7:16])


@pytest.mark.parametrize("r", [64, 100, 512])
def test_spmm_n_decompositions_agree(r, tune):
    """One wave per row, 2048-entry row chunks, the merge path (equal shares of entries + rows,
    cut wherever the row boundaries fall) and the planned decomposition (forced panels and swept
    pieces) of A H^T on ragged rows, some of them empty: the same sums up to fp32 order, each
    against fp64."""
    tune("panels", 8)
    tune("sweep_bytes", 300 * 4 * min(r, 256))
    tune("sweep_min", 0)
    rowptr, colind, vals, norms = d.synth_pef_host(300, 40000, k_min=8, k_max=6000, seed=r)
    # rows 5, 6 and the last one emptied: end markers only on the merge path
    keep = np.ones(len(colind), dtype=bool)
    lens = np.diff(rowptr)
    for i in (5, 6, 299):
        keep[rowptr[i]:rowptr[i + 1]] = False
        lens[i] = 0
    colind, vals = colind[keep], vals[keep]
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    A = d.Csr.from_host(rowptr, colind, vals, 40000)
    rng = np.random.default_rng(r)
    H = rng.random((40000, r)).astype(np.float32)
    dH, dN = d.DeviceArray.from_numpy(H), d.DeviceArray((300, r))
    N64 = orc.spmm_n_f64(rowptr, colind, vals, H)
    for variant in (1, 2, 3, 0):
        dN = d.DeviceArray.from_numpy(np.full((300, r), np.nan, dtype=np.float32))  # every element must be written
        d.binding._check(d.lib.dnpeff_op_spmm_n_variant(A._h, r, dH.ptr, dN.ptr, variant))
        d.sync()
        N = dN.numpy()
        assert (np.abs(N - N64).max(axis=1) / np.maximum(np.abs(N64).max(axis=1), 1e-30)).max() < TOL
    with pytest.raises(d.DnpeffError, match="variant"):
        d.binding._check(d.lib.dnpeff_op_spmm_n_variant(A._h, r, dH.ptr, dN.ptr, 7))
    A.close()
