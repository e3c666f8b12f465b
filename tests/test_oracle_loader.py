"""Pins the integer/byte part of the CPU oracle: the reference's own known-answer vectors,
the compiled reference routines (oracle/_ref) on random inputs, and brute force over dense
matrices for what neither covers.  No GPU."""

import numpy as np
import pytest

from conftest import csr_to_dense, random_csr
from oracle import oracle as orc


def _dense_to_csr(dense):
    return orc.csr_from_dense(np.array(dense, dtype=np.float32))


# ---- reference known-answer vectors ---------------------------------------------------------
def test_column_pruning_golden(golden):
    for case in golden["column_pruning"]:
        dense = np.array(case["dense"], dtype=np.float32)
        r, c, v = _dense_to_csr(dense)
        r2, c2, v2, n2o = orc.compact_columns(r, c, v, dense.shape[1], case["min_nnz_per_col"])
        er, ec, ev = _dense_to_csr(case["expected_dense"])
        assert np.array_equal(r2, er), case["source"]
        assert np.array_equal(c2, ec), case["source"]
        assert np.array_equal(v2, ev), case["source"]
        assert n2o.tolist() == case["expected_new_to_old"], case["source"]


def test_csr_from_dense_golden(golden):
    for case in golden["csr_from_row_major"]:
        r, c, v = orc.csr_from_dense(np.array(case["dense"], dtype=np.float32), case["threshold"])
        assert r.tolist() == case["row_offsets"]
        assert c.tolist() == case["col_indices"]
        assert v.tolist() == case["values"]
    for case in golden["csr_from_col_major"]:
        dense = np.array(case["col_major_data"], dtype=np.float32).reshape(case["n_cols"], case["n_rows"]).T
        r, c, v = orc.csr_from_dense(dense)
        assert r.tolist() == case["row_offsets"]
        assert c.tolist() == case["col_indices"]
        assert v.tolist() == case["values"]


def test_validate_indices_golden(golden):
    for case in golden["validate_indices"]:
        got = orc.validate_indices(case["row_offsets"], case["col_indices"], case["n_cols"], case["nnz"])
        assert got == case["valid"], case["source"]


def test_validate_indices_rejects_duplicates():
    assert not orc.validate_indices([0, 3], [1, 2, 1], 4)
    assert orc.validate_indices([0, 3], [1, 2, 3], 4)


def test_fixed_width_rowptr_golden(golden):
    case = golden["construct_csr_fixed_width"]
    vals = np.array(case["values"], dtype=np.float32)
    n, k = vals.shape
    assert orc.pef_rowptr(n, k).tolist() == case["expected_row_offsets_one_row_per_example"]


# ---- the compiled reference routine on random inputs ---------------------------------------
@pytest.mark.skipif(not orc.have_ref(), reason="oracle/_ref not built")
@pytest.mark.parametrize("seed", range(6))
def test_compact_columns_matches_compiled_reference(seed):
    rng = np.random.default_rng(seed)
    n, m = int(rng.integers(1, 40)), int(rng.integers(1, 60))
    # the reference routine assumes the last row is not empty after an empty tail; keep tails full
    r, c, v = random_csr(rng, n, m, 12, empty_rows={1, 5} if n > 6 else set())
    for min_count in (1, 2, 3):
        got = orc.compact_columns(r, c, v, m, min_count)
        ref = orc.ref_prune_columns(r, c, v, m, min_count)
        # rows that trail the matrix without entries keep stale offsets in the reference; compare
        # up to the last non-empty row and require our tail to equal the new nnz
        last = max([i for i in range(n) if r[i + 1] > r[i]], default=-1)
        assert np.array_equal(got[0][: last + 2], ref[0][: last + 2])
        assert np.all(got[0][last + 1 :] == got[0][-1])
        for a, b in zip(got[1:], ref[1:]):
            assert np.array_equal(a, b)


@pytest.mark.skipif(not orc.have_ref(), reason="oracle/_ref not built")
def test_csr_from_dense_and_validate_match_compiled_reference(golden):
    rng = np.random.default_rng(3)
    dense = (rng.random((7, 9)) * (rng.random((7, 9)) < 0.4)).astype(np.float32)
    for thr in (0.0, 0.3):
        a, b = orc.csr_from_dense(dense, thr), orc.ref_csr_from_row_major(dense, thr)
        for x, y in zip(a, b):
            assert np.array_equal(x, y)
    for case in golden["validate_indices"]:
        assert orc.ref_validate_indices(case["row_offsets"], case["col_indices"], case["n_cols"], case["nnz"]) == case["valid"]
    g = golden["convert_numeric_arrays"]
    assert orc.ref_convert_i32_to_i64(g["src_int32"]).tolist() == g["dst_int64"]


# ---- brute force / invariants ---------------------------------------------------------------
@pytest.mark.parametrize("seed", range(4))
def test_compact_columns_invariants(seed):
    rng = np.random.default_rng(100 + seed)
    n, m = 30, 50
    r, c, v = random_csr(rng, n, m, 10, empty_rows={0, 7, n - 1})
    D = csr_to_dense(r, c, v, m)
    counts = (D != 0).sum(axis=0)
    for min_count in (1, 2, 4):
        r2, c2, v2, n2o = orc.compact_columns(r, c, v, m, min_count)
        kept = np.nonzero(counts >= min_count)[0]
        assert np.array_equal(n2o, kept)  # ascending original order
        assert np.all(np.diff(n2o) > 0) or len(n2o) <= 1
        assert r2[0] == 0 and r2[-1] == len(c2) and np.all(np.diff(r2) >= 0)
        assert np.array_equal(csr_to_dense(r2, c2, v2, len(n2o)), D[:, kept])
        # in-row order preserved: surviving original ids appear in the original order
        for i in range(n):
            orig = [x for x in c[r[i] : r[i + 1]] if counts[x] >= min_count]
            assert n2o[c2[r2[i] : r2[i + 1]]].tolist() == orig


@pytest.mark.parametrize("seed", range(3))
def test_retain_columns_brute_force(seed):
    rng = np.random.default_rng(200 + seed)
    n, m = 20, 40
    r, c, v = random_csr(rng, n, m, 9, empty_rows={3})
    D = csr_to_dense(r, c, v, m)
    kept = rng.choice(m, size=17, replace=False).astype(np.int32)  # arbitrary order
    r2, c2, v2 = orc.retain_columns(r, c, v, m, kept)
    assert np.array_equal(csr_to_dense(r2, c2, v2, len(kept)), D[:, kept])
    for i in range(n):  # in-row order preserved
        pos = {int(k): j for j, k in enumerate(kept)}
        want = [pos[int(x)] for x in c[r[i] : r[i + 1]] if int(x) in pos]
        assert c2[r2[i] : r2[i + 1]].tolist() == want


def test_size_of_split_closed_form():
    for total in (0, 1, 10, 17, 1000003):
        for n_splits in (1, 2, 3, 8):
            sizes = [orc.size_of_split(total, n_splits, i) for i in range(n_splits)]
            assert sum(sizes) == total
            assert all(s == total // n_splits for s in sizes[:-1])
            assert sizes[-1] == total // n_splits + total % n_splits
            assert orc.size_of_split(total, n_splits, n_splits) == -1


def test_split_row_wise_and_column_wise_brute_force():
    rng = np.random.default_rng(7)
    n, m = 23, 31
    r, c, v = random_csr(rng, n, m, 8)
    D = csr_to_dense(r, c, v, m)
    for n_splits in (1, 2, 4, 5):
        rs, es = orc.split_row_wise(r, n_splits)
        assert rs[0] == 0 and rs[-1] == n and es[-1] == r[-1]
        for s in range(n_splits):
            assert rs[s + 1] - rs[s] == orc.size_of_split(n, n_splits, s)
            assert es[s] == r[rs[s]]
        col0 = 0
        for s in range(n_splits):
            w = orc.size_of_split(m, n_splits, s)
            sr, sc, sv = orc.split_column_wise(r, c, v, m, n_splits, s)
            assert np.array_equal(csr_to_dense(sr, sc, sv, w), D[:, col0 : col0 + w])
            col0 += w


@pytest.mark.parametrize("seed", range(3))
def test_transpose_is_canonical(seed):
    rng = np.random.default_rng(300 + seed)
    n, m = 25, 35
    r, c, v = random_csr(rng, n, m, 12, empty_rows={2})
    cp, ri, tv = orc.transpose(r, c, v, m)
    D = csr_to_dense(r, c, v, m)
    assert np.array_equal(csr_to_dense(cp, ri, tv, n), D.T)
    for j in range(m):  # ascending rows inside every column
        assert np.all(np.diff(ri[cp[j] : cp[j + 1]]) > 0)
    # (A^T)^T = A with sorted columns
    r3, c3, v3 = orc.transpose(cp, ri, tv, n)
    assert np.array_equal(r3, r)
    for i in range(n):
        order = np.argsort(c[r[i] : r[i + 1]], kind="stable")
        assert np.array_equal(c3[r[i] : r[i + 1]], c[r[i] : r[i + 1]][order])
        assert np.array_equal(v3[r[i] : r[i + 1]], v[r[i] : r[i + 1]][order])


def test_normalize_rows_is_fp32_division():
    rng = np.random.default_rng(11)
    r, c, v = random_csr(rng, 9, 20, 6)
    norms = rng.random(9).astype(np.float32) + np.float32(0.1)
    out = orc.normalize_rows(r, v, norms, 1e-9)
    for i in range(9):
        d = np.float32(norms[i] + np.float32(1e-9))
        assert np.array_equal(out[r[i] : r[i + 1]], (v[r[i] : r[i + 1]] / d).astype(np.float32))
