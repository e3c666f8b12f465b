"""GPU loader through the C ABI vs the CPU oracle: bit-exact CSR construction, row
normalisation, column compaction / retention, transposed CSR, and the device generator vs its
host twin."""

import numpy as np
import pytest

import npeff_ref_amd as d
from conftest import csr_to_dense, random_csr
from oracle import oracle as orc

pytestmark = pytest.mark.gpu


def _dense_to_csr(dense):
    return orc.csr_from_dense(np.array(dense, dtype=np.float32))


def test_column_pruning_golden_on_device(golden):
    for case in golden["column_pruning"]:
        dense = np.array(case["dense"], dtype=np.float32)
        r, c, v = _dense_to_csr(dense)
        A = d.Csr.from_host(r, c, v, dense.shape[1])
        A.compact_columns(case["min_nnz_per_col"])
        r2, c2, v2 = A.download()
        er, ec, ev = _dense_to_csr(case["expected_dense"])
        assert np.array_equal(r2, er) and np.array_equal(c2, ec) and np.array_equal(v2, ev), case["source"]
        assert A.kept_indices().tolist() == case["expected_new_to_old"]
        assert A.n_cols == len(case["expected_new_to_old"]) and A.full_dense_size == dense.shape[1]
        A.close()


def test_from_pef_golden(golden):
    case = golden["construct_csr_fixed_width"]
    A = d.Csr.from_pef(case["indices"], case["values"], case["n_parameters"])
    r, c, v = A.download()
    assert r.tolist() == case["expected_row_offsets_one_row_per_example"]
    assert c.tolist() == case["expected_col_indices"]
    assert v.tolist() == case["expected_values"]
    A.close()


@pytest.mark.parametrize("seed", range(4))
def test_loader_pipeline_bit_exact(seed):
    rng = np.random.default_rng(seed)
    n, m = int(rng.integers(5, 300)), int(rng.integers(50, 5000))
    r, c, v = random_csr(rng, n, m, 200, empty_rows={0, 3, n - 1})
    norms = (rng.random(n) + 0.01).astype(np.float32)
    for min_count in (1, 2, 3):
        A = d.Csr.from_host(r, c, v, m)
        A.normalize_rows(norms, 1e-9)
        vn = orc.normalize_rows(r, v, norms, 1e-9)
        assert np.array_equal(A.download()[2], vn)
        A.compact_columns(min_count)
        er, ec, ev, en2o = orc.compact_columns(r, c, vn, m, min_count)
        gr, gc, gv = A.download()
        assert np.array_equal(gr, er) and np.array_equal(gc, ec) and np.array_equal(gv, ev)
        assert np.array_equal(A.kept_indices(), en2o)
        assert (A.n_rows, A.n_cols, A.nnz) == (n, len(en2o), len(ec))
        # transposed CSR is the canonical counting-sort transpose
        cp, ri, tv = A.download_transpose()
        ecp, eri, etv = orc.transpose(er, ec, ev, len(en2o))
        assert np.array_equal(cp, ecp) and np.array_equal(ri, eri) and np.array_equal(tv, etv)
        np.testing.assert_allclose(A.sq_norm(), np.sum(ev.astype(np.float64) ** 2), rtol=1e-12)
        A.close()


def test_retain_columns_bit_exact():
    rng = np.random.default_rng(17)
    n, m = 120, 3000
    r, c, v = random_csr(rng, n, m, 150, empty_rows={5})
    kept = rng.choice(m, size=1100, replace=False).astype(np.int32)
    A = d.Csr.from_host(r, c, v, m)
    A.retain_columns(kept)
    er, ec, ev = orc.retain_columns(r, c, v, m, kept)
    gr, gc, gv = A.download()
    assert np.array_equal(gr, er) and np.array_equal(gc, ec) and np.array_equal(gv, ev)
    assert np.array_equal(A.kept_indices(), kept) and A.n_cols == len(kept)
    A.close()


def test_edge_cases_empty_matrix_and_all_columns_dropped():
    A = d.Csr.from_host([0, 0, 0], [], [], 10)
    A.compact_columns(1)
    assert (A.n_rows, A.n_cols, A.nnz) == (2, 0, 0)
    assert A.download()[0].tolist() == [0, 0, 0]
    A.close()
    A = d.Csr.from_host([0, 1, 2], [3, 4], [1.0, 2.0], 6)
    A.compact_columns(2)
    assert (A.n_cols, A.nnz) == (0, 0) and A.download()[0].tolist() == [0, 0, 0]
    A.close()


def test_invalid_input_is_refused():
    with pytest.raises(d.DnpeffError):
        d.Csr.from_host([0, 2], [1, 7], [1.0, 1.0], 5)  # column id out of range
    with pytest.raises(d.DnpeffError):
        d.Csr.from_host([0, 2, 1], [1, 2], [1.0, 1.0], 5)  # offsets decrease


def test_large_scan_paths():
    """More than one scan tile in every scan: many columns, many entries, min_count > 1."""
    rng = np.random.default_rng(23)
    n, m, k = 300, 200000, 700
    rowptr, colind, vals, norms = d.synth_pef_host(n, m, k_fixed=k, zipf_s=1.1, seed=5)
    A = d.Csr.from_host(rowptr, colind, vals, m)
    A.normalize_rows(norms)
    vn = orc.normalize_rows(rowptr, vals, norms)
    A.compact_columns(2)
    er, ec, ev, en2o = orc.compact_columns(rowptr, colind, vn, m, 2)
    gr, gc, gv = A.download()
    assert np.array_equal(gr, er) and np.array_equal(gc, ec) and np.array_equal(gv, ev)
    assert np.array_equal(A.kept_indices(), en2o)
    cp, ri, tv = A.download_transpose()
    ecp, eri, etv = orc.transpose(er, ec, ev, len(en2o))
    assert np.array_equal(cp, ecp) and np.array_equal(ri, eri) and np.array_equal(tv, etv)
    A.close()


@pytest.mark.parametrize("kw", [dict(k_fixed=600, zipf_s=1.1), dict(k_fixed=300, zipf_s=1.3), dict(k_min=16, k_max=2048, zipf_s=1.1)])
def test_device_generator_equals_host_generator(kw):
    n, m = 96, 500000
    A, norms = d.Csr.synth(n, m, seed=99, **kw)
    hr, hc, hv, hn = d.synth_pef_host(n, m, seed=99, **kw)
    gr, gc, gv = A.download()
    assert np.array_equal(gr, hr) and np.array_equal(gc, hc)
    assert np.array_equal(gv, hv) and np.array_equal(norms, hn)
    assert orc.validate_indices(gr, gc, m)
    A.close()
