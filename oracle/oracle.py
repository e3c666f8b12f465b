"""TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.

ctypes binding of oracle/liboracle.so (the C restatement in dnpeff_oracle.c) and, where it was
built, of oracle/_ref/libref.so (the reference's own host-only routines).  Only tests/,
__graft_entry__.smoke() and the cpu_baseline leg of bench.py import this module.
"""

from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liboracle.so")
REF_PATH = os.path.join(_HERE, "_ref", "libref.so")

if not os.path.exists(LIB_PATH):
    raise ImportError(f"{LIB_PATH} missing: run `make -C oracle`")
_lib = C.CDLL(LIB_PATH)
_ref = C.CDLL(REF_PATH) if os.path.exists(REF_PATH) else None

_i64, _i32, _f32, _f64, _p = C.c_int64, C.c_int32, C.c_float, C.c_double, C.c_void_p


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _sig(lib, name, res, args):
    f = getattr(lib, name)
    f.restype = res
    f.argtypes = args
    return f


_normalize = _sig(_lib, "orc_normalize_rows", None, [_i64, _p, _p, _p, _f32])
_pef_rowptr = _sig(_lib, "orc_pef_rowptr", None, [_i64, _i64, _p])
_compact = _sig(_lib, "orc_compact_columns", _i64, [_i64, _i64, _p, _p, _p, C.c_int, _p])
_retain = _sig(_lib, "orc_retain_columns", _i64, [_i64, _i64, _p, _p, _p, _p, _i64])
_size_of_split = _sig(_lib, "orc_size_of_split", _i64, [_i64, _i64, _i64])
_split_rows = _sig(_lib, "orc_split_row_wise", None, [_i64, _p, C.c_int, _p, _p])
_split_cols = _sig(_lib, "orc_split_column_wise", _i64, [_i64, _i64, _p, _p, _p, C.c_int, C.c_int, _p, _p, _p])
_csr_from_dense = _sig(_lib, "orc_csr_from_dense", _i64, [_p, _i64, _i64, _f32, _p, _p, _p])
_validate = _sig(_lib, "orc_validate_indices", C.c_int, [_i64, _i64, _i64, _p, _p])
_transpose = _sig(_lib, "orc_transpose", None, [_i64, _i64, _p, _p, _p, _p, _p, _p])
_nmf_f64 = _sig(_lib, "orc_nmf_f64", None, [_i64, _i64, _p, _p, _p, C.c_int, _f32, C.c_int, C.c_int, _p, _p, _p])
_loss_f64 = _sig(_lib, "orc_loss_f64", _f64, [_i64, _i64, _p, _p, _p, C.c_int, _p, _p, _p])
_spmm_n = _sig(_lib, "orc_spmm_n_f64", None, [_i64, _p, _p, _p, C.c_int, _p, _p])
_spmm_t = _sig(_lib, "orc_spmm_t_f64", None, [_i64, _i64, _p, _p, _p, C.c_int, _p, _p])
_gram = _sig(_lib, "orc_gram_f64", None, [_i64, C.c_int, _p, _p])
_xg_mu = _sig(_lib, "orc_xg_mu_f64", None, [_i64, C.c_int, _p, _p, _p, _f32, _p, _p])
_spsp = _sig(_lib, "orc_spsp_dense_f64", None, [_i64, _i64, _p, _p, _p, C.c_int, _p, _p, _p, _p])
_fit = _sig(_lib, "orc_fit_f64", None, [_i64, C.c_int, _p, _p, _f64, _f32, C.c_int, C.c_int, _p, _p, _p])
_f32_create = _sig(_lib, "orc_f32_create", _p, [_i64, _i64, _p, _p, _p, C.c_int, _f32, _p, _p])
_f32_create_mr = _sig(_lib, "orc_f32_create_mr", _p, [_i64, _i64, _p, _p, _p, C.c_int, _f32, _p, _p])
_f32_step = _sig(_lib, "orc_f32_step", None, [_p, C.c_int])
_f32_step_timed = _sig(_lib, "orc_f32_step_timed", None, [_p, C.c_int, _p])
_f32_spsp_timed = _sig(_lib, "orc_f32_spsp_timed", _f64, [_i64, _p, _p, _p, C.c_int, _p, _p, _p, _p])
_f32_fit_timed = _sig(_lib, "orc_f32_fit_steps_timed", _f64, [_i64, C.c_int, _p, _p, _f32, C.c_int, _p])
_f32_get = _sig(_lib, "orc_f32_get", None, [_p, _p, _p])
_f32_destroy = _sig(_lib, "orc_f32_destroy", None, [_p])
_num_threads = _sig(_lib, "orc_num_threads", C.c_int, [])
_sparsify_cols = _sig(_lib, "orc_sparsify_columns", C.c_int, [_i64, C.c_int, _p, _f32, _f32])


def _csr(rowptr, colind, vals):
    return (
        np.ascontiguousarray(rowptr, dtype=np.int64),
        np.ascontiguousarray(colind, dtype=np.int32),
        np.ascontiguousarray(vals, dtype=np.float32),
    )


# ---- loader ---------------------------------------------------------------------------------
def normalize_rows(rowptr, vals, norms, eps=1e-9):
    rowptr = np.ascontiguousarray(rowptr, dtype=np.int64)
    out = np.array(vals, dtype=np.float32, copy=True)
    norms = np.ascontiguousarray(norms, dtype=np.float32)
    _normalize(len(rowptr) - 1, _ptr(rowptr), _ptr(out), _ptr(norms), eps)
    return out


def pef_rowptr(n_rows, k):
    out = np.zeros(n_rows + 1, dtype=np.int64)
    _pef_rowptr(n_rows, k, _ptr(out))
    return out


def compact_columns(rowptr, colind, vals, n_cols, min_count=1):
    """-> (rowptr, colind, vals, new_to_og) after removeSmallestL0NormColumns_inPlace."""
    rowptr, colind, vals = (np.array(a, copy=True) for a in _csr(rowptr, colind, vals))
    new_to_og = np.zeros(max(n_cols, 1), dtype=np.int32)
    m = _compact(len(rowptr) - 1, n_cols, _ptr(rowptr), _ptr(colind), _ptr(vals), min_count, _ptr(new_to_og))
    nnz = int(rowptr[-1])
    return rowptr, colind[:nnz].copy(), vals[:nnz].copy(), new_to_og[:m].copy()


def retain_columns(rowptr, colind, vals, n_cols, kept):
    rowptr, colind, vals = (np.array(a, copy=True) for a in _csr(rowptr, colind, vals))
    kept = np.ascontiguousarray(kept, dtype=np.int32)
    nnz = _retain(len(rowptr) - 1, n_cols, _ptr(rowptr), _ptr(colind), _ptr(vals), _ptr(kept), len(kept))
    return rowptr, colind[:nnz].copy(), vals[:nnz].copy()


def size_of_split(total, n_splits, idx):
    return _size_of_split(total, n_splits, idx)


def split_row_wise(rowptr, n_splits):
    rowptr = np.ascontiguousarray(rowptr, dtype=np.int64)
    rs = np.zeros(n_splits + 1, dtype=np.int64)
    es = np.zeros(n_splits + 1, dtype=np.int64)
    _split_rows(len(rowptr) - 1, _ptr(rowptr), n_splits, _ptr(rs), _ptr(es))
    return rs, es


def split_column_wise(rowptr, colind, vals, n_cols, n_splits, split):
    rowptr, colind, vals = _csr(rowptr, colind, vals)
    n = len(rowptr) - 1
    orow = np.zeros(n + 1, dtype=np.int64)
    ocol = np.zeros(len(colind), dtype=np.int32)
    oval = np.zeros(len(colind), dtype=np.float32)
    k = _split_cols(n, n_cols, _ptr(rowptr), _ptr(colind), _ptr(vals), n_splits, split, _ptr(orow), _ptr(ocol), _ptr(oval))
    return orow, ocol[:k].copy(), oval[:k].copy()


def csr_from_dense(dense, threshold=0.0):
    dense = np.ascontiguousarray(dense, dtype=np.float32)
    n, m = dense.shape
    rowptr = np.zeros(n + 1, dtype=np.int64)
    colind = np.zeros(n * m, dtype=np.int32)
    vals = np.zeros(n * m, dtype=np.float32)
    k = _csr_from_dense(_ptr(dense), n, m, threshold, _ptr(rowptr), _ptr(colind), _ptr(vals))
    return rowptr, colind[:k].copy(), vals[:k].copy()


def validate_indices(rowptr, colind, n_cols, nnz=None):
    rowptr = np.ascontiguousarray(rowptr, dtype=np.int64)
    colind = np.ascontiguousarray(colind, dtype=np.int32)
    return bool(_validate(len(rowptr) - 1, n_cols, len(colind) if nnz is None else nnz, _ptr(rowptr), _ptr(colind)))


def transpose(rowptr, colind, vals, n_cols):
    rowptr, colind, vals = _csr(rowptr, colind, vals)
    colptr = np.zeros(n_cols + 1, dtype=np.int64)
    rowind = np.zeros(len(colind), dtype=np.int32)
    tvals = np.zeros(len(colind), dtype=np.float32)
    _transpose(len(rowptr) - 1, n_cols, _ptr(rowptr), _ptr(colind), _ptr(vals), _ptr(colptr), _ptr(rowind), _ptr(tvals))
    return colptr, rowind, tvals


# ---- fp64 NMF -------------------------------------------------------------------------------
def nmf_f64(rowptr, colind, vals, n_cols, W0, H0, eps, iters, log_every=10):
    """Reference update sequence in fp64.  W0 [n, r], H0 [r, m] -> (W, H, losses)."""
    rowptr, colind, vals = _csr(rowptr, colind, vals)
    W = np.array(W0, dtype=np.float64, copy=True, order="C")
    H = np.array(H0, dtype=np.float64, copy=True, order="C")
    n, r = W.shape
    assert H.shape == (r, n_cols)
    n_log = iters // log_every if log_every > 0 else 0
    losses = np.zeros(max(n_log, 1), dtype=np.float64)
    _nmf_f64(n, n_cols, _ptr(rowptr), _ptr(colind), _ptr(vals), r, eps, iters, log_every, _ptr(W), _ptr(H), _ptr(losses))
    return W, H, losses[:n_log]


def loss_f64(rowptr, colind, vals, n_cols, W, H):
    rowptr, colind, vals = _csr(rowptr, colind, vals)
    W = np.ascontiguousarray(W, dtype=np.float64)
    H = np.ascontiguousarray(H, dtype=np.float64)
    terms = np.zeros(3, dtype=np.float64)
    v = _loss_f64(W.shape[0], n_cols, _ptr(rowptr), _ptr(colind), _ptr(vals), W.shape[1], _ptr(W), _ptr(H), _ptr(terms))
    return v, terms


def spmm_n_f64(rowptr, colind, vals, Ht_mr):
    rowptr, colind, vals = _csr(rowptr, colind, vals)
    Ht = np.ascontiguousarray(Ht_mr, dtype=np.float64)
    n, r = len(rowptr) - 1, Ht.shape[1]
    out = np.zeros((n, r), dtype=np.float64)
    _spmm_n(n, _ptr(rowptr), _ptr(colind), _ptr(vals), r, _ptr(Ht), _ptr(out))
    return out


def spmm_t_f64(rowptr, colind, vals, n_cols, W_nr):
    rowptr, colind, vals = _csr(rowptr, colind, vals)
    W = np.ascontiguousarray(W_nr, dtype=np.float64)
    n, r = W.shape
    out = np.zeros((n_cols, r), dtype=np.float64)
    _spmm_t(n, n_cols, _ptr(rowptr), _ptr(colind), _ptr(vals), r, _ptr(W), _ptr(out))
    return out


def gram_f64(X):
    X = np.ascontiguousarray(X, dtype=np.float64)
    G = np.zeros((X.shape[1], X.shape[1]), dtype=np.float64)
    _gram(X.shape[0], X.shape[1], _ptr(X), _ptr(G))
    return G


def xg_mu_f64(X, G, num, eps):
    X = np.ascontiguousarray(X, dtype=np.float64)
    G = np.ascontiguousarray(G, dtype=np.float64)
    num = np.ascontiguousarray(num, dtype=np.float64)
    out = np.zeros_like(X)
    D = np.zeros_like(X)
    _xg_mu(X.shape[0], X.shape[1], _ptr(X), _ptr(G), _ptr(num), eps, _ptr(out), _ptr(D))
    return out, D


def spsp_dense_f64(a_csr, n_cols, b_csr, r):
    ar, ac, av = _csr(*a_csr)
    br, bc, bv = _csr(*b_csr)
    n = len(ar) - 1
    out = np.zeros((n, r), dtype=np.float64)
    _spsp(n, n_cols, _ptr(ar), _ptr(ac), _ptr(av), r, _ptr(br), _ptr(bc), _ptr(bv), _ptr(out))
    return out


def fit_f64(AH, HH, sq_norm_A, W0, eps, iters, log_every=25):
    AH = np.ascontiguousarray(AH, dtype=np.float64)
    HH = np.ascontiguousarray(HH, dtype=np.float64)
    W = np.array(W0, dtype=np.float64, copy=True, order="C")
    n, r = W.shape
    n_log = iters // log_every if log_every > 0 else 0
    ref = np.zeros(max(n_log, 1), dtype=np.float64)
    tru = np.zeros(max(n_log, 1), dtype=np.float64)
    _fit(n, r, _ptr(AH), _ptr(HH), sq_norm_A, eps, iters, log_every, _ptr(W), _ptr(ref), _ptr(tru))
    return W, ref[:n_log], tru[:n_log]


# ---- fp32 OpenMP baseline -------------------------------------------------------------------
class F32Baseline:
    """The reference update loop in fp32 on the host cores (timed cpu_baseline)."""

    def __init__(self, rowptr, colind, vals, n_cols, W0, H0=None, eps=1e-8, Ht0_mr=None):
        self._csr = _csr(rowptr, colind, vals)  # keep alive: the context borrows them
        W0 = np.ascontiguousarray(W0, dtype=np.float32)
        self.n, self.r = W0.shape
        self.m = n_cols
        if Ht0_mr is not None:
            Ht0 = np.ascontiguousarray(Ht0_mr, dtype=np.float32)
            self._h = _f32_create_mr(self.n, self.m, *map(_ptr, self._csr), self.r, eps, _ptr(W0), _ptr(Ht0))
        else:
            H0 = np.ascontiguousarray(H0, dtype=np.float32)
            self._h = _f32_create(self.n, self.m, *map(_ptr, self._csr), self.r, eps, _ptr(W0), _ptr(H0))

    def step(self, n_steps=1):
        _f32_step(self._h, n_steps)

    PARTS = ("spmm_n", "gram_H", "xg_mu_W", "spmm_t", "gram_W", "xg_mu_H")

    def step_timed(self, n_steps=1):
        """Seconds spent in each part of n_steps iterations, keyed like the device kernel classes."""
        secs = np.zeros(6, dtype=np.float64)
        _f32_step_timed(self._h, n_steps, _ptr(secs))
        return dict(zip(self.PARTS, secs.tolist()))

    def get(self):
        W = np.zeros((self.n, self.r), dtype=np.float32)
        H = np.zeros((self.r, self.m), dtype=np.float32)
        _f32_get(self._h, _ptr(W), _ptr(H))
        return W, H

    def close(self):
        if self._h:
            _f32_destroy(self._h)
            self._h = None

    @staticmethod
    def num_threads():
        return _num_threads()


def spsp_f32_timed(a_csr, b_transposed, r):
    """fp32 OpenMP A B^T (first stage of the learner) on the host cores: (out [n, r], seconds).
    b_transposed = (colptr, component ids, values) of B's transposed CSR."""
    ar, ac, av = _csr(*a_csr)
    bp, bc, bv = _csr(*b_transposed)
    n = len(ar) - 1
    out = np.zeros((n, r), dtype=np.float32)
    secs = _f32_spsp_timed(n, _ptr(ar), _ptr(ac), _ptr(av), r, _ptr(bp), _ptr(bc), _ptr(bv), _ptr(out))
    return out, secs


def fit_steps_f32_timed(AH, HH, W0, eps, n_steps):
    """n_steps of the learner's W update in fp32 on the host cores: (W, seconds)."""
    AH = np.ascontiguousarray(AH, dtype=np.float32)
    HH = np.ascontiguousarray(HH, dtype=np.float32)
    W = np.array(W0, dtype=np.float32, copy=True, order="C")
    n, r = W.shape
    secs = _f32_fit_timed(n, r, _ptr(AH), _ptr(HH), eps, n_steps, _ptr(W))
    return W, secs


# ---- compiled reference routines (oracle/_ref) ----------------------------------------------
def sparsify_H(W, H_rm, threshold):
    """Dense decomposition -> (W', values, row_offsets, column_indices): every row of H scaled to
    unit L2 norm (sum of squares in fp64, norm and division in fp32), the matching column of W
    multiplied by the norm, then per row the entries >= threshold in ascending column order.
    scripts/sparsify_d_npeff.py:27-49 (to_csr) and :56 (the normalisation it intends)."""
    H = np.asarray(H_rm, dtype=np.float32)
    W2 = np.array(W, dtype=np.float32, copy=True)
    thr = np.float32(threshold)
    vals, cols, offs = [], [], [0]
    for k in range(H.shape[0]):
        norm = np.float32(np.sqrt(np.sum(H[k].astype(np.float64) ** 2)))
        div = norm if norm > 0 else np.float32(1.0)
        row = (H[k] / div).astype(np.float32)
        mask = row >= thr
        vals.append(row[mask])
        cols.append(np.nonzero(mask)[0].astype(np.int32))
        offs.append(offs[-1] + int(mask.sum()))
        W2[:, k] *= div
    return (W2, np.concatenate(vals).astype(np.float32), np.array(offs, dtype=np.int64),
            np.concatenate(cols).astype(np.int32))


def sparsify_columns(W, l1_norm, l2_norm=1.0):
    """(W', passes): every column of the row-major W moved to non-negative entries that sum to
    l1_norm by the reference's iteration (dense_factor_sparsity_constraints.h:205-237)."""
    out = np.array(W, dtype=np.float32, order="C", copy=True)
    passes = _sparsify_cols(out.shape[0], out.shape[1], _ptr(out), l1_norm, l2_norm)
    return out, passes


def topk_rows(x, k):
    """Per row: the k largest entries in descending order, equal values by ascending index
    (tf.math.top_k's rule), and the L2 norm of the whole row.
    npeff/fishers/d_pefs_computer.py:126-129, :48-50."""
    x = np.asarray(x, dtype=np.float32)
    order = np.argsort(-x.astype(np.float64), axis=1, kind="stable")[:, :k]
    vals = np.take_along_axis(x, order, axis=1)
    norms = np.sqrt(np.sum(x.astype(np.float64) ** 2, axis=1)).astype(np.float32)
    return vals, order.astype(np.int32), norms


def have_ref():
    return _ref is not None


def ref_prune_columns(rowptr, colind, vals, n_cols, min_nnz_per_col):
    """prune_columns_in_place of the reference (int32 offsets)."""
    f = _sig(_ref, "ref_prune_columns_i32", _i64, [_i64, _i64, _i64, _p, _p, _p, _i64, _p, C.POINTER(_i64)])
    ro = np.array(rowptr, dtype=np.int32, copy=True)
    ci = np.array(colind, dtype=np.int32, copy=True)
    va = np.array(vals, dtype=np.float32, copy=True)
    n2o = np.zeros(max(n_cols, 1), dtype=np.int32)
    nnz_out = _i64(0)
    m = f(len(ro) - 1, n_cols, len(ci), _ptr(ro), _ptr(ci), _ptr(va), min_nnz_per_col, _ptr(n2o), C.byref(nnz_out))
    z = nnz_out.value
    return ro.astype(np.int64), ci[:z].copy(), va[:z].copy(), n2o[:m].copy()


def ref_csr_from_row_major(dense, threshold=0.0):
    f = _sig(_ref, "ref_csr_from_row_major", _i64, [_p, _i64, _i64, _f32, _p, _p, _p])
    dense = np.ascontiguousarray(dense, dtype=np.float32)
    n, m = dense.shape
    ro = np.zeros(n + 1, dtype=np.int32)
    ci = np.zeros(n * m, dtype=np.int32)
    va = np.zeros(n * m, dtype=np.float32)
    k = f(_ptr(dense), n, m, threshold, _ptr(ro), _ptr(ci), _ptr(va))
    return ro.astype(np.int64), ci[:k].copy(), va[:k].copy()


def ref_validate_indices(rowptr, colind, n_cols, nnz):
    f = _sig(_ref, "ref_validate_indices", C.c_int, [_i64, _i64, _i64, _p, _p])
    ro = np.ascontiguousarray(rowptr, dtype=np.int32)
    ci = np.ascontiguousarray(colind, dtype=np.int32)
    return bool(f(len(ro) - 1, n_cols, nnz, _ptr(ro), _ptr(ci)))


def ref_convert_i32_to_i64(src):
    f = _sig(_ref, "ref_convert_i32_to_i64", None, [_p, _p, _i64])
    src = np.ascontiguousarray(src, dtype=np.int32)
    dst = np.zeros(len(src), dtype=np.int64)
    f(_ptr(dst), _ptr(src), len(src))
    return dst
