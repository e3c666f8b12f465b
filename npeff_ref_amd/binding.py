"""ctypes binding of libdnpeff_hip.so (C ABI: include/dnpeff.h)."""

from __future__ import annotations

import ctypes as C
import math
import os
import time
from dataclasses import dataclass
from typing import Callable, Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libdnpeff_hip.so")


class DnpeffError(RuntimeError):
    """A C-ABI call returned a non-zero status."""


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "(or `make -C npeff_ref_amd/csrc`). There is no CPU fallback."
        )
    return C.CDLL(LIB_PATH)


lib = _load()

_i64 = C.c_int64
_i32 = C.c_int32
_u64 = C.c_uint64
_f32 = C.c_float
_f64 = C.c_double
_p = C.c_void_p
_pp = C.POINTER(C.c_void_p)

# name -> (restype, argtypes); every exported function of include/dnpeff.h
SIGNATURES = {
    "dnpeff_last_error": (C.c_char_p, []),
    "dnpeff_device_count": (C.c_int, [C.POINTER(C.c_int)]),
    "dnpeff_device_info": (C.c_int, [C.c_char_p, C.c_int, C.POINTER(_i64), C.POINTER(C.c_int)]),
    "dnpeff_sync": (C.c_int, []),
    "dnpeff_stream": (_p, []),
    "dnpeff_device_memory": (C.c_int, [C.POINTER(_i64), C.POINTER(_i64)]),
    "dnpeff_tuning_set": (C.c_int, [C.c_char_p, _f64]),
    "dnpeff_tuning_get": (C.c_int, [C.c_char_p, C.POINTER(_f64)]),
    "dnpeff_plan_estimate": (C.c_int, [_i64, _i64, _i64, _i64, C.c_int, C.c_int, C.c_int, _i64, C.POINTER(_f64)]),
    "dnpeff_tuning_reset": (C.c_int, []),
    "dnpeff_dev_malloc": (C.c_int, [_i64, _pp]),
    "dnpeff_dev_free": (C.c_int, [_p]),
    "dnpeff_dev_upload": (C.c_int, [_p, _p, _i64]),
    "dnpeff_dev_download": (C.c_int, [_p, _p, _i64]),
    "dnpeff_csr_from_host": (C.c_int, [_i64, _i64, _i64, _p, _p, _p, _pp]),
    "dnpeff_csr_from_pef": (C.c_int, [_i64, _i64, _i64, _p, _p, _pp]),
    "dnpeff_csr_normalize_rows": (C.c_int, [_p, _p, _f32]),
    "dnpeff_csr_compact_columns": (C.c_int, [_p, C.c_int]),
    "dnpeff_csr_retain_columns": (C.c_int, [_p, _p, _i64]),
    "dnpeff_csr_shape": (C.c_int, [_p, C.POINTER(_i64), C.POINTER(_i64), C.POINTER(_i64)]),
    "dnpeff_csr_full_dense_size": (C.c_int, [_p, C.POINTER(_i64)]),
    "dnpeff_csr_download": (C.c_int, [_p, _p, _p, _p]),
    "dnpeff_csr_kept_indices": (C.c_int, [_p, _p]),
    "dnpeff_csr_sq_norm": (C.c_int, [_p, C.POINTER(_f64)]),
    "dnpeff_csr_build_transpose": (C.c_int, [_p]),
    "dnpeff_topk_rows": (C.c_int, [C.c_int64, C.c_int64, C.c_int64, _p, _p, _p, _p]),
    "dnpeff_op_threshold_compact": (C.c_int, [C.c_int64, _p, C.c_float, C.c_float, _p, _p, C.POINTER(C.c_int64)]),
    "dnpeff_csr_split_dense_head": (C.c_int, [_p, C.c_double, C.POINTER(C.c_int64)]),
    "dnpeff_csr_head_info": (C.c_int, [_p, C.POINTER(C.c_int64), C.POINTER(C.c_int64)]),
    "dnpeff_csr_products_info": (C.c_int, [_p, _p]),
    "dnpeff_csr_download_transpose": (C.c_int, [_p, _p, _p, _p]),
    "dnpeff_csr_release": (C.c_int, [_p, C.c_int]),
    "dnpeff_csr_destroy": (C.c_int, [_p]),
    "dnpeff_size_of_split": (_i64, [_i64, _i64, _i64]),
    "dnpeff_synth_pef": (C.c_int, [_i64, _i64, _i64, _i64, _i64, _f64, _f64, _f64, _u64, _p, _pp]),
    "dnpeff_synth_pef_host": (
        C.c_int,
        [_i64, _i64, _i64, _i64, _i64, _f64, _f64, _f64, _u64, _p, _p, _p, _p],
    ),
    "dnpeff_synth_pef_host_rows": (
        C.c_int,
        [_i64, _i64, _i64, _i64, _i64, _i64, _f64, _f64, _f64, _u64, _p, _p, _p, _p],
    ),
    "dnpeff_csr_get_row": (C.c_int, [_p, _i64, _i64, C.POINTER(_i64), _p, _p]),
    "dnpeff_csr_get_column": (C.c_int, [_p, _i64, _i64, C.POINTER(_i64), _p, _p]),
    "dnpeff_op_gather_rows": (C.c_int, [_i64, C.c_int, _p, _p, _p]),
    "dnpeff_uniform_at": (_f32, [_u64, C.c_int, _i64, _i64, _i64]),
    "dnpeff_nmf_create": (C.c_int, [_p, C.c_int, _f32, _i64, _pp]),
    "dnpeff_nmf_create_ex": (C.c_int, [_p, C.c_int, _f32, _i64, C.c_uint, _pp]),
    "dnpeff_nmf_info": (C.c_int, [_p, C.POINTER(C.c_int), C.POINTER(_i64)]),
    "dnpeff_nmf_init_factors": (C.c_int, [_p]),
    "dnpeff_nmf_set_factors": (C.c_int, [_p, _p, _p]),
    "dnpeff_nmf_step": (C.c_int, [_p, C.c_int]),
    "dnpeff_nmf_update_W": (C.c_int, [_p]),
    "dnpeff_nmf_update_H": (C.c_int, [_p]),
    "dnpeff_nmf_loss": (C.c_int, [_p, C.POINTER(_f64)]),
    "dnpeff_nmf_loss_terms": (C.c_int, [_p, C.POINTER(_f64), C.POINTER(_f64), C.POINTER(_f64)]),
    "dnpeff_nmf_check_products": (C.c_int, [_p, C.POINTER(_f64), C.POINTER(_f64)]),
    "dnpeff_nmf_sparsify_W": (C.c_int, [_p, _f32, _f32, C.POINTER(C.c_int)]),
    "dnpeff_nmf_get_W": (C.c_int, [_p, _p]),
    "dnpeff_nmf_get_H": (C.c_int, [_p, _p]),
    "dnpeff_nmf_device_factors": (C.c_int, [_p, _pp, _pp]),
    "dnpeff_nmf_set_profiling": (C.c_int, [_p, C.c_int]),
    "dnpeff_nmf_timings": (C.c_int, [_p, _p, _p, C.c_int]),
    "dnpeff_nmf_destroy": (C.c_int, [_p]),
    "dnpeff_fit_create": (C.c_int, [_p, _p, _f32, _i64, _pp]),
    "dnpeff_fit_init_W": (C.c_int, [_p]),
    "dnpeff_fit_set_W": (C.c_int, [_p, _p]),
    "dnpeff_fit_step": (C.c_int, [_p, C.c_int]),
    "dnpeff_fit_loss": (C.c_int, [_p, C.POINTER(_f64), C.POINTER(_f64)]),
    "dnpeff_fit_get_W": (C.c_int, [_p, _p]),
    "dnpeff_fit_get_products": (C.c_int, [_p, _p, _p, C.POINTER(_f64)]),
    "dnpeff_fit_destroy": (C.c_int, [_p]),
    "dnpeff_op_mu": (C.c_int, [_i64, _p, _p, _p, _f32]),
    "dnpeff_op_sparsify_columns": (C.c_int, [_i64, C.c_int, _p, _f32, _f32, C.POINTER(C.c_int)]),
    "dnpeff_op_spmm_n": (C.c_int, [_p, C.c_int, _p, _p]),
    "dnpeff_op_spmm_n_variant": (C.c_int, [_p, C.c_int, _p, _p, C.c_int]),
    "dnpeff_op_spmm_t": (C.c_int, [_p, C.c_int, _p, _p]),
    "dnpeff_op_spmm_t_tile": (C.c_int, [_p, C.c_int, _p, _i64, _i64, _p]),
    "dnpeff_op_gram": (C.c_int, [_i64, C.c_int, _p, _p]),
    "dnpeff_op_gram_static": (C.c_int, [_i64, C.c_int, _p, _p]),
    "dnpeff_op_xg_mu": (C.c_int, [_i64, C.c_int, _p, _p, _p, _f32, _p, _p]),
    "dnpeff_op_xg_mu_gram": (C.c_int, [_i64, _p, _p, _p, _f32, _p, _p]),
    "dnpeff_op_dot": (C.c_int, [_i64, _p, _p, C.POINTER(_f64)]),
    "dnpeff_op_spsp_dense": (C.c_int, [_p, _p, _p]),
    "dnpeff_op_copy": (C.c_int, [_i64, _p, _p]),
    "dnpeff_op_init_uniform": (C.c_int, [C.c_int, _i64, _i64, _u64, _p]),
}

for _name, (_res, _args) in SIGNATURES.items():
    _fn = getattr(lib, _name)
    _fn.restype = _res
    _fn.argtypes = _args

KERNEL_CLASSES = ["spmm_n", "spmm_n_reduce", "gram_H", "xg_mu_W", "spmm_t", "gram_W", "xg_mu_H"]


def _check(status: int):
    if status != 0:
        raise DnpeffError(lib.dnpeff_last_error().decode("utf-8", "replace"))


def _ptr(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _arr(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def device_count() -> int:
    c = C.c_int(0)
    _check(lib.dnpeff_device_count(C.byref(c)))
    return c.value


def device_info():
    name = C.create_string_buffer(256)
    total = _i64(0)
    cus = C.c_int(0)
    _check(lib.dnpeff_device_info(name, 256, C.byref(total), C.byref(cus)))
    return name.value.decode(), total.value, cus.value


def sync():
    _check(lib.dnpeff_sync())


def device_memory():
    """(free, total) bytes of device memory."""
    f, t = _i64(0), _i64(0)
    _check(lib.dnpeff_device_memory(C.byref(f), C.byref(t)))
    return f.value, t.value


PLAN_FIELDS = ("factors", "partials", "segments", "offsets", "reserve", "sparse_copies", "head_blocks",
               "head_workspace")


def plan_estimate(n_rows, n_cols, nnz_sparse, n_dense, rank, tiled, sweeps=True, total_bytes=309_220_868_096):
    """The byte table of the memory plan (dnpeff_plan_estimate) as a dict; needs no GPU."""
    out = (_f64 * 8)()
    _check(lib.dnpeff_plan_estimate(n_rows, n_cols, nnz_sparse, n_dense, rank, int(bool(tiled)), int(bool(sweeps)),
                                    total_bytes, out))
    return dict(zip(PLAN_FIELDS, [float(x) for x in out]))


def tuning_set(name: str, value: float):
    _check(lib.dnpeff_tuning_set(name.encode(), float(value)))


def tuning_get(name: str) -> float:
    v = _f64(0)
    _check(lib.dnpeff_tuning_get(name.encode(), C.byref(v)))
    return v.value


def tuning_reset():
    _check(lib.dnpeff_tuning_reset())


def size_of_split(total: int, n_splits: int, split_index: int) -> int:
    """getSizeOfSplit (cc/cuda_d_npeff/src/util/matrix_util.h:10-21); raises where it throws."""
    v = lib.dnpeff_size_of_split(total, n_splits, split_index)
    if v < 0:
        raise DnpeffError("split index out of range")
    return v


def uniform_at(seed: int, matrix_id: int, row: int, col: int, n_cols: int) -> float:
    return lib.dnpeff_uniform_at(seed & 0xFFFFFFFFFFFFFFFF, matrix_id, row, col, n_cols)


def synth_pef_host(n_rows, n_cols, k_fixed=0, k_min=0, k_max=0, zipf_s=1.1, mu=-8.0, sigma=2.0, seed=0):
    """Single-threaded host twin of the device generator; returns rowptr, colind, vals, norms."""
    rowptr = np.zeros(n_rows + 1, dtype=np.int64)
    args = (n_rows, n_cols, k_fixed, k_min, k_max, zipf_s, mu, sigma, seed & 0xFFFFFFFFFFFFFFFF)
    _check(lib.dnpeff_synth_pef_host(*args, _ptr(rowptr), None, None, None))
    nnz = int(rowptr[-1])
    colind = np.zeros(nnz, dtype=np.int32)
    vals = np.zeros(nnz, dtype=np.float32)
    norms = np.zeros(n_rows, dtype=np.float32)
    _check(lib.dnpeff_synth_pef_host(*args, _ptr(rowptr), _ptr(colind), _ptr(vals), _ptr(norms)))
    return rowptr, colind, vals, norms


def synth_pef_host_rows(row0, n_rows, n_cols, k_fixed=0, k_min=0, k_max=0, zipf_s=1.1, mu=-8.0, sigma=2.0,
                        seed=0):
    """Rows [row0, row0 + n_rows) of the device generator's matrix, made on the host."""
    rowptr = np.zeros(n_rows + 1, dtype=np.int64)
    args = (row0, n_rows, n_cols, k_fixed, k_min, k_max, zipf_s, mu, sigma, seed & 0xFFFFFFFFFFFFFFFF)
    _check(lib.dnpeff_synth_pef_host_rows(*args, _ptr(rowptr), None, None, None))
    nnz = int(rowptr[-1])
    colind = np.zeros(nnz, dtype=np.int32)
    vals = np.zeros(nnz, dtype=np.float32)
    norms = np.zeros(n_rows, dtype=np.float32)
    _check(lib.dnpeff_synth_pef_host_rows(*args, _ptr(rowptr), _ptr(colind), _ptr(vals), _ptr(norms)))
    return rowptr, colind, vals, norms


def gather_rows(dev_ptr, r: int, rows) -> np.ndarray:
    """Rows `rows` of a device array of r floats per row, as a numpy array."""
    rows = np.ascontiguousarray(rows, dtype=np.int32)
    idx = DeviceArray.from_numpy(rows, dtype=np.int32)
    out = DeviceArray((len(rows), r))
    _check(lib.dnpeff_op_gather_rows(len(rows), r, C.c_void_p(dev_ptr), idx.ptr, out.ptr))
    sync()
    res = out.numpy()
    idx.free()
    out.free()
    return res


class DeviceArray:
    """A plain device buffer holding a numpy array (for the dnpeff_op_* entry points)."""

    def __init__(self, shape, dtype=np.float32):
        self.shape = tuple(int(x) for x in np.atleast_1d(shape))
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = C.c_void_p()
        _check(lib.dnpeff_dev_malloc(self.nbytes, C.byref(p)))
        self.ptr = p

    @staticmethod
    def from_numpy(a, dtype=np.float32) -> "DeviceArray":
        a = np.ascontiguousarray(a, dtype=dtype)
        d = DeviceArray(a.shape, a.dtype)
        _check(lib.dnpeff_dev_upload(d.ptr, _ptr(a), d.nbytes))
        return d

    def numpy(self) -> np.ndarray:
        out = np.zeros(self.shape, dtype=self.dtype)
        _check(lib.dnpeff_dev_download(_ptr(out), self.ptr, self.nbytes))
        return out

    def free(self):
        if self.ptr is not None:
            lib.dnpeff_dev_free(self.ptr)
            self.ptr = None

    def __del__(self):  # pragma: no cover
        try:
            self.free()
        except Exception:
            pass


def op_mu(F: DeviceArray, num: DeviceArray, den: DeviceArray, eps: float):
    _check(lib.dnpeff_op_mu(int(np.prod(F.shape)), F.ptr, num.ptr, den.ptr, eps))


def op_sparsify_columns(W_nr: DeviceArray, l1_norm: float, l2_norm: float = 1.0) -> int:
    """The reference's sparseness projection of every column of W [n, r], in place; returns the
    number of passes of its loop (DenseFactorSparsityContext::sparsifyF,
    dense_factor_sparsity_constraints.h:205-237)."""
    rounds = C.c_int(0)
    _check(lib.dnpeff_op_sparsify_columns(W_nr.shape[0], W_nr.shape[1], W_nr.ptr, l1_norm, l2_norm,
                                          C.byref(rounds)))
    return rounds.value


def op_spmm_n(A: "Csr", r: int, H_mr: DeviceArray, N_nr: DeviceArray):
    _check(lib.dnpeff_op_spmm_n(A._h, r, H_mr.ptr, N_nr.ptr))


def op_spmm_t(A: "Csr", r: int, W_nr: DeviceArray, T_mr: DeviceArray):
    _check(lib.dnpeff_op_spmm_t(A._h, r, W_nr.ptr, T_mr.ptr))


def op_gram(X: DeviceArray, G: DeviceArray):
    _check(lib.dnpeff_op_gram(X.shape[0], X.shape[1], X.ptr, G.ptr))


def op_gram_static(X: DeviceArray, G: DeviceArray, rows: Optional[int] = None):
    """G = X^T X of the first `rows` rows of X through the entry point that allocates nothing."""
    _check(lib.dnpeff_op_gram_static(X.shape[0] if rows is None else rows, X.shape[1], X.ptr, G.ptr))


def op_xg_mu(X: DeviceArray, G: DeviceArray, num: DeviceArray, eps: float, out: DeviceArray, D_out=None):
    _check(
        lib.dnpeff_op_xg_mu(X.shape[0], X.shape[1], X.ptr, G.ptr, num.ptr, eps, out.ptr,
                            None if D_out is None else D_out.ptr)
    )


def op_xg_mu_gram(X: DeviceArray, G: DeviceArray, num: DeviceArray, eps: float, out: DeviceArray,
                  Gout: DeviceArray):
    """Rank 128: out = X * num / (X G + eps) and Gout = out^T out in one pass."""
    assert X.shape[1] == 128
    _check(lib.dnpeff_op_xg_mu_gram(X.shape[0], X.ptr, G.ptr, num.ptr, eps, out.ptr, Gout.ptr))


def op_dot(x: DeviceArray, y: DeviceArray) -> float:
    v = _f64(0)
    _check(lib.dnpeff_op_dot(int(np.prod(x.shape)), x.ptr, y.ptr, C.byref(v)))
    return v.value


def op_spsp_dense(A: "Csr", B: "Csr", out: DeviceArray):
    _check(lib.dnpeff_op_spsp_dense(A._h, B._h, out.ptr))


def op_init_uniform(matrix_id: int, logical_rows: int, logical_cols: int, seed: int, x: DeviceArray):
    _check(lib.dnpeff_op_init_uniform(matrix_id, logical_rows, logical_cols, seed & 0xFFFFFFFFFFFFFFFF, x.ptr))


def topk_rows(x: "DeviceArray", k: int):
    """(values [n, k], indices [n, k], norms [n]) of the k largest entries of each row of x."""
    n, count = x.shape
    vals = DeviceArray((n, k), dtype=np.float32)
    idx = DeviceArray((n, k), dtype=np.int32)
    norms = DeviceArray((n,), dtype=np.float32)
    _check(lib.dnpeff_topk_rows(n, count, k, x.ptr, vals.ptr, idx.ptr, norms.ptr))
    sync()
    return vals.numpy(), idx.numpy(), norms.numpy()


def op_threshold_compact(x: "DeviceArray", divisor: float, threshold: float):
    """(positions, values) of the elements with x / divisor >= threshold, as numpy arrays."""
    n = int(np.prod(x.shape))
    idx = DeviceArray((max(n, 1),), dtype=np.int32)
    val = DeviceArray((max(n, 1),), dtype=np.float32)
    kept = _i64(0)
    _check(lib.dnpeff_op_threshold_compact(n, x.ptr, float(divisor), float(threshold), idx.ptr, val.ptr,
                                           C.byref(kept)))
    return idx.numpy()[:kept.value].copy(), val.numpy()[:kept.value].copy()


class Csr:
    """Device-resident CSR matrix: the reference's ElCsrMatrix / Host::CsrMatrix plus the
    loader steps that the mains apply to it (cc/cuda_d_npeff/src/util/matrices.h:172-199)."""

    def __init__(self, handle):
        self._h = handle

    # -- construction -------------------------------------------------------
    @staticmethod
    def from_host(rowptr, colind, vals, n_cols: int) -> "Csr":
        rowptr = _arr(rowptr, np.int64)
        colind = _arr(colind, np.int32)
        vals = _arr(vals, np.float32)
        h = C.c_void_p()
        _check(
            lib.dnpeff_csr_from_host(
                len(rowptr) - 1, n_cols, len(colind), _ptr(rowptr), _ptr(colind), _ptr(vals), C.byref(h)
            )
        )
        return Csr(h)

    @staticmethod
    def from_pef(indices, values, dense_fisher_size: int) -> "Csr":
        """PefSparseFishers::read's CSR (cc/cuda_d_npeff/src/io/pef_fisher_h5.h:170-177)."""
        indices = _arr(indices, np.int32)
        values = _arr(values, np.float32)
        assert indices.ndim == 2 and indices.shape == values.shape
        h = C.c_void_p()
        _check(
            lib.dnpeff_csr_from_pef(
                indices.shape[0], indices.shape[1], dense_fisher_size, _ptr(indices), _ptr(values), C.byref(h)
            )
        )
        return Csr(h)

    @staticmethod
    def synth(n_rows, n_cols, k_fixed=0, k_min=0, k_max=0, zipf_s=1.1, mu=-8.0, sigma=2.0, seed=0):
        """Device generator; returns (Csr, norms)."""
        norms = np.zeros(n_rows, dtype=np.float32)
        h = C.c_void_p()
        _check(
            lib.dnpeff_synth_pef(
                n_rows, n_cols, k_fixed, k_min, k_max, zipf_s, mu, sigma, seed & 0xFFFFFFFFFFFFFFFF,
                _ptr(norms), C.byref(h),
            )
        )
        return Csr(h), norms

    # -- loader steps -------------------------------------------------------
    def normalize_rows(self, norms, eps: float = 1e-9):
        norms = _arr(norms, np.float32)
        assert len(norms) == self.n_rows
        _check(lib.dnpeff_csr_normalize_rows(self._h, _ptr(norms), eps))

    def compact_columns(self, min_count: int = 1):
        _check(lib.dnpeff_csr_compact_columns(self._h, min_count))

    def retain_columns(self, kept):
        kept = _arr(kept, np.int32)
        _check(lib.dnpeff_csr_retain_columns(self._h, _ptr(kept), len(kept)))

    # -- inspection ---------------------------------------------------------
    def _shape3(self):
        a, b, c = _i64(0), _i64(0), _i64(0)
        _check(lib.dnpeff_csr_shape(self._h, C.byref(a), C.byref(b), C.byref(c)))
        return a.value, b.value, c.value

    @property
    def n_rows(self):
        return self._shape3()[0]

    @property
    def n_cols(self):
        return self._shape3()[1]

    @property
    def nnz(self):
        return self._shape3()[2]

    @property
    def full_dense_size(self):
        v = _i64(0)
        _check(lib.dnpeff_csr_full_dense_size(self._h, C.byref(v)))
        return v.value

    def density(self) -> float:
        n, m, z = self._shape3()
        return z / float(n * m)

    def download(self):
        n, _, z = self._shape3()
        rowptr = np.zeros(n + 1, dtype=np.int64)
        colind = np.zeros(z, dtype=np.int32)
        vals = np.zeros(z, dtype=np.float32)
        _check(lib.dnpeff_csr_download(self._h, _ptr(rowptr), _ptr(colind), _ptr(vals)))
        return rowptr, colind, vals

    def kept_indices(self):
        out = np.zeros(self.n_cols, dtype=np.int32)
        _check(lib.dnpeff_csr_kept_indices(self._h, _ptr(out)))
        return out

    def get_row(self, row: int):
        """(cols, vals) of one row as the products hold it (works on a consumed matrix)."""
        cnt = _i64(0)
        _check(lib.dnpeff_csr_get_row(self._h, row, 0, C.byref(cnt), None, None))
        cols = np.zeros(cnt.value, dtype=np.int32)
        vals = np.zeros(cnt.value, dtype=np.float32)
        _check(lib.dnpeff_csr_get_row(self._h, row, cnt.value, C.byref(cnt), _ptr(cols), _ptr(vals)))
        return cols, vals

    def get_column(self, col: int):
        """(rows, vals) of one column as the products hold it."""
        cnt = _i64(0)
        _check(lib.dnpeff_csr_get_column(self._h, col, 0, C.byref(cnt), None, None))
        rows = np.zeros(cnt.value, dtype=np.int32)
        vals = np.zeros(cnt.value, dtype=np.float32)
        _check(lib.dnpeff_csr_get_column(self._h, col, cnt.value, C.byref(cnt), _ptr(rows), _ptr(vals)))
        return rows, vals

    def sq_norm(self) -> float:
        v = _f64(0)
        _check(lib.dnpeff_csr_sq_norm(self._h, C.byref(v)))
        return v.value

    def split_dense_head(self, min_fill: float) -> int:
        """Moves the columns held by at least min_fill of the rows into a dense block
        (min_fill <= 0 undoes it); returns the number of such columns."""
        nd = _i64(0)
        _check(lib.dnpeff_csr_split_dense_head(self._h, float(min_fill), C.byref(nd)))
        return nd.value

    def head_info(self):
        nd, zs = _i64(0), _i64(0)
        _check(lib.dnpeff_csr_head_info(self._h, C.byref(nd), C.byref(zs)))
        return nd.value, zs.value

    def products_info(self):
        """dict(panels, plain, swept_pieces, tail_floor, list_entries, list_batches) of the sparse part."""
        out = np.zeros(6, dtype=np.int64)
        _check(lib.dnpeff_csr_products_info(self._h, _ptr(out)))
        return dict(zip(("panels", "plain", "swept_pieces", "tail_floor", "list_entries", "list_batches"),
                        (int(v) for v in out)))

    def build_transpose(self):
        _check(lib.dnpeff_csr_build_transpose(self._h))

    def download_transpose(self):
        _, m, z = self._shape3()
        colptr = np.zeros(m + 1, dtype=np.int64)
        rowind = np.zeros(z, dtype=np.int32)
        vals = np.zeros(z, dtype=np.float32)
        _check(lib.dnpeff_csr_download_transpose(self._h, _ptr(colptr), _ptr(rowind), _ptr(vals)))
        return colptr, rowind, vals

    def close(self):
        if self._h is not None:
            lib.dnpeff_csr_destroy(self._h)
            self._h = None

    def __del__(self):  # pragma: no cover
        try:
            self.close()
        except Exception:
            pass


@dataclass
class MuNmfParams:
    """MuNmfParams (multi_mu_dense_factors_device_contexts1.h:36-46); defaults as set by
    run_nmf_on_pefs (cc/cuda_d_npeff/mains/run_nmf_on_pefs.cu:189-200)."""

    rank: int
    max_iters: int
    eps: float = 1e-8
    seed: int = 43190432042
    log_every: int = 10


class MuNmf:
    """Dense-factor multiplicative-update NMF on one GPU (MuNmf<IndT>,
    multi_mu_dense_factors_nmf1.h:42-375)."""

    def __init__(self, A: Csr, params: MuNmfParams, consume_matrix: bool = False):
        """consume_matrix: the context may free the arrays of A that its products do not read
        (DNPEFF_NMF_CONSUME_MATRIX), for matrices that only fit the device that way."""
        self.A = A
        self.params = params
        self.n_rows, self.n_cols, _ = A._shape3()
        h = C.c_void_p()
        _check(lib.dnpeff_nmf_create_ex(A._h, params.rank, params.eps, params.seed,
                                        1 if consume_matrix else 0, C.byref(h)))
        self._h = h
        self._initialized = False

    def info(self):
        """(tiled H update?, tile width in columns)."""
        t, c = C.c_int(0), _i64(0)
        _check(lib.dnpeff_nmf_info(self._h, C.byref(t), C.byref(c)))
        return bool(t.value), c.value

    def device_factors(self):
        """Device addresses of W [n, r] and H [m, r]."""
        w, h = C.c_void_p(), C.c_void_p()
        _check(lib.dnpeff_nmf_device_factors(self._h, C.byref(w), C.byref(h)))
        return w.value, h.value

    def initialize(self):
        """_initializeBeforeRun (nmf1.h:128-150): W then H ~ U[0,1) from the seed."""
        _check(lib.dnpeff_nmf_init_factors(self._h))
        self._initialized = True

    def set_factors(self, W=None, H=None):
        W = None if W is None else _arr(W, np.float32)
        H = None if H is None else _arr(H, np.float32)
        if W is not None:
            assert W.shape == (self.n_rows, self.params.rank)
        if H is not None:
            assert H.shape == (self.params.rank, self.n_cols)
        _check(lib.dnpeff_nmf_set_factors(self._h, _ptr(W), _ptr(H)))
        self._initialized = True

    def step(self, n_steps: int = 1):
        _check(lib.dnpeff_nmf_step(self._h, n_steps))

    def update_W(self):
        _check(lib.dnpeff_nmf_update_W(self._h))

    def update_H(self):
        _check(lib.dnpeff_nmf_update_H(self._h))

    def run(self, log: Callable[[str], None] = print):
        """MuNmf::run (nmf1.h:152-205): W-update, H-update; every log_every steps the loss and
        the mean ms/step of the window, loss time excluded.  Returns [(step, loss, ms_per_step)]."""
        if not self._initialized:
            self.initialize()
        p = self.params
        history = []
        sync()
        t0 = time.perf_counter()
        for step in range(p.max_iters):
            self.step(1)
            if p.log_every > 0 and (step + 1) % p.log_every == 0:
                sync()
                elapsed_ms = (time.perf_counter() - t0) * 1e3
                loss = self.computeUncachedLoss()
                ms = elapsed_ms / p.log_every
                log(f"step {step + 1}: {loss:g} [{ms:g} ms/step]")
                history.append((step + 1, loss, ms))
                t0 = time.perf_counter()
        sync()
        return history

    def computeUncachedLoss(self) -> float:
        v = _f64(0)
        _check(lib.dnpeff_nmf_loss(self._h, C.byref(v)))
        return v.value

    def loss_terms(self):
        a, p, q = _f64(0), _f64(0), _f64(0)
        _check(lib.dnpeff_nmf_loss_terms(self._h, C.byref(a), C.byref(p), C.byref(q)))
        return a.value, p.value, q.value

    def check_products(self):
        """(<A H^T, W> via the row-ordered kernels, <A^T W, H> via the column-ordered ones)."""
        a, b = _f64(0), _f64(0)
        _check(lib.dnpeff_nmf_check_products(self._h, C.byref(a), C.byref(b)))
        return a.value, b.value

    def sparsify_W(self, l1_norm: float, l2_norm: float = 1.0) -> int:
        """sparseContextW->sparsifyF() on the context's W (the call that the reference leaves
        commented out at multi_mu_dense_factors_nmf1.h:161-162); returns the passes taken."""
        rounds = C.c_int(0)
        _check(lib.dnpeff_nmf_sparsify_W(self._h, l1_norm, l2_norm, C.byref(rounds)))
        return rounds.value

    def loadWToHostSync(self) -> np.ndarray:
        """W as [n, r] row-major (after the reference's toRowMajor_inPlace)."""
        W = np.zeros((self.n_rows, self.params.rank), dtype=np.float32)
        _check(lib.dnpeff_nmf_get_W(self._h, _ptr(W)))
        return W

    def loadHToHostSync(self) -> np.ndarray:
        """H as [r, m] row-major (after the reference's toRowMajor_inPlace)."""
        H = np.zeros((self.params.rank, self.n_cols), dtype=np.float32)
        _check(lib.dnpeff_nmf_get_H(self._h, _ptr(H)))
        return H

    def set_profiling(self, enable: bool):
        _check(lib.dnpeff_nmf_set_profiling(self._h, 1 if enable else 0))

    def timings(self, reset: bool = False):
        ms = np.zeros(len(KERNEL_CLASSES), dtype=np.float64)
        cnt = np.zeros(len(KERNEL_CLASSES), dtype=np.int64)
        _check(lib.dnpeff_nmf_timings(self._h, _ptr(ms), _ptr(cnt), 1 if reset else 0))
        return {k: (float(ms[i]), int(cnt[i])) for i, k in enumerate(KERNEL_CLASSES)}

    def close(self):
        if self._h is not None:
            lib.dnpeff_nmf_destroy(self._h)
            self._h = None

    def __del__(self):  # pragma: no cover
        try:
            self.close()
        except Exception:
            pass


@dataclass
class LearnerParams:
    """LearnerParams (cc/cuda_d_npeff/src/nmf/sparse2/only_W_learner_params.h:15-62); eps as set
    by fit_coeffs_to_sparse_H (cc/cuda_d_npeff/mains/fit_coeffs_to_sparse_H.cu:185)."""

    max_iters: int
    eps: float = 1e-7
    seed: int = 43190432042
    log_every_n_steps: int = 25


class Learner:
    """W-only learner against a fixed sparse H (Nmf::OnlyW::SparseH::Learner,
    nmf_sparse_H.h:42-345)."""

    def __init__(self, A: Csr, H: Csr, params: LearnerParams):
        self.params = params
        self.n_examples = A.n_rows
        self.n_components = H.n_rows
        h = C.c_void_p()
        _check(lib.dnpeff_fit_create(A._h, H._h, params.eps, params.seed, C.byref(h)))  # first stage
        self._h = h
        self._initialized = False

    def initialize(self):
        _check(lib.dnpeff_fit_init_W(self._h))
        self._initialized = True

    def set_W(self, W):
        W = _arr(W, np.float32)
        assert W.shape == (self.n_examples, self.n_components)
        _check(lib.dnpeff_fit_set_W(self._h, _ptr(W)))
        self._initialized = True

    def step(self, n_steps: int = 1):
        _check(lib.dnpeff_fit_step(self._h, n_steps))

    def losses(self):
        """(reference_loss, true_loss); see dnpeff_fit_loss."""
        a, b = _f64(0), _f64(0)
        _check(lib.dnpeff_fit_loss(self._h, C.byref(a), C.byref(b)))
        return a.value, b.value

    def Run(self, log: Callable[[str], None] = print):
        """RunSecondStage (nmf_sparse_H.h:298-340); the first stage ran in the constructor."""
        if not self._initialized:
            self.initialize()
        p = self.params
        history = []
        sync()
        t0 = time.perf_counter()
        for i in range(p.max_iters):
            self.step(1)
            if p.log_every_n_steps > 0 and (i + 1) % p.log_every_n_steps == 0:
                sync()
                elapsed_ms = (time.perf_counter() - t0) * 1e3
                ref_loss, true_loss = self.losses()
                ms = elapsed_ms / p.log_every_n_steps
                log(f"step {i + 1}: {ref_loss:g} [{ms:g} ms/step]")
                history.append((i + 1, ref_loss, true_loss, ms))
                t0 = time.perf_counter()
        sync()
        return history

    def GetOnHost_W(self) -> np.ndarray:
        W = np.zeros((self.n_examples, self.n_components), dtype=np.float32)
        _check(lib.dnpeff_fit_get_W(self._h, _ptr(W)))
        return W

    def products(self):
        AH = np.zeros((self.n_examples, self.n_components), dtype=np.float32)
        HH = np.zeros((self.n_components, self.n_components), dtype=np.float32)
        sq = _f64(0)
        _check(lib.dnpeff_fit_get_products(self._h, _ptr(AH), _ptr(HH), C.byref(sq)))
        return AH, HH, sq.value

    def close(self):
        if self._h is not None:
            lib.dnpeff_fit_destroy(self._h)
            self._h = None

    def __del__(self):  # pragma: no cover
        try:
            self.close()
        except Exception:
            pass
