#!/usr/bin/env python3
"""Times one kernel of the library through its C-ABI entry point (dnpeff_op_*), for profiling
with rocprofv3.

    python3 kernel_bench.py --op xg_mu --rows 8000000 --rank 128 --iters 5
    python3 kernel_bench.py --op spmm_n --n 10000 --m-full 110000000 --k 65536 --rank 128

Dense ops (mu, gram, xg_mu, copy) run on uniform random [rows, rank] operands; sparse ops
(spmm_n, spmm_t) on a synthetic PEF matrix (Zipf columns, compacted).  `copy` is a plain device
copy of rows*rank floats, the yardstick for scaling FETCH_SIZE / WRITE_SIZE counters."""

import argparse
import ctypes as C
import os
import sys
import time

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import npeff_ref_amd as d  # noqa: E402


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--op", required=True, choices=["mu", "gram", "xg_mu", "xg_mu_gram", "copy", "spmm_n", "spmm_t", "topk"])
    ap.add_argument("--rows", type=int, default=4_000_000)
    ap.add_argument("--rank", type=int, default=128)
    ap.add_argument("--iters", type=int, default=5)
    ap.add_argument("--n", type=int, default=2000)
    ap.add_argument("--m-full", type=int, default=22_000_000)
    ap.add_argument("--k", type=int, default=32768)
    ap.add_argument("--zipf", type=float, default=1.1)
    ap.add_argument("--seed", type=int, default=1)
    a = ap.parse_args()
    r = a.rank

    def uniform(rows, cols, seed):
        x = d.DeviceArray((rows, cols))
        d.op_init_uniform(0, rows, cols, seed, x)
        return x

    if a.op in ("spmm_n", "spmm_t"):
        A, norms = d.Csr.synth(a.n, a.m_full, k_fixed=a.k, zipf_s=a.zipf, seed=a.seed)
        A.normalize_rows(norms)
        A.compact_columns(1)
        A.build_transpose()
        n, m, z = A.n_rows, A.n_cols, A.nnz
        H, W = uniform(m, r, 2), uniform(n, r, 3)
        N, T = d.DeviceArray((n, r)), d.DeviceArray((m, r))
        fn = (lambda: d.op_spmm_n(A, r, H, N)) if a.op == "spmm_n" else (lambda: d.op_spmm_t(A, r, W, T))
        work = 8 * z + 4 * (n + 1 if a.op == "spmm_n" else m + 1) + 4 * r * m + 4 * n * r
        desc = f"n={n} m={m} nnz={z} r={r}"
    elif a.op == "topk":
        # --rows examples of --m-full dense Fisher values each, the --k largest kept
        rows, count, k = a.rows, a.m_full, a.k
        X = uniform(rows, count, 2)
        vals, idx = d.DeviceArray((rows, k)), d.DeviceArray((rows, k), dtype=np.int32)
        norms = d.DeviceArray((rows,))
        fn = lambda: d.binding._check(d.lib.dnpeff_topk_rows(rows, count, k, X.ptr, vals.ptr, idx.ptr, norms.ptr))
        work = 4 * rows * count
        desc = f"rows={rows} count={count} k={k}"
    else:
        rows = a.rows
        X = uniform(rows, r, 2)
        desc = f"rows={rows} r={r}"
        if a.op == "gram":
            G = d.DeviceArray((r, r))
            fn = lambda: d.op_gram(X, G)
            work = 2 * rows * r * r
        elif a.op == "xg_mu":
            G, num, out = uniform(r, r, 4), uniform(rows, r, 5), d.DeviceArray((rows, r))
            fn = lambda: d.op_xg_mu(X, G, num, 1e-12, out)
            work = 2 * rows * r * r
        elif a.op == "xg_mu_gram":
            # the H update of the factorisation at rank 128: in place on the numerator
            G, num, Gout = uniform(r, r, 4), uniform(rows, r, 5), d.DeviceArray((r, r))
            fn = lambda: d.op_xg_mu_gram(X, G, num, 1e-12, num, Gout)
            work = 12 * rows * r
        elif a.op == "mu":
            num, den = uniform(rows, r, 5), uniform(rows, r, 6)
            fn = lambda: d.op_mu(X, num, den, 1e-12)
            work = 16 * rows * r
        else:
            out = d.DeviceArray((rows, r))
            fn = lambda: d.binding._check(d.lib.dnpeff_op_copy(rows * r, X.ptr, out.ptr))
            work = 8 * rows * r
    fn()
    d.sync()
    t0 = time.perf_counter()
    for _ in range(a.iters):
        fn()
    d.sync()
    ms = (time.perf_counter() - t0) * 1e3 / a.iters
    unit = "TFLOP/s" if a.op in ("gram", "xg_mu") else "GB/s"
    rate = work / ms / (1e9 if unit == "TFLOP/s" else 1e6)
    print(f"{a.op} {desc}: {ms:.3f} ms per call, {rate:.1f} {unit} (algorithmic)")


if __name__ == "__main__":
    main()
