#!/usr/bin/env python3
"""D-NPEFF NMF benchmark on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W [--config c3|c1|c2|c4|...]

Default workload: BASELINE.json configs[3], the configuration the target is quoted on (20,000
examples x 350M features, 262,144 entries per row = 5.24e9 entries, Zipf 1.3 columns, r = 256).
`--config c1` is configs[1] (10,000 x 110M, 65,536 per row, r = 128), `--config c2` the
fit_coeffs_to_sparse_H path of configs[2] (first stage + W-only loop against a fixed sparse H),
`--config c4` the ragged-row case of configs[4] with the comparison of work decompositions.

Prints ONE JSON line.  A step is one MU iteration (W-update then H-update) with the matrix and
the factors already resident in HBM; the loss is not evaluated inside the timed region, exactly
as the reference's own timer excludes it
(cc/cuda_d_npeff/src/nmf/sparse/multi_mu_dense_factors_nmf1.h:188-200).  Per-kernel times come
from HIP events on the library's stream.  The run checks itself: the two sparse products must
agree on <A H^T, W> = <A^T W, H> over every entry, and the loss must decrease."""

import argparse
import ctypes as C
import json
import os
import platform
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12  # B/s, MI355X HBM3E
MFMA_FP32_PEAK = 157.3e12  # flop/s, dense fp32 matrix
MFMA_BF16_PEAK = 2.5e15  # flop/s, dense bf16 matrix

CONFIGS = {
    "c0": dict(kind="nmf", name="configs[0] CPU plumbing shape", n=512, m_full=1 << 20, k=4096, kmin=0, kmax=0,
               s=1.1, r=16),
    "c1": dict(kind="nmf", name="configs[1] D-NPEFF NMF", n=10_000, m_full=110_000_000, k=65_536, kmin=0, kmax=0,
               s=1.1, r=128),
    "c1-small": dict(kind="nmf", name="configs[1] downscaled 10 x 10 x 4", n=1_000, m_full=11_000_000, k=16_384,
                     kmin=0, kmax=0, s=1.1, r=128),
    "c2": dict(kind="fit", name="configs[2] fit_coeffs_to_sparse_H", n=50_000, m_full=110_000_000, k=65_536,
               s=1.1, r=256, density=0.01),
    "c2-small": dict(kind="fit", name="configs[2] downscaled (5,000 new examples)", n=5_000,
                     m_full=110_000_000, k=65_536, s=1.1, r=256, density=0.01),
    "c3": dict(kind="nmf", name="configs[3] large D-NPEFF NMF", n=20_000, m_full=350_000_000, k=262_144, kmin=0,
               kmax=0, s=1.3, r=256),
    "c3-small": dict(kind="nmf", name="configs[3] downscaled (5,000 x 90M, 65,536 per row)", n=5_000,
                     m_full=90_000_000, k=65_536, kmin=0, kmax=0, s=1.3, r=256),
    "c4": dict(kind="nmf", name="configs[4] ragged rows", n=40_000, m_full=110_000_000, k=0, kmin=1_024,
               kmax=524_288, s=1.1, r=512, compare_rows=6_000),
    "c4-small": dict(kind="nmf", name="configs[4] downscaled (5,000 rows, 1,024..131,072 per row)", n=5_000,
                     m_full=40_000_000, k=0, kmin=1_024, kmax=131_072, s=1.1, r=512, compare_rows=5_000),
}


def log(msg):
    print(f"[bench {time.strftime('%H:%M:%S')}] {msg}", file=sys.stderr, flush=True)


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return platform.processor() or "unknown"


def physical_cores():
    """Distinct (package, core) pairs among the CPUs this process may run on; None where /proc does
    not tell."""
    try:
        allowed = os.sched_getaffinity(0)
        seen, cur = set(), {}
        for line in open("/proc/cpuinfo"):
            if ":" in line:
                k, v = (x.strip() for x in line.split(":", 1))
                cur[k] = v
            elif cur:
                if int(cur.get("processor", -1)) in allowed:
                    seen.add((cur.get("physical id", "0"), cur.get("core id", cur.get("processor"))))
                cur = {}
        if cur and int(cur.get("processor", -1)) in allowed:
            seen.add((cur.get("physical id", "0"), cur.get("core id", cur.get("processor"))))
        return len(seen) or None
    except Exception:
        return None


def algorithmic(cls, n, m, z, r, fused_gram=False, split_bf16=False):
    """Compulsory work of one product / update over the whole matrix, every operand touched once:
    (bytes, fp32 flops, split).  flops = 0 for the kernels without a matrix product.  With
    fused_gram the H update also produces H^T H (no separate gram_H launch): its class carries
    both products.  split = the products run on the bf16 matrix cores (every fp32 operand as the
    sum of three bf16 numbers, six partial products, fp32 accumulation): the launch then executes
    6 x flops on a peak that is 16 times the fp32 cores'."""
    P = 4 if z < 2**31 else 8
    tiles = split_bf16 and r > 128 and r % 128 == 0  # the 128 x 128 tile kernels
    if cls == "spmm_n":
        return 8 * z + P * (n + 1) + 4 * r * m + 4 * n * r, 0, False
    if cls == "spmm_n_reduce":
        return 8 * n * r, 0, False
    if cls == "spmm_t":
        return 8 * z + P * (m + 1) + 4 * n * r + 4 * r * m, 0, False
    # a Gram matrix is symmetric: r (r + 1) / 2 distinct dot products of length e
    if cls == "gram_H":
        return 4 * m * r + 4 * r * r, m * r * (r + 1), tiles and m >= 1024
    if cls == "gram_W":
        return 4 * n * r + 4 * r * r, n * r * (r + 1), tiles and n >= 1024
    if cls == "xg_mu_H":
        if fused_gram:
            return 12 * m * r + 8 * r * r, 2 * m * r * r + m * r * (r + 1), split_bf16
        return 12 * m * r + 4 * r * r, 2 * m * r * r, tiles and m >= 256
    if cls == "xg_mu_W":
        return 12 * n * r + 4 * r * r, 2 * n * r * r, tiles and n >= 256
    raise KeyError(cls)


def price(cls, n, m, z, r, step_s, fused_gram, split_bf16):
    """The roofline that binds a class that takes step_s seconds per MU iteration (one launch, or
    the launches of all column tiles together): the larger of its HBM fraction and its
    matrix-core fraction (fp32 cores, or bf16 cores for the split-operand kernels)."""
    nbytes, flops, split = algorithmic(cls, n, m, z, r, fused_gram, split_bf16)
    f_hbm = nbytes / step_s / HBM_PEAK
    f_mm = (6 * flops / step_s / MFMA_BF16_PEAK) if split else (flops / step_s / MFMA_FP32_PEAK)
    if f_mm > f_hbm:
        done = 6 * flops if split else flops
        return dict(bound="mfma", achieved=done / step_s / 1e12, unit="TFLOP/s",
                    peak=(MFMA_BF16_PEAK if split else MFMA_FP32_PEAK) / 1e12, frac=f_mm,
                    hbm_frac=f_hbm, arithmetic="bf16 x 6 (split fp32 operands)" if split else "fp32")
    return dict(bound="hbm", achieved=nbytes / step_s / 1e9, unit="GB/s", peak=HBM_PEAK / 1e9,
                frac=f_hbm)


def traffic_from_profile(config, cls):
    """HBM-side bytes per MU iteration of a kernel class, read from the committed counter summary
    profiles/nmf_<config>_hbm_traffic.md, or fit_<config>_hbm_traffic.md for the fit path (a line
    `traffic_bytes <class> <bytes>`); (None, None)
    when there is no such file or line: counters cannot be read from inside this process."""
    kind = "fit" if CONFIGS.get(config, {}).get("kind") == "fit" else "nmf"
    path = os.path.join(ROOT, "profiles", f"{kind}_{config}_hbm_traffic.md")
    try:
        for line in open(path):
            mm = re.match(r"\s*`?traffic_bytes\s+(\w+)\s+([0-9.eE+]+)`?", line)
            if mm and mm.group(1) == cls:
                return float(mm.group(2)), os.path.relpath(path, ROOT)
    except OSError:
        pass
    return None, None


# ------------------------------------------------------------------------------------------
# CPU baseline: the fp32 OpenMP port of the reference loop on the host cores, on a bounded sample
# ------------------------------------------------------------------------------------------
def cpu_sample_rows(cfg, rows=0):
    """Rows of the sample: all of them while n k r stays within ~1e11 multiply-adds per product
    (configs[1] in full), else the first rows of the matrix up to ~3.5e10 (about 10 s per iteration
    of the port on 16 threads); `rows` > 0 (--cpu-rows) overrides the rule."""
    if rows > 0:
        return min(cfg["n"], rows)
    k_mean = cfg["k"] if cfg["k"] else (cfg["kmax"] - cfg["kmin"]) / np.log(cfg["kmax"] / cfg["kmin"])
    if cfg["n"] * k_mean * cfg["r"] <= 1.0e11:
        return cfg["n"]
    return max(64, min(cfg["n"], int(3.5e10 / (k_mean * cfg["r"]))))


def prepare_cpu_sample(d, cfg, seed, rows):
    """The first `rows` rows of the workload's matrix (the generator keys rows by their number),
    loaded like the whole matrix (normalised, its own empty columns dropped), on the host."""
    t0 = time.perf_counter()
    A, norms = d.Csr.synth(rows, cfg["m_full"], k_fixed=cfg["k"], k_min=cfg["kmin"], k_max=cfg["kmax"],
                           zipf_s=cfg["s"], seed=seed)
    A.normalize_rows(norms)
    A.compact_columns(1)
    rp, ci, va = A.download()
    m_s = A.n_cols
    A.close()
    log(f"cpu baseline: sample of {rows} rows ({len(ci)} entries, {m_s} columns) on the host in "
        f"{time.perf_counter() - t0:.1f} s")
    return rp, ci, va, m_s


def run_cpu_baseline(sample, cfg, n, m, z, r, eps, iters=3):
    """Times `iters` MU iterations of the port on the sample, one by one (the loss is not evaluated,
    as the reference's own timer leaves it out, multi_mu_dense_factors_nmf1.h:188-200), and scales
    each part by its own unit count to the whole workload: the sparse products by entries, the
    H-sized dense parts by columns, the W-sized ones by rows.  `value` comes from the median
    iteration; the fastest one is reported beside it."""
    from oracle import oracle as orc

    rp, ci, va, m_s = sample
    n_s, z_s = len(rp) - 1, len(ci)
    rng = np.random.default_rng(0)
    W0 = rng.random((n_s, r), dtype=np.float32)
    Ht0 = rng.random((m_s, r), dtype=np.float32)
    t0 = time.perf_counter()
    base = orc.F32Baseline(rp, ci, va, m_s, W0, eps=eps, Ht0_mr=Ht0)
    del Ht0
    threads = orc.F32Baseline.num_threads()
    cores = physical_cores()
    log(f"cpu baseline: context (host transposed CSR) in {time.perf_counter() - t0:.1f} s, {threads} threads on "
        f"{cores} physical cores, {cpu_model()}")
    scale = {"spmm_n": z / z_s, "spmm_t": z / z_s, "gram_H": m / m_s, "xg_mu_H": m / m_s,
             "gram_W": n / n_s, "xg_mu_W": n / n_s}
    runs = []
    for it in range(max(1, iters)):
        parts = base.step_timed(1)
        runs.append((sum(parts[k] * scale[k] for k in parts), sum(parts.values()), parts))
        log(f"cpu baseline: iteration {it + 1} on the sample {runs[-1][1]:.2f} s -> {runs[-1][0]:.1f} s for the "
            "whole workload; parts " + ", ".join(f"{k} {v:.2f}" for k, v in parts.items()))
    base.close()
    order = sorted(range(len(runs)), key=lambda i: runs[i][0])
    full_s, sample_s, parts = runs[order[len(order) // 2]]  # the median iteration
    best_s = runs[order[0]][0]
    whole = n_s == n
    return {"value": 1.0 / full_s, "unit": "MU iterations/s", "cores": threads, "physical_cores": cores,
            "kind": "port", "cpu_model": cpu_model(), "iterations_timed": len(runs),
            "seconds_per_iteration_whole_workload": {"median": full_s, "min": best_s,
                                                     "all": [x[0] for x in runs]},
            "sample": (f"{len(runs)} MU iterations of the fp32 OpenMP port of the reference loop (loss excluded), "
                       "timed one by one, on "
                       + (f"the whole workload (n={n}, m={m}, nnz={z}, r={r}): median {full_s:.2f} s, fastest "
                          f"{best_s:.2f} s" if whole else
                          f"the first {n_s} of {n} rows with their {m_s} non-empty columns ({z_s} entries, r={r}): "
                          f"median {sample_s:.2f} s; scaled to the whole workload part by part (sparse products by "
                          f"entries x{z / z_s:.1f}, H-sized parts by columns x{m / m_s:.2f}, W-sized by rows): "
                          f"median {full_s:.1f} s, fastest {best_s:.1f} s")),
            "sample_seconds": sample_s, "parts_seconds_sample": parts}


def run_scipy_baseline(sample, n, m, z, r, eps, max_entries=3.0e7):
    """The same iteration with scipy.sparse products (one thread) and numpy BLAS for the dense
    parts, on a smaller row sample, scaled the same way.  None when scipy is missing."""
    try:
        import scipy.sparse as sp
    except Exception:
        return None
    rp, ci, va, m_s = sample
    rows = int(np.searchsorted(rp, max_entries, side="right")) - 1
    rows = max(1, min(rows, len(rp) - 1))
    z_s = int(rp[rows])
    A = sp.csr_matrix((va[:z_s], ci[:z_s], rp[: rows + 1]), shape=(rows, m_s))
    At = A.T.tocsr()
    rng = np.random.default_rng(1)
    W = rng.random((rows, r), dtype=np.float32)
    Ht = rng.random((m_s, r), dtype=np.float32)
    e = np.float32(eps)
    t = {}
    t0 = time.perf_counter(); N = A @ Ht; t["spmm_n"] = time.perf_counter() - t0
    t0 = time.perf_counter(); G = Ht.T @ Ht; t["gram_H"] = time.perf_counter() - t0
    t0 = time.perf_counter(); W *= N / (W @ G + e); t["xg_mu_W"] = time.perf_counter() - t0
    t0 = time.perf_counter(); T = At @ W; t["spmm_t"] = time.perf_counter() - t0
    t0 = time.perf_counter(); G = W.T @ W; t["gram_W"] = time.perf_counter() - t0
    t0 = time.perf_counter()
    blk = 1 << 20  # (bounds the temporary of the dense product)
    for c0 in range(0, m_s, blk):
        Ht[c0:c0 + blk] *= T[c0:c0 + blk] / (Ht[c0:c0 + blk] @ G + e)
    t["xg_mu_H"] = time.perf_counter() - t0
    scale = {"spmm_n": z / z_s, "spmm_t": z / z_s, "gram_H": m / m_s, "xg_mu_H": m / m_s,
             "gram_W": n / rows, "xg_mu_W": n / rows}
    full_s = sum(t[k] * scale[k] for k in t)
    log(f"scipy baseline: {rows} rows ({z_s} entries, {m_s} columns) {sum(t.values()):.2f} s -> {full_s:.1f} s "
        "for the whole workload")
    return {"value": 1.0 / full_s, "unit": "MU iterations/s", "kind": "scipy.sparse CSR @ dense (1 thread) + "
            "numpy BLAS", "sample": f"first {rows} rows ({z_s} entries) over the {m_s} columns of the port's "
            f"sample, one iteration {sum(t.values()):.2f} s, scaled part by part to {full_s:.1f} s",
            "parts_seconds_sample": t}


# ------------------------------------------------------------------------------------------
# dense-factor NMF (run_nmf_on_pefs)
# ------------------------------------------------------------------------------------------
def compare_decompositions(d, cfg, seed, r):
    """A H^T on the first rows of the ragged matrix under four work decompositions of the sparse
    part: one wavefront per row, 2048-entry row chunks, the merge path (equal shares of entries +
    rows, cut wherever the row boundaries fall) and the planned one (column panels + swept pieces
    + dense head).  Twice: with the row lengths of the configuration (1,024 .. 524,288, where a
    chunk split is the merge path up to the last, shorter chunk of each row) and with lengths from
    16 up, where thousands of short rows separate the two."""
    rows = cfg.get("compare_rows")
    if not rows:
        return None
    out = {}
    for label, kmin in (("as_configured", cfg["kmin"]), ("short_rows_too", 16)):
        A, norms = d.Csr.synth(rows, cfg["m_full"], k_fixed=cfg["k"], k_min=kmin, k_max=cfg["kmax"],
                               zipf_s=cfg["s"], seed=seed)
        A.normalize_rows(norms)
        A.compact_columns(1)
        n, m, z = A.n_rows, A.n_cols, A.nnz
        lens = np.diff(A.download()[0])
        hist, edges = np.histogram(np.log2(lens), bins=np.arange(4, 20.01, 2.0))
        H = d.DeviceArray((m, r))
        d.op_init_uniform(0, m, r, seed, H)
        N = d.DeviceArray((n, r))
        res = {"rows": n, "columns": m, "entries": z, "rank": r,
               "row_length_histogram_log2": {f"2^{int(a)}..2^{int(b)}": int(c)
                                             for a, b, c in zip(edges[:-1], edges[1:], hist)},
               "row_length_min_max": [int(lens.min()), int(lens.max())]}
        ref = None
        for variant, name in ((1, "wave_per_row"), (2, "row_chunks_2048"), (3, "merge_path_4096"),
                              (0, "planned_panels_sweeps_head")):
            for _ in range(2):
                d.binding._check(d.lib.dnpeff_op_spmm_n_variant(A._h, r, H.ptr, N.ptr, variant))
            d.sync()
            t0 = time.perf_counter()
            reps = 3
            for _ in range(reps):
                d.binding._check(d.lib.dnpeff_op_spmm_n_variant(A._h, r, H.ptr, N.ptr, variant))
            d.sync()
            ms = (time.perf_counter() - t0) * 1e3 / reps
            got = N.numpy()
            if ref is None:
                ref = got.astype(np.float64)
            err = float(np.max(np.abs(got - ref)) / np.max(np.abs(ref)))
            res[name] = {"ms": ms, "max_rel_diff_vs_wave_per_row": err}
            log(f"  A H^T on {n} ragged rows of {lens.min()}..{lens.max()} entries ({z} in all), {name}: "
                f"{ms:.2f} ms (diff {err:.1e})")
        dense_cols, z_sparse = A.head_info()
        res["dense_head_columns"], res["entries_sparse_part"] = dense_cols, z_sparse
        H.free(); N.free(); A.close()
        out[label] = res
    return out


def run_nmf(d, args, cfg):
    r = cfg["r"]
    cpu_rows = cpu_sample_rows(cfg, args.cpu_rows) if args.cpu_steps > 0 else 0
    sample = prepare_cpu_sample(d, cfg, args.seed, cpu_rows) if 0 < cpu_rows < cfg["n"] else None
    comparison = (compare_decompositions(d, cfg, args.seed, r)
                  if cfg.get("compare_rows") and not args.no_compare else None)

    free0, total = d.device_memory()
    t0 = time.perf_counter()
    A, norms = d.Csr.synth(cfg["n"], cfg["m_full"], k_fixed=cfg["k"], k_min=cfg["kmin"], k_max=cfg["kmax"],
                           zipf_s=cfg["s"], seed=args.seed)
    log(f"generated {A.nnz} entries on the device in {time.perf_counter() - t0:.1f} s")
    t0 = time.perf_counter()
    A.normalize_rows(norms)
    A.compact_columns(1)
    n, m, z = A.n_rows, A.n_cols, A.nnz
    log(f"normalised + compacted: n={n} m={m} (of {cfg['m_full']}) nnz={z} in {time.perf_counter() - t0:.1f} s")
    if sample is None and args.cpu_steps > 0:  # the whole matrix is the sample: copy it before it is consumed
        t0 = time.perf_counter()
        sample = A.download() + (m,)
        log(f"cpu baseline: whole matrix on the host in {time.perf_counter() - t0:.1f} s")
    t0 = time.perf_counter()
    nmf = d.MuNmf(A, d.MuNmfParams(rank=r, max_iters=0, eps=args.eps, seed=args.seed), consume_matrix=True)
    nmf.initialize()
    d.sync()
    n_dense, z_sparse = A.head_info()
    tiled, tile_cols = nmf.info()
    free1, _ = d.device_memory()
    log(f"context in {time.perf_counter() - t0:.1f} s: dense head of {n_dense} columns, {z_sparse} entries stay "
        f"sparse, {'tiled H update, ' + str(tile_cols) + ' columns per tile' if tiled else 'full-size H update'}; "
        f"device memory {(total - free1) / 1e9:.1f} of {total / 1e9:.1f} GB in use")

    nmf.step(args.warmup)
    d.sync()
    loss_before = nmf.computeUncachedLoss()
    # (the loss leaves A H^T behind for the next W update: one more untimed step, so that every
    # timed step computes both products)
    nmf.step(1)
    d.sync()
    nmf.set_profiling(True)
    nmf.timings(reset=True)
    d.sync()
    t0 = time.perf_counter()
    nmf.step(args.steps)
    d.sync()
    elapsed = time.perf_counter() - t0
    tim = nmf.timings(reset=True)
    nmf.set_profiling(False)
    loss = nmf.computeUncachedLoss()
    ms_per_step = elapsed * 1e3 / args.steps
    log(f"{args.steps} steps in {elapsed:.3f} s -> {ms_per_step:.2f} ms/step, loss {loss_before:.10g} -> {loss:.10g}")

    # the run checks itself
    via_rows, via_cols = nmf.check_products()
    products_rel = abs(via_rows - via_cols) / abs(via_rows)
    log(f"<A H^T, W> = {via_rows:.12g} (row-ordered kernels), <A^T W, H> = {via_cols:.12g} (column-ordered): "
        f"relative difference {products_rel:.1e}")
    ok = np.isfinite(loss) and loss < loss_before and products_rel < 1e-5
    if not ok:
        print("bench.py: self-check failed (loss must decrease, the two products must agree to 1e-5)",
              file=sys.stderr)

    kernels = {}
    fused_gram = tim.get("gram_H", (0.0, 0))[1] == 0
    split_bf16 = d.tuning_get("split_bf16") != 0.0
    for cls, (ms_sum, cnt) in tim.items():
        if cnt == 0:
            continue
        step_s = ms_sum / args.steps * 1e-3
        k = price(cls, n, m, z, r, step_s, fused_gram, split_bf16)
        k.update(ms=ms_sum / args.steps, launches_per_step=cnt / args.steps, share=ms_sum / (elapsed * 1e3))
        kernels[cls] = k
        log(f"  {cls:14s} {k['ms']:9.3f} ms/step ({k['launches_per_step']:.0f} launches)  {k['achieved']:9.1f} "
            f"{k['unit']:8s} frac {k['frac']:.3f}")
    dom = max((k for k in kernels if k != "spmm_n_reduce"), key=lambda k: kernels[k]["ms"])
    kd = kernels[dom]
    traffic, traffic_src = traffic_from_profile(args.config, dom)
    roofline = dict(kernel=dom, bound=kd["bound"], achieved=kd["achieved"], peak=kd["peak"], unit=kd["unit"],
                    frac=kd["frac"], traffic=traffic, traffic_source=traffic_src,
                    per="MU iteration (all launches of the class: one per column tile in the tiled H update)")

    # the same steps with the matrix products on the fp32 matrix cores
    fp32_ms = None
    if args.fp32_steps > 0 and split_bf16:
        d.tuning_set("split_bf16", 0)
        try:
            nmf.step(1)
            d.sync()
            t0 = time.perf_counter()
            nmf.step(args.fp32_steps)
            d.sync()
            fp32_ms = (time.perf_counter() - t0) * 1e3 / args.fp32_steps
            log(f"products on the fp32 matrix cores: {fp32_ms:.2f} ms/step")
        except d.DnpeffError as e:
            log(f"products on the fp32 matrix cores: not measured ({e})")
        d.tuning_set("split_bf16", 1)
    sparse_plan = A.products_info()
    nmf.close()
    A.close()

    cpu_baseline = scipy_baseline = None
    if args.cpu_steps > 0:
        cpu_baseline = run_cpu_baseline(sample, cfg, n, m, z, r, args.eps, args.cpu_steps)
        if not args.no_scipy:
            scipy_baseline = run_scipy_baseline(sample, n, m, z, r, args.eps)

    # The gather models beside the algorithmic bytes: what a product moves into the CUs when every
    # gathered entry brings a whole row of a factor (4 r bytes).  "untiled": every entry of the matrix
    # gathers; "planned": only the entries of the sparse part do, the dense head reads each of its
    # factor rows once and its own block.  Rates are bytes over the measured time of the class, as a
    # fraction of the HBM peak: above 1 means the caches served gathers, far below it with traffic near
    # these bytes means the gathers went to the fabric.
    P = 4 if z < 2**31 else 8
    head_bytes = 4 * n_dense * (n + r)
    gather_model = {}
    for cls, ptr_bytes, streamed in (("spmm_n", P * (n + 1), 4 * n * r), ("spmm_t", P * (m + 1), 4 * n * r + 4 * r * m)):
        if cls not in kernels:
            continue
        sec = kernels[cls]["ms"] / 1e3
        untiled = 8 * z + ptr_bytes + 4 * r * z + (4 * n * r if cls == "spmm_n" else 4 * r * m)
        planned = 8 * z_sparse + ptr_bytes + 4 * r * z_sparse + head_bytes + streamed
        gather_model[cls] = {"bytes_untiled": untiled, "bytes_planned": planned,
                             "untiled_frac_of_hbm_peak": untiled / sec / HBM_PEAK,
                             "planned_frac_of_hbm_peak": planned / sec / HBM_PEAK,
                             "planned_GBps": planned / sec / 1e9}
    out = {
        "metric": "NMF MU iterations/sec + SpMM achieved HBM GB/s (% of peak), 1 MI355X",
        "value": args.steps / elapsed,
        "unit": "MU iterations/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": cfg["name"], "n_examples": n, "n_features_full": cfg["m_full"],
                   "n_features_kept": m, "nnz": z, "nnz_per_row": cfg["k"] or [cfg["kmin"], cfg["kmax"]],
                   "zipf_s": cfg["s"], "rank": r, "eps": args.eps, "seed": args.seed,
                   "dense_head_columns": n_dense, "nnz_sparse_part": z_sparse, "tiled_H_update": tiled,
                   "H_tile_columns": tile_cols, "sparse_part_of_A_Ht": sparse_plan,
                   "H_gram_in_W_update": ("second stream, ahead of the dense head of A H^T; the class times count "
                                          "the time both run only once (under gram_H)"
                                          if d.tuning_get("gram_beside") != 0.0 and not fused_gram
                                          else "library stream"),
                   "device_memory_used_gb": (total - free1) / 1e9,
                   "device_memory_total_gb": total / 1e9},
        "roofline": roofline,
        "roofline_gather_model": gather_model,
        "cpu_baseline": cpu_baseline,
        "cpu_baseline_scipy": scipy_baseline,
        "gpu_over_cpu": (args.steps / elapsed) / cpu_baseline["value"] if cpu_baseline else None,
        "kernels": kernels,
        "fused_gram_in_H_update": fused_gram,
        "matrix_products": ("bf16 MFMA on fp32 operands split in three (6 partial products, fp32 "
                            "accumulation, fp32 accuracy) where the kernel table says so"
                            if split_bf16 else "fp32 MFMA"),
        "fp32_mfma_ms_per_step": fp32_ms,
        "spmm_hbm_frac": {k: (kernels[k]["hbm_frac"] if "hbm_frac" in kernels[k] else kernels[k]["frac"])
                          for k in ("spmm_n", "spmm_t") if k in kernels},
        "self_check": {"ok": bool(ok), "loss_before": loss_before, "loss_after": loss,
                       "products_relative_difference": products_rel},
        "load_balancing_comparison": comparison,
        "loss_after": loss,
    }
    print(json.dumps(out), flush=True)
    return 0 if ok else 4


# ------------------------------------------------------------------------------------------
# fixed sparse H, W-only learner (fit_coeffs_to_sparse_H)
# ------------------------------------------------------------------------------------------
def synth_sparse_H(r, m, density, seed):
    """Seeded r x m sparse H in CSR: every entry present with probability `density` (geometric
    gaps between the columns of a row), values exp(N(-8, 2^2)), ascending columns."""
    rng = np.random.default_rng(seed)
    rp, cols = [0], []
    for _ in range(r):
        gaps = rng.geometric(density, size=int(m * density * 1.05) + 64)
        idx = np.cumsum(gaps) - 1
        idx = idx[idx < m].astype(np.int32)
        cols.append(idx)
        rp.append(rp[-1] + len(idx))
    ci = np.concatenate(cols)
    va = np.exp(rng.normal(-8.0, 2.0, size=len(ci))).astype(np.float32)
    return np.array(rp, dtype=np.int64), ci, va


def run_fit(d, args, cfg):
    from oracle import oracle as orc

    r, m = cfg["r"], cfg["m_full"]
    t0 = time.perf_counter()
    hrp, hci, hva = synth_sparse_H(r, m, cfg["density"], args.seed)
    zh = len(hci)
    log(f"sparse H: {r} x {m}, {zh} entries ({zh / (r * m):.4f}) generated on the host in "
        f"{time.perf_counter() - t0:.1f} s")
    H = d.Csr.from_host(hrp, hci, hva, m)
    t0 = time.perf_counter()
    A, norms = d.Csr.synth(cfg["n"], m, k_fixed=cfg["k"], zipf_s=cfg["s"], seed=args.seed)
    A.normalize_rows(norms)
    # (H's reduce_kept_indices is the identity over all columns: RetainColumns_InPlace keeps every entry)
    d.sync()
    n, z = A.n_rows, A.nnz
    log(f"A: {n} new examples, {z} entries, generated and normalised in {time.perf_counter() - t0:.1f} s")

    # CPU sample: the first rows of A on the host, before the first stage may reorganise anything
    cpu = None
    if args.cpu_steps > 0:
        rows = max(16, min(n, int(2.0e8 / cfg["k"])))
        As, ns = d.Csr.synth(rows, m, k_fixed=cfg["k"], zipf_s=cfg["s"], seed=args.seed)
        As.normalize_rows(ns)
        cpu = As.download()
        As.close()

    d.sync()
    t0 = time.perf_counter()
    L = d.Learner(A, H, d.LearnerParams(max_iters=0, eps=1e-7, seed=args.seed))
    d.sync()
    stage1_s = time.perf_counter() - t0
    # the same first stage again on warm structures, kernel by kernel
    AH, HH = d.DeviceArray((n, r)), d.DeviceArray((r, r))
    d.op_spsp_dense(H, H, HH); d.sync()
    t0 = time.perf_counter(); d.op_spsp_dense(H, H, HH); d.sync(); hh_s = time.perf_counter() - t0
    d.op_spsp_dense(A, H, AH); d.sync()
    t0 = time.perf_counter(); d.op_spsp_dense(A, H, AH); d.sync(); ah_s = time.perf_counter() - t0
    spsp_bytes = 8 * z + 8 * zh
    log(f"first stage (transposed H, H H^T, A H^T, ||A||^2): {stage1_s:.3f} s; A H^T alone {ah_s * 1e3:.1f} ms "
        f"({spsp_bytes / ah_s / 1e9:.0f} GB/s algorithmic), H H^T {hh_s * 1e3:.1f} ms")
    L.initialize()
    L.step(args.warmup * 5)
    d.sync()
    steps = max(args.steps, 100)  # configs[2]: 100 iterations
    hist = []
    elapsed = 0.0
    t0 = time.perf_counter()
    log_every = 25  # log_every_n_steps (only_W_learner_params.h:35); the loss is not timed
    for i in range(steps):
        if i % log_every == 0:  # the steps up to the next logged one in one call of the library
            L.step(min(log_every, steps - i))
        if (i + 1) % log_every == 0:
            d.sync()
            elapsed += time.perf_counter() - t0
            hist.append((i + 1,) + L.losses())
            t0 = time.perf_counter()
    d.sync()
    elapsed += time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / steps
    ref_losses = [h[1] for h in hist]
    log(f"second stage: {steps} W updates, {ms_per_step:.4f} ms/step; logged loss {ref_losses}")
    # the run checks itself: the W update works row by row, so the first rows can be followed on
    # the host in fp64 from the same seeded start (H H^T and their rows of A H^T from the device)
    total_steps = args.warmup * 5 + steps
    chk = min(n, 48)
    W0 = np.array([[d.uniform_at(args.seed, 0, i, c, r) for c in range(r)] for i in range(chk)], dtype=np.float32)
    W64, _, _ = orc.fit_f64(AH.numpy()[:chk], HH.numpy(), 1.0, W0, np.float32(1e-7), total_steps, log_every=0)
    W_dev = L.GetOnHost_W()[:chk]
    w_err = float(np.linalg.norm(W_dev - W64) / np.linalg.norm(W64))
    log(f"W of the first {chk} examples after {total_steps} updates vs the fp64 host loop: {w_err:.1e}")
    ok = all(np.isfinite(ref_losses)) and w_err < 1e-4
    xg_bytes = 16 * n * r + 4 * r * r  # W, AH in; W, WHH out
    xg_flops = 2 * n * r * r

    cpu_baseline = None
    if cpu is not None:
        rp, ci, va = cpu
        ns_, zs_ = len(rp) - 1, len(ci)
        t0 = time.perf_counter()
        bt = orc.transpose(hrp, hci, hva, m)
        log(f"cpu baseline: transposed H on the host in {time.perf_counter() - t0:.1f} s")
        AH_s, s1 = orc.spsp_f32_timed((rp, ci, va), bt, r)
        got = AH.numpy()[:ns_]
        err = float(np.max(np.abs(got - AH_s)) / np.max(np.abs(AH_s)))
        ok = ok and err < 1e-4
        HHh = HH.numpy()
        rng = np.random.default_rng(0)
        Wc = rng.random((min(n, 8192), r), dtype=np.float32)
        _, s2 = orc.fit_steps_f32_timed(np.tile(AH_s, (len(Wc) // ns_ + 1, 1))[: len(Wc)], HHh, Wc, np.float32(1e-7), 5)
        s2_full = s2 / 5 * n / len(Wc)
        s1_full = s1 * z / zs_
        threads = orc.F32Baseline.num_threads()
        log(f"cpu baseline: A H^T on {ns_} rows {s1:.2f} s -> {s1_full:.1f} s for all rows; W update "
            f"{s2_full * 1e3:.1f} ms/step; GPU A H^T rows agree with the host port to {err:.1e}")
        cpu_baseline = {"value": 1.0 / s2_full, "unit": "W updates/s", "cores": threads, "kind": "port",
                        "cpu_model": cpu_model(),
                        "sample": f"second stage: 5 W updates on {len(Wc)} of {n} rows, scaled by rows; first stage "
                                  f"A H^T on the first {ns_} rows ({zs_} entries) in {s1:.2f} s, scaled by entries to "
                                  f"{s1_full:.1f} s (GPU: {ah_s:.3f} s)",
                        "first_stage_seconds": s1_full, "first_stage_gpu_over_cpu": s1_full / ah_s}
    out = {
        "metric": "fit_coeffs_to_sparse_H: W updates/sec (second stage) + first-stage sparse x sparse product, 1 MI355X",
        "value": steps / elapsed, "unit": "W updates/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup * 5,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": cfg["name"], "n_examples": n, "n_features": m, "nnz_A": z, "nnz_per_row": cfg["k"],
                   "rank": r, "nnz_H": zh, "H_density": zh / (r * m), "eps": 1e-7, "seed": args.seed},
        "roofline": {"kernel": "k_spsp (A H^T of the first stage)", "bound": "hbm", "achieved": spsp_bytes / ah_s / 1e9,
                     "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": spsp_bytes / ah_s / HBM_PEAK,
                     "traffic": traffic_from_profile(args.config, "spsp_AHt")[0],
                     "traffic_source": traffic_from_profile(args.config, "spsp_AHt")[1]},
        "first_stage": {"seconds_total": stage1_s, "AHt_ms": ah_s * 1e3, "HHt_ms": hh_s * 1e3,
                        "algorithmic_bytes": spsp_bytes},
        "second_stage": {"ms_per_step": ms_per_step, "hbm_frac": xg_bytes / (ms_per_step * 1e-3) / HBM_PEAK,
                         "tflops": xg_flops / (ms_per_step * 1e-3) / 1e12, "logged_losses": ref_losses},
        "cpu_baseline": cpu_baseline,
        "self_check": {"ok": bool(ok), "W_rows_vs_fp64_host_loop": w_err},
    }
    print(json.dumps(out), flush=True)
    return 0 if ok else 4


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--config", default="c3", choices=sorted(CONFIGS))
    ap.add_argument("--eps", type=float, default=1e-12)
    ap.add_argument("--seed", type=int, default=43190432042)
    ap.add_argument("--cpu-steps", type=int, default=3,
                    help="iterations of the host-core port that are timed (0 skips the host-core baselines)")
    ap.add_argument("--cpu-rows", type=int, default=0,
                    help="rows of the host-core sample (0 = about 10 s per iteration)")
    ap.add_argument("--fp32-steps", type=int, default=2,
                    help="steps timed with the matrix products on the fp32 matrix cores (0 = skip)")
    ap.add_argument("--no-scipy", action="store_true")
    ap.add_argument("--no-compare", action="store_true",
                    help="configs[4]: skip the comparison of the A H^T decompositions on the first rows")
    args = ap.parse_args()

    if args.gpus != 1:
        print("bench.py: this build drives exactly one GPU (no collectives are built); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import npeff_ref_amd as d

    if d.device_count() < 1:
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    cfg = CONFIGS[args.config]
    name, hbm_bytes, cus = d.device_info()
    log(f"device {name}, {hbm_bytes / 2**30:.0f} GiB, {cus} CUs; workload {args.config}: {cfg}")
    rc = run_fit(d, args, cfg) if cfg["kind"] == "fit" else run_nmf(d, args, cfg)
    sys.exit(rc)


if __name__ == "__main__":
    main()
