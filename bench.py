#!/usr/bin/env python3
"""D-NPEFF NMF benchmark on one MI355X: MU iterations/sec on BASELINE.json configs[1]
(10,000 examples x 110M features, 65,536 nnz/row, Zipf 1.1 columns, r = 128), per-kernel
roofline fractions from HIP events, and the same update loop timed on the host cores.

    python bench.py --gpus 1 --steps K --warmup W

Prints ONE JSON line.  A step is one MU iteration (W-update then H-update) with the CSR
matrix and the factors already resident in HBM; the loss is not evaluated inside the timed
region, exactly as the reference's own timer excludes it
(cc/cuda_d_npeff/src/nmf/sparse/multi_mu_dense_factors_nmf1.h:188-200)."""

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12  # B/s, MI355X HBM3E
MFMA_FP32_PEAK = 157.3e12  # flop/s, dense fp32 matrix
MFMA_BF16_PEAK = 2.5e15  # flop/s, dense bf16 matrix

CONFIGS = {
    "c0": dict(n=512, m_full=1 << 20, k=4096, kmin=0, kmax=0, s=1.1, r=16),
    "c1": dict(n=10_000, m_full=110_000_000, k=65_536, kmin=0, kmax=0, s=1.1, r=128),
    "c1-small": dict(n=1_000, m_full=11_000_000, k=16_384, kmin=0, kmax=0, s=1.1, r=128),
    # downscaled shapes of configs[3] (Zipf 1.3, r = 256) and configs[4] (ragged rows, r = 512)
    "c3-small": dict(n=5_000, m_full=90_000_000, k=65_536, kmin=0, kmax=0, s=1.3, r=256),
    "c4-small": dict(n=5_000, m_full=40_000_000, k=0, kmin=1_024, kmax=131_072, s=1.1, r=512),
}


# HBM-side bytes per launch of the long kernel of each class on configs[1], from rocprofv3 --pmc
# FETCH_SIZE (x 2.0) + WRITE_SIZE (x 1.0), the factors being what the same counters read for a
# plain copy of known size; counters cannot be read from inside this process, so the figures of
# the committed profile are carried here and apply to the unchanged c1 workload only.
TRAFFIC_C1 = {
    "spmm_n": 65.8e9 + 0.7e9 + 18.3e9 + 0.1e9 + 5.6e9,  # plain panels, swept pieces, dense head
    "spmm_t": 65.5e9 + 33.7e9 + 7.4e9 + 0.1e9 + 5.6e9,
    "gram_H": 33.8e9 + 0.1e9,
    "xg_mu_H": 67.5e9 + 33.9e9,  # the fused update: H, numerator in, new H out
}


def log(msg):
    print(f"[bench {time.strftime('%H:%M:%S')}] {msg}", file=sys.stderr, flush=True)


def algorithmic(cls, n, m, z, r, fused_gram=False, split_bf16=False):
    """Compulsory work of one launch, every operand touched once: (bytes, fp32 flops, split).
    flops = 0 for the kernels without a matrix product.  With fused_gram the H update also
    produces H^T H (no separate gram_H launch): its class carries both products.  split = the
    products run on the bf16 matrix cores (every fp32 operand as the sum of three bf16 numbers,
    six partial products, fp32 accumulation): the launch then executes 6 x flops on a peak that
    is 16 times the fp32 cores'."""
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


def price(cls, n, m, z, r, avg_s, fused_gram, split_bf16):
    """The roofline that binds a launch of mean duration avg_s: the larger of its HBM fraction and
    its matrix-core fraction (fp32 cores, or bf16 cores for the split-operand kernels)."""
    nbytes, flops, split = algorithmic(cls, n, m, z, r, fused_gram, split_bf16)
    f_hbm = nbytes / avg_s / HBM_PEAK
    f_mm = (6 * flops / avg_s / MFMA_BF16_PEAK) if split else (flops / avg_s / MFMA_FP32_PEAK)
    if f_mm > f_hbm:
        done = 6 * flops if split else flops
        return dict(bound="mfma", achieved=done / avg_s / 1e12, unit="TFLOP/s",
                    peak=(MFMA_BF16_PEAK if split else MFMA_FP32_PEAK) / 1e12, frac=f_mm,
                    arithmetic="bf16 x 6 (split fp32 operands)" if split else "fp32")
    return dict(bound="hbm", achieved=nbytes / avg_s / 1e9, unit="GB/s", peak=HBM_PEAK / 1e9,
                frac=f_hbm)


def prepare_cpu_baseline(d, A, nmf, n, m, r, eps):
    """Copies the CSR matrix and the initial factors to the host for the fp32 OpenMP port of the
    reference loop (oracle/dnpeff_oracle.c: orc_f32_step)."""
    from oracle import oracle as orc

    t0 = time.perf_counter()
    rp, ci, va = A.download()
    W0 = nmf.loadWToHostSync()
    Ht0 = np.empty((m, r), dtype=np.float32)
    wdev, hdev = C.c_void_p(), C.c_void_p()
    d.binding._check(d.lib.dnpeff_nmf_device_factors(nmf._h, C.byref(wdev), C.byref(hdev)))
    d.binding._check(d.lib.dnpeff_dev_download(Ht0.ctypes.data_as(C.c_void_p), hdev, Ht0.nbytes))
    log(f"cpu baseline: inputs on the host in {time.perf_counter() - t0:.1f} s")
    t0 = time.perf_counter()
    base = orc.F32Baseline(rp, ci, va, m, W0, eps=eps, Ht0_mr=Ht0)
    del Ht0
    log(f"cpu baseline: context (host transposed CSR) in {time.perf_counter() - t0:.1f} s, "
        f"{orc.F32Baseline.num_threads()} threads")
    return base


def run_cpu_baseline(base, steps, n, m, z, r):
    from oracle import oracle as orc

    t0 = time.perf_counter()
    base.step(steps)
    el = time.perf_counter() - t0
    base.close()
    log(f"cpu baseline: {steps} step(s) in {el:.2f} s")
    return {"value": steps / el, "unit": "MU iterations/s", "cores": orc.F32Baseline.num_threads(),
            "kind": "port",
            "sample": f"{steps} full MU iteration(s) of the same workload (n={n}, m={m}, nnz={z}, r={r}), "
                      "fp32 OpenMP port of the reference loop, loss excluded"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--config", default="c1", choices=sorted(CONFIGS))
    ap.add_argument("--eps", type=float, default=1e-12)
    ap.add_argument("--seed", type=int, default=43190432042)
    ap.add_argument("--cpu-steps", type=int, default=1,
                    help="MU iterations timed on the host cores (0 = skip)")
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
    log(f"device {name}, {hbm_bytes / 2**30:.0f} GiB, {cus} CUs; workload {args.config} {cfg}")

    t0 = time.perf_counter()
    A, norms = d.Csr.synth(cfg["n"], cfg["m_full"], k_fixed=cfg["k"], k_min=cfg["kmin"],
                           k_max=cfg["kmax"], zipf_s=cfg["s"], seed=args.seed)
    log(f"generated {A.nnz} entries on the device in {time.perf_counter() - t0:.1f} s")
    t0 = time.perf_counter()
    A.normalize_rows(norms)
    A.compact_columns(1)
    n, m, z = A.n_rows, A.n_cols, A.nnz
    log(f"normalised + compacted: n={n} m={m} (of {cfg['m_full']}) nnz={z} "
        f"in {time.perf_counter() - t0:.1f} s")
    r = cfg["r"]
    t0 = time.perf_counter()
    nmf = d.MuNmf(A, d.MuNmfParams(rank=r, max_iters=0, eps=args.eps, seed=args.seed))
    nmf.initialize()
    d.sync()
    n_dense, z_sparse = A.head_info()
    log(f"context (dense head of {n_dense} columns, {z_sparse} entries stay sparse, transposed CSR, "
        f"factors) in {time.perf_counter() - t0:.1f} s")

    # the CPU baseline starts from the same factors, so copy them before the GPU loop runs
    cpu = prepare_cpu_baseline(d, A, nmf, n, m, r, args.eps) if args.cpu_steps > 0 else None

    nmf.step(args.warmup)
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
    log(f"{args.steps} steps in {elapsed:.3f} s -> {ms_per_step:.2f} ms/step, loss {loss:.10g}")

    kernels = {}
    fused_gram = tim.get("gram_H", (0.0, 0))[1] == 0
    split_bf16 = os.environ.get("DNPEFF_SPLIT_BF16", "1") != "0"
    for cls, (ms_sum, cnt) in tim.items():
        if cnt == 0:
            continue
        avg_s = ms_sum / cnt * 1e-3
        k = price(cls, n, m, z, r, avg_s, fused_gram, split_bf16)
        k.update(ms=ms_sum / cnt, share=ms_sum / (elapsed * 1e3))
        kernels[cls] = k
        log(f"  {cls:14s} {k['ms']:9.3f} ms  {k['achieved']:9.1f} {k['unit']:8s} frac {k['frac']:.3f}")
    dom = max((k for k in kernels if k != "spmm_n_reduce"), key=lambda k: kernels[k]["ms"])
    kd = kernels[dom]
    roofline = dict(kernel=dom, bound=kd["bound"], achieved=kd["achieved"], peak=kd["peak"],
                    unit=kd["unit"], frac=kd["frac"],
                    traffic=TRAFFIC_C1.get(dom) if args.config == "c1" else None)

    cpu_baseline = run_cpu_baseline(cpu, args.cpu_steps, n, m, z, r) if cpu is not None else None

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
        "config": {"workload": "configs[1] D-NPEFF NMF" if args.config == "c1" else args.config,
                   "n_examples": n, "n_features_full": cfg["m_full"], "n_features_kept": m,
                   "nnz": z, "nnz_per_row": cfg["k"], "zipf_s": cfg["s"], "rank": r,
                   "eps": args.eps, "seed": args.seed, "dense_head_columns": n_dense,
                   "nnz_sparse_part": z_sparse},
        "roofline": roofline,
        "cpu_baseline": cpu_baseline,
        "kernels": kernels,
        "fused_gram_in_H_update": fused_gram,
        "matrix_products": ("bf16 MFMA on fp32 operands split in three (6 partial products, fp32 "
                            "accumulation, fp32 accuracy) where the kernel table says so"
                            if split_bf16 else "fp32 MFMA"),
        "spmm_hbm_frac": {k: kernels[k]["frac"] for k in ("spmm_n", "spmm_t") if k in kernels},
        "loss_after": loss,
    }
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
