"""The C-ABI library loads and exports every function include/dnpeff.h declares; host-only
entry points (split sizes, seeded uniform, host generator).  No compute on a GPU."""

import os
import re

import numpy as np
import pytest

import npeff_ref_amd as d
from npeff_ref_amd import binding

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "dnpeff.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dnpeff_[A-Za-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    names = _declared_functions()
    assert len(names) >= 50
    for name in names:
        assert hasattr(binding.lib, name), f"{name} not exported by libdnpeff_hip.so"
        assert name in binding.SIGNATURES, f"{name} has no ctypes signature"
    assert sorted(binding.SIGNATURES) == names


def test_product_does_not_touch_the_oracle():
    """Nothing under npeff_ref_amd/ may include, import or link the oracle."""
    pkg = os.path.join(ROOT, "npeff_ref_amd")
    for dirpath, _, files in os.walk(pkg):
        if os.sep + "build" in dirpath or os.sep + "lib" in dirpath:
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h", ".cc", ".c", "Makefile")):
                text = open(os.path.join(dirpath, f), errors="replace").read()
                assert "oracle" not in text.lower(), f"{f} mentions the oracle"


def test_size_of_split_matches_reference_rule():
    assert [d.size_of_split(10, 3, i) for i in range(3)] == [3, 3, 4]
    assert d.size_of_split(7, 1, 0) == 7
    with pytest.raises(d.DnpeffError):
        d.size_of_split(10, 3, 3)


def test_uniform_at_range_and_keying():
    seed = 43190432042
    v = np.array([d.uniform_at(seed, 0, i, c, 16) for i in range(200) for c in range(16)])
    assert v.min() >= 0.0 and v.max() < 1.0
    assert abs(v.mean() - 0.5) < 0.02 and abs(v.var() - 1 / 12) < 0.01
    assert d.uniform_at(seed, 0, 3, 4, 16) == d.uniform_at(seed, 0, 3, 4, 16)
    assert d.uniform_at(seed, 0, 3, 4, 16) != d.uniform_at(seed, 1, 3, 4, 16)
    assert d.uniform_at(seed, 0, 3, 4, 16) != d.uniform_at(seed + 1, 0, 3, 4, 16)
    # keyed by the logical element index row * n_cols + col
    assert d.uniform_at(seed, 0, 1, 0, 16) == d.uniform_at(seed, 0, 0, 16, 32)


def test_host_generator_shape_distinctness_and_norms():
    n, m, k = 64, 100000, 512
    rowptr, colind, vals, norms = d.synth_pef_host(n, m, k_fixed=k, zipf_s=1.1, seed=7)
    assert rowptr.tolist() == [i * k for i in range(n + 1)]
    assert colind.min() >= 0 and colind.max() < m
    for i in range(n):
        row = colind[i * k : (i + 1) * k]
        assert len(np.unique(row)) == k  # sampling without replacement
        want = np.float32(np.sqrt(np.sum(vals[i * k : (i + 1) * k].astype(np.float64) ** 2)))
        assert abs(norms[i] - want) <= np.spacing(want)
    assert vals.dtype == np.float32 and vals.min() > 0
    # log-normal(-8, 2): mean and spread of log(values)
    lv = np.log(vals.astype(np.float64))
    assert abs(lv.mean() + 8.0) < 0.05 and abs(lv.std() - 2.0) < 0.05
    # Zipf head: id 0 is in (almost) every row, the first draw is id 0 about 1/H(m, s) of the time
    assert np.mean([0 in colind[i * k : (i + 1) * k] for i in range(n)]) > 0.95
    # reproducible, seed-dependent
    again = d.synth_pef_host(n, m, k_fixed=k, zipf_s=1.1, seed=7)
    assert np.array_equal(again[1], colind) and np.array_equal(again[2], vals)
    other = d.synth_pef_host(n, m, k_fixed=k, zipf_s=1.1, seed=8)
    assert not np.array_equal(other[1], colind)


def test_host_generator_first_draw_follows_zipf():
    # the first draw of each row is a plain Zipf(s) sample: compare head frequencies
    n, m, s = 4000, 1000, 1.3
    rowptr, colind, _, _ = d.synth_pef_host(n, m, k_fixed=1, zipf_s=s, seed=3)
    p = np.arange(1, m + 1, dtype=np.float64) ** (-s)
    p /= p.sum()
    freq = np.bincount(colind, minlength=m) / n
    for i in range(4):
        assert abs(freq[i] - p[i]) < 4 * np.sqrt(p[i] * (1 - p[i]) / n) + 1e-3


def test_host_generator_ragged_rows():
    rowptr, colind, vals, norms = d.synth_pef_host(50, 200000, k_min=16, k_max=4096, seed=11)
    lens = np.diff(rowptr)
    assert lens.min() >= 16 and lens.max() <= 4096 and len(np.unique(lens)) > 10
    assert rowptr[-1] == len(colind) == len(vals)


def test_generator_rejects_impossible_requests():
    with pytest.raises(d.DnpeffError):
        d.synth_pef_host(2, 10, k_fixed=8)  # k > n_cols / 2
    with pytest.raises(d.DnpeffError):
        d.synth_pef_host(2, 1000, k_fixed=8, zipf_s=1.0)


def test_tuning_switches_round_trip_and_reject_unknown_names():
    assert d.tuning_get("sweep_spin") == 400.0
    d.tuning_set("sweep_spin", 3)
    assert d.tuning_get("sweep_spin") == 3.0
    d.tuning_reset()
    assert d.tuning_get("sweep_spin") == 400.0
    with pytest.raises(d.DnpeffError, match="no tuning switch"):
        d.tuning_set("no_such_switch", 1)
    with pytest.raises(d.DnpeffError, match="no tuning switch"):
        d.tuning_get("no_such_switch")


def test_host_generator_row_range_matches_the_whole_matrix():
    rowptr, colind, vals, norms = d.synth_pef_host(30, 80000, k_fixed=200, zipf_s=1.3, seed=9)
    rp, ci, va, nr = d.synth_pef_host_rows(11, 4, 80000, k_fixed=200, zipf_s=1.3, seed=9)
    assert rp.tolist() == [0, 200, 400, 600, 800]
    assert np.array_equal(ci, colind[11 * 200:15 * 200]) and np.array_equal(va, vals[11 * 200:15 * 200])
    assert np.array_equal(nr, norms[11:15])


def test_bench_work_model_and_sample_sizes():
    """bench.py's algorithmic bytes follow the formulas of the measurement plan, and the CPU
    sample is the whole matrix for configs[1] and a few hundred rows for configs[3]."""
    import bench

    n, m, z, r = 20_000, 211_311_151, 5_242_880_000, 256
    assert bench.algorithmic("spmm_n", n, m, z, r)[0] == 8 * z + 8 * (n + 1) + 4 * r * m + 4 * n * r
    assert bench.algorithmic("spmm_t", n, m, z, r)[0] == 8 * z + 8 * (m + 1) + 4 * n * r + 4 * r * m
    assert bench.algorithmic("spmm_n", 10, 100, 1000, 4)[0] == 8 * 1000 + 4 * 11 + 4 * 4 * 100 + 4 * 10 * 4
    b, f, split = bench.algorithmic("xg_mu_H", n, m, z, r, split_bf16=True)
    assert b == 12 * m * r + 4 * r * r and f == 2 * m * r * r and split
    assert bench.cpu_sample_rows(bench.CONFIGS["c1"]) == 10_000
    assert 256 <= bench.cpu_sample_rows(bench.CONFIGS["c3"]) <= 1024
    # the value is whatever the committed counter summary holds (it changes with every refresh of
    # the profile): parse the file here, independently, and compare
    import os, re
    path = os.path.join(bench.ROOT, "profiles", "nmf_c3_hbm_traffic.md")
    held = [float(x) for x in re.findall(r"traffic_bytes\s+spmm_n\s+([0-9.eE+]+)", open(path).read())]
    got, src = bench.traffic_from_profile("c3", "spmm_n")
    assert held and got == held[0] and got > 8 * z and src == "profiles/nmf_c3_hbm_traffic.md"
    assert bench.traffic_from_profile("c3", "no_such_class") == (None, None)
    assert bench.traffic_from_profile("c0", "spmm_n") == (None, None)


def test_memory_plan_arithmetic_for_the_benchmark_shapes():
    """dnpeff_plan_estimate needs no GPU: the byte table of the memory plan for the shapes of
    BASELINE configs[1], [3] and [4] as generated (kept columns, entries of the sparse part and head
    columns as the full-size runs report them) follows the sizing rules, fits the 309.2 GB the
    device reports, and prices a larger head higher."""
    total = 309_220_868_096
    n, m, r = 20_000, 211_311_151, 256
    c3 = d.plan_estimate(n, m, 2_355_000_000, 437_520, r, tiled=True, total_bytes=total)
    full = d.plan_estimate(n, m, 2_355_000_000, 437_520, r, tiled=False, total_bytes=total)
    tile = (768 * 2**20 // (4 * r)) // 128 * 128  # h_tile_mb = 768 MiB of the factor, a multiple of 128 columns
    assert tile == 786_432
    # full-size: H and A^T W as two [m, r] arrays; tiled: [m + tile, r] and [tile, r]
    assert full["factors"] - c3["factors"] == 4.0 * r * (m - 2 * tile)
    assert c3["factors"] > 4.0 * r * (m + 2 * tile) + 3 * 4.0 * n * r
    # plain panels capped so that their partial sums stay within 3 GB, plus one set per XCD
    panels = int(3.0e9 // (4 * n * r))
    assert panels == 146 and c3["partials"] == 4.0 * r * n * (panels + 8)
    assert c3["segments"] == 8.0 * n * (3072 + 1)
    assert 8.0 * (m + 1) < c3["offsets"] < 8.5 * (m + 1)
    assert c3["reserve"] == total / 64
    assert c3["sparse_copies"] == 16.0 * 2_355_000_000
    assert c3["head_blocks"] == 4.0 * 20_096 * 437_632  # one block, rows and columns padded to 128
    assert 0 < c3["head_workspace"] < 0.1 * c3["head_blocks"]
    assert sum(c3.values()) < total < sum(full.values())  # only the tiled update fits
    bigger = d.plan_estimate(n, m, 2_000_000_000, 600_000, r, tiled=True, total_bytes=total)
    assert bigger["head_blocks"] > c3["head_blocks"] and bigger["head_workspace"] >= c3["head_workspace"]
    assert sum(bigger.values()) > total  # the head at fill 1/16 does not fit beside H: the threshold rises
    c1 = d.plan_estimate(10_000, 65_941_155, 382_000_000, 120_802, 128, tiled=False, total_bytes=total)
    assert sum(c1.values()) < 0.3 * total and c1["head_blocks"] == 2 * 4.0 * 10_112 * 120_832 / 2
    c4 = d.plan_estimate(40_000, 107_300_000, 2_000_000_000, 100_000, 512, tiled=True, total_bytes=total)
    assert sum(c4.values()) < total
    # a small device: the reserve never goes below 1 GiB
    assert d.plan_estimate(512, 900_000, 2_097_152, 0, 16, False, total_bytes=8 * 2**30)["reserve"] == 2.0**30
    with pytest.raises(d.DnpeffError):
        d.plan_estimate(10, 5, 1, 6, 16, False)  # more head columns than columns
