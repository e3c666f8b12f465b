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
