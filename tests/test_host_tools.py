"""The C++ host executables: flag behaviour and file layouts on the CPU; the full pipelines
(hdf5 in -> GPU NMF -> hdf5 out) on the GPU, compared with the same fit driven through the
C ABI from Python."""

import os
import subprocess

import numpy as np
import pytest

import h5lite
import npeff_ref_amd as d
from oracle import oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "npeff_ref_amd", "bin")

pytestmark = pytest.mark.skipif(
    not (h5lite.available and os.path.exists(os.path.join(BIN, "run_nmf_on_pefs"))),
    reason="host executables / HDF5 library not built",
)


def run(prog, *flags, check=False):
    p = subprocess.run([os.path.join(BIN, prog), *flags], capture_output=True, text=True, timeout=600)
    if check:
        assert p.returncode == 0, p.stdout + p.stderr
    return p


def make_pef(tmp_path, n=24, m=20000, k=300, seed=3, **extra):
    path = str(tmp_path / "pef.h5")
    flags = [f"--output_path={path}", f"--n_examples={n}", f"--n_parameters={m}", f"--n_fisher_values={k}",
             f"--seed={seed}"] + [f"--{a}={b}" for a, b in extra.items()]
    run("synth_pef_h5", *flags, check=True)
    return path


# ---- CPU: flags and schemas -----------------------------------------------------------------
def test_missing_required_flag_is_fatal(tmp_path):
    p = run("run_nmf_on_pefs", "--output_path=/tmp/x.h5")
    assert p.returncode != 0 and "Missing flag: per_example_fishers" in p.stdout
    p = run("fit_coeffs_to_sparse_H", "--output_path=/tmp/x.h5", "--pef_path=a")
    assert p.returncode != 0 and "Missing flag: H_path" in p.stdout


def test_fit_rejects_unknown_flags_but_nmf_ignores_them(tmp_path):
    p = run("fit_coeffs_to_sparse_H", "--output_path=o", "--pef_path=a", "--H_path=b", "--n_splits_sparse_matmul=1",
            "--n_row_splits_pefs=1", "--nmf_max_iter=1", "--bogus=3")
    assert p.returncode != 0 and "Unrecognized flags." in p.stdout


def test_synthetic_pef_file_has_the_reference_schema(tmp_path):
    path = make_pef(tmp_path, n=10, m=5000, k=64, seed=9)
    vals, idx = h5lite.read(path, "data/fisher/values"), h5lite.read(path, "data/fisher/indices")
    norms = h5lite.read(path, "data/dense_fisher_norms")
    assert vals.dtype == np.float32 and vals.shape == (10, 64)
    assert idx.dtype == np.int32 and idx.shape == (10, 64)
    assert norms.dtype == np.float32 and norms.shape == (10,)
    a, shape = h5lite.attr(path, "data/fisher", "dense_fisher_size")
    assert a.dtype == np.int32 and a.itemsize == 4 and int(a[0]) == 5000
    hr, hc, hv, hn = d.synth_pef_host(10, 5000, k_fixed=64, seed=9)
    assert np.array_equal(idx.ravel(), hc) and np.array_equal(vals.ravel(), hv) and np.array_equal(norms, hn)


def test_truncation_flags_larger_than_the_file_are_fatal(tmp_path):
    path = make_pef(tmp_path, n=4, m=1000, k=16)
    p = run("run_nmf_on_pefs", f"--output_path={tmp_path}/o.h5", f"--per_example_fishers={path}",
            "--nmf_n_components=2", "--nmf_max_iter=1", "--n_examples=5")
    assert p.returncode != 0 and "n_examples exceeds" in p.stdout


# ---- GPU: the pipelines ---------------------------------------------------------------------
@pytest.mark.gpu
def test_run_nmf_on_pefs_end_to_end(tmp_path):
    n, m_full, k, r, iters = 40, 30000, 500, 16, 20
    pef = make_pef(tmp_path, n=n + 8, m=m_full, k=k + 40, seed=11)
    out = str(tmp_path / "decomp.h5")
    p = run("run_nmf_on_pefs", f"--output_path={out}", f"--per_example_fishers={pef}", f"--nmf_n_components={r}",
            f"--nmf_max_iter={iters}", f"--n_examples={n}", f"--n_fisher_values={k}", "--min_values_per_parameter=2",
            "--sparsity_W=0.5", "--some_unknown_flag=1", check=True)
    lines = p.stdout.splitlines()
    assert "Using 32 bit indices." in lines and "PEFS read in." in lines and "Running NMF." in lines
    assert f"n_cols before reduction: {m_full}" in lines
    steps = [l for l in lines if l.startswith("step ")]
    assert [s.split(":")[0] for s in steps] == ["step 10", "step 20"] and all("ms/step]" in s for s in steps)

    # the same fit through the C ABI from Python, with the reference defaults (eps 1e-8, seed)
    vals = h5lite.read(pef, "data/fisher/values")[:n, :k]
    idx = h5lite.read(pef, "data/fisher/indices")[:n, :k]
    norms = h5lite.read(pef, "data/dense_fisher_norms")[:n]
    A = d.Csr.from_pef(idx, vals, m_full)
    A.normalize_rows(norms)
    A.compact_columns(2)
    nmf = d.MuNmf(A, d.MuNmfParams(rank=r, max_iters=iters))
    hist = nmf.run(log=lambda s: None)
    W, H, kept = h5lite.read(out, "data/W"), h5lite.read(out, "data/H"), h5lite.read(out, "data/reduce_kept_indices")
    assert W.dtype == np.float32 and W.shape == (n, r) and H.shape == (r, A.n_cols)
    assert np.array_equal(W, nmf.loadWToHostSync()) and np.array_equal(H, nmf.loadHToHostSync())
    assert kept.dtype == np.int32 and np.array_equal(kept, A.kept_indices())
    fds, shape = h5lite.attr(out, "data/reduce_kept_indices", "full_dense_size")
    assert shape == (1,) and int(fds[0]) == m_full  # the reference writes shape (1,) here
    logged = float(steps[-1].split(":")[1].split("[")[0])
    assert abs(logged - hist[-1][1]) / hist[-1][1] < 1e-5
    # and against the fp64 oracle
    rp, ci, va = A.download()
    W0 = np.array([[d.uniform_at(43190432042, 0, i, c, r) for c in range(r)] for i in range(n)], np.float32)
    nmf2 = d.MuNmf(A, d.MuNmfParams(rank=r, max_iters=0))
    nmf2.initialize()
    assert np.array_equal(nmf2.loadWToHostSync(), W0)
    W64, H64, losses = orc.nmf_f64(rp, ci, va, A.n_cols, W0, nmf2.loadHToHostSync(), np.float32(1e-8), iters, 10)
    assert np.linalg.norm(W - W64) / np.linalg.norm(W64) < 1e-4
    assert np.linalg.norm(H - H64) / np.linalg.norm(H64) < 1e-4
    assert abs(logged - losses[-1]) / losses[-1] < 1e-4


@pytest.mark.gpu
def test_run_nmf_on_pefs_wide_index_schema(tmp_path):
    """The reference's writer with IndT = int64 (nmf_decomp_h5.h:58-75) stores reduce_kept_indices and
    full_dense_size as int64; it is reached when the PEF file was read with 64-bit indices and
    the pruned matrix holds no more than INT32_MAX entries (run_nmf_on_pefs.cu:236-247 with
    matrices.h:219-224).  --index_width=64 forces that branch on a small file; the values are the
    same, and the fit path reads such a file."""
    n, m_full, k, r = 24, 9000, 300, 8
    pef = make_pef(tmp_path, n=n, m=m_full, k=k, seed=5)
    out32, out64 = str(tmp_path / "d32.h5"), str(tmp_path / "d64.h5")
    common = [f"--per_example_fishers={pef}", f"--nmf_n_components={r}", "--nmf_max_iter=3"]
    p = run("run_nmf_on_pefs", f"--output_path={out32}", *common, check=True)
    assert "Using 32 bit indices." in p.stdout.splitlines()
    assert "Running NMF using 32 bit indices." in p.stdout.splitlines()
    p = run("run_nmf_on_pefs", f"--output_path={out64}", "--index_width=64", *common, check=True)
    assert "Running NMF using 64 bit indices." in p.stdout.splitlines()
    k32, k64 = h5lite.read(out32, "data/reduce_kept_indices"), h5lite.read(out64, "data/reduce_kept_indices")
    assert k32.dtype == np.int32 and k64.dtype == np.int64 and np.array_equal(k32, k64)
    f32, s32 = h5lite.attr(out32, "data/reduce_kept_indices", "full_dense_size")
    f64, s64 = h5lite.attr(out64, "data/reduce_kept_indices", "full_dense_size")
    assert f32.dtype == np.int32 and f64.dtype == np.int64 and s32 == s64 == (1,)
    assert int(f32[0]) == int(f64[0]) == m_full
    assert np.array_equal(h5lite.read(out32, "data/H"), h5lite.read(out64, "data/H"))
    # the sparsifier reads the wide file as it reads the narrow one
    sp32, sp64 = str(tmp_path / "s32.h5"), str(tmp_path / "s64.h5")
    run("sparsify_d_npeff", f"--decomposition_filepath={out32}", f"--output_filepath={sp32}", "--H_threshold=1e-3",
        check=True)
    run("sparsify_d_npeff", f"--decomposition_filepath={out64}", f"--output_filepath={sp64}", "--H_threshold=1e-3",
        check=True)
    assert np.array_equal(h5lite.read(sp32, "data/H/values"), h5lite.read(sp64, "data/H/values"))


@pytest.mark.gpu
def test_fit_coeffs_to_sparse_H_end_to_end(tmp_path):
    n, m_full, k, r, iters = 50, 20000, 400, 8, 50
    pef = make_pef(tmp_path, n=n, m=m_full, k=k, seed=21, sparse_H_output_path=str(tmp_path / "H.h5"), rank=r,
                   H_density=0.02)
    hpath, out = str(tmp_path / "H.h5"), str(tmp_path / "fit.h5")
    p = run("fit_coeffs_to_sparse_H", f"--output_path={out}", f"--pef_path={pef}", f"--H_path={hpath}",
            "--n_splits_sparse_matmul=4", "--n_row_splits_pefs=2", f"--nmf_max_iter={iters}", check=True)
    lines = p.stdout.splitlines()
    assert "Finished running first stage." in lines and "Finished running second stage." in lines
    steps = [l for l in lines if l.startswith("step ")]
    assert [s.split(":")[0] for s in steps] == ["step 25", "step 50"]
    # output layout: new W, unchanged sparse H, scalar full_dense_size
    for name in ("values", "row_indices", "column_indices"):
        assert np.array_equal(h5lite.read(out, f"data/H/{name}"), h5lite.read(hpath, f"data/H/{name}"))
    assert h5lite.read(out, "data/H/row_indices").dtype == np.int64
    shape_attr, _ = h5lite.attr(out, "data/H", "shape")
    assert shape_attr.tolist() == [r, m_full]
    fds, shape = h5lite.attr(out, "data/reduce_kept_indices", "full_dense_size")
    assert shape == () and int(fds[0]) == m_full
    W = h5lite.read(out, "data/W")
    assert W.shape == (n, r)
    # fp64 oracle of both stages on the same inputs
    vals, idx = h5lite.read(pef, "data/fisher/values"), h5lite.read(pef, "data/fisher/indices")
    norms = h5lite.read(pef, "data/dense_fisher_norms")
    rp = orc.pef_rowptr(n, k)
    va = orc.normalize_rows(rp, vals.ravel(), norms)
    kept = h5lite.read(hpath, "data/reduce_kept_indices")
    rp2, ci2, va2 = orc.retain_columns(rp, idx.ravel(), va, m_full, kept)
    b = (h5lite.read(hpath, "data/H/row_indices"), h5lite.read(hpath, "data/H/column_indices"),
         h5lite.read(hpath, "data/H/values"))
    AH = orc.spsp_dense_f64((rp2, ci2, va2), m_full, b, r)
    HH = orc.spsp_dense_f64(b, m_full, b, r)
    W0 = np.array([[d.uniform_at(43190432042, 0, i, c, r) for c in range(r)] for i in range(n)], np.float32)
    W64, ref, tru = orc.fit_f64(AH, HH, float(np.sum(va2.astype(np.float64) ** 2)), W0, np.float32(1e-7), iters, 25)
    assert np.linalg.norm(W - W64) / np.linalg.norm(W64) < 1e-4
    logged = [float(s.split(":")[1].split("[")[0]) for s in steps]
    assert np.all(np.abs(np.array(logged) - ref) / ref < 1e-4)


@pytest.mark.gpu
def test_fit_row_split_check_is_kept(tmp_path):
    """A split with nnz >= INT32_MAX is fatal in the reference; with small inputs the check passes
    for any number of splits, including more splits than rows' worth of remainder."""
    pef = make_pef(tmp_path, n=7, m=3000, k=50, seed=2, sparse_H_output_path=str(tmp_path / "H.h5"), rank=4,
                   H_density=0.05)
    p = run("fit_coeffs_to_sparse_H", f"--output_path={tmp_path}/o.h5", f"--pef_path={pef}",
            f"--H_path={tmp_path}/H.h5", "--n_splits_sparse_matmul=1", "--n_row_splits_pefs=3", "--nmf_max_iter=2",
            "--DEV_n_cols=1000", check=True)
    assert "NOTE: Using flag intended only for development purposes." in p.stdout
    shape_attr, _ = h5lite.attr(f"{tmp_path}/o.h5", "data/H", "shape")
    assert shape_attr.tolist() == [4, 1000]


@pytest.mark.gpu
def test_sparsify_d_npeff_feeds_the_fit(tmp_path):
    """run_nmf_on_pefs -> sparsify_d_npeff -> fit_coeffs_to_sparse_H: the sparsifier's file has the
    sparse schema with unit-norm thresholded rows of H and rescaled W, and the fit accepts it."""
    n, m_full, k, r = 40, 30000, 500, 8
    pef = make_pef(tmp_path, n=n, m=m_full, k=k, seed=5)
    dense, sparse, fit = (str(tmp_path / f) for f in ("decomp.h5", "sparse.h5", "fit.h5"))
    run("run_nmf_on_pefs", f"--output_path={dense}", f"--per_example_fishers={pef}", f"--nmf_n_components={r}",
        "--nmf_max_iter=30", check=True)
    thr = 0.004
    p = run("sparsify_d_npeff", f"--decomposition_filepath={dense}", f"--output_filepath={sparse}",
            f"--H_threshold={thr}", check=True)
    W, H = h5lite.read(dense, "data/W"), h5lite.read(dense, "data/H")
    W2, vals, offs, cols = orc.sparsify_H(W, H, thr)
    assert f"Dense size: {H.size}" in p.stdout and f"Sparse NNZ: {len(vals)}" in p.stdout
    assert 0 < len(vals) < H.size
    assert np.array_equal(h5lite.read(sparse, "data/H/values"), vals)
    assert np.array_equal(h5lite.read(sparse, "data/H/column_indices"), cols)
    got_offs = h5lite.read(sparse, "data/H/row_indices")
    assert got_offs.dtype == np.int64 and np.array_equal(got_offs, offs)
    assert np.array_equal(h5lite.read(sparse, "data/W"), W2)
    assert np.array_equal(h5lite.read(sparse, "data/reduce_kept_indices"), h5lite.read(dense, "data/reduce_kept_indices"))
    shape_attr, _ = h5lite.attr(sparse, "data/H", "shape")
    assert shape_attr.tolist() == list(H.shape)
    fds, _ = h5lite.attr(sparse, "data/reduce_kept_indices", "full_dense_size")
    assert int(fds[0]) == m_full
    # missing threshold is fatal, as the script's assert
    q = run("sparsify_d_npeff", f"--decomposition_filepath={dense}", f"--output_filepath={sparse}.x")
    assert q.returncode != 0 and "Missing flag: H_threshold" in q.stdout
    # the other executable takes the file
    run("fit_coeffs_to_sparse_H", f"--output_path={fit}", f"--pef_path={pef}", f"--H_path={sparse}",
        "--n_splits_sparse_matmul=1", "--n_row_splits_pefs=1", "--nmf_max_iter=25", check=True)
    assert h5lite.read(fit, "data/W").shape == (n, r)


@pytest.mark.gpu
def test_run_nmf_on_pefs_at_a_realistic_size(tmp_path):
    """configs[1] downscaled (1,000 examples x 16,384 values of 11M parameters, a 130 MB file made by
    the device generator, rank 128, dense head and column panels in use): the executable's W, H and
    reduce_kept_indices equal, bit for bit, those of the same fit driven through the C ABI."""
    n, m_full, k, r, iters = 1000, 11_000_000, 16_384, 128, 10
    pef = make_pef(tmp_path, n=n, m=m_full, k=k, seed=19, on_device=1)
    assert os.path.getsize(pef) > 8 * n * k
    out = str(tmp_path / "decomp.h5")
    p = run("run_nmf_on_pefs", f"--output_path={out}", f"--per_example_fishers={pef}", f"--nmf_n_components={r}",
            f"--nmf_max_iter={iters}", check=True)
    lines = p.stdout.splitlines()
    assert "Using 32 bit indices." in lines and "Running NMF using 32 bit indices." in lines
    steps = [l for l in lines if l.startswith("step ")]
    assert [s.split(":")[0] for s in steps] == ["step 10"]
    vals, idx = h5lite.read(pef, "data/fisher/values"), h5lite.read(pef, "data/fisher/indices")
    norms = h5lite.read(pef, "data/dense_fisher_norms")
    A = d.Csr.from_pef(idx, vals, m_full)
    A.normalize_rows(norms)
    A.compact_columns(1)
    nmf = d.MuNmf(A, d.MuNmfParams(rank=r, max_iters=iters), consume_matrix=True)
    hist = nmf.run(log=lambda s: None)
    W, H, kept = h5lite.read(out, "data/W"), h5lite.read(out, "data/H"), h5lite.read(out, "data/reduce_kept_indices")
    assert W.shape == (n, r) and H.shape == (r, A.n_cols) and A.n_cols > 1_000_000
    assert np.array_equal(kept, A.kept_indices())
    assert np.array_equal(W, nmf.loadWToHostSync()) and np.array_equal(H, nmf.loadHToHostSync())
    logged = float(steps[-1].split(":")[1].split("[")[0])
    assert abs(logged - hist[-1][1]) / hist[-1][1] < 1e-5
    nmf.close()
    A.close()


@pytest.mark.gpu
@pytest.mark.timeout(1200)
def test_wide_index_branch_from_a_file_past_int32(tmp_path):
    """A PEF file with n_examples x n_fisher_values = 32,800 x 65,536 = 2,149,580,800 > INT32_MAX
    (17 GB): the executable reads it with 64-bit indices (pef_fisher_h5.h:57-90); pruning the
    parameters held by one example only brings the entries under INT32_MAX, so, by the
    reference's rule, the factorisation is run and saved with IndT = int64
    (run_nmf_on_pefs.cu:236-247, nmf_decomp_h5.h:58-75) without any override."""
    import shutil

    n, k, m_full, r = 32_800, 65_536, 110_000_000, 8
    need_disk, need_ram = 30e9, 80e9
    free_disk = shutil.disk_usage(str(tmp_path)).free
    if free_disk < need_disk:
        pytest.skip(f"needs {need_disk / 1e9:.0f} GB of scratch disk, {free_disk / 1e9:.0f} GB free")
    ram = os.sysconf("SC_PAGE_SIZE") * os.sysconf("SC_AVPHYS_PAGES")
    if ram < need_ram:
        pytest.skip(f"needs {need_ram / 1e9:.0f} GB of free host memory, {ram / 1e9:.0f} GB available")
    free, total = d.device_memory()
    if free < 100e9:
        pytest.skip("needs 100 GB of device memory")
    pef = make_pef(tmp_path, n=n, m=m_full, k=k, seed=23, on_device=1)
    assert os.path.getsize(pef) > 8 * n * k > 8 * 2**31
    out = str(tmp_path / "wide.h5")
    p = run("run_nmf_on_pefs", f"--output_path={out}", f"--per_example_fishers={pef}", f"--nmf_n_components={r}",
            "--nmf_max_iter=2", "--min_values_per_parameter=2", check=True)
    os.remove(pef)
    lines = p.stdout.splitlines()
    assert "Reading in PEFs using 64 bit indices." in lines
    assert "Running NMF using 64 bit indices." in lines
    kept = h5lite.read(out, "data/reduce_kept_indices")
    fds, shape = h5lite.attr(out, "data/reduce_kept_indices", "full_dense_size")
    assert kept.dtype == np.int64 and fds.dtype == np.int64 and shape == (1,) and int(fds[0]) == m_full
    assert np.all(np.diff(kept) > 0) and 0 <= kept[0] and kept[-1] < m_full
    W, H = h5lite.read(out, "data/W"), h5lite.read(out, "data/H")
    assert W.shape == (n, r) and H.shape == (r, len(kept))
    assert np.isfinite(W).all() and W.min() >= 0 and np.isfinite(H).all() and H.min() >= 0
