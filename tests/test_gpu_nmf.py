"""The two hot loops end to end through the C ABI vs the fp64 CPU oracle running the
reference's exact update sequence on the same seeded factors.

Bar (from the task statement): W, H and the logged loss within 1e-4 relative after 50
iterations.  W and H are compared norm-wise (||X - X64||_F / ||X64||_F): entries that MU drives
to ~0 make an element-wise relative error meaningless."""

import numpy as np
import pytest

import npeff_ref_amd as d
from conftest import random_csr
from oracle import oracle as orc

pytestmark = pytest.mark.gpu

REL = 1e-4


def _nrm(a, b):
    return np.linalg.norm(a.astype(np.float64) - b) / np.linalg.norm(b)


def _seeded_factors(seed, n, r, m):
    W0 = np.array([[d.uniform_at(seed, 0, i, c, r) for c in range(r)] for i in range(n)], dtype=np.float32)
    return W0


def _run_case(n, m_full, k, r, eps, iters, seed, zipf_s=1.1, log_every=10):
    A, norms = d.Csr.synth(n, m_full, k_fixed=k, zipf_s=zipf_s, seed=seed)
    A.normalize_rows(norms)
    A.compact_columns(1)
    rp, ci, va = A.download()
    m = A.n_cols
    nmf = d.MuNmf(A, d.MuNmfParams(rank=r, max_iters=iters, eps=eps, seed=seed, log_every=log_every))
    nmf.initialize()
    W0, H0 = nmf.loadWToHostSync(), nmf.loadHToHostSync()
    hist = nmf.run(log=lambda s: None)
    W, H = nmf.loadWToHostSync(), nmf.loadHToHostSync()
    W64, H64, losses64 = orc.nmf_f64(rp, ci, va, m, W0, H0, np.float32(eps), iters, log_every)
    return nmf, A, (W0, H0), (W, H), (W64, H64), hist, losses64


def test_config0_50_iterations_within_1e4():
    """BASELINE configs[0]: 512 x 1,048,576, 4096 nnz/row, Zipf 1.1, r = 16, eps 1e-12, 50 its."""
    nmf, A, (W0, H0), (W, H), (W64, H64), hist, losses64 = _run_case(
        512, 1 << 20, 4096, 16, 1e-12, 50, seed=20240607)
    assert W0.min() >= 0 and W0.max() < 1 and H0.min() >= 0 and H0.max() < 1
    assert W0[3, 5] == np.float32(d.uniform_at(20240607, 0, 3, 5, 16))
    assert H0[5, 77] == np.float32(d.uniform_at(20240607, 1, 5, 77, A.n_cols))
    assert _nrm(W, W64) < REL and _nrm(H, H64) < REL
    got = np.array([h[1] for h in hist])
    assert len(got) == 5 and np.all(np.abs(got - losses64) / losses64 < REL)
    assert np.all(np.diff(losses64) < 0)  # MU decreases the loss
    assert W.min() >= 0 and H.min() >= 0
    nmf.close()
    A.close()


@pytest.mark.parametrize("r,k,n,eps", [(128, 2048, 300, 1e-8), (256, 1500, 260, 1e-8), (100, 700, 150, 1e-12)])
def test_larger_ranks_50_iterations(r, k, n, eps):
    nmf, A, _, (W, H), (W64, H64), hist, losses64 = _run_case(n, 300000, k, r, eps, 50, seed=r)
    assert _nrm(W, W64) < REL and _nrm(H, H64) < REL
    got = np.array([h[1] for h in hist])
    assert np.all(np.abs(got - losses64) / losses64 < REL)
    nmf.close()
    A.close()


def test_loss_terms_against_oracle_and_explicit_residual():
    rng = np.random.default_rng(3)
    n, m, r = 40, 900, 16
    rp, ci, va = random_csr(rng, n, m, 300)
    A = d.Csr.from_host(rp, ci, va, m)
    nmf = d.MuNmf(A, d.MuNmfParams(rank=r, max_iters=0))
    W, H = rng.random((n, r)).astype(np.float32), rng.random((r, m)).astype(np.float32)
    nmf.set_factors(W, H)
    assert np.array_equal(nmf.loadWToHostSync(), W) and np.array_equal(nmf.loadHToHostSync(), H)
    sq, pos, neg = nmf.loss_terms()
    loss64, terms = orc.loss_f64(rp, ci, va, m, W, H)
    np.testing.assert_allclose([sq, pos, neg], terms, rtol=2e-6)
    np.testing.assert_allclose(nmf.computeUncachedLoss(), loss64, rtol=1e-5)
    nmf.close()
    A.close()


def test_run_is_reproducible_bit_for_bit():
    outs = []
    for _ in range(2):
        A, norms = d.Csr.synth(200, 100000, k_fixed=1000, seed=4)
        A.normalize_rows(norms)
        A.compact_columns(1)
        nmf = d.MuNmf(A, d.MuNmfParams(rank=64, max_iters=5, log_every=0))
        nmf.run(log=lambda s: None)
        outs.append((nmf.loadWToHostSync(), nmf.loadHToHostSync(), nmf.computeUncachedLoss()))
        nmf.close()
        A.close()
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])
    assert outs[0][2] == outs[1][2]


@pytest.mark.parametrize("rank", [64, 128, 256])
def test_loss_evaluations_do_not_change_the_run(rank):
    """The loss leaves A H^T behind for the next W update (and takes H^T H from the fused H update
    at rank 128; at rank 256 a W update that finds A H^T there does not start H^T H on the second
    stream): a run that evaluates the loss after every step and between the two updates ends
    on the same bits as one that never does, and the loss values agree with a fresh evaluation."""
    outs = []
    for with_loss in (False, True):
        A, norms = d.Csr.synth(200, 150000, k_fixed=1500, seed=9)
        A.normalize_rows(norms)
        A.compact_columns(1)
        nmf = d.MuNmf(A, d.MuNmfParams(rank=rank, max_iters=4, log_every=0))
        nmf.initialize()
        losses = []
        for _ in range(4):
            nmf.update_W()
            if with_loss:
                losses.append(nmf.computeUncachedLoss())
            nmf.update_H()
            if with_loss:
                losses.append(nmf.computeUncachedLoss())
                losses.append(nmf.computeUncachedLoss())  # twice: everything cached
        outs.append((nmf.loadWToHostSync(), nmf.loadHToHostSync(), nmf.computeUncachedLoss(), losses))
        nmf.close()
        A.close()
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])
    assert outs[0][2] == outs[1][2] == outs[1][3][-1] == outs[1][3][-2]


@pytest.mark.parametrize("rank,n", [(256, 1500), (64, 300)])
def test_gram_beside_the_sparse_product_gives_the_same_bits(rank, n, tune):
    """The gram_beside switch only moves H^T H of the W update to a second stream, beside A H^T: the
    same kernels on the same operands, so six iterations end on the same bits (rank 256 with a
    dense head, panels and swept pieces forced on; rank 64 without)."""
    outs = []
    for beside in (0, 1):
        tune("gram_beside", beside)
        tune("panels", 8)
        tune("sweep_bytes", 300 * 4 * min(rank, 256))
        tune("sweep_min", 0)
        A, norms = d.Csr.synth(n, 200000, k_fixed=1500, zipf_s=1.3, seed=21)
        A.normalize_rows(norms)
        A.compact_columns(1)
        nmf = d.MuNmf(A, d.MuNmfParams(rank=rank, max_iters=6, log_every=3))
        nmf.initialize()
        hist = nmf.run(log=lambda s: None)
        outs.append((nmf.loadWToHostSync(), nmf.loadHToHostSync(), [h[1] for h in hist]))
        nmf.close()
        A.close()
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])
    assert outs[0][2] == outs[1][2]


@pytest.mark.parametrize("fill", [1.0 / 16.0, 0.0])
def test_second_context_on_a_consumed_matrix(fill, tune):
    """A matrix whose arrays a consuming create has released still serves a later context of the
    same rank (with a dense head: only head and tail are left; without: only the transposed and
    regrouped copies): same ||A||^2, same factors, same loss, bit for bit."""
    tune("dense_fill", fill)
    A, norms = d.Csr.synth(1500, 200000, k_fixed=1500, zipf_s=1.3, seed=33)
    A.normalize_rows(norms)
    A.compact_columns(1)
    outs = []
    for _ in range(2):
        nmf = d.MuNmf(A, d.MuNmfParams(rank=128, max_iters=3, log_every=0), consume_matrix=True)
        assert (A.head_info()[0] > 0) == (fill > 0)
        nmf.initialize()
        nmf.step(3)
        outs.append((nmf.loss_terms(), nmf.loadWToHostSync(), nmf.loadHToHostSync()))
        nmf.close()
    assert outs[0][0] == outs[1][0]
    assert np.array_equal(outs[0][1], outs[1][1]) and np.array_equal(outs[0][2], outs[1][2])
    A.close()


def test_more_rows_than_columns_is_refused():
    A = d.Csr.from_host([0, 1, 2, 3], [0, 1, 0], [1.0, 1.0, 1.0], 2)
    with pytest.raises(d.DnpeffError, match="more rows than columns"):
        d.MuNmf(A, d.MuNmfParams(rank=2, max_iters=1))
    A.close()


def test_profiling_counts_launches():
    A, norms = d.Csr.synth(64, 50000, k_fixed=500, seed=1)
    A.normalize_rows(norms)
    A.compact_columns(1)
    nmf = d.MuNmf(A, d.MuNmfParams(rank=32, max_iters=3, log_every=0))
    nmf.initialize()
    nmf.set_profiling(True)
    nmf.step(3)
    t = nmf.timings(reset=True)
    assert all(t[k][1] == 3 and t[k][0] > 0 for k in d.KERNEL_CLASSES)
    assert all(v == (0.0, 0) for v in nmf.timings().values())
    nmf.close()
    A.close()


def test_fit_path_first_stage_and_loop():
    """fit_coeffs_to_sparse_H: stage-1 products and the W loop, incl. the logged (stale-WHH) loss."""
    rng = np.random.default_rng(12)
    n, m, r = 300, 40000, 64
    ar, ac, av, norms = d.synth_pef_host(n, m, k_fixed=1200, seed=6)
    av = orc.normalize_rows(ar, av, norms)
    b = random_csr(rng, r, m, 900, sort_cols=True)
    A, H = d.Csr.from_host(ar, ac, av, m), d.Csr.from_host(*b, m)
    iters, eps = 50, 1e-7
    lrn = d.Learner(A, H, d.LearnerParams(max_iters=iters, eps=eps, log_every_n_steps=25))
    AH, HH, sq = lrn.products()
    AH64 = orc.spsp_dense_f64((ar, ac, av), m, b, r)
    HH64 = orc.spsp_dense_f64(b, m, b, r)
    assert np.abs(AH - AH64).max() / np.abs(AH64).max() < 2e-5
    assert np.abs(HH - HH64).max() / np.abs(HH64).max() < 2e-5
    np.testing.assert_allclose(sq, np.sum(av.astype(np.float64) ** 2), rtol=1e-12)
    lrn.initialize()
    W0 = lrn.GetOnHost_W()
    assert W0[2, 3] == np.float32(d.uniform_at(lrn.params.seed, 0, 2, 3, r))
    hist = lrn.Run(log=lambda s: None)
    W = lrn.GetOnHost_W()
    W64, ref64, true64 = orc.fit_f64(AH64, HH64, sq, W0, np.float32(eps), iters, 25)
    assert _nrm(W, W64) < REL
    assert np.all(np.abs(np.array([h[1] for h in hist]) - ref64) / ref64 < REL)
    assert np.all(np.abs(np.array([h[2] for h in hist]) - true64) / true64 < REL)
    lrn.close()
    A.close()
    H.close()


@pytest.mark.parametrize("n", [2000 + 80, 1024])
def test_fit_steps_in_one_call_and_one_by_one_rank_256(n):
    """The W loop of the fixed-H learner at rank 256 (matrix-core update kernel; with n = 2080 the
    last 32 rows go through another kernel, on the second stream): seven steps in one call, seven
    calls of one step and a 3 + 4 split give the same W bit for bit, and the oracle's within the
    bar."""
    rng = np.random.default_rng(n)
    m, r, eps = 30000, 256, 1e-7
    ar, ac, av, norms = d.synth_pef_host(n, m, k_fixed=600, seed=8)
    av = orc.normalize_rows(ar, av, norms)
    b = random_csr(rng, r, m, 700, sort_cols=True)
    A, H = d.Csr.from_host(ar, ac, av, m), d.Csr.from_host(*b, m)
    lrn = d.Learner(A, H, d.LearnerParams(max_iters=7, eps=eps, log_every_n_steps=0))
    AH, HH, sq = lrn.products()
    lrn.initialize()
    W0 = lrn.GetOnHost_W()
    lrn.step(7)
    W7 = lrn.GetOnHost_W()
    lrn.set_W(W0)
    for _ in range(7):
        lrn.step(1)
    assert np.array_equal(lrn.GetOnHost_W(), W7)
    lrn.set_W(W0)
    lrn.step(3)
    lrn.losses()
    lrn.step(4)
    assert np.array_equal(lrn.GetOnHost_W(), W7)
    W64, _, _ = orc.fit_f64(AH.astype(np.float64), HH.astype(np.float64), sq, W0, np.float32(eps), 7, 0)
    assert _nrm(W7, W64) < REL
    lrn.close()
    A.close()
    H.close()


def test_dense_head_run_matches_oracle_and_unsplit_run(tune):
    """n >= 1024 rows and r >= 64: dnpeff_nmf_create moves the columns most rows hold into the
    dense block by itself; the run stays within the bar of the fp64 oracle and close to the run
    with the split switched off."""
    n, m_full, k, r, eps, iters, seed = 1100, 60000, 3000, 64, 1e-8, 50, 77
    nmf, A, (W0, H0), (W, H), (W64, H64), hist, losses64 = _run_case(n, m_full, k, r, eps, iters, seed)
    nd, z_sparse = A.head_info()
    assert nd > 100 and z_sparse < A.nnz
    assert _nrm(W, W64) < REL and _nrm(H, H64) < REL
    got = np.array([h[1] for h in hist])
    assert np.all(np.abs(got - losses64) / losses64 < REL)
    nmf.close()
    A.close()
    tune("dense_fill", 0)
    nmf2, A2, _, (W2, H2), _, hist2, _ = _run_case(n, m_full, k, r, eps, iters, seed)
    assert A2.head_info()[0] == 0
    assert _nrm(W2, W64) < REL and _nrm(H2, H64) < REL
    nmf2.close()
    A2.close()


def test_column_panel_run_matches_oracle(tune):
    tune("panels", 12)
    nmf, A, _, (W, H), (W64, H64), hist, losses64 = _run_case(300, 40000, 2048, 128, 1e-8, 50, seed=5)
    assert _nrm(W, W64) < REL and _nrm(H, H64) < REL
    got = np.array([h[1] for h in hist])
    assert np.all(np.abs(got - losses64) / losses64 < REL)
    nmf.close()
    A.close()


@pytest.mark.parametrize("r,waves,piece_cols", [(128, 14, 40), (64, 3, 2000)])
def test_swept_piece_run_matches_oracle(r, waves, piece_cols, tune):
    """Column panels cut into small pieces that the XCDs sweep (forced on, any density; at 40
    columns per piece all 6 panels are cut, at 2000 the 3 narrow ones stay whole and both kernels
    share the product): 50 iterations stay within the bar, and a second run gives the same bits."""
    tune("panels", 6)
    tune("sweep_bytes", piece_cols * 4 * r)
    tune("sweep_min", 0)
    tune("sweep_waves", waves)
    nmf, A, _, (W, H), (W64, H64), hist, losses64 = _run_case(300, 40000, 2048, r, 1e-8, 50, seed=9)
    assert _nrm(W, W64) < REL and _nrm(H, H64) < REL
    got = np.array([h[1] for h in hist])
    assert np.all(np.abs(got - losses64) / losses64 < REL)
    nmf.close()
    A.close()
    nmf2, A2, _, (W2, H2), _, _, _ = _run_case(300, 40000, 2048, r, 1e-8, 50, seed=9)
    assert np.array_equal(W2, W) and np.array_equal(H2, H)
    nmf2.close()
    A2.close()


def test_ragged_rows_rank_512(tune):
    """Row lengths drawn log-uniformly over two decades (the ragged-row case), r = 512: the tiled
    X G kernel, the tile-pair Gram and the grouped A^T W at their widest, with column panels
    forced on so that short rows leave empty segments."""
    tune("panels", 24)
    n, m_full, r, eps, iters, seed = 260, 60000, 512, 1e-8, 50, 31
    A, norms = d.Csr.synth(n, m_full, k_fixed=0, k_min=16, k_max=4096, zipf_s=1.1, seed=seed)
    A.normalize_rows(norms)
    A.compact_columns(1)
    rp, ci, va = A.download()
    lens = np.diff(rp)
    assert lens.min() < 64 and lens.max() > 2000
    m = A.n_cols
    nmf = d.MuNmf(A, d.MuNmfParams(rank=r, max_iters=iters, eps=eps, seed=seed, log_every=10))
    nmf.initialize()
    W0, H0 = nmf.loadWToHostSync(), nmf.loadHToHostSync()
    hist = nmf.run(log=lambda s: None)
    W64, H64, losses64 = orc.nmf_f64(rp, ci, va, m, W0, H0, np.float32(eps), iters, 10)
    assert _nrm(nmf.loadWToHostSync(), W64) < REL and _nrm(nmf.loadHToHostSync(), H64) < REL
    got = np.array([h[1] for h in hist])
    assert np.all(np.abs(got - losses64) / losses64 < REL)
    nmf.close()
    A.close()


def test_heavier_skew_rank_256_with_dense_head():
    """Zipf 1.3 columns, r = 256, enough rows for the dense head: every r > 128 kernel plus the
    head products in one run."""
    nmf, A, _, (W, H), (W64, H64), hist, losses64 = _run_case(1030, 200000, 1500, 256, 1e-8, 50, seed=13, zipf_s=1.3)
    assert A.head_info()[0] > 50
    assert _nrm(W, W64) < REL and _nrm(H, H64) < REL
    got = np.array([h[1] for h in hist])
    assert np.all(np.abs(got - losses64) / losses64 < REL)
    nmf.close()
    A.close()


def test_fit_after_nmf_on_the_same_matrix():
    """A matrix that an NMF has split (dense head, tail) is handed to the fit path afterwards:
    the sparse-sparse product undoes the split and gives the same A H^T as on a fresh matrix."""
    n, m_full, k, r = 1100, 60000, 3000, 64
    A, norms = d.Csr.synth(n, m_full, k_fixed=k, zipf_s=1.1, seed=77)
    A.normalize_rows(norms)
    A.compact_columns(1)
    rp, ci, va = A.download()
    m = A.n_cols
    nmf = d.MuNmf(A, d.MuNmfParams(rank=r, max_iters=2, eps=1e-8, seed=1))
    nmf.initialize()
    nmf.run(log=lambda s: None)
    assert A.head_info()[0] > 0
    nmf.close()
    rng = np.random.default_rng(0)
    hr, hc, hv = random_csr(rng, 8, m, 300, sort_cols=True)
    B = d.Csr.from_host(hr, hc, hv, m)
    out = d.DeviceArray((n, 8))
    d.op_spsp_dense(A, B, out)
    assert A.head_info()[0] == 0
    want = orc.spsp_dense_f64((rp, ci, va), m, (hr, hc, hv), 8)
    got = out.numpy()
    assert np.abs(got - want).max() / np.abs(want).max() < 2e-5
    A.close()
    B.close()


def test_fused_gram_in_H_update_matches_the_two_pass_path(tune):
    """r = 128: the H update accumulates H^T H of its own output, the W update uses it; rows past
    the last 64-row tile go through the plain kernels and are added.  Same bar against the oracle
    with the fusion switched off, and the two runs agree far inside it."""
    args = (300, 40000, 2048, 128, 1e-8, 50)
    nmf, A, _, (W, H), (W64, H64), hist, losses64 = _run_case(*args, seed=5)
    assert A.n_cols % 64 != 0  # exercises the tail rows
    assert _nrm(W, W64) < REL and _nrm(H, H64) < REL
    nmf.close()
    A.close()
    tune("fused_gram", 0)
    nmf2, A2, _, (W2, H2), _, hist2, _ = _run_case(*args, seed=5)
    assert _nrm(W2, W64) < REL and _nrm(H2, H64) < REL
    assert _nrm(W, W2.astype(np.float64)) < 1e-5 and _nrm(H, H2.astype(np.float64)) < 1e-5
    assert abs(hist[-1][1] - hist2[-1][1]) / hist2[-1][1] < 1e-6
    nmf2.close()
    A2.close()


def _steps(A, r, seed, steps, consume=False):
    nmf = d.MuNmf(A, d.MuNmfParams(rank=r, max_iters=0, eps=1e-8, seed=seed), consume_matrix=consume)
    nmf.initialize()
    nmf.step(steps)
    d.sync()
    return nmf


@pytest.mark.parametrize("r,n,k,tile_mb", [(256, 1100, 3000, 0.9), (64, 300, 2000, 0.05), (512, 300, 2500, 1.5)])
def test_tiled_H_update_with_the_next_product_beside_it(r, n, k, tile_mb, tune):
    """`h_overlap`: A^T W of tile q + 1 on the library stream beside the update of tile q on a
    second stream, through two tile buffers.  Same kernels on the same operands in an order that
    the events between the streams fix: the same bits as the tiled update on one stream, after
    odd and even numbers of steps, and the calls that follow (loss, factors to the host) see
    the finished update."""
    tune("fused_gram", 0)
    tune("tiled_h", 1)
    tune("h_tile_mb", tile_mb)
    seed = 300 + r
    A, norms = d.Csr.synth(n, 60000, k_fixed=k, zipf_s=1.2, seed=seed)
    A.normalize_rows(norms)
    A.compact_columns(1)
    ref = _steps(A, r, seed, 3)
    tiled, tile_cols = ref.info()
    assert tiled and 3 * tile_cols < A.n_cols
    W3, H3, loss3 = ref.loadWToHostSync(), ref.loadHToHostSync(), ref.computeUncachedLoss()
    ref.step(2)
    W5, H5, loss5 = ref.loadWToHostSync(), ref.loadHToHostSync(), ref.computeUncachedLoss()
    ref.close()
    tune("h_overlap", 1)
    ovl = _steps(A, r, seed, 3)
    assert ovl.info() == (tiled, tile_cols)
    assert np.array_equal(ovl.loadWToHostSync(), W3) and np.array_equal(ovl.loadHToHostSync(), H3)
    assert ovl.computeUncachedLoss() == loss3
    ovl.step(2)
    assert np.array_equal(ovl.loadWToHostSync(), W5) and np.array_equal(ovl.loadHToHostSync(), H5)
    assert ovl.computeUncachedLoss() == loss5
    ovl.close()


@pytest.mark.parametrize("r,n,k,tile_mb", [(256, 1100, 3000, 0.9), (128, 1100, 3000, 0.4), (64, 300, 2000, 0.05),
                                           (48, 130, 800, 0.03)])
def test_tiled_H_update_gives_the_same_bits(r, n, k, tile_mb, tune):
    """The H update on column tiles (A^T W of a tile, then the tile's update written one tile
    away inside the buffer of H; forced here, used by itself when a second [m, r] array does not
    fit) against the full-size update: same factors bit for bit after an odd and an even number
    of steps (H sits at either end of its buffer), dense head and long columns included; the
    consuming create frees the caller's arrays and changes nothing else."""
    tune("fused_gram", 0)  # (at rank 128 the fused update sums in another order)
    seed = 100 + r
    A, norms = d.Csr.synth(n, 60000, k_fixed=k, zipf_s=1.2, seed=seed)
    A.normalize_rows(norms)
    A.compact_columns(1)
    ref = _steps(A, r, seed, 3)
    assert ref.info() == (False, 0)
    W3, H3 = ref.loadWToHostSync(), ref.loadHToHostSync()
    ref.step(1)
    W4, H4, loss4 = ref.loadWToHostSync(), ref.loadHToHostSync(), ref.computeUncachedLoss()
    ref.close()
    tune("tiled_h", 1)
    tune("h_tile_mb", tile_mb)
    til = _steps(A, r, seed, 3, consume=True)
    tiled, tile_cols = til.info()
    assert tiled and tile_cols % 128 == 0 and 2 * tile_cols < A.n_cols
    if r >= 64 and n >= 1024:
        assert A.head_info()[0] > 0
    assert np.array_equal(til.loadWToHostSync(), W3) and np.array_equal(til.loadHToHostSync(), H3)
    til.step(1)
    assert np.array_equal(til.loadWToHostSync(), W4) and np.array_equal(til.loadHToHostSync(), H4)
    assert til.computeUncachedLoss() == loss4
    # factors loaded from the host go through the same tiles
    til.set_factors(W3, H3)
    assert np.array_equal(til.loadHToHostSync(), H3)
    til.step(1)
    assert np.array_equal(til.loadHToHostSync(), H4)
    # the consumed matrix still knows its shape and column map, and refuses to be read back
    assert len(A.kept_indices()) == A.n_cols
    if A.head_info()[0] > 0:  # (without head or panels the products read the caller's arrays)
        with pytest.raises(d.DnpeffError, match="released"):
            A.download()
        with pytest.raises(d.DnpeffError, match="released"):
            A.compact_columns(1)
    else:
        assert len(A.download()[1]) == A.nnz
    til.close()
    A.close()


def test_two_contexts_of_different_rank_on_one_matrix():
    """A second context (or a single-kernel call) at another rank plans the matrix's work lists
    and partial-sum buffers again; the first context must notice and still give its own results."""
    seed = 12
    A, norms = d.Csr.synth(600, 200000, k_fixed=4000, zipf_s=1.1, seed=seed)
    A.normalize_rows(norms)
    A.compact_columns(1)
    alone = _steps(A, 128, seed, 2)
    W_ref, H_ref = alone.loadWToHostSync(), alone.loadHToHostSync()
    alone.close()
    big = _steps(A, 128, seed, 1)
    small = _steps(A, 32, seed, 1)  # plans the matrix for rank 32: smaller partial sums
    big.step(1)                     # rank 128 again
    small.step(1)
    assert np.array_equal(big.loadWToHostSync(), W_ref) and np.array_equal(big.loadHToHostSync(), H_ref)
    small_alone = _steps(A, 32, seed, 2)
    assert np.array_equal(small.loadWToHostSync(), small_alone.loadWToHostSync())
    small_alone.close()
    big.close()
    small.close()
    A.close()
