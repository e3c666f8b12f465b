// Handles of the two hot loops behind the C ABI: the dense-factor MU NMF of
// run_nmf_on_pefs and the W-only learner of fit_coeffs_to_sparse_H.
#include <chrono>
#include "dnpeff_internal.hpp"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <utility>
#include <vector>

using namespace dn;

// ---------------------------------------------------------------------------
// Per-kernel timing with HIP events on the library stream
// ---------------------------------------------------------------------------
// A mark is one event on the stream; the time from a mark to the next one belongs to the class
// that the mark opens (none for a mark that only closes).  Classes that follow one another
// without anything between them share the mark between them (next()).
struct Mark {
  hipEvent_t ev = nullptr;
  int cls = -1;
  bool counts = true;  // the segment is a launch of its class (not the continuation of one)
};

struct Profiler {
  bool enabled = false;
  std::vector<Mark> pool;        // every event ever created
  size_t used = 0;               // marks in flight since the last collect
  double ms_sum[DNPEFF_K_COUNT] = {0};
  int64_t launches[DNPEFF_K_COUNT] = {0};

  int mark(int cls, bool counts = true) {
    if (used == pool.size()) {
      Mark m;
      DN_HIP(hipEventCreate(&m.ev));
      pool.push_back(m);
    }
    pool[used].cls = cls;
    pool[used].counts = counts;
    DN_HIP(hipEventRecord(pool[used].ev, stream()));
    used++;
    return 0;
  }
  int begin(int cls) { return enabled ? mark(cls) : 0; }
  // goes on with a class that was interrupted (its time, not another launch)
  int resume(int cls) { return enabled ? mark(cls, false) : 0; }
  // closes the open class and opens cls with the same event
  int next(int cls) { return enabled ? mark(cls) : 0; }
  int end() {
    if (!enabled) return 0;
    DN_TRY(mark(-1));
    if (used >= 32768) return collect();
    return 0;
  }
  int collect() {
    if (used == 0) return 0;
    DN_HIP(hipStreamSynchronize(stream()));
    for (size_t i = 0; i + 1 < used; i++) {
      if (pool[i].cls < 0) continue;
      float ms = 0.0f;
      DN_HIP(hipEventElapsedTime(&ms, pool[i].ev, pool[i + 1].ev));
      if (ms < 0.0f) ms = 0.0f;  // (marks on two streams: the later mark's work ended first)
      ms_sum[pool[i].cls] += (double)ms;
      if (pool[i].counts) launches[pool[i].cls] += 1;
    }
    used = 0;
    return 0;
  }
  void reset() {
    for (int i = 0; i < DNPEFF_K_COUNT; i++) {
      ms_sum[i] = 0.0;
      launches[i] = 0;
    }
  }
  ~Profiler() {
    for (auto& m : pool)
      if (m.ev) (void)hipEventDestroy(m.ev);
  }
};

// ---------------------------------------------------------------------------
// Dense-factor MU NMF
// ---------------------------------------------------------------------------
struct dnpeff_nmf {
  dnpeff_csr* A = nullptr;
  int r = 0;
  float eps = 0.0f;
  uint64_t seed = 0;
  int64_t n = 0, m = 0;
  float* W = nullptr;        // [n, r]
  float* W2 = nullptr;       // [n, r] output buffer of the W update
  float* Nw = nullptr;       // [n, r] A H^T
  float* H = nullptr;        // [m, r] (points into Hbuf)
  float* S = nullptr;        // [m, r] A^T W, then the updated H; tiled: [tile_cols, r], A^T W of a tile
  float* S2 = nullptr;       // tiled, h_overlap: a second tile buffer
  float* Hbuf = nullptr;     // allocation that holds H; tiled: [m + tile_cols, r]
  // Tiled H update (when a second [m, r] array does not fit): A^T W is formed for tile_cols
  // columns at a time and the updated tile is written one tile below (or above) the place of the
  // old one inside Hbuf, so the update needs no full-size output: H alternates between
  // Hbuf and Hbuf + tile_cols r.
  bool tiled = false;
  int64_t tile_cols = 0;
  float* G = nullptr;        // [r, r]
  float* G2 = nullptr;       // [r, r]
  float* gram_ws = nullptr;  // slice partials of the Gram kernel
  double* dot_ws = nullptr;  // DOT_BLOCKS partials + 2 results
  float* GH = nullptr;       // [r, r] H^T H from the fused H update (valid while gh_valid)
  float* gpart = nullptr;    // its partial sums
  bool gh_valid = false;
  bool nw_valid = false;     // Nw holds A H^T of the current H (left there by the loss)
  double sq_norm_A = 0.0;
  Profiler prof;
};

DN_API int dnpeff_nmf_destroy(dnpeff_nmf* nmf) {
  if (!nmf) return 0;
  (void)hipStreamSynchronize(stream());
  dfree(nmf->W); dfree(nmf->W2); dfree(nmf->Nw); dfree(nmf->Hbuf); dfree(nmf->S); dfree(nmf->S2);
  dfree(nmf->G); dfree(nmf->G2); dfree(nmf->gram_ws); dfree(nmf->dot_ws);
  dfree(nmf->GH); dfree(nmf->gpart);
  delete nmf;
  return 0;
}

// The H update also produces H^T H (one pass over H instead of two) when the rank is 128 and
// the factor is large enough for the pass to matter (fused_gram switch: 0 = off).
static bool fused_update(const dnpeff_nmf* h) {
  if (tuning().fused_gram == 0.0 || h->tiled) return false;
  return h->r == 128 && h->m >= 4096;
}

// Columns of a tile of the tiled H update: h_tile_mb MiB of the factor, a multiple of 128.
static int64_t tile_cols_for(int64_t m, int rank) {
  double mb = tuning().h_tile_mb;
  if (mb < 0.001) mb = 0.001;
  int64_t t = (int64_t)(mb * 1024.0 * 1024.0 / (4.0 * rank)) / 128 * 128;
  if (t < 128) t = 128;
  const int64_t m_pad = ceil_div(m, 128) * 128;
  return t < m_pad ? t : m_pad;
}

// Bytes of device memory that the handle allocates besides the structures of the matrix.
static double factor_bytes(int64_t n, int64_t m, int rank, bool tiled) {
  const double nr = 4.0 * (double)n * rank, mr = 4.0 * (double)m * rank;
  double ws = (double)gram_workspace_floats(m, rank), ws_n = (double)gram_workspace_floats(n, rank);
  if (ws_n > ws) ws = ws_n;
  const double tile = 4.0 * (double)tile_cols_for(m, rank) * rank;
  return 3.0 * nr + (tiled ? mr + 2.0 * tile : 2.0 * mr) + 4.0 * ws + 3.0 * 4.0 * rank * rank +
         4.0 * (double)xg_mu_gram_workspace_floats(m);
}

// What the products' own buffers take besides the two sparse copies (16 bytes per entry of the
// sparse part), the dense blocks and the head's workspace, which the choice of the head prices
// per candidate: upper bounds from the same rules that size the allocations.
struct plan_table {
  double factors = 0.0;   // W, its double buffer, A H^T, H (+ tile), A^T W (or its tile), Grams, workspaces
  double partials = 0.0;  // partial sums of A H^T: per 2048-entry chunk, or per (row, plain panel / XCD)
  double segments = 0.0;  // offsets of the (row, panel) segments
  double offsets = 0.0;   // column offsets, long-column list, row offsets and chunk counts
  double reserve = 0.0;   // left free (1/64 of the device, at least 1 GiB): allocation granularity, code objects, the runtime's own
  double total() const { return factors + partials + segments + offsets + reserve; }
};

static plan_table plan_overheads(int64_t n, int64_t m, int64_t nnz_sparse, int rank, bool tiled, bool sweeps,
                                 double total_bytes) {
  plan_table t;
  t.factors = factor_bytes(n, m, rank, tiled);
  const int64_t P = coarse_panels_for(n, m, rank, sweeps);
  const double by_chunks = 4.0 * rank * ((double)nnz_sparse / (double)SPMM_N_CHUNK + (double)n);
  const double by_panels = P > 0 ? 4.0 * rank * (double)n * (double)(P + SWEEP_XCDS) : 0.0;
  t.partials = by_chunks > by_panels ? by_chunks : by_panels;
  // (a coarse panel may be cut into swept pieces: up to max_panels() panels and pieces in all)
  t.segments = P > 0 ? 8.0 * (double)n * (double)((sweeps ? max_panels() : P) + 1) : 0.0;
  const double n_long = std::min((double)m, (double)nnz_sparse / (double)(SPMM_T_LONG + 1));
  t.offsets = 8.0 * (double)(m + 1) + 4.0 * n_long + 2.0 * 8.0 * (double)(n + 1) + 2.0 * 8.0 * 64.0;
  t.reserve = std::max(1073741824.0, total_bytes / 64.0);
  return t;
}

// For tests and capacity planning without a GPU: the table above and, for a head of n_dense columns,
// its blocks and workspace.  out[0..7] = factors, partials, segments, offsets, reserve, sparse
// copies, head blocks, head workspace (bytes).
DN_API int dnpeff_plan_estimate(int64_t n_rows, int64_t n_cols, int64_t nnz_sparse, int64_t n_dense, int rank,
                                int tiled, int sweeps, int64_t total_bytes, double* out) {
  clear_error();
  DN_CHECK(out != nullptr, "out is NULL");
  DN_CHECK(n_rows >= 0 && n_cols >= 0 && nnz_sparse >= 0 && n_dense >= 0 && n_dense <= n_cols,
           "negative size");
  DN_CHECK(rank >= 1 && rank <= 1024, "rank %d outside [1, 1024]", rank);
  const plan_table t = plan_overheads(n_rows, n_cols, nnz_sparse, rank, tiled != 0, sweeps != 0, (double)total_bytes);
  out[0] = t.factors; out[1] = t.partials; out[2] = t.segments; out[3] = t.offsets; out[4] = t.reserve;
  out[5] = 16.0 * (double)nnz_sparse;
  out[6] = n_dense ? 4.0 * head_blocks_for_rank(rank) * (double)(ceil_div(n_rows, 128) * 128) *
                         (double)(ceil_div(n_dense, 128) * 128)
                   : 0.0;
  out[7] = 4.0 * (double)head_workspace_floats(n_rows, n_dense, rank);
  return 0;
}

// Splits off the dense head when the products can use it: rank a multiple of 4 and at least 64
// (below that a column of the dense block costs more than its entries do as gathers), enough
// rows for the fill fraction to mean something.  A column goes to the head when at least 1/16 of
// the rows hold it (dense_fill switch; 0 = never split); the fraction is raised until the dense
// blocks and both sparse copies of the rest fit the memory left beside the factors.  *tiled
// receives whether the H update must run on column tiles for everything to fit.
static int plan_matrix(dnpeff_csr* A, int rank, bool consume, bool* tiled) {
  const tuning_t& tn = tuning();
  size_t free_b = 0, total_b = 0;
  DN_HIP(hipMemGetInfo(&free_b, &total_b));
  const dnpeff_csr* S0 = sparse_part(A);
  // memory that the matrix structures may take: what is free now, plus what a consuming create
  // releases, plus what the structures hold already
  double avail = (double)free_b;
  if (consume && A->colind && A->vals) avail += 8.0 * (double)A->nnz;
  if (A->tail) {
    avail += (A->head.rm ? 8.0 : 4.0) * (double)A->head.n_pad * (double)A->head.n_d_pad;
    if (S0->colind) avail += 8.0 * (double)S0->nnz;
  }
  if (S0->colptr) avail += 8.0 * (double)S0->nnz;
  if (S0->pcol || S0->nl.pairs) avail += 8.0 * (double)S0->nnz;
  const bool sweeps = sweeps_for_rank(rank);
  const plan_table t_full = plan_overheads(A->n_rows, A->n_cols, A->nnz, rank, false, sweeps, (double)total_b);
  const plan_table t_tiled = plan_overheads(A->n_rows, A->n_cols, A->nnz, rank, true, sweeps, (double)total_b);
  const double budget_full = avail - t_full.total();
  const double budget_tiled = avail - t_tiled.total();
  const bool can_split = rank % 4 == 0 && rank >= 64 && A->n_rows >= 1024;
  double fill = tn.dense_fill;
  if (fill > 1.0) fill = 0.0;
  *tiled = tn.tiled_h > 0.0;
  if (A->tail) {
    if (rank % 4 == 0) {  // split by the caller (or an earlier handle): keep it
      const double foot = 4.0 * head_blocks_for_rank(rank) * (double)A->head.n_pad * (double)A->head.n_d_pad +
                          16.0 * (double)S0->nnz + 4.0 * (double)head_workspace_floats(A->n_rows, A->head.n_d, rank);
      if (tn.tiled_h < 0.0) *tiled = foot > budget_full;
      return 0;
    }
    DN_TRY(dnpeff_csr_split_dense_head(A, 0.0, nullptr));
    fill = 0.0;
  }
  if (!can_split) fill = 0.0;
  if (!has_row_major(A)) {  // consumed by an earlier handle without a head: nothing to choose
    if (tn.tiled_h < 0.0) *tiled = 16.0 * (double)A->nnz > budget_full;
    return 0;
  }
  head_choice c;
  const int n_blocks = head_blocks_for_rank(rank);
  DN_TRY(choose_dense_head(A, fill, *tiled ? budget_tiled : budget_full, n_blocks, rank, &c));
  if (!c.fits && tn.tiled_h < 0.0 && !*tiled) {
    *tiled = true;
    DN_TRY(choose_dense_head(A, fill, budget_tiled, n_blocks, rank, &c));
  }
  if (tn.verbose != 0.0) {
    const plan_table& t = *tiled ? t_tiled : t_full;
    fprintf(stderr,
            "dnpeff: plan for rank %d: %.1f GB free, budget for the matrix %.1f GB (%s H update); dense "
            "head of %lld columns (>= %lld entries), footprint %.1f GB%s\n"
            "dnpeff: plan bytes: factors %.2f GB, partial sums %.2f GB, segment offsets %.2f GB, column "
            "offsets %.2f GB, reserve %.2f GB\n",
            rank, (double)free_b / 1e9, (*tiled ? budget_tiled : budget_full) / 1e9,
            *tiled ? "tiled" : "full-size", (long long)c.n_d, (long long)c.thr, c.footprint / 1e9,
            c.fits ? "" : " (over budget)", t.factors / 1e9, t.partials / 1e9, t.segments / 1e9,
            t.offsets / 1e9, t.reserve / 1e9);
  }
  if (c.thr == 0) return 0;  // no head (there is none to undo either)
  return split_dense_head_at(A, c.thr, nullptr);
}

static int nmf_create_impl(dnpeff_csr* A, int rank, float eps, int64_t seed, unsigned flags,
                           dnpeff_nmf** out) {
  clear_error();
  DN_CHECK(out != nullptr, "out is NULL");
  *out = nullptr;
  DN_CHECK(A != nullptr, "matrix is NULL");
  DN_CHECK(rank >= 1 && rank <= 1024, "rank %d outside [1, 1024]", rank);
  DN_CHECK((flags & ~(unsigned)DNPEFF_NMF_CONSUME_MATRIX) == 0, "unknown flags 0x%x", flags);
  // multi_mu_dense_factors_nmf1.h:95-99
  DN_CHECK(A->n_rows <= A->n_cols, "Error: Not handling matrices with more rows than columns yet.");
  const bool consume = (flags & DNPEFF_NMF_CONSUME_MATRIX) != 0;
  // with verbose set: seconds of each phase of the set-up (the stream is drained at every mark)
  const bool timed = tuning().verbose != 0.0;
  auto t_last = std::chrono::steady_clock::now();
  auto mark = [&](const char* what) {
    if (!timed) return;
    (void)hipStreamSynchronize(stream());
    const auto t = std::chrono::steady_clock::now();
    fprintf(stderr, "dnpeff: set-up: %-44s %7.3f s\n", what, std::chrono::duration<double>(t - t_last).count());
    t_last = t;
  };
  double sq_norm = 0.0;
  DN_TRY(dnpeff_csr_sq_norm(A, &sq_norm));
  mark("||A||^2");
  bool tiled = false;
  DN_TRY(plan_matrix(A, rank, consume, &tiled));
  mark("memory plan, dense head and sparse tail");
  if (consume && A->tail) {  // the tail and the head hold everything the products read
    DN_HIP(hipStreamSynchronize(stream()));
    dfree(A->colind); A->colind = nullptr;
    dfree(A->vals); A->vals = nullptr;
  }
  DN_TRY(csr_ensure_products(A, rank));
  mark("transposed copy, panels, pieces, work lists");
  if (consume) DN_TRY(csr_consume_for_products(A));
  mark("release of what the products do not read");
  dnpeff_nmf* h = new dnpeff_nmf();
  h->A = A; h->r = rank; h->eps = eps; h->seed = (uint64_t)seed;
  h->n = A->n_rows; h->m = A->n_cols;
  h->sq_norm_A = sq_norm;
  h->tiled = tiled && A->n_cols > 0;
  h->tile_cols = h->tiled ? tile_cols_for(h->m, rank) : 0;
  const int64_t nr = h->n * rank, mr = h->m * rank;
  const int64_t h_floats = h->tiled ? (h->m + h->tile_cols) * rank : mr;
  const int64_t s_floats = h->tiled ? h->tile_cols * rank : mr;
  int64_t ws = gram_workspace_floats(h->m, rank);
  int64_t ws_n = gram_workspace_floats(h->n, rank);
  if (ws_n > ws) ws = ws_n;
  int s = dmalloc(&h->W, nr) || dmalloc(&h->W2, nr) || dmalloc(&h->Nw, nr) ||
          dmalloc(&h->Hbuf, h_floats) || dmalloc(&h->S, s_floats) ||
          dmalloc(&h->G, (int64_t)rank * rank) || dmalloc(&h->G2, (int64_t)rank * rank) ||
          dmalloc(&h->gram_ws, ws) || dmalloc(&h->dot_ws, DOT_BLOCKS + 2);
  h->H = h->Hbuf;
  if (!s && fused_update(h))
    s = dmalloc(&h->GH, (int64_t)rank * rank) || dmalloc(&h->gpart, xg_mu_gram_workspace_floats(h->m));
  if (!s && h->tiled && tuning().h_overlap != 0.0) s = dmalloc(&h->S2, s_floats);
  if (!s && h->tiled) s = csr_tile_lists(A);
  if (s) { dnpeff_nmf_destroy(h); return s; }
  mark("factors and workspaces");
  if (tuning().verbose != 0.0) {
    size_t free_b = 0, total_b = 0;
    (void)hipMemGetInfo(&free_b, &total_b);
    fprintf(stderr, "dnpeff: factors allocated (%s H update%s), %.1f GB of %.1f GB left free\n",
            h->tiled ? "tiled" : "full-size", consume ? ", matrix consumed" : "", (double)free_b / 1e9,
            (double)total_b / 1e9);
  }
  *out = h;
  return 0;
}

DN_API int dnpeff_nmf_create(dnpeff_csr* A, int rank, float eps, int64_t seed, dnpeff_nmf** out) {
  return nmf_create_impl(A, rank, eps, seed, 0u, out);
}

DN_API int dnpeff_nmf_create_ex(dnpeff_csr* A, int rank, float eps, int64_t seed, unsigned flags,
                                dnpeff_nmf** out) {
  return nmf_create_impl(A, rank, eps, seed, flags, out);
}

DN_API int dnpeff_nmf_info(const dnpeff_nmf* nmf, int* tiled, int64_t* tile_cols) {
  DN_CHECK(nmf != nullptr, "handle is NULL");
  if (tiled) *tiled = nmf->tiled ? 1 : 0;
  if (tile_cols) *tile_cols = nmf->tile_cols;
  return 0;
}

DN_API int dnpeff_nmf_init_factors(dnpeff_nmf* nmf) {
  clear_error();
  DN_CHECK(nmf != nullptr, "handle is NULL");
  nmf->gh_valid = false;
  nmf->nw_valid = false;
  DN_TRY(launch_init_uniform(0, nmf->n, nmf->r, nmf->seed, nmf->W));
  DN_TRY(launch_init_uniform(1, nmf->r, nmf->m, nmf->seed, nmf->H));
  return 0;
}

DN_API int dnpeff_nmf_set_factors(dnpeff_nmf* nmf, const float* W_nr, const float* H_rm) {
  clear_error();
  DN_CHECK(nmf != nullptr, "handle is NULL");
  DN_HIP(hipStreamSynchronize(stream()));
  if (W_nr)
    DN_HIP(hipMemcpy(nmf->W, W_nr, sizeof(float) * nmf->n * nmf->r, hipMemcpyHostToDevice));
  if (H_rm) {
    nmf->gh_valid = false;
    nmf->nw_valid = false;
    // [r, m] row-major on the host -> [m, r] on the device, through S, a column tile at a time
    // when S holds no more
    const int64_t step = nmf->tiled ? nmf->tile_cols : nmf->m;
    for (int64_t c0 = 0; c0 < nmf->m; c0 += step) {
      const int64_t len = nmf->m - c0 < step ? nmf->m - c0 : step;
      DN_HIP(hipMemcpy2D(nmf->S, sizeof(float) * len, H_rm + c0, sizeof(float) * nmf->m,
                         sizeof(float) * len, (size_t)nmf->r, hipMemcpyHostToDevice));
      DN_TRY(launch_transpose(nmf->r, len, nmf->S, nmf->H + c0 * nmf->r));
      DN_HIP(hipStreamSynchronize(stream()));
    }
  }
  return 0;
}

// The matrix may have been planned again for another rank since this handle was made (a second
// handle, a single-kernel call): make its work lists and workspaces fit this rank again.
static int products_for(dnpeff_nmf* h) {
  DN_TRY(csr_ensure_products(h->A, h->r));
  if (h->tiled) DN_TRY(csr_tile_lists(h->A));
  return 0;
}

DN_API int dnpeff_nmf_update_W(dnpeff_nmf* h) {
  DN_CHECK(h != nullptr, "handle is NULL");
  dnpeff_csr* A = h->A;
  bool gram_done = false;
  if (!h->nw_valid && !h->gh_valid && tuning().gram_beside != 0.0) {
    // H^T H on the second stream, the dense head of A H^T on the library stream behind it: the
    // head's workgroups take the CUs as those of H^T H leave them, and the rest of A H^T (kernels
    // that need the whole chip) starts when both are done.  Timing: H^T H from its start to its
    // end; A H^T from the end of H^T H to the end of the head (what the head adds), then the rest.
    DN_TRY(products_for(h));
    struct guard {
      ~guard() { side_stream_route(false); }
    } g;
    DN_TRY(side_stream_begin());
    int st = h->prof.begin(DNPEFF_K_GRAM_H);
    if (!st) st = launch_gram(h->m, h->r, h->H, h->G, h->gram_ws);
    if (!st) st = h->prof.next(DNPEFF_K_SPMM_N);
    DN_TRY(side_stream_end());
    DN_TRY(st);
    gram_done = true;
    DN_TRY(launch_spmm_n(A, h->r, h->H, 1));
    DN_TRY(h->prof.end());
    DN_TRY(side_stream_join());
    DN_TRY(h->prof.resume(DNPEFF_K_SPMM_N));
    DN_TRY(launch_spmm_n(A, h->r, h->H, 2));
    DN_TRY(h->prof.end());
    DN_TRY(h->prof.begin(DNPEFF_K_SPMM_N_REDUCE));
    DN_TRY(launch_spmm_n_reduce(A, h->r, h->Nw));
    DN_TRY(h->prof.end());
    h->nw_valid = true;
  }
  if (!h->nw_valid) {  // a loss evaluation since the last H update has left A H^T in Nw
    DN_TRY(products_for(h));
    DN_TRY(h->prof.begin(DNPEFF_K_SPMM_N));
    DN_TRY(launch_spmm_n(A, h->r, h->H));
    DN_TRY(h->prof.end());
    DN_TRY(h->prof.begin(DNPEFF_K_SPMM_N_REDUCE));
    DN_TRY(launch_spmm_n_reduce(A, h->r, h->Nw));
    DN_TRY(h->prof.end());
    h->nw_valid = true;
  }
  const float* Gh = h->GH;
  DN_TRY(side_stream_join());
  if (gram_done) {
    Gh = h->G;
  } else if (!h->gh_valid) {
    DN_TRY(h->prof.begin(DNPEFF_K_GRAM_H));
    DN_TRY(launch_gram(h->m, h->r, h->H, h->G, h->gram_ws));
    DN_TRY(h->prof.end());
    Gh = h->G;
  }
  DN_TRY(h->prof.begin(DNPEFF_K_XG_MU_W));
  DN_TRY(launch_xg_mu(h->n, h->r, h->W, Gh, h->Nw, h->eps, h->W2, nullptr));
  DN_TRY(h->prof.end());
  std::swap(h->W, h->W2);
  return 0;
}

// The H update on column tiles: A^T W of a tile into S, then the tile's update written one tile
// away from the old tile inside Hbuf.  H at the start of Hbuf: the new H goes one tile up and
// the tiles are walked from the last to the first (a new tile then lands on old tiles that were
// read already); H one tile up: the new H goes to the start, first tile first.  The tiles are
// independent of one another, so the order does not change any sum.
// The same with A^T W of tile q + 1 (library stream) running beside the update of tile q (second
// stream of the same priority), through two tile buffers.  The updates follow one another on
// their stream, so the rule about where a new tile may land holds as it does above; a product
// waits for the update that last read its buffer.  Same kernels on the same operands: same bits.
static int update_H_tiled_overlapped(dnpeff_nmf* h) {
  dnpeff_csr* A = h->A;
  const int r = h->r;
  const int64_t tile = h->tile_cols, n_tiles = ceil_div(h->m, tile);
  const bool up = h->H == h->Hbuf;
  float* Hnew = up ? h->Hbuf + tile * r : h->Hbuf;
  static hipEvent_t ev_t[2] = {nullptr, nullptr}, ev_x[2] = {nullptr, nullptr}, fork = nullptr;
  if (!fork) {
    DN_HIP(hipEventCreateWithFlags(&fork, hipEventDisableTiming));
    for (int b = 0; b < 2; b++) {
      DN_HIP(hipEventCreateWithFlags(&ev_t[b], hipEventDisableTiming));
      DN_HIP(hipEventCreateWithFlags(&ev_x[b], hipEventDisableTiming));
    }
  }
  hipStream_t s0 = stream(), s1 = side_stream_handle();
  DN_CHECK(s1 != nullptr, "second stream");
  struct guard {  // whatever happens, the library stream is where later launches go
    ~guard() { side_stream_route(false); xg_mu_release_g(); }
  } g;
  DN_TRY(h->prof.begin(DNPEFF_K_SPMM_T));
  DN_TRY(launch_head_t_product(A, r, h->W));
  DN_TRY(h->prof.end());
  DN_TRY(xg_mu_hold_g(h->G, r));
  DN_HIP(hipEventRecord(fork, s0));
  DN_HIP(hipStreamWaitEvent(s1, fork, 0));
  for (int64_t q = 0; q < n_tiles; q++) {
    const int64_t t = up ? n_tiles - 1 - q : q;
    const int64_t c0 = t * tile, c1 = c0 + tile < h->m ? c0 + tile : h->m;
    const int b = (int)(q & 1);
    float* Sb = b ? h->S2 : h->S;
    if (q >= 2) DN_HIP(hipStreamWaitEvent(s0, ev_x[b], 0));
    DN_TRY(h->prof.begin(DNPEFF_K_SPMM_T));
    DN_TRY(launch_spmm_t_tile(A, r, h->W, c0, c1, Sb));
    DN_TRY(h->prof.end());
    DN_HIP(hipEventRecord(ev_t[b], s0));
    DN_HIP(hipStreamWaitEvent(s1, ev_t[b], 0));
    side_stream_route(true);
    DN_TRY(h->prof.begin(DNPEFF_K_XG_MU_H));
    DN_TRY(launch_xg_mu(c1 - c0, r, h->H + c0 * r, h->G, Sb, h->eps, Hnew + c0 * r, nullptr));
    DN_TRY(h->prof.end());
    side_stream_route(false);
    DN_HIP(hipEventRecord(ev_x[b], s1));
  }
  DN_HIP(hipStreamWaitEvent(s0, ev_x[0], 0));
  if (n_tiles > 1) DN_HIP(hipStreamWaitEvent(s0, ev_x[1], 0));
  h->H = Hnew;
  h->gh_valid = false;
  return 0;
}

static int update_H_tiled(dnpeff_nmf* h) {
  if (h->S2) return update_H_tiled_overlapped(h);
  dnpeff_csr* A = h->A;
  const int r = h->r;
  const int64_t tile = h->tile_cols, n_tiles = ceil_div(h->m, tile);
  const bool up = h->H == h->Hbuf;
  float* Hnew = up ? h->Hbuf + tile * r : h->Hbuf;
  DN_TRY(h->prof.begin(DNPEFF_K_SPMM_T));
  DN_TRY(launch_head_t_product(A, r, h->W));
  DN_TRY(h->prof.end());
  struct held_g {  // G transposed once for all tiles
    ~held_g() { xg_mu_release_g(); }
  } hold;
  DN_TRY(xg_mu_hold_g(h->G, r));
  for (int64_t q = 0; q < n_tiles; q++) {
    const int64_t t = up ? n_tiles - 1 - q : q;
    const int64_t c0 = t * tile, c1 = c0 + tile < h->m ? c0 + tile : h->m;
    // (one event per change of class: a tile's product starts where the tile before ended)
    DN_TRY(q == 0 ? h->prof.begin(DNPEFF_K_SPMM_T) : h->prof.next(DNPEFF_K_SPMM_T));
    DN_TRY(launch_spmm_t_tile(A, r, h->W, c0, c1, h->S));
    DN_TRY(h->prof.next(DNPEFF_K_XG_MU_H));
    DN_TRY(launch_xg_mu(c1 - c0, r, h->H + c0 * r, h->G, h->S, h->eps, Hnew + c0 * r, nullptr));
  }
  DN_TRY(h->prof.end());
  h->H = Hnew;
  h->gh_valid = false;
  return 0;
}

DN_API int dnpeff_nmf_update_H(dnpeff_nmf* h) {
  DN_CHECK(h != nullptr, "handle is NULL");
  dnpeff_csr* A = h->A;
  DN_TRY(products_for(h));
  DN_TRY(h->prof.begin(DNPEFF_K_GRAM_W));
  DN_TRY(launch_gram(h->n, h->r, h->W, h->G, h->gram_ws));
  DN_TRY(h->prof.end());
  h->nw_valid = false;
  if (h->tiled) return update_H_tiled(h);
  DN_TRY(h->prof.begin(DNPEFF_K_SPMM_T));
  DN_TRY(launch_spmm_t(A, h->r, h->W, h->S));
  DN_TRY(h->prof.end());
  DN_TRY(h->prof.begin(DNPEFF_K_XG_MU_H));
  if (h->GH && ((uintptr_t)h->H % 16) == 0) {
    DN_TRY(launch_xg_mu_gram(h->m, h->H, h->G, h->S, h->eps, h->S, h->GH, h->gpart, h->G2, h->gram_ws));
    h->gh_valid = true;
  } else {
    DN_TRY(launch_xg_mu(h->m, h->r, h->H, h->G, h->S, h->eps, h->S, nullptr));
    h->gh_valid = false;
  }
  DN_TRY(h->prof.end());
  std::swap(h->H, h->S);
  h->Hbuf = h->H;
  return 0;
}

DN_API int dnpeff_nmf_step(dnpeff_nmf* nmf, int n_steps) {
  clear_error();
  DN_CHECK(nmf != nullptr, "handle is NULL");
  for (int s = 0; s < n_steps; s++) {
    DN_TRY(dnpeff_nmf_update_W(nmf));
    DN_TRY(dnpeff_nmf_update_H(nmf));
  }
  return 0;
}

DN_API int dnpeff_nmf_loss_terms(dnpeff_nmf* h, double* sq_norm_A, double* pos, double* neg) {
  clear_error();
  DN_CHECK(h != nullptr, "handle is NULL");
  dnpeff_csr* A = h->A;
  // neg = <W^T A, H> = <A H^T, W>
  if (!h->nw_valid) {
    DN_TRY(products_for(h));
    DN_TRY(launch_spmm_n(A, h->r, h->H));
    DN_TRY(launch_spmm_n_reduce(A, h->r, h->Nw));
    h->nw_valid = true;
  }
  DN_TRY(launch_dot(h->n * h->r, h->Nw, h->W, h->dot_ws, h->dot_ws + DOT_BLOCKS));
  // pos = <H, (W^T W) H> = <W^T W, H H^T>
  // (H^T H of the current H is at hand when the last H update produced it)
  const float* Gh = h->G;
  if (h->GH && h->gh_valid)
    Gh = h->GH;
  else
    DN_TRY(launch_gram(h->m, h->r, h->H, h->G, h->gram_ws));
  DN_TRY(launch_gram(h->n, h->r, h->W, h->G2, h->gram_ws));
  DN_TRY(launch_dot((int64_t)h->r * h->r, Gh, h->G2, h->dot_ws, h->dot_ws + DOT_BLOCKS + 1));
  double res[2];
  DN_HIP(hipStreamSynchronize(stream()));
  DN_HIP(hipMemcpy(res, h->dot_ws + DOT_BLOCKS, sizeof(double) * 2, hipMemcpyDeviceToHost));
  if (sq_norm_A) *sq_norm_A = h->sq_norm_A;
  if (neg) *neg = res[0];
  if (pos) *pos = res[1];
  return 0;
}

DN_API int dnpeff_nmf_check_products(dnpeff_nmf* h, double* via_rows, double* via_columns) {
  clear_error();
  DN_CHECK(h && via_rows && via_columns, "NULL argument");
  dnpeff_csr* A = h->A;
  DN_TRY(products_for(h));
  // <A H^T, W> through the row-ordered structures
  DN_TRY(launch_spmm_n(A, h->r, h->H));
  DN_TRY(launch_spmm_n_reduce(A, h->r, h->Nw));
  h->nw_valid = true;
  DN_TRY(launch_dot(h->n * h->r, h->Nw, h->W, h->dot_ws, h->dot_ws + DOT_BLOCKS));
  DN_HIP(hipStreamSynchronize(stream()));
  DN_HIP(hipMemcpy(via_rows, h->dot_ws + DOT_BLOCKS, sizeof(double), hipMemcpyDeviceToHost));
  // <A^T W, H> through the column-ordered ones (S is free between two H updates)
  double sum = 0.0;
  const int64_t step = h->tiled ? h->tile_cols : h->m;
  if (h->tiled) DN_TRY(launch_head_t_product(A, h->r, h->W));
  for (int64_t c0 = 0; c0 < h->m; c0 += step) {
    const int64_t c1 = c0 + step < h->m ? c0 + step : h->m;
    if (h->tiled)
      DN_TRY(launch_spmm_t_tile(A, h->r, h->W, c0, c1, h->S));
    else
      DN_TRY(launch_spmm_t(A, h->r, h->W, h->S));
    DN_TRY(launch_dot((c1 - c0) * h->r, h->S, h->H + c0 * h->r, h->dot_ws, h->dot_ws + DOT_BLOCKS + 1));
    double part = 0.0;
    DN_HIP(hipStreamSynchronize(stream()));
    DN_HIP(hipMemcpy(&part, h->dot_ws + DOT_BLOCKS + 1, sizeof(double), hipMemcpyDeviceToHost));
    sum += part;
  }
  *via_columns = sum;
  return 0;
}

DN_API int dnpeff_nmf_loss(dnpeff_nmf* nmf, double* out) {
  DN_CHECK(out != nullptr, "out is NULL");
  double a, p, q;
  DN_TRY(dnpeff_nmf_loss_terms(nmf, &a, &p, &q));
  *out = std::sqrt(a + p - 2.0 * q);
  return 0;
}

DN_API int dnpeff_nmf_sparsify_W(dnpeff_nmf* nmf, float l1_norm, float l2_norm, int* rounds) {
  clear_error();
  DN_CHECK(nmf, "NULL argument");
  // (H^T H and A H^T kept between calls depend on H only)
  return sparsify_columns(nmf->n, nmf->r, nmf->W, l1_norm, l2_norm, rounds);
}

DN_API int dnpeff_nmf_get_W(dnpeff_nmf* nmf, float* W_nr) {
  clear_error();
  DN_CHECK(nmf && W_nr, "NULL argument");
  DN_HIP(hipStreamSynchronize(stream()));
  DN_HIP(hipMemcpy(W_nr, nmf->W, sizeof(float) * nmf->n * nmf->r, hipMemcpyDeviceToHost));
  return 0;
}

DN_API int dnpeff_nmf_get_H(dnpeff_nmf* nmf, float* H_rm) {
  clear_error();
  DN_CHECK(nmf && H_rm, "NULL argument");
  // [m, r] on the device -> [r, m] row-major on the host, through S: all at once, or a column
  // tile at a time when S holds no more (the tiled H update)
  const int64_t step = nmf->tiled ? nmf->tile_cols : nmf->m;
  for (int64_t c0 = 0; c0 < nmf->m; c0 += step) {
    const int64_t len = nmf->m - c0 < step ? nmf->m - c0 : step;
    DN_TRY(launch_transpose(len, nmf->r, nmf->H + c0 * nmf->r, nmf->S));
    DN_HIP(hipStreamSynchronize(stream()));
    DN_HIP(hipMemcpy2D(H_rm + c0, sizeof(float) * nmf->m, nmf->S, sizeof(float) * len,
                       sizeof(float) * len, (size_t)nmf->r, hipMemcpyDeviceToHost));
  }
  return 0;
}

DN_API int dnpeff_nmf_device_factors(dnpeff_nmf* nmf, void** W_dev, void** H_dev) {
  DN_CHECK(nmf != nullptr, "handle is NULL");
  if (W_dev) *W_dev = nmf->W;
  if (H_dev) *H_dev = nmf->H;
  return 0;
}

DN_API int dnpeff_nmf_set_profiling(dnpeff_nmf* nmf, int enable) {
  DN_CHECK(nmf != nullptr, "handle is NULL");
  DN_TRY(nmf->prof.collect());
  nmf->prof.enabled = enable != 0;
  return 0;
}

DN_API int dnpeff_nmf_timings(dnpeff_nmf* nmf, double* ms_sum, int64_t* launches, int reset) {
  DN_CHECK(nmf != nullptr, "handle is NULL");
  DN_TRY(nmf->prof.collect());
  for (int i = 0; i < DNPEFF_K_COUNT; i++) {
    if (ms_sum) ms_sum[i] = nmf->prof.ms_sum[i];
    if (launches) launches[i] = nmf->prof.launches[i];
  }
  if (reset) nmf->prof.reset();
  return 0;
}

// ---------------------------------------------------------------------------
// Fixed sparse H, W-only learner
// ---------------------------------------------------------------------------
struct dnpeff_fit {
  int64_t n = 0;
  int r = 0;
  float eps = 0.0f;
  uint64_t seed = 0;
  float* AH = nullptr;   // [n, r]
  float* HH = nullptr;   // [r, r]
  float* W = nullptr;    // [n, r]
  float* W2 = nullptr;   // [n, r]
  float* WHH = nullptr;  // [n, r] W (H H^T) of the W before the last step
  float* tmp = nullptr;  // [n, r]
  double* dot_ws = nullptr;
  double sq_norm_A = 0.0;
  bool whh_valid = false;
};

DN_API int dnpeff_fit_destroy(dnpeff_fit* f) {
  if (!f) return 0;
  (void)hipStreamSynchronize(stream());
  dfree(f->AH); dfree(f->HH); dfree(f->W); dfree(f->W2); dfree(f->WHH); dfree(f->tmp);
  dfree(f->dot_ws);
  delete f;
  return 0;
}

DN_API int dnpeff_fit_create(dnpeff_csr* A, dnpeff_csr* H, float eps, int64_t seed,
                             dnpeff_fit** out) {
  clear_error();
  DN_CHECK(out != nullptr, "out is NULL");
  *out = nullptr;
  DN_CHECK(A && H, "matrix is NULL");
  DN_CHECK(A->n_cols == H->n_cols, "A has %lld columns but H has %lld", (long long)A->n_cols,
           (long long)H->n_cols);
  const int r = (int)H->n_rows;
  DN_CHECK(r >= 1 && r <= 1024, "rank %d outside [1, 1024]", r);
  dnpeff_fit* f = new dnpeff_fit();
  f->n = A->n_rows; f->r = r; f->eps = eps; f->seed = (uint64_t)seed;
  const int64_t nr = f->n * r;
  int s = dmalloc(&f->AH, nr) || dmalloc(&f->HH, (int64_t)r * r) || dmalloc(&f->W, nr) ||
          dmalloc(&f->W2, nr) || dmalloc(&f->WHH, nr) || dmalloc(&f->tmp, nr) ||
          dmalloc(&f->dot_ws, DOT_BLOCKS + 2);
  if (!s) s = dnpeff_op_spsp_dense(H, H, f->HH);
  if (!s) s = dnpeff_op_spsp_dense(A, H, f->AH);
  if (!s) s = dnpeff_csr_sq_norm(A, &f->sq_norm_A);
  if (!s && hipStreamSynchronize(stream()) != hipSuccess) {
    set_error("first stage kernels failed");
    s = 1;
  }
  if (s) { dnpeff_fit_destroy(f); return s; }
  *out = f;
  return 0;
}

DN_API int dnpeff_fit_init_W(dnpeff_fit* f) {
  clear_error();
  DN_CHECK(f != nullptr, "handle is NULL");
  f->whh_valid = false;
  return launch_init_uniform(0, f->n, f->r, f->seed, f->W);
}

DN_API int dnpeff_fit_set_W(dnpeff_fit* f, const float* W_nr) {
  clear_error();
  DN_CHECK(f && W_nr, "NULL argument");
  DN_HIP(hipStreamSynchronize(stream()));
  DN_HIP(hipMemcpy(f->W, W_nr, sizeof(float) * f->n * f->r, hipMemcpyHostToDevice));
  f->whh_valid = false;
  return 0;
}

DN_API int dnpeff_fit_step(dnpeff_fit* f, int n_steps) {
  clear_error();
  DN_CHECK(f != nullptr, "handle is NULL");
  struct held_g {  // H H^T is the same in every step: one transposed copy for all of them
    ~held_g() { xg_mu_release_g(); }
  } hold;
  DN_TRY(xg_mu_hold_g(f->HH, f->r));
  for (int s = 0; s < n_steps; s++) {
    DN_TRY(launch_xg_mu(f->n, f->r, f->W, f->HH, f->AH, f->eps, f->W2, f->WHH));
    std::swap(f->W, f->W2);
    f->whh_valid = true;
  }
  return 0;
}

DN_API int dnpeff_fit_loss(dnpeff_fit* f, double* reference_loss, double* true_loss) {
  clear_error();
  DN_CHECK(f != nullptr, "handle is NULL");
  const int64_t nr = f->n * f->r;
  double res[2];
  // neg = <A H^T, W>
  DN_TRY(launch_dot(nr, f->AH, f->W, f->dot_ws, f->dot_ws + DOT_BLOCKS));
  // pos of the current W; W2 receives an update that is discarded
  DN_TRY(launch_xg_mu(f->n, f->r, f->W, f->HH, f->AH, f->eps, f->W2, f->tmp));
  DN_TRY(launch_dot(nr, f->tmp, f->W, f->dot_ws, f->dot_ws + DOT_BLOCKS + 1));
  DN_HIP(hipStreamSynchronize(stream()));
  DN_HIP(hipMemcpy(res, f->dot_ws + DOT_BLOCKS, sizeof(double) * 2, hipMemcpyDeviceToHost));
  const double neg = res[0], pos_true = res[1];
  if (true_loss) *true_loss = std::sqrt(f->sq_norm_A + pos_true - 2.0 * neg);
  if (reference_loss) {
    double pos_ref = pos_true;
    if (f->whh_valid) {
      DN_TRY(launch_dot(nr, f->WHH, f->W, f->dot_ws, f->dot_ws + DOT_BLOCKS));
      DN_HIP(hipStreamSynchronize(stream()));
      DN_HIP(hipMemcpy(&pos_ref, f->dot_ws + DOT_BLOCKS, sizeof(double), hipMemcpyDeviceToHost));
    }
    *reference_loss = std::sqrt(f->sq_norm_A + pos_ref - 2.0 * neg);
  }
  return 0;
}

DN_API int dnpeff_fit_get_W(dnpeff_fit* f, float* W_nr) {
  clear_error();
  DN_CHECK(f && W_nr, "NULL argument");
  DN_HIP(hipStreamSynchronize(stream()));
  DN_HIP(hipMemcpy(W_nr, f->W, sizeof(float) * f->n * f->r, hipMemcpyDeviceToHost));
  return 0;
}

DN_API int dnpeff_fit_get_products(dnpeff_fit* f, float* AH_nr, float* HH_rr, double* sq_norm_A) {
  clear_error();
  DN_CHECK(f != nullptr, "handle is NULL");
  DN_HIP(hipStreamSynchronize(stream()));
  if (AH_nr) DN_HIP(hipMemcpy(AH_nr, f->AH, sizeof(float) * f->n * f->r, hipMemcpyDeviceToHost));
  if (HH_rr)
    DN_HIP(hipMemcpy(HH_rr, f->HH, sizeof(float) * f->r * f->r, hipMemcpyDeviceToHost));
  if (sq_norm_A) *sq_norm_A = f->sq_norm_A;
  return 0;
}
