/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * CPU restatement of the D-NPEFF NMF hot path of mmatena/npeff_ref, used only
 * as the checker in tests/, in __graft_entry__.smoke() and as the timed
 * cpu_baseline leg of bench.py.  Nothing under npeff_ref_amd/ may include,
 * link or call this file.
 *
 * Every function cites the reference lines it follows (paths relative to the
 * reference root).  Integer/byte functions (orc_normalize_rows .. orc_transpose)
 * are meant to be bit-exact with the reference; the floating-point NMF loops are
 * the reference's update sequence evaluated in fp64 (orc_nmf_f64, orc_fit_f64)
 * or in fp32 with OpenMP (orc_nmf_f32, the timed baseline).
 *
 * Pinning (what fixes each function independently of this text):
 *   orc_compact_columns  -- the reference's own known-answer tests
 *                           cc/cuda_lrm_npeff/src/preprocess/column_pruning_test.cc:24-105
 *                           (tests/golden/column_pruning.json) and the compiled
 *                           reference routine in oracle/_ref.
 *   orc_csr_from_dense, orc_validate_indices
 *                        -- cc/cuda_lrm_npeff/src/containers/conversions_test.cc:8-62,
 *                           sparse_matrix_test.cc:26-88, and oracle/_ref.
 *   orc_retain_columns   -- brute force over dense matrices (tests/test_oracle_loader.py);
 *                           the reference holds no test for it.
 *   orc_normalize_rows, orc_size_of_split, orc_split_row_wise, orc_split_column_wise
 *                        -- closed forms / brute force.
 *   orc_transpose        -- (A^T)^T = A and a dense transpose on tiny inputs.
 *   orc_nmf_f64, orc_fit_f64
 *                        -- dense numpy evaluation of the same update rules and the
 *                           explicit residual ||A - W H||_F on tiny inputs; MU
 *                           monotonicity of the true loss.  The reference holds no
 *                           numeric fixture for these ("parity unpinned" against the
 *                           reference's own cuSPARSE/cuBLAS bits, by construction).
 *   orc_sparsify_columns -- what its iteration fixes whatever the step length: every column
 *                           ends non-negative with the prescribed sum, entries keep their
 *                           order, a column that needs no second pass is an affine image of
 *                           its input; and what the reference's step length fixes:
 *                           ||column||^2 = l2^2 + l1^2 / (entries left non-zero), against l2^2
 *                           for Hoyer's own (tests/test_oracle_sparsify.py).  The reference
 *                           never runs this code and holds no vector for it: "parity
 *                           unpinned" against the reference's bits.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------- */
/* Loader                                                                     */
/* ------------------------------------------------------------------------- */

/* v /= (norm_i + eps) per row, fp32.
 * cc/cuda_d_npeff/src/io/pef_fisher_h5.h:38-52 */
ORC_API void orc_normalize_rows(int64_t n_rows, const int64_t* rowptr, float* vals,
                                const float* norms, float eps) {
  for (int64_t row = 0; row < n_rows; row++) {
    float example_norm = norms[row] + eps;
    for (int64_t j = rowptr[row]; j < rowptr[row + 1]; j++) vals[j] /= example_norm;
  }
}

/* Fixed-width PEF block -> row offsets i*k.
 * cc/cuda_d_npeff/src/io/pef_fisher_h5.h:175-177 */
ORC_API void orc_pef_rowptr(int64_t n_rows, int64_t k, int64_t* rowptr) {
  for (int64_t i = 0; i < n_rows + 1; i++) rowptr[i] = i * k;
}

/* Column compaction, in place.  Returns the new column count; rowptr[n_rows]
 * is the new nnz; new_to_og needs room for n_cols entries.
 * cc/cuda_d_npeff/src/util/sparse_util.h:78-159 (same sweep as
 * cc/cuda_lrm_npeff/src/preprocess/column_pruning.h:14-82) */
ORC_API int64_t orc_compact_columns(int64_t n_rows, int64_t n_cols, int64_t* rowptr,
                                    int32_t* colind, float* vals, int min_count,
                                    int32_t* new_to_og) {
  int64_t nnz = rowptr[n_rows];
  int* col_count = (int*)calloc((size_t)(n_cols > 0 ? n_cols : 1), sizeof(int));
  for (int64_t i = 0; i < nnz; i++) col_count[colind[i]] += 1; /* :94-97 */

  int32_t* og_to_new = (int32_t*)malloc(sizeof(int32_t) * (size_t)(n_cols > 0 ? n_cols : 1));
  int64_t new_index = 0;
  for (int64_t i = 0; i < n_cols; i++) { /* :108-117 */
    if (col_count[i] >= min_count) {
      og_to_new[i] = (int32_t)new_index;
      new_to_og[new_index] = (int32_t)i;
      new_index++;
    } else {
      og_to_new[i] = -1;
    }
  }

  int64_t i2 = 0, row_index = 0;
  for (int64_t i = 0; i < nnz; i++) { /* :130-148 */
    int32_t new_col = og_to_new[colind[i]];
    while (row_index <= n_rows && i == rowptr[row_index]) rowptr[row_index++] = i2;
    if (new_col != -1) {
      colind[i2] = new_col;
      vals[i2] = vals[i];
      i2++;
    }
  }
  /* Rows that end the matrix with no entries are still pending here; the
   * reference writes only one offset (:151-152), which is enough for its
   * fixed-width input.  All pending offsets equal the new nnz. */
  while (row_index <= n_rows) rowptr[row_index++] = i2;

  free(col_count);
  free(og_to_new);
  return new_index;
}

/* Keep columns listed in kept[], renumber to the position in kept[].  Returns
 * new nnz.  cc/cuda_d_npeff/src/cuda/host/sparse_matrix.h:141-170 */
ORC_API int64_t orc_retain_columns(int64_t n_rows, int64_t n_cols, int64_t* rowptr,
                                   int32_t* colind, float* vals, const int32_t* kept,
                                   int64_t n_kept) {
  int64_t nnz = rowptr[n_rows];
  int32_t* old_to_new = (int32_t*)malloc(sizeof(int32_t) * (size_t)(n_cols > 0 ? n_cols : 1));
  for (int64_t i = 0; i < n_cols; i++) old_to_new[i] = -1;
  for (int64_t i = 0; i < n_kept; i++) old_to_new[kept[i]] = (int32_t)i;

  int64_t i2 = 0, row_index = 0;
  for (int64_t i = 0; i < nnz; i++) {
    int32_t new_col = old_to_new[colind[i]];
    while (row_index <= n_rows && i == rowptr[row_index]) rowptr[row_index++] = i2;
    if (new_col != -1) {
      colind[i2] = new_col;
      vals[i2] = vals[i];
      i2++;
    }
  }
  while (row_index <= n_rows) rowptr[row_index++] = i2;
  free(old_to_new);
  return i2;
}

/* cc/cuda_d_npeff/src/util/matrix_util.h:10-21;
 * cc/cuda_d_npeff/src/cuda/host/sparse_matrix.h:107-117.  -1 where the
 * reference throws. */
ORC_API int64_t orc_size_of_split(int64_t total, int64_t n_splits, int64_t split_index) {
  int64_t base = total / n_splits;
  if (split_index >= n_splits) return -1;
  if (split_index == n_splits - 1) return base + (total % n_splits);
  return base;
}

/* Row-wise split: for split s, first row and first entry offset; a split's
 * arrays are the slices [entry_start[s], entry_start[s+1]) with row offsets
 * rebased to 0.  cc/cuda_d_npeff/src/cuda/host/sparse_matrix.h:219-245 */
ORC_API void orc_split_row_wise(int64_t n_rows, const int64_t* rowptr, int n_splits,
                                int64_t* row_start /*[n_splits+1]*/,
                                int64_t* entry_start /*[n_splits+1]*/) {
  int64_t start_row = 0;
  for (int i = 0; i < n_splits; i++) {
    row_start[i] = start_row;
    entry_start[i] = rowptr[start_row];
    start_row += orc_size_of_split(n_rows, n_splits, i);
  }
  row_start[n_splits] = start_row;
  entry_start[n_splits] = rowptr[start_row];
}

/* Column-wise split number `split` of `n_splits`: writes the slice as its own
 * CSR (column ids rebased) and returns its nnz.
 * cc/cuda_d_npeff/src/util/matrix_util.h:23-69 */
ORC_API int64_t orc_split_column_wise(int64_t n_rows, int64_t n_cols, const int64_t* rowptr,
                                      const int32_t* colind, const float* vals, int n_splits,
                                      int split, int64_t* out_rowptr, int32_t* out_colind,
                                      float* out_vals) {
  int64_t start_col = 0;
  for (int i = 0; i < split; i++) start_col += orc_size_of_split(n_cols, n_splits, i);
  int64_t end_col = start_col + orc_size_of_split(n_cols, n_splits, split);
  int64_t k = 0;
  for (int64_t row = 0; row < n_rows; row++) {
    out_rowptr[row] = k;
    for (int64_t j = rowptr[row]; j < rowptr[row + 1]; j++) {
      if (start_col <= colind[j] && colind[j] < end_col) {
        if (out_colind) {
          out_vals[k] = vals[j];
          out_colind[k] = (int32_t)(colind[j] - start_col);
        }
        k++;
      }
    }
  }
  out_rowptr[n_rows] = k;
  return k;
}

/* CSR from a row-major dense array, entries with |x| > threshold kept.
 * cc/cuda_lrm_npeff/src/containers/conversions.h:53-92,113-122 */
ORC_API int64_t orc_csr_from_dense(const float* dense, int64_t n_rows, int64_t n_cols,
                                   float threshold, int64_t* rowptr, int32_t* colind,
                                   float* vals) {
  int64_t k = 0;
  rowptr[0] = 0;
  for (int64_t i = 0; i < n_rows; i++) {
    for (int64_t j = 0; j < n_cols; j++) {
      float e = dense[i * n_cols + j];
      if (fabsf(e) > threshold) {
        vals[k] = e;
        colind[k] = (int32_t)j;
        k++;
      }
    }
    rowptr[i + 1] = k;
  }
  return k;
}

/* 1 if the CSR indices are valid: first offset 0, last == nnz, offsets
 * non-decreasing, column ids in range, no duplicate column in a row.
 * cc/cuda_lrm_npeff/src/containers/sparse_matrix.h:81-110 */
static int cmp_i32(const void* a, const void* b) {
  int32_t x = *(const int32_t*)a, y = *(const int32_t*)b;
  return (x > y) - (x < y);
}
ORC_API int orc_validate_indices(int64_t n_rows, int64_t n_cols, int64_t nnz,
                                 const int64_t* rowptr, const int32_t* colind) {
  if (rowptr[0] != 0 || rowptr[n_rows] != nnz) return 0;
  for (int64_t i = 0; i < n_rows; i++)
    if (rowptr[i] > rowptr[i + 1]) return 0;
  for (int64_t i = 0; i < nnz; i++)
    if (colind[i] < 0 || colind[i] >= n_cols) return 0;
  for (int64_t i = 0; i < n_rows; i++) {
    int64_t len = rowptr[i + 1] - rowptr[i];
    if (len < 2) continue;
    int32_t* tmp = (int32_t*)malloc(sizeof(int32_t) * (size_t)len);
    memcpy(tmp, colind + rowptr[i], sizeof(int32_t) * (size_t)len);
    qsort(tmp, (size_t)len, sizeof(int32_t), cmp_i32);
    int dup = 0;
    for (int64_t j = 1; j < len; j++)
      if (tmp[j] == tmp[j - 1]) dup = 1;
    free(tmp);
    if (dup) return 0;
  }
  return 1;
}

/* Transposed CSR by counting sort: per column the (row, value) pairs in
 * ascending row order.  This canonical order is what the reference's
 * cusparseCsr2cscEx2 produces and what its atomics-based int64 path leaves
 * undefined (cc/cuda_d_npeff/src/cuda/ops/transpose.h:82-115,296-331). */
ORC_API void orc_transpose(int64_t n_rows, int64_t n_cols, const int64_t* rowptr,
                           const int32_t* colind, const float* vals, int64_t* colptr,
                           int32_t* rowind, float* tvals) {
  int64_t nnz = rowptr[n_rows];
  for (int64_t j = 0; j <= n_cols; j++) colptr[j] = 0;
  for (int64_t e = 0; e < nnz; e++) colptr[colind[e] + 1]++;
  for (int64_t j = 0; j < n_cols; j++) colptr[j + 1] += colptr[j];
  int64_t* cur = (int64_t*)malloc(sizeof(int64_t) * (size_t)(n_cols > 0 ? n_cols : 1));
  memcpy(cur, colptr, sizeof(int64_t) * (size_t)n_cols);
  for (int64_t i = 0; i < n_rows; i++)
    for (int64_t e = rowptr[i]; e < rowptr[i + 1]; e++) {
      int64_t p = cur[colind[e]]++;
      rowind[p] = (int32_t)i;
      tvals[p] = vals[e];
    }
  free(cur);
}

/* ------------------------------------------------------------------------- */
/* fp64 evaluation of the reference update sequence                           */
/* Internally H is kept as Ht [m, r] (r contiguous), which is the reference's  */
/* column-major r x m array.                                                  */
/* ------------------------------------------------------------------------- */

/* out[n, r] = A * Ht   (A H^T: computeLocalAH,
 * multi_mu_dense_factors_device_contexts1.h:315-318) */
static void spmm_n_f64(int64_t n, const int64_t* rowptr, const int32_t* colind,
                       const float* vals, int r, const double* Ht, double* out) {
#pragma omp parallel for schedule(dynamic, 4)
  for (int64_t i = 0; i < n; i++) {
    double* o = out + i * r;
    for (int c = 0; c < r; c++) o[c] = 0.0;
    for (int64_t e = rowptr[i]; e < rowptr[i + 1]; e++) {
      const double* h = Ht + (int64_t)colind[e] * r;
      double a = (double)vals[e];
      for (int c = 0; c < r; c++) o[c] += a * h[c];
    }
  }
}

/* out[m, r] = A^T * W  (spmmAW, device_contexts1.h:260-265,301) */
static void spmm_t_f64(int64_t m, const int64_t* colptr, const int32_t* rowind,
                       const float* tvals, int r, const double* W, double* out) {
#pragma omp parallel for schedule(dynamic, 1024)
  for (int64_t j = 0; j < m; j++) {
    double* o = out + j * r;
    for (int c = 0; c < r; c++) o[c] = 0.0;
    for (int64_t p = colptr[j]; p < colptr[j + 1]; p++) {
      const double* w = W + (int64_t)rowind[p] * r;
      double a = (double)tvals[p];
      for (int c = 0; c < r; c++) o[c] += a * w[c];
    }
  }
}

/* G[r, r] = X^T X for X [rows, r]  (denseMatMul for HH^T and W^T W,
 * device_contexts1.h:303,322) */
static void gram_f64(int64_t rows, int r, const double* X, double* G) {
  for (int i = 0; i < r * r; i++) G[i] = 0.0;
#pragma omp parallel
  {
    double* loc = (double*)calloc((size_t)r * r, sizeof(double));
#pragma omp for schedule(static)
    for (int64_t k = 0; k < rows; k++) {
      const double* x = X + k * r;
      for (int a = 0; a < r; a++) {
        double xa = x[a];
        for (int b = 0; b < r; b++) loc[a * r + b] += xa * x[b];
      }
    }
#pragma omp critical
    for (int i = 0; i < r * r; i++) G[i] += loc[i];
    free(loc);
  }
}

/* D[rows, r] = X G  (W (HH^T), (W^T W) H; device_contexts1.h:306,329) */
static void xg_f64(int64_t rows, int r, const double* X, const double* G, double* D) {
#pragma omp parallel for schedule(static)
  for (int64_t k = 0; k < rows; k++) {
    const double* x = X + k * r;
    double* d = D + k * r;
    for (int b = 0; b < r; b++) d[b] = 0.0;
    for (int a = 0; a < r; a++) {
      double xa = x[a];
      const double* g = G + a * r;
      for (int b = 0; b < r; b++) d[b] += xa * g[b];
    }
  }
}

/* F *= num / (den + eps): divide first, then multiply
 * (cc/cuda_d_npeff/src/nmf/sparse/kernels.h:24-34) */
static void mu_f64(int64_t count, double* F, const double* num, const double* den, double eps) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < count; i++) F[i] *= num[i] / (den[i] + eps);
}

static double dot_f64(int64_t count, const double* x, const double* y) {
  double s = 0.0;
#pragma omp parallel for reduction(+ : s) schedule(static)
  for (int64_t i = 0; i < count; i++) s += x[i] * y[i];
  return s;
}

static void transpose_to_mr(int64_t m, int r, const double* H_rm, double* Ht) {
  for (int c = 0; c < r; c++)
    for (int64_t j = 0; j < m; j++) Ht[j * r + c] = H_rm[(int64_t)c * m + j];
}
static void transpose_to_rm(int64_t m, int r, const double* Ht, double* H_rm) {
  for (int c = 0; c < r; c++)
    for (int64_t j = 0; j < m; j++) H_rm[(int64_t)c * m + j] = Ht[j * r + c];
}

/* Loss through the reference's trace identity
 * (device_contexts1.h:337-354; combine at multi_mu_dense_factors_nmf1.h:242-274):
 * pos = <H, (W^T W) H>, neg = <W^T A, H>. */
static double loss_f64(int64_t n, int64_t m, int r, const int64_t* colptr, const int32_t* rowind,
                       const float* tvals, double sq_norm_A, const double* W, const double* Ht,
                       double* buf_num, double* buf_den, double* terms) {
  double* G = (double*)malloc(sizeof(double) * r * r);
  gram_f64(n, r, W, G);
  xg_f64(m, r, Ht, G, buf_den);
  double pos = dot_f64(m * r, Ht, buf_den);
  spmm_t_f64(m, colptr, rowind, tvals, r, W, buf_num);
  double neg = dot_f64(m * r, buf_num, Ht);
  free(G);
  if (terms) {
    terms[0] = sq_norm_A;
    terms[1] = pos;
    terms[2] = neg;
  }
  return sqrt(sq_norm_A + pos - 2.0 * neg);
}

/* MU NMF, reference order: per step W-update then H-update with the new W; the
 * loss after every `log_every` steps (MuNmf::run,
 * multi_mu_dense_factors_nmf1.h:152-205; updateW :293-305; updateH
 * device_contexts1.h:296-309).  W [n, r] row-major, H [r, m] row-major, both
 * in/out.  losses receives floor(iters/log_every) values (may be NULL). */
ORC_API void orc_nmf_f64(int64_t n, int64_t m, const int64_t* rowptr, const int32_t* colind,
                         const float* vals, int r, float eps_f, int iters, int log_every,
                         double* W, double* H_rm, double* losses) {
  int64_t nnz = rowptr[n];
  double eps = (double)eps_f;
  int64_t big = (n > m ? n : m);
  double* Ht = (double*)malloc(sizeof(double) * m * r);
  double* num = (double*)malloc(sizeof(double) * big * r);
  double* den = (double*)malloc(sizeof(double) * big * r);
  double* G = (double*)malloc(sizeof(double) * r * r);
  int64_t* colptr = (int64_t*)malloc(sizeof(int64_t) * (m + 1));
  int32_t* rowind = (int32_t*)malloc(sizeof(int32_t) * (nnz > 0 ? nnz : 1));
  float* tvals = (float*)malloc(sizeof(float) * (nnz > 0 ? nnz : 1));
  orc_transpose(n, m, rowptr, colind, vals, colptr, rowind, tvals);
  transpose_to_mr(m, r, H_rm, Ht);

  double sq_norm_A = 0.0; /* computeASqNorm, device_contexts1.h:274-294 */
  for (int64_t e = 0; e < nnz; e++) sq_norm_A += (double)vals[e] * (double)vals[e];

  int n_logged = 0;
  for (int step = 0; step < iters; step++) {
    /* updateW */
    spmm_n_f64(n, rowptr, colind, vals, r, Ht, num);
    gram_f64(m, r, Ht, G);
    xg_f64(n, r, W, G, den);
    mu_f64(n * r, W, num, den, eps);
    /* updateH */
    spmm_t_f64(m, colptr, rowind, tvals, r, W, num);
    gram_f64(n, r, W, G);
    xg_f64(m, r, Ht, G, den);
    mu_f64(m * r, Ht, num, den, eps);
    if (log_every > 0 && (step + 1) % log_every == 0 && losses)
      losses[n_logged++] =
          loss_f64(n, m, r, colptr, rowind, tvals, sq_norm_A, W, Ht, num, den, NULL);
  }
  transpose_to_rm(m, r, Ht, H_rm);
  free(Ht); free(num); free(den); free(G); free(colptr); free(rowind); free(tvals);
}

/* Loss of given factors and its three terms {||A||^2, pos, neg}. */
ORC_API double orc_loss_f64(int64_t n, int64_t m, const int64_t* rowptr, const int32_t* colind,
                            const float* vals, int r, const double* W, const double* H_rm,
                            double* terms) {
  int64_t nnz = rowptr[n];
  double* Ht = (double*)malloc(sizeof(double) * m * r);
  double* num = (double*)malloc(sizeof(double) * m * r);
  double* den = (double*)malloc(sizeof(double) * m * r);
  int64_t* colptr = (int64_t*)malloc(sizeof(int64_t) * (m + 1));
  int32_t* rowind = (int32_t*)malloc(sizeof(int32_t) * (nnz > 0 ? nnz : 1));
  float* tvals = (float*)malloc(sizeof(float) * (nnz > 0 ? nnz : 1));
  orc_transpose(n, m, rowptr, colind, vals, colptr, rowind, tvals);
  transpose_to_mr(m, r, H_rm, Ht);
  double sq = 0.0;
  for (int64_t e = 0; e < nnz; e++) sq += (double)vals[e] * (double)vals[e];
  double loss = loss_f64(n, m, r, colptr, rowind, tvals, sq, W, Ht, num, den, terms);
  free(Ht); free(num); free(den); free(colptr); free(rowind); free(tvals);
  return loss;
}

/* Single products in fp64, for per-kernel parity tests. */
ORC_API void orc_spmm_n_f64(int64_t n, const int64_t* rowptr, const int32_t* colind,
                            const float* vals, int r, const double* Ht_mr, double* out_nr) {
  spmm_n_f64(n, rowptr, colind, vals, r, Ht_mr, out_nr);
}
ORC_API void orc_spmm_t_f64(int64_t n, int64_t m, const int64_t* rowptr, const int32_t* colind,
                            const float* vals, int r, const double* W_nr, double* out_mr) {
  int64_t nnz = rowptr[n];
  int64_t* colptr = (int64_t*)malloc(sizeof(int64_t) * (m + 1));
  int32_t* rowind = (int32_t*)malloc(sizeof(int32_t) * (nnz > 0 ? nnz : 1));
  float* tvals = (float*)malloc(sizeof(float) * (nnz > 0 ? nnz : 1));
  orc_transpose(n, m, rowptr, colind, vals, colptr, rowind, tvals);
  spmm_t_f64(m, colptr, rowind, tvals, r, W_nr, out_mr);
  free(colptr); free(rowind); free(tvals);
}
ORC_API void orc_gram_f64(int64_t rows, int r, const double* X, double* G) {
  gram_f64(rows, r, X, G);
}
ORC_API void orc_xg_mu_f64(int64_t rows, int r, const double* X, const double* G,
                           const double* num, float eps, double* out, double* D_out) {
  double* D = (double*)malloc(sizeof(double) * rows * r);
  xg_f64(rows, r, X, G, D);
  for (int64_t i = 0; i < rows * r; i++) out[i] = X[i] * (num[i] / (D[i] + (double)eps));
  if (D_out) memcpy(D_out, D, sizeof(double) * rows * r);
  free(D);
}

/* ------------------------------------------------------------------------- */
/* Fixed sparse H, W-only learner in fp64                                     */
/* ------------------------------------------------------------------------- */

/* out[n, r] = A B^T for CSR A [n, m] and CSR B [r, m], via B densified by
 * column lists (ComputeProductWithHT, nmf/sparse2/nmf_sparse_H.h:264-272;
 * cuda/ops/spsp_matmul.h:95-131). */
ORC_API void orc_spsp_dense_f64(int64_t n, int64_t m, const int64_t* a_rowptr,
                                const int32_t* a_colind, const float* a_vals, int r,
                                const int64_t* b_rowptr, const int32_t* b_colind,
                                const float* b_vals, double* out_nr) {
  int64_t bnnz = b_rowptr[r];
  int64_t* colptr = (int64_t*)malloc(sizeof(int64_t) * (m + 1));
  int32_t* comp = (int32_t*)malloc(sizeof(int32_t) * (bnnz > 0 ? bnnz : 1));
  float* tv = (float*)malloc(sizeof(float) * (bnnz > 0 ? bnnz : 1));
  orc_transpose(r, m, b_rowptr, b_colind, b_vals, colptr, comp, tv);
#pragma omp parallel for schedule(dynamic, 4)
  for (int64_t i = 0; i < n; i++) {
    double* o = out_nr + i * r;
    for (int c = 0; c < r; c++) o[c] = 0.0;
    for (int64_t e = a_rowptr[i]; e < a_rowptr[i + 1]; e++) {
      int64_t j = a_colind[e];
      double a = (double)a_vals[e];
      for (int64_t p = colptr[j]; p < colptr[j + 1]; p++) o[comp[p]] += a * (double)tv[p];
    }
  }
  free(colptr); free(comp); free(tv);
}

/* Stage 2 of the learner (RunSecondStage / DoMuStep,
 * nmf/sparse2/nmf_sparse_H.h:298-345).  AH [n, r], HH [r, r], W [n, r] in/out.
 * ref_losses: the value the reference logs, which pairs WHH computed BEFORE the
 * step's update with the W AFTER it (:319,327-331).  true_losses: same formula
 * with WHH recomputed from the updated W.  One value per `log_every` steps. */
ORC_API void orc_fit_f64(int64_t n, int r, const double* AH, const double* HH, double sq_norm_A,
                         float eps_f, int iters, int log_every, double* W, double* ref_losses,
                         double* true_losses) {
  double eps = (double)eps_f;
  double* WHH = (double*)malloc(sizeof(double) * n * r);
  double* tmp = (double*)malloc(sizeof(double) * n * r);
  int n_logged = 0;
  for (int i = 0; i < iters; i++) {
    xg_f64(n, r, W, HH, WHH);
    mu_f64(n * r, W, AH, WHH, eps);
    if (log_every > 0 && (i + 1) % log_every == 0) {
      double neg = dot_f64(n * r, AH, W);
      double pos_ref = dot_f64(n * r, WHH, W);
      xg_f64(n, r, W, HH, tmp);
      double pos_true = dot_f64(n * r, tmp, W);
      if (ref_losses) ref_losses[n_logged] = sqrt(sq_norm_A + pos_ref - 2.0 * neg);
      if (true_losses) true_losses[n_logged] = sqrt(sq_norm_A + pos_true - 2.0 * neg);
      n_logged++;
    }
  }
  free(WHH); free(tmp);
}

/* ------------------------------------------------------------------------- */
/* fp32 OpenMP port of the same loop: the timed CPU baseline                  */
/* ------------------------------------------------------------------------- */

typedef struct {
  int64_t n, m, nnz;
  int r;
  float eps;
  const int64_t* rowptr;
  const int32_t* colind;
  const float* vals;
  int64_t* colptr;
  int32_t* rowind;
  float* tvals;
  float *W, *Ht, *num, *G;
  double sq_norm_A;
} orc_f32_ctx;

static void spmm_n_f32(const orc_f32_ctx* c, float* out) {
  const int r = c->r;
#pragma omp parallel for schedule(dynamic, 1)
  for (int64_t i = 0; i < c->n; i++) {
    float* o = out + i * r;
    for (int k = 0; k < r; k++) o[k] = 0.0f;
    for (int64_t e = c->rowptr[i]; e < c->rowptr[i + 1]; e++) {
      const float* h = c->Ht + (int64_t)c->colind[e] * r;
      float a = c->vals[e];
#pragma omp simd
      for (int k = 0; k < r; k++) o[k] += a * h[k];
    }
  }
}

static void spmm_t_f32(const orc_f32_ctx* c, float* out) {
  const int r = c->r;
#pragma omp parallel for schedule(dynamic, 4096)
  for (int64_t j = 0; j < c->m; j++) {
    float* o = out + j * r;
    for (int k = 0; k < r; k++) o[k] = 0.0f;
    for (int64_t p = c->colptr[j]; p < c->colptr[j + 1]; p++) {
      const float* w = c->W + (int64_t)c->rowind[p] * r;
      float a = c->tvals[p];
#pragma omp simd
      for (int k = 0; k < r; k++) o[k] += a * w[k];
    }
  }
}

/* G = X^T X (the cublasSgemm at device_contexts1.h:303,322), register-blocked: eight rows of
 * X are applied to a row of the local block at a time, so that each element of the block is read
 * and written once per eight rank-1 updates.  Each thread sums runs of 1024 rows in fp32; the
 * runs are combined in fp64. */
#define ORC_RB 8
static void gram_f32(int64_t rows, int r, const float* X, float* G) {
  double* acc = (double*)calloc((size_t)r * r, sizeof(double));
#pragma omp parallel
  {
    float* loc = (float*)malloc(sizeof(float) * r * r);
    double* mine = (double*)calloc((size_t)r * r, sizeof(double));
    const int64_t blk = 1024;
#pragma omp for schedule(static)
    for (int64_t k0 = 0; k0 < rows; k0 += blk) {
      int64_t k1 = k0 + blk < rows ? k0 + blk : rows;
      for (int i = 0; i < r * r; i++) loc[i] = 0.0f;
      int64_t k = k0;
      for (; k + ORC_RB <= k1; k += ORC_RB) {
        const float* x0 = X + k * r;
        const float *x1 = x0 + r, *x2 = x1 + r, *x3 = x2 + r, *x4 = x3 + r, *x5 = x4 + r,
                    *x6 = x5 + r, *x7 = x6 + r;
        for (int a = 0; a < r; a++) {
          const float a0 = x0[a], a1 = x1[a], a2 = x2[a], a3 = x3[a], a4 = x4[a], a5 = x5[a],
                      a6 = x6[a], a7 = x7[a];
          float* l = loc + a * r;
#pragma omp simd
          for (int b = 0; b < r; b++)
            l[b] += ((a0 * x0[b] + a1 * x1[b]) + (a2 * x2[b] + a3 * x3[b])) +
                    ((a4 * x4[b] + a5 * x5[b]) + (a6 * x6[b] + a7 * x7[b]));
        }
      }
      for (; k < k1; k++) {
        const float* x = X + k * r;
        for (int a = 0; a < r; a++) {
          float xa = x[a];
          float* l = loc + a * r;
#pragma omp simd
          for (int b = 0; b < r; b++) l[b] += xa * x[b];
        }
      }
      for (int i = 0; i < r * r; i++) mine[i] += (double)loc[i];
    }
#pragma omp critical
    for (int i = 0; i < r * r; i++) acc[i] += mine[i];
    free(loc);
    free(mine);
  }
  for (int i = 0; i < r * r; i++) G[i] = (float)acc[i];
  free(acc);
}

/* X <- X * num / (X G + eps) (cublasSgemm + kernelNmfMuUpdate, device_contexts1.h:306-308,
 * 329-332), eight rows at a time so that a row of G is loaded once per eight rows of X; fused
 * like the device path. */
static void xg_mu_f32(int64_t rows, int r, float* X, const float* G, const float* num,
                      float eps) {
#pragma omp parallel
  {
    float* d = (float*)malloc(sizeof(float) * r * ORC_RB);
#pragma omp for schedule(static)
    for (int64_t k0 = 0; k0 < rows; k0 += ORC_RB) {
      const int nb = rows - k0 < ORC_RB ? (int)(rows - k0) : ORC_RB;
      for (int i = 0; i < r * ORC_RB; i++) d[i] = 0.0f;
      if (nb == ORC_RB) {
        const float* x0 = X + k0 * r;
        for (int a = 0; a < r; a++) {
          const float* g = G + a * r;
          const float a0 = x0[a], a1 = x0[r + a], a2 = x0[2 * r + a], a3 = x0[3 * r + a],
                      a4 = x0[4 * r + a], a5 = x0[5 * r + a], a6 = x0[6 * r + a], a7 = x0[7 * r + a];
          float *d0 = d, *d1 = d + r, *d2 = d + 2 * r, *d3 = d + 3 * r, *d4 = d + 4 * r,
                *d5 = d + 5 * r, *d6 = d + 6 * r, *d7 = d + 7 * r;
#pragma omp simd
          for (int b = 0; b < r; b++) {
            const float gb = g[b];
            d0[b] += a0 * gb; d1[b] += a1 * gb; d2[b] += a2 * gb; d3[b] += a3 * gb;
            d4[b] += a4 * gb; d5[b] += a5 * gb; d6[b] += a6 * gb; d7[b] += a7 * gb;
          }
        }
      } else {
        for (int q = 0; q < nb; q++) {
          const float* x = X + (k0 + q) * r;
          float* dq = d + q * r;
          for (int a = 0; a < r; a++) {
            const float xa = x[a];
            const float* g = G + a * r;
#pragma omp simd
            for (int b = 0; b < r; b++) dq[b] += xa * g[b];
          }
        }
      }
      for (int q = 0; q < nb; q++) {
        float* x = X + (k0 + q) * r;
        const float* nu = num + (k0 + q) * r;
        const float* dq = d + q * r;
#pragma omp simd
        for (int b = 0; b < r; b++) x[b] *= nu[b] / (dq[b] + eps);
      }
    }
    free(d);
  }
}

/* Create the fp32 baseline context; W [n, r] and H [r, m] row-major initial
 * factors are copied in.  Returns an opaque pointer. */
ORC_API void* orc_f32_create(int64_t n, int64_t m, const int64_t* rowptr, const int32_t* colind,
                             const float* vals, int r, float eps, const float* W,
                             const float* H_rm) {
  orc_f32_ctx* c = (orc_f32_ctx*)calloc(1, sizeof(orc_f32_ctx));
  c->n = n; c->m = m; c->nnz = rowptr[n]; c->r = r; c->eps = eps;
  c->rowptr = rowptr; c->colind = colind; c->vals = vals;
  int64_t big = n > m ? n : m;
  c->colptr = (int64_t*)malloc(sizeof(int64_t) * (m + 1));
  c->rowind = (int32_t*)malloc(sizeof(int32_t) * (c->nnz > 0 ? c->nnz : 1));
  c->tvals = (float*)malloc(sizeof(float) * (c->nnz > 0 ? c->nnz : 1));
  orc_transpose(n, m, rowptr, colind, vals, c->colptr, c->rowind, c->tvals);
  c->W = (float*)malloc(sizeof(float) * n * r);
  c->Ht = (float*)malloc(sizeof(float) * m * r);
  c->num = (float*)malloc(sizeof(float) * big * r);
  c->G = (float*)malloc(sizeof(float) * r * r);
  memcpy(c->W, W, sizeof(float) * n * r);
#pragma omp parallel for schedule(static)
  for (int64_t j = 0; j < m; j++)
    for (int k = 0; k < r; k++) c->Ht[j * r + k] = H_rm[(int64_t)k * m + j];
  double sq = 0.0;
  for (int64_t e = 0; e < c->nnz; e++) sq += (double)vals[e] * (double)vals[e];
  c->sq_norm_A = sq;
  return c;
}

/* Same, but H is drawn inside (value_at callback-free): Ht[j*r+k] = init_H[j*r+k]
 * given directly in the [m, r] layout, avoiding an [r, m] staging copy. */
ORC_API void* orc_f32_create_mr(int64_t n, int64_t m, const int64_t* rowptr,
                                const int32_t* colind, const float* vals, int r, float eps,
                                const float* W, const float* Ht_mr) {
  orc_f32_ctx* c = (orc_f32_ctx*)calloc(1, sizeof(orc_f32_ctx));
  c->n = n; c->m = m; c->nnz = rowptr[n]; c->r = r; c->eps = eps;
  c->rowptr = rowptr; c->colind = colind; c->vals = vals;
  int64_t big = n > m ? n : m;
  c->colptr = (int64_t*)malloc(sizeof(int64_t) * (m + 1));
  c->rowind = (int32_t*)malloc(sizeof(int32_t) * (c->nnz > 0 ? c->nnz : 1));
  c->tvals = (float*)malloc(sizeof(float) * (c->nnz > 0 ? c->nnz : 1));
  orc_transpose(n, m, rowptr, colind, vals, c->colptr, c->rowind, c->tvals);
  c->W = (float*)malloc(sizeof(float) * n * r);
  c->Ht = (float*)malloc(sizeof(float) * m * r);
  c->num = (float*)malloc(sizeof(float) * big * r);
  c->G = (float*)malloc(sizeof(float) * r * r);
  memcpy(c->W, W, sizeof(float) * n * r);
  memcpy(c->Ht, Ht_mr, sizeof(float) * m * r);
  c->sq_norm_A = 0.0;
  for (int64_t e = 0; e < c->nnz; e++) c->sq_norm_A += (double)vals[e] * (double)vals[e];
  return c;
}

/* One MU iteration in the reference order (W-update, then H-update). */
ORC_API void orc_f32_step(void* ctx, int n_steps) {
  orc_f32_ctx* c = (orc_f32_ctx*)ctx;
  for (int s = 0; s < n_steps; s++) {
    spmm_n_f32(c, c->num);
    gram_f32(c->m, c->r, c->Ht, c->G);
    xg_mu_f32(c->n, c->r, c->W, c->G, c->num, c->eps);
    spmm_t_f32(c, c->num);
    gram_f32(c->n, c->r, c->W, c->G);
    xg_mu_f32(c->m, c->r, c->Ht, c->G, c->num, c->eps);
  }
}

static double orc_now(void) {
#ifdef _OPENMP
  return omp_get_wtime();
#else
  return (double)clock() / CLOCKS_PER_SEC;
#endif
}

/* The same iteration with the seconds spent in each part added to secs[0..5]:
 * A H^T, H^T H, W update, A^T W, W^T W, H update. */
ORC_API void orc_f32_step_timed(void* ctx, int n_steps, double* secs) {
  orc_f32_ctx* c = (orc_f32_ctx*)ctx;
  for (int s = 0; s < n_steps; s++) {
    double t0 = orc_now(), t1;
    spmm_n_f32(c, c->num);
    t1 = orc_now(); secs[0] += t1 - t0; t0 = t1;
    gram_f32(c->m, c->r, c->Ht, c->G);
    t1 = orc_now(); secs[1] += t1 - t0; t0 = t1;
    xg_mu_f32(c->n, c->r, c->W, c->G, c->num, c->eps);
    t1 = orc_now(); secs[2] += t1 - t0; t0 = t1;
    spmm_t_f32(c, c->num);
    t1 = orc_now(); secs[3] += t1 - t0; t0 = t1;
    gram_f32(c->n, c->r, c->W, c->G);
    t1 = orc_now(); secs[4] += t1 - t0; t0 = t1;
    xg_mu_f32(c->m, c->r, c->Ht, c->G, c->num, c->eps);
    t1 = orc_now(); secs[5] += t1 - t0;
  }
}

/* fp32 OpenMP port of the first stage of the learner for timing: out[n, r] = A B^T with B given
 * by its transposed CSR (per column: component ids and values), the product loop of
 * Partitioned_SpSpMatmul_ToDense (cuda/ops/spsp_matmul.h:95-131).  Returns the seconds taken. */
ORC_API double orc_f32_spsp_timed(int64_t n, const int64_t* a_rowptr, const int32_t* a_colind,
                                  const float* a_vals, int r, const int64_t* b_colptr,
                                  const int32_t* b_comp, const float* b_tvals, float* out_nr) {
  const double t0 = orc_now();
#pragma omp parallel for schedule(dynamic, 4)
  for (int64_t i = 0; i < n; i++) {
    float* o = out_nr + i * r;
    for (int c = 0; c < r; c++) o[c] = 0.0f;
    for (int64_t e = a_rowptr[i]; e < a_rowptr[i + 1]; e++) {
      const int64_t j = a_colind[e];
      const float a = a_vals[e];
      for (int64_t p = b_colptr[j]; p < b_colptr[j + 1]; p++) o[b_comp[p]] += a * b_tvals[p];
    }
  }
  return orc_now() - t0;
}

/* fp32 port of the learner's second stage for timing: n_steps of W <- W * AH / (W HH + eps). */
ORC_API double orc_f32_fit_steps_timed(int64_t n, int r, const float* AH, const float* HH, float eps,
                                       int n_steps, float* W) {
  const double t0 = orc_now();
  for (int s = 0; s < n_steps; s++) xg_mu_f32(n, r, W, HH, AH, eps);
  return orc_now() - t0;
}

ORC_API void orc_f32_get(void* ctx, float* W, float* H_rm) {
  orc_f32_ctx* c = (orc_f32_ctx*)ctx;
  if (W) memcpy(W, c->W, sizeof(float) * c->n * c->r);
  if (H_rm)
    for (int64_t j = 0; j < c->m; j++)
      for (int k = 0; k < c->r; k++) H_rm[(int64_t)k * c->m + j] = c->Ht[j * c->r + k];
}

ORC_API void orc_f32_destroy(void* ctx) {
  orc_f32_ctx* c = (orc_f32_ctx*)ctx;
  free(c->colptr); free(c->rowind); free(c->tvals);
  free(c->W); free(c->Ht); free(c->num); free(c->G);
  free(c);
}

/* The sparseness projection of the columns of a row-major factor W [n, r], in place; returns the
 * largest number of passes any column took.  One column at a time (the reference steps all
 * columns together and leaves those without negative entries alone: the same values).
 * DenseFactorSparsityContext::sparsifyF, cc/cuda_d_npeff/src/nmf/sparse/
 * dense_factor_sparsity_constraints.h:205-237; element arithmetic of
 * sparsity_constraint_kernels.h:16-141 in fp32; the column sums (cublasSgemv /
 * cublasSgemmStridedBatched there, :405-452) in fp64, rounded to fp32. */
ORC_API int orc_sparsify_columns(int64_t n, int r, float* W, float l1, float l2) {
  int most = 0;
  float* s = (float*)malloc(sizeof(float) * (size_t)n);
  float* y = (float*)malloc(sizeof(float) * (size_t)n);
  for (int c = 0; c < r; c++) {
    double acc = 0.0;
    for (int64_t i = 0; i < n; i++) { s[i] = W[i * r + c]; y[i] = 1.0f; acc += (double)s[i]; } /* :240-257 */
    const float sum_x = (float)acc;
    for (int64_t i = 0; i < n; i++) s[i] += (l1 - sum_x) / (float)n; /* kernel_computeInitialS :16-27 */
    int passes = 0;
    for (;;) {
      passes++;
      double yy_d = 0.0, ss_d = 0.0, sy_d = 0.0; /* :222, :281-286 */
      for (int64_t i = 0; i < n; i++) {
        yy_d += (double)y[i];
        ss_d += (double)(s[i] * s[i]);
        sy_d += (double)(s[i] * y[i]);
      }
      const float YY = (float)yy_d, SS = (float)ss_d, SY = (float)sy_d;
      /* kernel_computeAlpha :41-66 */
      const float L2 = sqrtf(l2 * l2);
      const float beta = l1 / YY;
      const float m2 = beta * beta * YY;
      const float ms = beta * SY;
      const float m_s_2 = fmaxf(1e-9f, beta * beta * YY + SS - 2.0f * beta * SY);
      const float alpha = (L2 * sqrtf(m_s_2) + m2 - ms) / m_s_2;
      /* kernel_updateSAfterAlpha :69-88 */
      int64_t negative = 0;
      for (int64_t i = 0; i < n; i++) {
        const float m = y[i] * l1 / YY;
        const float v = m + alpha * (s[i] - m);
        s[i] = v;
        negative += v < 0.0f;
      }
      if (negative == 0) break; /* :352-374 */
      /* kernel_updateYAndS :91-113 */
      for (int64_t i = 0; i < n; i++) {
        if (y[i] != 0.0f && s[i] < 0.0f) y[i] = 0.0f;
        if (y[i] == 0.0f) s[i] = 0.0f;
      }
      /* kernel_updateSLastStep :116-141 with the sums of :391-392 */
      double sum_s = 0.0, sum_y = 0.0;
      for (int64_t i = 0; i < n; i++) { sum_s += (double)s[i]; sum_y += (double)y[i]; }
      const float cshift = ((float)sum_s - l1) / (float)sum_y;
      for (int64_t i = 0; i < n; i++)
        if (y[i] != 0.0f) s[i] -= cshift;
      if (passes > n + 1) break; /* cannot happen: every pass fixes one more entry at zero */
    }
    for (int64_t i = 0; i < n; i++) W[i * r + c] = s[i];
    if (passes > most) most = passes;
  }
  free(s);
  free(y);
  return most;
}

ORC_API int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
