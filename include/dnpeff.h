/*
 * dnpeff.h -- C ABI of the MI355X D-NPEFF NMF library (libdnpeff_hip.so).
 *
 * Plain pointers and sizes only.  Every function returns 0 on success and a
 * non-zero status on failure; dnpeff_last_error() then holds a message.  The
 * reference aborts the process on every error (print + bare `throw;`,
 * cc/cuda_d_npeff/src/cuda/cuda_statuses.h:15-38); hosts that want that
 * behaviour turn a non-zero status into message + abort.
 *
 * Storage conventions
 *   - A is CSR with 64-bit row offsets and 32-bit column ids.
 *   - Host-visible W is [n, r] row-major, host-visible H is [r, m] row-major:
 *     the layouts the reference writes to "data/W" and "data/H"
 *     (cc/cuda_d_npeff/src/io/nmf_decomp_h5.h:38-56).
 *   - On the device both factors are kept "tall and skinny" with the r
 *     components of one row/column contiguous: W as [n, r], H as [m, r].
 *     [m, r] row-major is byte-for-byte the reference's column-major r x m H
 *     (multi_mu_dense_factors_device_contexts1.h:158).  Entry points that take
 *     device factor pointers (dnpeff_op_*) use this device layout.
 *
 * Threading: handles are not thread safe; one host thread drives one handle.
 * All work of the library runs on one HIP stream of default priority.
 */
#ifndef DNPEFF_H_
#define DNPEFF_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct dnpeff_csr dnpeff_csr; /* device-resident CSR matrix + loader state   */
typedef struct dnpeff_nmf dnpeff_nmf; /* dense-factor MU NMF (MuNmf + DeviceContext)  */
typedef struct dnpeff_fit dnpeff_fit; /* fixed sparse-H, W-only learner (Learner)     */

/* ------------------------------------------------------------------------- */
/* Library state                                                              */
/* ------------------------------------------------------------------------- */

/* Message of the last failing call on this thread ("" if none). */
const char* dnpeff_last_error(void);

/* Number of visible GPUs.  Replaces cudaGetDeviceCount at
 * cc/cuda_d_npeff/mains/run_nmf_on_pefs.cu:126 and Cuda::GetDeviceCount at
 * cc/cuda_d_npeff/mains/fit_coeffs_to_sparse_H.cu:74-78. */
int dnpeff_device_count(int* count);

/* Name and total memory of device 0. */
int dnpeff_device_info(char* name, int name_len, int64_t* total_bytes, int* n_cus);

/* Block until everything queued on the library's stream has finished
 * (cudaStreamSynchronize, multi_mu_dense_factors_nmf1.h:351-356). */
int dnpeff_sync(void);

/* Library stream as a hipStream_t, for callers that order their own work. */
void* dnpeff_stream(void);

/* Free and total memory of the current device in bytes (hipMemGetInfo); either pointer may be
 * NULL.  The reference prints the same figures through NVML
 * (cc/cuda_d_npeff/src/cuda/debugging/). */
int dnpeff_device_memory(int64_t* free_bytes, int64_t* total_bytes);

/* The byte table behind the memory plan of dnpeff_nmf_create, computable without a GPU (capacity
 * planning, tests): for a matrix of n_rows x n_cols whose sparse part holds nnz_sparse entries
 * and whose dense head holds n_dense columns, at the given rank, with the tiled (1) or full-size
 * (0) H update, on a device of total_bytes; sweeps = 1 when A H^T has swept pieces (ranks 32, 64,
 * 128, 256 and multiples of 128 above, on a device whose workgroups go to the XCDs round-robin).
 * out[0..7] = factors and their workspaces, partial sums of A H^T, segment offsets, column/row
 * offsets, reserve left free, both sparse copies, dense blocks of the head, workspace of the
 * head's products; all in bytes, upper bounds from the rules that size the allocations.  The
 * reference sizes its buffers inside the constructor
 * (multi_mu_dense_factors_device_contexts1.h:128-200) and has no such call. */
int dnpeff_plan_estimate(int64_t n_rows, int64_t n_cols, int64_t nnz_sparse, int64_t n_dense, int rank,
                         int tiled, int sweeps, int64_t total_bytes, double* out);

/* Switches for experiments and for tests that must reach a particular code path; no counterpart
 * in the reference.  Names: dense_fill, panels, sweep_bytes, sweep_min, sweep_waves, sweep_lag,
 * sweep_spin, spmm_t_slices, split_bf16, fused_gram, h_tile_mb, tiled_h, topk_fast_cap, verbose,
 * h_overlap (1: tiled H update with A^T W of the next tile on the library stream beside the
 * update of this tile on a second stream, through two tile buffers; off by default),
 * xg_wgs (3: the update kernel of ranks from 256 with three workgroups per CU on LDS planes
 * without padding where the launch fills the CUs eight times over; 4: always; 2: two, on padded
 * planes with two operand stages),
 * gram_beside (1: H^T H of the W update on a second stream with the dense head of A H^T behind
 * it; 0: after A H^T on the library stream), gram_fold (2: X^T X with
 * its diagonal squares of 256 columns each in one workgroup where the rank is a multiple of 256;
 * 1: diagonal tiles of 128 columns with their symmetry used; 0: without), n_lists (A H^T from slot lists on component slices of 32: -1 =
 * the far tail of the sparse part where that was measured to pay, 2 = wherever possible, 1 = the
 * whole sparse part, 0 = never), t_lists (1: A^T W in column blocks on such slices), nl_piece_cols,
 * nl_lag, nl_spin, nl_wgs (their piece size, lock step and launch shape), nl_extra_mb (memory the
 * far tail's lists may take beyond the panel copy they replace).
 * Each starts from the environment variable DNPEFF_<NAME IN CAPITALS> (read once, when the
 * library is first used) or its default; plans take the values when they are made
 * (dnpeff_nmf_create, the first product on a matrix).  dnpeff_tuning_reset() goes back to the
 * starting values.  An unknown name is an error. */
int dnpeff_tuning_set(const char* name, double value);
int dnpeff_tuning_get(const char* name, double* value);
int dnpeff_tuning_reset(void);

/* Plain device buffers for callers of the dnpeff_op_* entry points that have
 * no device allocator of their own (DeviceCudaContext::dmalloc / dfree and the
 * copies of cc/cuda_d_npeff/src/cuda/cuda_context.h:58-69, transfers.h).
 * Copies wait for the library stream first and are synchronous. */
int dnpeff_dev_malloc(int64_t bytes, void** out);
int dnpeff_dev_free(void* p);
int dnpeff_dev_upload(void* dst_dev, const void* src_host, int64_t bytes);
int dnpeff_dev_download(void* dst_host, const void* src_dev, int64_t bytes);

/* ------------------------------------------------------------------------- */
/* Loader: CSR on the device, row normalisation, column compaction            */
/* ------------------------------------------------------------------------- */

/* Upload a host CSR matrix.  Replaces ElCsrMatrix<IndT> + moveAToDeviceAsync
 * (cc/cuda_d_npeff/src/util/matrices.h:172-199;
 * multi_mu_dense_factors_device_contexts1.h:182-195).  Column ids inside a row
 * need not be sorted.  Host buffers are only read during the call. */
int dnpeff_csr_from_host(int64_t n_rows, int64_t n_cols, int64_t nnz,
                         const int64_t* rowptr, const int32_t* colind,
                         const float* vals, dnpeff_csr** out);

/* Build the CSR matrix of a fixed-width PEF block: values/indices are
 * [n_rows, k] row-major, row offsets are i*k.  Replaces
 * PefSparseFishers<IndT>::read's construction
 * (cc/cuda_d_npeff/src/io/pef_fisher_h5.h:170-177). */
int dnpeff_csr_from_pef(int64_t n_rows, int64_t k, int64_t dense_fisher_size,
                        const int32_t* indices, const float* values,
                        dnpeff_csr** out);

/* vals[row] /= (norms[row] + eps), fp32.  Replaces normalizeFishers_inPlace
 * (cc/cuda_d_npeff/src/io/pef_fisher_h5.h:38-52; eps default 1e-9f there). */
int dnpeff_csr_normalize_rows(dnpeff_csr* A, const float* norms_host, float eps);

/* Drop every column with fewer than min_count entries and renumber the rest in
 * ascending original order; entries of dropped columns are removed, in-row
 * order is kept.  Bit-exact replacement of removeSmallestL0NormColumns_inPlace
 * (cc/cuda_d_npeff/src/util/sparse_util.h:78-159).  Afterwards
 * dnpeff_csr_kept_indices returns newToOgIndex. */
int dnpeff_csr_compact_columns(dnpeff_csr* A, int min_count);

/* Keep only entries whose column id appears in kept[0..n_kept) and renumber
 * them to their position in kept.  Bit-exact replacement of
 * Cuda::Host::CsrMatrix::RetainColumns_InPlace
 * (cc/cuda_d_npeff/src/cuda/host/sparse_matrix.h:141-170). */
int dnpeff_csr_retain_columns(dnpeff_csr* A, const int32_t* kept, int64_t n_kept);

int dnpeff_csr_shape(const dnpeff_csr* A, int64_t* n_rows, int64_t* n_cols, int64_t* nnz);

/* Column count before the last compaction (fisherDenseSize,
 * cc/cuda_d_npeff/mains/run_nmf_on_pefs.cu:174). */
int dnpeff_csr_full_dense_size(const dnpeff_csr* A, int64_t* out);

/* Copy the matrix back: rowptr[n_rows+1], colind[nnz], vals[nnz]; any pointer
 * may be NULL to skip that array. */
int dnpeff_csr_download(const dnpeff_csr* A, int64_t* rowptr, int32_t* colind, float* vals);

/* newToOgIndex[n_cols] of the last compact/retain call (identity if none). */
int dnpeff_csr_kept_indices(const dnpeff_csr* A, int32_t* new_to_og);

/* Sum of squares of all values, accumulated in fp64.  Replaces
 * computeASqNorm (multi_mu_dense_factors_device_contexts1.h:274-294) and
 * ComputeAndAccumulate_SquaredNormA (nmf/sparse2/nmf_sparse_H.h:250-262). */
int dnpeff_csr_sq_norm(const dnpeff_csr* A, double* out);

/* Build (once) the transposed CSR on the device: column offsets, and per
 * column the (row, value) pairs in ascending row order.  Deterministic
 * replacement of CsrTranspose (cc/cuda_d_npeff/src/cuda/ops/transpose.h:170-439). */
int dnpeff_csr_build_transpose(dnpeff_csr* A);

/* Split off the dense head: every column held by at least ceil(min_fill * n_rows) rows
 * leaves the sparse structures and is stored as a dense block, so that its share of A H^T and
 * A^T W runs as a matrix product on the matrix cores; the other entries stay sparse.  The
 * products of the split matrix are the same sums in another order; they then need a rank that
 * is a multiple of 4.  dnpeff_csr_download and the loader calls still see the whole matrix;
 * any call that edits the matrix undoes the split.  The threshold is raised until both dense
 * blocks fit an eighth of the device memory.  min_fill <= 0 removes the split.  n_dense (may
 * be NULL) receives the number of columns in the head.  A matrix in which a row holds the same
 * column twice is refused by the products (dnpeff_csr_build_transpose reports it).
 * No counterpart in the reference, which hands the whole matrix to cusparseSpMM
 * (device_contexts1.h:255-265); dnpeff_nmf_create applies it by itself (fill 1/16, rank >= 64
 * and a multiple of 4, at least 1024 rows) unless the caller has split the matrix already. */
int dnpeff_csr_split_dense_head(dnpeff_csr* A, double min_fill, int64_t* n_dense);

/* Columns in the dense head (0 = not split) and entries left in the sparse part. */
int dnpeff_csr_head_info(const dnpeff_csr* A, int64_t* n_dense, int64_t* nnz_sparse);

/* How the sparse part is organised for A H^T once a product or a context has planned it:
 * out6 = column panels, of which plain, swept pieces, first column of the far tail that runs from
 * slot lists (0 = none), entries and batches of 64 in the slot lists (0 = none).  No counterpart in
 * the reference (cusparseSpMM_preprocess, device_contexts1.h:255-265, keeps its plan to itself). */
int dnpeff_csr_products_info(const dnpeff_csr* A, int64_t* out6);

/* Copy the transposed CSR back: colptr[n_cols+1], rowind[nnz], vals[nnz]. */
int dnpeff_csr_download_transpose(dnpeff_csr* A, int64_t* colptr, int32_t* rowind, float* vals);

/* One row / one column of the matrix as the products hold it (dense head block plus sparse
 * part), to the host: *count receives the number of entries; cols/rows and vals (may be NULL
 * to ask for the count only) must hold cap >= count entries.  Order: head entries first, then
 * the sparse part's (a row: in its stored order; a column: ascending rows).  Works on a matrix
 * consumed by dnpeff_nmf_create_ex.  Counterpart of the inspection helpers of
 * cc/cuda_d_npeff/src/util/matrices.h:258-324 (asDenseMatrix / areEqual), for validation. */
int dnpeff_csr_get_row(dnpeff_csr* A, int64_t row, int64_t cap, int64_t* count, int32_t* cols,
                       float* vals);
int dnpeff_csr_get_column(dnpeff_csr* A, int64_t col, int64_t cap, int64_t* count, int32_t* rows,
                          float* vals);

/* Release the arrays that only dnpeff_op_spmm_n / dnpeff_nmf_* need (row-major
 * copy) or only spmm_t needs (transposed copy).  which: 1 = row-major copy,
 * 2 = transposed copy. */
int dnpeff_csr_release(dnpeff_csr* A, int which);

int dnpeff_csr_destroy(dnpeff_csr* A);

/* Contiguous split sizes: total/n_splits each, remainder added to the last.
 * Replaces getSizeOfSplit (cc/cuda_d_npeff/src/util/matrix_util.h:10-21) and
 * CsrMatrix::GetSizeOfSplit (cuda/host/sparse_matrix.h:107-117).  Returns -1
 * for split_index >= n_splits (the reference throws). */
int64_t dnpeff_size_of_split(int64_t total, int64_t n_splits, int64_t split_index);

/* ------------------------------------------------------------------------- */
/* Synthetic PEF generator (benchmark / test inputs, not part of the reference)*/
/* ------------------------------------------------------------------------- */

/* Per row i: k_i distinct column ids by successive Zipf(s) draws over
 * [0, n_cols) rejecting duplicates, draw order kept; values exp(N(mu, sigma^2))
 * in fp32.  k_i = k_fixed, or, when k_min > 0, round(exp(U(ln k_min, ln k_max))).
 * norms_out_host[n_rows] (may be NULL) receives the fp32 L2 norm of each row
 * so that dnpeff_csr_normalize_rows L2-normalises it. */
int dnpeff_synth_pef(int64_t n_rows, int64_t n_cols, int64_t k_fixed,
                     int64_t k_min, int64_t k_max, double zipf_s,
                     double mu, double sigma, uint64_t seed,
                     float* norms_out_host, dnpeff_csr** out);

/* Same generator on the host, one thread; arrays sized by the caller
 * (rowptr[n_rows+1] is written first when colind == NULL so the caller can
 * size colind/vals). */
int dnpeff_synth_pef_host(int64_t n_rows, int64_t n_cols, int64_t k_fixed,
                          int64_t k_min, int64_t k_max, double zipf_s,
                          double mu, double sigma, uint64_t seed,
                          int64_t* rowptr, int32_t* colind, float* vals,
                          float* norms);

/* Rows [row0, row0 + n_rows) of the matrix that dnpeff_synth_pef makes for the same other
 * arguments (rows are keyed by their absolute number), for checks of a large device-made matrix
 * on sampled rows; rowptr[n_rows + 1] is relative to the first of these rows. */
int dnpeff_synth_pef_host_rows(int64_t row0, int64_t n_rows, int64_t n_cols, int64_t k_fixed,
                               int64_t k_min, int64_t k_max, double zipf_s, double mu, double sigma,
                               uint64_t seed, int64_t* rowptr, int32_t* colind, float* vals,
                               float* norms);

/* U[0,1) initial factor value of logical element (row, col) of matrix
 * matrix_id (0 = W [n, r], 1 = H [r, m]); host mirror of the device
 * initialiser.  Replaces curandGenerateUniform
 * (multi_mu_dense_factors_device_contexts1.h:197-207). */
float dnpeff_uniform_at(uint64_t seed, int matrix_id, int64_t row, int64_t col, int64_t n_cols);

/* ------------------------------------------------------------------------- */
/* Dense-factor MU NMF (run_nmf_on_pefs hot loop)                             */
/* ------------------------------------------------------------------------- */

/* Create the context for A ~= W H with W [n, r], H [r, m].  Builds the
 * transposed CSR, allocates W, H and one [max(n, m), r] scratch, computes
 * ||A||^2.  A stays owned by the caller and must outlive the context.
 * Replaces MuNmf<IndT>::MuNmf + DeviceContext ctor
 * (multi_mu_dense_factors_nmf1.h:81-122;
 * multi_mu_dense_factors_device_contexts1.h:129-170,384-434).
 * Like the reference it refuses n_rows > n_cols. */
int dnpeff_nmf_create(dnpeff_csr* A, int rank, float eps, int64_t seed, dnpeff_nmf** out);

/* The same with flags.  DNPEFF_NMF_CONSUME_MATRIX: the context may free every array of A that
 * its products do not read (the caller's row-major arrays once the dense head, the transposed
 * copy and the regrouped copy exist), as the reference's host matrix can be dropped once
 * moveAToDeviceAsync has copied it (device_contexts1.h:182-195).  Afterwards A still answers
 * dnpeff_csr_shape, dnpeff_csr_kept_indices and dnpeff_csr_full_dense_size and serves this and
 * later contexts of the same rank, but dnpeff_csr_download and the loader calls fail with an
 * error.  This is what lets a matrix whose copies and factors fill the device fit.
 * When a second [m, r] array does not fit beside H, the context updates H on column tiles
 * (A^T W of a tile, then the tile's update) with the same results. */
enum { DNPEFF_NMF_CONSUME_MATRIX = 1 };
int dnpeff_nmf_create_ex(dnpeff_csr* A, int rank, float eps, int64_t seed, unsigned flags,
                         dnpeff_nmf** out);

/* Whether the context updates H on column tiles, and the tile width in columns (0 if not). */
int dnpeff_nmf_info(const dnpeff_nmf* nmf, int* tiled, int64_t* tile_cols);

/* W then H ~ U[0,1) from the seed (initializeW / initializeH,
 * multi_mu_dense_factors_device_contexts1.h:197-233). */
int dnpeff_nmf_init_factors(dnpeff_nmf* nmf);

/* Load caller-chosen factors: W [n, r] row-major, H [r, m] row-major (either
 * may be NULL to keep the current one). */
int dnpeff_nmf_set_factors(dnpeff_nmf* nmf, const float* W_nr, const float* H_rm);

/* n_steps iterations of: W-update, then H-update with the new W
 * (MuNmf::run loop body, multi_mu_dense_factors_nmf1.h:175-182).  Returns
 * without waiting for the device. */
int dnpeff_nmf_step(dnpeff_nmf* nmf, int n_steps);

/* W <- W * (A H^T) / (W (H H^T) + eps)   (updateW, nmf1.h:293-305). */
int dnpeff_nmf_update_W(dnpeff_nmf* nmf);
/* H <- H * (W^T A) / ((W^T W) H + eps)   (updateH, device_contexts1.h:296-309). */
int dnpeff_nmf_update_H(dnpeff_nmf* nmf);

/* sqrt(||A||^2 + <W^T W, H H^T> - 2 <A H^T, W>) with fp64 accumulation of the
 * reductions: the quantity of computeUncachedLoss (nmf1.h:242-274,
 * device_contexts1.h:337-354) through the same trace identity. */
int dnpeff_nmf_loss(dnpeff_nmf* nmf, double* out);

/* The three terms of the loss: ||A||^2, <H,(W^T W)H>, <W^T A,H>. */
int dnpeff_nmf_loss_terms(dnpeff_nmf* nmf, double* sq_norm_A, double* pos, double* neg);

/* Consistency of the two sparse products on the current factors: <A H^T, W> computed through
 * the row-ordered structures (the kernels of the W update) and <A^T W, H> through the
 * column-ordered ones (the kernels of the H update, tile by tile when H is updated so).  The
 * two are the same number, the third term of the loss (multi_mu_dense_factors_nmf1.h:270-273);
 * an entry lost, doubled or misplaced in either copy of the matrix makes them differ.  Costs one
 * A H^T and one A^T W; does not change the factors. */
int dnpeff_nmf_check_products(dnpeff_nmf* nmf, double* via_rows, double* via_columns);

/* The sparseness projection of the columns of W that the reference builds for --sparsity_W and
 * never runs: sparseContextW->sparsifyF() (dense_factor_sparsity_constraints.h:205-237; the one
 * call, at multi_mu_dense_factors_nmf1.h:161-162, is commented out, and so no loop of this
 * library calls it either).  l1_norm is FactorSparsenessConstraints::l1_norm (the flag's value),
 * l2_norm its l2_norm (1 in the reference).  *rounds (may be NULL) receives the number of passes of
 * its loop.  See dnpeff_op_sparsify_columns. */
int dnpeff_nmf_sparsify_W(dnpeff_nmf* nmf, float l1_norm, float l2_norm, int* rounds);

/* Copy the factors to the host in the output-file layout: W [n, r] row-major
 * (loadWToHostSync + toRowMajor_inPlace, nmf1.h:207-220, matrices.h:49-62),
 * H [r, m] row-major (loadHToHostSync + toRowMajor_inPlace, nmf1.h:222-240). */
int dnpeff_nmf_get_W(dnpeff_nmf* nmf, float* W_nr);
int dnpeff_nmf_get_H(dnpeff_nmf* nmf, float* H_rm);

/* Device pointers of W [n, r] and H [m, r] (device layout). */
int dnpeff_nmf_device_factors(dnpeff_nmf* nmf, void** W_dev, void** H_dev);

/* Per-kernel timing with HIP events on the library stream.  enable != 0 turns
 * it on for subsequent steps; dnpeff_nmf_timings waits for the stream and
 * returns, per kernel class, summed milliseconds and launch counts since the
 * last reset.  Classes (DNPEFF_K_*) below. */
enum {
  DNPEFF_K_SPMM_N = 0,   /* A H^T                     */
  DNPEFF_K_SPMM_N_REDUCE = 1,
  DNPEFF_K_GRAM_H = 2,   /* H H^T  (k = m)            */
  DNPEFF_K_XG_MU_W = 3,  /* W (H H^T) fused with MU   */
  DNPEFF_K_SPMM_T = 4,   /* A^T W                     */
  DNPEFF_K_GRAM_W = 5,   /* W^T W  (k = n)            */
  DNPEFF_K_XG_MU_H = 6,  /* (W^T W) H fused with MU   */
  DNPEFF_K_COUNT = 7
};
int dnpeff_nmf_set_profiling(dnpeff_nmf* nmf, int enable);
int dnpeff_nmf_timings(dnpeff_nmf* nmf, double* ms_sum /*[DNPEFF_K_COUNT]*/,
                       int64_t* launches /*[DNPEFF_K_COUNT]*/, int reset);

int dnpeff_nmf_destroy(dnpeff_nmf* nmf);

/* ------------------------------------------------------------------------- */
/* Fixed sparse H, W-only learner (fit_coeffs_to_sparse_H)                    */
/* ------------------------------------------------------------------------- */

/* Stage 1: H H^T (r x r) and A H^T (n x r) from sparse A [n, m] and sparse H
 * [r, m], plus ||A||^2.  Replaces Learner::RunFirstStage
 * (cc/cuda_d_npeff/src/nmf/sparse2/nmf_sparse_H.h:157-292;
 * cuda/ops/spsp_matmul.h:95-131).  A and H may be destroyed afterwards. */
int dnpeff_fit_create(dnpeff_csr* A, dnpeff_csr* H, float eps, int64_t seed, dnpeff_fit** out);

/* W ~ U[0,1) from the seed / caller-chosen W [n, r] row-major. */
int dnpeff_fit_init_W(dnpeff_fit* fit);
int dnpeff_fit_set_W(dnpeff_fit* fit, const float* W_nr);

/* n_steps of WHH = W (H H^T); W <- W * (A H^T) / (WHH + eps)
 * (DoMuStep, nmf_sparse_H.h:342-345).  Several steps in one call give the same W as as many
 * calls of one step, and cost less: what the steps share (H H^T in the layout the kernel reads)
 * is prepared once per call. */
int dnpeff_fit_step(dnpeff_fit* fit, int n_steps);

/* reference_loss: sqrt(||A||^2 + <WHH, W> - 2 <A H^T, W>) with WHH as left by
 * the last step, i.e. computed from W before that step's update -- the value
 * the reference logs (nmf_sparse_H.h:319-331).  true_loss uses W (H H^T) of
 * the current W.  Either pointer may be NULL. */
int dnpeff_fit_loss(dnpeff_fit* fit, double* reference_loss, double* true_loss);

int dnpeff_fit_get_W(dnpeff_fit* fit, float* W_nr);
/* Stage-1 products: AH [n, r] row-major, HH [r, r]. */
int dnpeff_fit_get_products(dnpeff_fit* fit, float* AH_nr, float* HH_rr, double* sq_norm_A);
int dnpeff_fit_destroy(dnpeff_fit* fit);

/* ------------------------------------------------------------------------- */
/* Single kernels on device pointers (parity tests and profiling)             */
/* All factor pointers are device memory in the device layout ([rows, r]).    */
/* They are queued on the library stream; call dnpeff_sync() before reading.  */
/* ------------------------------------------------------------------------- */

/* F[i] *= num[i] / (den[i] + eps), i < count.  kernelNmfMuUpdate
 * (cc/cuda_d_npeff/src/nmf/sparse/kernels.h:24-34) and
 * MultiplicativeUpdate_Kernel (nmf/kernels/mu.h:32-38). */
int dnpeff_op_mu(int64_t count, float* F, const float* num, const float* den, float eps);

/* Every column of the row-major factor W [n_rows, rank] is moved, in place, to non-negative
 * entries that sum to l1_norm, by the iteration of DenseFactorSparsityContext::sparsifyF
 * (dense_factor_sparsity_constraints.h:205-237) with the arithmetic of its kernels
 * (sparsity_constraint_kernels.h:16-141): Hoyer's projection, except that the step length is the
 * reference's expression (:51-65), which leaves ||column||^2 = l2_norm^2 + l1_norm^2 / (entries
 * left non-zero) rather than l2_norm^2.  Column sums are taken in fp64 in a fixed order where the
 * reference calls cublasSgemv / cublasSgemmStridedBatched (:405-452).  Synchronises once per pass
 * (the reference's isFinishedSync, :363-374).  Fails for l1_norm <= 0 (a null constraint, :41-43). */
int dnpeff_op_sparsify_columns(int64_t n_rows, int rank, float* W_nr, float l1_norm, float l2_norm,
                               int* rounds);

/* N[n, r] = A H^T with H given as [m, r].  cusparseSpMM(N, T) at
 * device_contexts1.h:255-258,317. */
int dnpeff_op_spmm_n(dnpeff_csr* A, int r, const float* H_mr, float* N_nr);

/* The same product with the work decomposition of the sparse part chosen by the caller, for
 * comparisons on ragged rows: 0 = as planned (column panels and swept pieces where the factor
 * is large, else row chunks), 1 = one wavefront per row, 2 = chunks of 2048 entries of a row with
 * a second pass over the chunk sums, 3 = merge path: every wavefront takes 4096 consecutive steps
 * of the path that consumes each row's entries and then its end marker, wherever the row
 * boundaries fall (the nnz-balanced split of cc/cuda_d_npeff/src/cuda/ops/sp_slicing.h:314-403
 * taken down to wavefronts), with a pass that adds the sums of the rows cut between shares.
 * 1, 2 and 3 need the row-major arrays. */
int dnpeff_op_spmm_n_variant(dnpeff_csr* A, int r, const float* H_mr, float* N_nr, int variant);

/* T[m, r] = A^T W with W [n, r]; needs dnpeff_csr_build_transpose.
 * cusparseSpMM(T, T) at device_contexts1.h:260-265,301. */
int dnpeff_op_spmm_t(dnpeff_csr* A, int r, const float* W_nr, float* T_mr);

/* Rows [col0, col1) of A^T W into T_tile [col1 - col0, r]: the product on a column tile, as the
 * tiled H update of dnpeff_nmf_update_H forms it. */
int dnpeff_op_spmm_t_tile(dnpeff_csr* A, int r, const float* W_nr, int64_t col0, int64_t col1,
                          float* T_tile);

/* Keeps the elements with x[i] / divisor >= threshold (fp32 division, then the comparison):
 * idx_out receives their positions in ascending order, val_out the divided values, *n_kept
 * (host) their number; idx_out and val_out are device buffers of `count` elements.  One row of
 * the dense-to-sparse conversion of H, to_csr in scripts/sparsify_d_npeff.py:27-49, after the
 * row has been scaled to unit norm (:56). */
int dnpeff_op_threshold_compact(int64_t count, const float* x, float divisor, float threshold,
                                int32_t* idx_out, float* val_out, int64_t* n_kept);

/* Per-example top-k of dense rows x[n_rows, count] (device): vals_out / idx_out [n_rows, k] get
 * the k largest entries of each row in descending order, equal values in ascending index
 * order, norms_out [n_rows] (may be NULL) the L2 norm of the whole row (sum of squares in
 * fp64).  All buffers are device memory.  Replaces tf.math.top_k and the einsum norm in the
 * PEF producer (npeff/fishers/d_pefs_computer.py:126-129 and :48-50); the outputs are the
 * data/fisher/values, data/fisher/indices and data/dense_fisher_norms rows of the PEF file. */
int dnpeff_topk_rows(int64_t n_rows, int64_t count, int64_t k, const float* x, float* vals_out,
                     int32_t* idx_out, float* norms_out);

/* G[r, r] = X^T X for X [rows, r].  cublasSgemm at device_contexts1.h:303,322. */
int dnpeff_op_gram(int64_t rows, int r, const float* X, float* G_rr);

/* The same product for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): no counterpart in the
 * reference.  The slice partials that dnpeff_op_gram keeps in a buffer it allocates go to a
 * static 8 MiB device array instead; the call allocates and frees nothing and does not wait for
 * the device (call dnpeff_sync() before reading G).  Limits: 1 <= r <= 128; any number of rows at
 * r <= 32, at most 52,224 rows above (a larger request is refused with an error).  Same kernels,
 * same summation order, same bits as dnpeff_op_gram.  All calls on one GPU share the array:
 * calls queued on the library stream run one after the other, calls that overlap on one GPU
 * (other threads, other streams) race. */
int dnpeff_op_gram_static(int64_t rows, int r, const float* X, float* G_rr);

/* out = X * num / (X G + eps) with X, num, out [rows, r], G [r, r] symmetric.
 * out may alias num but not X.  D_out (may be NULL) receives X G.
 * cublasSgemm + kernelNmfMuUpdate at device_contexts1.h:306-308,329-332. */
int dnpeff_op_xg_mu(int64_t rows, int r, const float* X, const float* G_rr,
                    const float* num, float eps, float* out, float* D_out);

/* The same update for r = 128 that also returns the Gram matrix of its result:
 * out = X * num / (X G + eps), Gout = out^T out, in one pass over the rows
 * (rows >= 64; out may alias num but not X).  This is what dnpeff_nmf_update_H
 * runs at rank 128; the reference has no counterpart (it calls cublasSgemm for
 * H^T H separately, device_contexts1.h:303).  For tests and benchmarks. */
int dnpeff_op_xg_mu_gram(int64_t rows, const float* X, const float* G_rr,
                         const float* num, float eps, float* out, float* Gout_rr);

/* <x, y> over count floats, fp64 accumulation; result to the host.
 * frobeniusProductToHost (device_contexts1.h:503-537). */
int dnpeff_op_dot(int64_t count, const float* x, const float* y, double* out_host);

/* out[n, r] = A B^T for sparse A [n, m] and sparse B [r, m] (both CSR); B's
 * transposed copy is built if missing.  Partitioned_SpSpMatmul_ToDense
 * (cc/cuda_d_npeff/src/cuda/ops/spsp_matmul.h:95-131). */
int dnpeff_op_spsp_dense(dnpeff_csr* A, dnpeff_csr* B, float* out_nr);

/* out[k, :] = X[rows_dev[k], :] for k < count: rows of r floats picked from a device array by a
 * device index list (test and validation helper: sampled rows of a factor). */
int dnpeff_op_gather_rows(int64_t count, int r, const float* X, const int32_t* rows_dev, float* out);

/* dst[i] = src[i], i < count: a plain streaming copy of known size, the yardstick
 * that hardware-counter readings (FETCH_SIZE, WRITE_SIZE) are scaled by. */
int dnpeff_op_copy(int64_t count, const float* src, float* dst);

/* x[i] = U[0,1) value of logical element i of matrix matrix_id, written in the
 * device layout (see dnpeff_uniform_at). */
int dnpeff_op_init_uniform(int matrix_id, int64_t logical_rows, int64_t logical_cols,
                           uint64_t seed, float* x);

#ifdef __cplusplus
}
#endif
#endif /* DNPEFF_H_ */
