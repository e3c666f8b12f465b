// Internal declarations shared by the translation units of libdnpeff_hip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <vector>

#include "../../include/dnpeff.h"

#define DN_API extern "C" __attribute__((visibility("default")))

namespace dn {

// Records the message returned by dnpeff_last_error().
void set_error(const char* fmt, ...);
void clear_error();

// The library's single stream (default priority), created on first use.
hipStream_t stream();
// Compute units of device 0.
int n_cus();
// A second stream for work that may run beside the library stream (see loader.hip).
int side_stream_begin();
int side_stream_end();
int side_stream_join();
hipStream_t side_stream_handle();
void side_stream_route(bool on);
bool side_stream_routed();
bool side_stream_pending();

}  // namespace dn

#define DN_HIP(expr)                                                                 \
  do {                                                                               \
    hipError_t dn_e_ = (expr);                                                       \
    if (dn_e_ != hipSuccess) {                                                       \
      dn::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(dn_e_), __FILE__, \
                    __LINE__);                                                       \
      return 1;                                                                      \
    }                                                                                \
  } while (0)

#define DN_CHECK(cond, ...)       \
  do {                            \
    if (!(cond)) {                \
      dn::set_error(__VA_ARGS__); \
      return 2;                   \
    }                             \
  } while (0)

#define DN_TRY(expr)          \
  do {                        \
    int dn_s_ = (expr);       \
    if (dn_s_) return dn_s_;  \
  } while (0)

#define DN_LAUNCH_CHECK() DN_HIP(hipGetLastError())

namespace dn {

template <class T>
inline int dmalloc(T** p, int64_t count) {
  *p = nullptr;
  size_t bytes = sizeof(T) * (size_t)(count > 0 ? count : 1);
  hipError_t e = hipMalloc((void**)p, bytes);
  if (e != hipSuccess) {
    set_error("hipMalloc of %zu bytes failed: %s", bytes, hipGetErrorString(e));
    return 1;
  }
  return 0;
}

inline void dfree(void* p) {
  if (p) (void)hipFree(p);
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// A device buffer that is freed when it goes out of scope, for temporaries of functions with
// several exits; release() hands the pointer over to a longer-lived owner.
template <class T>
struct dbuf {
  T* p = nullptr;
  dbuf() = default;
  dbuf(const dbuf&) = delete;
  dbuf& operator=(const dbuf&) = delete;
  ~dbuf() { dfree(p); }
  int alloc(int64_t count) {
    dfree(p);
    return dmalloc(&p, count);
  }
  void reset() {
    dfree(p);
    p = nullptr;
  }
  T* release() {
    T* q = p;
    p = nullptr;
    return q;
  }
  operator T*() const { return p; }
};

// ---- scans (loader.hip) ----
// out[i] = sum_{i' < i} (count[i'] >= min_count), i in [0, n]; out has n+1 entries.
int scan_keep_mask(const int* count, int min_count, int64_t n, int32_t* out);
// out[i] = sum_{i' < i} count[i'], i in [0, n].
int scan_counts_i64(const int* count, int64_t n, int64_t* out);
// out[e] = number of kept entries before e (table[colind[e]] != -1), e in [0, nnz].
int scan_kept_entries(const int32_t* colind, const int32_t* table, int64_t nnz, int64_t* out);
// out[i] = sum_{i' < i} ceil(len_i' / chunk), i in [0, n].
int scan_row_chunks(const int64_t* rowptr, int64_t chunk, int64_t n, int64_t* out);
// out[j] = number of columns j' < j longer than `limit`, j in [0, n].
int scan_long_cols(const int64_t* colptr, int64_t limit, int64_t n, int32_t* out);

// ---- dense kernels (dense.hip) ----
int launch_mu(int64_t count, float* F, const float* num, const float* den, float eps);
// Needs a workspace of gram_workspace_floats(rows, r) floats.
int64_t gram_workspace_floats(int64_t rows, int r);
int launch_gram(int64_t rows, int r, const float* X, float* G, float* workspace);
// ranks 256, 384, ..., 1024 (head.hip)
int64_t gram_tiles_workspace_floats(int64_t rows, int r);
int launch_gram_tiles(int64_t rows, int r, const float* X, float* G, float* workspace);
// Between the two, launch_xg_mu calls with this G reuse one transposed copy of it (the caller
// must not change G in between).
int xg_mu_hold_g(const float* G, int r);
void xg_mu_release_g();
int launch_xg_mu(int64_t rows, int r, const float* X, const float* G, const float* num, float eps,
                 float* out, float* D_out);
// r = 128: the update and the Gram matrix of its output in one pass (dense.hip).
int64_t xg_mu_gram_workspace_floats(int64_t rows);
int launch_xg_mu_gram(int64_t rows, const float* X, const float* G, const float* num, float eps,
                      float* out, float* Gout, float* gpart, float* G_tmp, float* gram_ws);
// dot with fp64 accumulation; result lands in *out_dev (one double, device).
// partials: workspace of DOT_BLOCKS doubles.
constexpr int DOT_BLOCKS = 2048;
int launch_dot(int64_t count, const float* x, const float* y, double* partials, double* out_dev);
int launch_init_uniform(int matrix_id, int64_t logical_rows, int64_t logical_cols, uint64_t seed,
                        float* x);
// out[c * rows + i] = in[i * cols + c]   (in is [rows, cols] row-major)
int launch_transpose(int64_t rows, int64_t cols, const float* in, float* out);

// ---- sparse kernels (spmm.hip) ----
constexpr int64_t SPMM_N_CHUNK = 2048;  // entries of one row handled by one workgroup
constexpr int64_t SPMM_T_LONG = 256;    // columns longer than this get a whole workgroup
// A H^T in two steps (partial sums, then their reduction); both cover the sparse part and the
// dense head of A.  Need csr_ensure_products(A, r).
int launch_spmm_n(const dnpeff_csr* A, int r, const float* H_mr, int part = 0);
int launch_spmm_n_reduce(const dnpeff_csr* A, int r, float* N_nr);
int launch_spmm_t(const dnpeff_csr* A, int r, const float* W_nr, float* T_mr);
int launch_spsp(const dnpeff_csr* A, dnpeff_csr* B, float* partials);
// sparsity.hip: the sparseness projection of the columns of a row-major [n, r] factor, in place
int sparsify_columns(int64_t n, int r, float* W, float l1, float l2, int* rounds_out);
int launch_chunk_reduce(const dnpeff_csr* A, int r, const float* partials, float* N_nr);

// Switches for experiments and for tests that force a code path.  Each has an environment
// variable DNPEFF_<NAME IN CAPITALS> that is read once, when the library is first used, and can be
// set afterwards with dnpeff_tuning_set(); plans (panels, head, tiles) take their values when they
// are made, launch paths read no environment.
struct tuning_t {
  double dense_fill = 1.0 / 16.0;  // columns held by this fraction of the rows form the dense head (0 = none)
  double panels = -1.0;            // coarse column panels of A H^T (-1 = by the size of the factor, 0 = none)
  double sweep_bytes = 3.0 * 1024 * 1024;  // bytes of the factor per swept piece (0 = no swept pieces)
  double sweep_min = -1.0;         // entries a row must hold per piece on average (-1 = default rule)
  double sweep_waves = 0.0;        // waves per workgroup of the sweep kernel (0 = as many as fit)
  double sweep_lag = 0.0;          // pieces the workgroups of an XCD may be apart
  double sweep_spin = 400.0;       // polls before a workgroup of the sweep stops waiting
  double spmm_t_slices = 0.0;      // component slices of A^T W (0 = by the size of W)
  double split_bf16 = 1.0;         // matrix products on the bf16 cores with split fp32 operands (0 = fp32 cores)
  double fused_gram = 1.0;         // rank 128: the H update also produces H^T H
  double h_tile_mb = 768.0;        // size of a column tile of the tiled H update, MiB of the factor
  double tiled_h = -1.0;           // tiled H update: 1 = always, 0 = never, -1 = when the full-size buffer does not fit
  double topk_fast_cap = -1.0;     // top-k: candidate list length that ends the histogram passes (-1 = default)
  double n_lists = -1.0;           // A H^T from slot lists on component slices: 0 = never, 1 = the whole sparse
                                   // part, 2 = its far tail, -1 = the far tail where that pays (see use_nlists_tail)
  double t_lists = 0.0;            // A^T W in column blocks on component slices (1 = on)
  double nl_piece_cols = 32768.0;  // columns per piece of the slot lists
  double nl_extra_mb = -1.0;       // MB the far tail's slot lists may take beyond their panel copy (-1: 1/128 of the device)
  double nl_lag = 0.0;             // pieces the workgroups of an XCD may be apart
  double gram_beside = 1.0;        // H^T H of the W update on a second stream beside the dense head and the plain panels of A H^T (0 = after A H^T)
  double h_overlap = 0.0;          // tiled H update: A^T W of the next tile beside the update of this one (two streams, two tile buffers)
  double xg_wgs = 3.0;             // workgroups per CU of the r >= 256 update kernel: 3 where the launch fills the CUs eight times, 4 = three always, 2 = two (padded planes, two operand stages)
  double gram_fold = 2.0;          // X^T X on tiles: 2 = diagonal squares of 256 columns in one workgroup where the rank is a
                                   // multiple of 256, else as 1 = diagonal tiles of 128 with their symmetry; 0 = all sixteen blocks
  double nl_wgs = 64.0;            // workgroups of the slot-list kernel per XCD (two per CU)
  double nl_spin = 50000.0;        // polls (about 1 us each) before a workgroup of the slot-list kernel stops waiting
  double verbose = 0.0;
};
tuning_t& tuning();

// Products of the large matrix-core kernels run on the bf16 matrix cores with every fp32 operand
// split in three (split_bf16.hpp) unless the split_bf16 switch selects the fp32 matrix cores.
inline bool use_split_bf16() { return tuning().split_bf16 != 0.0; }

// Columns present in many rows, held as a dense block in both orientations (head.hip).
struct dense_head {
  int64_t n_d = 0;      // columns in the head
  int64_t n_d_pad = 0;  // n_d rounded up to 128
  int64_t n_pad = 0;    // rows rounded up to 128
  int32_t* cols = nullptr;  // [n_d] column of each head slot, ascending
  float* cm = nullptr;      // [n_d_pad, n_pad]: cm[k * n_pad + i] = A[i, cols[k]]
  // [n_pad, n_d_pad]: rm[i * n_d_pad + k] = A[i, cols[k]]; made from cm when a product needs it
  // (the fp32 matrix-core kernel of A^T W; the split-operand kernels read cm in both directions)
  float* rm = nullptr;
  float* ws = nullptr;      // gathered factor rows + slice partials of the products
  int64_t ws_floats = 0;
};

// How the columns of a sparse part are cut into panels for A H^T: `coarse` panels with equal
// numbers of entries; a coarse panel wider than sweep_cols columns in which a row holds at least
// sweep_min entries per sweep_cols columns on average is cut into pieces of at most sweep_cols
// columns, which are swept (spmm.hip).
struct panel_plan {
  int coarse = 0;
  int sweep_cols = 0;
  double sweep_min = 0.0;
  bool tail_lists = false;  // the plain panels past the last swept one go to slot lists instead
  bool operator==(const panel_plan& o) const {
    return coarse == o.coarse && sweep_cols == o.sweep_cols && sweep_min == o.sweep_min &&
           tail_lists == o.tail_lists;
  }
};

// Slot lists of A H^T on component slices (lists.hip): the entries of the sparse part as one
// stream of (local row, local column, value) per wave slot, ordered by column piece.
struct slot_lists {
  int piece_cols = 0, n_pieces = 0, n_parts = 0, rpw = 0, wgs = 0;
  int32_t floor_col = 0;          // the lists hold the entries of columns floor_col .. only
  int64_t n_batches = 0, n_entries = 0;
  uint2* pairs = nullptr;         // [n_batches + 8][64]
  int64_t* slot_base = nullptr;   // [n_slots + 1] first batch of each slot
  uint32_t* off = nullptr;        // [n_slots][n_pieces + 1] batches of the slot before piece p
  int32_t* slot_rows = nullptr;   // [n_slots][rpw] row of each local row, -1 = none
  int32_t* row_slot = nullptr;    // [n_rows] slot * 128 + local row
  int* progress = nullptr;        // progress counters of the XCDs
  std::vector<int32_t> h_row_slot;
  std::vector<int64_t> h_slot_base;
};

// Column blocks of A^T W on component slices (lists.hip): cols[b] = first column of block b.
struct col_blocks {
  int32_t* cols = nullptr;  // [n_blocks + 1]
  int64_t n_blocks = 0;
  std::vector<int64_t> h_first;  // first block of every aligned group of 64 columns
};

}  // namespace dn

struct dnpeff_csr {
  int64_t n_rows = 0, n_cols = 0, nnz = 0;
  int64_t full_dense_size = 0;
  // ||A||_F^2 as first computed (from the row-major values, in their order); the loader calls that
  // change entries clear it.  Kept so that a matrix whose arrays a context has consumed still
  // gives later contexts the same number.
  double sq_norm = 0.0;
  bool sq_norm_valid = false;
  // row-major copy
  int64_t* rowptr = nullptr;
  int32_t* colind = nullptr;
  float* vals = nullptr;
  // newToOgIndex of the last compaction / retain (nullptr = identity)
  int32_t* kept = nullptr;
  // transposed copy: per column the (row, value) pairs in ascending row order
  int64_t* colptr = nullptr;
  int32_t* rowind = nullptr;
  float* tvals = nullptr;
  // as the sparse factor of dnpeff_op_spsp_dense: per column 32 bytes holding its first four
  // (row, value) pairs and, in the upper half of the first row word, its length
  uint4* slots = nullptr;
  // work decomposition of A H^T: chunk_base[i] = chunks of rows before i
  int64_t* chunk_base = nullptr;
  int64_t n_chunks = 0;
  // columns longer than SPMM_T_LONG
  int32_t* long_cols = nullptr;
  int64_t n_long = 0;
  // workspace for the per-chunk partial sums of A H^T ([n_chunks, r])
  float* partials = nullptr;
  int64_t partials_floats = 0;
  // column panels of A H^T: the entries of every row regrouped by panel (original order kept
  // inside a panel), seg[row * (n_panels + 1) + p] = first entry of the (row, p) segment
  int n_panels = 0;
  int32_t* panel_bounds = nullptr;  // [n_panels + 1] first column of each panel
  // panel_ids[0 .. n_plain): panels handled one wave per (row, panel) segment, in grid order;
  // panel_ids[n_plain .. n_plain + n_swept): swept panels
  int n_plain = 0, n_swept = 0;
  int32_t* panel_ids = nullptr;
  int* sweep_progress = nullptr;  // per-XCD counters of the sweep kernel (256 ints)
  int32_t* sweep_perm = nullptr;  // the rows in the order the sweep kernel takes them
  int64_t sweep_perm_key = 0;     // the launch shape that order was made for
  dn::panel_plan plan;
  int64_t* seg = nullptr;
  int32_t* pcol = nullptr;
  float* pval = nullptr;
  // tail_floor > 0: the panels hold the entries of columns below tail_floor only (row i's at
  // prow[i] .. prow[i + 1] of pcol / pval), the others are in the slot lists nl
  int32_t tail_floor = 0;
  int64_t* prow = nullptr;
  bool tail_declined = false;  // the far tail's slot lists did not fit the memory bound: it stays panels
  // after dnpeff_csr_split_dense_head: the dense block and the matrix of the remaining entries
  // (same shape, owned), which carries the derived structures the products use
  dn::slot_lists nl;
  dn::col_blocks tb;
  dn::dense_head head;
  dnpeff_csr* tail = nullptr;
  // host copies of head.cols and long_cols (ascending), made when a product runs on column tiles
  std::vector<int32_t> h_head_cols, h_long_cols;
  bool h_lists_valid = false;
};

namespace dn {
inline dnpeff_csr* sparse_part(dnpeff_csr* A) { return A->tail ? A->tail : A; }
inline const dnpeff_csr* sparse_part(const dnpeff_csr* A) { return A->tail ? A->tail : A; }
int csr_ensure_chunks(dnpeff_csr* A);
int csr_ensure_partials(dnpeff_csr* A, int r);
// Builds (or drops) the column panels of a matrix without dense head / of a sparse part;
// needs the transposed copy.  plan.coarse = 0 removes them.
int csr_set_panels(dnpeff_csr* S, const panel_plan& plan);
// Swept panels are summed per XCD: one slot of partial sums per plain panel plus SWEEP_XCDS.
constexpr int SWEEP_XCDS = 8;
// With a far tail on slot lists (tail_floor > 0) their sums take one more slot, the last.
inline int64_t panel_slots(const dnpeff_csr* S) {
  return S->n_plain + (S->n_swept > 0 ? SWEEP_XCDS : 0) + (S->tail_floor > 0 ? 1 : 0);
}
// Whether the workgroups of a launch go to the SWEEP_XCDS XCDs round-robin (probed once).
bool xcd_round_robin();
// Ranks the sweep kernel of A H^T handles.
// Components that one launch of the sweep kernel sums: the rank itself up to 256, else slices of
// 256 or 128 components (0 = the rank has no sweep kernel).
inline int sweep_width(int r) {
  if (r == 32 || r == 64 || r == 128 || r == 256) return r;
  if (r > 256 && r % 256 == 0) return 256;
  if (r > 256 && r % 128 == 0) return 128;
  return 0;
}
inline bool spmm_n_sweep_supported(int r) { return sweep_width(r) != 0; }
// Everything A H^T and A^T W at rank r need: transposed copy and work lists of the sparse part,
// workspaces of the sparse part and of the dense head.
int csr_ensure_products(dnpeff_csr* A, int r);
int head_ensure_workspace(dnpeff_csr* A, int r);
int launch_head_n(const dnpeff_csr* A, int r, const float* H_mr);
int launch_head_n_add(const dnpeff_csr* A, int r, float* N_nr);
int launch_head_t(const dnpeff_csr* A, int r, const float* W_nr, float* T_mr);
// The same in two steps for a result that is produced in column tiles: the product into the head's
// workspace once, then the rows of the head slots [k0, k1) to T_tile[cols[k] - col0].
int launch_head_t_product(const dnpeff_csr* A, int r, const float* W_nr);
int launch_head_t_scatter(const dnpeff_csr* A, int r, int64_t k0, int64_t k1, int64_t col0,
                          float* T_tile);
// Rows [col0, col1) of A^T W into T_tile (row j - col0), sparse part and dense head; the head's
// product must have been launched (launch_head_t_product) and csr_tile_lists(A) built.
int launch_spmm_t_tile(const dnpeff_csr* A, int r, const float* W_nr, int64_t col0, int64_t col1,
                       float* T_tile);
int csr_tile_lists(dnpeff_csr* A);
// True while the arrays of the row-major copy that the loader calls and dnpeff_csr_download use
// are there (dnpeff_csr_release or a consuming dnpeff_nmf_create_ex frees them).
inline bool has_row_major(const dnpeff_csr* A) {
  return A->rowptr != nullptr && (A->nnz == 0 || (A->colind != nullptr && A->vals != nullptr));
}
// lists.hip
bool nlists_supported(const dnpeff_csr* S, int r);
// max_extra_bytes >= 0: the lists are not built (*declined = true) when they would take more than
// that beyond the 8 bytes per entry of the panel copy they replace
int nlists_build(dnpeff_csr* S, int r, int32_t floor_col = 0, double max_extra_bytes = -1.0,
                 bool* declined = nullptr);
int nlists_slots(int64_t n_rows, int r);  // wave slots (of eight lane groups) the lists of rank r use
int csr_rows_count_below(const dnpeff_csr* S, int32_t col, int* d_below);
void nlists_drop(dnpeff_csr* S);
int launch_spmm_n_lists(const dnpeff_csr* S, int r, const float* H_mr, float* part, int64_t stride);
int nlists_get_row(const dnpeff_csr* S, int64_t row, std::vector<int32_t>& cols, std::vector<float>& vals);
bool tlists_supported(const dnpeff_csr* S, int r);
int tblocks_build(dnpeff_csr* S);
void tblocks_drop(dnpeff_csr* S);
int launch_spmm_t_lists(const dnpeff_csr* S, int r, const float* W_nr, float* T, int64_t col0, int64_t col1);
// Whether the products of the sparse part S at rank r run from the slot lists / column blocks.
bool use_nlists(const dnpeff_csr* S, int r);       // the whole sparse part on slot lists
bool use_nlists_tail(const dnpeff_csr* S, int r);  // its far tail only
bool use_tlists(const dnpeff_csr* S, int r);
struct head_choice {
  int64_t thr = 0;   // columns with at least thr entries form the head (0 = no head)
  int64_t n_d = 0;
  double footprint = 0.0;  // bytes of the dense blocks + both sparse copies of the rest
  bool fits = true;        // footprint within the budget given
};
constexpr double NO_BUDGET = 1e300;
// rank > 0: the footprint also counts the head's workspace at that rank
int choose_dense_head(dnpeff_csr* A, double min_fill, double budget, int n_blocks, int rank, head_choice* out);
int64_t head_workspace_floats(int64_t n_rows, int64_t n_d, int r);
// Sizes that the memory plan shares with the code that allocates (loader.hip).
constexpr double PANEL_PARTIALS_BYTES = 3.0e9;  // the plain panels' partial sums stay within this
int64_t coarse_panels_for(int64_t n_rows, int64_t n_cols, int r, bool sweeps);
bool sweeps_for_rank(int r);
int max_panels();
// Dense blocks that the head's products at rank r read (1 or 2), see dense_head::rm.
int head_blocks_for_rank(int r);
int split_dense_head_at(dnpeff_csr* A, int64_t thr, int64_t* n_dense);
// Frees every array of A that the products A H^T and A^T W do not read.
int csr_consume_for_products(dnpeff_csr* A);
}  // namespace dn
