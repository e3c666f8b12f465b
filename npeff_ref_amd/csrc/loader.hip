// CSR loader on the device: upload, row normalisation, column compaction,
// column retention, transposed CSR, ||A||^2.  Integer results are bit-exact
// with the reference's host code; see include/dnpeff.h for the citations.
#include "dnpeff_internal.hpp"
#include "scan.hpp"

#include <cmath>
#include <cstdlib>

#include <cstdarg>
#include <cstring>
#include <vector>

namespace dn {

// ---------------------------------------------------------------------------
// Library state
// ---------------------------------------------------------------------------
static thread_local char g_error[1024] = "";
static hipStream_t g_stream = nullptr;
static int g_n_cus = 0;

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
void clear_error() { g_error[0] = 0; }

hipStream_t stream() {
  if (!g_stream) {
    if (hipStreamCreate(&g_stream) != hipSuccess) {
      fprintf(stderr, "dnpeff: hipStreamCreate failed (no usable GPU?)\n");
      abort();
    }
  }
  return g_stream;
}

int n_cus() {
  if (!g_n_cus) {
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, 0) == hipSuccess) g_n_cus = p.multiProcessorCount;
    if (g_n_cus <= 0) g_n_cus = 256;
  }
  return g_n_cus;
}

struct KeepMaskF {
  const int* count;
  int min_count;
  __device__ int64_t operator()(int64_t i) const { return count[i] >= min_count ? 1 : 0; }
};
struct CountsF {
  const int* count;
  __device__ int64_t operator()(int64_t i) const { return count[i]; }
};
struct KeptEntryF {
  const int32_t* colind;
  const int32_t* table;
  __device__ int64_t operator()(int64_t e) const { return table[colind[e]] != -1 ? 1 : 0; }
};
struct RowChunksF {
  const int64_t* rowptr;
  int64_t chunk;
  __device__ int64_t operator()(int64_t i) const {
    int64_t len = rowptr[i + 1] - rowptr[i];
    return (len + chunk - 1) / chunk;
  }
};
struct LongColF {
  const int64_t* colptr;
  int64_t limit;
  __device__ int64_t operator()(int64_t j) const {
    return (colptr[j + 1] - colptr[j]) > limit ? 1 : 0;
  }
};

struct GeThresholdF {
  const float* x;
  float divisor, threshold;
  __device__ int64_t operator()(int64_t i) const { return x[i] / divisor >= threshold ? 1 : 0; }
};

int scan_keep_mask(const int* count, int min_count, int64_t n, int32_t* out) {
  return exclusive_scan(KeepMaskF{count, min_count}, n, out);
}
int scan_counts_i64(const int* count, int64_t n, int64_t* out) {
  return exclusive_scan(CountsF{count}, n, out);
}
int scan_kept_entries(const int32_t* colind, const int32_t* table, int64_t nnz, int64_t* out) {
  return exclusive_scan(KeptEntryF{colind, table}, nnz, out);
}
int scan_row_chunks(const int64_t* rowptr, int64_t chunk, int64_t n, int64_t* out) {
  return exclusive_scan(RowChunksF{rowptr, chunk}, n, out);
}
int scan_long_cols(const int64_t* colptr, int64_t limit, int64_t n, int32_t* out) {
  return exclusive_scan(LongColF{colptr, limit}, n, out);
}

// ---------------------------------------------------------------------------
// Loader kernels
// ---------------------------------------------------------------------------

__global__ void __launch_bounds__(256) k_pef_rowptr(int64_t n_rows, int64_t k, int64_t* rowptr) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i <= n_rows; i += stride)
    rowptr[i] = i * k;
}

// vals[e] /= (norms[row] + eps); one workgroup walks one row at a time.
__global__ void __launch_bounds__(256) k_normalize_rows(const int64_t* __restrict__ rowptr,
                                                        float* __restrict__ vals,
                                                        const float* __restrict__ norms, float eps,
                                                        int64_t n_rows) {
  for (int64_t row = blockIdx.x; row < n_rows; row += gridDim.x) {
    const float d = norms[row] + eps;
    const int64_t e1 = rowptr[row + 1];
    for (int64_t e = rowptr[row] + threadIdx.x; e < e1; e += 256) vals[e] = vals[e] / d;
  }
}

__global__ void __launch_bounds__(256)
    k_col_hist(const int32_t* __restrict__ colind, int64_t nnz, int* __restrict__ count) {
  int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < nnz; e += stride)
    atomicAdd(&count[colind[e]], 1);
}

// og_to_new[i] = pos[i] if kept else -1; new_to_og[pos[i]] = i.
__global__ void __launch_bounds__(256)
    k_build_maps(const int* __restrict__ count, int min_count, const int32_t* __restrict__ pos,
                 int64_t n_cols, int32_t* __restrict__ og_to_new, int32_t* __restrict__ new_to_og) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n_cols; i += stride) {
    if (count[i] >= min_count) {
      og_to_new[i] = pos[i];
      new_to_og[pos[i]] = (int32_t)i;
    } else {
      og_to_new[i] = -1;
    }
  }
}

// table[c] = -1 for the columns of the head, c for the others
__global__ void __launch_bounds__(256)
    k_tail_table(const int32_t* __restrict__ og_to_new, int64_t n_cols, int32_t* __restrict__ table) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n_cols; i += stride)
    table[i] = og_to_new[i] >= 0 ? -1 : (int32_t)i;
}

// Entries of the head's columns into both dense blocks; a workgroup per row.  Entries that
// repeat a (row, column) pair add up, as they do in the sparse products.
__global__ void __launch_bounds__(256)
    k_head_fill(const int64_t* __restrict__ rowptr, const int32_t* __restrict__ colind,
                const float* __restrict__ vals, int64_t n_rows, const int32_t* __restrict__ slot_of,
                float* __restrict__ cm, int64_t n_pad, float* __restrict__ rm, int64_t n_d_pad) {
  for (int64_t row = blockIdx.x; row < n_rows; row += gridDim.x) {
    const int64_t e1 = rowptr[row + 1];
    for (int64_t e = rowptr[row] + threadIdx.x; e < e1; e += 256) {
      const int32_t k = slot_of[colind[e]];
      if (k >= 0) {
        atomicAdd(&cm[(int64_t)k * n_pad + row], vals[e]);
        atomicAdd(&rm[row * n_d_pad + k], vals[e]);
      }
    }
  }
}

// bounds[p] = first column c with colptr[c] >= p * nnz / P  (bounds[0] = 0, bounds[P] = n_cols):
// P panels of consecutive columns with about the same number of entries each.
__global__ void __launch_bounds__(256)
    k_panel_bounds(const int64_t* __restrict__ colptr, int64_t n_cols, int64_t nnz, int P,
                   int32_t* __restrict__ bounds) {
  const int p = blockIdx.x * 256 + threadIdx.x;
  if (p > P) return;
  if (p == 0) { bounds[0] = 0; return; }
  if (p == P) { bounds[P] = (int32_t)n_cols; return; }
  const int64_t target = (int64_t)(((__int128)nnz * p) / P);
  int64_t lo = 0, hi = n_cols;  // smallest c in [0, n_cols] with colptr[c] >= target
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (colptr[mid] >= target) hi = mid; else lo = mid + 1;
  }
  bounds[p] = (int32_t)lo;
}

// Regroups the entries of each row by column panel, keeping their order inside a panel (a
// stable split, so the result does not depend on how the hardware schedules the lanes), and
// records where each (row, panel) segment starts.  One workgroup per row at a time: a counting
// pass, a scan over the panels, then tiles of 256 entries in order; within a tile an entry's
// rank among the entries of its panel comes from wave ballots over the bits of the panel
// number plus the per-wave counts of the earlier waves.
constexpr int MAX_PANELS = 3072;

__global__ void __launch_bounds__(256)
    k_panel_split(const int64_t* __restrict__ rowptr, const int32_t* __restrict__ colind,
                  const float* __restrict__ vals, int64_t n_rows, int P, int bits,
                  const int32_t* __restrict__ bounds, int64_t* __restrict__ seg,
                  int32_t* __restrict__ pcol, float* __restrict__ pval) {
  __shared__ int32_t bnd[MAX_PANELS + 1];
  __shared__ int hist[MAX_PANELS];
  __shared__ int cursor[MAX_PANELS];         // next free position of each panel, relative to e0
  __shared__ uint8_t wcnt[4][MAX_PANELS];    // entries of a panel in one wave of a tile (<= 64)
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  for (int i = tid; i <= P; i += 256) bnd[i] = bounds[i];
  auto panel_of = [&](int32_t col) {
    int lo = 0, hi = P;  // largest p < P with bnd[p] <= col
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (bnd[mid] <= col) lo = mid; else hi = mid;
    }
    return lo;
  };
  for (int64_t row = blockIdx.x; row < n_rows; row += gridDim.x) {
    const int64_t e0 = rowptr[row], e1 = rowptr[row + 1];
    __syncthreads();
    for (int i = tid; i < P; i += 256) {
      hist[i] = 0;
      wcnt[0][i] = wcnt[1][i] = wcnt[2][i] = wcnt[3][i] = 0;
    }
    __syncthreads();
    for (int64_t e = e0 + tid; e < e1; e += 256) atomicAdd(&hist[panel_of(colind[e])], 1);
    __syncthreads();
    // exclusive scan of the panel counts: each thread sums a run of consecutive panels, the
    // run totals are scanned by thread 0
    {
      const int per = (P + 255) / 256, p0 = tid * per;
      int s = 0;
      for (int q = p0; q < p0 + per && q < P; q++) s += hist[q];
      __syncthreads();
      if (p0 < P) cursor[p0] = s;  // run total, parked in the run's first slot
      __syncthreads();
      if (tid == 0) {
        int run = 0;
        for (int q = 0; q < P; q += per) {
          const int t = cursor[q];
          cursor[q] = run;
          run += t;
        }
      }
      __syncthreads();
      if (p0 < P) {
        int run = cursor[p0];
        for (int q = p0; q < p0 + per && q < P; q++) {
          cursor[q] = run;
          seg[row * (P + 1) + q] = e0 + run;
          run += hist[q];
        }
      }
    }
    if (tid == 0) seg[row * (P + 1) + P] = e1;
    __syncthreads();
    for (int64_t base = e0; base < e1; base += 256) {
      const int64_t e = base + tid;
      const bool active = e < e1;
      int32_t col = 0;
      float v = 0.0f;
      int pid = 0;
      if (active) {
        col = colind[e];
        v = vals[e];
        pid = panel_of(col);
      }
      unsigned long long mask = __ballot(active);
      for (int b = 0; b < bits; b++) {
        const bool bit = (pid >> b) & 1;
        const unsigned long long bal = __ballot(active && bit);
        mask &= bit ? bal : ~bal;
      }
      const int rank = __popcll(mask & ((1ull << lane) - 1ull));
      if (active && rank == 0) wcnt[wave][pid] = (uint8_t)__popcll(mask);
      __syncthreads();
      int off = 0, tot = 0;
      if (active) {
        for (int w = 0; w < 4; w++) {
          const int c = wcnt[w][pid];
          if (w < wave) off += c;
          tot += c;
        }
        const int64_t pos = e0 + cursor[pid] + off + rank;
        pcol[pos] = col;
        pval[pos] = v;
      }
      __syncthreads();
      // the last entry of each panel in the tile (last wave that holds it, last lane of its
      // mask) moves the panel's cursor on and clears its counts
      if (active) {
        bool last_wave = true;
        for (int w = wave + 1; w < 4; w++) last_wave = last_wave && wcnt[w][pid] == 0;
        if (last_wave && rank == __popcll(mask) - 1) cursor[pid] += tot;
      }
      __syncthreads();
      if (active && rank == 0) wcnt[wave][pid] = 0;
    }
  }
}

// idx_out / val_out [pos[i]] = (i, x[i] / divisor) for the elements that pass the threshold
__global__ void __launch_bounds__(256)
    k_threshold_write(const float* __restrict__ x, float divisor, float threshold, int64_t n,
                      const int64_t* __restrict__ pos, int32_t* __restrict__ idx_out,
                      float* __restrict__ val_out) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
    const float v = x[i] / divisor;
    if (v >= threshold) {
      idx_out[pos[i]] = (int32_t)i;
      val_out[pos[i]] = v;
    }
  }
}

__global__ void __launch_bounds__(256) k_fill_i32(int32_t* p, int64_t n, int32_t v) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) p[i] = v;
}

// old_to_new[kept[i]] = i; for a column listed twice the last position wins,
// as in the reference's sequential loop.
__global__ void __launch_bounds__(256)
    k_retain_table(const int32_t* __restrict__ kept, int64_t n_kept, int32_t* __restrict__ table) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n_kept; i += stride)
    atomicMax(&table[kept[i]], (int32_t)i);
}

__global__ void __launch_bounds__(256)
    k_remap_cols(int32_t* __restrict__ colind, int64_t nnz, const int32_t* __restrict__ table) {
  int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < nnz; e += stride)
    colind[e] = table[colind[e]];
}

// Order-preserving removal of entries whose column was dropped.
__global__ void __launch_bounds__(256)
    k_compact_entries(const int32_t* __restrict__ colind, const float* __restrict__ vals,
                      int64_t nnz, const int32_t* __restrict__ table,
                      const int64_t* __restrict__ newpos, int32_t* __restrict__ out_col,
                      float* __restrict__ out_val) {
  int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < nnz; e += stride) {
    int32_t c = table[colind[e]];
    if (c != -1) {
      int64_t p = newpos[e];
      out_col[p] = c;
      out_val[p] = vals[e];
    }
  }
}

__global__ void __launch_bounds__(256)
    k_remap_rowptr(int64_t* __restrict__ rowptr, int64_t n_rows, const int64_t* __restrict__ newpos) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i <= n_rows; i += stride)
    rowptr[i] = newpos[rowptr[i]];
}

// One row of the stable transposition: entry e of this row goes to the next
// free slot of its column.  Rows are issued in ascending order on one stream
// and a row holds each column at most once, so every column ends up in
// ascending row order.
__global__ void __launch_bounds__(256)
    k_transpose_row(int32_t row, int64_t e0, int64_t e1, const int32_t* __restrict__ colind,
                    const float* __restrict__ vals, const int64_t* __restrict__ colptr,
                    int* __restrict__ cursor, int32_t* __restrict__ rowind,
                    float* __restrict__ tvals) {
  int64_t e = e0 + (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= e1) return;
  int32_t j = colind[e];
  int64_t p = colptr[j] + atomicAdd(&cursor[j], 1);
  rowind[p] = row;
  tvals[p] = vals[e];
}

__global__ void __launch_bounds__(256)
    k_collect_long(const int64_t* __restrict__ colptr, int64_t limit, int64_t n_cols,
                   const int32_t* __restrict__ pos, int32_t* __restrict__ long_cols) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x; j < n_cols; j += stride)
    if (colptr[j + 1] - colptr[j] > limit) long_cols[pos[j]] = (int32_t)j;
}

__global__ void __launch_bounds__(256)
    k_sq_norm_partial(const float* __restrict__ v, int64_t n, double* __restrict__ partials) {
  __shared__ double sh[256];
  double s = 0.0;
  int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
    double x = (double)v[i];
    s += x * x;
  }
  sh[threadIdx.x] = s;
  __syncthreads();
  for (int off = 128; off > 0; off >>= 1) {
    if (threadIdx.x < off) sh[threadIdx.x] += sh[threadIdx.x + off];
    __syncthreads();
  }
  if (threadIdx.x == 0) partials[blockIdx.x] = sh[0];
}

// Grid of a grid-stride kernel over n items (every kernel launched with it loops); a launch is
// limited to 2^32 threads in total, so grids are capped well below that.
static unsigned grid_for(int64_t n, int64_t cap = 1 << 20) {
  int64_t g = ceil_div(n, 256);
  if (g < 1) g = 1;
  if (g > cap) g = cap;
  return (unsigned)g;
}

// Drops entries whose table[col] == -1 and renumbers the rest (in place on A).
static int apply_column_table(dnpeff_csr* A, const int32_t* table, int64_t new_n_cols) {
  hipStream_t st = stream();
  int64_t* newpos = nullptr;
  DN_TRY(dmalloc(&newpos, A->nnz + 1));
  DN_TRY(scan_kept_entries(A->colind, table, A->nnz, newpos));
  int64_t new_nnz = 0;
  DN_HIP(hipMemcpy(&new_nnz, newpos + A->nnz, sizeof(int64_t), hipMemcpyDeviceToHost));
  if (new_nnz == A->nnz) {
    hipLaunchKernelGGL(k_remap_cols, dim3(grid_for(A->nnz)), dim3(256), 0, st, A->colind, A->nnz,
                       table);
    DN_LAUNCH_CHECK();
  } else {
    int32_t* out_col = nullptr;
    float* out_val = nullptr;
    DN_TRY(dmalloc(&out_col, new_nnz));
    DN_TRY(dmalloc(&out_val, new_nnz));
    hipLaunchKernelGGL(k_compact_entries, dim3(grid_for(A->nnz)), dim3(256), 0, st, A->colind,
                       A->vals, A->nnz, table, newpos, out_col, out_val);
    hipLaunchKernelGGL(k_remap_rowptr, dim3(grid_for(A->n_rows + 1)), dim3(256), 0, st, A->rowptr,
                       A->n_rows, newpos);
    DN_LAUNCH_CHECK();
    DN_HIP(hipStreamSynchronize(st));
    dfree(A->colind);
    dfree(A->vals);
    A->colind = out_col;
    A->vals = out_val;
    A->nnz = new_nnz;
  }
  DN_HIP(hipStreamSynchronize(st));
  dfree(newpos);
  A->n_cols = new_n_cols;
  return 0;
}

static void drop_head(dnpeff_csr* A) {
  if (A->tail) {
    dnpeff_csr_destroy(A->tail);
    A->tail = nullptr;
  }
  dfree(A->head.cols); dfree(A->head.cm); dfree(A->head.rm); dfree(A->head.ws);
  A->head = dense_head();
}

static void drop_panels(dnpeff_csr* A) {
  dfree(A->panel_bounds); A->panel_bounds = nullptr;
  dfree(A->panel_ids); A->panel_ids = nullptr;
  dfree(A->sweep_progress); A->sweep_progress = nullptr;
  dfree(A->seg); A->seg = nullptr;
  dfree(A->pcol); A->pcol = nullptr;
  dfree(A->pval); A->pval = nullptr;
  if (A->n_panels) {  // the partial sums were sized for the panels
    dfree(A->partials); A->partials = nullptr; A->partials_floats = 0;
  }
  A->n_panels = A->n_plain = A->n_swept = 0;
  A->plan = panel_plan();
}

static void drop_derived(dnpeff_csr* A) {
  drop_head(A);
  drop_panels(A);
  dfree(A->colptr); A->colptr = nullptr;
  dfree(A->rowind); A->rowind = nullptr;
  dfree(A->tvals); A->tvals = nullptr;
  dfree(A->chunk_base); A->chunk_base = nullptr; A->n_chunks = 0;
  dfree(A->long_cols); A->long_cols = nullptr; A->n_long = 0;
  dfree(A->partials); A->partials = nullptr; A->partials_floats = 0;
}

int csr_ensure_chunks(dnpeff_csr* A) {
  if (A->chunk_base) return 0;
  DN_CHECK(A->rowptr != nullptr, "row-major copy of the matrix was released");
  DN_TRY(dmalloc(&A->chunk_base, A->n_rows + 1));
  DN_TRY(scan_row_chunks(A->rowptr, SPMM_N_CHUNK, A->n_rows, A->chunk_base));
  DN_HIP(hipMemcpy(&A->n_chunks, A->chunk_base + A->n_rows, sizeof(int64_t),
                   hipMemcpyDeviceToHost));
  return 0;
}

int csr_set_panels(dnpeff_csr* S, const panel_plan& plan) {
  if (plan == S->plan) return 0;
  drop_panels(S);
  const int P0 = plan.coarse;
  if (P0 <= 0) return 0;
  DN_CHECK(P0 <= MAX_PANELS, "at most %d column panels", MAX_PANELS);
  DN_CHECK(S->rowptr && S->colptr, "column panels need both copies of the matrix");
  hipStream_t st = stream();
  // coarse panels: equal numbers of entries
  std::vector<int32_t> coarse((size_t)P0 + 1);
  {
    int32_t* d_coarse = nullptr;
    DN_TRY(dmalloc(&d_coarse, (int64_t)P0 + 1));
    hipLaunchKernelGGL(k_panel_bounds, dim3((unsigned)ceil_div(P0 + 1, 256)), dim3(256), 0, st,
                       S->colptr, S->n_cols, S->nnz, P0, d_coarse);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e == hipSuccess)
      e = hipMemcpy(coarse.data(), d_coarse, sizeof(int32_t) * coarse.size(), hipMemcpyDeviceToHost);
    dfree(d_coarse);
    DN_CHECK(e == hipSuccess, "building the column panels failed: %s", hipGetErrorString(e));
  }
  // A coarse panel whose part of the factor does not fit one L2 is cut into pieces that do, when
  // the rows hold entries enough per piece to be worth a segment each; those pieces are swept
  // (spmm.hip).  A raised threshold keeps the number of panels within bounds.
  std::vector<int32_t> bounds, ids, swept;
  double min_seg = plan.sweep_min;
  for (;;) {
    bounds.clear(); ids.clear(); swept.clear();
    const double per_coarse = (double)S->nnz / P0 / (double)(S->n_rows > 0 ? S->n_rows : 1);
    for (int c = 0; c < P0; c++) {
      const int64_t w = (int64_t)coarse[c + 1] - coarse[c];
      const bool sweep = plan.sweep_cols > 0 && w > plan.sweep_cols + plan.sweep_cols / 4 &&
                         per_coarse * (double)plan.sweep_cols / (double)w >= min_seg;
      const int64_t parts = sweep ? ceil_div(w, plan.sweep_cols) : 1;
      for (int64_t q = 0; q < parts; q++) {
        (sweep ? swept : ids).push_back((int32_t)bounds.size());
        bounds.push_back((int32_t)(coarse[c] + w * q / parts));
      }
    }
    if ((int64_t)bounds.size() <= MAX_PANELS) break;
    min_seg = min_seg > 0.0 ? min_seg * 1.5 : 1.0;
  }
  bounds.push_back((int32_t)S->n_cols);
  const int P = (int)bounds.size() - 1;
  const int n_plain = (int)ids.size(), n_swept = (int)swept.size();
  ids.insert(ids.end(), swept.begin(), swept.end());

  int bits = 0;
  while ((1 << bits) < P) bits++;
  int s = dmalloc(&S->panel_bounds, (int64_t)P + 1) || dmalloc(&S->panel_ids, (int64_t)P) ||
          dmalloc(&S->sweep_progress, 256) ||
          dmalloc(&S->seg, S->n_rows * (P + 1)) || dmalloc(&S->pcol, S->nnz + 64) ||
          dmalloc(&S->pval, S->nnz + 64);  // (the sweep kernel reads 64 pairs at a time)
  if (!s) {
    hipError_t e = hipMemcpy(S->panel_bounds, bounds.data(), sizeof(int32_t) * bounds.size(),
                             hipMemcpyHostToDevice);
    if (e == hipSuccess)
      e = hipMemcpy(S->panel_ids, ids.data(), sizeof(int32_t) * ids.size(), hipMemcpyHostToDevice);
    if (e == hipSuccess) {
      int64_t wgs = S->n_rows < 8192 ? S->n_rows : 8192;
      hipLaunchKernelGGL(k_panel_split, dim3((unsigned)(wgs < 1 ? 1 : wgs)), dim3(256), 0, st,
                         S->rowptr, S->colind, S->vals, S->n_rows, P, bits, S->panel_bounds, S->seg,
                         S->pcol, S->pval);
      e = hipGetLastError();
      if (e == hipSuccess) e = hipStreamSynchronize(st);
    }
    if (e != hipSuccess) {
      set_error("building the column panels failed: %s", hipGetErrorString(e));
      s = 1;
    }
  }
  if (s) { drop_panels(S); return s; }
  S->n_panels = P;
  S->n_plain = n_plain;
  S->n_swept = n_swept;
  S->plan = plan;
  if (getenv("DNPEFF_VERBOSE"))
    fprintf(stderr, "dnpeff: %d column panels: %d plain, %d cut into %d swept pieces\n", P0, n_plain,
            P0 - n_plain, n_swept);
  dfree(S->partials); S->partials = nullptr; S->partials_floats = 0;
  return 0;
}

// Panels pay when the gathered factor [n_cols, r] is far larger than the caches and there are
// rows enough to share a panel's part of it: one coarse panel per ~48 MB of the factor, 8..512
// (per ~96 MB, 8..256, at the ranks that have swept pieces), and few enough for the (panel, 4
// rows) workgroups to fit one launch.  On 10,000 x 65.9M,
// r = 128 (33.7 GB factor): no panels 29.3 ms, 32: 27.8, 128: 23.9, 256: 21.8, 512: 20.1 ms for
// the gathers, plus 0.1 to 0.8 ms for the sum over panels; 1024 gains 1.1 ms and loses 0.7.
// DNPEFF_PANELS overrides the number (0 = none).  Swept pieces hold DNPEFF_SWEEP_BYTES of the
// factor each (default 3 MB of the 4 MB L2 of an XCD; 0 = no sweeps) and are made where a row
// holds DNPEFF_SWEEP_MIN entries per piece on average (default 4, more when there are few rows).
static panel_plan panel_policy(const dnpeff_csr* S, int r) {
  int64_t P = 0;
  const double bytes = 4.0 * (double)S->n_cols * r;
  bool sweeps = spmm_n_sweep_supported(r);
  if (const char* e = getenv("DNPEFF_SWEEP_BYTES")) sweeps = sweeps && atof(e) > 0.0;
  if (bytes >= 512e6 && S->n_rows >= 64) {
    // with swept pieces for the panels in between, half as many coarse panels do as well for the
    // gathers and halve the sum over the panels (configs[1]: 19.8 -> 19.4 ms for both)
    P = (int64_t)ceil(bytes / (sweeps ? 96e6 : 48e6));
    if (P < 8) P = 8;
    if (P > (sweeps ? 256 : 512)) P = sweeps ? 256 : 512;
  }
  if (const char* e = getenv("DNPEFF_PANELS")) P = atoi(e);
  if (P > 512) P = 512;
  const int64_t row_groups = ceil_div(S->n_rows, 4);
  while (P > 1 && P * row_groups >= ((int64_t)1 << 24)) P /= 2;
  if (P < 2 || S->nnz == 0) P = 0;
  panel_plan plan;
  plan.coarse = (int)P;
  if (P > 0 && sweeps) {
    double sweep_bytes = 3.0 * 1024 * 1024;
    if (const char* e = getenv("DNPEFF_SWEEP_BYTES")) sweep_bytes = atof(e);
    if (sweep_bytes > 1e9) sweep_bytes = 1e9;  // (the kernel addresses a piece with 32 bits)
    plan.sweep_cols = (int)(sweep_bytes / (4.0 * r));
    // a piece must also bring work enough for a sweep step (a wait for the other workgroups of
    // the XCD and two barriers): 20,000 entries over all rows
    plan.sweep_min = 4.0;
    if (S->n_rows > 0 && 20000.0 / (double)S->n_rows > plan.sweep_min)
      plan.sweep_min = 20000.0 / (double)S->n_rows;
    if (const char* e = getenv("DNPEFF_SWEEP_MIN")) plan.sweep_min = atof(e);
    if (plan.sweep_cols <= 0) plan.sweep_cols = 0, plan.sweep_min = 0.0;
  }
  return plan;
}

int csr_ensure_products(dnpeff_csr* A, int r) {
  dnpeff_csr* S = sparse_part(A);
  DN_TRY(dnpeff_csr_build_transpose(S));
  DN_TRY(csr_set_panels(S, panel_policy(S, r)));
  DN_TRY(csr_ensure_partials(S, r));
  return head_ensure_workspace(A, r);
}

int csr_ensure_partials(dnpeff_csr* A, int r) {
  DN_TRY(csr_ensure_chunks(A));
  int64_t need = A->n_chunks * (int64_t)r;
  if (A->n_panels > 0 && A->n_rows * panel_slots(A) * (int64_t)r > need)
    need = A->n_rows * panel_slots(A) * (int64_t)r;
  if (need <= A->partials_floats && A->partials) return 0;
  dfree(A->partials);
  A->partials = nullptr;
  DN_TRY(dmalloc(&A->partials, need));
  A->partials_floats = need;
  return 0;
}

}  // namespace dn

using namespace dn;

// ---------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------

DN_API const char* dnpeff_last_error(void) { return g_error; }

DN_API int dnpeff_device_count(int* count) {
  DN_CHECK(count != nullptr, "count is NULL");
  int c = 0;
  hipError_t e = hipGetDeviceCount(&c);
  if (e != hipSuccess) c = 0;
  *count = c;
  return 0;
}

DN_API int dnpeff_device_info(char* name, int name_len, int64_t* total_bytes, int* n_cus_out) {
  hipDeviceProp_t p;
  DN_HIP(hipGetDeviceProperties(&p, 0));
  if (name && name_len > 0) {
    strncpy(name, p.name, (size_t)name_len - 1);
    name[name_len - 1] = 0;
  }
  if (total_bytes) *total_bytes = (int64_t)p.totalGlobalMem;
  if (n_cus_out) *n_cus_out = p.multiProcessorCount;
  return 0;
}

DN_API int dnpeff_sync(void) {
  DN_HIP(hipStreamSynchronize(stream()));
  return 0;
}

DN_API void* dnpeff_stream(void) { return (void*)stream(); }

DN_API int dnpeff_dev_malloc(int64_t bytes, void** out) {
  clear_error();
  DN_CHECK(out != nullptr && bytes >= 0, "bad arguments");
  char* p = nullptr;
  DN_TRY(dmalloc(&p, bytes));
  *out = p;
  return 0;
}

DN_API int dnpeff_dev_free(void* p) {
  if (!p) return 0;
  DN_HIP(hipStreamSynchronize(stream()));
  DN_HIP(hipFree(p));
  return 0;
}

DN_API int dnpeff_dev_upload(void* dst_dev, const void* src_host, int64_t bytes) {
  clear_error();
  DN_CHECK(bytes >= 0 && (bytes == 0 || (dst_dev && src_host)), "bad arguments");
  DN_HIP(hipStreamSynchronize(stream()));
  if (bytes) DN_HIP(hipMemcpy(dst_dev, src_host, (size_t)bytes, hipMemcpyHostToDevice));
  return 0;
}

DN_API int dnpeff_dev_download(void* dst_host, const void* src_dev, int64_t bytes) {
  clear_error();
  DN_CHECK(bytes >= 0 && (bytes == 0 || (dst_host && src_dev)), "bad arguments");
  DN_HIP(hipStreamSynchronize(stream()));
  if (bytes) DN_HIP(hipMemcpy(dst_host, src_dev, (size_t)bytes, hipMemcpyDeviceToHost));
  return 0;
}

DN_API int64_t dnpeff_size_of_split(int64_t total, int64_t n_splits, int64_t split_index) {
  if (n_splits <= 0 || split_index < 0 || split_index >= n_splits) return -1;
  int64_t base = total / n_splits;
  return split_index == n_splits - 1 ? base + total % n_splits : base;
}

static int validate_host_csr(int64_t n_rows, int64_t n_cols, int64_t nnz, const int64_t* rowptr) {
  DN_CHECK(n_rows >= 0 && n_cols >= 0 && nnz >= 0, "negative matrix dimension");
  DN_CHECK(n_rows < (int64_t)INT32_MAX && n_cols < (int64_t)INT32_MAX,
           "n_rows and n_cols must fit 32-bit ids");
  DN_CHECK(rowptr != nullptr, "rowptr is NULL");
  DN_CHECK(rowptr[0] == 0 && rowptr[n_rows] == nnz, "rowptr[0] must be 0 and rowptr[n_rows] == nnz");
  for (int64_t i = 0; i < n_rows; i++)
    DN_CHECK(rowptr[i] <= rowptr[i + 1], "rowptr decreases at row %lld", (long long)i);
  return 0;
}

__global__ void __launch_bounds__(256)
    k_check_cols(const int32_t* __restrict__ colind, int64_t nnz, int64_t n_cols, int* bad) {
  int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < nnz; e += stride) {
    int32_t c = colind[e];
    if (c < 0 || c >= n_cols) atomicAdd(bad, 1);
  }
}

static int check_cols_in_range(const dnpeff_csr* A) {
  int* bad = nullptr;
  DN_TRY(dmalloc(&bad, 1));
  DN_HIP(hipMemsetAsync(bad, 0, sizeof(int), stream()));
  hipLaunchKernelGGL(k_check_cols, dim3(grid_for(A->nnz)), dim3(256), 0, stream(), A->colind,
                     A->nnz, A->n_cols, bad);
  DN_LAUNCH_CHECK();
  int h = 0;
  DN_HIP(hipMemcpy(&h, bad, sizeof(int), hipMemcpyDeviceToHost));
  dfree(bad);
  DN_CHECK(h == 0, "%d column ids outside [0, n_cols)", h);
  return 0;
}

DN_API int dnpeff_csr_from_host(int64_t n_rows, int64_t n_cols, int64_t nnz, const int64_t* rowptr,
                                const int32_t* colind, const float* vals, dnpeff_csr** out) {
  clear_error();
  DN_CHECK(out != nullptr, "out is NULL");
  *out = nullptr;
  DN_TRY(validate_host_csr(n_rows, n_cols, nnz, rowptr));
  DN_CHECK(nnz == 0 || (colind && vals), "colind/vals are NULL");
  dnpeff_csr* A = new dnpeff_csr();
  A->n_rows = n_rows; A->n_cols = n_cols; A->nnz = nnz; A->full_dense_size = n_cols;
  int s = dmalloc(&A->rowptr, n_rows + 1) || dmalloc(&A->colind, nnz) || dmalloc(&A->vals, nnz);
  if (s) { dnpeff_csr_destroy(A); return 1; }
  hipError_t e = hipMemcpy(A->rowptr, rowptr, sizeof(int64_t) * (n_rows + 1), hipMemcpyHostToDevice);
  if (e == hipSuccess && nnz)
    e = hipMemcpy(A->colind, colind, sizeof(int32_t) * nnz, hipMemcpyHostToDevice);
  if (e == hipSuccess && nnz)
    e = hipMemcpy(A->vals, vals, sizeof(float) * nnz, hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    set_error("upload of the CSR arrays failed: %s", hipGetErrorString(e));
    dnpeff_csr_destroy(A);
    return 1;
  }
  if (check_cols_in_range(A)) { dnpeff_csr_destroy(A); return 2; }
  *out = A;
  return 0;
}

DN_API int dnpeff_csr_from_pef(int64_t n_rows, int64_t k, int64_t dense_fisher_size,
                               const int32_t* indices, const float* values, dnpeff_csr** out) {
  clear_error();
  DN_CHECK(out != nullptr, "out is NULL");
  *out = nullptr;
  DN_CHECK(n_rows >= 0 && k >= 0 && dense_fisher_size >= 0, "negative dimension");
  DN_CHECK(n_rows < (int64_t)INT32_MAX && dense_fisher_size < (int64_t)INT32_MAX,
           "n_rows and dense_fisher_size must fit 32-bit ids");
  int64_t nnz = n_rows * k;
  DN_CHECK(nnz == 0 || (indices && values), "indices/values are NULL");
  dnpeff_csr* A = new dnpeff_csr();
  A->n_rows = n_rows; A->n_cols = dense_fisher_size; A->nnz = nnz;
  A->full_dense_size = dense_fisher_size;
  int s = dmalloc(&A->rowptr, n_rows + 1) || dmalloc(&A->colind, nnz) || dmalloc(&A->vals, nnz);
  if (s) { dnpeff_csr_destroy(A); return 1; }
  hipLaunchKernelGGL(k_pef_rowptr, dim3(grid_for(n_rows + 1)), dim3(256), 0, stream(), n_rows, k,
                     A->rowptr);
  hipError_t e = hipGetLastError();
  if (e == hipSuccess && nnz)
    e = hipMemcpy(A->colind, indices, sizeof(int32_t) * nnz, hipMemcpyHostToDevice);
  if (e == hipSuccess && nnz)
    e = hipMemcpy(A->vals, values, sizeof(float) * nnz, hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipStreamSynchronize(stream());
  if (e != hipSuccess) {
    set_error("upload of the PEF arrays failed: %s", hipGetErrorString(e));
    dnpeff_csr_destroy(A);
    return 1;
  }
  if (check_cols_in_range(A)) { dnpeff_csr_destroy(A); return 2; }
  *out = A;
  return 0;
}

DN_API int dnpeff_csr_normalize_rows(dnpeff_csr* A, const float* norms_host, float eps) {
  clear_error();
  DN_CHECK(A && A->rowptr, "matrix is NULL or released");
  DN_CHECK(norms_host != nullptr || A->n_rows == 0, "norms is NULL");
  if (A->n_rows == 0) return 0;
  float* norms = nullptr;
  DN_TRY(dmalloc(&norms, A->n_rows));
  DN_HIP(hipMemcpy(norms, norms_host, sizeof(float) * A->n_rows, hipMemcpyHostToDevice));
  unsigned grid = (unsigned)(A->n_rows < 65536 ? A->n_rows : 65536);
  hipLaunchKernelGGL(k_normalize_rows, dim3(grid), dim3(256), 0, stream(), A->rowptr, A->vals,
                     norms, eps, A->n_rows);
  DN_LAUNCH_CHECK();
  DN_HIP(hipStreamSynchronize(stream()));
  dfree(norms);
  drop_derived(A);
  return 0;
}

DN_API int dnpeff_csr_compact_columns(dnpeff_csr* A, int min_count) {
  clear_error();
  DN_CHECK(A && A->rowptr, "matrix is NULL or released");
  hipStream_t st = stream();
  drop_derived(A);
  const int64_t m_full = A->n_cols;
  int* count = nullptr;
  int32_t *pos = nullptr, *og_to_new = nullptr, *new_to_og = nullptr;
  DN_TRY(dmalloc(&count, m_full));
  DN_HIP(hipMemsetAsync(count, 0, sizeof(int) * (size_t)(m_full > 0 ? m_full : 1), st));
  hipLaunchKernelGGL(k_col_hist, dim3(grid_for(A->nnz, 65536)), dim3(256), 0, st, A->colind, A->nnz,
                     count);
  DN_LAUNCH_CHECK();
  DN_TRY(dmalloc(&pos, m_full + 1));
  DN_TRY(scan_keep_mask(count, min_count, m_full, pos));
  int32_t m_new = 0;
  DN_HIP(hipMemcpy(&m_new, pos + m_full, sizeof(int32_t), hipMemcpyDeviceToHost));
  DN_TRY(dmalloc(&og_to_new, m_full));
  DN_TRY(dmalloc(&new_to_og, (int64_t)m_new));
  hipLaunchKernelGGL(k_build_maps, dim3(grid_for(m_full)), dim3(256), 0, st, count, min_count, pos,
                     m_full, og_to_new, new_to_og);
  DN_LAUNCH_CHECK();
  DN_HIP(hipStreamSynchronize(st));
  dfree(count);
  dfree(pos);
  A->full_dense_size = m_full;
  int s = apply_column_table(A, og_to_new, (int64_t)m_new);
  dfree(og_to_new);
  if (s) { dfree(new_to_og); return s; }
  dfree(A->kept);
  A->kept = new_to_og;
  return 0;
}

DN_API int dnpeff_csr_retain_columns(dnpeff_csr* A, const int32_t* kept, int64_t n_kept) {
  clear_error();
  DN_CHECK(A && A->rowptr, "matrix is NULL or released");
  DN_CHECK(n_kept >= 0 && (kept || n_kept == 0), "kept is NULL");
  for (int64_t i = 0; i < n_kept; i++)
    DN_CHECK(kept[i] >= 0 && kept[i] < A->n_cols, "kept[%lld] = %d outside [0, %lld)",
             (long long)i, kept[i], (long long)A->n_cols);
  hipStream_t st = stream();
  drop_derived(A);
  int32_t *table = nullptr, *kept_dev = nullptr;
  DN_TRY(dmalloc(&table, A->n_cols));
  DN_TRY(dmalloc(&kept_dev, n_kept));
  if (n_kept) DN_HIP(hipMemcpy(kept_dev, kept, sizeof(int32_t) * n_kept, hipMemcpyHostToDevice));
  hipLaunchKernelGGL(k_fill_i32, dim3(grid_for(A->n_cols)), dim3(256), 0, st, table, A->n_cols, -1);
  hipLaunchKernelGGL(k_retain_table, dim3(grid_for(n_kept)), dim3(256), 0, st, kept_dev, n_kept,
                     table);
  DN_LAUNCH_CHECK();
  A->full_dense_size = A->n_cols;
  int s = apply_column_table(A, table, n_kept);
  dfree(table);
  if (s) { dfree(kept_dev); return s; }
  dfree(A->kept);
  A->kept = kept_dev;
  return 0;
}

DN_API int dnpeff_csr_shape(const dnpeff_csr* A, int64_t* n_rows, int64_t* n_cols, int64_t* nnz) {
  DN_CHECK(A != nullptr, "matrix is NULL");
  if (n_rows) *n_rows = A->n_rows;
  if (n_cols) *n_cols = A->n_cols;
  if (nnz) *nnz = A->nnz;
  return 0;
}

DN_API int dnpeff_csr_full_dense_size(const dnpeff_csr* A, int64_t* out) {
  DN_CHECK(A && out, "NULL argument");
  *out = A->full_dense_size;
  return 0;
}

DN_API int dnpeff_csr_download(const dnpeff_csr* A, int64_t* rowptr, int32_t* colind, float* vals) {
  clear_error();
  DN_CHECK(A && A->rowptr, "matrix is NULL or released");
  DN_HIP(hipStreamSynchronize(stream()));
  if (rowptr)
    DN_HIP(hipMemcpy(rowptr, A->rowptr, sizeof(int64_t) * (A->n_rows + 1), hipMemcpyDeviceToHost));
  if (colind && A->nnz)
    DN_HIP(hipMemcpy(colind, A->colind, sizeof(int32_t) * A->nnz, hipMemcpyDeviceToHost));
  if (vals && A->nnz)
    DN_HIP(hipMemcpy(vals, A->vals, sizeof(float) * A->nnz, hipMemcpyDeviceToHost));
  return 0;
}

DN_API int dnpeff_csr_kept_indices(const dnpeff_csr* A, int32_t* new_to_og) {
  clear_error();
  DN_CHECK(A && new_to_og, "NULL argument");
  if (A->kept) {
    if (A->n_cols)
      DN_HIP(hipMemcpy(new_to_og, A->kept, sizeof(int32_t) * A->n_cols, hipMemcpyDeviceToHost));
  } else {
    for (int64_t i = 0; i < A->n_cols; i++) new_to_og[i] = (int32_t)i;
  }
  return 0;
}

DN_API int dnpeff_csr_sq_norm(const dnpeff_csr* A, double* out) {
  clear_error();
  DN_CHECK(A && out, "NULL argument");
  const float* v = A->vals ? A->vals : A->tvals;
  DN_CHECK(v != nullptr || A->nnz == 0, "both copies of the matrix were released");
  const int blocks = 1024;
  double* partials = nullptr;
  DN_TRY(dmalloc(&partials, blocks));
  hipLaunchKernelGGL(k_sq_norm_partial, dim3(blocks), dim3(256), 0, stream(), v, A->nnz, partials);
  DN_LAUNCH_CHECK();
  std::vector<double> h(blocks);
  DN_HIP(hipMemcpy(h.data(), partials, sizeof(double) * blocks, hipMemcpyDeviceToHost));
  dfree(partials);
  double s = 0.0;
  for (int i = 0; i < blocks; i++) s += h[i];
  *out = s;
  return 0;
}

DN_API int dnpeff_csr_split_dense_head(dnpeff_csr* A, double min_fill, int64_t* n_dense) {
  clear_error();
  DN_CHECK(A && A->rowptr, "matrix is NULL or released");
  DN_CHECK(min_fill <= 1.0, "min_fill %g above 1", min_fill);
  hipStream_t st = stream();
  drop_derived(A);
  if (n_dense) *n_dense = 0;
  if (min_fill <= 0.0) return 0;
  const int64_t m = A->n_cols, n = A->n_rows;
  if (m == 0 || n == 0 || A->nnz == 0) return 0;
  int64_t thr = (int64_t)ceil(min_fill * (double)n);
  if (thr < 1) thr = 1;
  int* count = nullptr;
  int32_t *pos = nullptr, *slot_of = nullptr, *cols = nullptr, *table = nullptr;
  DN_TRY(dmalloc(&count, m));
  DN_HIP(hipMemsetAsync(count, 0, sizeof(int) * (size_t)m, st));
  hipLaunchKernelGGL(k_col_hist, dim3(grid_for(A->nnz, 65536)), dim3(256), 0, st, A->colind, A->nnz,
                     count);
  DN_LAUNCH_CHECK();
  DN_TRY(dmalloc(&pos, m + 1));
  // both dense blocks together stay below an eighth of the device memory: raise the bar
  // until they do
  size_t free_b = 0, total_b = 0;
  DN_HIP(hipMemGetInfo(&free_b, &total_b));
  const int64_t n_pad = ceil_div(n, 128) * 128;
  int32_t n_d = 0;
  for (;;) {
    DN_CHECK(thr <= (int64_t)INT32_MAX, "dense head: threshold overflow");
    DN_TRY(scan_keep_mask(count, (int)thr, m, pos));
    DN_HIP(hipMemcpy(&n_d, pos + m, sizeof(int32_t), hipMemcpyDeviceToHost));
    const double bytes = 2.0 * 4.0 * (double)n_pad * (double)(ceil_div(n_d, 128) * 128);
    if (bytes <= (double)total_b / 8.0 || thr > n) break;
    thr *= 2;
  }
  if (n_d == 0 || thr > n) {
    dfree(count); dfree(pos);
    return 0;
  }
  const int64_t n_d_pad = ceil_div(n_d, 128) * 128;
  int s = dmalloc(&slot_of, m) || dmalloc(&cols, (int64_t)n_d) || dmalloc(&table, m);
  if (!s) {
    hipLaunchKernelGGL(k_build_maps, dim3(grid_for(m)), dim3(256), 0, st, count, (int)thr, pos, m,
                       slot_of, cols);
    hipLaunchKernelGGL(k_tail_table, dim3(grid_for(m)), dim3(256), 0, st, slot_of, m, table);
  }
  dense_head& h = A->head;
  if (!s) s = dmalloc(&h.cm, n_d_pad * n_pad) || dmalloc(&h.rm, n_pad * n_d_pad);
  if (!s && (hipMemsetAsync(h.cm, 0, sizeof(float) * (size_t)(n_d_pad * n_pad), st) != hipSuccess ||
             hipMemsetAsync(h.rm, 0, sizeof(float) * (size_t)(n_pad * n_d_pad), st) != hipSuccess)) {
    set_error("dense head: clearing the blocks failed");
    s = 1;
  }
  if (!s) {
    hipLaunchKernelGGL(k_head_fill, dim3(grid_for(n * 256)), dim3(256), 0, st, A->rowptr, A->colind,
                       A->vals, n, slot_of, h.cm, n_pad, h.rm, n_d_pad);
    if (hipGetLastError() != hipSuccess) { set_error("dense head: launch failed"); s = 1; }
  }
  // the remaining entries: a copy of the row-major arrays without the head's columns
  dnpeff_csr* T = nullptr;
  if (!s) {
    T = new dnpeff_csr();
    T->n_rows = n; T->n_cols = m; T->nnz = A->nnz; T->full_dense_size = A->full_dense_size;
    s = dmalloc(&T->rowptr, n + 1) || dmalloc(&T->colind, A->nnz) || dmalloc(&T->vals, A->nnz);
    if (!s && (hipMemcpyAsync(T->rowptr, A->rowptr, sizeof(int64_t) * (n + 1), hipMemcpyDeviceToDevice, st) != hipSuccess ||
               hipMemcpyAsync(T->colind, A->colind, sizeof(int32_t) * A->nnz, hipMemcpyDeviceToDevice, st) != hipSuccess ||
               hipMemcpyAsync(T->vals, A->vals, sizeof(float) * A->nnz, hipMemcpyDeviceToDevice, st) != hipSuccess)) {
      set_error("dense head: copying the entries failed");
      s = 1;
    }
    if (!s) s = apply_column_table(T, table, m);
  }
  (void)hipStreamSynchronize(st);
  dfree(count); dfree(pos); dfree(slot_of); dfree(table);
  if (s) {
    if (T) dnpeff_csr_destroy(T);
    dfree(cols);
    drop_head(A);
    return s;
  }
  h.n_d = n_d; h.n_d_pad = n_d_pad; h.n_pad = n_pad; h.cols = cols;
  A->tail = T;
  if (n_dense) *n_dense = n_d;
  return 0;
}

DN_API int dnpeff_op_threshold_compact(int64_t count, const float* x, float divisor, float threshold,
                                       int32_t* idx_out, float* val_out, int64_t* n_kept) {
  clear_error();
  DN_CHECK(count >= 0 && count <= (int64_t)INT32_MAX, "count %lld outside [0, 2^31)", (long long)count);
  DN_CHECK((x && idx_out && val_out) || count == 0, "NULL argument");
  DN_CHECK(n_kept != nullptr, "n_kept is NULL");
  DN_CHECK(divisor != 0.0f, "divisor is zero");
  *n_kept = 0;
  if (count == 0) return 0;
  int64_t* pos = nullptr;
  DN_TRY(dmalloc(&pos, count + 1));
  int s = exclusive_scan(GeThresholdF{x, divisor, threshold}, count, pos);
  if (!s) {
    hipLaunchKernelGGL(k_threshold_write, dim3(grid_for(count)), dim3(256), 0, stream(), x, divisor,
                       threshold, count, pos, idx_out, val_out);
    if (hipGetLastError() != hipSuccess ||
        hipMemcpy(n_kept, pos + count, sizeof(int64_t), hipMemcpyDeviceToHost) != hipSuccess) {
      set_error("threshold compaction failed");
      s = 1;
    }
  }
  (void)hipStreamSynchronize(stream());
  dfree(pos);
  return s;
}

DN_API int dnpeff_csr_head_info(const dnpeff_csr* A, int64_t* n_dense, int64_t* nnz_sparse) {
  DN_CHECK(A != nullptr, "matrix is NULL");
  if (n_dense) *n_dense = A->head.n_d;
  if (nnz_sparse) *nnz_sparse = sparse_part(A)->nnz;
  return 0;
}

DN_API int dnpeff_csr_build_transpose(dnpeff_csr* A) {
  clear_error();
  DN_CHECK(A != nullptr, "matrix is NULL");
  if (A->colptr) return 0;
  DN_CHECK(A->rowptr != nullptr, "row-major copy of the matrix was released");
  hipStream_t st = stream();
  const int64_t m = A->n_cols;
  int* count = nullptr;
  DN_TRY(dmalloc(&count, m));
  DN_HIP(hipMemsetAsync(count, 0, sizeof(int) * (size_t)(m > 0 ? m : 1), st));
  hipLaunchKernelGGL(k_col_hist, dim3(grid_for(A->nnz, 65536)), dim3(256), 0, st, A->colind, A->nnz,
                     count);
  DN_LAUNCH_CHECK();
  DN_TRY(dmalloc(&A->colptr, m + 1));
  DN_TRY(scan_counts_i64(count, m, A->colptr));
  DN_TRY(dmalloc(&A->rowind, A->nnz));
  DN_TRY(dmalloc(&A->tvals, A->nnz));
  DN_HIP(hipMemsetAsync(count, 0, sizeof(int) * (size_t)(m > 0 ? m : 1), st));
  std::vector<int64_t> rowptr((size_t)A->n_rows + 1);
  DN_HIP(hipMemcpy(rowptr.data(), A->rowptr, sizeof(int64_t) * (A->n_rows + 1),
                   hipMemcpyDeviceToHost));
  for (int64_t i = 0; i < A->n_rows; i++) {
    int64_t len = rowptr[i + 1] - rowptr[i];
    if (len <= 0) continue;
    hipLaunchKernelGGL(k_transpose_row, dim3((unsigned)ceil_div(len, 256)), dim3(256), 0, st,
                       (int32_t)i, rowptr[i], rowptr[i + 1], A->colind, A->vals, A->colptr, count,
                       A->rowind, A->tvals);
  }
  DN_LAUNCH_CHECK();
  DN_HIP(hipStreamSynchronize(st));
  dfree(count);
  // list of long columns for A^T W
  int32_t* pos = nullptr;
  DN_TRY(dmalloc(&pos, m + 1));
  DN_TRY(scan_long_cols(A->colptr, SPMM_T_LONG, m, pos));
  int32_t n_long = 0;
  DN_HIP(hipMemcpy(&n_long, pos + m, sizeof(int32_t), hipMemcpyDeviceToHost));
  A->n_long = n_long;
  DN_TRY(dmalloc(&A->long_cols, (int64_t)n_long));
  if (n_long) {
    hipLaunchKernelGGL(k_collect_long, dim3(grid_for(m)), dim3(256), 0, st, A->colptr, SPMM_T_LONG,
                       m, pos, A->long_cols);
    DN_LAUNCH_CHECK();
  }
  DN_HIP(hipStreamSynchronize(st));
  dfree(pos);
  return 0;
}

DN_API int dnpeff_csr_download_transpose(dnpeff_csr* A, int64_t* colptr, int32_t* rowind,
                                         float* vals) {
  clear_error();
  DN_TRY(dnpeff_csr_build_transpose(A));
  if (colptr)
    DN_HIP(hipMemcpy(colptr, A->colptr, sizeof(int64_t) * (A->n_cols + 1), hipMemcpyDeviceToHost));
  if (rowind && A->nnz)
    DN_HIP(hipMemcpy(rowind, A->rowind, sizeof(int32_t) * A->nnz, hipMemcpyDeviceToHost));
  if (vals && A->nnz)
    DN_HIP(hipMemcpy(vals, A->tvals, sizeof(float) * A->nnz, hipMemcpyDeviceToHost));
  return 0;
}

DN_API int dnpeff_csr_release(dnpeff_csr* A, int which) {
  clear_error();
  DN_CHECK(A != nullptr, "matrix is NULL");
  DN_HIP(hipStreamSynchronize(stream()));
  if (which == 1) {
    dfree(A->colind); A->colind = nullptr;
    dfree(A->vals); A->vals = nullptr;
    dfree(A->rowptr); A->rowptr = nullptr;
    dfree(A->chunk_base); A->chunk_base = nullptr; A->n_chunks = 0;
    dfree(A->partials); A->partials = nullptr; A->partials_floats = 0;
  } else if (which == 2) {
    dfree(A->colptr); A->colptr = nullptr;
    dfree(A->rowind); A->rowind = nullptr;
    dfree(A->tvals); A->tvals = nullptr;
    dfree(A->long_cols); A->long_cols = nullptr; A->n_long = 0;
  } else {
    DN_CHECK(false, "which must be 1 (row-major copy) or 2 (transposed copy)");
  }
  return 0;
}

DN_API int dnpeff_csr_destroy(dnpeff_csr* A) {
  if (!A) return 0;
  (void)hipStreamSynchronize(stream());
  drop_derived(A);
  dfree(A->rowptr);
  dfree(A->colind);
  dfree(A->vals);
  dfree(A->kept);
  delete A;
  return 0;
}
