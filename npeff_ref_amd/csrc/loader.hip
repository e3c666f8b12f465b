// CSR loader on the device: upload, row normalisation, column compaction,
// column retention, transposed CSR, ||A||^2.  Integer results are bit-exact
// with the reference's host code; see include/dnpeff.h for the citations.
#include "dnpeff_internal.hpp"
#include "scan.hpp"

#include <cmath>
#include <cstdlib>

#include <algorithm>
#include <cctype>
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

static hipStream_t g_side_stream = nullptr;
static bool g_on_side_stream = false;
static hipEvent_t g_side_done = nullptr;  // recorded on the side stream; nullptr = nothing pending

hipStream_t stream() {
  if (g_on_side_stream) return g_side_stream;
  if (!g_stream) {
    if (hipStreamCreate(&g_stream) != hipSuccess) {
      fprintf(stderr, "dnpeff: hipStreamCreate failed (no usable GPU?)\n");
      abort();
    }
  }
  return g_stream;
}

// Work launched between side_stream_begin() and side_stream_end() goes to a second stream of the
// same (default) priority: it starts once everything launched so far on the library stream has
// finished, and runs beside what the library stream gets afterwards, until side_stream_join()
// makes the library stream wait for it.
int side_stream_begin() {
  if (!g_side_stream) DN_HIP(hipStreamCreate(&g_side_stream));
  static hipEvent_t fork = nullptr;
  if (!fork) DN_HIP(hipEventCreateWithFlags(&fork, hipEventDisableTiming));
  DN_HIP(hipEventRecord(fork, stream()));
  DN_HIP(hipStreamWaitEvent(g_side_stream, fork, 0));
  g_on_side_stream = true;
  return 0;
}
int side_stream_end() {
  static hipEvent_t done = nullptr;
  if (!done) DN_HIP(hipEventCreateWithFlags(&done, hipEventDisableTiming));
  g_on_side_stream = false;
  DN_HIP(hipEventRecord(done, g_side_stream));
  g_side_done = done;
  return 0;
}
int side_stream_join() {
  if (!g_side_done) return 0;
  hipEvent_t e = g_side_done;
  g_side_done = nullptr;
  DN_HIP(hipStreamWaitEvent(stream(), e, 0));
  return 0;
}

// The two streams by themselves, and where stream() points, for callers that order work between
// them with events of their own.
hipStream_t side_stream_handle() {
  if (!g_side_stream && hipStreamCreate(&g_side_stream) != hipSuccess) return nullptr;
  return g_side_stream;
}
void side_stream_route(bool on) { g_on_side_stream = on && g_side_stream != nullptr; }
bool side_stream_routed() { return g_on_side_stream; }
bool side_stream_pending() { return g_side_done != nullptr; }

int n_cus() {
  if (!g_n_cus) {
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, 0) == hipSuccess) g_n_cus = p.multiProcessorCount;
    if (g_n_cus <= 0) g_n_cus = 256;
  }
  return g_n_cus;
}

struct tuning_entry {
  const char* name;
  double tuning_t::*field;
};
static const tuning_entry g_tuning_table[] = {
    {"dense_fill", &tuning_t::dense_fill},       {"panels", &tuning_t::panels},
    {"sweep_bytes", &tuning_t::sweep_bytes},     {"sweep_min", &tuning_t::sweep_min},
    {"sweep_waves", &tuning_t::sweep_waves},     {"sweep_lag", &tuning_t::sweep_lag},
    {"sweep_spin", &tuning_t::sweep_spin},       {"spmm_t_slices", &tuning_t::spmm_t_slices},
    {"split_bf16", &tuning_t::split_bf16},       {"fused_gram", &tuning_t::fused_gram},
    {"h_tile_mb", &tuning_t::h_tile_mb},         {"tiled_h", &tuning_t::tiled_h},
    {"topk_fast_cap", &tuning_t::topk_fast_cap}, {"verbose", &tuning_t::verbose},
    {"n_lists", &tuning_t::n_lists},             {"t_lists", &tuning_t::t_lists},
    {"nl_piece_cols", &tuning_t::nl_piece_cols}, {"nl_lag", &tuning_t::nl_lag},
    {"nl_extra_mb", &tuning_t::nl_extra_mb},
    {"nl_spin", &tuning_t::nl_spin},             {"nl_wgs", &tuning_t::nl_wgs},
    {"gram_beside", &tuning_t::gram_beside},
    {"gram_fold", &tuning_t::gram_fold},         {"xg_wgs", &tuning_t::xg_wgs},
    {"h_overlap", &tuning_t::h_overlap},
};

static tuning_t tuning_from_env() {
  tuning_t t;
  for (const tuning_entry& e : g_tuning_table) {
    char var[64] = "DNPEFF_";
    size_t k = strlen(var);
    for (const char* c = e.name; *c && k + 1 < sizeof(var); c++) var[k++] = (char)toupper((unsigned char)*c);
    var[k] = 0;
    if (const char* v = getenv(var)) t.*(e.field) = atof(v);
  }
  return t;
}

tuning_t& tuning() {
  static tuning_t t = tuning_from_env();
  return t;
}

// ids[b] = XCD that workgroup b of the probe runs on (hardware register XCC_ID, bits 3:0)
__global__ void k_xcd_probe(int* ids) {
  if (threadIdx.x == 0) ids[blockIdx.x] = __builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11)) & 15;
}

// The kernels that pin work to an XCD (swept pieces of A H^T, component slices of A^T W) count on
// the dispatcher dealing the workgroups of a launch to SWEEP_XCDS XCDs round-robin by their
// number: workgroups b, b + 8, b + 16, ... on one XCD, the eight classes on eight different ones
// (which XCD a class gets does not matter).  Checked once per process with a probe launch; where
// it does not hold (another partition mode, another part) those plans are not made: plain
// panels, one slice.
bool xcd_round_robin() {
  static int state = -1;
  if (state >= 0) return state == 1;
  state = 0;
  constexpr int N = 64 * SWEEP_XCDS;
  int* ids = nullptr;
  if (dmalloc(&ids, N)) return false;
  int h[N];
  hipLaunchKernelGGL(k_xcd_probe, dim3(N), dim3(64), 0, stream(), ids);
  if (hipGetLastError() == hipSuccess &&
      hipMemcpy(h, ids, sizeof(int) * N, hipMemcpyDeviceToHost) == hipSuccess) {
    bool ok = true;
    unsigned seen = 0;
    for (int x = 0; x < SWEEP_XCDS; x++) {
      for (int b = x; b < N; b += SWEEP_XCDS) ok = ok && h[b] == h[x];
      ok = ok && !(seen & (1u << h[x]));
      seen |= 1u << h[x];
    }
    state = ok ? 1 : 0;
  }
  dfree(ids);
  clear_error();
  if (state == 0 && tuning().verbose != 0.0)
    fprintf(stderr, "dnpeff: workgroups are not dealt to %d XCDs round-robin: no swept pieces, no "
                    "component slices\n", SWEEP_XCDS);
  return state == 1;
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

// Entries of the head's columns into the dense block; a workgroup per row.  Every element must
// receive one addition: an addition that finds something other than zero in its element means
// that the row holds the column twice (*repeats counts them; a repeat whose earlier values were
// all exactly zero goes unnoticed and changes nothing: 0 + x has one value whatever the order).
__global__ void __launch_bounds__(256)
    k_head_fill(const int64_t* __restrict__ rowptr, const int32_t* __restrict__ colind,
                const float* __restrict__ vals, int64_t n_rows, const int32_t* __restrict__ slot_of,
                float* __restrict__ cm, int64_t n_pad, int* __restrict__ repeats) {
  for (int64_t row = blockIdx.x; row < n_rows; row += gridDim.x) {
    const int64_t e1 = rowptr[row + 1];
    for (int64_t e = rowptr[row] + threadIdx.x; e < e1; e += 256) {
      const int32_t k = slot_of[colind[e]];
      if (k >= 0 && atomicAdd(&cm[(int64_t)k * n_pad + row], vals[e]) != 0.0f) atomicAdd(repeats, 1);
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
                  int32_t* __restrict__ pcol, float* __restrict__ pval,
                  const int64_t* __restrict__ out_begin) {
  // out_begin (or NULL): the panels end below the matrix's last column; row i's entries below
  // bounds[P] (out_begin[i + 1] - out_begin[i] of them, anywhere in the row) go to
  // out_begin[i] .. of pcol / pval, and the segment offsets count from there; the others are left
  // out
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
    const int64_t o0 = out_begin ? out_begin[row] : e0;
    const int64_t o1 = out_begin ? out_begin[row + 1] : e1;
    const int32_t col_end = bounds[P];
    __syncthreads();
    for (int i = tid; i < P; i += 256) {
      hist[i] = 0;
      wcnt[0][i] = wcnt[1][i] = wcnt[2][i] = wcnt[3][i] = 0;
    }
    __syncthreads();
    for (int64_t e = e0 + tid; e < e1; e += 256)
      if (colind[e] < col_end) atomicAdd(&hist[panel_of(colind[e])], 1);
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
          seg[row * (P + 1) + q] = o0 + run;
          run += hist[q];
        }
      }
    }
    if (tid == 0) seg[row * (P + 1) + P] = o1;
    __syncthreads();
    for (int64_t base = e0; base < e1; base += 256) {
      const int64_t e = base + tid;
      bool active = e < e1;
      int32_t col = 0;
      float v = 0.0f;
      int pid = 0;
      if (active) {
        col = colind[e];
        active = col < col_end;
      }
      if (active) {
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
        const int64_t pos = o0 + cursor[pid] + off + rank;
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

// sum over the columns with count >= thr of their counts (an integer sum: any order)
__global__ void __launch_bounds__(256)
    k_sum_selected(const int* __restrict__ count, int64_t n, int thr, unsigned long long* out) {
  __shared__ unsigned long long sh[256];
  unsigned long long s = 0;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
    const int c = count[i];
    if (c >= thr) s += (unsigned long long)c;
  }
  sh[threadIdx.x] = s;
  __syncthreads();
  for (int off = 128; off > 0; off >>= 1) {
    if (threadIdx.x < off) sh[threadIdx.x] += sh[threadIdx.x + off];
    __syncthreads();
  }
  if (threadIdx.x == 0 && sh[0]) atomicAdd(out, sh[0]);
}

// bad += 1 for every column that holds the same row twice in a row of its list (after the stable
// transposition the entries of one row of a column are adjacent)
__global__ void __launch_bounds__(256)
    k_check_repeats(const int64_t* __restrict__ colptr, const int32_t* __restrict__ rowind,
                    int64_t n_cols, int* __restrict__ bad) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x; j < n_cols; j += stride) {
    const int64_t p1 = colptr[j + 1];
    int32_t prev = -1;
    bool rep = false;
    for (int64_t p = colptr[j]; p < p1; p++) {
      const int32_t i = rowind[p];
      rep = rep || i == prev;
      prev = i;
    }
    if (rep) atomicAdd(bad, 1);
  }
}

// Drops entries whose table[col] == -1 and renumbers the rest (in place on A).
static int apply_column_table(dnpeff_csr* A, const int32_t* table, int64_t new_n_cols) {
  hipStream_t st = stream();
  dbuf<int64_t> newpos;
  DN_TRY(newpos.alloc(A->nnz + 1));
  DN_TRY(scan_kept_entries(A->colind, table, A->nnz, newpos));
  int64_t new_nnz = 0;
  DN_HIP(hipMemcpy(&new_nnz, newpos + A->nnz, sizeof(int64_t), hipMemcpyDeviceToHost));
  if (new_nnz == A->nnz) {
    hipLaunchKernelGGL(k_remap_cols, dim3(grid_for(A->nnz)), dim3(256), 0, st, A->colind, A->nnz,
                       table);
    DN_LAUNCH_CHECK();
  } else {
    dbuf<int32_t> out_col;
    dbuf<float> out_val;
    DN_TRY(out_col.alloc(new_nnz));
    DN_TRY(out_val.alloc(new_nnz));
    hipLaunchKernelGGL(k_compact_entries, dim3(grid_for(A->nnz)), dim3(256), 0, st, A->colind,
                       A->vals, A->nnz, table, newpos.p, out_col.p, out_val.p);
    hipLaunchKernelGGL(k_remap_rowptr, dim3(grid_for(A->n_rows + 1)), dim3(256), 0, st, A->rowptr,
                       A->n_rows, newpos.p);
    DN_LAUNCH_CHECK();
    DN_HIP(hipStreamSynchronize(st));
    dfree(A->colind);
    dfree(A->vals);
    A->colind = out_col.release();
    A->vals = out_val.release();
    A->nnz = new_nnz;
  }
  DN_HIP(hipStreamSynchronize(st));
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
  dfree(A->sweep_perm); A->sweep_perm = nullptr; A->sweep_perm_key = 0;
  dfree(A->seg); A->seg = nullptr;
  dfree(A->pcol); A->pcol = nullptr;
  dfree(A->pval); A->pval = nullptr;
  dfree(A->prow); A->prow = nullptr;
  A->tail_floor = 0;
  if (A->n_panels) {  // the partial sums were sized for the panels
    dfree(A->partials); A->partials = nullptr; A->partials_floats = 0;
  }
  A->n_panels = A->n_plain = A->n_swept = 0;
  A->plan = panel_plan();
}

static void drop_derived(dnpeff_csr* A) {
  A->h_lists_valid = false;
  A->tail_declined = false;
  drop_head(A);
  drop_panels(A);
  nlists_drop(A);
  tblocks_drop(A);
  dfree(A->colptr); A->colptr = nullptr;
  dfree(A->rowind); A->rowind = nullptr;
  dfree(A->tvals); A->tvals = nullptr;
  dfree(A->slots); A->slots = nullptr;
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
  DN_CHECK(has_row_major(S) && S->colptr, "column panels need both copies of the matrix");
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
  int P_used = P0;  // coarse panels that stay panels
  for (;;) {
    bounds.clear(); ids.clear(); swept.clear();
    const double per_coarse = (double)S->nnz / P0 / (double)(S->n_rows > 0 ? S->n_rows : 1);
    auto sweeps = [&](int c) {
      const int64_t w = (int64_t)coarse[c + 1] - coarse[c];
      return plan.sweep_cols > 0 && w > plan.sweep_cols + plan.sweep_cols / 4 &&
             per_coarse * (double)plan.sweep_cols / (double)w >= min_seg;
    };
    // The far tail: the plain panels past the last swept one.  With tail_lists their entries go
    // to slot lists and the panels end at the first of them.
    P_used = P0;
    if (plan.tail_lists) {
      int last_swept = -1;
      for (int c = 0; c < P0; c++)
        if (sweeps(c)) last_swept = c;
      if (last_swept >= 0 && last_swept + 1 < P0 && coarse[last_swept + 1] > 0) P_used = last_swept + 1;
    }
    for (int c = 0; c < P_used; c++) {
      const int64_t w = (int64_t)coarse[c + 1] - coarse[c];
      const bool sweep = sweeps(c);
      const int64_t parts = sweep ? ceil_div(w, plan.sweep_cols) : 1;
      for (int64_t q = 0; q < parts; q++) {
        (sweep ? swept : ids).push_back((int32_t)bounds.size());
        bounds.push_back((int32_t)(coarse[c] + w * q / parts));
      }
    }
    if ((int64_t)bounds.size() <= MAX_PANELS) break;
    min_seg = min_seg > 0.0 ? min_seg * 1.5 : 1.0;
  }
  const int32_t tail_floor = P_used < P0 ? coarse[P_used] : 0;
  bounds.push_back(tail_floor > 0 ? tail_floor : (int32_t)S->n_cols);
  const int P = (int)bounds.size() - 1;
  // rows' places in the panel copy when it leaves the far tail out
  int64_t nnz_panels = S->nnz;
  if (tail_floor > 0) {
    dbuf<int> below;
    int s0 = below.alloc(S->n_rows) || dmalloc(&S->prow, S->n_rows + 1) ||
             csr_rows_count_below(S, tail_floor, below.p) ||
             scan_counts_i64(below.p, S->n_rows, S->prow);
    if (!s0 && hipMemcpy(&nnz_panels, S->prow + S->n_rows, sizeof(int64_t), hipMemcpyDeviceToHost) != hipSuccess) {
      set_error("building the column panels failed (row prefixes)");
      s0 = 1;
    }
    if (s0) { drop_panels(S); return 1; }
  }
  const int n_plain = (int)ids.size(), n_swept = (int)swept.size();
  ids.insert(ids.end(), swept.begin(), swept.end());

  int bits = 0;
  while ((1 << bits) < P) bits++;
  int s = dmalloc(&S->panel_bounds, (int64_t)P + 1) || dmalloc(&S->panel_ids, (int64_t)P) ||
          dmalloc(&S->sweep_progress, 256) ||
          dmalloc(&S->seg, S->n_rows * (P + 1)) || dmalloc(&S->pcol, nnz_panels + 64) ||
          dmalloc(&S->pval, nnz_panels + 64);  // (the sweep kernel reads 64 pairs at a time)
  if (!s) {
    hipError_t e = hipMemcpy(S->panel_bounds, bounds.data(), sizeof(int32_t) * bounds.size(),
                             hipMemcpyHostToDevice);
    if (e == hipSuccess)
      e = hipMemcpy(S->panel_ids, ids.data(), sizeof(int32_t) * ids.size(), hipMemcpyHostToDevice);
    if (e == hipSuccess) {
      int64_t wgs = S->n_rows < 8192 ? S->n_rows : 8192;
      hipLaunchKernelGGL(k_panel_split, dim3((unsigned)(wgs < 1 ? 1 : wgs)), dim3(256), 0, st,
                         S->rowptr, S->colind, S->vals, S->n_rows, P, bits, S->panel_bounds, S->seg,
                         S->pcol, S->pval, (const int64_t*)S->prow);
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
  S->tail_floor = tail_floor;
  if (tuning().verbose != 0.0) {
    fprintf(stderr, "dnpeff: %d column panels: %d plain, %d cut into %d swept pieces", P_used, n_plain,
            P_used - n_plain, n_swept);
    if (tail_floor > 0)
      fprintf(stderr, "; the %d panels from column %d on (%lld entries) go to slot lists", P0 - P_used,
              (int)tail_floor, (long long)(S->nnz - nnz_panels));
    fprintf(stderr, "\n");
  }
  dfree(S->partials); S->partials = nullptr; S->partials_floats = 0;
  return 0;
}

// Panels pay when the gathered factor [n_cols, r] is far larger than the caches and there are
// rows enough to share a panel's part of it: one coarse panel per ~48 MB of the factor, 8..512
// (per ~96 MB, 8..256, at the ranks that have swept pieces), few enough for the (panel, 4
// rows) workgroups to fit one launch and for the partial sums (one [n_rows, r] block per plain
// panel) to stay within 3 GB.  On 10,000 x 65.9M,
// r = 128 (33.7 GB factor): no panels 29.3 ms, 32: 27.8, 128: 23.9, 256: 21.8, 512: 20.1 ms for
// the gathers, plus 0.1 to 0.8 ms for the sum over panels; 1024 gains 1.1 ms and loses 0.7.
// The `panels` switch overrides the number (0 = none).  Swept pieces hold `sweep_bytes` of the
// factor each (default 3 MB of the 4 MB L2 of an XCD; 0 = no sweeps) and are made where a row
// holds `sweep_min` entries per piece on average (default 4, more when there are few rows).
// Coarse panels for a sparse part of n_rows x n_cols at rank r (0 = none); `sweeps`: the rank and
// the machine have swept pieces.
int64_t coarse_panels_for(int64_t n_rows, int64_t n_cols, int r, bool sweeps) {
  const tuning_t& tn = tuning();
  int64_t P = 0;
  const double bytes = 4.0 * (double)n_cols * r;
  if (bytes >= 512e6 && n_rows >= 64) {
    // with swept pieces for the panels in between, half as many coarse panels do as well for the
    // gathers and halve the sum over the panels (configs[1]: 19.8 -> 19.4 ms for both)
    P = (int64_t)ceil(bytes / (sweeps ? 96e6 : 48e6));
    if (P < 8) P = 8;
    if (P > (sweeps ? 256 : 512)) P = sweeps ? 256 : 512;
    const int64_t by_partials = (int64_t)(PANEL_PARTIALS_BYTES / (4.0 * (double)n_rows * r));
    if (P > by_partials) P = by_partials < 8 ? 8 : by_partials;
  }
  if (tn.panels >= 0.0) P = (int64_t)tn.panels;
  if (P > 512) P = 512;
  const int64_t row_groups = ceil_div(n_rows, 4);
  while (P > 1 && P * row_groups >= ((int64_t)1 << 24)) P /= 2;
  return P < 2 ? 0 : P;
}
bool sweeps_for_rank(int r) { return spmm_n_sweep_supported(r) && tuning().sweep_bytes > 0.0 && xcd_round_robin(); }
int max_panels() { return MAX_PANELS; }

static panel_plan panel_policy(const dnpeff_csr* S, int r) {
  const tuning_t& tn = tuning();
  const bool sweeps = sweeps_for_rank(r);
  int64_t P = coarse_panels_for(S->n_rows, S->n_cols, r, sweeps);
  if (S->nnz == 0) P = 0;
  panel_plan plan;
  plan.coarse = (int)P;
  if (P > 0 && sweeps) {
    double sweep_bytes = tn.sweep_bytes;
    if (sweep_bytes > 1e9) sweep_bytes = 1e9;  // (the kernel addresses a piece with 32 bits)
    plan.sweep_cols = (int)(sweep_bytes / (4.0 * sweep_width(r)));  // (a piece of one slice)
    // a piece must also bring work enough for a sweep step (a wait for the other workgroups of
    // the XCD and two barriers): 20,000 entries over all rows
    plan.sweep_min = 4.0;
    if (S->n_rows > 0 && 20000.0 / (double)S->n_rows > plan.sweep_min)
      plan.sweep_min = 20000.0 / (double)S->n_rows;
    if (tn.sweep_min >= 0.0) plan.sweep_min = tn.sweep_min;
    if (plan.sweep_cols <= 0) plan.sweep_cols = 0, plan.sweep_min = 0.0;
  }
  return plan;
}

// The products of a sparse part run on component slices (lists.hip) only when the switches
// n_lists / t_lists ask for it (1): at the sizes measured they are slower than the panels, swept
// pieces and 4-slice column kernel that the plan uses otherwise.  Needs a rank that is a multiple
// of 32 and workgroups dealt to the XCDs round-robin.
bool use_nlists(const dnpeff_csr* S, int r) {
  return tuning().n_lists == 1.0 && nlists_supported(S, r) && xcd_round_robin();
}
// The far tail only (the plain panels past the last swept one) on slot lists, beside the panels
// and swept pieces of the columns before it: n_lists = 2 wherever the lists can be built; left to
// itself (n_lists < 0) where it was measured to pay: ranks from 256 (eight slices or more: one per
// XCD, the entry streams read once per slice) and four rows or more per lane group (with fewer,
// the groups' lists of a piece are short and uneven, and most of a batch is filler): 195 against
// 221 ms for A H^T at 20,000 x 211M, r = 256, 397 against 462 ms at 40,000 ragged rows, r = 512,
// but 20.6 against 19.6 ms at 10,000 rows, r = 128.
bool use_nlists_tail(const dnpeff_csr* S, int r) {
  const double sw = tuning().n_lists;
  if (!(sw == 2.0 || sw < 0.0) || !nlists_supported(S, r) || !xcd_round_robin()) return false;
  if (sw == 2.0) return true;
  return r >= 256 && S->n_rows >= 4 * 8 * (int64_t)nlists_slots(S->n_rows, r);
}
bool use_tlists(const dnpeff_csr* S, int r) {
  return tuning().t_lists > 0.0 && tlists_supported(S, r) && xcd_round_robin();
}

int csr_ensure_products(dnpeff_csr* A, int r) {
  dnpeff_csr* S = sparse_part(A);
  DN_TRY(dnpeff_csr_build_transpose(S));
  if (use_nlists(S, r)) {
    DN_TRY(csr_set_panels(S, panel_plan()));
    DN_TRY(nlists_build(S, r));
  } else {
    panel_plan plan = panel_policy(S, r);
    plan.tail_lists = plan.coarse > 0 && plan.sweep_cols > 0 && use_nlists_tail(S, r) && !S->tail_declined;
    DN_TRY(csr_set_panels(S, plan));
    if (S->tail_floor > 0) {
      // Left to itself, the plan gives the lists what the panel copy of the same entries would
      // take plus half of the memory that the plan keeps free; beyond that the tail stays panels.
      bool declined = false;
      double bound = -1.0;
      if (!(S->nl.pairs && S->nl.floor_col == S->tail_floor)) {  // (lists that exist are not judged again)
        size_t free_b = 0, total_b = 0;
        DN_HIP(hipMemGetInfo(&free_b, &total_b));
        if (tuning().n_lists < 0.0) bound = (double)total_b / 128.0;
        if (tuning().nl_extra_mb >= 0.0) bound = tuning().nl_extra_mb * 1048576.0;
      }
      DN_TRY(nlists_build(S, r, S->tail_floor, bound, &declined));
      if (declined) {
        S->tail_declined = true;  // (later calls must come to the same plan: the matrix may be consumed by then)
        plan.tail_lists = false;
        DN_TRY(csr_set_panels(S, plan));
      }
    } else {
      nlists_drop(S);
    }
  }
  if (use_tlists(S, r)) DN_TRY(tblocks_build(S));
  DN_TRY(csr_ensure_partials(S, r));
  return head_ensure_workspace(A, r);
}

int csr_consume_for_products(dnpeff_csr* A) {
  DN_HIP(hipStreamSynchronize(stream()));
  dnpeff_csr* S = sparse_part(A);
  if (A->tail) {  // the products read the dense head and the tail, not the whole matrix
    dfree(A->colind); A->colind = nullptr;
    dfree(A->vals); A->vals = nullptr;
    dfree(A->chunk_base); A->chunk_base = nullptr; A->n_chunks = 0;
    dfree(A->partials); A->partials = nullptr; A->partials_floats = 0;
  }
  if ((S->n_panels > 0 || S->nl.pairs) && S->nnz > 0) {  // A H^T reads the regrouped copy / the slot lists
    DN_TRY(csr_ensure_chunks(S));  // (sizes the partial sums; needs the row offsets only)
    dfree(S->colind); S->colind = nullptr;
    dfree(S->vals); S->vals = nullptr;
  }
  return 0;
}

int csr_tile_lists(dnpeff_csr* A) {
  if (A->h_lists_valid) return 0;
  const dnpeff_csr* S = sparse_part(A);
  A->h_head_cols.assign((size_t)A->head.n_d, 0);
  A->h_long_cols.assign((size_t)S->n_long, 0);
  DN_HIP(hipStreamSynchronize(stream()));
  if (A->head.n_d)
    DN_HIP(hipMemcpy(A->h_head_cols.data(), A->head.cols, sizeof(int32_t) * A->head.n_d,
                     hipMemcpyDeviceToHost));
  if (S->n_long)
    DN_HIP(hipMemcpy(A->h_long_cols.data(), S->long_cols, sizeof(int32_t) * S->n_long,
                     hipMemcpyDeviceToHost));
  A->h_lists_valid = true;
  return 0;
}

int csr_ensure_partials(dnpeff_csr* A, int r) {
  DN_TRY(csr_ensure_chunks(A));
  int64_t need = A->n_chunks * (int64_t)r;
  if (A->n_panels > 0 && A->n_rows * panel_slots(A) * (int64_t)r > need)
    need = A->n_rows * panel_slots(A) * (int64_t)r;
  if (A->nl.pairs && A->n_rows * (int64_t)r > need) need = A->n_rows * (int64_t)r;
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

DN_API int dnpeff_tuning_set(const char* name, double value) {
  clear_error();
  DN_CHECK(name != nullptr, "name is NULL");
  for (const tuning_entry& e : g_tuning_table)
    if (strcmp(e.name, name) == 0) {
      tuning().*(e.field) = value;
      return 0;
    }
  DN_CHECK(false, "no tuning switch named '%s'", name);
  return 0;
}

DN_API int dnpeff_tuning_get(const char* name, double* value) {
  clear_error();
  DN_CHECK(name && value, "NULL argument");
  for (const tuning_entry& e : g_tuning_table)
    if (strcmp(e.name, name) == 0) {
      *value = tuning().*(e.field);
      return 0;
    }
  DN_CHECK(false, "no tuning switch named '%s'", name);
  return 0;
}

DN_API int dnpeff_tuning_reset(void) {
  tuning() = tuning_from_env();
  return 0;
}

DN_API int dnpeff_device_memory(int64_t* free_bytes, int64_t* total_bytes) {
  clear_error();
  size_t f = 0, t = 0;
  DN_HIP(hipMemGetInfo(&f, &t));
  if (free_bytes) *free_bytes = (int64_t)f;
  if (total_bytes) *total_bytes = (int64_t)t;
  return 0;
}

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
  DN_CHECK(A && has_row_major(A), "matrix is NULL or its row-major arrays were released");
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
  A->sq_norm_valid = false;
  return 0;
}

DN_API int dnpeff_csr_compact_columns(dnpeff_csr* A, int min_count) {
  clear_error();
  DN_CHECK(A && has_row_major(A), "matrix is NULL or its row-major arrays were released");
  hipStream_t st = stream();
  drop_derived(A);
  A->sq_norm_valid = false;
  const int64_t m_full = A->n_cols;
  dbuf<int> count;
  dbuf<int32_t> pos, og_to_new, new_to_og;
  DN_TRY(count.alloc(m_full));
  DN_HIP(hipMemsetAsync(count, 0, sizeof(int) * (size_t)(m_full > 0 ? m_full : 1), st));
  hipLaunchKernelGGL(k_col_hist, dim3(grid_for(A->nnz, 65536)), dim3(256), 0, st, A->colind, A->nnz,
                     count.p);
  DN_LAUNCH_CHECK();
  DN_TRY(pos.alloc(m_full + 1));
  DN_TRY(scan_keep_mask(count, min_count, m_full, pos));
  int32_t m_new = 0;
  DN_HIP(hipMemcpy(&m_new, pos + m_full, sizeof(int32_t), hipMemcpyDeviceToHost));
  DN_TRY(og_to_new.alloc(m_full));
  DN_TRY(new_to_og.alloc((int64_t)m_new));
  hipLaunchKernelGGL(k_build_maps, dim3(grid_for(m_full)), dim3(256), 0, st, count.p, min_count,
                     pos.p, m_full, og_to_new.p, new_to_og.p);
  DN_LAUNCH_CHECK();
  DN_HIP(hipStreamSynchronize(st));
  count.reset();
  pos.reset();
  A->full_dense_size = m_full;
  DN_TRY(apply_column_table(A, og_to_new, (int64_t)m_new));
  dfree(A->kept);
  A->kept = new_to_og.release();
  return 0;
}

DN_API int dnpeff_csr_retain_columns(dnpeff_csr* A, const int32_t* kept, int64_t n_kept) {
  clear_error();
  DN_CHECK(A && has_row_major(A), "matrix is NULL or its row-major arrays were released");
  DN_CHECK(n_kept >= 0 && (kept || n_kept == 0), "kept is NULL");
  for (int64_t i = 0; i < n_kept; i++)
    DN_CHECK(kept[i] >= 0 && kept[i] < A->n_cols, "kept[%lld] = %d outside [0, %lld)",
             (long long)i, kept[i], (long long)A->n_cols);
  hipStream_t st = stream();
  drop_derived(A);
  A->sq_norm_valid = false;
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
  DN_CHECK(A && has_row_major(A), "matrix is NULL or its row-major arrays were released");
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
  if (A->sq_norm_valid) {
    *out = A->sq_norm;
    return 0;
  }
  // (with a dense head the whole matrix's values only exist in the row-major copy)
  const float* v = A->vals ? A->vals : (A->tail ? nullptr : A->tvals);
  DN_CHECK(v != nullptr || A->nnz == 0, "the row-major copy of the matrix was released before its norm was taken");
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
  dnpeff_csr* M = const_cast<dnpeff_csr*>(A);
  M->sq_norm = s;
  M->sq_norm_valid = true;
  return 0;
}

// rowptr_out[i] = newpos[rowptr[i]]
__global__ void __launch_bounds__(256)
    k_map_rowptr(const int64_t* __restrict__ rowptr, int64_t n_rows, const int64_t* __restrict__ newpos,
                 int64_t* __restrict__ rowptr_out) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i <= n_rows; i += stride)
    rowptr_out[i] = newpos[rowptr[i]];
}

namespace dn {

// Which columns form the dense head.  Candidates are the thresholds thr0, 2 thr0, 4 thr0, ...
// (thr0 = ceil(min_fill n_rows)) and "no head"; a candidate is admissible when its dense blocks
// (n_blocks of them: one where the products read it in both directions, two otherwise) stay
// below a sixth of the device memory; its footprint is the blocks plus both sparse copies of
// the remaining entries (16 bytes each).  The choice is the first admissible candidate
// whose footprint is within `budget` bytes (NO_BUDGET: the first admissible one), else the
// admissible candidate with the smallest footprint (fits = false).
int choose_dense_head(dnpeff_csr* A, double min_fill, double budget, int n_blocks, int rank, head_choice* out) {
  *out = head_choice();
  out->footprint = 16.0 * (double)A->nnz;
  out->fits = out->footprint <= budget;
  const int64_t m = A->n_cols, n = A->n_rows;
  if (min_fill <= 0.0 || m == 0 || n == 0 || A->nnz == 0) return 0;
  DN_CHECK(has_row_major(A), "matrix is NULL or its row-major arrays were released");
  hipStream_t st = stream();
  dbuf<int> count;
  dbuf<int32_t> pos;
  dbuf<unsigned long long> zsum;
  DN_TRY(count.alloc(m));
  DN_TRY(pos.alloc(m + 1));
  DN_TRY(zsum.alloc(1));
  DN_HIP(hipMemsetAsync(count, 0, sizeof(int) * (size_t)m, st));
  hipLaunchKernelGGL(k_col_hist, dim3(grid_for(A->nnz, 65536)), dim3(256), 0, st, A->colind, A->nnz,
                     count.p);
  DN_LAUNCH_CHECK();
  size_t free_b = 0, total_b = 0;
  DN_HIP(hipMemGetInfo(&free_b, &total_b));
  const int64_t n_pad = ceil_div(n, 128) * 128;
  int64_t thr = (int64_t)ceil(min_fill * (double)n);
  if (thr < 1) thr = 1;
  head_choice best = *out;  // "no head"
  bool have_fit = false;
  // candidates a fifth apart (a doubled threshold can leave a quarter of the budget unused)
  for (; thr <= n && thr <= (int64_t)INT32_MAX; thr = std::max(thr + 1, thr + thr / 5)) {
    int32_t n_d = 0;
    unsigned long long z_head = 0;
    DN_TRY(scan_keep_mask(count, (int)thr, m, pos));
    DN_HIP(hipMemcpy(&n_d, pos + m, sizeof(int32_t), hipMemcpyDeviceToHost));
    if (n_d == 0) break;
    DN_HIP(hipMemsetAsync(zsum, 0, sizeof(unsigned long long), st));
    hipLaunchKernelGGL(k_sum_selected, dim3(grid_for(m, 4096)), dim3(256), 0, st, count.p, m, (int)thr,
                       zsum.p);
    DN_LAUNCH_CHECK();
    DN_HIP(hipMemcpy(&z_head, zsum, sizeof(unsigned long long), hipMemcpyDeviceToHost));
    const double blocks = n_blocks * 4.0 * (double)n_pad * (double)(ceil_div(n_d, 128) * 128);
    if (blocks > (double)total_b / 6.0) continue;
    head_choice c;
    c.thr = thr;
    c.n_d = n_d;
    c.footprint = blocks + 16.0 * (double)(A->nnz - (int64_t)z_head) +
                  (rank > 0 ? 4.0 * (double)head_workspace_floats(n, n_d, rank) : 0.0);
    c.fits = c.footprint <= budget;
    if (c.fits) {
      best = c;
      have_fit = true;
      break;
    }
    if (c.footprint < best.footprint) best = c;
  }
  if (!have_fit && out->fits) return 0;  // no head fits the budget, a head does not
  *out = best;
  return 0;
}

// Moves the columns with at least thr entries into the dense head.
int split_dense_head_at(dnpeff_csr* A, int64_t thr, int64_t* n_dense) {
  hipStream_t st = stream();
  drop_derived(A);
  if (n_dense) *n_dense = 0;
  const int64_t m = A->n_cols, n = A->n_rows;
  if (thr <= 0 || thr > n || m == 0 || A->nnz == 0) return 0;
  DN_CHECK(has_row_major(A), "matrix is NULL or its row-major arrays were released");
  dbuf<int> count;
  dbuf<int32_t> pos, slot_of, cols, table;
  DN_TRY(count.alloc(m));
  DN_HIP(hipMemsetAsync(count, 0, sizeof(int) * (size_t)m, st));
  hipLaunchKernelGGL(k_col_hist, dim3(grid_for(A->nnz, 65536)), dim3(256), 0, st, A->colind, A->nnz,
                     count.p);
  DN_LAUNCH_CHECK();
  DN_TRY(pos.alloc(m + 1));
  DN_TRY(scan_keep_mask(count, (int)thr, m, pos));
  int32_t n_d = 0;
  DN_HIP(hipMemcpy(&n_d, pos + m, sizeof(int32_t), hipMemcpyDeviceToHost));
  if (n_d == 0) return 0;
  const int64_t n_pad = ceil_div(n, 128) * 128, n_d_pad = ceil_div(n_d, 128) * 128;
  DN_TRY(slot_of.alloc(m));
  DN_TRY(cols.alloc((int64_t)n_d));
  DN_TRY(table.alloc(m));
  hipLaunchKernelGGL(k_build_maps, dim3(grid_for(m)), dim3(256), 0, st, count.p, (int)thr, pos.p, m,
                     slot_of.p, cols.p);
  hipLaunchKernelGGL(k_tail_table, dim3(grid_for(m)), dim3(256), 0, st, slot_of.p, m, table.p);
  DN_LAUNCH_CHECK();
  DN_HIP(hipStreamSynchronize(st));
  count.reset();
  pos.reset();
  dbuf<float> cm;
  DN_TRY(cm.alloc(n_d_pad * n_pad));
  DN_HIP(hipMemsetAsync(cm, 0, sizeof(float) * (size_t)(n_d_pad * n_pad), st));
  {
    dbuf<int> repeats;
    DN_TRY(repeats.alloc(1));
    DN_HIP(hipMemsetAsync(repeats, 0, sizeof(int), st));
    hipLaunchKernelGGL(k_head_fill, dim3(grid_for(n * 256)), dim3(256), 0, st, A->rowptr, A->colind,
                       A->vals, n, slot_of.p, cm.p, n_pad, repeats.p);
    DN_LAUNCH_CHECK();
    int n_rep = 0;
    DN_HIP(hipMemcpy(&n_rep, repeats.p, sizeof(int), hipMemcpyDeviceToHost));
    DN_CHECK(n_rep == 0,
             "%d entries of the dense head's columns repeat a (row, column) pair: duplicate entries are "
             "not supported by the products",
             n_rep);
  }
  // the remaining entries: the row-major arrays without the head's columns, written straight
  // into the tail's own arrays (positions from a scan over the entries)
  dnpeff_csr* T = new dnpeff_csr();
  T->n_rows = n; T->n_cols = m; T->full_dense_size = A->full_dense_size;
  int status = 0;
  {
    dbuf<int64_t> newpos;
    status = newpos.alloc(A->nnz + 1) || scan_kept_entries(A->colind, table, A->nnz, newpos);
    if (!status && hipMemcpy(&T->nnz, newpos + A->nnz, sizeof(int64_t), hipMemcpyDeviceToHost) != hipSuccess) {
      set_error("dense head: reading the size of the sparse part failed");
      status = 1;
    }
    if (!status)
      status = dmalloc(&T->rowptr, n + 1) || dmalloc(&T->colind, T->nnz) || dmalloc(&T->vals, T->nnz);
    if (!status) {
      hipLaunchKernelGGL(k_compact_entries, dim3(grid_for(A->nnz)), dim3(256), 0, st, A->colind,
                         A->vals, A->nnz, table.p, newpos.p, T->colind, T->vals);
      hipLaunchKernelGGL(k_map_rowptr, dim3(grid_for(n + 1)), dim3(256), 0, st, A->rowptr, n, newpos.p,
                         T->rowptr);
      if (hipGetLastError() != hipSuccess || hipStreamSynchronize(st) != hipSuccess) {
        set_error("dense head: building the sparse part failed");
        status = 1;
      }
    }
  }
  if (status) {
    dnpeff_csr_destroy(T);
    return status;
  }
  dense_head& h = A->head;
  h.n_d = n_d; h.n_d_pad = n_d_pad; h.n_pad = n_pad;
  h.cols = cols.release(); h.cm = cm.release();
  A->tail = T;
  if (n_dense) *n_dense = n_d;
  return 0;
}

}  // namespace dn

DN_API int dnpeff_csr_split_dense_head(dnpeff_csr* A, double min_fill, int64_t* n_dense) {
  clear_error();
  DN_CHECK(A && has_row_major(A), "matrix is NULL or its row-major arrays were released");
  DN_CHECK(min_fill <= 1.0, "min_fill %g above 1", min_fill);
  if (n_dense) *n_dense = 0;
  if (min_fill <= 0.0) {
    drop_derived(A);
    return 0;
  }
  head_choice c;
  DN_TRY(choose_dense_head(A, min_fill, NO_BUDGET, 2, 0, &c));
  return split_dense_head_at(A, c.thr, n_dense);
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

DN_API int dnpeff_csr_products_info(const dnpeff_csr* A, int64_t* out6) {
  DN_CHECK(A != nullptr && out6 != nullptr, "NULL argument");
  const dnpeff_csr* S = sparse_part(A);
  out6[0] = S->n_panels;
  out6[1] = S->n_plain;
  out6[2] = S->n_swept;
  out6[3] = S->tail_floor;
  out6[4] = S->nl.pairs ? S->nl.n_entries : 0;
  out6[5] = S->nl.pairs ? S->nl.n_batches : 0;
  return 0;
}

DN_API int dnpeff_csr_build_transpose(dnpeff_csr* A) {
  clear_error();
  DN_CHECK(A != nullptr, "matrix is NULL");
  if (A->colptr) return 0;
  DN_CHECK(has_row_major(A), "row-major copy of the matrix was released");
  hipStream_t st = stream();
  const int64_t m = A->n_cols;
  dbuf<int> count;
  dbuf<int64_t> colptr;
  dbuf<int32_t> rowind, pos, long_cols;
  dbuf<float> tvals;
  DN_TRY(count.alloc(m + 1));  // (the last element counts columns with a repeated row)
  DN_HIP(hipMemsetAsync(count, 0, sizeof(int) * (size_t)(m + 1), st));
  hipLaunchKernelGGL(k_col_hist, dim3(grid_for(A->nnz, 65536)), dim3(256), 0, st, A->colind, A->nnz,
                     count.p);
  DN_LAUNCH_CHECK();
  DN_TRY(colptr.alloc(m + 1));
  DN_TRY(scan_counts_i64(count, m, colptr));
  DN_TRY(rowind.alloc(A->nnz));
  DN_TRY(tvals.alloc(A->nnz));
  DN_HIP(hipMemsetAsync(count, 0, sizeof(int) * (size_t)(m + 1), st));
  std::vector<int64_t> rowptr((size_t)A->n_rows + 1);
  DN_HIP(hipMemcpy(rowptr.data(), A->rowptr, sizeof(int64_t) * (A->n_rows + 1),
                   hipMemcpyDeviceToHost));
  for (int64_t i = 0; i < A->n_rows; i++) {
    int64_t len = rowptr[i + 1] - rowptr[i];
    if (len <= 0) continue;
    hipLaunchKernelGGL(k_transpose_row, dim3((unsigned)ceil_div(len, 256)), dim3(256), 0, st,
                       (int32_t)i, rowptr[i], rowptr[i + 1], A->colind, A->vals, colptr.p, count.p,
                       rowind.p, tvals.p);
  }
  DN_LAUNCH_CHECK();
  // A row that holds a column twice puts two entries of that row next to each other in the
  // column's list, in an order that the hardware decides: such a matrix has no deterministic
  // transposed copy (nor is it a valid PEF matrix: top-k indices are distinct) and is refused.
  hipLaunchKernelGGL(k_check_repeats, dim3(grid_for(m, 65536)), dim3(256), 0, st, colptr.p, rowind.p, m,
                     count.p + m);
  DN_LAUNCH_CHECK();
  int repeats = 0;
  DN_HIP(hipMemcpy(&repeats, count.p + m, sizeof(int), hipMemcpyDeviceToHost));
  DN_CHECK(repeats == 0,
           "%d column(s) hold the same row more than once: duplicate (row, column) entries are not "
           "supported by the products",
           repeats);
  count.reset();
  // list of long columns for A^T W
  DN_TRY(pos.alloc(m + 1));
  DN_TRY(scan_long_cols(colptr, SPMM_T_LONG, m, pos));
  int32_t n_long = 0;
  DN_HIP(hipMemcpy(&n_long, pos + m, sizeof(int32_t), hipMemcpyDeviceToHost));
  DN_TRY(long_cols.alloc((int64_t)n_long));
  if (n_long) {
    hipLaunchKernelGGL(k_collect_long, dim3(grid_for(m)), dim3(256), 0, st, colptr.p, SPMM_T_LONG, m,
                       pos.p, long_cols.p);
    DN_LAUNCH_CHECK();
  }
  DN_HIP(hipStreamSynchronize(st));
  A->colptr = colptr.release();
  A->rowind = rowind.release();
  A->tvals = tvals.release();
  A->long_cols = long_cols.release();
  A->n_long = n_long;
  A->h_lists_valid = false;
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

// out[k] = X[rows[k]] for k < count (rows of r floats)
__global__ void __launch_bounds__(256)
    k_gather_rows(const float* __restrict__ X, const int32_t* __restrict__ rows, int64_t count, int r,
                  float* __restrict__ out) {
  const int64_t total = count * r, stride = (int64_t)gridDim.x * 256;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += stride)
    out[e] = X[(int64_t)rows[e / r] * r + e % r];
}

DN_API int dnpeff_op_gather_rows(int64_t count, int r, const float* X, const int32_t* rows_dev,
                                 float* out) {
  clear_error();
  DN_CHECK(count >= 0 && r >= 1, "bad arguments");
  if (count == 0) return 0;
  DN_CHECK(X && rows_dev && out, "NULL argument");
  hipLaunchKernelGGL(k_gather_rows, dim3(grid_for(count * r)), dim3(256), 0, stream(), X, rows_dev,
                     count, r, out);
  DN_LAUNCH_CHECK();
  return 0;
}

// out[k] = cm[k * n_pad + row]: one row of the dense head's block
__global__ void __launch_bounds__(256)
    k_head_row(const float* __restrict__ cm, int64_t n_pad, int64_t row, int64_t n_d,
               float* __restrict__ out) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t k = (int64_t)blockIdx.x * 256 + threadIdx.x; k < n_d; k += stride)
    out[k] = cm[k * n_pad + row];
}

// Entries of one row / one column of the matrix as the products hold it: the dense head's block
// plus the sparse part (its regrouped or plain row-major copy, its transposed copy).
DN_API int dnpeff_csr_get_row(dnpeff_csr* A, int64_t row, int64_t cap, int64_t* count, int32_t* cols,
                              float* vals) {
  clear_error();
  DN_CHECK(A && count, "NULL argument");
  DN_CHECK(row >= 0 && row < A->n_rows, "row %lld outside [0, %lld)", (long long)row,
           (long long)A->n_rows);
  DN_HIP(hipStreamSynchronize(stream()));
  const dnpeff_csr* S = sparse_part(A);
  DN_CHECK(S->rowptr != nullptr, "matrix has no row offsets");
  int64_t e[2];
  DN_HIP(hipMemcpy(e, S->rowptr + row, sizeof(e), hipMemcpyDeviceToHost));
  const int32_t* src_c = S->colind ? S->colind : S->pcol;
  const float* src_v = S->vals ? S->vals : S->pval;
  std::vector<int32_t> list_cols;
  std::vector<float> list_vals;
  const int64_t row_entries = e[1] - e[0];
  if (!S->colind && S->pcol && S->tail_floor > 0 && S->nl.pairs) {
    // the panels hold the row's entries below tail_floor, the slot lists the others
    DN_TRY(nlists_get_row(S, row, list_cols, list_vals));
    DN_HIP(hipMemcpy(e, S->prow + row, sizeof(e), hipMemcpyDeviceToHost));
    DN_CHECK((int64_t)list_cols.size() + (e[1] - e[0]) == row_entries,
             "panels and slot lists hold %lld entries of row %lld, not %lld",
             (long long)((int64_t)list_cols.size() + (e[1] - e[0])), (long long)row, (long long)row_entries);
    std::vector<int32_t> pc((size_t)(e[1] - e[0]));
    std::vector<float> pv((size_t)(e[1] - e[0]));
    if (e[1] > e[0]) {
      DN_HIP(hipMemcpy(pc.data(), S->pcol + e[0], sizeof(int32_t) * pc.size(), hipMemcpyDeviceToHost));
      DN_HIP(hipMemcpy(pv.data(), S->pval + e[0], sizeof(float) * pv.size(), hipMemcpyDeviceToHost));
    }
    list_cols.insert(list_cols.begin(), pc.begin(), pc.end());
    list_vals.insert(list_vals.begin(), pv.begin(), pv.end());
  } else if (!(src_c && src_v) && S->nl.pairs) {  // the sparse part is held as slot lists
    DN_TRY(nlists_get_row(S, row, list_cols, list_vals));
    DN_CHECK((int64_t)list_cols.size() == row_entries, "slot lists hold %lld entries of row %lld, not %lld",
             (long long)list_cols.size(), (long long)row, (long long)row_entries);
  } else {
    DN_CHECK(e[1] == e[0] || (src_c && src_v), "matrix holds no row-major copy of its sparse part");
  }
  int64_t got = row_entries;
  std::vector<float> head_row;
  std::vector<int32_t> head_cols;
  if (A->head.n_d) {
    head_row.resize((size_t)A->head.n_d);
    head_cols.resize((size_t)A->head.n_d);
    dbuf<float> tmp;
    DN_TRY(tmp.alloc(A->head.n_d));
    hipLaunchKernelGGL(k_head_row, dim3(grid_for(A->head.n_d, 4096)), dim3(256), 0, stream(), A->head.cm,
                       A->head.n_pad, row, A->head.n_d, tmp.p);
    DN_LAUNCH_CHECK();
    DN_HIP(hipStreamSynchronize(stream()));
    DN_HIP(hipMemcpy(head_row.data(), tmp.p, sizeof(float) * A->head.n_d, hipMemcpyDeviceToHost));
    DN_HIP(hipMemcpy(head_cols.data(), A->head.cols, sizeof(int32_t) * A->head.n_d,
                     hipMemcpyDeviceToHost));
    for (float v : head_row) got += v != 0.0f;
  }
  *count = got;
  if (!cols || !vals) return 0;
  DN_CHECK(cap >= got, "row %lld holds %lld entries, the buffers %lld", (long long)row, (long long)got,
           (long long)cap);
  int64_t w = 0;
  for (size_t k = 0; k < head_row.size(); k++)
    if (head_row[k] != 0.0f) {
      cols[w] = head_cols[k];
      vals[w++] = head_row[k];
    }
  if (!list_cols.empty()) {
    memcpy(cols + w, list_cols.data(), sizeof(int32_t) * list_cols.size());
    memcpy(vals + w, list_vals.data(), sizeof(float) * list_vals.size());
  } else if (e[1] > e[0]) {
    DN_HIP(hipMemcpy(cols + w, src_c + e[0], sizeof(int32_t) * (e[1] - e[0]), hipMemcpyDeviceToHost));
    DN_HIP(hipMemcpy(vals + w, src_v + e[0], sizeof(float) * (e[1] - e[0]), hipMemcpyDeviceToHost));
  }
  return 0;
}

DN_API int dnpeff_csr_get_column(dnpeff_csr* A, int64_t col, int64_t cap, int64_t* count,
                                 int32_t* rows, float* vals) {
  clear_error();
  DN_CHECK(A && count, "NULL argument");
  DN_CHECK(col >= 0 && col < A->n_cols, "column %lld outside [0, %lld)", (long long)col,
           (long long)A->n_cols);
  dnpeff_csr* S = sparse_part(A);
  DN_TRY(dnpeff_csr_build_transpose(S));
  DN_TRY(csr_tile_lists(A));
  DN_HIP(hipStreamSynchronize(stream()));
  const std::vector<int32_t>& hc = A->h_head_cols;
  const auto it = std::lower_bound(hc.begin(), hc.end(), (int32_t)col);
  if (it != hc.end() && *it == (int32_t)col) {  // a column of the dense head
    const int64_t k = it - hc.begin();
    std::vector<float> c((size_t)A->n_rows);
    DN_HIP(hipMemcpy(c.data(), A->head.cm + k * A->head.n_pad, sizeof(float) * A->n_rows,
                     hipMemcpyDeviceToHost));
    int64_t got = 0;
    for (float v : c) got += v != 0.0f;
    *count = got;
    if (!rows || !vals) return 0;
    DN_CHECK(cap >= got, "column %lld holds %lld entries, the buffers %lld", (long long)col,
             (long long)got, (long long)cap);
    int64_t w = 0;
    for (int64_t i = 0; i < A->n_rows; i++)
      if (c[(size_t)i] != 0.0f) {
        rows[w] = (int32_t)i;
        vals[w++] = c[(size_t)i];
      }
    return 0;
  }
  int64_t p[2];
  DN_HIP(hipMemcpy(p, S->colptr + col, sizeof(p), hipMemcpyDeviceToHost));
  *count = p[1] - p[0];
  if (!rows || !vals) return 0;
  DN_CHECK(cap >= p[1] - p[0], "column %lld holds %lld entries, the buffers %lld", (long long)col,
           (long long)(p[1] - p[0]), (long long)cap);
  if (p[1] > p[0]) {
    DN_HIP(hipMemcpy(rows, S->rowind + p[0], sizeof(int32_t) * (p[1] - p[0]), hipMemcpyDeviceToHost));
    DN_HIP(hipMemcpy(vals, S->tvals + p[0], sizeof(float) * (p[1] - p[0]), hipMemcpyDeviceToHost));
  }
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
    dfree(A->slots); A->slots = nullptr;
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
