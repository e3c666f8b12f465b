// Internal declarations shared by the translation units of libdnpeff_hip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>

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
int launch_xg_mu(int64_t rows, int r, const float* X, const float* G, const float* num, float eps,
                 float* out, float* D_out);
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
int launch_spmm_n(const dnpeff_csr* A, int r, const float* H_mr, float* N_nr, float* partials);
int launch_spmm_n_reduce(const dnpeff_csr* A, int r, const float* partials, float* N_nr);
int launch_spmm_t(const dnpeff_csr* A, int r, const float* W_nr, float* T_mr);
int launch_spsp(const dnpeff_csr* A, const dnpeff_csr* B, float* partials);

}  // namespace dn

struct dnpeff_csr {
  int64_t n_rows = 0, n_cols = 0, nnz = 0;
  int64_t full_dense_size = 0;
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
  // work decomposition of A H^T: chunk_base[i] = chunks of rows before i
  int64_t* chunk_base = nullptr;
  int64_t n_chunks = 0;
  // columns longer than SPMM_T_LONG
  int32_t* long_cols = nullptr;
  int64_t n_long = 0;
  // workspace for the per-chunk partial sums of A H^T ([n_chunks, r])
  float* partials = nullptr;
  int64_t partials_floats = 0;
};

namespace dn {
int csr_ensure_chunks(dnpeff_csr* A);
int csr_ensure_partials(dnpeff_csr* A, int r);
}  // namespace dn
