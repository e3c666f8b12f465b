// Synthetic PEF generator (benchmark and test inputs): per row, distinct
// column ids by successive Zipf draws with rejection of duplicates (draw order
// kept), log-normal fp32 values, per-row L2 norms.  The device generator and
// the single-threaded host generator share synth_rng.h and give the same bits.
// Compiled with -ffp-contract=off.
#include "dnpeff_internal.hpp"
#include "synth_rng.h"

#include <vector>

namespace dn {

constexpr uint64_t SLOT_EMPTY = 0xffffffffffffffffULL;

// Draw budget of one row: generous for Zipf exponents up to ~1.3 at the sizes
// used here, and a hard stop so that every workgroup terminates.
__host__ __device__ inline uint64_t draw_budget(int64_t k) {
  uint64_t b = 256ull * (uint64_t)k + (1ull << 20);
  return b < 0xffffff00ull ? b : 0xffffff00ull;
}

__host__ __device__ inline uint64_t slot_hash(uint64_t id) { return dn_mix64(id + 0x632be59bd9b4e019ULL); }

__global__ void __launch_bounds__(256)
    k_row_lengths(int64_t n_rows, int64_t k_fixed, int64_t k_min, int64_t k_max, uint64_t seed,
                  int* __restrict__ len) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n_rows) len[i] = (int)dn_row_length(seed, (uint64_t)i, k_fixed, k_min, k_max);
}

// One workgroup draws one row at a time.  Batches of 256 SYNTH_D draws (thread tid holds the
// draws batch base + SYNTH_D tid + q, q < SYNTH_D) are inserted into a per-workgroup
// open-addressing table keyed by id holding the smallest draw index seen; a draw is accepted iff
// it is the first occurrence of its id, and accepted draws are written in draw order.  This
// reproduces sequential sampling with rejection exactly.  Most draws of a skewed distribution
// repeat an id that an earlier batch has put into the table: such a draw sees the id with a
// smaller draw index on a plain read and needs no atomic operation.
constexpr int SYNTH_D = 8;

__global__ void __launch_bounds__(256)
    k_synth_cols(dn_zipf z, uint64_t seed, int64_t n_rows, const int64_t* __restrict__ rowptr,
                 int32_t* __restrict__ colind, unsigned long long* table_all, uint64_t cap,
                 int* __restrict__ failed) {
  __shared__ int sh[256];
  unsigned long long* table = table_all + (uint64_t)blockIdx.x * cap;
  const int tid = threadIdx.x;
  const uint64_t mask = cap - 1;

  for (int64_t row = blockIdx.x; row < n_rows; row += gridDim.x) {
    const int64_t base = rowptr[row];
    const int64_t k = rowptr[row + 1] - base;
    for (uint64_t i = tid; i < cap; i += 256) table[i] = SLOT_EMPTY;
    __threadfence();
    __syncthreads();

    int64_t count = 0;
    const uint64_t budget = draw_budget(k);
    for (uint64_t t_base = 0; count < k && t_base < budget; t_base += 256 * SYNTH_D) {
      uint64_t ids[SYNTH_D], slots[SYNTH_D];
      bool maybe[SYNTH_D];  // not yet known to repeat an earlier draw
#pragma unroll
      for (int q = 0; q < SYNTH_D; q++) {
        const uint64_t t = t_base + (uint64_t)tid * SYNTH_D + q;
        const uint64_t id = (uint64_t)dn_zipf_draw(&z, seed, (uint64_t)row, t);
        const unsigned long long packed = (id << 32) | t;
        uint64_t slot = slot_hash(id) & mask;
        bool open = true;
        for (;;) {
          unsigned long long cur = __hip_atomic_load(&table[slot], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if (cur == SLOT_EMPTY) {
            cur = atomicCAS(&table[slot], SLOT_EMPTY, packed);
            if (cur == SLOT_EMPTY) break;
          }
          if ((cur >> 32) == id) {
            if ((cur & 0xffffffffULL) < t) open = false;  // an earlier draw holds the id
            else atomicMin(&table[slot], packed);
            break;
          }
          slot = (slot + 1) & mask;
        }
        ids[q] = id;
        slots[q] = slot;
        maybe[q] = open;
      }
      __threadfence();
      __syncthreads();
      // first occurrence of its id?  (the slot of an id never moves)
      int wins = 0;
      bool win[SYNTH_D];
#pragma unroll
      for (int q = 0; q < SYNTH_D; q++) {
        win[q] = false;
        if (maybe[q]) {
          const uint64_t t = t_base + (uint64_t)tid * SYNTH_D + q;
          const unsigned long long cur =
              __hip_atomic_load(&table[slots[q]], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          win[q] = (cur & 0xffffffffULL) == t;
        }
        wins += win[q] ? 1 : 0;
      }
      // exclusive scan of the per-thread counts over the workgroup, in draw order
      sh[tid] = wins;
      __syncthreads();
      for (int off = 1; off < 256; off <<= 1) {
        int add = tid >= off ? sh[tid - off] : 0;
        __syncthreads();
        sh[tid] += add;
        __syncthreads();
      }
      const int incl = sh[tid];
      const int total = sh[255];
      __syncthreads();
      int64_t pos = count + incl - wins;
#pragma unroll
      for (int q = 0; q < SYNTH_D; q++)
        if (win[q]) {
          if (pos < k) colind[base + pos] = (int32_t)ids[q];
          pos++;
        }
      count += total;
    }
    if (count < k && tid == 0) atomicAdd(failed, 1);
    __syncthreads();
  }
}

__global__ void __launch_bounds__(256)
    k_synth_vals(int64_t n_rows, const int64_t* __restrict__ rowptr, uint64_t seed, double mu,
                 double sigma, float* __restrict__ vals) {
  for (int64_t row = blockIdx.x; row < n_rows; row += gridDim.x) {
    const int64_t base = rowptr[row];
    const int64_t len = rowptr[row + 1] - base;
    for (int64_t p = threadIdx.x; p < len; p += 256)
      vals[base + p] = dn_lognormal_at(seed, (uint64_t)row, (uint64_t)p, mu, sigma);
  }
}

// fp32 L2 norm of each row: squares summed in fp64 in entry order (the same
// order as the host generator), then rounded.
__global__ void __launch_bounds__(64)
    k_row_norms(int64_t n_rows, const int64_t* __restrict__ rowptr, const float* __restrict__ vals,
                float* __restrict__ norms) {
  int64_t row = (int64_t)blockIdx.x * 64 + threadIdx.x;
  if (row >= n_rows) return;
  double s = 0.0;
  for (int64_t e = rowptr[row]; e < rowptr[row + 1]; e++) {
    double v = (double)vals[e];
    s = fma(v, v, s);
  }
  norms[row] = (float)sqrt(s);
}

static int validate_synth(int64_t n_rows, int64_t n_cols, int64_t k_fixed, int64_t k_min,
                          int64_t k_max, double zipf_s) {
  DN_CHECK(n_rows >= 0 && n_cols >= 1, "bad shape");
  DN_CHECK(n_rows < (int64_t)INT32_MAX && n_cols < (int64_t)INT32_MAX, "shape must fit 32-bit ids");
  DN_CHECK(zipf_s > 1.0 && zipf_s < 8.0, "zipf exponent must be in (1, 8)");
  if (k_min > 0) {
    DN_CHECK(k_min <= k_max, "k_min > k_max");
    DN_CHECK(k_max * 2 <= n_cols, "k_max must be at most n_cols / 2");
  } else {
    DN_CHECK(k_fixed >= 0 && k_fixed * 2 <= n_cols, "k must be at most n_cols / 2");
  }
  return 0;
}

}  // namespace dn

using namespace dn;

DN_API int dnpeff_synth_pef(int64_t n_rows, int64_t n_cols, int64_t k_fixed, int64_t k_min,
                            int64_t k_max, double zipf_s, double mu, double sigma, uint64_t seed,
                            float* norms_out_host, dnpeff_csr** out) {
  clear_error();
  DN_CHECK(out != nullptr, "out is NULL");
  *out = nullptr;
  DN_TRY(validate_synth(n_rows, n_cols, k_fixed, k_min, k_max, zipf_s));
  hipStream_t st = stream();
  dnpeff_csr* A = new dnpeff_csr();
  A->n_rows = n_rows; A->n_cols = n_cols; A->full_dense_size = n_cols;
  int* len = nullptr;
  int* failed = nullptr;
  unsigned long long* tables = nullptr;
  float* norms = nullptr;
  int status = 0;
  auto fail = [&](int s) {
    dfree(len); dfree(failed); dfree(tables); dfree(norms);
    dnpeff_csr_destroy(A);
    return s;
  };
  if (dmalloc(&len, n_rows) || dmalloc(&A->rowptr, n_rows + 1) || dmalloc(&failed, 1)) return fail(1);
  if (n_rows > 0) {
    hipLaunchKernelGGL(k_row_lengths, dim3((unsigned)ceil_div(n_rows, 256)), dim3(256), 0, st,
                       n_rows, k_fixed, k_min, k_max, seed, len);
  }
  if ((status = scan_counts_i64(len, n_rows, A->rowptr))) return fail(status);
  if (hipMemcpy(&A->nnz, A->rowptr + n_rows, sizeof(int64_t), hipMemcpyDeviceToHost) != hipSuccess)
    return fail(1);
  if (dmalloc(&A->colind, A->nnz) || dmalloc(&A->vals, A->nnz)) return fail(1);

  const int64_t kmax_eff = k_min > 0 ? k_max : k_fixed;
  uint64_t cap = 1024;
  while (cap < 2 * (uint64_t)(kmax_eff + 256)) cap <<= 1;
  // the draws are long chains of fp64 arithmetic: as many workgroups as the tables leave room for
  // (one table each, at most 24 GB together), up to 8 per CU
  int64_t wgs = 8 * (int64_t)n_cus();
  while (wgs > 2 * (int64_t)n_cus() && (double)wgs * (double)cap * 8.0 > 24e9) wgs /= 2;
  if (wgs > n_rows) wgs = n_rows;
  if (wgs < 1) wgs = 1;
  if (dmalloc(&tables, (int64_t)(cap * (uint64_t)wgs))) return fail(1);
  (void)hipMemsetAsync(failed, 0, sizeof(int), st);

  dn_zipf z;
  dn_zipf_init(&z, zipf_s, n_cols);
  if (n_rows > 0) {
    hipLaunchKernelGGL(k_synth_cols, dim3((unsigned)wgs), dim3(256), 0, st, z, seed, n_rows,
                       A->rowptr, A->colind, tables, cap, failed);
    hipLaunchKernelGGL(k_synth_vals, dim3((unsigned)(n_rows < 65536 ? n_rows : 65536)), dim3(256),
                       0, st, n_rows, A->rowptr, seed, mu, sigma, A->vals);
  }
  if (hipGetLastError() != hipSuccess) { set_error("generator launch failed"); return fail(1); }
  int h_failed = 0;
  if (hipMemcpy(&h_failed, failed, sizeof(int), hipMemcpyDeviceToHost) != hipSuccess) {
    set_error("generator kernel failed");
    return fail(1);
  }
  if (h_failed) {
    set_error("%d rows exhausted their draw budget before reaching k distinct ids", h_failed);
    return fail(2);
  }
  if (norms_out_host && n_rows > 0) {
    if (dmalloc(&norms, n_rows)) return fail(1);
    hipLaunchKernelGGL(k_row_norms, dim3((unsigned)ceil_div(n_rows, 64)), dim3(64), 0, st, n_rows,
                       A->rowptr, A->vals, norms);
    if (hipMemcpy(norms_out_host, norms, sizeof(float) * n_rows, hipMemcpyDeviceToHost) !=
        hipSuccess) {
      set_error("norm kernel failed");
      return fail(1);
    }
  }
  (void)hipStreamSynchronize(st);
  dfree(len); dfree(failed); dfree(tables); dfree(norms);
  *out = A;
  return 0;
}

// rows [row0, row0 + n_rows) of the matrix that dnpeff_synth_pef makes for the same arguments
static int synth_host_rows(int64_t row0, int64_t n_rows, int64_t n_cols, int64_t k_fixed,
                           int64_t k_min, int64_t k_max, double zipf_s, double mu, double sigma,
                           uint64_t seed, int64_t* rowptr, int32_t* colind, float* vals, float* norms) {
  DN_CHECK(rowptr != nullptr, "rowptr is NULL");
  rowptr[0] = 0;
  int64_t kmax_eff = 0;
  for (int64_t i = 0; i < n_rows; i++) {
    int64_t k = dn_row_length(seed, (uint64_t)(row0 + i), k_fixed, k_min, k_max);
    rowptr[i + 1] = rowptr[i] + k;
    if (k > kmax_eff) kmax_eff = k;
  }
  if (!colind) return 0;  // sizing pass
  DN_CHECK(vals != nullptr, "vals is NULL");
  dn_zipf z;
  dn_zipf_init(&z, zipf_s, n_cols);
  uint64_t cap = 1024;
  while (cap < 2 * (uint64_t)(kmax_eff + 256)) cap <<= 1;
  std::vector<uint64_t> table(cap);
  const uint64_t mask = cap - 1;
  for (int64_t i = 0; i < n_rows; i++) {
    const uint64_t row = (uint64_t)(row0 + i);
    const int64_t base = rowptr[i], k = rowptr[i + 1] - base;
    std::fill(table.begin(), table.end(), SLOT_EMPTY);
    int64_t count = 0;
    const uint64_t budget = draw_budget(k);
    for (uint64_t t = 0; count < k && t < budget; t++) {
      const uint64_t id = (uint64_t)dn_zipf_draw(&z, seed, row, t);
      uint64_t slot = slot_hash(id) & mask;
      bool seen = false;
      while (table[slot] != SLOT_EMPTY) {
        if (table[slot] == id) { seen = true; break; }
        slot = (slot + 1) & mask;
      }
      if (seen) continue;
      table[slot] = id;
      colind[base + count++] = (int32_t)id;
    }
    DN_CHECK(count == k, "row %lld exhausted its draw budget", (long long)row);
    double s = 0.0;
    for (int64_t p = 0; p < k; p++) {
      float v = dn_lognormal_at(seed, row, (uint64_t)p, mu, sigma);
      vals[base + p] = v;
      s = fma((double)v, (double)v, s);
    }
    if (norms) norms[i] = (float)sqrt(s);
  }
  return 0;
}

DN_API int dnpeff_synth_pef_host(int64_t n_rows, int64_t n_cols, int64_t k_fixed, int64_t k_min,
                                 int64_t k_max, double zipf_s, double mu, double sigma,
                                 uint64_t seed, int64_t* rowptr, int32_t* colind, float* vals,
                                 float* norms) {
  clear_error();
  DN_TRY(validate_synth(n_rows, n_cols, k_fixed, k_min, k_max, zipf_s));
  return synth_host_rows(0, n_rows, n_cols, k_fixed, k_min, k_max, zipf_s, mu, sigma, seed, rowptr,
                         colind, vals, norms);
}

DN_API int dnpeff_synth_pef_host_rows(int64_t row0, int64_t n_rows, int64_t n_cols, int64_t k_fixed,
                                      int64_t k_min, int64_t k_max, double zipf_s, double mu,
                                      double sigma, uint64_t seed, int64_t* rowptr, int32_t* colind,
                                      float* vals, float* norms) {
  clear_error();
  DN_CHECK(row0 >= 0, "row0 is negative");
  DN_TRY(validate_synth(row0 + n_rows, n_cols, k_fixed, k_min, k_max, zipf_s));
  return synth_host_rows(row0, n_rows, n_cols, k_fixed, k_min, k_max, zipf_s, mu, sigma, seed, rowptr,
                         colind, vals, norms);
}
