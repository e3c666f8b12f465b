// Sparse kernels: A H^T (row-major CSR, gather rows of H), A^T W (transposed
// CSR, gather rows of W, no atomics) and sparse x sparse -> dense for the
// fixed-H learner.  A wavefront owns one output row; lane l holds components
// l, l+64, l+128, ... so every gathered row is read as contiguous 256-byte
// segments.  (col, val) pairs are streamed 64 at a time, one per lane, and
// broadcast from registers.  All summation orders are fixed by the matrix
// structure, so results are reproducible run to run.
#include "dnpeff_internal.hpp"

namespace dn {

__device__ inline int bcast_i(int v, int src_lane) { return __builtin_amdgcn_readlane(v, src_lane); }
__device__ inline float bcast_f(float v, int src_lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src_lane));
}

// acc[t] += sum_{p in [p0, p1)} val[p] * X[idx[p] * r + lane + 64 t], p ascending.
template <int VPL>
__device__ inline void gather_rows(const int32_t* __restrict__ idx, const float* __restrict__ val,
                                   int64_t p0, int64_t p1, const float* __restrict__ X, int r,
                                   int lane, const bool (&ok)[VPL], float (&acc)[VPL]) {
  for (int64_t p = p0; p < p1; p += 64) {
    const int cnt = (p1 - p) < 64 ? (int)(p1 - p) : 64;
    int my_i = 0;
    float my_v = 0.0f;
    if (lane < cnt) {
      my_i = idx[p + lane];
      my_v = val[p + lane];
    }
    int u = 0;
    for (; u + 4 <= cnt; u += 4) {
      const float* x0 = X + (int64_t)bcast_i(my_i, u) * r + lane;
      const float* x1 = X + (int64_t)bcast_i(my_i, u + 1) * r + lane;
      const float* x2 = X + (int64_t)bcast_i(my_i, u + 2) * r + lane;
      const float* x3 = X + (int64_t)bcast_i(my_i, u + 3) * r + lane;
      const float a0 = bcast_f(my_v, u), a1 = bcast_f(my_v, u + 1);
      const float a2 = bcast_f(my_v, u + 2), a3 = bcast_f(my_v, u + 3);
      float h0[VPL], h1[VPL], h2[VPL], h3[VPL];
#pragma unroll
      for (int t = 0; t < VPL; t++) {
        h0[t] = ok[t] ? x0[64 * t] : 0.0f;
        h1[t] = ok[t] ? x1[64 * t] : 0.0f;
        h2[t] = ok[t] ? x2[64 * t] : 0.0f;
        h3[t] = ok[t] ? x3[64 * t] : 0.0f;
      }
#pragma unroll
      for (int t = 0; t < VPL; t++) {
        acc[t] = fmaf(a0, h0[t], acc[t]);
        acc[t] = fmaf(a1, h1[t], acc[t]);
        acc[t] = fmaf(a2, h2[t], acc[t]);
        acc[t] = fmaf(a3, h3[t], acc[t]);
      }
    }
    for (; u < cnt; u++) {
      const float* x0 = X + (int64_t)bcast_i(my_i, u) * r + lane;
      const float a0 = bcast_f(my_v, u);
#pragma unroll
      for (int t = 0; t < VPL; t++) {
        float h = ok[t] ? x0[64 * t] : 0.0f;
        acc[t] = fmaf(a0, h, acc[t]);
      }
    }
  }
}

// Row that owns work chunk `chunk`: chunk_base[row] <= chunk < chunk_base[row + 1].
__device__ inline int64_t chunk_to_row(const int64_t* __restrict__ chunk_base, int64_t n_rows,
                                       int64_t chunk) {
  int64_t lo = 0, hi = n_rows;
  while (lo < hi) {
    int64_t mid = (lo + hi + 1) >> 1;
    if (chunk_base[mid] <= chunk) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// ---------------------------------------------------------------------------
// partials[chunk, :] = sum over the chunk's entries of val * H[col, :]
// A workgroup owns SPMM_N_CHUNK consecutive entries of one row; its 4 waves
// take a quarter each and are combined in wave order.
// ---------------------------------------------------------------------------
template <int VPL>
__global__ void __launch_bounds__(256)
    k_spmm_n(const int64_t* __restrict__ rowptr, const int32_t* __restrict__ colind,
             const float* __restrict__ vals, const int64_t* __restrict__ chunk_base, int64_t n_rows,
             int r, const float* __restrict__ H, float* __restrict__ partials) {
  __shared__ float red[4][64 * VPL];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int64_t chunk = blockIdx.x;
  const int64_t row = chunk_to_row(chunk_base, n_rows, chunk);
  const int64_t e0 = rowptr[row] + (chunk - chunk_base[row]) * SPMM_N_CHUNK;
  int64_t e1 = e0 + SPMM_N_CHUNK;
  if (e1 > rowptr[row + 1]) e1 = rowptr[row + 1];
  int64_t w0 = e0 + wave * (SPMM_N_CHUNK / 4);
  int64_t w1 = w0 + SPMM_N_CHUNK / 4;
  if (w0 > e1) w0 = e1;
  if (w1 > e1) w1 = e1;

  bool ok[VPL];
  float acc[VPL];
#pragma unroll
  for (int t = 0; t < VPL; t++) {
    ok[t] = lane + 64 * t < r;
    acc[t] = 0.0f;
  }
  gather_rows<VPL>(colind, vals, w0, w1, H, r, lane, ok, acc);
#pragma unroll
  for (int t = 0; t < VPL; t++) red[wave][lane + 64 * t] = acc[t];
  __syncthreads();
  for (int c = threadIdx.x; c < r; c += 256) {
    float s = red[0][c];
    s += red[1][c];
    s += red[2][c];
    s += red[3][c];
    partials[chunk * r + c] = s;
  }
}

// N[row, :] = sum of the row's chunk partials, in chunk order.
__global__ void __launch_bounds__(256)
    k_chunk_reduce(const int64_t* __restrict__ chunk_base, int r,
                   const float* __restrict__ partials, float* __restrict__ N) {
  const int64_t row = blockIdx.x;
  const int64_t c0 = chunk_base[row], c1 = chunk_base[row + 1];
  for (int c = threadIdx.x; c < r; c += 256) {
    float s = 0.0f;
    for (int64_t k = c0; k < c1; k++) s += partials[k * r + c];
    N[row * r + c] = s;
  }
}

// ---------------------------------------------------------------------------
// T[j, :] = sum over column j's entries (ascending row) of val * W[row, :]
// ---------------------------------------------------------------------------
template <int VPL>
__global__ void __launch_bounds__(256)
    k_spmm_t_short(const int64_t* __restrict__ colptr, const int32_t* __restrict__ rowind,
                   const float* __restrict__ tvals, int64_t m, int r, const float* __restrict__ W,
                   float* __restrict__ T) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int64_t j = (int64_t)blockIdx.x * 4 + wave;
  if (j >= m) return;
  const int64_t p0 = colptr[j], p1 = colptr[j + 1];
  if (p1 - p0 > SPMM_T_LONG) return;  // written by k_spmm_t_long
  bool ok[VPL];
  float acc[VPL];
#pragma unroll
  for (int t = 0; t < VPL; t++) {
    ok[t] = lane + 64 * t < r;
    acc[t] = 0.0f;
  }
  gather_rows<VPL>(rowind, tvals, p0, p1, W, r, lane, ok, acc);
#pragma unroll
  for (int t = 0; t < VPL; t++)
    if (ok[t]) T[j * r + lane + 64 * t] = acc[t];
}

template <int VPL>
__global__ void __launch_bounds__(256)
    k_spmm_t_long(const int32_t* __restrict__ long_cols, const int64_t* __restrict__ colptr,
                  const int32_t* __restrict__ rowind, const float* __restrict__ tvals, int r,
                  const float* __restrict__ W, float* __restrict__ T) {
  __shared__ float red[4][64 * VPL];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int64_t j = long_cols[blockIdx.x];
  const int64_t p0 = colptr[j], p1 = colptr[j + 1];
  const int64_t per = (((p1 - p0) + 3) / 4 + 63) / 64 * 64;  // quarter, rounded up to 64
  int64_t w0 = p0 + wave * per, w1 = w0 + per;
  if (w0 > p1) w0 = p1;
  if (w1 > p1) w1 = p1;
  bool ok[VPL];
  float acc[VPL];
#pragma unroll
  for (int t = 0; t < VPL; t++) {
    ok[t] = lane + 64 * t < r;
    acc[t] = 0.0f;
  }
  gather_rows<VPL>(rowind, tvals, w0, w1, W, r, lane, ok, acc);
#pragma unroll
  for (int t = 0; t < VPL; t++) red[wave][lane + 64 * t] = acc[t];
  __syncthreads();
  for (int c = threadIdx.x; c < r; c += 256) {
    float s = red[0][c];
    s += red[1][c];
    s += red[2][c];
    s += red[3][c];
    T[j * r + c] = s;
  }
}

// ---------------------------------------------------------------------------
// partials[chunk, :] = sum over the chunk's entries (j, a) of a * B[:, j] for a
// sparse B given by its transposed CSR (per column j: component ids and
// values).  Each wave keeps its r running sums in LDS.  The entries of an A-row
// chunk are applied strictly one after the other; within one entry the
// components of column j are distinct, so lane k applies the k-th of them.
// Every component therefore receives its additions in entry order.  Each lane
// prefetches the first SPSP_PREFETCH components of "its" entry so that the
// serial part touches registers and LDS only.
// ---------------------------------------------------------------------------
constexpr int SPSP_PREFETCH = 4;

template <int VPL>
__global__ void __launch_bounds__(256)
    k_spsp(const int64_t* __restrict__ rowptr, const int32_t* __restrict__ colind,
           const float* __restrict__ vals, const int64_t* __restrict__ chunk_base, int64_t n_rows,
           int r, const int64_t* __restrict__ b_colptr, const int32_t* __restrict__ b_comp,
           const float* __restrict__ b_vals, float* __restrict__ partials) {
  __shared__ float red[4][64 * VPL];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int64_t chunk = blockIdx.x;
  const int64_t row = chunk_to_row(chunk_base, n_rows, chunk);
  const int64_t e0 = rowptr[row] + (chunk - chunk_base[row]) * SPMM_N_CHUNK;
  int64_t e1 = e0 + SPMM_N_CHUNK;
  if (e1 > rowptr[row + 1]) e1 = rowptr[row + 1];
  int64_t w0 = e0 + wave * (SPMM_N_CHUNK / 4);
  int64_t w1 = w0 + SPMM_N_CHUNK / 4;
  if (w0 > e1) w0 = e1;
  if (w1 > e1) w1 = e1;

  float* acc = red[wave];
#pragma unroll
  for (int t = 0; t < VPL; t++) acc[lane + 64 * t] = 0.0f;

  for (int64_t e = w0; e < w1; e += 64) {
    const int cnt = (w1 - e) < 64 ? (int)(w1 - e) : 64;
    float my_a = 0.0f;
    int64_t q0 = 0;
    int len = 0;
    int pc[SPSP_PREFETCH];
    float pv[SPSP_PREFETCH];
    if (lane < cnt) {
      const int32_t j = colind[e + lane];
      my_a = vals[e + lane];
      q0 = b_colptr[j];
      len = (int)(b_colptr[j + 1] - q0);
    }
#pragma unroll
    for (int k = 0; k < SPSP_PREFETCH; k++) {
      pc[k] = 0;
      pv[k] = 0.0f;
      if (k < len) {
        pc[k] = b_comp[q0 + k];
        pv[k] = b_vals[q0 + k];
      }
    }
    const int q0_lo = (int)(uint32_t)(q0 & 0xffffffffLL), q0_hi = (int)(q0 >> 32);
    for (int u = 0; u < cnt; u++) {
      const int len_u = bcast_i(len, u);
      if (len_u == 0) continue;
      const float a_u = bcast_f(my_a, u);
      int c = bcast_i(pc[0], u);
      float h = bcast_f(pv[0], u);
#pragma unroll
      for (int k = 1; k < SPSP_PREFETCH; k++) {
        const int ck = bcast_i(pc[k], u);
        const float hk = bcast_f(pv[k], u);
        if (lane == k) {
          c = ck;
          h = hk;
        }
      }
      const int first = len_u < SPSP_PREFETCH ? len_u : SPSP_PREFETCH;
      if (lane < first) acc[c] = fmaf(a_u, h, acc[c]);
      if (len_u > SPSP_PREFETCH) {
        const int64_t q =
            ((int64_t)bcast_i(q0_hi, u) << 32) | (int64_t)(uint32_t)bcast_i(q0_lo, u);
        for (int k0 = SPSP_PREFETCH; k0 < len_u; k0 += 64) {
          if (k0 + lane < len_u) {
            const int cc = b_comp[q + k0 + lane];
            const float hh = b_vals[q + k0 + lane];
            acc[cc] = fmaf(a_u, hh, acc[cc]);
          }
        }
      }
    }
  }
  __syncthreads();
  for (int c = threadIdx.x; c < r; c += 256) {
    float s = red[0][c];
    s += red[1][c];
    s += red[2][c];
    s += red[3][c];
    partials[chunk * r + c] = s;
  }
}

// ---------------------------------------------------------------------------
// Host launchers
// ---------------------------------------------------------------------------
static int vpl_for(int r) {
  int v = (r + 63) / 64;
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

#define DN_DISPATCH_VPL(vpl, CALL)                        \
  switch (vpl) {                                          \
    case 1: { constexpr int V = 1; CALL; } break;         \
    case 2: { constexpr int V = 2; CALL; } break;         \
    case 4: { constexpr int V = 4; CALL; } break;         \
    case 8: { constexpr int V = 8; CALL; } break;         \
    case 16: { constexpr int V = 16; CALL; } break;       \
    default: set_error("rank too large for the sparse kernels (max 1024)"); return 2; \
  }

int launch_spmm_n(const dnpeff_csr* A, int r, const float* H_mr, float* /*N_nr*/, float* partials) {
  DN_CHECK(r >= 1 && r <= 1024, "rank %d outside [1, 1024]", r);
  DN_CHECK(A->rowptr && A->chunk_base, "matrix has no row-major copy / work list");
  if (A->n_chunks == 0) return 0;
  DN_CHECK(A->n_chunks < (int64_t)INT32_MAX, "too many work chunks");
  dim3 grid((unsigned)A->n_chunks), block(256);
  DN_DISPATCH_VPL(vpl_for(r), hipLaunchKernelGGL((k_spmm_n<V>), grid, block, 0, stream(), A->rowptr,
                                                 A->colind, A->vals, A->chunk_base, A->n_rows, r,
                                                 H_mr, partials));
  DN_LAUNCH_CHECK();
  return 0;
}

int launch_spmm_n_reduce(const dnpeff_csr* A, int r, const float* partials, float* N_nr) {
  if (A->n_rows == 0) return 0;
  hipLaunchKernelGGL(k_chunk_reduce, dim3((unsigned)A->n_rows), dim3(256), 0, stream(),
                     A->chunk_base, r, partials, N_nr);
  DN_LAUNCH_CHECK();
  return 0;
}

int launch_spmm_t(const dnpeff_csr* A, int r, const float* W_nr, float* T_mr) {
  DN_CHECK(r >= 1 && r <= 1024, "rank %d outside [1, 1024]", r);
  DN_CHECK(A->colptr != nullptr, "matrix has no transposed copy");
  if (A->n_cols == 0) return 0;
  dim3 grid((unsigned)ceil_div(A->n_cols, 4)), block(256);
  DN_DISPATCH_VPL(vpl_for(r), hipLaunchKernelGGL((k_spmm_t_short<V>), grid, block, 0, stream(),
                                                 A->colptr, A->rowind, A->tvals, A->n_cols, r,
                                                 W_nr, T_mr));
  if (A->n_long > 0) {
    dim3 grid_l((unsigned)A->n_long);
    DN_DISPATCH_VPL(vpl_for(r), hipLaunchKernelGGL((k_spmm_t_long<V>), grid_l, block, 0, stream(),
                                                   A->long_cols, A->colptr, A->rowind, A->tvals, r,
                                                   W_nr, T_mr));
  }
  DN_LAUNCH_CHECK();
  return 0;
}

int launch_spsp(const dnpeff_csr* A, const dnpeff_csr* B, float* partials) {
  const int r = (int)B->n_rows;
  DN_CHECK(r >= 1 && r <= 1024, "rank %d outside [1, 1024]", r);
  DN_CHECK(A->rowptr && A->chunk_base, "matrix has no row-major copy / work list");
  DN_CHECK(B->colptr != nullptr, "sparse factor has no transposed copy");
  DN_CHECK(A->n_cols == B->n_cols, "column counts differ (%lld vs %lld)", (long long)A->n_cols,
           (long long)B->n_cols);
  if (A->n_chunks == 0) return 0;
  dim3 grid((unsigned)A->n_chunks), block(256);
  DN_DISPATCH_VPL(vpl_for(r), hipLaunchKernelGGL((k_spsp<V>), grid, block, 0, stream(), A->rowptr,
                                                 A->colind, A->vals, A->chunk_base, A->n_rows, r,
                                                 B->colptr, B->rowind, B->tvals, partials));
  DN_LAUNCH_CHECK();
  return 0;
}

}  // namespace dn

using namespace dn;

DN_API int dnpeff_op_spmm_n(dnpeff_csr* A, int r, const float* H_mr, float* N_nr) {
  clear_error();
  DN_CHECK(A && H_mr && N_nr, "NULL argument");
  DN_TRY(csr_ensure_partials(A, r));
  DN_TRY(launch_spmm_n(A, r, H_mr, N_nr, A->partials));
  return launch_spmm_n_reduce(A, r, A->partials, N_nr);
}

DN_API int dnpeff_op_spmm_t(dnpeff_csr* A, int r, const float* W_nr, float* T_mr) {
  clear_error();
  DN_CHECK(A && W_nr && T_mr, "NULL argument");
  DN_TRY(dnpeff_csr_build_transpose(A));
  return launch_spmm_t(A, r, W_nr, T_mr);
}

DN_API int dnpeff_op_spsp_dense(dnpeff_csr* A, dnpeff_csr* B, float* out_nr) {
  clear_error();
  DN_CHECK(A && B && out_nr, "NULL argument");
  DN_TRY(dnpeff_csr_build_transpose(B));
  const int r = (int)B->n_rows;
  DN_TRY(csr_ensure_partials(A, r));
  DN_TRY(launch_spsp(A, B, A->partials));
  return launch_spmm_n_reduce(A, r, A->partials, out_nr);
}
