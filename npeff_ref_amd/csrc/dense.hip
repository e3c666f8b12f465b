// Dense kernels of the MU iteration for tall-skinny factors X [rows, r] with the
// r components contiguous: Gram X^T X and X G on fp32 MFMA (32x32x2), the
// multiplicative update fused into the X G epilogue, dot products with fp64
// accumulation, seeded initialisation and the [m, r] <-> [r, m] transposition.
#include "dnpeff_internal.hpp"
#include "synth_rng.h"

namespace dn {

typedef float acc16 __attribute__((ext_vector_type(16)));

// ---------------------------------------------------------------------------
// F[i] *= num[i] / (den[i] + eps)      (divide first, then multiply)
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
    k_mu(int64_t count, float* __restrict__ F, const float* __restrict__ num,
         const float* __restrict__ den, float eps) {
  int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += stride)
    F[i] *= num[i] / (den[i] + eps);
}

int launch_mu(int64_t count, float* F, const float* num, const float* den, float eps) {
  if (count <= 0) return 0;
  int64_t g = ceil_div(count, 256);
  if (g > 65536 * 16) g = 65536 * 16;
  hipLaunchKernelGGL(k_mu, dim3((unsigned)g), dim3(256), 0, stream(), count, F, num, den, eps);
  DN_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// Gram  G = X^T X
//
// One workgroup (4 waves) owns a 128 x 128 tile of G over a slice of the rows of
// X; wave w owns the 64 x 64 quadrant (w/2, w%2) as 2 x 2 MFMA blocks.  Operand
// layout of v_mfma_f32_32x32x2f32: lane l supplies A[i = l%32][k = l/32] and
// B[k = l/32][j = l%32]; both come straight from two consecutive rows of X, so
// every load is a pair of 128-byte row segments.  Accumulators are flushed into
// a second set every GRAM_FLUSH rows so no fp32 running sum grows long.  Slice
// partials are summed in fp64 in slice order by k_gram_reduce.
// ---------------------------------------------------------------------------
constexpr int GRAM_TILE = 128;
constexpr int64_t GRAM_FLUSH = 4096;
constexpr int GRAM_MAX_SLICES = 1024;

static int64_t gram_slices(int64_t rows) {
  int64_t s = ceil_div(rows, 256);
  if (s > GRAM_MAX_SLICES) s = GRAM_MAX_SLICES;
  if (s < 1) s = 1;
  return s;
}

int64_t gram_workspace_floats(int64_t rows, int r) {
  int64_t tiles = ceil_div(r, GRAM_TILE);
  return gram_slices(rows) * tiles * tiles * GRAM_TILE * GRAM_TILE;
}

__global__ void __launch_bounds__(256)
    k_gram(const float* __restrict__ X, int64_t rows, int r, int64_t rows_per_slice, int tiles,
           float* __restrict__ partials) {
  const int slice = blockIdx.x;
  const int tile_a = blockIdx.y / tiles, tile_b = blockIdx.y % tiles;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int ca = tile_a * GRAM_TILE + (wave >> 1) * 64 + l32;  // column of X feeding A, block 0
  const int cb = tile_b * GRAM_TILE + (wave & 1) * 64 + l32;   // column of X feeding B, block 0
  const bool a0ok = ca < r, a1ok = ca + 32 < r, b0ok = cb < r, b1ok = cb + 32 < r;

  int64_t k0 = (int64_t)slice * rows_per_slice;
  int64_t k1 = k0 + rows_per_slice;
  if (k1 > rows) k1 = rows;

  acc16 acc[4], tot[4];
  for (int i = 0; i < 4; i++)
    for (int v = 0; v < 16; v++) {
      acc[i][v] = 0.0f;
      tot[i][v] = 0.0f;
    }

  for (int64_t kf = k0; kf < k1; kf += GRAM_FLUSH) {
    int64_t kend = kf + GRAM_FLUSH < k1 ? kf + GRAM_FLUSH : k1;
    int64_t k = kf;
    // full groups of 8 row pairs, loads issued ahead of the MFMAs
    for (; k + 16 <= kend; k += 16) {
      float a0[8], a1[8], b0[8], b1[8];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const float* row = X + (k + 2 * u + half) * (int64_t)r;
        a0[u] = a0ok ? row[ca] : 0.0f;
        a1[u] = a1ok ? row[ca + 32] : 0.0f;
        b0[u] = b0ok ? row[cb] : 0.0f;
        b1[u] = b1ok ? row[cb + 32] : 0.0f;
      }
#pragma unroll
      for (int u = 0; u < 8; u++) {
        acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[u], b0[u], acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[u], b1[u], acc[1], 0, 0, 0);
        acc[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[u], b0[u], acc[2], 0, 0, 0);
        acc[3] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[u], b1[u], acc[3], 0, 0, 0);
      }
    }
    for (; k < kend; k += 2) {
      int64_t kr = k + half;
      bool rok = kr < kend;
      const float* row = X + kr * (int64_t)r;
      float a0 = (rok && a0ok) ? row[ca] : 0.0f;
      float a1 = (rok && a1ok) ? row[ca + 32] : 0.0f;
      float b0 = (rok && b0ok) ? row[cb] : 0.0f;
      float b1 = (rok && b1ok) ? row[cb + 32] : 0.0f;
      acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0], 0, 0, 0);
      acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[1], 0, 0, 0);
      acc[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[2], 0, 0, 0);
      acc[3] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[3], 0, 0, 0);
    }
    for (int i = 0; i < 4; i++)
      for (int v = 0; v < 16; v++) {
        tot[i][v] += acc[i][v];
        acc[i][v] = 0.0f;
      }
  }

  // D layout of the 32x32 block: reg v of lane l holds row 8*(v/4) + 4*(l/32) + v%4,
  // column l%32.
  float* out = partials + ((int64_t)slice * tiles * tiles + blockIdx.y) * (GRAM_TILE * GRAM_TILE);
  for (int i = 0; i < 4; i++) {
    int rb = (wave >> 1) * 64 + (i >> 1) * 32;
    int cbk = (wave & 1) * 64 + (i & 1) * 32;
    for (int v = 0; v < 16; v++) {
      int rr = rb + 8 * (v >> 2) + 4 * half + (v & 3);
      out[rr * GRAM_TILE + cbk + l32] = tot[i][v];
    }
  }
}

__global__ void __launch_bounds__(256)
    k_gram_reduce(const float* __restrict__ partials, int64_t slices, int tiles, int r,
                  float* __restrict__ G) {
  int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= r * r) return;
  int a = idx / r, b = idx % r;
  int tile = (a / GRAM_TILE) * tiles + (b / GRAM_TILE);
  int off = (a % GRAM_TILE) * GRAM_TILE + (b % GRAM_TILE);
  double s = 0.0;
  for (int64_t sl = 0; sl < slices; sl++)
    s += (double)partials[(sl * tiles * tiles + tile) * (GRAM_TILE * GRAM_TILE) + off];
  G[idx] = (float)s;
}

int launch_gram(int64_t rows, int r, const float* X, float* G, float* workspace) {
  DN_CHECK(r >= 1 && r <= 4096, "rank %d outside [1, 4096]", r);
  int tiles = (int)ceil_div(r, GRAM_TILE);
  int64_t slices = gram_slices(rows);
  int64_t rps = ceil_div(rows > 0 ? rows : 1, slices);
  rps = ceil_div(rps, 2) * 2;  // slices start on even rows
  hipLaunchKernelGGL(k_gram, dim3((unsigned)slices, (unsigned)(tiles * tiles)), dim3(256), 0,
                     stream(), X, rows, r, rps, tiles, workspace);
  hipLaunchKernelGGL(k_gram_reduce, dim3((unsigned)ceil_div((int64_t)r * r, 256)), dim3(256), 0,
                     stream(), workspace, slices, tiles, r, G);
  DN_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// out = X * num / (X G + eps)
//
// A wave owns 32 rows of X and up to 128 output columns (4 MFMA blocks); the
// workgroup's 4 waves own 128 consecutive rows.  The contraction runs over the
// r components in steps of 8: lane (row = l%32, half = l/32) loads
// X[row][k0 + 4*half .. +3], and MFMA step s contracts the component pair
// (k0 + s, k0 + 4 + s) against the matching two rows of G.
// ---------------------------------------------------------------------------
template <bool VEC4>
__global__ void __launch_bounds__(256)
    k_xg_mu(const float* __restrict__ X, const float* __restrict__ G, const float* num, float eps,
            int64_t rows, int r, float* out,
            float* __restrict__ D_out) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int64_t row0 = (int64_t)blockIdx.x * 128 + wave * 32;
  if (row0 >= rows) return;
  const int c0 = blockIdx.y * 128;
  const int64_t arow = row0 + l32;
  const bool arow_ok = arow < rows;
  const float* xrow = X + (arow_ok ? arow : 0) * (int64_t)r;

  acc16 acc[4];
  for (int i = 0; i < 4; i++)
    for (int v = 0; v < 16; v++) acc[i][v] = 0.0f;

  bool cok[4];
  for (int i = 0; i < 4; i++) cok[i] = (c0 + 32 * i + l32) < r;

  for (int k0 = 0; k0 < r; k0 += 8) {
    const int kk = k0 + 4 * half;
    float xa[4];
    if (VEC4) {
      // r % 8 == 0 here, so kk + 3 < r
      float4 t = arow_ok ? *reinterpret_cast<const float4*>(xrow + kk) : make_float4(0, 0, 0, 0);
      xa[0] = t.x; xa[1] = t.y; xa[2] = t.z; xa[3] = t.w;
    } else {
#pragma unroll
      for (int s = 0; s < 4; s++) xa[s] = (arow_ok && kk + s < r) ? xrow[kk + s] : 0.0f;
    }
#pragma unroll
    for (int s = 0; s < 4; s++) {
      const int kg = kk + s;
      const bool kok = kg < r;
      const float* grow = G + (int64_t)(kok ? kg : 0) * r + c0 + l32;
      float g0 = (kok && cok[0]) ? grow[0] : 0.0f;
      float g1 = (kok && cok[1]) ? grow[32] : 0.0f;
      float g2 = (kok && cok[2]) ? grow[64] : 0.0f;
      float g3 = (kok && cok[3]) ? grow[96] : 0.0f;
      acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(xa[s], g0, acc[0], 0, 0, 0);
      acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(xa[s], g1, acc[1], 0, 0, 0);
      acc[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(xa[s], g2, acc[2], 0, 0, 0);
      acc[3] = __builtin_amdgcn_mfma_f32_32x32x2f32(xa[s], g3, acc[3], 0, 0, 0);
    }
  }

  for (int i = 0; i < 4; i++) {
    if (!cok[i]) continue;
    const int col = c0 + 32 * i + l32;
    for (int v = 0; v < 16; v++) {
      int64_t row = row0 + 8 * (v >> 2) + 4 * half + (v & 3);
      if (row < rows) {
        int64_t idx = row * (int64_t)r + col;
        float d = acc[i][v];
        float x = X[idx];
        float q = num[idx] / (d + eps);
        out[idx] = x * q;
        if (D_out) D_out[idx] = d;
      }
    }
  }
}

int launch_xg_mu(int64_t rows, int r, const float* X, const float* G, const float* num, float eps,
                 float* out, float* D_out) {
  DN_CHECK(r >= 1 && r <= 4096, "rank %d outside [1, 4096]", r);
  DN_CHECK(out != X, "xg_mu: out must not alias X");
  if (rows <= 0) return 0;
  dim3 grid((unsigned)ceil_div(rows, 128), (unsigned)ceil_div(r, 128));
  if (r % 8 == 0 && ((uintptr_t)X % 16 == 0))
    hipLaunchKernelGGL((k_xg_mu<true>), grid, dim3(256), 0, stream(), X, G, num, eps, rows, r, out,
                       D_out);
  else
    hipLaunchKernelGGL((k_xg_mu<false>), grid, dim3(256), 0, stream(), X, G, num, eps, rows, r,
                       out, D_out);
  DN_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// <x, y> with fp64 accumulation; fixed grid, fixed order.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
    k_dot_partial(int64_t count, const float* __restrict__ x, const float* __restrict__ y,
                  double* __restrict__ partials) {
  __shared__ double sh[256];
  double s = 0.0;
  int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += stride)
    s += (double)x[i] * (double)y[i];
  sh[threadIdx.x] = s;
  __syncthreads();
  for (int off = 128; off > 0; off >>= 1) {
    if (threadIdx.x < off) sh[threadIdx.x] += sh[threadIdx.x + off];
    __syncthreads();
  }
  if (threadIdx.x == 0) partials[blockIdx.x] = sh[0];
}

__global__ void __launch_bounds__(256)
    k_dot_final(const double* __restrict__ partials, int n, double* __restrict__ out) {
  __shared__ double sh[256];
  double s = 0.0;
  for (int i = threadIdx.x; i < n; i += 256) s += partials[i];
  sh[threadIdx.x] = s;
  __syncthreads();
  for (int off = 128; off > 0; off >>= 1) {
    if (threadIdx.x < off) sh[threadIdx.x] += sh[threadIdx.x + off];
    __syncthreads();
  }
  if (threadIdx.x == 0) *out = sh[0];
}

int launch_dot(int64_t count, const float* x, const float* y, double* partials, double* out_dev) {
  hipLaunchKernelGGL(k_dot_partial, dim3(DOT_BLOCKS), dim3(256), 0, stream(), count, x, y,
                     partials);
  hipLaunchKernelGGL(k_dot_final, dim3(1), dim3(256), 0, stream(), partials, DOT_BLOCKS, out_dev);
  DN_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// Seeded U[0,1) factors, keyed by the logical element.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
    k_init_uniform(int matrix_id, int64_t lrows, int64_t lcols, uint64_t seed,
                   float* __restrict__ x) {
  int64_t total = lrows * lcols;
  int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
    if (matrix_id == 1) {
      // H is logically [r, m] = [lrows, lcols]; device layout [m, r]
      int64_t j = i / lrows, c = i % lrows;
      x[i] = dn_uniform_at(seed, 1, c, j, lcols);
    } else {
      x[i] = dn_uniform_at(seed, matrix_id, i / lcols, i % lcols, lcols);
    }
  }
}

int launch_init_uniform(int matrix_id, int64_t logical_rows, int64_t logical_cols, uint64_t seed,
                        float* x) {
  int64_t total = logical_rows * logical_cols;
  if (total <= 0) return 0;
  int64_t g = ceil_div(total, 256);
  if (g > 65536 * 4) g = 65536 * 4;
  hipLaunchKernelGGL(k_init_uniform, dim3((unsigned)g), dim3(256), 0, stream(), matrix_id,
                     logical_rows, logical_cols, seed, x);
  DN_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// out[c * rows + i] = in[i * cols + c], 32 x 32 tiles through LDS.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
    k_transpose(const float* __restrict__ in, int64_t rows, int64_t cols, float* __restrict__ out) {
  __shared__ float tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
  const int64_t tiles_c = (cols + 31) / 32;
  const int64_t tile_r = blockIdx.x / tiles_c, tile_c = blockIdx.x % tiles_c;
  const int64_t r0 = tile_r * 32, c0 = tile_c * 32;
  for (int i = ty; i < 32; i += 8) {
    int64_t rr = r0 + i, cc = c0 + tx;
    tile[i][tx] = (rr < rows && cc < cols) ? in[rr * cols + cc] : 0.0f;
  }
  __syncthreads();
  for (int i = ty; i < 32; i += 8) {
    int64_t cc = c0 + i, rr = r0 + tx;
    if (cc < cols && rr < rows) out[cc * rows + rr] = tile[tx][i];
  }
}

int launch_transpose(int64_t rows, int64_t cols, const float* in, float* out) {
  if (rows <= 0 || cols <= 0) return 0;
  int64_t tiles = ceil_div(rows, 32) * ceil_div(cols, 32);
  DN_CHECK(tiles < (int64_t)INT32_MAX, "matrix too large for the transposition grid");
  hipLaunchKernelGGL(k_transpose, dim3((unsigned)tiles), dim3(256), 0, stream(), in, rows, cols,
                     out);
  DN_LAUNCH_CHECK();
  return 0;
}

}  // namespace dn

using namespace dn;

DN_API float dnpeff_uniform_at(uint64_t seed, int matrix_id, int64_t row, int64_t col,
                               int64_t n_cols) {
  return dn_uniform_at(seed, matrix_id, row, col, n_cols);
}

DN_API int dnpeff_op_mu(int64_t count, float* F, const float* num, const float* den, float eps) {
  clear_error();
  return launch_mu(count, F, num, den, eps);
}

DN_API int dnpeff_op_gram(int64_t rows, int r, const float* X, float* G_rr) {
  clear_error();
  float* ws = nullptr;
  DN_TRY(dmalloc(&ws, gram_workspace_floats(rows, r)));
  int s = launch_gram(rows, r, X, G_rr, ws);
  if (!s && hipStreamSynchronize(stream()) != hipSuccess) {
    set_error("gram kernel failed");
    s = 1;
  }
  dfree(ws);
  return s;
}

DN_API int dnpeff_op_xg_mu(int64_t rows, int r, const float* X, const float* G_rr, const float* num,
                           float eps, float* out, float* D_out) {
  clear_error();
  return launch_xg_mu(rows, r, X, G_rr, num, eps, out, D_out);
}

DN_API int dnpeff_op_dot(int64_t count, const float* x, const float* y, double* out_host) {
  clear_error();
  DN_CHECK(out_host != nullptr, "out is NULL");
  double* ws = nullptr;
  DN_TRY(dmalloc(&ws, DOT_BLOCKS + 1));
  int s = launch_dot(count, x, y, ws, ws + DOT_BLOCKS);
  if (!s && hipMemcpy(out_host, ws + DOT_BLOCKS, sizeof(double), hipMemcpyDeviceToHost) != hipSuccess) {
    set_error("dot: copy of the result failed");
    s = 1;
  }
  dfree(ws);
  return s;
}

DN_API int dnpeff_op_init_uniform(int matrix_id, int64_t logical_rows, int64_t logical_cols,
                                  uint64_t seed, float* x) {
  clear_error();
  return launch_init_uniform(matrix_id, logical_rows, logical_cols, seed, x);
}
