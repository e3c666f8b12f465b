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
  DN_CHECK(r >= 1 && r <= 1024, "rank %d outside [1, 1024]", r);
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
// A workgroup stages a column chunk of G (all r rows, 32*NB columns) in LDS once
// and then walks over 128-row tiles of X; each of its 4 waves owns 32 rows and
// NB MFMA blocks (32*NB output columns).  The contraction runs over the r
// components in steps of 8: lane (row = l%32, half = l/32) loads
// X[row][k0 + 4*half .. +3] straight from global memory, and MFMA step s
// contracts the component pair (k0 + s, k0 + 4 + s) against the matching two
// rows of G.  In LDS the chunk is stored as [k][l%32][block], so one ds_read of
// NB floats gives a lane its B operands of all NB blocks for one step.  The
// multiplicative update is applied in the epilogue, so X G is never written.
// ---------------------------------------------------------------------------
template <int NB>
struct GVec;
template <>
struct GVec<4> { typedef float4 type; };
template <>
struct GVec<2> { typedef float2 type; };
template <>
struct GVec<1> { typedef float type; };

template <int NB>
__device__ inline void load_g(const float* p, float (&g)[NB]) {
  typename GVec<NB>::type v = *reinterpret_cast<const typename GVec<NB>::type*>(p);
  if constexpr (NB == 4) { g[0] = v.x; g[1] = v.y; g[2] = v.z; g[3] = v.w; }
  else if constexpr (NB == 2) { g[0] = v.x; g[1] = v.y; }
  else { g[0] = v; }
}

template <int NB, int PD, bool VEC4>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
    k_xg_mu(const float* __restrict__ X, const float* __restrict__ G, const float* num, float eps,
            int64_t rows, int r, int nsteps, float* out, float* __restrict__ D_out) {
  extern __shared__ float g_lds[];  // [8 * nsteps][32][NB]
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int l32 = lane & 31, half = lane >> 5;
  constexpr int CW = 32 * NB;
  const int c0 = blockIdx.y * CW;
  const int kpad = 8 * nsteps;

  for (int idx = threadIdx.x; idx < kpad * CW; idx += 256) {
    const int k = idx / CW, c = idx % CW, gc = c0 + c;
    const float v = (k < r && gc < r) ? G[(int64_t)k * r + gc] : 0.0f;
    g_lds[(k * 32 + (c & 31)) * NB + (c >> 5)] = v;
  }
  __syncthreads();

  bool cok[NB];
#pragma unroll
  for (int i = 0; i < NB; i++) cok[i] = (c0 + 32 * i + l32) < r;

  const int64_t n_tiles = (rows + 127) / 128;

  // A operands of step `step` of tile `tile`: X[row][8 step + 4 half .. +3] (zeros outside X).
  auto load_x = [&](int64_t tile, int step, float (&xa)[4]) {
    const int64_t arow = tile * 128 + wave * 32 + l32;
    const bool ok = tile < n_tiles && arow < rows;
    const float* xrow = X + (ok ? arow : 0) * (int64_t)r;
    const int kk = 8 * step + 4 * half;
    if (VEC4) {
      // r % 8 == 0 here, so kk + 3 < r whenever 8 step < r
      float4 t = (ok && 8 * step < r) ? *reinterpret_cast<const float4*>(xrow + kk)
                                      : make_float4(0, 0, 0, 0);
      xa[0] = t.x; xa[1] = t.y; xa[2] = t.z; xa[3] = t.w;
    } else {
#pragma unroll
      for (int s = 0; s < 4; s++) xa[s] = (ok && kk + s < r) ? xrow[kk + s] : 0.0f;
    }
  };

  // The X operands form one stream over (tile, step); PD steps are kept in flight, across the
  // epilogue and into the next tile, so the MFMAs never wait for a fresh global load.
  float xq[PD][4];
  int64_t tile = blockIdx.x;
#pragma unroll
  for (int d = 0; d < PD; d++) load_x(tile, d, xq[d]);

  while (tile < n_tiles) {
    const int64_t next_tile = tile + gridDim.x;
    const int64_t row0 = tile * 128 + wave * 32;
    acc16 acc[NB];
#pragma unroll
    for (int i = 0; i < NB; i++)
      for (int v = 0; v < 16; v++) acc[i][v] = 0.0f;

    // Epilogue operands (numerator and X in the accumulator layout) are requested now and
    // arrive while the MFMAs run.
    float pn[NB][16], px[NB][16];
#pragma unroll
    for (int i = 0; i < NB; i++) {
      const int col = c0 + 32 * i + l32;
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int64_t row = row0 + 8 * (v >> 2) + 4 * half + (v & 3);
        const bool ok = cok[i] && row < rows;
        const int64_t idx = ok ? row * (int64_t)r + col : 0;
        pn[i][v] = ok ? num[idx] : 0.0f;
        px[i][v] = ok ? X[idx] : 0.0f;
      }
    }

    for (int s0 = 0; s0 < nsteps; s0 += PD) {
      const bool last_round = s0 + PD >= nsteps;
#pragma unroll
      for (int d = 0; d < PD; d++) {
        const int step = s0 + d;
#pragma unroll
        for (int s = 0; s < 4; s++) {
          float g[NB];
          load_g<NB>(g_lds + ((8 * step + 4 * half + s) * 32 + l32) * NB, g);
#pragma unroll
          for (int i = 0; i < NB; i++)
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(xq[d][s], g[i], acc[i], 0, 0, 0);
        }
        if (last_round)
          load_x(next_tile, d, xq[d]);
        else
          load_x(tile, step + PD, xq[d]);
      }
    }

#pragma unroll
    for (int i = 0; i < NB; i++) {
      if (!cok[i]) continue;
      const int col = c0 + 32 * i + l32;
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int64_t row = row0 + 8 * (v >> 2) + 4 * half + (v & 3);
        if (row < rows) {
          const int64_t idx = row * (int64_t)r + col;
          const float d = acc[i][v];
          const float q = pn[i][v] / (d + eps);
          out[idx] = px[i][v] * q;
          if (D_out) D_out[idx] = d;
        }
      }
    }
    tile = next_tile;
  }
}

template <int NB, int PD, bool VEC4>
static int launch_xg_mu_inst(dim3 grid, size_t lds, const float* X, const float* G,
                             const float* num, float eps, int64_t rows, int r, int nsteps,
                             float* out, float* D_out) {
  static bool attr_set = false;
  if (!attr_set) {
    DN_HIP(hipFuncSetAttribute((const void*)k_xg_mu<NB, PD, VEC4>,
                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    attr_set = true;
  }
  hipLaunchKernelGGL((k_xg_mu<NB, PD, VEC4>), grid, dim3(256), lds, stream(), X, G, num, eps, rows,
                     r, nsteps, out, D_out);
  DN_LAUNCH_CHECK();
  return 0;
}

template <int NB>
static int launch_xg_mu_nb(int64_t rows, int r, const float* X, const float* G, const float* num,
                           float eps, float* out, float* D_out) {
  int nsteps = (r + 7) / 8;
  if (nsteps > 2 && (nsteps & 1)) nsteps++;  // zero-padded, so that two steps can be in flight
  const int pd = nsteps % 4 == 0 ? 4 : nsteps % 2 == 0 ? 2 : 1;
  const size_t lds = (size_t)nsteps * 8 * 32 * NB * sizeof(float);
  const bool vec4 = (r % 8 == 0) && ((uintptr_t)X % 16 == 0);
  int64_t tiles = ceil_div(rows, 128);
  int64_t wgs = (int64_t)n_cus() * (lds <= 72 * 1024 ? 2 : 1);
  if (wgs > tiles) wgs = tiles;
  dim3 grid((unsigned)wgs, (unsigned)ceil_div(r, 32 * NB));
#define DN_XG(PDV)                                                                              \
  (vec4 ? launch_xg_mu_inst<NB, PDV, true>(grid, lds, X, G, num, eps, rows, r, nsteps, out, D_out) \
        : launch_xg_mu_inst<NB, PDV, false>(grid, lds, X, G, num, eps, rows, r, nsteps, out, D_out))
  switch (pd) {
    case 4: return DN_XG(4);
    case 2: return DN_XG(2);
    default: return DN_XG(1);
  }
#undef DN_XG
}

int launch_xg_mu(int64_t rows, int r, const float* X, const float* G, const float* num, float eps,
                 float* out, float* D_out) {
  DN_CHECK(r >= 1 && r <= 1024, "rank %d outside [1, 1024]", r);
  DN_CHECK(out != X, "xg_mu: out must not alias X");
  if (rows <= 0) return 0;
  // widest column chunk whose slice of G fits 128 KB of LDS
  if (r <= 256) return launch_xg_mu_nb<4>(rows, r, X, G, num, eps, out, D_out);
  if (r <= 512) return launch_xg_mu_nb<2>(rows, r, X, G, num, eps, out, D_out);
  return launch_xg_mu_nb<1>(rows, r, X, G, num, eps, out, D_out);
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

__global__ void __launch_bounds__(256)
    k_copy(int64_t count, const float* __restrict__ src, float* __restrict__ dst) {
  int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += stride) dst[i] = src[i];
}

DN_API int dnpeff_op_copy(int64_t count, const float* src, float* dst) {
  clear_error();
  if (count <= 0) return 0;
  int64_t g = ceil_div(count, 256);
  if (g > 65536 * 16) g = 65536 * 16;
  hipLaunchKernelGGL(k_copy, dim3((unsigned)g), dim3(256), 0, stream(), count, src, dst);
  DN_LAUNCH_CHECK();
  return 0;
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
