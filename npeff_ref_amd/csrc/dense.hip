// Dense kernels of the MU iteration for tall-skinny factors X [rows, r] with the
// r components contiguous: Gram X^T X and X G on fp32 MFMA (32x32x2), the
// multiplicative update fused into the X G epilogue, dot products with fp64
// accumulation, seeded initialisation and the [m, r] <-> [r, m] transposition.
#include "dnpeff_internal.hpp"
#include "abt_b16.hpp"
#include "synth_rng.h"

#include <type_traits>

namespace dn {

typedef float acc16 __attribute__((ext_vector_type(16)));

// n / den from the reciprocal (1 ulp) and one correction step: 5 vector instructions where the
// IEEE division sequence takes 11.  For the epilogues of the split-operand updates, where
// den = (X G) + eps is positive and normal; within 2 ulp of the quotient.
__device__ __forceinline__ float mu_quotient(float n, float den) {
  const float rc = __builtin_amdgcn_rcpf(den), q0 = n * rc;
  return __builtin_fmaf(__builtin_fmaf(-den, q0, n), rc, q0);
}

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
// v_mfma_f32_32x32x2f32 takes from lane l the element A[i = l%32][k = l/32] and
// B[k = l/32][j = l%32].  Here k runs over two consecutive rows of X and the 32
// "columns" of an operand block are every fourth column of a 128-column tile:
// strided block sb = 4 t + a holds columns 128 t + 4 i + a, i < 32.  Lane l then
// needs X[k + l/32][128 t + 4 (l%32) + a] for a = 0..3: ONE 16-byte load per lane
// and row pair feeds all four strided blocks of the tile, i.e. the A and B
// operands of up to 16 MFMAs, and 16-byte loads are the only form that reaches
// the L1's full rate.  G is symmetric, so only block pairs (sbi <= sbj) are
// computed; the reduce kernel mirrors and un-strides them.  Pairs are numbered
// row by row; a wave owns two consecutive pairs over a slice of the rows of X, a
// workgroup of 5 waves owns 10 (all of G for r <= 128).  Accumulators are flushed
// are kept per slice (at most rows / 2048 rows each), and the slice partials are summed in
// fp64 in slice order by k_gram_reduce, so no fp32 running sum grows long.
// ---------------------------------------------------------------------------
constexpr int GRAM_MAX_SLICES = 2048;
constexpr int GRAM_UNR = 8;  // row pairs in flight per wave

static int64_t gram_slices(int64_t rows) {
  int64_t s = ceil_div(rows, 256);
  if (s > GRAM_MAX_SLICES) s = GRAM_MAX_SLICES;
  if (s < 1) s = 1;
  return s;
}

__host__ __device__ inline int gram_blocks(int r) { return 4 * ((r + 127) / 128); }
// Number of the block pair (bi <= bj) in row-major order over the upper triangle.
__host__ __device__ inline int gram_pair_index(int bi, int bj, int nb) {
  return bi * nb - bi * (bi - 1) / 2 + (bj - bi);
}
static int gram_pairs(int r) {
  int nb = gram_blocks(r);
  return nb * (nb + 1) / 2;
}

static bool gram_uses_tiles(int64_t rows, int r) { return r > 128 && r % 128 == 0 && rows >= 1024; }

static int64_t gram_small_wgs(int64_t rows);

int64_t gram_workspace_floats(int64_t rows, int r) {
  if (r <= 32) return gram_small_wgs(rows) * 1024;  // one 32 x 32 block per workgroup of k_gram_small
  if (gram_uses_tiles(rows, r)) return gram_tiles_workspace_floats(rows, r);
  return gram_slices(rows) * (int64_t)gram_pairs(r) * 1024;
}

template <int A>
__device__ inline float comp4(const float4& v) {
  return A == 0 ? v.x : A == 1 ? v.y : A == 2 ? v.z : v.w;
}

constexpr int GRAM_TILE_FLOATS = 4096;  // one LDS slot: KB rows x ld columns (16 KB)
constexpr int GRAM_STAGES = 3;          // row tiles in flight in registers
constexpr int GRAM_NP = 3;              // block pairs per wave

// LDS position of column c of a row: the four strided blocks of a 128-column tile are stored
// one after the other, 32 floats each, so that the 32 lanes reading one block touch 32
// different banks.
__device__ inline int gram_lds_col(int c) { return (c & ~127) + 32 * (c & 3) + ((c & 127) >> 2); }

// Streams row tiles of X through two LDS slots of `kb` rows each.  Every element is read from
// global memory once per workgroup, with 16-byte loads issued GRAM_STAGES tiles ahead of their
// use (global latency is several microseconds, one tile of MFMAs lasts about one), parked in
// registers and written to the free LDS slot one tile ahead.
template <int NW, bool VEC4>
struct GramPipe {
  static constexpr int THREADS = 64 * NW;
  static constexpr int NVEC = (GRAM_TILE_FLOATS / 4 + THREADS - 1) / THREADS;
  const float* __restrict__ X;
  int r, ld, kb;
  int64_t k1;  // number of rows of X
  float4 stage[GRAM_STAGES][NVEC];

  __device__ inline void fetch(int st, int64_t kt) {
    if (!VEC4) return;
    const int r4 = r >> 2;
#pragma unroll
    for (int q = 0; q < NVEC; q++) {
      const int f = threadIdx.x + q * THREADS;
      const int64_t row = kt + f / r4;
      const bool ok = f < kb * r4 && row < k1;
      stage[st][q] = ok ? *reinterpret_cast<const float4*>(X + row * (int64_t)r + 4 * (f % r4))
                        : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
  }
  __device__ inline void commit(int st, float* slot, int64_t kt) {
    if (VEC4) {
      const int r4 = r >> 2;
#pragma unroll
      for (int q = 0; q < NVEC; q++) {
        const int f = threadIdx.x + q * THREADS;
        if (f < kb * r4) {
          const int c4 = f % r4;  // columns 4 c4 .. 4 c4 + 3 = position c4 % 32 of blocks 0..3
          float* p = slot + (f / r4) * ld + (c4 >> 5) * 128 + (c4 & 31);
          p[0] = stage[st][q].x;
          p[32] = stage[st][q].y;
          p[64] = stage[st][q].z;
          p[96] = stage[st][q].w;
        }
      }
    } else {
      for (int e = threadIdx.x; e < kb * r; e += THREADS) {
        const int64_t row = kt + e / r;
        const int c = e % r;
        slot[(e / r) * ld + gram_lds_col(c)] = row < k1 ? X[row * (int64_t)r + c] : 0.0f;
      }
    }
  }
};

struct GramPairs {  // strided-block residues of a wave's block pairs within its tile pair
  int a[GRAM_NP], b[GRAM_NP], n;
};

// MFMAs of one LDS slot for the wave's NP block pairs.  KB > 0, LD > 0: tile height and LDS row
// length known at compile time (the loop is fully unrolled, LDS reads carry immediate offsets
// and are scheduled ahead of the MFMAs of the previous row group); KB = 0: run-time values.
template <int NP, int KB, int LD>
__device__ inline void gram_tile_mfma(const float* __restrict__ slot, int kb_rt, int ld_rt, int ta,
                                      int tb, const GramPairs& gp, int lane, acc16 (&acc)[GRAM_NP]) {
  const int l32 = lane & 31, half = lane >> 5;
  const int ld = KB > 0 ? LD : ld_rt;
  const int kb = KB > 0 ? KB : kb_rt;
  const float* pa[NP];
  const float* pb[NP];
#pragma unroll
  for (int i = 0; i < NP; i++) {
    pa[i] = slot + half * ld + 128 * ta + 32 * gp.a[i] + l32;
    pb[i] = slot + half * ld + 128 * tb + 32 * gp.b[i] + l32;
  }
  if (KB > 0) {
    constexpr int GRP = 4;  // row pairs whose operands are read together
#pragma unroll
    for (int g = 0; g < KB / 2; g += GRP) {
      float xa[GRP][NP], xb[GRP][NP];
#pragma unroll
      for (int u = 0; u < GRP; u++)
#pragma unroll
        for (int i = 0; i < NP; i++) {
          xa[u][i] = pa[i][2 * (g + u) * LD];
          xb[u][i] = pb[i][2 * (g + u) * LD];
        }
#pragma unroll
      for (int u = 0; u < GRP; u++)
#pragma unroll
        for (int i = 0; i < NP; i++)
          acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(xa[u][i], xb[u][i], acc[i], 0, 0, 0);
    }
  } else {
    for (int kk = 0; kk < kb; kk += 2) {
      float xa[NP], xb[NP];
#pragma unroll
      for (int i = 0; i < NP; i++) {
        xa[i] = pa[i][kk * ld];
        xb[i] = pb[i][kk * ld];
      }
#pragma unroll
      for (int i = 0; i < NP; i++)
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(xa[i], xb[i], acc[i], 0, 0, 0);
    }
  }
}

// The row tiles of X are dealt to the slices round-robin (slice s owns tiles s, s + S, ...), so
// that at any moment the workgroups read one contiguous window of X.
template <int NW, int NP, bool FAST, bool VEC4>
__device__ inline void gram_stream(const float* __restrict__ X, int r, int kb, int64_t rows,
                                   int slice, int n_slices, float* __restrict__ lds, int lane,
                                   int ta, int tb, const GramPairs& gp, float* __restrict__ base,
                                   int nb) {
  GramPipe<NW, VEC4> pipe;
  const int ld = 128 * ((r + 127) / 128);
  pipe.X = X; pipe.r = r; pipe.ld = ld; pipe.kb = kb; pipe.k1 = rows;
  const int64_t all_tiles = (rows + kb - 1) / kb;
  const int64_t n_tiles = all_tiles > slice ? (all_tiles - slice + n_slices - 1) / n_slices : 0;
  const int64_t k0 = (int64_t)slice * kb;         // first row of this slice's tile 0
  const int64_t tstride = (int64_t)n_slices * kb;  // rows between consecutive tiles of the slice
  acc16 acc[GRAM_NP];
  for (int i = 0; i < GRAM_NP; i++)
    for (int v = 0; v < 16; v++) acc[i][v] = 0.0f;
  if (!VEC4 || ld != r) {  // padding columns of the LDS rows are read as operands: zero them once
    for (int e = threadIdx.x; e < 2 * GRAM_TILE_FLOATS; e += 64 * NW) lds[e] = 0.0f;
    __syncthreads();
  }
#pragma unroll
  for (int st = 0; st < GRAM_STAGES; st++) pipe.fetch(st, k0 + (int64_t)st * tstride);
  if (n_tiles > 0) pipe.commit(0, lds, k0);
  __syncthreads();

  // iteration t: tile t is in slot t & 1; stage[t % S] is free and receives tile t + S;
  // tile t + 1 sits in stage[(t + 1) % S] and moves to the other slot after the MFMAs.
  auto step = [&](int64_t t, auto st_tag) {
    constexpr int ST = decltype(st_tag)::value;
    pipe.fetch(ST, k0 + (t + GRAM_STAGES) * tstride);
    gram_tile_mfma<NP, FAST ? 32 : 0, FAST ? 128 : 0>(lds + (t & 1) * GRAM_TILE_FLOATS, kb, ld, ta, tb,
                                                       gp, lane, acc);
    if (t + 1 < n_tiles)
      pipe.commit((ST + 1) % GRAM_STAGES, lds + ((t + 1) & 1) * GRAM_TILE_FLOATS,
                  k0 + (t + 1) * tstride);
    __syncthreads();
  };
  int64_t t = 0;
  for (; t + GRAM_STAGES <= n_tiles; t += GRAM_STAGES) {
    step(t, std::integral_constant<int, 0>{});
    step(t + 1, std::integral_constant<int, 1>{});
    step(t + 2, std::integral_constant<int, 2>{});
  }
  if (t < n_tiles) step(t, std::integral_constant<int, 0>{});
  if (t + 1 < n_tiles) step(t + 1, std::integral_constant<int, 1>{});

  const int l32 = lane & 31, half = lane >> 5;
  // D layout of the 32x32 block: reg v of lane l holds row 8*(v/4) + 4*(l/32) + v%4, column l%32.
#pragma unroll
  for (int i = 0; i < NP; i++) {
    {
      float* out = base + (int64_t)gram_pair_index(4 * ta + gp.a[i], 4 * tb + gp.b[i], nb) * 1024;
      for (int v = 0; v < 16; v++) {
        const int rr = 8 * (v >> 2) + 4 * half + (v & 3);
        out[rr * 32 + l32] = acc[i][v];
      }
    }
  }
}

// Tile pair number -> (ta <= tb), row by row over the upper triangle.
__device__ inline void gram_tile_pair(int p, int n_tiles, int& ta, int& tb) {
  ta = 0;
  int row_len = n_tiles;
  while (p >= row_len) {
    p -= row_len;
    ta++;
    row_len--;
  }
  tb = ta + p;
}

// One workgroup of 4 waves per (tile pair, slice).  A diagonal tile pair has 10 distinct block
// pairs (a <= b): waves take 3, 3, 3, 1.  An off-diagonal one has 16: two workgroups' worth is
// covered by launching it twice in grid.x (sub = 0: residues a in {0, 1}, sub = 1: {2, 3}),
// each wave taking a row half: 2 pairs.  Here: one kernel, NP chosen per wave at run time.
template <bool VEC4>
__global__ void __launch_bounds__(256)
    k_gram(const float* __restrict__ X, int64_t rows, int r, int kb, int n_pairs, int n_tiles,
           float* __restrict__ partials) {
  __shared__ __align__(16) float lds[2 * GRAM_TILE_FLOATS];
  const int slice = blockIdx.y, n_slices = gridDim.y;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int nb = gram_blocks(r);
  // grid.x: first the diagonal tile pairs (one workgroup each), then the off-diagonal ones
  // (two workgroups each)
  int ta, tb, sub = 0;
  bool diag;
  if ((int)blockIdx.x < n_tiles) {
    ta = tb = blockIdx.x;
    diag = true;
  } else {
    const int q = blockIdx.x - n_tiles;
    // off-diagonal pairs (ta < tb) numbered row by row
    int p = q >> 1, row_len = n_tiles - 1;
    ta = 0;
    while (p >= row_len) {
      p -= row_len;
      ta++;
      row_len--;
    }
    tb = ta + 1 + p;
    sub = q & 1;
    diag = false;
  }
  float* base = partials + (int64_t)slice * n_pairs * 1024;
  GramPairs gp;
  if (diag) {
    // (0,0)(0,1)(0,2) | (0,3)(1,1)(1,2) | (1,3)(2,2)(2,3) | (3,3)
    const int A[4][3] = {{0, 0, 0}, {0, 1, 1}, {1, 2, 2}, {3, 3, 3}};
    const int B[4][3] = {{0, 1, 2}, {3, 1, 2}, {3, 2, 3}, {3, 3, 3}};
    for (int i = 0; i < 3; i++) {
      gp.a[i] = A[wave][i];
      gp.b[i] = B[wave][i];
    }
    gp.n = wave == 3 ? 1 : 3;
  } else {
    // residue a = 2 sub + wave / 2, b in {2 (wave % 2), 2 (wave % 2) + 1}
    for (int i = 0; i < 3; i++) {
      gp.a[i] = 2 * sub + (wave >> 1);
      gp.b[i] = 2 * (wave & 1) + (i & 1);
    }
    gp.n = 2;
  }
  // r <= 128 has one tile of 128 LDS columns and 32 rows per slot: fully unrolled MFMA loop
  if (r <= 128) {
    if (gp.n == 3)
      gram_stream<4, 3, true, VEC4>(X, r, kb, rows, slice, n_slices, lds, lane, ta, tb, gp, base, nb);
    else
      gram_stream<4, 1, true, VEC4>(X, r, kb, rows, slice, n_slices, lds, lane, ta, tb, gp, base, nb);
  } else {
    if (gp.n == 3)
      gram_stream<4, 3, false, VEC4>(X, r, kb, rows, slice, n_slices, lds, lane, ta, tb, gp, base, nb);
    else if (gp.n == 2)
      gram_stream<4, 2, false, VEC4>(X, r, kb, rows, slice, n_slices, lds, lane, ta, tb, gp, base, nb);
    else
      gram_stream<4, 1, false, VEC4>(X, r, kb, rows, slice, n_slices, lds, lane, ta, tb, gp, base, nb);
  }
}

// One thread per element of a computed block: sums its slice partials (coalesced across
// threads) and writes the element and its mirror image.
__global__ void __launch_bounds__(256)
    k_gram_reduce(const float* __restrict__ partials, int64_t slices, int n_pairs, int r,
                  float* __restrict__ G) {
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= n_pairs * 1024) return;
  const int nb = gram_blocks(r);
  int pair = e >> 10, ba = 0, row_len = nb;
  while (pair >= row_len) {
    pair -= row_len;
    ba++;
    row_len--;
  }
  const int bb = ba + pair;
  const int ia = (e >> 5) & 31, ib = e & 31;
  // strided block sb holds columns 128 (sb / 4) + 4 i + sb % 4
  const int a = 128 * (ba >> 2) + 4 * ia + (ba & 3), b = 128 * (bb >> 2) + 4 * ib + (bb & 3);
  if (a >= r || b >= r) return;
  const int64_t stride = (int64_t)n_pairs * 1024;
  const float* p = partials + e;
  double s = 0.0;
  for (int64_t sl = 0; sl < slices; sl++) s += (double)p[sl * stride];
  G[(int64_t)a * r + b] = (float)s;
  G[(int64_t)b * r + a] = (float)s;
}

// ---------------------------------------------------------------------------
// G = X^T X for r <= 32: all of G is one 32x32 MFMA block, and for X^T X the A operand
// (A[i][k] = X[k][i]) and the B operand (B[k][j] = X[k][j]) of lane (l%32, k = l/32) are the
// same number, so a wave feeds the MFMA straight from one global load per row pair: no LDS
// staging, and the kernel runs at the rate the rows stream in.  A wave owns a contiguous run
// of row pairs; the four waves of a workgroup are summed through LDS into one partial block,
// and the partials are summed in fp64 by k_gram_small_reduce.
// ---------------------------------------------------------------------------
constexpr int GRAM_SMALL_MAX_WGS = 512;

static int64_t gram_small_wgs(int64_t rows) {
  int64_t s = ceil_div(rows, 1024);
  if (s > GRAM_SMALL_MAX_WGS) s = GRAM_SMALL_MAX_WGS;
  if (s < 1) s = 1;
  return s;
}

__global__ void __launch_bounds__(256)
    k_gram_small(const float* __restrict__ X, int64_t rows, int r, float* __restrict__ partials) {
  __shared__ float red[4 * 1024];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int64_t n_rp = (rows + 1) / 2;
  const int64_t n_waves = (int64_t)gridDim.x * 4;
  const int64_t per = (n_rp + n_waves - 1) / n_waves;
  const int64_t gw = (int64_t)blockIdx.x * 4 + wave;
  int64_t p0 = gw * per, p1 = p0 + per;
  if (p0 > n_rp) p0 = n_rp;
  if (p1 > n_rp) p1 = n_rp;
  const bool col_ok = l32 < r;
  const int col = col_ok ? l32 : 0;
  acc16 acc;
  for (int v = 0; v < 16; v++) acc[v] = 0.f;
  int64_t p = p0;
  // whole groups of GRAM_UNR complete row pairs (an odd row count leaves the last pair of X
  // without its second row): loads without a bounds check
  const int64_t p_full = p1 < rows / 2 ? p1 : rows / 2;
  for (; p + GRAM_UNR <= p_full; p += GRAM_UNR) {
    float x[GRAM_UNR];
#pragma unroll
    for (int u = 0; u < GRAM_UNR; u++) x[u] = X[(2 * (p + u) + half) * r + col];
#pragma unroll
    for (int u = 0; u < GRAM_UNR; u++) {
      const float v = col_ok ? x[u] : 0.f;
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(v, v, acc, 0, 0, 0);
    }
  }
  for (; p < p1; p++) {
    const int64_t row = 2 * p + half;
    const bool ok = col_ok && row < rows;
    const float v = ok ? X[(row < rows ? row : rows - 1) * r + col] : 0.f;
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(v, v, acc, 0, 0, 0);
  }
  // D layout of the 32x32 block: reg v of lane l holds row 8*(v/4) + 4*(l/32) + v%4, column l%32.
  for (int v = 0; v < 16; v++) red[wave * 1024 + (8 * (v >> 2) + 4 * half + (v & 3)) * 32 + l32] = acc[v];
  __syncthreads();
  float* out = partials + (int64_t)blockIdx.x * 1024;
  for (int e = threadIdx.x; e < 1024; e += 256)
    out[e] = (red[e] + red[1024 + e]) + (red[2048 + e] + red[3072 + e]);
}

// One workgroup per row of G: 8 groups of 32 threads each sum every 8th partial (four loads in
// flight), then the 8 sums are added in fp64 through LDS.
__global__ void __launch_bounds__(256)
    k_gram_small_reduce(const float* __restrict__ partials, int64_t n_parts, int r,
                        float* __restrict__ G) {
  __shared__ double red[256];
  const int a = blockIdx.x, b = threadIdx.x & 31, g = threadIdx.x >> 5;
  const float* p = partials + a * 32 + b;
  double s = 0.0;
  int64_t q = g;
  for (; q + 24 < n_parts; q += 32) {
    const float x0 = p[q * 1024], x1 = p[(q + 8) * 1024], x2 = p[(q + 16) * 1024],
                x3 = p[(q + 24) * 1024];
    s += ((double)x0 + (double)x1) + ((double)x2 + (double)x3);
  }
  for (; q < n_parts; q += 8) s += (double)p[q * 1024];
  red[threadIdx.x] = s;
  __syncthreads();
  if (g == 0 && b < r) {
    for (int k = 1; k < 8; k++) s += red[k * 32 + b];
    G[a * r + b] = (float)s;
  }
}

int launch_gram(int64_t rows, int r, const float* X, float* G, float* workspace) {
  DN_CHECK(r >= 1 && r <= 1024, "rank %d outside [1, 1024]", r);
  if (r <= 32 && rows >= 1) {
    const int64_t wgs = gram_small_wgs(rows);
    hipLaunchKernelGGL(k_gram_small, dim3((unsigned)wgs), dim3(256), 0, stream(), X, rows, r,
                       workspace);
    hipLaunchKernelGGL(k_gram_small_reduce, dim3((unsigned)r), dim3(256), 0, stream(), workspace, wgs, r, G);
    DN_LAUNCH_CHECK();
    return 0;
  }
  if (gram_uses_tiles(rows, r) && ((uintptr_t)X % 16) == 0)
    return launch_gram_tiles(rows, r, X, G, workspace);
  const int n_pairs = gram_pairs(r);
  const int n_tiles = (r + 127) / 128;
  int64_t slices = gram_slices(rows);
  const bool vec4 = r % 4 == 0 && ((uintptr_t)X % 16) == 0;
  // rows per LDS slot: even, a multiple of 8 where possible, with kb * ld <= GRAM_TILE_FLOATS
  const int ld = 128 * n_tiles;
  int kb = GRAM_TILE_FLOATS / ld;
  kb = kb >= 8 ? kb / 8 * 8 : kb / 2 * 2;
  dim3 grid((unsigned)(n_tiles + n_tiles * (n_tiles - 1)), (unsigned)slices);
  if (vec4)
    hipLaunchKernelGGL((k_gram<true>), grid, dim3(256), 0, stream(), X, rows, r, kb, n_pairs,
                       n_tiles, workspace);
  else
    hipLaunchKernelGGL((k_gram<false>), grid, dim3(256), 0, stream(), X, rows, r, kb, n_pairs,
                       n_tiles, workspace);
  hipLaunchKernelGGL(k_gram_reduce, dim3((unsigned)(n_pairs * 4)), dim3(256), 0, stream(), workspace,
                     slices, n_pairs, r, G);
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
        // element 0 stands in for the ones outside the matrix: unconditional loads, which the
        // compiler can issue together (a branch per load would serialise them)
        const bool ok = cok[i] && row < rows;
        const int64_t idx = ok ? row * (int64_t)r + col : 0;
        pn[i][v] = num[idx];
        px[i][v] = X[idx];
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

// ---------------------------------------------------------------------------
// out = X * num / (X G + eps) for r = 32, 64 or 128: G in registers, X through LDS.
//
// With r <= 128 the B operands of a wave -- the 32 columns of G of its column block, all r rows
// -- fit its registers (r / 2 per lane), so LDS is free for the X tiles: a workgroup streams
// tiles of ROWS rows through two LDS slots, fetched with coalesced 16-byte loads one tile
// ahead, and two workgroups share a CU, one running MFMAs while the other is in its epilogue.
// A wave owns column block cb and two row blocks; lane (i = l%32, half = l/32) reads
// X[row i][8 kg + 4 half .. + 3] of a row block with one 16-byte LDS read (rows padded by 4
// floats: conflict free) and MFMA step s contracts component 8 kg + 4 half + s against the
// matching row of G.  The X factor of the update comes from the same LDS tile.  The rank is a
// compile-time constant and the launch covers whole tiles only (the host hands the last rows to
// k_xg_mu): the epilogue is then straight-line code with one per-lane offset, whose loads, LDS
// reads and stores the compiler batches; code for partial tiles would cost registers that the
// main path needs.
// ---------------------------------------------------------------------------
// Consecutive tiles a workgroup takes at a time: a power of two, 16 where that leaves every
// workgroup several runs, less for short inputs.
static int xg_run(int64_t tiles, int64_t wgs_max) {
  int run = 16;
  while (run > 1 && tiles / run < 4 * wgs_max) run /= 2;
  return run;
}

template <int CB>
struct XgReg {
  static constexpr int WPC = 4 / CB;         // waves per column block
  static constexpr int RB = 2;               // row blocks per wave
  static constexpr int ROWS = 32 * RB * WPC;  // rows of a tile
  static constexpr int R = 32 * CB;           // rank
  static constexpr int LD = R + 4;
  static constexpr int KG = R / 8;
  static constexpr int C4 = R / 4;           // 16-byte columns of a tile row
  static constexpr int RSTEP = 256 / C4;
  static constexpr int NV = ROWS / RSTEP;    // 16-byte pieces per thread and tile
  static constexpr int SLOT = ROWS * LD;
};

template <int CB, bool WITH_D>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
    k_xg_mu_reg(const float* __restrict__ X, const float* __restrict__ G, const float* num,
                float eps, int64_t n_tiles, int run, float* out, float* __restrict__ D_out) {
  using C = XgReg<CB>;
  constexpr int r = C::R;
  extern __shared__ __align__(16) float xl[];  // 2 slots of ROWS x LD
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int cb = wave % CB, rg = wave / CB;
  const int col = 32 * cb + l32;

  float g[C::KG][4];
#pragma unroll
  for (int kg = 0; kg < C::KG; kg++)
#pragma unroll
    for (int s = 0; s < 4; s++) g[kg][s] = G[(8 * kg + 4 * half + s) * r + col];

  const int lc = threadIdx.x % C::C4, lr = threadIdx.x / C::C4;
  float4 R[C::NV];
  auto fetch = [&](int64_t tile) {
    const float* src = X + (tile * C::ROWS + lr) * (int64_t)r + 4 * lc;
#pragma unroll
    for (int q = 0; q < C::NV; q++)
      R[q] = tile < n_tiles ? *reinterpret_cast<const float4*>(src + q * C::RSTEP * r)
                            : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  };
  auto commit = [&](float* slot) {
#pragma unroll
    for (int q = 0; q < C::NV; q++)
      *reinterpret_cast<float4*>(slot + (lr + q * C::RSTEP) * C::LD + 4 * lc) = R[q];
  };

  // A workgroup takes runs of `run` (a power of two) consecutive tiles, the runs dealt
  // round-robin (single tiles dealt round-robin put a workgroup's tiles a fixed power-of-two
  // stride apart, which costs about 15 % of the streaming rate).
  auto after = [&](int64_t t) {
    return ((t + 1) & (run - 1)) != 0 ? t + 1 : t + 1 + ((int64_t)gridDim.x - 1) * run;
  };
  int64_t tile = (int64_t)blockIdx.x * run;
  fetch(tile);
  commit(xl);
  fetch(after(tile));
  __syncthreads();

  // element (b, v) of the accumulators sits 32 b + 8 (v / 4) + v % 4 rows below the lane's
  // first one: a uniform pointer per row plus one per-lane offset
  const int lrow0 = 32 * C::RB * rg + 4 * half;
  const unsigned off0 = (unsigned)(lrow0 * r + col);

  for (int it = 0; tile < n_tiles; it++, tile = after(tile)) {
    const float* slot = xl + (it & 1) * C::SLOT;
    const int64_t t0 = tile * C::ROWS * (int64_t)r;
    const float* tnum = num + t0;
    float* tout = out + t0;
    float* tD = WITH_D ? D_out + t0 : nullptr;
    // numerators in the accumulator layout: requested now, they arrive while the MFMAs run
    float pn[C::RB][16];
#pragma unroll
    for (int b = 0; b < C::RB; b++)
#pragma unroll
      for (int v = 0; v < 16; v++)
        pn[b][v] = (tnum + (32 * b + 8 * (v >> 2) + (v & 3)) * r)[off0];
    acc16 acc[C::RB];
#pragma unroll
    for (int b = 0; b < C::RB; b++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[b][v] = 0.0f;

    const float* arow = slot + (32 * C::RB * rg + l32) * C::LD + 4 * half;
#pragma unroll
    for (int kg = 0; kg < C::KG; kg++) {
      float4 a[C::RB];
#pragma unroll
      for (int b = 0; b < C::RB; b++)
        a[b] = *reinterpret_cast<const float4*>(arow + 32 * b * C::LD + 8 * kg);
#pragma unroll
      for (int b = 0; b < C::RB; b++) {
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[b].x, g[kg][0], acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[b].y, g[kg][1], acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[b].z, g[kg][2], acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[b].w, g[kg][3], acc[b], 0, 0, 0);
      }
    }

#pragma unroll
    for (int b = 0; b < C::RB; b++) {
      float x[16];
#pragma unroll
      for (int v = 0; v < 16; v++)
        x[v] = slot[(lrow0 + 32 * b + 8 * (v >> 2) + (v & 3)) * C::LD + col];
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int below = (32 * b + 8 * (v >> 2) + (v & 3)) * r;
        const float d = acc[b][v];
        const float q = pn[b][v] / (d + eps);
        (tout + below)[off0] = x[v] * q;
        if (WITH_D) (tD + below)[off0] = d;
      }
    }

    // the other slot was last read before the previous barrier: it takes the next tile, whose
    // loads were issued one tile ago; the registers then take the tile after it
    commit(xl + ((it + 1) & 1) * C::SLOT);
    fetch(after(after(tile)));
    __syncthreads();
  }
}

// rows must be a multiple of XgReg<CB>::ROWS
template <int CB>
static int launch_xg_mu_reg(int64_t rows, const float* X, const float* G, const float* num,
                            float eps, float* out, float* D_out) {
  using C = XgReg<CB>;
  const size_t lds = sizeof(float) * 2 * C::SLOT;
  static bool attr_set = false;
  if (!attr_set) {
    DN_HIP(hipFuncSetAttribute((const void*)k_xg_mu_reg<CB, false>,
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    DN_HIP(hipFuncSetAttribute((const void*)k_xg_mu_reg<CB, true>,
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set = true;
  }
  const int64_t tiles = rows / C::ROWS;
  if (tiles == 0) return 0;
  int64_t wgs = (int64_t)n_cus() * 2;
  const int run = xg_run(tiles, wgs);
  if (wgs > ceil_div(tiles, run)) wgs = ceil_div(tiles, run);
  const dim3 grid((unsigned)wgs), block(256);
  if (D_out)
    hipLaunchKernelGGL((k_xg_mu_reg<CB, true>), grid, block, lds, stream(), X, G, num, eps, tiles,
                       run, out, D_out);
  else
    hipLaunchKernelGGL((k_xg_mu_reg<CB, false>), grid, block, lds, stream(), X, G, num, eps, tiles,
                       run, out, D_out);
  DN_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// out = X * num / (X G + eps) for r a multiple of 128 above 128: both operands through LDS.
//
// A workgroup owns a 128 x 128 tile of X G (row tile, column chunk) and walks the r components
// in tiles of 32: the X part [128 rows][32 k] (rows padded to 36 floats: one conflict-free
// 16-byte LDS read gives a lane 4 consecutive components of its row) and the G part
// [32 k][128 columns] of the two LDS slots are fetched with coalesced 16-byte loads one tile
// ahead into registers and committed after the MFMAs of the current tile.  Wave (wm, wn) owns
// 64 rows x 64 columns (2 x 2 blocks of 32 x 32).  Workgroups of one row tile are neighbours in
// the grid, so the chunks after the first find the X tile in L2 / the memory-side cache.  The
// epilogue walks the four blocks with the operands of the next block in flight.
// ---------------------------------------------------------------------------
constexpr int XGT_KB = 32;
constexpr int XGT_XLD = XGT_KB + 4;
constexpr int XGT_XPART = 128 * XGT_XLD;        // floats
constexpr int XGT_SLOT = XGT_XPART + XGT_KB * 128;

template <bool WITH_D>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
    k_xg_mu_tile(const float* __restrict__ X, const float* __restrict__ G, const float* num,
                 float eps, int64_t rows, int r, int n_chunks, float* out,
                 float* __restrict__ D_out) {
  extern __shared__ __align__(16) float tl[];  // 2 slots
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;
  // Workgroups are dealt to the 8 XCDs round-robin by their number; the column chunks of one row
  // tile are numbered 8 apart so that they share an XCD, i.e. an L2, and X comes in once.
  const int64_t grp = blockIdx.x / (8 * n_chunks);
  const int rem = (int)(blockIdx.x % (8 * n_chunks));
  const int64_t tile = grp * 8 + rem % 8;
  if (tile * 128 >= rows) return;
  const int n0 = (rem / 8) * 128;
  const int64_t row0 = tile * 128;
  const int n_kt = r / XGT_KB;

  // loader roles: X: 16-byte column xc of rows xr + 32 q; G: 16-byte column gc of k gk + 8 q
  const int xc = threadIdx.x & 7, xr = threadIdx.x >> 3;
  const int gc = threadIdx.x & 31, gk = threadIdx.x >> 5;
  float4 RX[4], RG[4];
  auto fetch = [&](int kt) {
    const int k0 = kt * XGT_KB;
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const int64_t row = row0 + xr + 32 * q;
      RX[q] = (kt < n_kt && row < rows)
                  ? *reinterpret_cast<const float4*>(X + row * (int64_t)r + k0 + 4 * xc)
                  : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      RG[q] = kt < n_kt ? *reinterpret_cast<const float4*>(G + (int64_t)(k0 + gk + 8 * q) * r + n0 + 4 * gc)
                        : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
  };
  auto commit = [&](float* slot) {
#pragma unroll
    for (int q = 0; q < 4; q++) {
      *reinterpret_cast<float4*>(slot + (xr + 32 * q) * XGT_XLD + 4 * xc) = RX[q];
      *reinterpret_cast<float4*>(slot + XGT_XPART + (gk + 8 * q) * 128 + 4 * gc) = RG[q];
    }
  };

  acc16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

  // element (i, j, v): row 64 wm + 32 i + 8 (v / 4) + 4 half + v % 4, column n0 + 64 wn + 32 j + l32
  const int64_t t0 = (row0 + 64 * wm + 4 * half) * (int64_t)r + n0 + 64 * wn;
  const float* tnum = num + t0;
  const float* tx = X + t0;
  float* tout = out + t0;
  float* tD = WITH_D ? D_out + t0 : nullptr;
  const int64_t rows_left = rows - (row0 + 64 * wm + 4 * half);  // rows at and below the lane's first
  float pn[2][16], px[2][16];
  auto request = [&](int blk, float (&n_)[16], float (&x_)[16]) {
    const int i = blk >> 1, j = blk & 1;
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int below = 32 * i + 8 * (v >> 2) + (v & 3);
      // rows past the end are clamped to the lane's first row (never stored)
      const int64_t off = (below < rows_left ? below : 0) * (int64_t)r + 32 * j + l32;
      n_[v] = tnum[off];
      x_[v] = tx[off];
    }
  };
  // the epilogue operands of the first two blocks are requested before the contraction starts
  if (rows_left > 0) {
    request(0, pn[0], px[0]);
    request(1, pn[1], px[1]);
  }
  fetch(0);
  commit(tl);
  fetch(1);
  __syncthreads();
  for (int kt = 0; kt < n_kt; kt++) {
    const float* slot = tl + (kt & 1) * XGT_SLOT;
    const float* pa = slot + (64 * wm + l32) * XGT_XLD + 4 * half;
    const float* pb = slot + XGT_XPART + 4 * half * 128 + 64 * wn + l32;
#pragma unroll
    for (int kg = 0; kg < XGT_KB / 8; kg++) {
      float4 a[2];
      float b[2][4];
#pragma unroll
      for (int i = 0; i < 2; i++)
        a[i] = *reinterpret_cast<const float4*>(pa + 32 * i * XGT_XLD + 8 * kg);
#pragma unroll
      for (int j = 0; j < 2; j++)
#pragma unroll
        for (int s2 = 0; s2 < 4; s2++) b[j][s2] = pb[(8 * kg + s2) * 128 + 32 * j];
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i].x, b[j][0], acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i].y, b[j][1], acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i].z, b[j][2], acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i].w, b[j][3], acc[i][j], 0, 0, 0);
        }
    }
    if (kt + 1 < n_kt) {
      // the other slot was last read before the previous barrier
      commit(tl + ((kt + 1) & 1) * XGT_SLOT);
      fetch(kt + 2);
      __syncthreads();
    }
  }

  auto finish = [&](int blk, const float (&n_)[16], const float (&x_)[16]) {
    const int i = blk >> 1, j = blk & 1;
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int below = 32 * i + 8 * (v >> 2) + (v & 3);
      if (below < rows_left) {
        const int64_t off = below * (int64_t)r + 32 * j + l32;
        const float d = acc[i][j][v];
        const float q = n_[v] / (d + eps);
        tout[off] = x_[v] * q;
        if (WITH_D) tD[off] = d;
      }
    }
  };
  if (rows_left > 0) {
    finish(0, pn[0], px[0]);
    request(2, pn[0], px[0]);
    finish(1, pn[1], px[1]);
    request(3, pn[1], px[1]);
    finish(2, pn[0], px[0]);
    finish(3, pn[1], px[1]);
  }
}

static int launch_xg_mu_tile(int64_t rows, int r, const float* X, const float* G, const float* num,
                             float eps, float* out, float* D_out) {
  const size_t lds = sizeof(float) * 2 * XGT_SLOT;
  static bool attr_set = false;
  if (!attr_set) {
    DN_HIP(hipFuncSetAttribute((const void*)k_xg_mu_tile<false>,
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    DN_HIP(hipFuncSetAttribute((const void*)k_xg_mu_tile<true>,
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set = true;
  }
  const int n_chunks = r / 128;
  const int64_t wgs = ceil_div(ceil_div(rows, 128), 8) * 8 * n_chunks;
  DN_CHECK(wgs < ((int64_t)1 << 24), "xg_mu: too many tiles for one launch");
  const dim3 grid((unsigned)wgs), block(256);
  if (D_out)
    hipLaunchKernelGGL((k_xg_mu_tile<true>), grid, block, lds, stream(), X, G, num, eps, rows, r,
                       n_chunks, out, D_out);
  else
    hipLaunchKernelGGL((k_xg_mu_tile<false>), grid, block, lds, stream(), X, G, num, eps, rows, r,
                       n_chunks, out, D_out);
  DN_LAUNCH_CHECK();
  return 0;
}

// The same update on the bf16 matrix cores with split operands (abt_b16.hpp): X has the
// contraction index fast as it is, G is passed transposed (Gt[n][k] = G[k][n]).  Whole row tiles
// of 128 only; the caller hands the last rows to k_xg_mu_tile.
template <bool WITH_D>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
    k_xg_mu_tile_b16(const float* __restrict__ X, const float* __restrict__ Gt, const float* num,
                     float eps, int64_t n_row_tiles, int r, int n_chunks, float* out,
                     float* __restrict__ D_out) {
  extern __shared__ __align__(16) unsigned char ab[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;
  // Workgroups are dealt to the 8 XCDs round-robin by their number; the column chunks of one row
  // tile are numbered 8 apart so that they share an XCD, i.e. an L2, and X comes in once.
  const int64_t grp = blockIdx.x / (8 * n_chunks);
  const int rem = (int)(blockIdx.x % (8 * n_chunks));
  const int64_t tile = grp * 8 + rem % 8;
  if (tile >= n_row_tiles) return;
  const int n0 = (rem / 8) * 128;
  const int64_t row0 = tile * 128;

  // element (i, j, v): row 64 wm + 32 i + 8 (v / 4) + 4 half + v % 4, column n0 + 64 wn + 32 j + l32
  const int64_t t0 = (row0 + 64 * wm + 4 * half) * (int64_t)r + n0 + 64 * wn;
  const float* tnum = num + t0;
  const float* tx = X + t0;
  float* tout = out + t0;
  float* tD = WITH_D ? D_out + t0 : nullptr;
  float pn[2][16], px[2][16];
  auto request = [&](int blk, float (&n_)[16], float (&x_)[16]) {
    const int i = blk >> 1, j = blk & 1;
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int64_t off = (32 * i + 8 * (v >> 2) + (v & 3)) * (int64_t)r + 32 * j + l32;
      n_[v] = tnum[off];
      x_[v] = tx[off];
    }
  };
  acc16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;
  abt_mainloop<false, false, ABT_STAGES_XG>(X + row0 * r, r, Gt + (int64_t)n0 * r, r, 0, 1, r / ABT_KB, ab, acc);

  auto finish = [&](int blk, const float (&n_)[16], const float (&x_)[16]) {
    const int i = blk >> 1, j = blk & 1;
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int64_t off = (32 * i + 8 * (v >> 2) + (v & 3)) * (int64_t)r + 32 * j + l32;
      const float d = acc[i][j][v];
      const float q = mu_quotient(n_[v], d + eps);
      tout[off] = x_[v] * q;
      if (WITH_D) tD[off] = d;
    }
  };
  request(0, pn[0], px[0]);
  request(1, pn[1], px[1]);
  finish(0, pn[0], px[0]);
  request(2, pn[0], px[0]);
  finish(1, pn[1], px[1]);
  request(3, pn[1], px[1]);
  finish(2, pn[0], px[0]);
  finish(3, pn[1], px[1]);
}

// The same with three workgroups per CU (abt_mainloop64).
template <bool WITH_D>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3)))
    k_xg_mu_tile_b16_w3(const float* __restrict__ X, const float* __restrict__ Gt, const float* num,
                     float eps, int64_t n_row_tiles, int r, int n_chunks, float* out,
                     float* __restrict__ D_out) {
  extern __shared__ __align__(16) unsigned char ab[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;
  // Workgroups are dealt to the 8 XCDs round-robin by their number; the column chunks of one row
  // tile are numbered 8 apart so that they share an XCD, i.e. an L2, and X comes in once.
  const int64_t grp = blockIdx.x / (8 * n_chunks);
  const int rem = (int)(blockIdx.x % (8 * n_chunks));
  const int64_t tile = grp * 8 + rem % 8;
  if (tile >= n_row_tiles) return;
  const int n0 = (rem / 8) * 128;
  const int64_t row0 = tile * 128;

  // element (i, j, v): row 64 wm + 32 i + 8 (v / 4) + 4 half + v % 4, column n0 + 64 wn + 32 j + l32
  const int64_t t0 = (row0 + 64 * wm + 4 * half) * (int64_t)r + n0 + 64 * wn;
  const float* tnum = num + t0;
  const float* tx = X + t0;
  float* tout = out + t0;
  float* tD = WITH_D ? D_out + t0 : nullptr;
  float pn[2][16], px[2][16];
  auto request = [&](int blk, float (&n_)[16], float (&x_)[16]) {
    const int i = blk >> 1, j = blk & 1;
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int64_t off = (32 * i + 8 * (v >> 2) + (v & 3)) * (int64_t)r + 32 * j + l32;
      n_[v] = tnum[off];
      x_[v] = tx[off];
    }
  };
  acc16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;
  abt_mainloop64(X + row0 * r, r, Gt + (int64_t)n0 * r, r, r / ABT_KB, ab, acc);

  auto finish = [&](int blk, const float (&n_)[16], const float (&x_)[16]) {
    const int i = blk >> 1, j = blk & 1;
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int64_t off = (32 * i + 8 * (v >> 2) + (v & 3)) * (int64_t)r + 32 * j + l32;
      const float d = acc[i][j][v];
      const float q = mu_quotient(n_[v], d + eps);
      tout[off] = x_[v] * q;
      if (WITH_D) tD[off] = d;
    }
  };
  request(0, pn[0], px[0]);
  request(1, pn[1], px[1]);
  finish(0, pn[0], px[0]);
  request(2, pn[0], px[0]);
  finish(1, pn[1], px[1]);
  request(3, pn[1], px[1]);
  finish(2, pn[0], px[0]);
  finish(3, pn[1], px[1]);
}

// G transposed for the split-operand update: a buffer that grows to the largest rank seen and
// lives until the process ends (one host thread drives the library).
static float* g_gt = nullptr;
static int64_t g_gt_floats = 0;
// The G (and rank) whose transpose g_gt holds for a run of calls, between xg_mu_hold_g and
// xg_mu_release_g: the column tiles of one H update all multiply by the same G.
static const float* g_gt_of = nullptr;
static int g_gt_rank = 0;

static int xg_mu_transpose_g(const float* G, int r) {
  if (g_gt_floats < (int64_t)r * r) {
    DN_HIP(hipStreamSynchronize(stream()));
    dfree(g_gt);
    g_gt = nullptr;
    g_gt_floats = 0;
    g_gt_of = nullptr;
    DN_TRY(dmalloc(&g_gt, (int64_t)r * r));
    g_gt_floats = (int64_t)r * r;
  }
  return launch_transpose(r, r, G, g_gt);
}

int xg_mu_hold_g(const float* G, int r) {
  g_gt_of = nullptr;
  if (!(use_split_bf16() && r > 128 && r % 128 == 0 && ((uintptr_t)G % 16) == 0)) return 0;  // (no transposed G on that path)
  DN_TRY(xg_mu_transpose_g(G, r));
  g_gt_of = G;
  g_gt_rank = r;
  return 0;
}
void xg_mu_release_g() { g_gt_of = nullptr; }

static int launch_xg_mu_tile_b16(int64_t rows, int r, const float* X, const float* G, const float* num,
                                 float eps, float* out, float* D_out) {
  static bool attr_set = false;
  if (!attr_set) {
    DN_HIP(hipFuncSetAttribute((const void*)k_xg_mu_tile_b16<false>,
                               hipFuncAttributeMaxDynamicSharedMemorySize, ABT_LDS));
    DN_HIP(hipFuncSetAttribute((const void*)k_xg_mu_tile_b16<true>,
                               hipFuncAttributeMaxDynamicSharedMemorySize, ABT_LDS));
    attr_set = true;
  }
  if (!(g_gt_of == G && g_gt_rank == r)) DN_TRY(xg_mu_transpose_g(G, r));
  const int n_chunks = r / 128;
  const int64_t tiles = rows / 128;
  // The last rows (fewer than 128, through the fp32 kernel: two workgroups that take a third of
  // the time of a few hundred row tiles) run on the second stream beside the whole tiles.
  const int64_t head = tiles * 128;
  bool beside = false;
  if (head < rows && tiles > 0 && tiles <= 4096 && !side_stream_routed() && !side_stream_pending()) {
    DN_TRY(side_stream_begin());
    const int64_t off = head * r;
    int st = launch_xg_mu_tile(rows - head, r, X + off, G, num + off, eps, out + off, D_out ? D_out + off : nullptr);
    DN_TRY(side_stream_end());
    DN_TRY(st);
    beside = true;
  }
  if (tiles > 0) {
    const int64_t wgs = ceil_div(tiles, 8) * 8 * n_chunks;
    DN_CHECK(wgs < ((int64_t)1 << 24), "xg_mu: too many tiles for one launch");
    const dim3 grid((unsigned)wgs), block(256);
    // three workgroups per CU on planes without padding, where the launch fills them several
    // times over (a workgroup of three takes longer than one of two: few row tiles, as in the
    // fixed-H learner's W update, are done sooner two per CU)
    const bool three = tuning().xg_wgs >= 4.0 || (tuning().xg_wgs >= 3.0 && wgs >= 8 * 3 * (int64_t)n_cus());
    if (three && D_out)
      hipLaunchKernelGGL((k_xg_mu_tile_b16_w3<true>), grid, block, ABT_LDS64, stream(), X, g_gt, num, eps,
                         tiles, r, n_chunks, out, D_out);
    else if (three)
      hipLaunchKernelGGL((k_xg_mu_tile_b16_w3<false>), grid, block, ABT_LDS64, stream(), X, g_gt, num, eps,
                         tiles, r, n_chunks, out, D_out);
    else if (D_out)
      hipLaunchKernelGGL((k_xg_mu_tile_b16<true>), grid, block, ABT_LDS, stream(), X, g_gt, num, eps,
                         tiles, r, n_chunks, out, D_out);
    else
      hipLaunchKernelGGL((k_xg_mu_tile_b16<false>), grid, block, ABT_LDS, stream(), X, g_gt, num, eps,
                         tiles, r, n_chunks, out, D_out);
    DN_LAUNCH_CHECK();
  }
  if (beside) return side_stream_join();
  if (head < rows) {
    const int64_t off = head * r;
    DN_TRY(launch_xg_mu_tile(rows - head, r, X + off, G, num + off, eps, out + off,
                             D_out ? D_out + off : nullptr));
  }
  return 0;
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

// ---------------------------------------------------------------------------
// The same update for r = 128 that also accumulates the Gram matrix of its OUTPUT, so that the
// next A-side update does not have to read the new factor again: out = X * num / (X G + eps),
// Gout += out^T out.
//
// After the epilogue a lane holds out[row(v, half)][32 cb + l32] in register v, where rows
// row(v, 0) and row(v, 1) differ by 4: exactly the operand shape of v_mfma_f32_32x32x2f32 with
// the row pair as contraction index.  The diagonal block (cb, cb) of the Gram matrix therefore
// takes both operands from the registers; for the other blocks of the wave (cb, cb + 1 mod 4 and,
// for waves 0 and 1, cb + 2) the second operand is read from the LDS tile, where every wave has
// replaced X by its part of out (after a barrier: the other waves read X until their MFMAs and
// epilogue are done).  10 distinct blocks in all; the reduction kernel mirrors
// them.  The Gram accumulators are flushed every XGG_FLUSH tiles so that no fp32 sum runs over
// more than 32,768 rows; the partial sums are added in fp64 in a fixed order.
// ---------------------------------------------------------------------------
constexpr int XGG_FLUSH = 512;
constexpr int XGG_BLOCKS = 12;  // 4 waves x 3 block slots (the third is used by waves 0 and 1)

__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
    k_xg_mu_gram(const float* __restrict__ X, const float* __restrict__ G, const float* num,
                 float eps, int64_t n_tiles, int n_flush, float* out, float* __restrict__ gpart) {
  using C = XgReg<4>;
  constexpr int r = C::R;
  extern __shared__ __align__(16) float xl[];  // 2 slots of ROWS x LD
  const int cb = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int col = 32 * cb + l32;

  float g[C::KG][4];
#pragma unroll
  for (int kg = 0; kg < C::KG; kg++)
#pragma unroll
    for (int s = 0; s < 4; s++) g[kg][s] = G[(8 * kg + 4 * half + s) * r + col];

  const int lc = threadIdx.x % C::C4, lr = threadIdx.x / C::C4;
  float4 R[C::NV];
  auto fetch = [&](int64_t tile) {
    const float* src = X + (tile * C::ROWS + lr) * (int64_t)r + 4 * lc;
#pragma unroll
    for (int q = 0; q < C::NV; q++)
      R[q] = tile < n_tiles ? *reinterpret_cast<const float4*>(src + q * C::RSTEP * r)
                            : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  };
  auto commit = [&](float* slot) {
#pragma unroll
    for (int q = 0; q < C::NV; q++)
      *reinterpret_cast<float4*>(slot + (lr + q * C::RSTEP) * C::LD + 4 * lc) = R[q];
  };

  acc16 ga[3];
  auto ga_clear = [&]() {
#pragma unroll
    for (int k = 0; k < 3; k++)
#pragma unroll
      for (int v = 0; v < 16; v++) ga[k][v] = 0.0f;
  };
  auto ga_flush = [&](int chunk) {
    float* dst = gpart + (((int64_t)blockIdx.x * n_flush + chunk) * XGG_BLOCKS + 3 * cb) * 1024 + lane;
#pragma unroll
    for (int k = 0; k < 3; k++)
#pragma unroll
      for (int v = 0; v < 16; v++) dst[k * 1024 + v * 64] = ga[k][v];
  };
  ga_clear();

  int64_t tile = blockIdx.x;
  fetch(tile);
  commit(xl);
  fetch(tile + gridDim.x);
  __syncthreads();

  const int lrow0 = 4 * half;
  const unsigned off0 = (unsigned)(lrow0 * r + col);
  const int cb1 = (cb + 1) & 3, cb2 = (cb + 2) & 3;
  int it = 0;
  for (; tile < n_tiles; it++, tile += gridDim.x) {
    float* slot = xl + (it & 1) * C::SLOT;
    const int64_t t0 = tile * C::ROWS * (int64_t)r;
    const float* tnum = num + t0;
    float* tout = out + t0;
    float pn[C::RB][16];
#pragma unroll
    for (int b = 0; b < C::RB; b++)
#pragma unroll
      for (int v = 0; v < 16; v++)
        pn[b][v] = (tnum + (32 * b + 8 * (v >> 2) + (v & 3)) * r)[off0];
    acc16 acc[C::RB];
#pragma unroll
    for (int b = 0; b < C::RB; b++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[b][v] = 0.0f;

    const float* arow = slot + l32 * C::LD + 4 * half;
#pragma unroll
    for (int kg = 0; kg < C::KG; kg++) {
      float4 a[C::RB];
#pragma unroll
      for (int b = 0; b < C::RB; b++)
        a[b] = *reinterpret_cast<const float4*>(arow + 32 * b * C::LD + 8 * kg);
#pragma unroll
      for (int b = 0; b < C::RB; b++) {
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[b].x, g[kg][0], acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[b].y, g[kg][1], acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[b].z, g[kg][2], acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[b].w, g[kg][3], acc[b], 0, 0, 0);
      }
    }

    // the next tile goes to the other slot now (it was last read before the previous barrier),
    // which frees its registers for the rest of the iteration
    commit(xl + ((it + 1) & 1) * C::SLOT);

    // epilogue: the result replaces the numerator registers
#pragma unroll
    for (int b = 0; b < C::RB; b++) {
      float x[16];
#pragma unroll
      for (int v = 0; v < 16; v++)
        x[v] = slot[(lrow0 + 32 * b + 8 * (v >> 2) + (v & 3)) * C::LD + col];
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int below = 32 * b + 8 * (v >> 2) + (v & 3);
        const float q = pn[b][v] / (acc[b][v] + eps);
        const float o = x[v] * q;
        pn[b][v] = o;
        (tout + below * r)[off0] = o;
      }
    }
    __syncthreads();  // every wave is done with the X values of this slot
#pragma unroll
    for (int b = 0; b < C::RB; b++)
#pragma unroll
      for (int v = 0; v < 16; v++)
        slot[(lrow0 + 32 * b + 8 * (v >> 2) + (v & 3)) * C::LD + col] = pn[b][v];
    __syncthreads();

    // Gram blocks of the new tile; the block pairs two apart, (0, 2) and (1, 3), are taken by
    // waves 0 and 1 on even iterations and, transposed, by waves 2 and 3 on odd ones, so that
    // all four SIMDs carry the same number of MFMAs
    const bool third = (cb < 2) == ((it & 1) == 0);
#pragma unroll
    for (int b = 0; b < C::RB; b++) {
      float y1[16], y2[16];
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int lrow = lrow0 + 32 * b + 8 * (v >> 2) + (v & 3);
        y1[v] = slot[lrow * C::LD + 32 * cb1 + l32];
        y2[v] = slot[lrow * C::LD + 32 * cb2 + l32];
      }
#pragma unroll
      for (int v = 0; v < 16; v++) {
        ga[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(pn[b][v], pn[b][v], ga[0], 0, 0, 0);
        ga[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(pn[b][v], y1[v], ga[1], 0, 0, 0);
        if (third) ga[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(pn[b][v], y2[v], ga[2], 0, 0, 0);
      }
    }
    if ((it + 1) % XGG_FLUSH == 0) {
      ga_flush(it / XGG_FLUSH);
      ga_clear();
    }

    fetch(tile + 2 * (int64_t)gridDim.x);
    __syncthreads();
  }
  // the chunk in progress, then zeros for the chunks this workgroup never reached
  int chunk = it / XGG_FLUSH;
  if (it % XGG_FLUSH != 0 || it == 0) ga_flush(chunk++);
  ga_clear();
  for (; chunk < n_flush; chunk++) ga_flush(chunk);
}

// Gout[a][b] = sum of the partial blocks (fp64, fixed order), both triangles.  One thread per
// element of the upper block triangle.  Block slot (w, k) holds the block (w, w + k mod 4);
// element (i, j) of a block sits at register v = 4 (i / 8) + i % 4 of lane j + 32 ((i / 4) % 2).
__global__ void __launch_bounds__(256)
    k_xg_gram_reduce(const float* __restrict__ gpart, int64_t n_parts, float* __restrict__ Gout) {
  // 32 elements per workgroup, 8 threads per element: thread q sums the parts q, q + 8, ...,
  // the eight sums are added in order
  __shared__ double red[8][32];
  const int q = threadIdx.x >> 5;
  const int e = blockIdx.x * 32 + (threadIdx.x & 31);
  const int a = e >> 7, b = e & 127;
  const int ca = a >> 5, cbk = b >> 5, i = a & 31, j = b & 31;
  auto at = [](int w, int k, int ii, int jj) {
    return (3 * w + k) * 1024 + (4 * (ii >> 3) + (ii & 3)) * 64 + jj + 32 * ((ii >> 2) & 1);
  };
  double s = 0.0;
  // of a diagonal block only the upper triangle: the split-operand kernel's (i, j) and (j, i)
  // sums differ in their last bits, and Gout must be exactly symmetric
  const bool mine = ca < cbk || (ca == cbk && i <= j);
  if (mine) {
    int src0, src1 = -1;
    switch (cbk - ca) {
      case 0: src0 = at(ca, 0, i, j); break;
      case 1: src0 = at(ca, 1, i, j); break;
      case 2: src0 = at(ca, 2, i, j); src1 = at(cbk, 2, j, i); break;
      default: src0 = at(3, 1, j, i); break;  // (0, 3) is held as (3, 0)
    }
#pragma unroll 8
    for (int64_t p = q; p < n_parts; p += 8) s += (double)gpart[p * (XGG_BLOCKS * 1024) + src0];
    if (src1 >= 0) {
#pragma unroll 8
      for (int64_t p = q; p < n_parts; p += 8) s += (double)gpart[p * (XGG_BLOCKS * 1024) + src1];
    }
  }
  red[q][threadIdx.x & 31] = s;
  __syncthreads();
  if (q == 0 && mine) {
    double t = 0.0;
    for (int u = 0; u < 8; u++) t += red[u][threadIdx.x];
    Gout[a * 128 + b] = (float)t;
    Gout[b * 128 + a] = (float)t;
  }
}

// ---------------------------------------------------------------------------
// The fused update on the bf16 matrix cores, at fp32 accuracy.
//
// Every fp32 number is the exact sum of three bf16 numbers, x = h + m + l (each the round-to-
// nearest bf16 of what the ones before leave; 3 x 8 significant bits cover the 24 of fp32).  A
// product of two such numbers is then the sum of nine bf16 products, each exact in fp32; the
// six largest -- hh, hm, mh, hl, lh, mm -- carry everything down to 2^-24 of the result, which
// is the rounding error of an fp32 multiply.  v_mfma_f32_32x32x16_bf16 contracts 16 components
// in half the time v_mfma_f32_32x32x2f32 takes for 2, so six of them per 16 components are 2.7
// times faster than the fp32 matrix cores, with fp32 accumulation either way, and the kernel
// moves from the matrix-core bound to the HBM bound.
//
// Tiles of 32 rows.  X is split once per element on its way into LDS (three bf16 planes
// [row][k], rows padded to 272 bytes; the next tile is fetched into registers after the MFMAs
// of the update and stored after those of the Gram part, when no wave reads the planes any
// more), G is split once per workgroup into registers (lane (j, half) holds the 8
// components 16 st + 8 half .. + 7 of column j for each of the 8 steps: 32 registers a part).
// An A operand is one 16-byte LDS read; an fp32 copy of the tile beside the
// planes gives the epilogue its X factor.  The hardware contracts slot s of lane half `half` of A
// with the same slot of B, so only the agreement of the two sides matters, not the order of
// the 16 components inside an instruction.
//
// Gram part: the result tile is split again; a lane's registers hold, per column, rows
// 8 q + 4 half + t -- taken as contraction slots (MFMA u = 0, 1: q = 2u, 2u + 1; t = 0..3) they
// are the A operand of out^T out directly, and the B operand of the diagonal block.  For the
// other blocks the parts go to LDS transposed ([column][row], 72 bytes a column), where the
// four rows of a (q, half) group are 8 contiguous bytes: a B operand is two 8-byte reads.
// Block ownership, the flush of the accumulators and the partial sums are those of
// k_xg_mu_gram, with 32-row tiles.
// ---------------------------------------------------------------------------
constexpr int XB_ROWS = 32;
constexpr int XB_LDX = 272;                  // bytes per row of an X plane
constexpr int XB_PLANE = XB_ROWS * XB_LDX;
constexpr int XB_SLOT = 3 * XB_PLANE;
constexpr int XB_LDO = 72;                   // bytes per column of an out^T plane
constexpr int XB_OPLANE = 128 * XB_LDO;
constexpr int XB_LDR = 132;                  // floats per row of the fp32 copy of the X tile
constexpr int XB_RAW = XB_ROWS * XB_LDR * 4;
constexpr int XB_LDS = XB_SLOT + 3 * XB_OPLANE + XB_RAW;
constexpr int XB_FLUSH = 1024;               // tiles between flushes: 32,768 rows


__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
    k_xg_mu_gram_b16(const float* __restrict__ X, const float* __restrict__ G, const float* num,
                     float eps, int64_t n_tiles, int run, int n_flush, float* out,
                     float* __restrict__ gpart) {
  constexpr int r = 128;
  extern __shared__ __align__(16) unsigned char xb[];
  unsigned char* const oplanes = xb + XB_SLOT;
  float* const xraw = reinterpret_cast<float*>(xb + XB_SLOT + 3 * XB_OPLANE);
  const int cb = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int col = 32 * cb + l32;

  bf16x8 gh[8], gm[8], gl[8];
#pragma unroll
  for (int st = 0; st < 8; st++) {
    f32x4 g0, g1;
#pragma unroll
    for (int s = 0; s < 4; s++) {
      g0[s] = G[(16 * st + 8 * half + s) * r + col];
      g1[s] = G[(16 * st + 8 * half + 4 + s) * r + col];
    }
    bf16x4 h0, m0, l0, h1, m1, l1;
    split3(g0, h0, m0, l0);
    split3(g1, h1, m1, l1);
    gh[st] = cat8(h0, h1);
    gm[st] = cat8(m0, m1);
    gl[st] = cat8(l0, l1);
  }

  // a thread fetches 16 bytes of each of 4 rows (8 rows apart): whole rows per wave instruction
  const int lc = threadIdx.x & 31, lr = threadIdx.x >> 5;
  f32x4 R[4];
  auto fetch = [&](int64_t tile) {
    // past the last tile the loads are redirected to it (and what they bring is never used)
    const float* src = X + ((tile < n_tiles ? tile : n_tiles - 1) * XB_ROWS + lr) * (int64_t)r + 4 * lc;
#pragma unroll
    for (int q = 0; q < 4; q++) R[q] = *reinterpret_cast<const f32x4*>(src + q * 8 * r);
  };
  auto commit = [&](unsigned char* slot) {
#pragma unroll
    for (int q = 0; q < 4; q++) {
      bf16x4 h, m, l;
      split3(R[q], h, m, l);
      unsigned char* dst = slot + (lr + 8 * q) * XB_LDX + 8 * lc;
      *reinterpret_cast<bf16x4*>(dst) = h;
      *reinterpret_cast<bf16x4*>(dst + XB_PLANE) = m;
      *reinterpret_cast<bf16x4*>(dst + 2 * XB_PLANE) = l;
      *reinterpret_cast<f32x4*>(xraw + (lr + 8 * q) * XB_LDR + 4 * lc) = R[q];
    }
  };

  acc16 ga[3];
  auto ga_clear = [&]() {
#pragma unroll
    for (int k = 0; k < 3; k++)
#pragma unroll
      for (int v = 0; v < 16; v++) ga[k][v] = 0.0f;
  };
  auto ga_flush = [&](int chunk) {
    float* dst = gpart + (((int64_t)blockIdx.x * n_flush + chunk) * XGG_BLOCKS + 3 * cb) * 1024 + lane;
#pragma unroll
    for (int k = 0; k < 3; k++)
#pragma unroll
      for (int v = 0; v < 16; v++) dst[k * 1024 + v * 64] = ga[k][v];
  };
  ga_clear();

  // A workgroup takes runs of `run` (a power of two) consecutive tiles, the runs dealt
  // round-robin: with single tiles dealt round-robin, the tiles of a workgroup lie a fixed
  // power-of-two stride apart, and the three streams then reach 4.4 TB/s where runs reach 5.2.
  auto after = [&](int64_t t) {
    return ((t + 1) & (run - 1)) != 0 ? t + 1 : t + 1 + ((int64_t)gridDim.x - 1) * run;
  };
  int64_t tile = (int64_t)blockIdx.x * run;
  fetch(tile);
  commit(xb);
  const unsigned off0 = (unsigned)(4 * half * r + col);
  // numerators of a tile in the accumulator layout; past the last tile the loads are
  // redirected to it (and their values never used)
  float pn[16], pnn[16];
  auto numerators = [&](int64_t t, float (&dst)[16]) {
    const float* tnum = num + (t < n_tiles ? t : n_tiles - 1) * XB_ROWS * (int64_t)r;
#pragma unroll
    for (int v = 0; v < 16; v++) dst[v] = (tnum + (8 * (v >> 2) + (v & 3)) * r)[off0];
  };
  numerators(tile, pn);
  __syncthreads();

  const int cb1 = (cb + 1) & 3, cb2 = (cb + 2) & 3;
  int it = 0;
  for (; tile < n_tiles; it++, tile = after(tile)) {
    const unsigned char* slot = xb;
    float* tout = out + tile * XB_ROWS * (int64_t)r;
    // the next tile and its numerators travel during this iteration
    fetch(after(tile));

    acc16 a0;
#pragma unroll
    for (int v = 0; v < 16; v++) a0[v] = 0.0f;
    const unsigned char* arow = slot + l32 * XB_LDX + 16 * half;
#pragma unroll
    for (int st = 0; st < 8; st++) {
      const bf16x8 xh = *reinterpret_cast<const bf16x8*>(arow + 32 * st);
      const bf16x8 xm = *reinterpret_cast<const bf16x8*>(arow + 32 * st + XB_PLANE);
      const bf16x8 xl = *reinterpret_cast<const bf16x8*>(arow + 32 * st + 2 * XB_PLANE);
      a0 = DN_MFMA_B16(xh, gh[st], a0);
      a0 = DN_MFMA_B16(xh, gm[st], a0);
      a0 = DN_MFMA_B16(xm, gh[st], a0);
      a0 = DN_MFMA_B16(xh, gl[st], a0);
      a0 = DN_MFMA_B16(xl, gh[st], a0);
      a0 = DN_MFMA_B16(xm, gm[st], a0);
    }
    numerators(after(tile), pnn);

    // epilogue: the result replaces the numerators
    {
      float x[16];
#pragma unroll
      for (int v = 0; v < 16; v++) x[v] = xraw[(8 * (v >> 2) + 4 * half + (v & 3)) * XB_LDR + col];
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const float o = x[v] * mu_quotient(pn[v], a0[v] + eps);
        pn[v] = o;
        (tout + (8 * (v >> 2) + (v & 3)) * r)[off0] = o;
      }
    }
    // parts of the result: registers for the A side, LDS (transposed) for the other waves.
    // The planes were last read before the barrier that ended the previous iteration.
    bf16x4 oh[4], om[4], ol[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const f32x4 o = {pn[4 * q], pn[4 * q + 1], pn[4 * q + 2], pn[4 * q + 3]};
      split3(o, oh[q], om[q], ol[q]);
      unsigned char* dst = oplanes + col * XB_LDO + 2 * (8 * q + 4 * half);
      *reinterpret_cast<bf16x4*>(dst) = oh[q];
      *reinterpret_cast<bf16x4*>(dst + XB_OPLANE) = om[q];
      *reinterpret_cast<bf16x4*>(dst + 2 * XB_OPLANE) = ol[q];
    }
    __syncthreads();

    // Gram blocks of the new tile; the block pairs two apart, (0, 2) and (1, 3), are taken by
    // waves 0 and 1 on even iterations and, transposed, by waves 2 and 3 on odd ones
    const bool third = (cb < 2) == ((it & 1) == 0);
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const bf16x8 ah = cat8(oh[2 * u], oh[2 * u + 1]);
      const bf16x8 am = cat8(om[2 * u], om[2 * u + 1]);
      const bf16x8 al = cat8(ol[2 * u], ol[2 * u + 1]);
      auto side = [&](int cbb, int part) {
        const unsigned char* p =
            oplanes + part * XB_OPLANE + (32 * cbb + l32) * XB_LDO + 2 * (16 * u + 4 * half);
        return cat8(*reinterpret_cast<const bf16x4*>(p), *reinterpret_cast<const bf16x4*>(p + 16));
      };
      const bf16x8 bh = side(cb1, 0), bm = side(cb1, 1), bl = side(cb1, 2);
      ga[0] = DN_MFMA_B16(ah, ah, ga[0]);
      ga[1] = DN_MFMA_B16(ah, bh, ga[1]);
      ga[0] = DN_MFMA_B16(ah, am, ga[0]);
      ga[1] = DN_MFMA_B16(ah, bm, ga[1]);
      ga[0] = DN_MFMA_B16(am, ah, ga[0]);
      ga[1] = DN_MFMA_B16(am, bh, ga[1]);
      ga[0] = DN_MFMA_B16(ah, al, ga[0]);
      ga[1] = DN_MFMA_B16(ah, bl, ga[1]);
      ga[0] = DN_MFMA_B16(al, ah, ga[0]);
      ga[1] = DN_MFMA_B16(al, bh, ga[1]);
      ga[0] = DN_MFMA_B16(am, am, ga[0]);
      ga[1] = DN_MFMA_B16(am, bm, ga[1]);
      if (third) {
        const bf16x8 ch = side(cb2, 0), cm = side(cb2, 1), cl = side(cb2, 2);
        ga[2] = DN_MFMA_B16(ah, ch, ga[2]);
        ga[2] = DN_MFMA_B16(ah, cm, ga[2]);
        ga[2] = DN_MFMA_B16(am, ch, ga[2]);
        ga[2] = DN_MFMA_B16(ah, cl, ga[2]);
        ga[2] = DN_MFMA_B16(al, ch, ga[2]);
        ga[2] = DN_MFMA_B16(am, cm, ga[2]);
      }
    }
    if ((it + 1) % XB_FLUSH == 0) {
      ga_flush(it / XB_FLUSH);
      ga_clear();
    }

    // every wave has left the X planes behind at the barrier above: they take the next tile
    commit(xb);
#pragma unroll
    for (int v = 0; v < 16; v++) pn[v] = pnn[v];
    __syncthreads();
  }
  // the chunk in progress, then zeros for the chunks this workgroup never reached
  int chunk = it / XB_FLUSH;
  if (it % XB_FLUSH != 0 || it == 0) ga_flush(chunk++);
  ga_clear();
  for (; chunk < n_flush; chunk++) ga_flush(chunk);
}

// Number of partial Gram matrices of the fused update (workgroups x flushes) for `rows` rows;
// runs_of_tiles: a workgroup takes several consecutive tiles at a time (xg_run) instead of one.
static int64_t xgg_parts(int64_t rows, int tile_rows, int flush, bool runs_of_tiles, int64_t* wgs_out,
                         int64_t* n_flush_out, int* run_out = nullptr) {
  const int64_t tiles = rows / tile_rows;
  int64_t wgs = (int64_t)n_cus() * 2;
  const int run = runs_of_tiles ? xg_run(tiles, wgs) : 1;
  if (run_out) *run_out = run;
  const int64_t runs = ceil_div(tiles > 0 ? tiles : 1, run);
  if (wgs > runs) wgs = runs;
  const int64_t n_flush = ceil_div(ceil_div(runs, wgs) * run, flush);
  if (wgs_out) *wgs_out = wgs;
  if (n_flush_out) *n_flush_out = n_flush;
  return wgs * n_flush;
}

// Workspace of the fused update in floats, for `rows` rows.
int64_t xg_mu_gram_workspace_floats(int64_t rows) {
  const int64_t a = xgg_parts(rows, XgReg<4>::ROWS, XGG_FLUSH, false, nullptr, nullptr);
  const int64_t b = xgg_parts(rows, XB_ROWS, XB_FLUSH, true, nullptr, nullptr);
  return (a > b ? a : b) * XGG_BLOCKS * 1024;
}

// out = X * num / (X G + eps) and Gout = out^T out for r = 128; rows >= 64.  The rows past the
// last whole tile go through the plain kernels and their Gram matrix (workspace `gram_ws`, at
// least gram_workspace_floats(64, 128) floats; `G_tmp` r x r) is added.
__global__ void __launch_bounds__(256) k_add_inplace(float* __restrict__ a, const float* __restrict__ b, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) a[i] += b[i];
}

int launch_xg_mu_gram(int64_t rows, const float* X, const float* G, const float* num, float eps,
                      float* out, float* Gout, float* gpart, float* G_tmp, float* gram_ws) {
  using C = XgReg<4>;
  constexpr int r = 128;
  const bool split = use_split_bf16();
  const int tile_rows = split ? XB_ROWS : C::ROWS;
  const size_t lds = split ? (size_t)XB_LDS : sizeof(float) * 2 * C::SLOT;
  static bool attr_set[2] = {false, false};
  if (!attr_set[split]) {
    DN_HIP(hipFuncSetAttribute(split ? (const void*)k_xg_mu_gram_b16 : (const void*)k_xg_mu_gram,
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set[split] = true;
  }
  const int64_t tiles = rows / tile_rows;
  DN_CHECK(tiles >= 1, "fused update needs at least one whole tile");
  DN_CHECK(((uintptr_t)X % 16) == 0, "fused update: X must be 16-byte aligned");
  int64_t wgs, n_flush;
  int run;
  xgg_parts(rows, tile_rows, split ? XB_FLUSH : XGG_FLUSH, split, &wgs, &n_flush, &run);
  if (split)
    hipLaunchKernelGGL(k_xg_mu_gram_b16, dim3((unsigned)wgs), dim3(256), lds, stream(), X, G, num, eps,
                       tiles, run, (int)n_flush, out, gpart);
  else
    hipLaunchKernelGGL(k_xg_mu_gram, dim3((unsigned)wgs), dim3(256), lds, stream(), X, G, num, eps, tiles,
                       (int)n_flush, out, gpart);
  hipLaunchKernelGGL(k_xg_gram_reduce, dim3(128 * 128 / 32), dim3(256), 0, stream(), gpart,
                     wgs * n_flush, Gout);
  DN_LAUNCH_CHECK();
  const int64_t head = tiles * tile_rows;
  if (head < rows) {
    const int64_t off = head * r;
    DN_TRY(launch_xg_mu_nb<4>(rows - head, r, X + off, G, num + off, eps, out + off, nullptr));
    DN_TRY(launch_gram(rows - head, r, out + off, G_tmp, gram_ws));
    hipLaunchKernelGGL(k_add_inplace, dim3(r * r / 256), dim3(256), 0, stream(), Gout, G_tmp, r * r);
    DN_LAUNCH_CHECK();
  }
  return 0;
}

// Kernel-level entry point of the fused update (rank 128): allocates its workspaces per call.
DN_API int dnpeff_op_xg_mu_gram(int64_t rows, const float* X, const float* G_rr, const float* num,
                                float eps, float* out, float* Gout_rr) {
  clear_error();
  DN_CHECK(rows >= 64, "fused update needs at least 64 rows");
  float *gpart = nullptr, *G_tmp = nullptr, *gram_ws = nullptr;
  int s = dmalloc(&gpart, xg_mu_gram_workspace_floats(rows)) || dmalloc(&G_tmp, 128 * 128) ||
          dmalloc(&gram_ws, gram_workspace_floats(64, 128));
  if (!s) s = launch_xg_mu_gram(rows, X, G_rr, num, eps, out, Gout_rr, gpart, G_tmp, gram_ws);
  if (!s && hipStreamSynchronize(stream()) != hipSuccess) {
    set_error("fused update: kernel failed");
    s = 1;
  }
  dfree(gpart);
  dfree(G_tmp);
  dfree(gram_ws);
  return s;
}

int launch_xg_mu(int64_t rows, int r, const float* X, const float* G, const float* num, float eps,
                 float* out, float* D_out) {
  DN_CHECK(r >= 1 && r <= 1024, "rank %d outside [1, 1024]", r);
  DN_CHECK(out != X, "xg_mu: out must not alias X");
  if (rows <= 0) return 0;
  const bool aligned = ((uintptr_t)X % 16) == 0;
  if ((r == 32 || r == 64 || r == 128) && aligned && rows >= 256) {
    // whole tiles with the compile-time-rank kernel, the last rows below
    int64_t head;
    if (r == 128) {
      head = rows / XgReg<4>::ROWS * XgReg<4>::ROWS;
      DN_TRY(launch_xg_mu_reg<4>(head, X, G, num, eps, out, D_out));
    } else if (r == 64) {
      head = rows / XgReg<2>::ROWS * XgReg<2>::ROWS;
      DN_TRY(launch_xg_mu_reg<2>(head, X, G, num, eps, out, D_out));
    } else {
      head = rows / XgReg<1>::ROWS * XgReg<1>::ROWS;
      DN_TRY(launch_xg_mu_reg<1>(head, X, G, num, eps, out, D_out));
    }
    if (head == rows) return 0;
    const int64_t off = head * r;
    return launch_xg_mu_nb<4>(rows - head, r, X + off, G, num + off, eps, out + off,
                              D_out ? D_out + off : nullptr);
  }
  if (r > 128 && r % 128 == 0 && aligned && ((uintptr_t)G % 16) == 0 && rows >= 256 &&
      ceil_div(rows, 128) * (r / 128) < ((int64_t)1 << 24)) {
    if (use_split_bf16() && ((uintptr_t)num % 4) == 0)
      return launch_xg_mu_tile_b16(rows, r, X, G, num, eps, out, D_out);
    return launch_xg_mu_tile(rows, r, X, G, num, eps, out, D_out);
  }
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
  const int64_t tiles_c = (cols + 31) / 32, tiles_r = (rows + 31) / 32;
  for (int64_t t = blockIdx.x; t < tiles_c * tiles_r; t += gridDim.x) {
    const int64_t tile_r = t / tiles_c, tile_c = t % tiles_c;
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
    __syncthreads();
  }
}

int launch_transpose(int64_t rows, int64_t cols, const float* in, float* out) {
  if (rows <= 0 || cols <= 0) return 0;
  int64_t tiles = ceil_div(rows, 32) * ceil_div(cols, 32);
  if (tiles > ((int64_t)1 << 22)) tiles = (int64_t)1 << 22;  // the kernel loops over the rest
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

// ---------------------------------------------------------------------------
// The Gram product without any allocation: the slice partials go to a file-scope device array.
// Every GPU holds its own copy of the array at its own address, taken once per device with
// hipGetSymbolAddress; host code never uses the array's name as a pointer.
// ---------------------------------------------------------------------------
constexpr int64_t GRAM_STATIC_FLOATS = 2 * 1024 * 1024;  // 8 MiB per GPU, held until the process ends
constexpr int GRAM_STATIC_MAX_DEVICES = 64;
static __device__ __align__(256) float scratch[GRAM_STATIC_FLOATS];
static float* g_scratch_ptr[GRAM_STATIC_MAX_DEVICES] = {};

// Address of this device's copy of the scratch array (looked up on first use on a device).
static int gram_static_scratch(float** out) {
  int dev = 0;
  DN_HIP(hipGetDevice(&dev));
  DN_CHECK(dev >= 0 && dev < GRAM_STATIC_MAX_DEVICES, "device %d outside [0, %d)", dev,
           GRAM_STATIC_MAX_DEVICES);
  if (!g_scratch_ptr[dev]) {
    float* p = nullptr;
    DN_HIP(hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch)));
    DN_CHECK(p != nullptr, "no device address for the static scratch array");
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

DN_API int dnpeff_op_gram_static(int64_t rows, int r, const float* X, float* G_rr) {
  clear_error();
  DN_CHECK(X && G_rr, "NULL argument");
  DN_CHECK(rows >= 1, "rows must be at least 1 (got %lld)", (long long)rows);
  DN_CHECK(r >= 1 && r <= 128, "dnpeff_op_gram_static handles ranks 1..128 (got %d)", r);
  const int64_t need = gram_workspace_floats(rows, r);
  DN_CHECK(need <= GRAM_STATIC_FLOATS,
           "dnpeff_op_gram_static: %lld rows at rank %d need %lld floats of partial sums, the static "
           "scratch holds %lld (at most %lld rows at ranks above 32)",
           (long long)rows, r, (long long)need, (long long)GRAM_STATIC_FLOATS,
           (long long)(GRAM_STATIC_FLOATS / (gram_pairs(128) * 1024) * 256));
  float* ws = nullptr;
  DN_TRY(gram_static_scratch(&ws));
  // every partial block that the reduction reads is written by the product kernel of the same
  // call, so nothing of the last call's contents needs clearing
  return launch_gram(rows, r, X, G_rr, ws);
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
