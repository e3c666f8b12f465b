// Dense head of a sparse matrix: the columns that are present in a sizeable fraction of the
// rows are taken out of the CSR structures and kept as a dense block ("cm", one head column after
// the other; a second copy "rm" in the other orientation only for the fp32 kernel of A^T W).
// Their share of A H^T and A^T W is then a matrix product on fp32 MFMA (32x32x2) instead of one
// 4r-byte gather per entry; the remaining ("tail") entries stay sparse.
//
//   A H^T  = tail(A) H^T + D  Hd        D  [n, n_d] dense block, Hd = rows of H of the head
//   A^T W  : rows of the head  = D^T W, all other rows = tail(A)^T W
//
// Both products have the form C = P^T Q with P [K, ldp] and Q [K, r] sharing the contraction
// index K as their slow index: P = D^T ("cm", K = n_d) for the first, P = D ("rm", K = n) for
// the second.
#include "dnpeff_internal.hpp"
#include "abt_b16.hpp"


namespace dn {

typedef float acc16 __attribute__((ext_vector_type(16)));

// ---------------------------------------------------------------------------
// C[slice] = P[k in slice]^T Q[k in slice]
//
// A workgroup of 4 waves owns a 128 x 128 tile of C and one slice of K (every S-th tile of 32
// contraction rows), streamed through two LDS slots (P tile then Q tile, 20 KB each), fetched
// with 16-byte loads two tiles ahead into registers and written to LDS as they are (16-byte
// stores).  v_mfma_f32_32x32x2f32 takes from lane l A[i = l%32][k = l/32] and
// B[k = l/32][j = l%32]: a lane reads P[k][32 a + i] and Q[k][32 b + j] of its blocks with 4-byte
// LDS reads, the two half-waves on rows k and k + 1.  Wave (wm, wn) owns the 32-wide blocks
// {2 wm, 2 wm + 1} x {2 wn, 2 wn + 1} of the tile.
// ---------------------------------------------------------------------------
constexpr int PTQ_KB = 32;
constexpr int PTQ_LD = 160;              // LDS row: 128 floats + 32, so that the two half-waves
                                         // (rows k and k + 1) fall on different banks
constexpr int PTQ_HALF = PTQ_KB * PTQ_LD;  // floats of one operand tile
constexpr int PTQ_SLOT = 2 * PTQ_HALF;   // floats of one slot

struct PtqStage {
  float4 p[4], q[4];
};

__global__ void __launch_bounds__(256)
    k_ptq(const float* __restrict__ P, int64_t ldp, int64_t K, const float* __restrict__ Q, int r,
          int64_t M, int64_t M_pad, int upper_only,
          float* __restrict__ out) {
  extern __shared__ __align__(16) float lds[];  // 2 * PTQ_SLOT floats
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;
  // Symmetric product (upper_only = number of 128-wide tiles per side): grid.x numbers the tile
  // pairs (i <= j) row by row.  Every workgroup of the grid works: the hardware deals workgroups
  // to the XCDs round-robin by their linear number, and a grid with idle numbers at a fixed
  // stride would leave whole XCDs without work.
  int ti = blockIdx.x, tj = blockIdx.y;
  if (upper_only) {
    int p = blockIdx.x, row_len = upper_only;
    ti = 0;
    while (p >= row_len) {
      p -= row_len;
      ti++;
      row_len--;
    }
    tj = ti + p;
  }
  const int64_t m0 = (int64_t)ti * 128;
  const int n0 = tj * 128;
  // the K tiles are dealt to the slices round-robin (slice z owns tiles z, z + S, ...), so that
  // at any moment the workgroups read one contiguous window of P and Q
  const int64_t all_tiles = (K + PTQ_KB - 1) / PTQ_KB;
  const int64_t S = gridDim.z, z = blockIdx.z;
  const int64_t n_tiles = all_tiles > z ? (all_tiles - z + S - 1) / S : 0;

  // loader role of a thread: 16-byte column li of rows lr + 8 q of a tile
  const int li = threadIdx.x & 31, lr = threadIdx.x >> 5;
  const bool qcol_ok = n0 + 4 * li < r;
  const float* pP = P + m0 + 4 * li;
  const float* pQ = Q + n0 + 4 * li;

  auto fetch = [&](PtqStage& s, int64_t tile) {
    const int64_t kbase = (z + tile * S) * PTQ_KB + lr;
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const int64_t k = kbase + 8 * q;
      const bool ok = tile < n_tiles && k < K;
      s.p[q] = ok ? *reinterpret_cast<const float4*>(pP + k * ldp)
                  : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      s.q[q] = (ok && qcol_ok) ? *reinterpret_cast<const float4*>(pQ + k * (int64_t)r)
                               : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
  };
  auto commit = [&](const PtqStage& s, float* slot) {
#pragma unroll
    for (int q = 0; q < 4; q++) {
      float* a = slot + (lr + 8 * q) * PTQ_LD + 4 * li;
      *reinterpret_cast<float4*>(a) = s.p[q];
      *reinterpret_cast<float4*>(a + PTQ_HALF) = s.q[q];
    }
  };

  acc16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

  // Operands of 4 row pairs are read one group ahead of the MFMAs that use them; the scheduling
  // fences keep the compiler from sinking the LDS reads back to their first use, which would
  // expose the LDS latency once per 4 MFMAs.
  auto mfma_slot = [&](const float* slot) {
    const float* pa = slot + half * PTQ_LD + 64 * wm + l32;
    const float* pb = slot + PTQ_HALF + half * PTQ_LD + 64 * wn + l32;
    constexpr int GRP = 4, NG = PTQ_KB / 2 / GRP;
    float xa[2][GRP][2], xb[2][GRP][2];
    auto read_group = [&](int g, float (&ya)[GRP][2], float (&yb)[GRP][2]) {
#pragma unroll
      for (int u = 0; u < GRP; u++) {
        ya[u][0] = pa[2 * (g * GRP + u) * PTQ_LD];
        ya[u][1] = pa[2 * (g * GRP + u) * PTQ_LD + 32];
        yb[u][0] = pb[2 * (g * GRP + u) * PTQ_LD];
        yb[u][1] = pb[2 * (g * GRP + u) * PTQ_LD + 32];
      }
    };
    read_group(0, xa[0], xb[0]);
#pragma unroll
    for (int g = 0; g < NG; g++) {
      if (g + 1 < NG) read_group(g + 1, xa[(g + 1) & 1], xb[(g + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < GRP; u++)
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
          for (int j = 0; j < 2; j++)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(xa[g & 1][u][i], xb[g & 1][u][j],
                                                             acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  PtqStage s0, s1;
  fetch(s0, 0);
  fetch(s1, 1);
  if (n_tiles > 0) commit(s0, lds);
  __syncthreads();
  // iteration t: tile t sits in slot t & 1; its register stage is free and receives tile t + 2;
  // tile t + 1 moves from the other stage to the other slot after the MFMAs
  int64_t t = 0;
  for (; t + 2 <= n_tiles; t += 2) {
    fetch(s0, t + 2);
    mfma_slot(lds);
    commit(s1, lds + PTQ_SLOT);
    __syncthreads();
    fetch(s1, t + 3);
    mfma_slot(lds + PTQ_SLOT);
    if (t + 2 < n_tiles) commit(s0, lds);
    __syncthreads();
  }
  if (t < n_tiles) mfma_slot(lds);

  // D layout of a 32x32 block: reg v of lane l holds row 8 (v/4) + 4 (l/32) + v%4, column l%32;
  // block (i, j) of the wave covers rows 64 wm + 32 i.., columns 64 wn + 32 j.. of the tile.
  float* base = out + ((int64_t)blockIdx.z * M_pad + m0 + 64 * wm + 4 * half) * r + n0 + 64 * wn + l32;
#pragma unroll
  for (int j = 0; j < 2; j++) {
    if (n0 + 64 * wn + 32 * j + l32 >= r) continue;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int below = 32 * i + 8 * (v >> 2) + (v & 3);
        if (m0 + 64 * wm + 4 * half + below < M) base[(int64_t)below * r + 32 * j] = acc[i][j][v];
      }
  }
}

// slices of K so that the launch holds about a thousand workgroups
static int64_t ptq_slices(int64_t tiles_mn, int64_t k_tiles) {
  int64_t s = (4 * (int64_t)n_cus()) / (tiles_mn > 0 ? tiles_mn : 1);
  if (s > 64) s = 64;
  if (s > k_tiles) s = k_tiles;
  return s < 1 ? 1 : s;
}

static int launch_ptq(const float* P, int64_t ldp, int64_t K, const float* Q, int r, int64_t M,
                      int64_t M_pad, int64_t slices, float* out, int upper_only = 0) {
  static bool attr_set = false;
  const size_t lds = sizeof(float) * 2 * PTQ_SLOT;
  if (!attr_set) {
    DN_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_ptq),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set = true;
  }
  DN_CHECK(M_pad % 128 == 0 && ldp % 4 == 0 && r % 4 == 0, "dense product: misaligned operands");
  DN_CHECK(M_pad / 128 < ((int64_t)1 << 22), "dense product: too many row tiles");
  dim3 grid((unsigned)(M_pad / 128), (unsigned)ceil_div(r, 128), (unsigned)slices);
  if (upper_only) grid = dim3((unsigned)(upper_only * (upper_only + 1) / 2), 1, (unsigned)slices);
  hipLaunchKernelGGL(k_ptq, grid, dim3(256), lds, stream(), P, ldp, K, Q, r, M, M_pad,
                     upper_only, out);
  DN_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// C[slice] = A[:, k in slice] B[:, k in slice]^T on the bf16 matrix cores, at fp32 accuracy.
//
// Both operands have the contraction index as their FAST index (A [M_pad, lda], B [N, ldb]): a
// lane of v_mfma_f32_32x32x16_bf16 holds 8 consecutive contraction elements of one row, which
// is then one 16-byte LDS read.  Every fp32 element is split in three bf16 parts once, on its
// way into LDS (three planes per operand, rows of 32 elements padded to 80 bytes: conflict-free
// 16-byte reads), and a product is six MFMAs (split_bf16.hpp).  A workgroup of 4 waves owns a
// 128 x 128 tile of C (wave (wm, wn): 64 x 64) and one slice of the contraction tiles of 32,
// dealt round-robin; the next two tiles travel in registers while the MFMAs of the current one run.
// Per contraction tile a wave issues 48 MFMAs of 32 cycles and splits 32 elements (176 vector
// instructions): 2240 SIMD cycles against 4096 for the 64 v_mfma_f32_32x32x2f32 of k_ptq.
// Operands are zero-padded to whole tiles (rows to M_pad / N, the contraction to a multiple of
// 32 within lda / ldb), so the loads need no bounds.
// ---------------------------------------------------------------------------
// A_KN: A is stored with the contraction index slow (A[k * lda + row], lda >= M_pad).
template <bool A_KN>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
    k_abt_b16(const float* __restrict__ A, int64_t lda, const float* __restrict__ B, int64_t ldb,
              int64_t K, int N, int64_t M, int64_t M_pad, float* __restrict__ out) {
  extern __shared__ __align__(16) unsigned char ab[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;
  const int64_t m0 = (int64_t)blockIdx.x * 128;
  const int n0 = blockIdx.y * 128;
  const int64_t k_tiles = (K + ABT_KB - 1) / ABT_KB;
  const int64_t S = gridDim.z, z = blockIdx.z;
  const int64_t n_my = z < k_tiles ? (k_tiles - z + S - 1) / S : 0;

  acc16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;
  abt_mainloop<A_KN, false, ABT_STAGES_ABT>(A_KN ? A + m0 : A + m0 * lda, lda, B + (int64_t)n0 * ldb, ldb, z, S, n_my, ab,
                            acc);

  // D layout of a 32x32 block: reg v of lane l holds row 8 (v/4) + 4 (l/32) + v%4, column l%32;
  // block (i, j) of the wave covers rows 64 wm + 32 i.., columns 64 wn + 32 j.. of the tile.
  float* base = out + ((int64_t)blockIdx.z * M_pad + m0 + 64 * wm + 4 * half) * N + n0 + 64 * wn + l32;
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int below = 32 * i + 8 * (v >> 2) + (v & 3);
        if (m0 + 64 * wm + 4 * half + below < M) base[(int64_t)below * N + 32 * j] = acc[i][j][v];
      }
}

static int launch_abt_b16(const float* A, int64_t lda, const float* B, int64_t ldb, int64_t K, int N,
                          int64_t M, int64_t M_pad, int64_t slices, float* out, bool a_kn = false) {
  static bool attr_set = false;
  if (!attr_set) {
    DN_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_abt_b16<false>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, ABT_LDS));
    DN_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_abt_b16<true>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, ABT_LDS));
    attr_set = true;
  }
  const int64_t k_pad = ceil_div(K, ABT_KB) * ABT_KB;
  DN_CHECK(M_pad % 128 == 0 && N % 128 == 0 && lda % 4 == 0 && ldb % 4 == 0 &&
               (a_kn ? M_pad <= lda : k_pad <= lda) && k_pad <= ldb && ((uintptr_t)A % 16) == 0 &&
               ((uintptr_t)B % 16) == 0,
           "dense product: misaligned or unpadded operands");
  DN_CHECK(M_pad / 128 < ((int64_t)1 << 22), "dense product: too many row tiles");
  dim3 grid((unsigned)(M_pad / 128), (unsigned)(N / 128), (unsigned)slices);
  if (a_kn)
    hipLaunchKernelGGL(k_abt_b16<true>, grid, dim3(256), ABT_LDS, stream(), A, lda, B, ldb, K, N, M, M_pad, out);
  else
    hipLaunchKernelGGL(k_abt_b16<false>, grid, dim3(256), ABT_LDS, stream(), A, lda, B, ldb, K, N, M, M_pad, out);
  DN_LAUNCH_CHECK();
  return 0;
}

// out[c * ld + i] = in[i * cols + c] for i < rows, 0 for rows <= i < ld   (32 x 32 tiles via LDS)
__global__ void __launch_bounds__(256)
    k_transpose_pad(const float* __restrict__ in, int64_t rows, int cols, int64_t ld,
                    float* __restrict__ out) {
  __shared__ float tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const int64_t i0 = (int64_t)blockIdx.x * 32;
  const int c0 = blockIdx.y * 32;
  for (int q = ty; q < 32; q += 8) {
    const int64_t i = i0 + q;
    const int c = c0 + tx;
    tile[q][tx] = (i < rows && c < cols) ? in[i * cols + c] : 0.0f;
  }
  __syncthreads();
  for (int q = ty; q < 32; q += 8) {
    const int c = c0 + q;
    const int64_t i = i0 + tx;
    if (c < cols && i < ld) out[(int64_t)c * ld + i] = tile[tx][q];
  }
}

// out[j * ld + k] = H[cols[k]][j] for k < n_d, 0 for n_d <= k < ld
__global__ void __launch_bounds__(256)
    k_head_gather_t(const float* __restrict__ H, const int32_t* __restrict__ cols, int64_t n_d, int r,
                    int64_t ld, float* __restrict__ out) {
  __shared__ float tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const int64_t k0 = (int64_t)blockIdx.x * 32;
  const int j0 = blockIdx.y * 32;
  for (int q = ty; q < 32; q += 8) {
    const int64_t k = k0 + q;
    const int j = j0 + tx;
    tile[q][tx] = (k < n_d && j < r) ? H[(int64_t)cols[k] * r + j] : 0.0f;
  }
  __syncthreads();
  for (int q = ty; q < 32; q += 8) {
    const int j = j0 + q;
    const int64_t k = k0 + tx;
    if (j < r && k < ld) out[(int64_t)j * ld + k] = tile[tx][q];
  }
}

// ---------------------------------------------------------------------------
// Gram X^T X for ranks that are multiples of 128 above 128: the same tiles with P = Q = X, only
// the tile pairs (i <= j), K split into slices; the reduction sums the slices in fp64 and writes
// every element and its mirror image.
// ---------------------------------------------------------------------------
static int64_t gram_tiles_slices(int64_t rows, int r) {
  const int64_t t = r / 128, pairs = t * (t + 1) / 2;
  // two workgroups fit a CU: at most 2 rounds of 2 x 256 workgroups, never a few stragglers
  int64_t s = (4 * (int64_t)n_cus()) / pairs;
  const int64_t k_tiles = ceil_div(rows, PTQ_KB);
  if (s > k_tiles) s = k_tiles;
  return s < 1 ? 1 : s;
}

// The split-operand kernel runs the diagonal tile pairs and the others as two launches (a
// diagonal pair fetches and splits one tile, not two), each with the slices that fill the 2
// workgroup slots per CU once.
// paired: the diagonal tiles go two and two as squares of 256 columns (one workgroup of eight
// waves per CU), and the other launch takes the tile pairs that lie outside those squares.
static bool gram_paired(int r) { return tuning().gram_fold >= 2 && r % 256 == 0; }
static void gram_b16_slices(int64_t rows, int r, int64_t* s_diag, int64_t* s_off, bool paired = false) {
  const int64_t t = r / 128, slots = 2 * (int64_t)n_cus(), k_tiles = rows / 32;
  const int64_t n_off = t * (t - 1) / 2 - (paired ? t / 2 : 0);
  int64_t d = slots / t, o = n_off > 0 ? slots / n_off : 0;  // (paired: t / 2 squares, one slot per CU)
  if (d < 1) d = 1;
  if (n_off > 0 && o < 1) o = 1;
  if (d > k_tiles) d = k_tiles;
  if (o > k_tiles) o = k_tiles;
  *s_diag = d < 1 ? 1 : d;
  *s_off = n_off > 0 ? (o < 1 ? 1 : o) : 0;
}

int64_t gram_tiles_workspace_floats(int64_t rows, int r) {
  int64_t d, o, dp, op;
  gram_b16_slices(rows, r, &d, &o);
  gram_b16_slices(rows, r, &dp, &op, true);
  const int64_t s = std::max(std::max(gram_tiles_slices(rows, r), std::max(d, o)), std::max(dp, op));
  return (s + 1) * (int64_t)r * r;
}

// Diagonal tiles hold s_diag slices, the others s_off, and slice number `extra` (if >= 0) holds
// one more term of every tile (the last rows, from the fp32 kernel).
__global__ void __launch_bounds__(256)
    k_gram_tiles_reduce(const float* __restrict__ ws, int64_t s_diag, int64_t s_off, int64_t extra, int r,
                        int folded, float* __restrict__ G) {
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= r * r) return;
  const int a = e / r, b = e % r;
  if (a > b) return;  // upper triangle only
  double s = 0.0;
  const int64_t stride = (int64_t)r * r;
  // folded = 1: diagonal tiles of 128 from k_gram_diag_b16; 2: diagonal squares of 256 from
  // k_gram_pair_b16, where the block four block columns to the right of the diagonal comes in
  // two halves, one of them stored transposed below the diagonal
  const bool own = folded == 2 ? (a >> 8) == (b >> 8) : (a >> 7) == (b >> 7);
  const int64_t slices = own ? s_diag : s_off;
  if (folded && ((a >> 5) == (b >> 5) || (folded == 2 && own && (b >> 5) - (a >> 5) == 4))) {
    // the stored block plus (the stored block at the mirrored place) transposed
    const int et = b * r + a;
    for (int64_t sl = 0; sl < slices; sl++)
      s += (double)ws[sl * stride + e] + (double)ws[sl * stride + et];
  } else
  for (int64_t sl = 0; sl < slices; sl++) s += (double)ws[sl * stride + e];
  if (extra >= 0) s += (double)ws[extra * stride + e];
  G[(int64_t)a * r + b] = (float)s;
  G[(int64_t)b * r + a] = (float)s;
}

// The same on the bf16 matrix cores with split operands (abt_b16.hpp): both operand tiles are
// column tiles of X, read with the contraction index (the rows of X) slow.  Whole contraction
// tiles of 32 rows only; the caller adds the last rows.
// DIAG: grid.x numbers the diagonal tiles; otherwise the tile pairs (ti < tj) row by row: every
// workgroup of the grid works.
// paired (not DIAG): without the pairs (2 g, 2 g + 1), which k_gram_pair_b16 covers.
template <bool DIAG>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
    k_gram_tiles_b16(const float* __restrict__ X, int64_t k_tiles, int r, int n_tiles_side,
                     float* __restrict__ out, bool paired) {
  extern __shared__ __align__(16) unsigned char ab[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;
  int ti = blockIdx.x, tj = blockIdx.x;
  if (!DIAG) {
    int p = blockIdx.x;
    ti = 0;
    for (;;) {
      const int first = ti + 1 + ((paired && !(ti & 1)) ? 1 : 0), row_len = n_tiles_side - first;
      if (p < row_len || ti >= n_tiles_side - 1) {
        tj = first + p;
        break;
      }
      p -= row_len;
      ti++;
    }
    if (tj >= n_tiles_side) return;  // (a grid larger than the pairs: not launched)
  }
  const int64_t S = gridDim.z, z = blockIdx.z;
  const int64_t n_my = z < k_tiles ? (k_tiles - z + S - 1) / S : 0;
  acc16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;
  abt_mainloop<true, true, ABT_STAGES_GRAM, DIAG>(X + 128 * ti, r, X + 128 * tj, r, z, S, n_my, ab, acc);
  float* base = out + ((int64_t)z * r + 128 * ti + 64 * wm + 4 * half) * r + 128 * tj + 64 * wn + l32;
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int v = 0; v < 16; v++)
        base[(int64_t)(32 * i + 8 * (v >> 2) + (v & 3)) * r + 32 * j] = acc[i][j][v];
}

// The diagonal tiles with the work their symmetry leaves (gram_diag_mainloop): the ten upper
// blocks of 32 x 32 are stored, those on the diagonal as Q / 2 + P, so that the reduction gets
// Q + P + P^T as the sum of the stored block and its transpose.
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
    k_gram_diag_b16(const float* __restrict__ X, int64_t k_tiles, int r, float* __restrict__ out) {
  extern __shared__ __align__(16) unsigned char ab[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int ti = blockIdx.x;
  const int64_t S = gridDim.z, z = blockIdx.z;
  const int64_t n_my = z < k_tiles ? (k_tiles - z + S - 1) / S : 0;
  acc16 acc[5];
#pragma unroll
  for (int b = 0; b < 5; b++)
#pragma unroll
    for (int v = 0; v < 16; v++) acc[b][v] = 0.0f;
  gram_diag_mainloop<ABT_STAGES_GRAM>(X + 128 * ti, r, z, S, n_my, ab, acc);
  float* tile = out + ((int64_t)z * r + 128 * ti + 4 * half) * r + 128 * ti + l32;
  auto store = [&](int bi, int bj, const acc16& c) {
    float* base = tile + (int64_t)(32 * bi) * r + 32 * bj;
#pragma unroll
    for (int v = 0; v < 16; v++) base[(int64_t)(8 * (v >> 2) + (v & 3)) * r] = c[v];
  };
  if (wave < 2) {
    const int p = 2 * wave;
    store(p, p + 1, acc[0]);
    acc16 d0, d1;
#pragma unroll
    for (int v = 0; v < 16; v++) {
      d0[v] = 0.5f * acc[1][v] + acc[2][v];
      d1[v] = 0.5f * acc[3][v] + acc[4][v];
    }
    store(p, p, d0);
    store(p + 1, p + 1, d1);
  } else {
    store(wave - 2, 2, acc[0]);
    store(wave - 2, 3, acc[1]);
  }
}

// A diagonal square of 256 columns (gram_pair_mainloop): its 36 upper blocks of 32 x 32 are
// stored, those on the diagonal as Q / 2 + P; blocks that a wave holds as (w, j) with j < w are
// stored transposed at (j, w); the half block that waves 4-7 hold of (w - 4, w) stays as it is,
// below the diagonal at (w, w - 4), and the reduction adds its transpose to the other half.
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
    k_gram_pair_b16(const float* __restrict__ X, int64_t k_tiles, int r, float* __restrict__ out) {
  extern __shared__ __align__(16) unsigned char ab[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int l32 = lane & 31, half = lane >> 5;
  const int g = blockIdx.x;
  const int64_t S = gridDim.z, z = blockIdx.z;
  const int64_t n_my = z < k_tiles ? (k_tiles - z + S - 1) / S : 0;
  acc16 acc[6];
#pragma unroll
  for (int b = 0; b < 6; b++)
#pragma unroll
    for (int v = 0; v < 16; v++) acc[b][v] = 0.0f;
  gram_pair_mainloop<ABT_STAGES_GRAM>(X + 256 * g, r, z, S, n_my, ab, acc);
  float* square = out + ((int64_t)z * r + 256 * g) * r + 256 * g;
  // element (8 (v / 4) + v % 4 + 4 half, l32) of block (bi, bj)
  auto store = [&](int bi, int bj, const acc16& c) {
    float* base = square + (int64_t)(32 * bi + 4 * half) * r + 32 * bj + l32;
#pragma unroll
    for (int v = 0; v < 16; v++) base[(int64_t)(8 * (v >> 2) + (v & 3)) * r] = c[v];
  };
  auto store_transposed = [&](int bi, int bj, const acc16& c) {  // the block (bi, bj) to the place (bj, bi)
    float* base = square + (int64_t)(32 * bj + l32) * r + 32 * bi + 4 * half;
#pragma unroll
    for (int v = 0; v < 16; v++) base[8 * (v >> 2) + (v & 3)] = c[v];
  };
#pragma unroll
  for (int k = 1; k < 4; k++) {
    const int bj = (wave + k) & 7;
    if (bj > wave)
      store(wave, bj, acc[k - 1]);
    else
      store_transposed(wave, bj, acc[k - 1]);
  }
  acc16 d;
#pragma unroll
  for (int v = 0; v < 16; v++) d[v] = 0.5f * acc[3][v] + acc[4][v];
  store(wave, wave, d);
  store(wave, (wave + 4) & 7, acc[5]);
}

int launch_gram_tiles(int64_t rows, int r, const float* X, float* G, float* workspace) {
  const int t = r / 128;
  int64_t s_diag, s_off, extra = -1;
  int folded = 0;
  if (use_split_bf16() && rows >= ABT_KB) {
    static bool attr_set = false;
    if (!attr_set) {
      DN_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gram_tiles_b16<true>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, ABT_LDS));
      DN_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gram_tiles_b16<false>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, ABT_LDS));
      DN_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gram_diag_b16),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, ABT_LDS));
      DN_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gram_pair_b16),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, ABT_LDS_PAIR));
      attr_set = true;
    }
    // whole contraction tiles on the bf16 matrix cores, the last rows (fewer than 32) as one
    // more slice through the fp32 kernel
    const int64_t k_tiles = rows / ABT_KB, whole = k_tiles * ABT_KB;
    const bool paired = gram_paired(r);
    gram_b16_slices(rows, r, &s_diag, &s_off, paired);
    folded = paired ? 2 : tuning().gram_fold != 0 ? 1 : 0;
    const int n_off = t * (t - 1) / 2 - (paired ? t / 2 : 0);
    if (paired)
      hipLaunchKernelGGL(k_gram_pair_b16, dim3((unsigned)(t / 2), 1, (unsigned)s_diag), dim3(512), ABT_LDS_PAIR,
                         stream(), X, k_tiles, r, workspace);
    else if (folded)
      hipLaunchKernelGGL(k_gram_diag_b16, dim3((unsigned)t, 1, (unsigned)s_diag), dim3(256), ABT_LDS, stream(),
                         X, k_tiles, r, workspace);
    else
      hipLaunchKernelGGL(k_gram_tiles_b16<true>, dim3((unsigned)t, 1, (unsigned)s_diag), dim3(256), ABT_LDS,
                         stream(), X, k_tiles, r, t, workspace, false);
    if (n_off > 0)
      hipLaunchKernelGGL(k_gram_tiles_b16<false>, dim3((unsigned)n_off, 1, (unsigned)s_off),
                         dim3(256), ABT_LDS, stream(), X, k_tiles, r, t, workspace, paired);
    DN_LAUNCH_CHECK();
    if (whole < rows) {
      extra = std::max(s_diag, s_off);
      DN_TRY(launch_ptq(X + whole * r, r, rows - whole, X + whole * r, r, r, r, 1,
                        workspace + extra * (int64_t)r * r, t));
    }
  } else {
    s_diag = s_off = gram_tiles_slices(rows, r);
    DN_TRY(launch_ptq(X, r, rows, X, r, r, r, s_diag, workspace, t));
  }
  hipLaunchKernelGGL(k_gram_tiles_reduce, dim3((unsigned)ceil_div((int64_t)r * r, 256)), dim3(256), 0,
                     stream(), workspace, s_diag, s_off, extra, r, folded, G);
  DN_LAUNCH_CHECK();
  return 0;
}

// Hd[k] = H[cols[k]]
__global__ void __launch_bounds__(256)
    k_head_gather(const float* __restrict__ H, const int32_t* __restrict__ cols, int64_t n_d, int r,
                  float* __restrict__ Hd) {
  const int r4 = r >> 2;
  const int64_t total = n_d * r4, stride = (int64_t)gridDim.x * 256;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += stride) {
    const int64_t k = e / r4;
    const int c = (int)(e % r4);
    reinterpret_cast<float4*>(Hd + k * r)[c] =
        reinterpret_cast<const float4*>(H + (int64_t)cols[k] * r)[c];
  }
}

// N[i] += sum over slices of ws[s][i]   (slices summed in fp64, in slice order)
__global__ void __launch_bounds__(256)
    k_head_add(const float* __restrict__ ws, int64_t slices, int64_t rows, int64_t rows_pad, int r,
               float* __restrict__ N) {
  const int r4 = r >> 2;
  const int64_t total = rows * r4, stride = (int64_t)gridDim.x * 256;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += stride) {
    const int64_t i = e / r4;
    const int c = (int)(e % r4);
    double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
    for (int64_t s = 0; s < slices; s++) {
      const float4 v = reinterpret_cast<const float4*>(ws + (s * rows_pad + i) * r)[c];
      s0 += v.x; s1 += v.y; s2 += v.z; s3 += v.w;
    }
    float4* o = reinterpret_cast<float4*>(N + i * r) + c;
    float4 cur = *o;
    cur.x = (float)((double)cur.x + s0);
    cur.y = (float)((double)cur.y + s1);
    cur.z = (float)((double)cur.z + s2);
    cur.w = (float)((double)cur.w + s3);
    *o = cur;
  }
}

// T[cols[k] - col0] = sum over slices of ws[s][k], k0 <= k < k1
__global__ void __launch_bounds__(256)
    k_head_scatter(const float* __restrict__ ws, int64_t slices, int64_t k0, int64_t k1,
                   int64_t n_d_pad, int r, const int32_t* __restrict__ cols, int64_t col0,
                   float* __restrict__ T) {
  const int r4 = r >> 2;
  const int64_t total = (k1 - k0) * r4, stride = (int64_t)gridDim.x * 256;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += stride) {
    const int64_t k = k0 + e / r4;
    const int c = (int)(e % r4);
    float4 out;
    if (slices == 1) {
      out = reinterpret_cast<const float4*>(ws + k * r)[c];
    } else {
      double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
      for (int64_t s = 0; s < slices; s++) {
        const float4 v = reinterpret_cast<const float4*>(ws + (s * n_d_pad + k) * r)[c];
        s0 += v.x; s1 += v.y; s2 += v.z; s3 += v.w;
      }
      out = make_float4((float)s0, (float)s1, (float)s2, (float)s3);
    }
    reinterpret_cast<float4*>(T + ((int64_t)cols[k] - col0) * r)[c] = out;
  }
}

static unsigned elem_grid(int64_t count) {
  int64_t g = ceil_div(count, 256);
  if (g > (1 << 20)) g = 1 << 20;
  return (unsigned)(g < 1 ? 1 : g);
}

// At ranks that are multiples of 128 the head products run on the bf16 matrix cores with split
// operands (k_abt_b16), otherwise (and with DNPEFF_SPLIT_BF16=0) on the fp32 ones (k_ptq).
static bool head_uses_split(int r) { return r % 128 == 0 && use_split_bf16(); }
int head_blocks_for_rank(int r) { return head_uses_split(r) ? 1 : 2; }
static int64_t head_gather_floats(const dense_head& h, int r) {
  return (h.n_d_pad > h.n_pad ? h.n_d_pad : h.n_pad) * (int64_t)r;
}

// Slices of the contraction: enough workgroups to fill the chip, and no fp32 running sum longer
// than 8192 products (the slices are added in fp64).
static int64_t head_slices_for(int64_t tiles_mn, int64_t K) {
  const int64_t k_tiles = ceil_div(K, PTQ_KB);
  int64_t s = ptq_slices(tiles_mn, k_tiles);
  const int64_t by_length = ceil_div(K, 8192);
  if (s < by_length) s = by_length;
  return s < k_tiles ? s : (k_tiles > 0 ? k_tiles : 1);
}
static int64_t head_slices_n(const dense_head& h, int r) {
  return head_slices_for((h.n_pad / 128) * ceil_div(r, 128), h.n_d);
}
static int64_t head_slices_t(const dense_head& h, int r, int64_t n) {
  return head_slices_for((h.n_d_pad / 128) * ceil_div(r, 128), n);
}

// Floats of the workspace that the products of a head of n_d columns over n_rows rows use at rank r:
// the gathered rows of H of the head, or W transposed (the split-operand product wants the
// contraction index fast), plus the slice partials of the larger of the two products.
int64_t head_workspace_floats(int64_t n_rows, int64_t n_d, int r) {
  if (n_d <= 0) return 0;
  dense_head h;
  h.n_d = n_d;
  h.n_d_pad = ceil_div(n_d, 128) * 128;
  h.n_pad = ceil_div(n_rows, 128) * 128;
  const int64_t gather = head_gather_floats(h, r);
  const int64_t wn = head_slices_n(h, r) * h.n_pad * r;
  const int64_t wt = head_slices_t(h, r, n_rows) * h.n_d_pad * r;
  return gather + (wn > wt ? wn : wt);
}

int head_ensure_workspace(dnpeff_csr* A, int r) {
  dense_head& h = A->head;
  if (h.n_d == 0) return 0;
  DN_CHECK(r % 4 == 0, "a matrix with a dense head needs a rank that is a multiple of 4 (got %d)", r);
  const int64_t need = head_workspace_floats(A->n_rows, h.n_d, r);
  if (!head_uses_split(r) && !h.rm) {  // the fp32 kernel of A^T W wants the block row by row
    if (dmalloc(&h.rm, h.n_pad * h.n_d_pad)) {
      // no room for the second copy: at ranks that the split-operand kernel handles the head's
      // share of A^T W stays on it (said once), other ranks cannot go on
      h.rm = nullptr;
      (void)hipGetLastError();  // (the failed allocation must not surface at the next launch check)
      DN_CHECK(r % 128 == 0, "dense head: no memory for the row-major block (%lld bytes)",
               (long long)(4 * h.n_pad * h.n_d_pad));
      clear_error();
      static bool told = false;
      if (!told) {
        told = true;
        fprintf(stderr, "dnpeff: no memory for the row-major copy of the dense head: its share of A^T W "
                        "stays on the split-operand kernel\n");
      }
    } else {
      DN_TRY(launch_transpose(h.n_d_pad, h.n_pad, h.cm, h.rm));
    }
  }
  if (h.ws && h.ws_floats >= need) return 0;
  dfree(h.ws);
  h.ws = nullptr;
  DN_TRY(dmalloc(&h.ws, need));
  h.ws_floats = need;
  return 0;
}

// slice partials of D Hd into the workspace
int launch_head_n(const dnpeff_csr* A, int r, const float* H_mr) {
  const dense_head& h = A->head;
  if (h.n_d == 0) return 0;
  DN_CHECK(h.ws && r % 4 == 0 && ((uintptr_t)H_mr % 16) == 0, "dense head: workspace or alignment");
  float* Hd = h.ws;
  float* part = h.ws + head_gather_floats(h, r);
  if (head_uses_split(r)) {
    // D [n, n_d] (cm, read with the contraction index slow) times the gathered rows, transposed:
    // contraction over the head slots
    dim3 tg((unsigned)ceil_div(h.n_d_pad, 32), (unsigned)ceil_div(r, 32));
    hipLaunchKernelGGL(k_head_gather_t, tg, dim3(256), 0, stream(), H_mr, h.cols, h.n_d, r, h.n_d_pad, Hd);
    return launch_abt_b16(h.cm, h.n_pad, Hd, h.n_d_pad, h.n_d, r, A->n_rows, h.n_pad,
                          head_slices_n(h, r), part, /*a_kn=*/true);
  }
  hipLaunchKernelGGL(k_head_gather, dim3(elem_grid(h.n_d * (r / 4))), dim3(256), 0, stream(), H_mr,
                     h.cols, h.n_d, r, Hd);
  return launch_ptq(h.cm, h.n_pad, h.n_d, Hd, r, A->n_rows, h.n_pad, head_slices_n(h, r), part);
}

// N += D Hd from the slice partials
int launch_head_n_add(const dnpeff_csr* A, int r, float* N_nr) {
  const dense_head& h = A->head;
  if (h.n_d == 0) return 0;
  const float* part = h.ws + head_gather_floats(h, r);
  hipLaunchKernelGGL(k_head_add, dim3(elem_grid(A->n_rows * (r / 4))), dim3(256), 0, stream(), part,
                     head_slices_n(h, r), A->n_rows, h.n_pad, r, N_nr);
  DN_LAUNCH_CHECK();
  return 0;
}

// slice partials of D^T W into the workspace
int launch_head_t_product(const dnpeff_csr* A, int r, const float* W_nr) {
  const dense_head& h = A->head;
  if (h.n_d == 0) return 0;
  DN_CHECK(h.ws && r % 4 == 0 && ((uintptr_t)W_nr % 16) == 0, "dense head: workspace or alignment");
  float* part = h.ws + head_gather_floats(h, r);
  const int64_t slices = head_slices_t(h, r, A->n_rows);
  if (head_uses_split(r) || (r % 128 == 0 && !h.rm)) {
    // D^T [n_d, n] (cm) times W transposed: contraction over the rows of the matrix
    float* Wt = h.ws;
    dim3 tg((unsigned)ceil_div(h.n_pad, 32), (unsigned)ceil_div(r, 32));
    hipLaunchKernelGGL(k_transpose_pad, tg, dim3(256), 0, stream(), W_nr, A->n_rows, r, h.n_pad, Wt);
    return launch_abt_b16(h.cm, h.n_pad, Wt, h.n_pad, A->n_rows, r, h.n_d, h.n_d_pad, slices, part);
  }
  DN_CHECK(h.rm != nullptr, "dense head: no row-major block for the fp32 product");
  return launch_ptq(h.rm, h.n_d_pad, A->n_rows, W_nr, r, h.n_d, h.n_d_pad, slices, part);
}

// rows of the head slots [k0, k1) of A^T W from the slice partials, to T_tile[cols[k] - col0]
// (overwrites what the sparse kernels stored there)
int launch_head_t_scatter(const dnpeff_csr* A, int r, int64_t k0, int64_t k1, int64_t col0,
                          float* T_tile) {
  const dense_head& h = A->head;
  if (h.n_d == 0 || k1 <= k0) return 0;
  DN_CHECK(h.ws && r % 4 == 0 && ((uintptr_t)T_tile % 16) == 0, "dense head: workspace or alignment");
  DN_CHECK(k0 >= 0 && k1 <= h.n_d, "dense head: slots [%lld, %lld) outside the head", (long long)k0,
           (long long)k1);
  const float* part = h.ws + head_gather_floats(h, r);
  hipLaunchKernelGGL(k_head_scatter, dim3(elem_grid((k1 - k0) * (r / 4))), dim3(256), 0, stream(), part,
                     head_slices_t(h, r, A->n_rows), k0, k1, h.n_d_pad, r, h.cols, col0, T_tile);
  DN_LAUNCH_CHECK();
  return 0;
}

int launch_head_t(const dnpeff_csr* A, int r, const float* W_nr, float* T_mr) {
  DN_TRY(launch_head_t_product(A, r, W_nr));
  return launch_head_t_scatter(A, r, 0, A->head.n_d, 0, T_mr);
}

}  // namespace dn
