// Main loop of the split-operand matrix products: C (128 x 128 per workgroup) +=
// A (128 x K) B (128 x K)^T on the bf16 matrix cores at fp32 accuracy (split_bf16.hpp).
#pragma once
#include "split_bf16.hpp"

namespace dn {

typedef float abt_acc16 __attribute__((ext_vector_type(16)));

constexpr int ABT_KB = 32;
constexpr int ABT_LD = 80;                // bytes per row of a plane: 32 bf16 + 16 of padding
constexpr int ABT_PLANE = 128 * ABT_LD;   // one part of one operand tile
constexpr int ABT_LDS = 6 * ABT_PLANE;    // A: h, m, l; B: h, m, l
#ifndef ABT_STAGES_XG
#define ABT_STAGES_XG 2
#endif
#ifndef ABT_STAGES_ABT
#define ABT_STAGES_ABT 2
#endif
#ifndef ABT_STAGES_GRAM
#define ABT_STAGES_GRAM 2
#endif

// One operand tile (128 rows x 32 contraction elements) on its way from global memory to the
// three bf16 planes in LDS, 16-byte loads either way.  KN = false: the source has the
// contraction index fast (src[row * ld + k]): a thread takes 4 contraction elements of 4 rows,
// 8 threads per row.  KN = true: the source has it slow (src[k * ld + row], e.g. a tile of X for
// X^T X): a thread takes a 4 x 4 block, 4 rows of each of 4 consecutive contraction elements, and
// turns it in registers; 8 consecutive threads hold the 32 contraction elements of 4 rows, so
// that their LDS stores fall into different banks.  (With 4-byte loads, 16 per thread, the
// address unit and not the matrix cores set the pace of X^T X.)  Either way four consecutive
// contraction elements of a row make one 8-byte LDS store per part.
template <bool KN>
struct AbtOperand {
  f32x4 r[4];
  __device__ __forceinline__ void fetch(const float* __restrict__ src, int64_t ld, int64_t k0) {
    if constexpr (!KN) {
      const int fr = threadIdx.x >> 3, fk = 4 * (threadIdx.x & 7);
#pragma unroll
      for (int q = 0; q < 4; q++)
        r[q] = *reinterpret_cast<const f32x4*>(src + (int64_t)(fr + 32 * q) * ld + k0 + fk);
    } else {
      const int row4 = 4 * (threadIdx.x >> 3), kb = 4 * (threadIdx.x & 7);
      const float* p = src + (k0 + kb) * ld + row4;
#pragma unroll
      for (int q = 0; q < 4; q++) r[q] = *reinterpret_cast<const f32x4*>(p + q * ld);
    }
  }
  // PLANE: bytes between the parts of the tile (a tile of 256 rows from a workgroup of 512 has
  // planes of twice the size)
  template <int PLANE = ABT_PLANE>
  __device__ __forceinline__ void commit(unsigned char* planes) const {
#pragma unroll
    for (int q = 0; q < 4; q++) {
      bf16x4 h, m, l;
      unsigned char* dst;
      if constexpr (!KN) {
        const int fr = threadIdx.x >> 3, fk = 4 * (threadIdx.x & 7);
        split3(r[q], h, m, l);
        dst = planes + (fr + 32 * q) * ABT_LD + 2 * fk;
      } else {
        const int row4 = 4 * (threadIdx.x >> 3), kb = 4 * (threadIdx.x & 7);
        split3(f32x4{r[0][q], r[1][q], r[2][q], r[3][q]}, h, m, l);
        dst = planes + (row4 + q) * ABT_LD + 2 * kb;
      }
      *reinterpret_cast<bf16x4*>(dst) = h;
      *reinterpret_cast<bf16x4*>(dst + PLANE) = m;
      *reinterpret_cast<bf16x4*>(dst + 2 * PLANE) = l;
    }
  }
};

// acc += A B^T over the contraction tiles first, first + stride, ... (n_tiles of them).  Wave
// (wm, wn) of the four owns the 64 x 64 quarter of the tile: blocks (i, j) of 32 x 32.  STAGES
// contraction tiles travel in registers while the 48 MFMAs of the current one run (one tile of
// MFMAs lasts 0.65 us, a trip to HBM three or four times that), and every fp32 element is split
// once, on its way into LDS.  The loads are unconditional, so that the waits for them are counted
// exactly: past the last tile they fetch the last one again.  The sources must be readable for
// whole tiles (zero padding, or rows clamped by the caller's pointer arithmetic); with A_KN /
// B_KN the source and its leading dimension must be 16-byte aligned.
// SAME_AB: B is A (a diagonal tile of X^T X): the tile is fetched, split and stored once and both
// operands are read from A's planes (a compile-time switch: a branch around the loads of B would
// cost the exact waits).
template <bool A_KN, bool B_KN, int STAGES = 1, bool SAME_AB = false>
__device__ __forceinline__ void abt_mainloop(const float* __restrict__ a_src, int64_t lda,
                                             const float* __restrict__ b_src, int64_t ldb,
                                             int64_t first, int64_t stride, int64_t n_tiles,
                                             unsigned char* ab, abt_acc16 (&acc)[2][2]) {
  static_assert(STAGES == 1 || STAGES == 2, "one or two tiles in registers");
  if (n_tiles <= 0) return;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l32 = lane & 31, half = lane >> 5, wm = wave >> 1, wn = wave & 1;
  AbtOperand<A_KN> oa[STAGES];
  AbtOperand<B_KN> ob[STAGES];
  auto fetch = [&](int s, int64_t t) {
    const int64_t k0 = (first + (t < n_tiles ? t : n_tiles - 1) * stride) * ABT_KB;
    oa[s].fetch(a_src, lda, k0);
    if constexpr (!SAME_AB) ob[s].fetch(b_src, ldb, k0);
  };
  auto commit = [&](int s) {
    oa[s].commit(ab);
    if constexpr (!SAME_AB) ob[s].commit(ab + 3 * ABT_PLANE);
  };
  const unsigned char* a_row = ab + (64 * wm + l32) * ABT_LD + 16 * half;
  const unsigned char* b_row = ab + (SAME_AB ? 0 : 3 * ABT_PLANE) + (64 * wn + l32) * ABT_LD + 16 * half;
  auto mfma_tile = [&]() {
#pragma unroll
    for (int st = 0; st < 2; st++) {
      bf16x8 ah[2], am[2], al[2], bh[2], bm[2], bl[2];
#pragma unroll
      for (int i = 0; i < 2; i++) {
        const unsigned char* pa = a_row + 32 * i * ABT_LD + 32 * st;
        ah[i] = *reinterpret_cast<const bf16x8*>(pa);
        am[i] = *reinterpret_cast<const bf16x8*>(pa + ABT_PLANE);
        al[i] = *reinterpret_cast<const bf16x8*>(pa + 2 * ABT_PLANE);
        const unsigned char* pb = b_row + 32 * i * ABT_LD + 32 * st;
        bh[i] = *reinterpret_cast<const bf16x8*>(pb);
        bm[i] = *reinterpret_cast<const bf16x8*>(pb + ABT_PLANE);
        bl[i] = *reinterpret_cast<const bf16x8*>(pb + 2 * ABT_PLANE);
      }
      // term by term over the four blocks: no instruction waits for the one before it
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = DN_MFMA_B16(ah[i], bh[j], acc[i][j]);
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = DN_MFMA_B16(ah[i], bm[j], acc[i][j]);
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = DN_MFMA_B16(am[i], bh[j], acc[i][j]);
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = DN_MFMA_B16(ah[i], bl[j], acc[i][j]);
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = DN_MFMA_B16(al[i], bh[j], acc[i][j]);
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = DN_MFMA_B16(am[i], bm[j], acc[i][j]);
    }
  };
  // At the top of tile t: the planes hold tile t, and register stage (t + 1 + s) % STAGES holds
  // tile t + 1 + s for s = 0 ... STAGES - 1 (requested, maybe not arrived).
  fetch(0, 0);
  commit(0);
#pragma unroll
  for (int s = 0; s < STAGES; s++) fetch((1 + s) % STAGES, 1 + s);
  __syncthreads();
  for (int64_t t = 0; t < n_tiles; t += STAGES) {
#pragma unroll
    for (int u = 0; u < STAGES; u++) {
      if (t + u < n_tiles) {
        mfma_tile();
        __syncthreads();  // every wave is done with the planes
        commit((u + 1) % STAGES);
        fetch((u + 1) % STAGES, t + u + 1 + STAGES);
        __syncthreads();
      }
    }
  }
}

// The product of abt_mainloop for operands with the contraction index fast, on planes without
// padding (64 bytes per row: 48 KB for the six planes, so that three workgroups fit a CU): the
// four 16-byte pieces of a row are stored at piece ^ (row / 4 % 4), which spreads the sixteen rows
// that a 16-byte LDS read instruction takes at a time over all banks.  One tile travels in
// registers (a third workgroup per CU hides what a second stage would).
constexpr int ABT_LD64 = 64;
constexpr int ABT_PLANE64 = 128 * ABT_LD64;
constexpr int ABT_LDS64 = 6 * ABT_PLANE64;

__device__ __forceinline__ void abt_fetch_kfast(f32x4 (&r)[4], const float* __restrict__ src, int64_t ld, int64_t k0) {
  const int fr = threadIdx.x >> 3, fk = 4 * (threadIdx.x & 7);
#pragma unroll
  for (int q = 0; q < 4; q++) r[q] = *reinterpret_cast<const f32x4*>(src + (int64_t)(fr + 32 * q) * ld + k0 + fk);
}
__device__ __forceinline__ void abt_commit64(const f32x4 (&r)[4], unsigned char* planes) {
  const int fr = threadIdx.x >> 3, fk = 4 * (threadIdx.x & 7);
#pragma unroll
  for (int q = 0; q < 4; q++) {
    bf16x4 h, m, l;
    split3(r[q], h, m, l);
    const int row = fr + 32 * q;
    unsigned char* dst = planes + row * ABT_LD64 + (((fk >> 3) ^ ((row >> 2) & 3)) << 4) + 2 * (fk & 7);
    *reinterpret_cast<bf16x4*>(dst) = h;
    *reinterpret_cast<bf16x4*>(dst + ABT_PLANE64) = m;
    *reinterpret_cast<bf16x4*>(dst + 2 * ABT_PLANE64) = l;
  }
}

__device__ __forceinline__ void abt_mainloop64(const float* __restrict__ a_src, int64_t lda,
                                               const float* __restrict__ b_src, int64_t ldb, int n_tiles,
                                               unsigned char* ab, abt_acc16 (&acc)[2][2]) {
  if (n_tiles <= 0) return;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l32 = lane & 31, half = lane >> 5, wm = wave >> 1, wn = wave & 1;
  f32x4 oa[4], ob[4];
  auto fetch = [&](int t) {
    const int64_t k0 = (int64_t)(t < n_tiles ? t : n_tiles - 1) * ABT_KB;
    abt_fetch_kfast(oa, a_src, lda, k0);
    abt_fetch_kfast(ob, b_src, ldb, k0);
  };
  const int swz = (l32 >> 2) & 3;
  const unsigned char* a_row = ab + (64 * wm + l32) * ABT_LD64;
  const unsigned char* b_row = ab + 3 * ABT_PLANE64 + (64 * wn + l32) * ABT_LD64;
  auto mfma_tile = [&]() {
#pragma unroll
    for (int st = 0; st < 2; st++) {
      const int at = ((2 * st + half) ^ swz) << 4;
      bf16x8 ah[2], am[2], al[2], bh[2], bm[2], bl[2];
#pragma unroll
      for (int i = 0; i < 2; i++) {
        const unsigned char* pa = a_row + 32 * i * ABT_LD64 + at;
        ah[i] = *reinterpret_cast<const bf16x8*>(pa);
        am[i] = *reinterpret_cast<const bf16x8*>(pa + ABT_PLANE64);
        al[i] = *reinterpret_cast<const bf16x8*>(pa + 2 * ABT_PLANE64);
        const unsigned char* pb = b_row + 32 * i * ABT_LD64 + at;
        bh[i] = *reinterpret_cast<const bf16x8*>(pb);
        bm[i] = *reinterpret_cast<const bf16x8*>(pb + ABT_PLANE64);
        bl[i] = *reinterpret_cast<const bf16x8*>(pb + 2 * ABT_PLANE64);
      }
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = DN_MFMA_B16(ah[i], bh[j], acc[i][j]);
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = DN_MFMA_B16(ah[i], bm[j], acc[i][j]);
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = DN_MFMA_B16(am[i], bh[j], acc[i][j]);
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = DN_MFMA_B16(ah[i], bl[j], acc[i][j]);
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = DN_MFMA_B16(al[i], bh[j], acc[i][j]);
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = DN_MFMA_B16(am[i], bm[j], acc[i][j]);
    }
  };
  fetch(0);
  abt_commit64(oa, ab);
  abt_commit64(ob, ab + 3 * ABT_PLANE64);
  fetch(1);
  __syncthreads();
  for (int t = 0; t < n_tiles; t++) {
    mfma_tile();
    __syncthreads();
    abt_commit64(oa, ab);
    abt_commit64(ob, ab + 3 * ABT_PLANE64);
    fetch(t + 2);
    __syncthreads();
  }
}

// A diagonal tile of X^T X (128 columns of X against themselves) with the work that its symmetry
// leaves: of the 4 x 4 blocks of 32 x 32 only the ten with block row <= block column are formed,
// and a block on the diagonal needs four of the six partial products, because h^T m and m^T h
// (and h^T l, l^T h) are transposes of each other there:
//   G_bb = Q + P + P^T,  Q = h^T h + m^T m,  P = h^T m + h^T l.
// Waves 0 and 1 take the block pairs (0, 1) and (2, 3): the block between the two (six products)
// and the two diagonal blocks (Q and P apart, two products each): 14 matrix instructions per 16
// contraction elements.  Waves 2 and 3 take blocks (0, 2), (0, 3) and (1, 2), (1, 3): 12.  (All
// sixteen blocks with six products are 24 per wave.)  The operand tile is fetched, split and
// stored once; a block row of it serves as first and as second operand alike (both are read as
// [row][8 contraction elements per half wave]).
// acc: pair waves: [0] = block (p, p + 1), [1] = Q_p, [2] = P_p, [3] = Q_p+1, [4] = P_p+1 with
// p = 2 wave; the others: [0] = block (a, 2), [1] = block (a, 3) with a = wave - 2.
template <int STAGES>
__device__ __forceinline__ void gram_diag_mainloop(const float* __restrict__ src, int64_t ld,
                                                   int64_t first, int64_t stride, int64_t n_tiles,
                                                   unsigned char* ab, abt_acc16 (&acc)[5]) {
  static_assert(STAGES == 1 || STAGES == 2, "one or two tiles in registers");
  if (n_tiles <= 0) return;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l32 = lane & 31, half = lane >> 5;
  const bool pair = wave < 2;
  AbtOperand<true> oa[STAGES];
  auto fetch = [&](int s, int64_t t) {
    const int64_t k0 = (first + (t < n_tiles ? t : n_tiles - 1) * stride) * ABT_KB;
    oa[s].fetch(src, ld, k0);
  };
  const unsigned char* lane_at = ab + l32 * ABT_LD + 16 * half;
  const unsigned char* row_x = lane_at + 32 * (pair ? 2 * wave : wave - 2) * ABT_LD;
  const unsigned char* row_y = lane_at + 32 * (pair ? 2 * wave + 1 : 2) * ABT_LD;
  const unsigned char* row_w = lane_at + 32 * 3 * ABT_LD;
  auto planes = [&](const unsigned char* p, bf16x8& h, bf16x8& m, bf16x8& l) {
    h = *reinterpret_cast<const bf16x8*>(p);
    m = *reinterpret_cast<const bf16x8*>(p + ABT_PLANE);
    l = *reinterpret_cast<const bf16x8*>(p + 2 * ABT_PLANE);
  };
  auto mfma_tile = [&]() {
#pragma unroll
    for (int st = 0; st < 2; st++) {
      bf16x8 xh, xm, xl, yh, ym, yl;
      planes(row_x + 32 * st, xh, xm, xl);
      planes(row_y + 32 * st, yh, ym, yl);
      if (pair) {
        // the six products of the block between alternate with the eight of the diagonal blocks
        acc[0] = DN_MFMA_B16(xh, yh, acc[0]);
        acc[1] = DN_MFMA_B16(xh, xh, acc[1]);
        acc[0] = DN_MFMA_B16(xh, ym, acc[0]);
        acc[3] = DN_MFMA_B16(yh, yh, acc[3]);
        acc[0] = DN_MFMA_B16(xm, yh, acc[0]);
        acc[2] = DN_MFMA_B16(xh, xm, acc[2]);
        acc[0] = DN_MFMA_B16(xh, yl, acc[0]);
        acc[4] = DN_MFMA_B16(yh, ym, acc[4]);
        acc[0] = DN_MFMA_B16(xl, yh, acc[0]);
        acc[1] = DN_MFMA_B16(xm, xm, acc[1]);
        acc[0] = DN_MFMA_B16(xm, ym, acc[0]);
        acc[3] = DN_MFMA_B16(ym, ym, acc[3]);
        acc[2] = DN_MFMA_B16(xh, xl, acc[2]);
        acc[4] = DN_MFMA_B16(yh, yl, acc[4]);
      } else {
        bf16x8 wh, wm, wl;
        planes(row_w + 32 * st, wh, wm, wl);
        acc[0] = DN_MFMA_B16(xh, yh, acc[0]);
        acc[1] = DN_MFMA_B16(xh, wh, acc[1]);
        acc[0] = DN_MFMA_B16(xh, ym, acc[0]);
        acc[1] = DN_MFMA_B16(xh, wm, acc[1]);
        acc[0] = DN_MFMA_B16(xm, yh, acc[0]);
        acc[1] = DN_MFMA_B16(xm, wh, acc[1]);
        acc[0] = DN_MFMA_B16(xh, yl, acc[0]);
        acc[1] = DN_MFMA_B16(xh, wl, acc[1]);
        acc[0] = DN_MFMA_B16(xl, yh, acc[0]);
        acc[1] = DN_MFMA_B16(xl, wh, acc[1]);
        acc[0] = DN_MFMA_B16(xm, ym, acc[0]);
        acc[1] = DN_MFMA_B16(xm, wm, acc[1]);
      }
    }
  };
  fetch(0, 0);
  oa[0].commit(ab);
#pragma unroll
  for (int s = 0; s < STAGES; s++) fetch((1 + s) % STAGES, 1 + s);
  __syncthreads();
  for (int64_t t = 0; t < n_tiles; t += STAGES) {
#pragma unroll
    for (int u = 0; u < STAGES; u++) {
      if (t + u < n_tiles) {
        mfma_tile();
        __syncthreads();  // every wave is done with the planes
        oa[(u + 1) % STAGES].commit(ab);
        fetch((u + 1) % STAGES, t + u + 1 + STAGES);
        __syncthreads();
      }
    }
  }
}

// A diagonal square of 256 columns of X^T X in one workgroup of eight waves: the 8 x 8 blocks of
// 32 x 32 with the work the symmetry leaves, and every element of X fetched, split and stored
// once for all of them.  Wave w owns block row w of the operand tile as first operand and forms
//   the blocks (w, w + 1), (w, w + 2), (w, w + 3) (indices modulo 8; six products each),
//   the diagonal block (w, w) as Q and P apart (four products, see gram_diag_mainloop),
//   half of the block (w, w + 4): waves 0-3 the products h h, h m, m h, waves 4-7 (which hold the
//   block as (w, w - 4), the transpose) h l, l h, m m;
// 25 matrix instructions per 16 contraction elements and wave, where all 64 blocks with six
// products take 48.  The planes are kept twice: the next tile is stored while slower waves still
// read the current one, and one barrier per tile is enough.
// acc: [0..2] = blocks (w, w + 1 .. w + 3), [3] = Q, [4] = P, [5] = the half block.
constexpr int ABT_PLANE2 = 256 * ABT_LD;
constexpr int ABT_LDS_PAIR = 2 * 3 * ABT_PLANE2;

template <int STAGES>
__device__ __forceinline__ void gram_pair_mainloop(const float* __restrict__ src, int64_t ld,
                                                   int64_t first, int64_t stride, int64_t n_tiles,
                                                   unsigned char* ab, abt_acc16 (&acc)[6]) {
  static_assert(STAGES == 1 || STAGES == 2, "one or two tiles in registers");
  if (n_tiles <= 0) return;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l32 = lane & 31, half = lane >> 5;
  const bool low = wave < 4;
  AbtOperand<true> oa[STAGES];
  auto fetch = [&](int s, int64_t t) {
    const int64_t k0 = (first + (t < n_tiles ? t : n_tiles - 1) * stride) * ABT_KB;
    oa[s].fetch(src, ld, k0);
  };
  const int lane_at = l32 * ABT_LD + 16 * half;
  int row_at[5];
#pragma unroll
  for (int k = 0; k < 5; k++) row_at[k] = lane_at + 32 * ((wave + k) & 7) * ABT_LD;
  auto planes = [&](const unsigned char* p, bf16x8& h, bf16x8& m, bf16x8& l) {
    h = *reinterpret_cast<const bf16x8*>(p);
    m = *reinterpret_cast<const bf16x8*>(p + ABT_PLANE2);
    l = *reinterpret_cast<const bf16x8*>(p + 2 * ABT_PLANE2);
  };
  auto mfma_tile = [&](const unsigned char* buf) {
#pragma unroll
    for (int st = 0; st < 2; st++) {
      bf16x8 xh, xm, xl, yh, ym, yl;
      planes(buf + row_at[0] + 32 * st, xh, xm, xl);
      planes(buf + row_at[1] + 32 * st, yh, ym, yl);
      acc[0] = DN_MFMA_B16(xh, yh, acc[0]);
      acc[3] = DN_MFMA_B16(xh, xh, acc[3]);
      acc[0] = DN_MFMA_B16(xh, ym, acc[0]);
      acc[4] = DN_MFMA_B16(xh, xm, acc[4]);
      acc[0] = DN_MFMA_B16(xm, yh, acc[0]);
      acc[3] = DN_MFMA_B16(xm, xm, acc[3]);
      acc[0] = DN_MFMA_B16(xh, yl, acc[0]);
      acc[4] = DN_MFMA_B16(xh, xl, acc[4]);
      acc[0] = DN_MFMA_B16(xl, yh, acc[0]);
      acc[0] = DN_MFMA_B16(xm, ym, acc[0]);
#pragma unroll
      for (int k = 2; k < 4; k++) {
        planes(buf + row_at[k] + 32 * st, yh, ym, yl);
        acc[k - 1] = DN_MFMA_B16(xh, yh, acc[k - 1]);
        acc[k - 1] = DN_MFMA_B16(xh, ym, acc[k - 1]);
        acc[k - 1] = DN_MFMA_B16(xm, yh, acc[k - 1]);
        acc[k - 1] = DN_MFMA_B16(xh, yl, acc[k - 1]);
        acc[k - 1] = DN_MFMA_B16(xl, yh, acc[k - 1]);
        acc[k - 1] = DN_MFMA_B16(xm, ym, acc[k - 1]);
      }
      planes(buf + row_at[4] + 32 * st, yh, ym, yl);
      if (low) {
        acc[5] = DN_MFMA_B16(xh, yh, acc[5]);
        acc[5] = DN_MFMA_B16(xh, ym, acc[5]);
        acc[5] = DN_MFMA_B16(xm, yh, acc[5]);
      } else {
        acc[5] = DN_MFMA_B16(xh, yl, acc[5]);
        acc[5] = DN_MFMA_B16(xl, yh, acc[5]);
        acc[5] = DN_MFMA_B16(xm, ym, acc[5]);
      }
    }
  };
  // At the top of tile t: buffer t % 2 holds tile t, and register stage (t + 1 + s) % STAGES holds
  // tile t + 1 + s.  Buffer (t + 1) % 2 was last read for tile t - 1, before that tile's barrier.
  fetch(0, 0);
  oa[0].template commit<ABT_PLANE2>(ab);
#pragma unroll
  for (int s = 0; s < STAGES; s++) fetch((1 + s) % STAGES, 1 + s);
  __syncthreads();
  for (int64_t t = 0; t < n_tiles; t += STAGES) {
#pragma unroll
    for (int u = 0; u < STAGES; u++) {
      if (t + u < n_tiles) {
        const int cur = (int)((t + u) & 1);
        mfma_tile(ab + cur * (3 * ABT_PLANE2));
        oa[(u + 1) % STAGES].template commit<ABT_PLANE2>(ab + (cur ^ 1) * (3 * ABT_PLANE2));
        fetch((u + 1) % STAGES, t + u + 1 + STAGES);
        __syncthreads();
      }
    }
  }
}

}  // namespace dn
