// Sparse kernels: A H^T (row-major CSR, gather rows of H), A^T W (transposed
// CSR, gather rows of W, no atomics) and sparse x sparse -> dense for the
// fixed-H learner.  A wavefront owns one output row.  (index, value) pairs are
// streamed 64 at a time, one per lane, and handed out from registers.  When
// the rank is a multiple of 4 a gathered row is read as 16-byte pieces: r/4
// lanes cover one row, so a wave fetches 64/(r/4) rows with one instruction
// (two for r = 128) and keeps several such instructions in flight.  Other
// ranks use 4-byte loads, lane l holding components l, l+64, ...  All
// summation orders are fixed by the matrix structure, so results are
// reproducible run to run.
#include "dnpeff_internal.hpp"

#include <algorithm>
#include <cstdlib>
#include <type_traits>
#include <utility>

namespace dn {

__device__ inline int bcast_i(int v, int src_lane) { return __builtin_amdgcn_readlane(v, src_lane); }
__device__ inline float bcast_f(float v, int src_lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src_lane));
}

// ---------------------------------------------------------------------------
// Gatherers: acc += sum_{p in [p0, p1)} val[p] * X[idx[p], :], then store(dst).
// ---------------------------------------------------------------------------

// Any rank: lane l holds components l + 64 t; every entry is applied by the whole wave.
template <int VPL>
struct GatherDword {
  static constexpr int UNR = VPL <= 2 ? 8 : VPL <= 4 ? 4 : 2;
  float acc[VPL];
  bool ok[VPL];
  int lane;
  bool small = false;  // (unused here) X smaller than 4 GB

  // `width` components starting at the pointers given to run() and store()
  __device__ inline void init(int lane_, int width) {
    lane = lane_;
#pragma unroll
    for (int t = 0; t < VPL; t++) {
      ok[t] = lane + 64 * t < width;
      acc[t] = 0.0f;
    }
  }

  __device__ inline void run(const int32_t* __restrict__ idx, const float* __restrict__ val,
                             int64_t p0, int64_t p1, const float* __restrict__ X, int r) {
    for (int64_t p = p0; p < p1; p += 64) {
      const int cnt = (p1 - p) < 64 ? (int)(p1 - p) : 64;
      int my_i = 0;
      float my_v = 0.0f;
      if (lane < cnt) {
        my_i = idx[p + lane];
        my_v = val[p + lane];
      }
      int u = 0;
      for (; u + UNR <= cnt; u += UNR) {
        float h[UNR][VPL];
        float a[UNR];
#pragma unroll
        for (int q = 0; q < UNR; q++) {
          const float* x = X + (int64_t)bcast_i(my_i, u + q) * r + lane;
          a[q] = bcast_f(my_v, u + q);
#pragma unroll
          for (int t = 0; t < VPL; t++) h[q][t] = ok[t] ? x[64 * t] : 0.0f;
        }
#pragma unroll
        for (int q = 0; q < UNR; q++)
#pragma unroll
          for (int t = 0; t < VPL; t++) acc[t] = fmaf(a[q], h[q][t], acc[t]);
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

  __device__ inline void store(float* dst) const {
#pragma unroll
    for (int t = 0; t < VPL; t++)
      if (ok[t]) dst[lane + 64 * t] = acc[t];
  }
};

// Rank a multiple of 4.  LPR lanes cover one gathered row with 16-byte loads (T
// loads per lane when the row is wider than 64 such pieces); the wave's 64/LPR
// lane groups take the entries of a batch round-robin, so group g applies
// entries g, g + G, g + 2G, ... in order, and the groups are added at the end in
// a fixed butterfly order.  FULL: the width is 4 LPR T, every lane holds components and the
// loads need no predicates.
template <int LPR, int T, bool FULL = false>
struct GatherVec4 {
  static constexpr int G = 64 / LPR;
  static constexpr int UNR = T >= 4 ? 1 : T == 2 ? 2 : 4;
  float4 acc[T];
  bool ok[T];
  int lane, sub, grp;
  bool small = false;  // X smaller than 4 GB: 32-bit row offsets

  // `width` components starting at the pointers given to run() and store()
  __device__ inline void init(int lane_, int width) {
    lane = lane_;
    sub = lane % LPR;
    grp = lane / LPR;
#pragma unroll
    for (int t = 0; t < T; t++) {
      ok[t] = FULL || 4 * (sub + 64 * t) < width;
      acc[t] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
  }

  __device__ inline void run(const int32_t* __restrict__ idx, const float* __restrict__ val,
                             int64_t p0, int64_t p1, const float* __restrict__ X, int r) {
    for (int64_t p = p0; p < p1; p += 64) {
      const int cnt = (p1 - p) < 64 ? (int)(p1 - p) : 64;
      int my_i = 0;
      float my_v = 0.0f;
      if (lane < cnt) {
        my_i = idx[p + lane];
        my_v = val[p + lane];
      }
      // Lanes past the batch hold (row 0, value 0): a padded step gathers row 0 with weight 0,
      // so the steps need no predicates.  Row offsets are 32-bit when X is smaller than 4 GB
      // (one multiply-add per gathered row).
      const int nsteps = (cnt + G - 1) / G;
      for (int q = 0; q < nsteps; q += UNR) {
        float4 h[UNR][T];
        float a[UNR];
#pragma unroll
        for (int uu = 0; uu < UNR; uu++) {
          const int u = ((q + uu) * G + grp) & 63;
          const int j = __shfl(my_i, u);
          a[uu] = __shfl(my_v, u);
          const float* x = small ? X + ((unsigned)j * (unsigned)r + 4u * (unsigned)sub)
                                 : X + (int64_t)j * r + 4 * sub;
#pragma unroll
          for (int t = 0; t < T; t++)
            h[uu][t] = FULL || ok[t] ? *reinterpret_cast<const float4*>(x + 256 * t)
                                     : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
#pragma unroll
        for (int uu = 0; uu < UNR; uu++)
#pragma unroll
          for (int t = 0; t < T; t++) {
            acc[t].x = fmaf(a[uu], h[uu][t].x, acc[t].x);
            acc[t].y = fmaf(a[uu], h[uu][t].y, acc[t].y);
            acc[t].z = fmaf(a[uu], h[uu][t].z, acc[t].z);
            acc[t].w = fmaf(a[uu], h[uu][t].w, acc[t].w);
          }
      }
    }
  }

  __device__ inline void store(float* dst) {
#pragma unroll
    for (int off = 32; off >= LPR; off >>= 1) {
#pragma unroll
      for (int t = 0; t < T; t++) {
        acc[t].x += __shfl_xor(acc[t].x, off);
        acc[t].y += __shfl_xor(acc[t].y, off);
        acc[t].z += __shfl_xor(acc[t].z, off);
        acc[t].w += __shfl_xor(acc[t].w, off);
      }
    }
    if (grp == 0) {
#pragma unroll
      for (int t = 0; t < T; t++)
        if (FULL || ok[t]) *reinterpret_cast<float4*>(dst + 4 * (sub + 64 * t)) = acc[t];
    }
  }
};

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

constexpr int MAX_RANK = 1024;

// ---------------------------------------------------------------------------
// partials[chunk, :] = sum over the chunk's entries of val * H[col, :]
// A workgroup owns SPMM_N_CHUNK consecutive entries of one row; its 4 waves
// take a quarter each and are combined in wave order.
// ---------------------------------------------------------------------------
template <class GT>
__global__ void __launch_bounds__(256)
    k_spmm_n(const int64_t* __restrict__ rowptr, const int32_t* __restrict__ colind,
             const float* __restrict__ vals, const int64_t* __restrict__ chunk_base, int64_t n_rows,
             int r, const float* __restrict__ H, float* __restrict__ partials) {
  extern __shared__ __align__(16) float red_dyn[];  // [4][r]
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

  GT g;
  g.init(lane, r);
  g.run(colind, vals, w0, w1, H, r);
  g.store(red_dyn + wave * r);
  __syncthreads();
  for (int c = threadIdx.x; c < r; c += 256) {
    float s = red_dyn[c];
    s += red_dyn[r + c];
    s += red_dyn[2 * r + c];
    s += red_dyn[3 * r + c];
    partials[chunk * r + c] = s;
  }
}

// One wave per row, the whole row: the plain row-per-wavefront decomposition, kept for the
// comparison of work decompositions on ragged rows (a long row then holds its wave for as long
// as its length says, while the waves of short rows have long finished).
template <class GT>
__global__ void __launch_bounds__(256)
    k_spmm_n_rowwave(const int64_t* __restrict__ rowptr, const int32_t* __restrict__ colind,
                     const float* __restrict__ vals, int64_t n_rows, int r,
                     const float* __restrict__ H, float* __restrict__ N) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;
  if (row >= n_rows) return;
  GT g;
  g.init(lane, r);
  g.run(colind, vals, rowptr[row], rowptr[row + 1], H, r);
  g.store(N + row * r);
}

// ---------------------------------------------------------------------------
// Merge-path decomposition, for the comparison of work decompositions on ragged rows: the path
// that consumes, row by row, a row's entries and then its end marker has nnz + n_rows steps; every
// wave takes MERGE_SHARE consecutive steps of it, wherever the row boundaries fall (a long row is
// cut over many waves, many short rows share one).  Diagonal d of the path lies at (rows closed,
// entries consumed) = (i, d - i) with i = the number of rows whose end marker, at step
// rowptr[i + 1] + i, comes before d.  A row that starts and ends inside a share is stored directly;
// the share's sums for the row that was open when it began / that stays open when it ends go to
// carry[share][0] / [1] and k_merge_fixup adds a row's carries in share order.
// ---------------------------------------------------------------------------
constexpr int64_t MERGE_SHARE = 4096;

__device__ inline int64_t merge_rows_closed(const int64_t* __restrict__ rowptr, int64_t n_rows, int64_t d) {
  int64_t lo = 0, hi = n_rows;  // number of i in [0, n_rows) with rowptr[i + 1] + i < d
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (rowptr[mid + 1] + mid < d) lo = mid + 1; else hi = mid;
  }
  return lo;
}

template <class GT>
__global__ void __launch_bounds__(256)
    k_spmm_n_merge(const int64_t* __restrict__ rowptr, const int32_t* __restrict__ colind,
                   const float* __restrict__ vals, int64_t n_rows, int64_t n_shares, int r,
                   const float* __restrict__ H, float* __restrict__ N, float* __restrict__ carry) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int64_t share = (int64_t)blockIdx.x * 4 + wave;
  if (share >= n_shares) return;
  const int64_t total = rowptr[n_rows] + n_rows;
  const int64_t d0 = share * MERGE_SHARE, d1 = d0 + MERGE_SHARE < total ? d0 + MERGE_SHARE : total;
  const int64_t i0 = merge_rows_closed(rowptr, n_rows, d0), i1 = merge_rows_closed(rowptr, n_rows, d1);
  const int64_t e0 = d0 - i0, e1 = d1 - i1;
  for (int64_t i = i0; i <= i1 && i < n_rows; i++) {
    const int64_t r0 = rowptr[i], r1 = rowptr[i + 1];
    const int64_t a = r0 > e0 ? r0 : e0, b = r1 < e1 ? r1 : e1;
    const bool opened_before = r0 < e0, closes_here = i < i1;
    if (i == i1 && !opened_before && b <= a && r0 >= e1) break;  // the next share's row: nothing of it here
    GT g;
    g.init(lane, r);
    g.run(colind, vals, a, b > a ? b : a, H, r);
    if (!opened_before && closes_here) g.store(N + i * r);
    else g.store(carry + (share * 2 + (opened_before ? 0 : 1)) * r);
  }
}

// N[row, :] of the rows that span several shares: the tail carry of the share where the row
// starts, then the head carries of the following shares up to the one with its end marker.
__global__ void __launch_bounds__(256)
    k_merge_fixup(const int64_t* __restrict__ rowptr, int64_t n_rows, int r, const float* __restrict__ carry,
                  float* __restrict__ N) {
  for (int64_t i = blockIdx.x; i < n_rows; i += gridDim.x) {
    const int64_t sa = (rowptr[i] + i) / MERGE_SHARE, sb = (rowptr[i + 1] + i) / MERGE_SHARE;
    if (sa == sb) continue;
    // (a row whose first step is the first step of share sa was not open before it)
    for (int c = threadIdx.x; c < r; c += 256) {
      float s = carry[(sa * 2 + 1) * r + c];
      for (int64_t sh = sa + 1; sh <= sb; sh++) s += carry[(sh * 2) * r + c];
      N[i * r + c] = s;
    }
  }
}

// ---------------------------------------------------------------------------
// Column panels.  When H is far larger than the caches, every gathered row of H comes from
// HBM unless the workgroups running at one time gather from the same part of H.  The entries of
// each row are therefore regrouped by column panel (same panels for all rows, equal numbers of
// entries per panel over the whole matrix), a wave owns one (row, panel) segment and the grid
// runs panel by panel: the rows of H of a panel are fetched from HBM once and then found in
// L2 / the memory-side cache by the other rows' segments.
// part[row, panel, :] = sum over the segment's entries of val * H[col, :]
// ---------------------------------------------------------------------------
template <class GT>
__global__ void __launch_bounds__(256)
    k_spmm_n_panel(const int64_t* __restrict__ seg, const int32_t* __restrict__ pcol,
                   const float* __restrict__ pval, int64_t n_rows, int64_t row_groups, int P,
                   const int32_t* __restrict__ ids, int slots, int r, const float* __restrict__ H,
                   float* __restrict__ part) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int64_t slot = blockIdx.x / row_groups;
  const int64_t row = (blockIdx.x % row_groups) * 4 + wave;
  if (row >= n_rows) return;
  const int64_t* sg = seg + row * (P + 1) + ids[slot];
  GT g;
  g.init(lane, r);
  g.run(pcol, pval, sg[0], sg[1], H, r);
  g.store(part + (row * slots + slot) * r);
}

// ---------------------------------------------------------------------------
// Swept panels.  Where a coarse panel's part of H is larger than an L2 and its columns still
// hold several entries each, the panel is cut into pieces that fit the 4 MB L2 of one XCD, and
// XCD x (workgroups x, x + 8, ... : the dispatcher deals workgroups to the XCDs round-robin)
// takes pieces x, x + 8, ... one after the other, for all rows of a pass: the rows of H of a
// piece then come from that XCD's L2 for every row after the first that uses them.
//
// All workgroups of the grid are resident at once (two per CU) and a workgroup keeps the running
// sums of its rows in LDS for the whole sweep, so nothing is written until the end of the pass.
// A wave owns the rows i * waves + wave of its workgroup and handles their (row, piece) segments
// one after the other: LPR = r / 4 lanes gather one row of H with 16-byte loads, the 64 / LPR
// lane groups take the entries of the segment round-robin and are added in a fixed butterfly
// order before the segment's sum goes to LDS.  The (column, value) pairs of a segment are
// requested two segments ahead, after the first gathers of a segment have been summed, and the
// segment bounds of a piece two pieces ahead, at the end of a piece (before the wait for the
// other workgroups): loads return in order, so a request from HBM placed before gathers holds
// their results up.  Rows of H are addressed as the piece's first row plus a 32-bit offset (one
// 24-bit multiply-add per gathered row), the pairs as a uniform base plus the lane.
//
// The workgroups of an XCD keep within `lag` pieces of each other: workgroups that ran ahead
// (their rows hold fewer entries) would otherwise widen the part of H in use beyond the L2.
// Each workgroup counts its finished pieces into a per-XCD counter and starts piece i only when
// the count says that all have finished piece i - 1 - lag.  The counter is only used by
// workgroups of one XCD, which share an L2, so it is bumped and polled with L2 atomics of
// workgroup scope (device scope costs a trip to the memory side per poll).  The wait is bounded
// (spin_max polls) and the first wait that runs out ends all later ones on that XCD (such a
// workgroup adds SWEEP_GIVE_UP = 2^22, far above any count waited for; the few workgroups that
// run out together each add it once: the grid has 64 per XCD), so a grid that is not resident
// as a whole loses the lock step but not much time, and the sums do not depend on the counter.
// One partial sum per (row, XCD): part[row, slot0 + x, :].
// ---------------------------------------------------------------------------
// Every lane of a row of 16 lanes reads lane K of that row (DPP row_newbcast).
template <int K>
__device__ inline int row_bcast(int v) {
  return __builtin_amdgcn_update_dpp(0, v, 0x150 + K, 0xf, 0xf, true);
}
// f(integral_constant<int, I>) for I = 0 .. n - 1, unrolled at compile time
template <class F, int... I>
__device__ inline void each_step(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}

constexpr int SWEEP_SYNC_STRIDE = 32;    // ints between the progress counters of two XCDs
constexpr int SWEEP_LDS_BYTES = 81920;   // running sums of a workgroup: half the LDS of a CU
constexpr int SWEEP_MAX_SEGS = 32;       // rows per wave (their offsets live in the 64 lanes)
constexpr int SWEEP_GIVE_UP = 1 << 22;   // added to a progress counter: every later wait ends at once

template <int LPR, bool A16>
__global__ void __launch_bounds__(1024)
    k_spmm_n_sweep(const int64_t* __restrict__ seg, const int32_t* __restrict__ pcol,
                   const float* __restrict__ pval, int64_t row0, int64_t row1, int P,
                   const int32_t* __restrict__ swept, int n_swept,
                   const int32_t* __restrict__ bounds_of, int slots, int slot0, int r, int stride,
                   const float* __restrict__ H, float* __restrict__ part,
                   int* __restrict__ progress, int lag, int spin_max, int rows_wg,
                   const int32_t* __restrict__ perm) {
  // [row0, row1) are positions in perm, the list of rows dealt so that every wave's rows hold
  // about the same number of entries (rows of very different lengths would otherwise make the
  // waves of a piece wait for the one with the longest rows).
  // r: components that this launch sums (4 LPR); stride: floats between two rows of H and of
  // the partial sums (the rank; r < stride for a launch on a slice of the components, whose H and
  // part pointers then start at the slice's first component)
  extern __shared__ __align__(16) float sums[];  // [rows_wg][r], row l = i * waves + wave
  constexpr int G = 64 / LPR;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int waves = blockDim.x >> 6;
  const int sub = lane % LPR, grp = lane / LPR;
  const int x = blockIdx.x % SWEEP_XCDS;
  const int64_t q = blockIdx.x / SWEEP_XCDS, nq = gridDim.x / SWEEP_XCDS;
  int* const counter = progress + x * SWEEP_SYNC_STRIDE;
  const int n_pi = (n_swept - x + SWEEP_XCDS - 1) / SWEEP_XCDS;  // pieces of this XCD
  auto pos_of = [&](int i) { return row0 + ((int64_t)i * waves + wave) * nq + q; };
  // rows of this wave: those with i * waves + wave < rows_wg (at least two, at most 32)
  const int n_i = (rows_wg - wave + waves - 1) / waves;

  for (int i = 0; i < n_i; i++)
    for (int c = lane; c < r; c += 64) sums[(size_t)(i * waves + wave) * r + c] = 0.0f;

  // Segment bounds live in the lanes: lane i holds the first pair and the length of the
  // (row_i, piece) segment of the current piece, lane 32 + i those of the next piece; a third
  // set (in the upper lanes of `st_*`) is on its way for the piece after that.  Lanes without a
  // row and pieces past the end hold empty segments.
  const int64_t my_pos = pos_of(lane & 31);
  const bool my_seg = (lane & 31) < n_i && my_pos < row1;
  const int64_t my_row = my_seg ? perm[my_pos] : 0;
  auto load_off = [&](int pi, int64_t& s0, int& len) {
    const bool ok = my_seg && pi < n_pi;
    const int piece = swept[x + SWEEP_XCDS * (pi < n_pi ? pi : 0)];
    const int64_t at = ok ? my_row * (P + 1) + piece : 0;
    const int64_t a = seg[at], b = seg[at + 1];
    s0 = ok ? a : 0;
    len = ok ? (int)(b - a) : 0;
  };
  auto bcast_i64 = [&](int64_t v, int src) {
    const int lo = (int)(uint32_t)(v & 0xffffffffLL), hi = (int)(v >> 32);
    return ((int64_t)bcast_i(hi, src) << 32) | (uint32_t)bcast_i(lo, src);
  };
  const unsigned r4 = 4u * (unsigned)stride, sub16 = 16u * (unsigned)sub;

  if (n_pi > 0) {  // (n_pi is the same for all waves of the workgroup)
    int64_t cm_s0, st_s0;
    int cm_len, st_len;
    {
      int64_t s0a, s0b;
      int lena, lenb;
      load_off(0, s0a, lena);
      load_off(1, s0b, lenb);
      cm_s0 = lane < 32 ? s0a : s0b;
      cm_len = lane < 32 ? lena : lenb;
      load_off(2, st_s0, st_len);
    }
    int pi = 0, i = 0;
    // rows of H of the current piece: Hp + 4 r (column - c0), a 32-bit offset
    int c0 = bounds_of[swept[x]];
    const char* Hp = reinterpret_cast<const char*>(H + (int64_t)c0 * stride);
    int ra_i, rb_i;
    float ra_v, rb_v;
    ra_i = (pcol + bcast_i64(cm_s0, 0))[lane];
    ra_v = (pval + bcast_i64(cm_s0, 0))[lane];
    rb_i = (pcol + bcast_i64(cm_s0, 1))[lane];  // (a wave owns at least two rows)
    rb_v = (pval + bcast_i64(cm_s0, 1))[lane];
    // One segment: (ri, rv) hold its first 64 pairs (and whatever follows them in memory: the
    // arrays end with 64 spare pairs) and are refilled with those of the segment after the next.
    auto segment = [&](int& ri, float& rv) {
      if (i == 0 && pi > lag) {
        if (threadIdx.x == 0) {
          const int want = (int)nq * (pi - lag);
          int spin = 0;
          for (; spin < spin_max; spin++) {
            // an L2 atomic that changes nothing (the counter is never negative) reads the counter
            if (__hip_atomic_fetch_max(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) >=
                want)
              break;
            __builtin_amdgcn_s_sleep(8);
          }
          // waited in vain (part of the grid is not running): nobody on this XCD waits again
          if (spin == spin_max)
            __hip_atomic_fetch_add(counter, SWEEP_GIVE_UP, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_WORKGROUP);
        }
        __syncthreads();
      }
      const int64_t s0 = bcast_i64(cm_s0, i);
      const int len = bcast_i(cm_len, i);
      // the segment after the next: two rows on, possibly in the next piece
      const int l2 = i + 2 < n_i ? i + 2 : 32 + i + 2 - n_i;
      const int32_t* pc2 = pcol + bcast_i64(cm_s0, l2);
      const float* pv2 = pval + bcast_i64(cm_s0, l2);

      float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      // lanes past the segment hold (first row of the piece, value 0): a padded step gathers
      // that row with weight 0
      int my_i = lane < len ? ri - c0 : 0;
      float my_v = lane < len ? rv : 0.0f;
      auto gather_at = [&](int j) -> float4 {
        const unsigned at = __umul24((unsigned)j, r4) + sub16;
        const float* hx = reinterpret_cast<const float*>(Hp + at);
        if (A16) return *reinterpret_cast<const float4*>(hx);
        return make_float4(hx[0], hx[1], hx[2], hx[3]);
      };
      auto sums_up = [&](auto u_tag, const float4* h, const float* a) {
        constexpr int U = decltype(u_tag)::value;
#pragma unroll
        for (int uu = 0; uu < U; uu++) {
          acc.x = fmaf(a[uu], h[uu].x, acc.x);
          acc.y = fmaf(a[uu], h[uu].y, acc.y);
          acc.z = fmaf(a[uu], h[uu].z, acc.z);
          acc.w = fmaf(a[uu], h[uu].w, acc.w);
        }
      };
      using U2 = std::integral_constant<int, 2>;
      using U4 = std::integral_constant<int, 4>;
      if constexpr (LPR >= 16) {
        // A lane group is one or more rows of 16 lanes.  One shuffle per 16 steps puts the pair
        // of step 16 s + k of a lane's group into lane k of its row; each step then takes its
        // pair with a row broadcast (a DPP operand, no LDS traffic): shuffles through the LDS
        // crossbar for every step kept that pipe busy 68 % of the time.
        const int row_lane = (lane & 15) * G + grp;
        auto arrange = [&](int s, int& ai, float& av) {
          const int src = (16 * G * s + row_lane) & 63;
          ai = __shfl(my_i, src);
          av = __shfl(my_v, src);
        };
        auto chunk = [&](auto st_tag, auto u_tag, int ai, float av) {
          constexpr int ST = decltype(st_tag)::value;
          constexpr int U = decltype(u_tag)::value;
          float4 h[U];
          float a[U];
          each_step(std::make_integer_sequence<int, U>{}, [&](auto uu_tag) {
            constexpr int uu = decltype(uu_tag)::value;
            a[uu] = __int_as_float(row_bcast<ST + uu>(__float_as_int(av)));
            h[uu] = gather_at(row_bcast<ST + uu>(ai));
          });
          sums_up(u_tag, h, a);
        };
        auto from = [&](auto st_tag, int n_s, int ai, float av) {  // steps ST .. of a sub-batch
          constexpr int ST = decltype(st_tag)::value;
          if (n_s - ST > 2) chunk(st_tag, U4{}, ai, av);
          else chunk(st_tag, U2{}, ai, av);
        };
        auto after_first = [&](int n_s, int ai, float av) {
          if (n_s > 4) from(std::integral_constant<int, 4>{}, n_s, ai, av);
          if (n_s > 8) from(std::integral_constant<int, 8>{}, n_s, ai, av);
          if (n_s > 12) from(std::integral_constant<int, 12>{}, n_s, ai, av);
        };
        int n_b = ((len < 64 ? len : 64) + G - 1) / G;  // steps of the batch
        int ai;
        float av;
        arrange(0, ai, av);
        // the first gathers of the segment and their sums (an empty segment gathers the piece's
        // first row twice with weight 0), then the request for the segment after the next
        from(std::integral_constant<int, 0>{}, n_b < 16 ? n_b : 16, ai, av);
        ri = pc2[lane];
        rv = pv2[lane];
        after_first(n_b < 16 ? n_b : 16, ai, av);
        for (int base = 0; base < len; base += 64) {
          if (base > 0) {
            my_i = (pcol + s0)[base + lane];
            my_v = (pval + s0)[base + lane];
            my_i = base + lane < len ? my_i - c0 : 0;
            my_v = base + lane < len ? my_v : 0.0f;
            n_b = ((len - base < 64 ? len - base : 64) + G - 1) / G;
          }
          for (int sb = base > 0 ? 0 : 1; 16 * sb < n_b; sb++) {
            const int n_s = n_b - 16 * sb < 16 ? n_b - 16 * sb : 16;
            arrange(sb, ai, av);
            from(std::integral_constant<int, 0>{}, n_s, ai, av);
            after_first(n_s, ai, av);
          }
        }
      } else {
        auto gathers = [&](auto u_tag, int st, float4* h, float* a) {
          constexpr int U = decltype(u_tag)::value;
#pragma unroll
          for (int uu = 0; uu < U; uu++) {
            const int u = ((st + uu) * G + grp) & 63;
            a[uu] = __shfl(my_v, u);
            h[uu] = gather_at(__shfl(my_i, u));
          }
        };
        // the first gathers of the segment and their sums, then the request for the segment
        // after the next
        int nsteps = ((len < 64 ? len : 64) + G - 1) / G;
        int st;
        if (nsteps > 2) {
          float4 h[4];
          float a[4];
          gathers(U4{}, 0, h, a);
          sums_up(U4{}, h, a);
          st = 4;
        } else {
          float4 h[2];
          float a[2];
          gathers(U2{}, 0, h, a);
          sums_up(U2{}, h, a);
          st = 2;
        }
        ri = pc2[lane];
        rv = pv2[lane];
        for (int base = 0; base < len; base += 64) {
          if (base > 0) {
            my_i = (pcol + s0)[base + lane];
            my_v = (pval + s0)[base + lane];
            my_i = base + lane < len ? my_i - c0 : 0;
            my_v = base + lane < len ? my_v : 0.0f;
            nsteps = ((len - base < 64 ? len - base : 64) + G - 1) / G;
            st = 0;
          }
          while (st < nsteps) {
            if (nsteps - st > 2) {
              float4 h[4];
              float a[4];
              gathers(U4{}, st, h, a);
              sums_up(U4{}, h, a);
              st += 4;
            } else {
              float4 h[2];
              float a[2];
              gathers(U2{}, st, h, a);
              sums_up(U2{}, h, a);
              st += 2;
            }
          }
        }
      }
      if (len > 0) {
#pragma unroll
        for (int off = 32; off >= LPR; off >>= 1) {
          acc.x += __shfl_xor(acc.x, off);
          acc.y += __shfl_xor(acc.y, off);
          acc.z += __shfl_xor(acc.z, off);
          acc.w += __shfl_xor(acc.w, off);
        }
        if (grp == 0) {
          float4* dst = reinterpret_cast<float4*>(sums + (size_t)(i * waves + wave) * r) + sub;
          float4 t = *dst;
          t.x += acc.x; t.y += acc.y; t.z += acc.z; t.w += acc.w;
          *dst = t;
        }
      }
      if (++i == n_i) {  // the piece is done
        // bounds: the next piece moves to the lower lanes, the one after it to the upper lanes,
        // and the request for a further one goes out before the wait for the other workgroups
        const int64_t lo_s0 = (int64_t)(((uint64_t)(uint32_t)__shfl((int)(cm_s0 >> 32), lane + 32) << 32) |
                                        (uint32_t)__shfl((int)(uint32_t)(cm_s0 & 0xffffffffLL), lane + 32));
        const int lo_len = __shfl(cm_len, lane + 32);
        cm_s0 = lane < 32 ? lo_s0 : st_s0;
        cm_len = lane < 32 ? lo_len : st_len;
        i = 0;
        pi++;
        load_off(pi + 2, st_s0, st_len);
        c0 = bounds_of[swept[x + SWEEP_XCDS * (pi < n_pi ? pi : 0)]];
        Hp = reinterpret_cast<const char*>(H + (int64_t)c0 * stride);
        __syncthreads();
        if (threadIdx.x == 0)
          __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
    };
    const int total = n_pi * n_i;
    for (int t = 0; t < total; t += 2) {
      segment(ra_i, ra_v);
      if (t + 1 < total) segment(rb_i, rb_v);
    }
  }

  for (int i = 0; i < n_i; i++) {
    const int64_t pos = pos_of(i);
    if (pos < row1) {
      const int64_t row = perm[pos];
      const float* src = sums + (size_t)(i * waves + wave) * r;
      float* dst = part + (row * slots + slot0 + x) * stride;
      for (int c = lane; c < r; c += 64) dst[c] = src[c];
    }
  }
}

// N[row, :] = sum of the row's panel partials, in panel order, accumulated in fp64.
__global__ void __launch_bounds__(256)
    k_panel_reduce(const float* __restrict__ part, int64_t n_rows, int P, int r,
                   float* __restrict__ N) {
  const int64_t total = n_rows * r, stride = (int64_t)gridDim.x * 256;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += stride) {
    const int64_t row = e / r;
    const int c = (int)(e % r);
    const float* src = part + row * P * r + c;
    double s = 0.0;
    for (int p = 0; p < P; p++) s += (double)src[(int64_t)p * r];
    N[e] = (float)s;
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
//
// The r components are cut into n_slices equal slices and workgroup b works on
// slice b % n_slices.  Workgroups are handed to the 8 XCDs round-robin, so each
// XCD only ever gathers from its own slice of W and that slice (n * r / n_slices
// floats) stays in the XCD's 4 MB L2 instead of being evicted by the other half.
// ---------------------------------------------------------------------------
template <class GT>
__global__ void __launch_bounds__(256)
    k_spmm_t_short(const int64_t* __restrict__ colptr, const int32_t* __restrict__ rowind,
                   const float* __restrict__ tvals, int64_t m, int r, int n_slices,
                   const float* __restrict__ W, float* __restrict__ T, bool w_small) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int slice = blockIdx.x % n_slices, width = r / n_slices;
  // gridDim.x is a multiple of n_slices: the slice of a workgroup never changes
  const int64_t group_stride = gridDim.x / n_slices;
  for (int64_t grp = blockIdx.x / n_slices; grp * 4 < m; grp += group_stride) {
    const int64_t j = grp * 4 + wave;
    if (j >= m) break;
    const int64_t p0 = colptr[j], p1 = colptr[j + 1];
    if (p1 - p0 > SPMM_T_LONG) continue;  // written by k_spmm_t_long
    GT g;
    g.init(lane, width);
    g.small = w_small;
    g.run(rowind, tvals, p0, p1, W + slice * width, r);
    g.store(T + j * r + slice * width);
  }
}

// Short and medium columns (at most SPMM_T_LONG entries), rank a multiple of 4: a wave owns
// SPMM_T_COLS consecutive columns and each of its 64/LPR lane groups walks whole columns on its
// own, so that a wave works on several columns at once, no cross-lane reduction is needed and
// the column offsets of all its columns come from one coalesced load.  A group reads up to LPR
// (row, value) pairs of its column with one load, hands them out with lane shuffles inside the
// group and gathers each W row with one 16-byte load per lane; entries are applied in order.
constexpr int SPMM_T_COLS = 32;

// FULL: r = 4 LPR T, every lane holds components (no predicates); SMALL: W has fewer than 2^24
// rows and 4 GB, a row is addressed as the (uniform) base of W plus a 32-bit offset made by one
// 24-bit multiply-add.
template <int LPR, int T, bool FULL, bool SMALL>
__global__ void __launch_bounds__(256)
    k_spmm_t_grouped(const int64_t* __restrict__ colptr, const int32_t* __restrict__ rowind,
                     const float* __restrict__ tvals, int64_t m, int r, int n_slices,
                     const float* __restrict__ W, float* __restrict__ Tout) {
  constexpr int G = 64 / LPR;
  constexpr int UNR = T >= 4 ? 1 : T == 2 ? 2 : 4;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int sub = lane % LPR, grp = lane / LPR, gbase = grp * LPR;
  // With component slices, workgroup b works on slice b % n_slices (4 LPR T components starting
  // at that multiple): the XCD it runs on gathers from its own slice of W only.
  const int slice = blockIdx.x % n_slices;
  W += slice * (4 * LPR * T);
  Tout += slice * (4 * LPR * T);
  const int64_t j0 = ((int64_t)(blockIdx.x / n_slices) * 4 + wave) * SPMM_T_COLS;
  if (j0 >= m) return;
  bool ok[T];
#pragma unroll
  for (int t = 0; t < T; t++) ok[t] = FULL || 4 * (sub + LPR * t) < r;
  const unsigned r4 = 4u * (unsigned)r, sub16 = 16u * (unsigned)sub;

  // colptr[j0 + lane] for lane <= SPMM_T_COLS, as two 32-bit halves for the shuffles
  const int64_t jc = j0 + lane < m ? j0 + lane : m;
  const int64_t cp = lane <= SPMM_T_COLS ? colptr[jc] : 0;
  const int cp_lo = (int)(uint32_t)(cp & 0xffffffffLL), cp_hi = (int)(cp >> 32);

  // The (row, value) pairs of a round's columns are requested one round ahead, so that their
  // latency overlaps the gathers of the round before: two dependent memory round trips per
  // column would otherwise bound the kernel.
  auto request = [&](int round, int64_t& p0, int& len, bool& active, int& e_i, float& e_v) {
    const int jl = round * G + grp;
    const int64_t j = j0 + jl;
    p0 = ((int64_t)__shfl(cp_hi, jl & 63) << 32) | (uint32_t)__shfl(cp_lo, jl & 63);
    const int64_t p1 =
        ((int64_t)__shfl(cp_hi, (jl + 1) & 63) << 32) | (uint32_t)__shfl(cp_lo, (jl + 1) & 63);
    active = jl < SPMM_T_COLS && j < m && (p1 - p0) <= SPMM_T_LONG;  // longer: k_spmm_t_long
    len = active ? (int)(p1 - p0) : 0;
    e_i = 0;
    e_v = 0.0f;
    if (sub < len) {
      e_i = rowind[p0 + sub];
      e_v = tvals[p0 + sub];
    }
  };
  int64_t nx_p0;
  int nx_len, nx_i;
  bool nx_active;
  float nx_v;
  request(0, nx_p0, nx_len, nx_active, nx_i, nx_v);

  for (int round = 0; round * G < SPMM_T_COLS; round++) {
    const int64_t j = j0 + round * G + grp;
    const int64_t p0 = nx_p0;
    const int len = nx_len;
    const bool active = nx_active;
    int my_i = nx_i;
    float my_v = nx_v;
    request(round + 1, nx_p0, nx_len, nx_active, nx_i, nx_v);
    float4 acc[T];
#pragma unroll
    for (int t = 0; t < T; t++) acc[t] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);

    for (int base = 0; __any(base < len); base += LPR) {
      if (base > 0) {  // columns longer than a lane group: further batches are loaded here
        const int e = base + sub;
        my_i = 0;
        my_v = 0.0f;
        if (e < len) {
          my_i = rowind[p0 + e];
          my_v = tvals[p0 + e];
        }
      }
      const int cnt = len - base;  // entries of this group in the batch (may be <= 0 or > LPR)
      // the wave walks to the largest count among its groups
      int cmax = 0;
#pragma unroll
      for (int g = 0; g < G; g++) {
        const int c = __builtin_amdgcn_readlane(cnt, g * LPR);
        cmax = c > cmax ? c : cmax;
      }
      if (cmax > LPR) cmax = LPR;
      // Whole blocks of UNR entries with their loads in flight together, then the rest one by
      // one: most columns hold one or two entries.  Lanes past a group's entries hold
      // (row 0, value 0), so a step that a shorter group only accompanies gathers row 0 with
      // weight 0 and needs no predicate.
      auto wrow = [&](int jrow) {
        if (SMALL)
          return reinterpret_cast<const float*>(reinterpret_cast<const char*>(W) +
                                                (__umul24((unsigned)jrow, r4) + sub16));
        return W + (int64_t)jrow * r + 4 * sub;
      };
      // U entries of every group with their gathers in flight together
      auto block = [&](auto u_tag, int u) {
        constexpr int U = decltype(u_tag)::value;
        float4 h[U][T];
        float a[U];
#pragma unroll
        for (int uu = 0; uu < U; uu++) {
          const float* x = wrow(__shfl(my_i, gbase + u + uu));
          a[uu] = __shfl(my_v, gbase + u + uu);
#pragma unroll
          for (int t = 0; t < T; t++)
            h[uu][t] = FULL || ok[t] ? *reinterpret_cast<const float4*>(x + 4 * LPR * t)
                                     : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
#pragma unroll
        for (int uu = 0; uu < U; uu++)
#pragma unroll
          for (int t = 0; t < T; t++) {
            acc[t].x = fmaf(a[uu], h[uu][t].x, acc[t].x);
            acc[t].y = fmaf(a[uu], h[uu][t].y, acc[t].y);
            acc[t].z = fmaf(a[uu], h[uu][t].z, acc[t].z);
            acc[t].w = fmaf(a[uu], h[uu][t].w, acc[t].w);
          }
      };
      int u = 0;
      for (; u + UNR <= cmax; u += UNR) block(std::integral_constant<int, UNR>{}, u);
      // what is left, also in one go: most columns hold one to three entries, and one at a time
      // each of them would wait for its own round trip
      if constexpr (UNR == 4) {
        if (cmax - u == 3) block(std::integral_constant<int, 3>{}, u);
        else if (cmax - u == 2) block(std::integral_constant<int, 2>{}, u);
        else if (cmax - u == 1) block(std::integral_constant<int, 1>{}, u);
      } else if constexpr (UNR == 2) {
        if (cmax - u == 1) block(std::integral_constant<int, 1>{}, u);
      }
    }
    if (active) {
#pragma unroll
      for (int t = 0; t < T; t++)
        if (FULL || ok[t]) *reinterpret_cast<float4*>(Tout + j * r + 4 * (sub + LPR * t)) = acc[t];
    }
  }
}

template <class GT>
__global__ void __launch_bounds__(256)
    k_spmm_t_long(const int32_t* __restrict__ long_cols, const int64_t* __restrict__ colptr,
                  const int32_t* __restrict__ rowind, const float* __restrict__ tvals, int r,
                  int n_slices, const float* __restrict__ W, float* __restrict__ T, bool w_small,
                  int64_t col0) {
  extern __shared__ __align__(16) float red_dyn[];  // [4][width]
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int slice = blockIdx.x % n_slices, width = r / n_slices;
  const int64_t j = long_cols[blockIdx.x / n_slices];
  const int64_t p0 = colptr[j], p1 = colptr[j + 1];
  const int64_t per = (((p1 - p0) + 3) / 4 + 63) / 64 * 64;  // quarter, rounded up to 64
  int64_t w0 = p0 + wave * per, w1 = w0 + per;
  if (w0 > p1) w0 = p1;
  if (w1 > p1) w1 = p1;
  GT g;
  g.init(lane, width);
  g.small = w_small;
  g.run(rowind, tvals, w0, w1, W + slice * width, r);
  g.store(red_dyn + wave * width);
  __syncthreads();
  for (int c = threadIdx.x; c < width; c += 256) {
    float s = red_dyn[c];
    s += red_dyn[width + c];
    s += red_dyn[2 * width + c];
    s += red_dyn[3 * width + c];
    T[(j - col0) * r + slice * width + c] = s;  // (T starts at column col0)
  }
}

// ---------------------------------------------------------------------------
// partials[chunk, :] = sum over the chunk's entries (j, a) of a * B[:, j] for a sparse B, a
// lane per entry.  B's transposed copy (per column j: component ids and values) is condensed
// into one 32-byte slot per column (its first four (component, value) pairs, the column's
// length in the upper half of the first component word), so that an entry of A costs one
// random sector instead of three dependent ones (column offsets, component ids, values); only
// columns longer than four go on to the transposed arrays.  Each wave keeps its r running sums
// in LDS and the lanes add into them with ds_add_f32: step k of a batch applies the k-th pair
// of all 64 entries at once, and where two lanes meet in a component the LDS adds them one
// after the other in lane order, the same way in every run.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
    k_spsp_build_slots(int64_t n_cols, const int64_t* __restrict__ colptr, const int32_t* __restrict__ comp,
                       const float* __restrict__ vals, uint4* __restrict__ slots) {
  const int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (j >= n_cols) return;
  const int64_t q0 = colptr[j];
  const int len = (int)(colptr[j + 1] - q0);
  unsigned w[8];
#pragma unroll
  for (int k = 0; k < 4; k++) {
    w[2 * k] = k < len ? (unsigned)comp[q0 + k] : 0u;
    w[2 * k + 1] = k < len ? __float_as_uint(vals[q0 + k]) : 0u;
  }
  w[0] |= (unsigned)len << 16;
  slots[2 * j] = make_uint4(w[0], w[1], w[2], w[3]);
  slots[2 * j + 1] = make_uint4(w[4], w[5], w[6], w[7]);
}

template <int VPL>
__global__ void __launch_bounds__(256)
    k_spsp_slots(const int64_t* __restrict__ rowptr, const int32_t* __restrict__ colind,
                 const float* __restrict__ vals, const int64_t* __restrict__ chunk_base, int64_t n_rows,
                 int r, const uint4* __restrict__ slots, const int64_t* __restrict__ b_colptr,
                 const int32_t* __restrict__ b_comp, const float* __restrict__ b_vals,
                 float* __restrict__ partials) {
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
    if (e + lane < w1) {
      const int32_t j = colind[e + lane];
      const float a = vals[e + lane];
      const uint4 s0 = slots[2 * (int64_t)j];
      const int len = (int)(s0.x >> 16);
      if (len > 0) atomicAdd(&acc[s0.x & 0xffffu], a * __uint_as_float(s0.y));
      if (len > 1) atomicAdd(&acc[s0.z], a * __uint_as_float(s0.w));
      if (len > 2) {
        const uint4 s1 = slots[2 * (int64_t)j + 1];
        atomicAdd(&acc[s1.x], a * __uint_as_float(s1.y));
        if (len > 3) atomicAdd(&acc[s1.z], a * __uint_as_float(s1.w));
        if (len > 4) {
          const int64_t q = b_colptr[j];
          for (int k = 4; k < len; k++) atomicAdd(&acc[b_comp[q + k]], a * b_vals[q + k]);
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

template <class T>
struct TypeTag {
  using type = T;
};

// Calls f(TypeTag<Gatherer>) with the gatherer that fits rank r and the alignment of X.
template <class F>
static int dispatch_gather(int r, bool aligned16, F&& f) {
  if (r % 4 == 0 && aligned16) {
    const int r4 = r / 4;
    if (r4 == 4) return f(TypeTag<GatherVec4<4, 1, true>>{});
    if (r4 == 8) return f(TypeTag<GatherVec4<8, 1, true>>{});
    if (r4 == 16) return f(TypeTag<GatherVec4<16, 1, true>>{});
    if (r4 == 32) return f(TypeTag<GatherVec4<32, 1, true>>{});
    if (r4 == 64) return f(TypeTag<GatherVec4<64, 1, true>>{});
    if (r4 == 128) return f(TypeTag<GatherVec4<64, 2, true>>{});
    if (r4 == 256) return f(TypeTag<GatherVec4<64, 4, true>>{});
    if (r4 <= 4) return f(TypeTag<GatherVec4<4, 1>>{});
    if (r4 <= 8) return f(TypeTag<GatherVec4<8, 1>>{});
    if (r4 <= 16) return f(TypeTag<GatherVec4<16, 1>>{});
    if (r4 <= 32) return f(TypeTag<GatherVec4<32, 1>>{});
    if (r4 <= 64) return f(TypeTag<GatherVec4<64, 1>>{});
    if (r4 <= 128) return f(TypeTag<GatherVec4<64, 2>>{});
    return f(TypeTag<GatherVec4<64, 4>>{});
  }
  switch (vpl_for(r)) {
    case 1: return f(TypeTag<GatherDword<1>>{});
    case 2: return f(TypeTag<GatherDword<2>>{});
    case 4: return f(TypeTag<GatherDword<4>>{});
    case 8: return f(TypeTag<GatherDword<8>>{});
    default: return f(TypeTag<GatherDword<16>>{});
  }
}

__global__ void k_sweep_clear(int* progress) { progress[threadIdx.x] = 0; }

// Shape of a sweep launch: two workgroups per CU, each with SWEEP_LDS_BYTES of running sums; the
// number of waves per workgroup is the largest (at most max_waves) that covers the rows in the
// fewest passes; DNPEFF_SWEEP_WAVES overrides it.  More rows than one launch covers take several
// passes of equal size.
struct sweep_shape {
  int waves, rows_wg;
  int64_t wgs, n_pass, rows_per_pass;
};
// max_waves: the most waves per workgroup that leave two workgroups resident per CU
static sweep_shape sweep_shape_for(int64_t n_rows, int r, int max_waves) {
  sweep_shape best{};
  const int64_t wgs = (int64_t)n_cus() * 2 / SWEEP_XCDS * SWEEP_XCDS;
  const int rows_cap = SWEEP_LDS_BYTES / (4 * r);
  int forced = (int)tuning().sweep_waves;
  if (forced < 1 || forced > max_waves) forced = 0;
  for (int waves = max_waves; waves >= 2; waves -= 2) {
    const int w = forced ? forced : waves;
    // every wave owns 2 to SWEEP_MAX_SEGS rows: the kernel looks two segments ahead within two
    // pieces and keeps the segment bounds of a piece in 32 lanes
    const int rows_wg = rows_cap < SWEEP_MAX_SEGS * w ? rows_cap : SWEEP_MAX_SEGS * w;
    if (rows_wg >= 2 * w) {
      const int64_t cover = wgs / SWEEP_XCDS * rows_wg;
      const int64_t n_pass = ceil_div(n_rows, cover);
      if (best.waves == 0 || n_pass < best.n_pass) best = sweep_shape{w, rows_wg, wgs, n_pass, 0};
    }
    if (forced) break;
  }
  best.rows_per_pass = ceil_div(n_rows, best.n_pass > 0 ? best.n_pass : 1);
  return best;
}

// Registers per SIMD lane that resident waves can share.  The file holds 512, but a launch of
// 8 waves per SIMD at 64 registers ran with 7 resident and one of 5 at 96 with 4 (the sweep's
// workgroups then wait for workgroups that have not started), so the shape is planned for 448.
constexpr int SWEEP_REGISTER_BUDGET = 448;

using sweep_kernel_t = void (*)(const int64_t*, const int32_t*, const float*, int64_t, int64_t, int,
                                const int32_t*, int, const int32_t*, int, int, int, int, const float*,
                                float*, int*, int, int, int, const int32_t*);

__global__ void __launch_bounds__(256)
    k_sweep_row_entries(const int64_t* __restrict__ seg, int64_t n_rows, int P, int64_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n_rows) out[i] = seg[i * (P + 1) + P] - seg[i * (P + 1)];
}

// The order in which the sweep kernel takes the rows: longest first, pass p takes every
// n_pass-th of them, and within a pass the rows go to the (workgroup, wave) slots back and forth
// (the slots of round i are the positions i * slots ... (i + 1) * slots - 1), so that the sums of
// the slots' row lengths come out close.  pass_start[p] = first position of pass p.
static int sweep_row_order(const dnpeff_csr* A, const sweep_shape& sh, std::vector<int64_t>& pass_start) {
  dnpeff_csr* M = const_cast<dnpeff_csr*>(A);
  const int64_t n = A->n_rows;
  const int64_t slots = (int64_t)sh.waves * (sh.wgs / SWEEP_XCDS);
  const int64_t key = (sh.n_pass << 32) ^ (slots << 8) ^ n;
  pass_start.assign(sh.n_pass + 1, 0);
  for (int64_t p = 0; p < sh.n_pass; p++)
    pass_start[p + 1] = pass_start[p] + (n - p + sh.n_pass - 1) / sh.n_pass;
  if (M->sweep_perm && M->sweep_perm_key == key) return 0;
  DN_HIP(hipStreamSynchronize(stream()));
  dfree(M->sweep_perm);
  M->sweep_perm = nullptr;
  dbuf<int64_t> counts;
  DN_TRY(counts.alloc(n));
  hipLaunchKernelGGL(k_sweep_row_entries, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, stream(), A->seg, n,
                     A->n_panels, counts.p);
  DN_LAUNCH_CHECK();
  std::vector<int64_t> h(n);
  DN_HIP(hipMemcpy(h.data(), counts.p, sizeof(int64_t) * n, hipMemcpyDeviceToHost));
  std::vector<int32_t> order(n), perm(n);
  for (int64_t i = 0; i < n; i++) order[i] = (int32_t)i;
  std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) { return h[a] > h[b]; });
  for (int64_t p = 0; p < sh.n_pass; p++) {
    const int64_t count = pass_start[p + 1] - pass_start[p];
    for (int64_t t = 0; t < count; t++) {
      const int64_t round = t / slots, first = round * slots;
      const int64_t in_round = count - first < slots ? count - first : slots;
      int64_t sl = t - first;
      if (round & 1) sl = in_round - 1 - sl;
      perm[pass_start[p] + first + sl] = order[p + t * sh.n_pass];
    }
  }
  DN_TRY(dmalloc(&M->sweep_perm, n));
  DN_HIP(hipMemcpy(M->sweep_perm, perm.data(), sizeof(int32_t) * n, hipMemcpyHostToDevice));
  M->sweep_perm_key = key;
  return 0;
}

// Ranks above 256 are swept in slices of 256 (or 128) components: one set of launches per slice,
// each with its slice of every row of H pinned in the L2s and its own running sums.
static int launch_spmm_n_sweep(const dnpeff_csr* A, int r, const float* H_mr, bool aligned,
                               int slots) {
  DN_CHECK(spmm_n_sweep_supported(r), "swept panels at rank %d", r);
  DN_CHECK(A->sweep_progress != nullptr, "matrix has no sweep counters");
  static const sweep_kernel_t kernels[8] = {
      k_spmm_n_sweep<8, false>,  k_spmm_n_sweep<8, true>,  k_spmm_n_sweep<16, false>,
      k_spmm_n_sweep<16, true>,  k_spmm_n_sweep<32, false>, k_spmm_n_sweep<32, true>,
      k_spmm_n_sweep<64, false>, k_spmm_n_sweep<64, true>};
  static int kernel_regs[8] = {0, 0, 0, 0, 0, 0, 0, 0};  // 0: attributes not yet set
  const int w = sweep_width(r);
  const int variant = (w == 32 ? 0 : w == 64 ? 2 : w == 128 ? 4 : 6) + (aligned ? 1 : 0);
  const sweep_kernel_t kernel = kernels[variant];
  if (kernel_regs[variant] == 0) {
    hipFuncAttributes attr;
    DN_HIP(hipFuncGetAttributes(&attr, (const void*)kernel));
    DN_HIP(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                               SWEEP_LDS_BYTES));
    kernel_regs[variant] = attr.numRegs > 0 ? attr.numRegs : 1;
  }
  const int regs = (kernel_regs[variant] + 7) / 8 * 8;
  // two workgroups per CU: a workgroup puts waves / 4 waves on each of the 4 SIMDs
  int max_waves = SWEEP_REGISTER_BUDGET / (regs > 0 ? regs : 8) * 4 / 2;
  if (max_waves > 14) max_waves = 14;
  max_waves &= ~1;
  DN_CHECK(max_waves >= 2, "the sweep kernel needs %d registers", kernel_regs[variant]);
  const sweep_shape sh = sweep_shape_for(A->n_rows, w, max_waves);
  DN_CHECK(sh.waves > 0, "no sweep shape for rank %d", r);
  static bool told = false;
  if (!told && tuning().verbose != 0.0) {
    told = true;
    fprintf(stderr,
            "dnpeff: sweep kernel with %d registers: %lld workgroups of %d waves, %d rows each, "
            "%lld pass(es) of %lld rows, %d slice(s) of %d components\n",
            kernel_regs[variant], (long long)sh.wgs, sh.waves, sh.rows_wg, (long long)sh.n_pass,
            (long long)sh.rows_per_pass, r / w, w);
  }
  std::vector<int64_t> pass_start;
  DN_TRY(sweep_row_order(A, sh, pass_start));
  const int32_t* swept = A->panel_ids + A->n_plain;
  int lag = (int)tuning().sweep_lag, spin_max = (int)tuning().sweep_spin;
  if (lag < 0) lag = 0;
  const size_t lds = sizeof(float) * (size_t)sh.rows_wg * w;
  for (int slice = 0; slice < r / w; slice++)
    for (int64_t pass = 0; pass < sh.n_pass; pass++) {
      const int64_t row0 = pass_start[pass], row1 = pass_start[pass + 1];
      hipLaunchKernelGGL(k_sweep_clear, dim3(1), dim3(SWEEP_XCDS * SWEEP_SYNC_STRIDE), 0, stream(),
                         A->sweep_progress);
      hipLaunchKernelGGL(kernel, dim3((unsigned)sh.wgs), dim3(64 * sh.waves), lds, stream(), A->seg,
                         A->pcol, A->pval, row0, row1, A->n_panels, swept, A->n_swept,
                         A->panel_bounds, slots, A->n_plain, w, r, H_mr + slice * w,
                         A->partials + slice * w, A->sweep_progress, lag, spin_max, sh.rows_wg,
                         A->sweep_perm);
      DN_LAUNCH_CHECK();
    }
  return 0;
}

// part: 0 = the whole product; 1 = what may run beside another kernel: the dense head, and the
// plain panels where they are the far tail (no slot lists: a long kernel that waits for the
// fabric); 2 = the rest (swept pieces and slot lists, whose workgroups walk in lock step and
// must all be resident; everything, where the product is not planned in panels).  1 then 2
// launch what 0 launches, in the same order.
int launch_spmm_n(const dnpeff_csr* A_full, int r, const float* H_mr, int part) {
  DN_CHECK(r >= 1 && r <= MAX_RANK, "rank %d outside [1, %d]", r, MAX_RANK);
  if (part != 2) DN_TRY(launch_head_n(A_full, r, H_mr));
  const dnpeff_csr* A = sparse_part(A_full);
  float* partials = A->partials;
  const bool planned = !(A->nl.pairs && use_nlists(A, r)) && A->n_panels > 0;
  if (part == 1 && !planned) return 0;
  if (A->nl.pairs && use_nlists(A, r)) {
    DN_CHECK(partials && A->partials_floats >= A->n_rows * (int64_t)r, "partial sums too small");
    return launch_spmm_n_lists(A, r, H_mr, partials, r);
  }
  if (A->n_panels > 0) {
    DN_CHECK(A->seg && A->pcol && A->panel_ids && partials, "matrix has no panel work list");
    const bool aligned = ((uintptr_t)H_mr % 16) == 0;
    const int slots = (int)panel_slots(A);
    const bool plain_early = A->tail_floor == 0;  // (in part 1)
    if (A->n_plain > 0 && (part == 0 || (part == 1) == plain_early)) {
      const int64_t row_groups = ceil_div(A->n_rows, 4);
      dim3 grid((unsigned)(row_groups * A->n_plain)), block(256);
      dispatch_gather(r, aligned, [&](auto tag) {
        using GT = typename decltype(tag)::type;
        hipLaunchKernelGGL((k_spmm_n_panel<GT>), grid, block, 0, stream(), A->seg, A->pcol,
                           A->pval, A->n_rows, row_groups, A->n_panels, A->panel_ids, slots, r, H_mr,
                           partials);
        return 0;
      });
      DN_LAUNCH_CHECK();
    }
    if (part == 1) return 0;
    // (the sweep kernel wants the CUs to itself: all its workgroups must be resident)
    if (A->n_swept > 0) {
      DN_TRY(side_stream_join());
      DN_TRY(launch_spmm_n_sweep(A, r, H_mr, aligned, slots));
    }
    // the far tail from its slot lists, into the last slot of the partial sums
    if (A->tail_floor > 0) {
      DN_CHECK(A->nl.pairs && A->nl.floor_col == A->tail_floor, "the far tail has no slot lists");
      DN_TRY(side_stream_join());
      DN_TRY(launch_spmm_n_lists(A, r, H_mr, partials + (int64_t)(slots - 1) * r, (int64_t)slots * r));
    }
    return 0;
  }
  DN_CHECK(A->rowptr && A->chunk_base && partials, "matrix has no row-major copy / work list");
  if (A->n_chunks == 0) return 0;
  DN_CHECK(A->n_chunks < (int64_t)INT32_MAX, "too many work chunks");
  dim3 grid((unsigned)A->n_chunks), block(256);
  const size_t lds = sizeof(float) * 4 * (size_t)r;
  dispatch_gather(r, ((uintptr_t)H_mr % 16) == 0, [&](auto tag) {
    using GT = typename decltype(tag)::type;
    hipLaunchKernelGGL((k_spmm_n<GT>), grid, block, lds, stream(), A->rowptr, A->colind, A->vals,
                       A->chunk_base, A->n_rows, r, H_mr, partials);
    return 0;
  });
  DN_LAUNCH_CHECK();
  return 0;
}

int launch_spmm_n_reduce(const dnpeff_csr* A_full, int r, float* N_nr) {
  const dnpeff_csr* A = sparse_part(A_full);
  const bool lists = A->nl.pairs && use_nlists(A, r);  // one set of sums, no panels
  if (lists || A->n_panels > 0) {
    if (A->n_rows > 0) {
      int64_t wgs = ceil_div(A->n_rows * r, 256);
      if (wgs > (1 << 20)) wgs = 1 << 20;
      hipLaunchKernelGGL(k_panel_reduce, dim3((unsigned)wgs), dim3(256), 0, stream(), A->partials,
                         A->n_rows, lists ? 1 : (int)panel_slots(A), r, N_nr);
      DN_LAUNCH_CHECK();
    }
  } else {
    DN_TRY(launch_chunk_reduce(A, r, A->partials, N_nr));
  }
  return launch_head_n_add(A_full, r, N_nr);
}

int launch_chunk_reduce(const dnpeff_csr* A, int r, const float* partials, float* N_nr) {
  if (A->n_rows == 0) return 0;
  hipLaunchKernelGGL(k_chunk_reduce, dim3((unsigned)A->n_rows), dim3(256), 0, stream(),
                     A->chunk_base, r, partials, N_nr);
  DN_LAUNCH_CHECK();
  return 0;
}

// Component slices for A^T W: workgroup b gathers slice b % n_slices of the rows of W, so an XCD
// (workgroups are dealt to the XCDs round-robin) only ever touches its own slice and keeps more
// of it in its 4 MB L2, at the price of reading the entries once per slice.  Measured with the
// grouped kernel, 1 / 2 / 4 / 8 slices: 10,000 x 128 (W 5.1 MB) 19.6 / 19.0 / 20.7 / 40.5 ms,
// 20,000 x 256 (W 20.5 MB) 352 / 294 / 230 / 246 ms.  Rule: the fewest slices (1, 2, 4, 8) that
// bring a slice of W to 6 MB or less, slices of at least 16 components; the spmm_t_slices
// switch overrides it (0 = this rule).
static int spmm_t_slices(int64_t n, int r) {
  auto ok = [&](int v) { return r % v == 0 && (r / v) % 16 == 0; };
  const int forced = (int)tuning().spmm_t_slices;
  if (forced == 1 || ((forced == 2 || forced == 4 || forced == 8) && ok(forced))) return forced;
  int v = 1;
  if (!xcd_round_robin()) return v;  // slices pay through the XCDs' own L2s only
  while (v < 8 && ok(2 * v) && 4.0 * (double)n * r / v > 6.0e6) v *= 2;
  return v;
}

// The sparse part of rows [col0, col1) of A^T W into T (row j - col0); long_cols[l0 .. l1) are the
// long columns in that range.
static int launch_spmm_t_sparse(const dnpeff_csr* A, int r, const float* W_nr, float* T, int64_t col0,
                                int64_t col1, int64_t l0, int64_t l1) {
  DN_CHECK(A->colptr != nullptr, "matrix has no transposed copy");
  const int64_t m = col1 - col0;
  if (m <= 0) return 0;
  const int64_t* colptr = A->colptr + col0;
  const bool aligned = ((uintptr_t)T % 16) == 0 && ((uintptr_t)W_nr % 16) == 0;
  if (A->tb.cols && aligned && col0 % 64 == 0 && (col1 % 64 == 0 || col1 == A->n_cols) && use_tlists(A, r))
    return launch_spmm_t_lists(A, r, W_nr, T, col0, col1);
  const int n_slices = (aligned && r % 4 == 0) ? spmm_t_slices(A->n_rows, r) : 1;
  const int width = r / n_slices;
  // one wave per (column, slice); a launch holds at most 2^32 threads, so beyond 2^23 workgroups
  // each one loops over several column groups
  int64_t wgs = ceil_div(m, 4) * n_slices;
  const int64_t max_wgs = ((int64_t)1 << 23) / n_slices * n_slices;
  if (wgs > max_wgs) wgs = max_wgs;
  dim3 grid((unsigned)wgs), block(256);
  // the grouped kernel handles whole slices of 16, 32, ..., 256 components (or the whole rank)
  const bool slice_ok = n_slices == 1 || width == 16 || width == 32 || width == 64 || width == 128 || width == 256;
  const bool grouped = aligned && r % 4 == 0 && slice_ok;
  const bool w_small = (double)A->n_rows * r * 4.0 < 4.0e9;  // 32-bit offsets into W
  if (grouped) {
    dim3 gg((unsigned)(ceil_div(m, 4 * SPMM_T_COLS) * n_slices));
    const int w4 = width / 4;
#define DN_GROUPED2(LPR, T_, FULL, SMALL)                                                     \
  hipLaunchKernelGGL((k_spmm_t_grouped<LPR, T_, FULL, SMALL>), gg, block, 0, stream(), colptr, \
                     A->rowind, A->tvals, m, r, n_slices, W_nr, T)
#define DN_GROUPED(LPR, T_)                                     \
  do {                                                          \
    const bool full = width == 4 * LPR * T_;                    \
    if (full && w_small24) DN_GROUPED2(LPR, T_, true, true);    \
    else if (full) DN_GROUPED2(LPR, T_, true, false);           \
    else if (w_small24) DN_GROUPED2(LPR, T_, false, true);      \
    else DN_GROUPED2(LPR, T_, false, false);                    \
  } while (0)
    const bool w_small24 = w_small && A->n_rows < ((int64_t)1 << 24);
    if (w4 <= 4) DN_GROUPED(4, 1);
    else if (w4 <= 8) DN_GROUPED(8, 1);
    else if (w4 <= 16) DN_GROUPED(16, 1);
    else if (w4 <= 32) DN_GROUPED(32, 1);
    else if (w4 <= 64) DN_GROUPED(64, 1);
    else if (w4 <= 128) DN_GROUPED(64, 2);
    else DN_GROUPED(64, 4);
#undef DN_GROUPED2
#undef DN_GROUPED
  }
  dispatch_gather(width, aligned, [&](auto tag) {
    using GT = typename decltype(tag)::type;
    if (!grouped)
      hipLaunchKernelGGL((k_spmm_t_short<GT>), grid, block, 0, stream(), colptr, A->rowind, A->tvals,
                         m, r, n_slices, W_nr, T, w_small);
    if (l1 > l0) {
      dim3 grid_l((unsigned)((l1 - l0) * n_slices));
      const size_t lds = sizeof(float) * 4 * (size_t)width;
      hipLaunchKernelGGL((k_spmm_t_long<GT>), grid_l, block, lds, stream(), A->long_cols + l0,
                         A->colptr, A->rowind, A->tvals, r, n_slices, W_nr, T, w_small, col0);
    }
    return 0;
  });
  DN_LAUNCH_CHECK();
  return 0;
}

int launch_spmm_t(const dnpeff_csr* A_full, int r, const float* W_nr, float* T_mr) {
  DN_CHECK(r >= 1 && r <= MAX_RANK, "rank %d outside [1, %d]", r, MAX_RANK);
  const dnpeff_csr* A = sparse_part(A_full);
  DN_TRY(launch_spmm_t_sparse(A, r, W_nr, T_mr, 0, A->n_cols, 0, A->n_long));
  // the head's rows of the result were stored as zeros above (its columns are empty in the
  // sparse part); the dense product overwrites them
  return launch_head_t(A_full, r, W_nr, T_mr);
}

int launch_spmm_t_tile(const dnpeff_csr* A_full, int r, const float* W_nr, int64_t col0,
                       int64_t col1, float* T_tile) {
  DN_CHECK(r >= 1 && r <= MAX_RANK, "rank %d outside [1, %d]", r, MAX_RANK);
  DN_CHECK(A_full->h_lists_valid, "matrix has no host lists for column tiles");
  const dnpeff_csr* A = sparse_part(A_full);
  DN_CHECK(0 <= col0 && col0 <= col1 && col1 <= A->n_cols, "column tile [%lld, %lld) outside the matrix",
           (long long)col0, (long long)col1);
  const std::vector<int32_t>& lc = A_full->h_long_cols;
  const int64_t l0 = std::lower_bound(lc.begin(), lc.end(), (int32_t)col0) - lc.begin();
  const int64_t l1 = std::lower_bound(lc.begin(), lc.end(), (int32_t)col1) - lc.begin();
  DN_TRY(launch_spmm_t_sparse(A, r, W_nr, T_tile, col0, col1, l0, l1));
  const std::vector<int32_t>& hc = A_full->h_head_cols;
  const int64_t k0 = std::lower_bound(hc.begin(), hc.end(), (int32_t)col0) - hc.begin();
  const int64_t k1 = std::lower_bound(hc.begin(), hc.end(), (int32_t)col1) - hc.begin();
  return launch_head_t_scatter(A_full, r, k0, k1, col0, T_tile);
}

int launch_spsp(const dnpeff_csr* A, dnpeff_csr* B, float* partials) {
  const int r = (int)B->n_rows;
  DN_CHECK(r >= 1 && r <= MAX_RANK, "rank %d outside [1, %d]", r, MAX_RANK);
  DN_CHECK(A->rowptr && A->chunk_base, "matrix has no row-major copy / work list");
  DN_CHECK(B->colptr != nullptr, "sparse factor has no transposed copy");
  DN_CHECK(A->n_cols == B->n_cols, "column counts differ (%lld vs %lld)", (long long)A->n_cols,
           (long long)B->n_cols);
  if (A->n_chunks == 0) return 0;
  if (!B->slots && B->n_cols > 0) {
    DN_TRY(dmalloc(&B->slots, 2 * B->n_cols));
    hipLaunchKernelGGL(k_spsp_build_slots, dim3((unsigned)ceil_div(B->n_cols, 256)), dim3(256), 0, stream(),
                       B->n_cols, B->colptr, B->rowind, B->tvals, B->slots);
    DN_LAUNCH_CHECK();
  }
  dim3 grid((unsigned)A->n_chunks), block(256);
#define DN_SPSP(V)                                                                               \
  hipLaunchKernelGGL((k_spsp_slots<V>), grid, block, 0, stream(), A->rowptr, A->colind, A->vals,   \
                     A->chunk_base, A->n_rows, r, B->slots, B->colptr, B->rowind, B->tvals, partials)
  switch (vpl_for(r)) {
    case 1: DN_SPSP(1); break;
    case 2: DN_SPSP(2); break;
    case 4: DN_SPSP(4); break;
    case 8: DN_SPSP(8); break;
    default: DN_SPSP(16); break;
  }
#undef DN_SPSP
  DN_LAUNCH_CHECK();
  return 0;
}

}  // namespace dn

using namespace dn;

DN_API int dnpeff_op_spmm_n(dnpeff_csr* A, int r, const float* H_mr, float* N_nr) {
  clear_error();
  DN_CHECK(A && H_mr && N_nr, "NULL argument");
  DN_TRY(csr_ensure_products(A, r));
  DN_TRY(launch_spmm_n(A, r, H_mr));
  return launch_spmm_n_reduce(A, r, N_nr);
}

DN_API int dnpeff_op_spmm_t(dnpeff_csr* A, int r, const float* W_nr, float* T_mr) {
  clear_error();
  DN_CHECK(A && W_nr && T_mr, "NULL argument");
  DN_TRY(csr_ensure_products(A, r));
  return launch_spmm_t(A, r, W_nr, T_mr);
}

DN_API int dnpeff_op_spmm_n_variant(dnpeff_csr* A_full, int r, const float* H_mr, float* N_nr,
                                    int variant) {
  clear_error();
  DN_CHECK(A_full && H_mr && N_nr, "NULL argument");
  DN_CHECK(r >= 1 && r <= MAX_RANK, "rank %d outside [1, %d]", r, MAX_RANK);
  if (variant == 0) return dnpeff_op_spmm_n(A_full, r, H_mr, N_nr);
  DN_CHECK(variant >= 1 && variant <= 3,
           "variant must be 0 (planned), 1 (a wave per row), 2 (row chunks) or 3 (merge path)");
  DN_TRY(csr_ensure_products(A_full, r));
  dnpeff_csr* A = sparse_part(A_full);
  DN_CHECK(has_row_major(A), "the row-major arrays of the sparse part were released");
  DN_TRY(launch_head_n(A_full, r, H_mr));
  const bool aligned = ((uintptr_t)H_mr % 16) == 0 && ((uintptr_t)N_nr % 16) == 0;
  if (variant == 1) {
    if (A->n_rows > 0) {
      dim3 grid((unsigned)ceil_div(A->n_rows, 4)), block(256);
      dispatch_gather(r, aligned, [&](auto tag) {
        using GT = typename decltype(tag)::type;
        hipLaunchKernelGGL((k_spmm_n_rowwave<GT>), grid, block, 0, stream(), A->rowptr, A->colind,
                           A->vals, A->n_rows, r, H_mr, N_nr);
        return 0;
      });
      DN_LAUNCH_CHECK();
    }
  } else if (variant == 3) {
    const int64_t n_shares = ceil_div(A->nnz + A->n_rows, MERGE_SHARE);
    if (n_shares > 0) {
      dbuf<float> carry;
      DN_TRY(carry.alloc(n_shares * 2 * (int64_t)r));
      DN_CHECK(ceil_div(n_shares, 4) < ((int64_t)1 << 24), "too many shares for one launch");
      dim3 grid((unsigned)ceil_div(n_shares, 4)), block(256);
      dispatch_gather(r, aligned, [&](auto tag) {
        using GT = typename decltype(tag)::type;
        hipLaunchKernelGGL((k_spmm_n_merge<GT>), grid, block, 0, stream(), A->rowptr, A->colind, A->vals,
                           A->n_rows, n_shares, r, H_mr, N_nr, carry.p);
        return 0;
      });
      int64_t wgs = A->n_rows < 65536 ? A->n_rows : 65536;
      hipLaunchKernelGGL(k_merge_fixup, dim3((unsigned)wgs), dim3(256), 0, stream(), A->rowptr, A->n_rows, r,
                         carry.p, N_nr);
      DN_LAUNCH_CHECK();
      DN_HIP(hipStreamSynchronize(stream()));  // (the carries are freed on return)
    }
  } else {
    DN_TRY(csr_ensure_chunks(A));
    DN_CHECK(A->partials && A->partials_floats >= A->n_chunks * (int64_t)r, "partial sums too small");
    if (A->n_chunks > 0) {
      DN_CHECK(A->n_chunks < (int64_t)INT32_MAX, "too many work chunks");
      dim3 grid((unsigned)A->n_chunks), block(256);
      const size_t lds = sizeof(float) * 4 * (size_t)r;
      dispatch_gather(r, ((uintptr_t)H_mr % 16) == 0, [&](auto tag) {
        using GT = typename decltype(tag)::type;
        hipLaunchKernelGGL((k_spmm_n<GT>), grid, block, lds, stream(), A->rowptr, A->colind, A->vals,
                           A->chunk_base, A->n_rows, r, H_mr, A->partials);
        return 0;
      });
      DN_LAUNCH_CHECK();
    }
    DN_TRY(launch_chunk_reduce(A, r, A->partials, N_nr));
  }
  return launch_head_n_add(A_full, r, N_nr);
}

DN_API int dnpeff_op_spmm_t_tile(dnpeff_csr* A, int r, const float* W_nr, int64_t col0, int64_t col1,
                                 float* T_tile) {
  clear_error();
  DN_CHECK(A && W_nr && T_tile, "NULL argument");
  DN_TRY(csr_ensure_products(A, r));
  DN_TRY(csr_tile_lists(A));
  DN_TRY(launch_head_t_product(A, r, W_nr));
  return launch_spmm_t_tile(A, r, W_nr, col0, col1, T_tile);
}

DN_API int dnpeff_op_spsp_dense(dnpeff_csr* A, dnpeff_csr* B, float* out_nr) {
  clear_error();
  DN_CHECK(A && B && out_nr, "NULL argument");
  // this product walks the plain CSR structures: a split left by an earlier NMF is undone
  if (A->tail) DN_TRY(dnpeff_csr_split_dense_head(A, 0.0, nullptr));
  if (B->tail) DN_TRY(dnpeff_csr_split_dense_head(B, 0.0, nullptr));
  DN_TRY(dnpeff_csr_build_transpose(B));
  const int r = (int)B->n_rows;
  DN_TRY(csr_ensure_partials(A, r));
  DN_TRY(launch_spsp(A, B, A->partials));
  return launch_chunk_reduce(A, r, A->partials, out_nr);
}
