// Component-sliced sparse products.
//
// A gathered entry of A H^T or A^T W moves a whole row of a factor (4 r bytes) into a CU, and a
// row-ordered gather finds the rows of a large factor in no cache: every entry then costs 4 r
// bytes of fabric traffic.  The kernels here cut the r components into slices of 32 (128 bytes)
// and give each XCD one slice (workgroup b runs on XCD b mod 8), so that what an XCD gathers from
// is eight times smaller and stays in its own L2:
//
//   A H^T  (k_spmm_n_lists): XCD x sums components [32 x, 32 x + 32) of every row of the result.
//     The running sums of all rows live in the LDS of the XCD's CUs (a wave slot owns up to 80
//     rows, 512 slots per XCD), and all slots walk the columns in the same order, piece by piece
//     (a piece: 32,768 columns, 4 MB of 128-byte row slices of H), so that a row slice of H is
//     fetched from HBM once and found in the L2 by the other rows that use it.  This is how the
//     far tail of a sparse part runs (the columns past the last swept piece, a few entries each,
//     which as panels bring every gathered row over the fabric: lists from a column floor on,
//     their sums in a slot of their own beside the panels' and the swept pieces'); the whole
//     sparse part can run this way too (n_lists = 1) and is slower than panels and pieces then.  The entries are
//     kept as one stream of (local row, local column, value) per slot, ordered by piece
//     ("slot lists").  Each of the 8 lane groups of a wave owns every eighth row of the slot
//     for good: it gathers one 128-byte slice per entry, sums the entries of a row in registers
//     and adds the sum to the row's place in LDS when its row changes.  No two groups ever touch
//     the same row, so the sums need no atomics (LDS float atomics run at one lane per ~3 cycles).
//
//   A^T W  (k_spmm_t_lists): XCD x produces components [32 x, 32 x + 32) of every row of the
//     result from its 128-byte slices of the rows of W (n x 128 bytes: L2 resident).  A wave owns
//     a block of up to 64 consecutive columns of the transposed copy; its 8 lane groups take
//     contiguous eighths of the block's entries, sum a column's entries in registers and add the
//     sum to the column's place in a small LDS tile when the column changes.
//
// All sums have an order fixed by the matrix structure.
#include "dnpeff_internal.hpp"

#include <algorithm>
#include <climits>
#include <cstring>
#include <type_traits>
#include <utility>
#include <vector>

namespace dn {

constexpr int NL_WAVES = 8;                      // waves per workgroup of the A H^T kernel
constexpr int NL_WGS_MAX = 96;                   // its workgroups per XCD: two (or three) per CU
constexpr int NL_ROW_BYTES = 128;                // one row of running sums in LDS: 32 floats
constexpr int NL_RPW_MAX = 80;                   // rows per wave slot (8 x 80 x 128 bytes = half the LDS)
constexpr int NL_SLICE = 32;                     // components per slice
constexpr int NL_MAX_SLOTS = 4096;
constexpr int NL_MAX_PIECES = 16000;             // (the builder keeps one counter per piece in LDS)
constexpr int NL_SYNC_STRIDE = 32;               // ints between the progress counters of two XCDs
constexpr int NL_GIVE_UP = 1 << 22;

// Lanes 0-7 of every row of 16 lanes read lane K of their row, lanes 8-15 lane 8 + K: every lane
// group of 8 reads the value of its K-th lane.
template <int K>
__device__ inline int bcast_octet(int v) {
  const int t = __builtin_amdgcn_mov_dpp(v, 0x150 + K, 0xf, 0xf, false);  // every lane: lane K of its row
  return __builtin_amdgcn_update_dpp(t, v, 0x150 + 8 + K, 0xf, 0xc, false);  // lanes 8-15: lane 8 + K
}
template <class F, int... I>
__device__ inline void for_steps(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
__device__ inline void add4(float4& a, const float4& b) {
  a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
}
__device__ inline void fma4(float4& a, float v, const float4& h) {
  a.x = fmaf(v, h.x, a.x); a.y = fmaf(v, h.y, a.y); a.z = fmaf(v, h.z, a.z); a.w = fmaf(v, h.w, a.w);
}

// ---------------------------------------------------------------------------
// A H^T from the slot lists
// ---------------------------------------------------------------------------
// pairs: per slot one stream of batches of 64 (index, value) pairs; index = (128 x local row)
// << 16 | local column.  Lane group g of the slot's wave owns the local rows 8 j + g; lane
// 8 g + k of batch t holds entry 8 t + k of the group's list for the piece, a list being sorted
// by row and filled up with (row of the entry before, column 0, 0.0f).  The batches of piece p of
// slot s are off[s][p] .. off[s][p + 1], counted from slot_base[s].
// Unit u = part * n_slices + slice; XCD x of a launch takes unit unit0 + x.
__global__ void __launch_bounds__(64 * NL_WAVES, 4)
    k_spmm_n_lists(const uint2* __restrict__ pairs, const int64_t* __restrict__ slot_base,
                   const uint32_t* __restrict__ off, int n_pieces, int piece_cols,
                   const int32_t* __restrict__ slot_rows, int rpw, int unit0, int n_units, int n_slices,
                   int r, const float* __restrict__ H, float* __restrict__ N, int64_t n_stride,
                   int* __restrict__ progress, int lag, int spin_max) {
  extern __shared__ __align__(16) float nl_sums[];  // [NL_WAVES][rpw][32]
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int x = blockIdx.x % SWEEP_XCDS, q = blockIdx.x / SWEEP_XCDS;
  const int nq = gridDim.x / SWEEP_XCDS;
  const int unit = unit0 + x;
  if (unit >= n_units) return;  // (the whole workgroup)
  const int slice = unit % n_slices, part = unit / n_slices;
  const int slot = (part * nq + q) * NL_WAVES + wave;
  int* const counter = progress + x * NL_SYNC_STRIDE;
  float* const my = nl_sums + wave * rpw * NL_SLICE;
  for (int i = lane; i < rpw * NL_SLICE; i += 64) my[i] = 0.0f;
  const int sub = lane & 7, grp = lane >> 3;
  const unsigned r4 = 4u * (unsigned)r, sub16 = 16u * (unsigned)sub;
  char* const lds_lane = reinterpret_cast<char*>(my) + 16 * sub;

  const uint2* st = pairs + slot_base[slot] * 64 + lane;
  const uint32_t* of = off + (size_t)slot * (n_pieces + 1);
  const int nb = (int)of[n_pieces];
  int p = 0;
  uint32_t e1 = of[1], e2 = of[n_pieces < 2 ? n_pieces : 2];
  const char* const Hs = reinterpret_cast<const char*>(H + slice * NL_SLICE);
  const char* Hp = Hs;
  int seen = 0;

  // The workgroup has issued everything of piece p: count it, and (wave 0) hold the workgroup back
  // while others on this XCD are more than `lag` pieces behind.  The other waves run on: they
  // meet wave 0 again at the next piece's barrier.  The wait is bounded; the first one that runs
  // out ends all later waits on this XCD.
  auto piece_done = [&]() {
    __builtin_amdgcn_s_barrier();
    p++;
    if (wave == 0) {
      int c = 0;
      if (lane == 0)
        c = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) + 1;
      c = __builtin_amdgcn_readfirstlane(c);
      if (seen < c) seen = c;
      const int want = nq * (p - lag);
      if (p > lag && p < n_pieces && seen < want) {
        int spin = 0;
        for (; spin < spin_max; spin++) {
          // an L2 atomic that changes nothing reads the counter (a plain load may hit the L1)
          if (lane == 0)
            c = __hip_atomic_fetch_max(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          c = __builtin_amdgcn_readfirstlane(c);
          if (c >= want) break;
          __builtin_amdgcn_s_sleep(32);
        }
        seen = c;
        if (spin == spin_max) {
          if (lane == 0)
            __hip_atomic_fetch_add(counter, NL_GIVE_UP, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          seen = INT_MAX;
        }
      }
    }
    e1 = e2;
    e2 = of[p + 2 < n_pieces ? p + 2 : n_pieces];
    Hp = Hs + (int64_t)p * piece_cols * (int64_t)r4;
  };

  unsigned cur_off = (unsigned)(grp * NL_ROW_BYTES);  // the group's first row
  float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  if (nb > 0) {
    // Four batches of pairs are held (A: batch b, B: b + 1, C: b + 2, D: b + 3) and the loop is
    // unrolled over their four roles, so that no register is copied while its load is in flight.
    // Batch b's eight steps each sum one gathered entry per lane group and then request the
    // gather of the same step of batch b + 1 into the registers just consumed: 7 or 8 gathers
    // are in flight at any time.  (nb is a multiple of 4.)
    uint2 A = st[0], B = st[64], C = st[128], D = st[192];
    while (0u >= e1) piece_done();
    float4 h[8];
    for_steps(std::make_integer_sequence<int, 8>{}, [&](auto k_tag) {
      constexpr int K = decltype(k_tag)::value;
      const int idx = bcast_octet<K>((int)A.x);
      h[K] = *reinterpret_cast<const float4*>(Hp + (__umul24((unsigned)idx & 0xffffu, r4) + sub16));
    });
    auto batch = [&](const uint2& cur, const uint2& nxt) {
      const char* const Hn = Hp;
      for_steps(std::make_integer_sequence<int, 8>{}, [&](auto k_tag) {
        constexpr int K = decltype(k_tag)::value;
        const unsigned ro = (unsigned)bcast_octet<K>((int)cur.x) >> 16;
        const float v = __int_as_float(bcast_octet<K>((int)cur.y));
        const float4 hv = h[K];
        if (ro != cur_off) {  // the group's row changes: its sum goes to LDS
          float4* a = reinterpret_cast<float4*>(lds_lane + cur_off);
          float4 t = *a;
          add4(t, acc);
          *a = t;
          acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
          cur_off = ro;
        }
        fma4(acc, v, hv);
        const int idn = bcast_octet<K>((int)nxt.x);
        h[K] = *reinterpret_cast<const float4*>(Hn + (__umul24((unsigned)idn & 0xffffu, r4) + sub16));
      });
    };
    for (int b = 0; b < nb; b += 4) {
      while ((uint32_t)(b + 1) >= e1) piece_done();
      batch(A, B);
      A = st[(size_t)(b + 4) * 64];
      while ((uint32_t)(b + 2) >= e1) piece_done();
      batch(B, C);
      B = st[(size_t)(b + 5) * 64];
      while ((uint32_t)(b + 3) >= e1) piece_done();
      batch(C, D);
      C = st[(size_t)(b + 6) * 64];
      if (b + 4 < nb) {
        while ((uint32_t)(b + 4) >= e1) piece_done();
      } else {
        A = make_uint2(0u, 0u);  // past the slot's last batch: gathers the piece's first row for nothing
      }
      batch(D, A);
      D = st[(size_t)(b + 7) * 64];
    }
  }
  while (p < n_pieces) piece_done();
  {
    float4* a = reinterpret_cast<float4*>(lds_lane + cur_off);
    float4 t = *a;
    add4(t, acc);
    *a = t;
  }
  // the wave's rows to N: a half wave writes the 128 bytes of one row
  const int c = lane & 31;
  for (int lr = lane >> 5; lr < rpw; lr += 2) {
    const int row = slot_rows[(size_t)slot * rpw + lr];
    if (row >= 0) N[(int64_t)row * n_stride + slice * NL_SLICE + c] = my[lr * NL_SLICE + c];
  }
}

// ---------------------------------------------------------------------------
// A^T W in blocks of columns
// ---------------------------------------------------------------------------
// tb[b] = first column of block b; a block holds up to 64 consecutive columns of one aligned
// group of 64.  Workgroup w of a launch: XCD x = w mod 8 takes slice slice0 + x mod n_sl of the
// components and every (8 / n_sl)-th group of four blocks; a wave takes one block.
// T (row j - col0 for column j) receives every column of the blocks, empty ones as zeros.
// A column's entries lie in the ranges of adjacent lane groups; a group adds its sum for a column
// to the LDS tile when it meets the next column (only the group whose range holds the column's
// end does that, so two groups never add to one column in the same step) and at the end of its
// range (groups that end in the same column then take turns).
__global__ void __launch_bounds__(256)
    k_spmm_t_lists(const int32_t* __restrict__ tb, int64_t blk0, int64_t blk1,
                   const int64_t* __restrict__ colptr, const int32_t* __restrict__ rowind,
                   const float* __restrict__ tvals, int r, int slice0, int n_sl,
                   const float* __restrict__ W, float* __restrict__ T, int64_t col0) {
  __shared__ __align__(16) float tiles[4][64 * NL_SLICE];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int x = blockIdx.x % SWEEP_XCDS;
  const int64_t rest = blockIdx.x / SWEEP_XCDS;
  const int slice = slice0 + x % n_sl, n_sub = SWEEP_XCDS / n_sl;
  const int64_t blk = blk0 + ((rest * n_sub + x / n_sl) * 4 + wave);
  if (blk >= blk1) return;
  const int j0 = tb[blk], nc = tb[blk + 1] - j0;  // 1 .. 64 columns
  float* const tile = tiles[wave];
  const int sub = lane & 7, grp = lane >> 3;
  const unsigned r4 = 4u * (unsigned)r, sub16 = 16u * (unsigned)sub;
  const char* const Ws = reinterpret_cast<const char*>(W + slice * NL_SLICE);
  float4* const tile_lane = reinterpret_cast<float4*>(tile) + sub;  // + 8 c: the lane's part of column c

  // column offsets of the block, relative to its first entry: lane l holds that of column l
  const int64_t cp = colptr[j0 + (lane < nc ? lane : nc)];
  const int64_t e0 = __shfl(cp, 0);
  const int64_t e_end = colptr[j0 + nc];
  const int L = (int)(e_end - e0);
  const int rel = lane < nc ? (int)(cp - e0) : INT_MAX;
  for (int i = lane; i < nc * 8; i += 64)
    reinterpret_cast<float4*>(tile)[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);

  if (L > 0) {
    // lane group g takes entries [g Lg, (g + 1) Lg) of the block, eight at a time (one per lane)
    const int Lg = (L + 7) / 8;
    const int g0 = grp * Lg, g1 = g0 + Lg < L ? g0 + Lg : L;
    const bool has = g0 < g1;
    const int nbt = (Lg + 7) / 8;
    const int32_t* ri = rowind + e0;
    const float* tv = tvals + e0;
    // (row, value, local column) of the lane's entry of batch t; lanes past the group's entries hold
    // (row 0, 0.0f, column of the group's last entry): they add nothing and make no column change.
    // The loads are unconditional, at a clamped position: a load under a branch would turn every
    // later wait for a gather into a wait for all outstanding loads.
    auto fetch = [&](int t, int& row, float& v, int& col) {
      const int qe = g0 + 8 * t + sub;
      const bool ok = qe < g1;
      const int qc = qe < L ? qe : L - 1;
      row = ri[qc];
      v = tv[qc];
      const int qs = ok ? qe : (has ? g1 - 1 : L - 1);
      int lo = 0;  // largest column c with rel[c] <= qs
#pragma unroll
      for (int step = 32; step >= 1; step >>= 1) {
        const int mid = lo + step;
        const int rv = __shfl(rel, mid & 63);
        if (mid < 64 && rv <= qs) lo = mid;
      }
      col = ok ? lo : (lo | 0x100);  // (bit 8: not an entry)
    };
    // Four batches are held (R0: batch t, .. R3: t + 3) and the loop is unrolled over their four
    // roles, so that no register is copied or combined while its load is in flight.
    int row0, row1, row2, row3, col0_, col1_, col2_, col3_;
    float val0, val1, val2, val3;
    fetch(0, row0, val0, col0_);
    fetch(1, row1, val1, col1_);
    fetch(2, row2, val2, col2_);
    fetch(3, row3, val3, col3_);
    float4 h[8];
    auto w_at = [&](int row, int col) {
      const unsigned rr = (col & 0x100) ? 0u : (unsigned)row;
      return *reinterpret_cast<const float4*>(Ws + (__umul24(rr, r4) + sub16));
    };
    for_steps(std::make_integer_sequence<int, 8>{}, [&](auto k_tag) {
      constexpr int K = decltype(k_tag)::value;
      h[K] = w_at(bcast_octet<K>(row0), bcast_octet<K>(col0_));
    });
    float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    int cur = bcast_octet<0>(col0_) & 0xff;
    auto batch = [&](float cval, int ccol, int nrow, int ncol) {
      for_steps(std::make_integer_sequence<int, 8>{}, [&](auto k_tag) {
        constexpr int K = decltype(k_tag)::value;
        const int cc = bcast_octet<K>(ccol);
        const int c = cc & 0xff;
        const float v = (cc & 0x100) ? 0.0f : __int_as_float(bcast_octet<K>(__float_as_int(cval)));
        const float4 hv = h[K];
        if (c != cur) {
          float4 s = tile_lane[8 * cur];
          add4(s, acc);
          tile_lane[8 * cur] = s;
          acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
          cur = c;
        }
        fma4(acc, v, hv);
        h[K] = w_at(bcast_octet<K>(nrow), bcast_octet<K>(ncol));
      });
    };
    for (int t = 0; t < nbt; t += 4) {
      batch(val0, col0_, row1, col1_);
      if (t + 1 >= nbt) break;
      fetch(t + 4, row0, val0, col0_);
      batch(val1, col1_, row2, col2_);
      if (t + 2 >= nbt) break;
      fetch(t + 5, row1, val1, col1_);
      batch(val2, col2_, row3, col3_);
      if (t + 3 >= nbt) break;
      fetch(t + 6, row2, val2, col2_);
      batch(val3, col3_, row0, col0_);
      fetch(t + 7, row3, val3, col3_);
    }
    // the groups' last sums: at once where the neighbours end in other columns, else in turn
    const int prev = __shfl(cur, (lane + 56) & 63), next = __shfl(cur, (lane + 8) & 63);
    const bool lone = has && (grp == 0 || prev != cur) && (grp == 7 || next != cur);
    if (lone) {
      float4 s = tile_lane[8 * cur];
      add4(s, acc);
      tile_lane[8 * cur] = s;
    }
    const bool pending = has && !lone;
    if (__any(pending)) {
      for (int g = 0; g < 8; g++) {
        if (pending && grp == g) {
          float4 s = tile_lane[8 * cur];
          add4(s, acc);
          tile_lane[8 * cur] = s;
        }
      }
    }
  }
  // the tile's rows to T: a lane group writes the 128 bytes of one column
  for (int c = grp; c < nc; c += 8)
    *reinterpret_cast<float4*>(T + ((int64_t)(j0 + c) - col0) * r + slice * NL_SLICE + 4 * sub) = tile_lane[8 * c];
}

// ---------------------------------------------------------------------------
// Building the slot lists from the row-major copy
// ---------------------------------------------------------------------------
// cnt[row][p] = entries of the row in piece p (one wave per row)
__global__ void __launch_bounds__(64)
    k_nl_row_count(const int64_t* __restrict__ rowptr, const int32_t* __restrict__ colind, int32_t floor_col,
                   int n_pieces, int piece_cols, uint32_t* __restrict__ cnt) {
  extern __shared__ int nl_lds[];
  const int64_t row = blockIdx.x;
  const int lane = threadIdx.x;
  for (int p = lane; p < n_pieces; p += 64) nl_lds[p] = 0;
  __syncthreads();
  const int64_t e1 = rowptr[row + 1];
  for (int64_t e = rowptr[row] + lane; e < e1; e += 64) {
    const int col = colind[e] - floor_col;  // (entries below the floor are not the lists')
    if (col >= 0) atomicAdd(&nl_lds[col / piece_cols], 1);
  }
  __syncthreads();
  for (int p = lane; p < n_pieces; p += 64) cnt[row * n_pieces + p] = (uint32_t)nl_lds[p];
}

// nbat[slot][p] = batches of (slot, p): the longest of the slot's eight group lists, in eights
__global__ void __launch_bounds__(256)
    k_nl_slot_batches(const uint32_t* __restrict__ cnt, const int32_t* __restrict__ slot_rows, int rpw,
                      int n_pieces, int n_slots, uint32_t* __restrict__ nbat) {
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= (int64_t)n_slots * n_pieces) return;
  const int s = (int)(id / n_pieces), p = (int)(id % n_pieces);
  uint32_t longest = 0;
  for (int g = 0; g < 8; g++) {
    uint32_t len = 0;
    for (int lr = g; lr < rpw; lr += 8) {
      const int row = slot_rows[(size_t)s * rpw + lr];
      if (row >= 0) len += cnt[(size_t)row * n_pieces + p];
    }
    longest = len > longest ? len : longest;
  }
  nbat[(size_t)s * n_pieces + p] = (longest + 7u) / 8u;
}

// off[slot][p] = batches of the slot's pieces before p (one workgroup per slot)
__global__ void __launch_bounds__(256)
    k_nl_slot_scan(const uint32_t* __restrict__ nbat, int n_pieces, uint32_t* __restrict__ off) {
  __shared__ uint32_t runs[256];
  const int s = blockIdx.x, tid = threadIdx.x;
  const int per = (n_pieces + 255) / 256, p0 = tid * per;
  const uint32_t* c = nbat + (size_t)s * n_pieces;
  uint32_t sum = 0;
  for (int p = p0; p < p0 + per && p < n_pieces; p++) sum += c[p];
  runs[tid] = sum;
  __syncthreads();
  if (tid == 0) {
    uint32_t run = 0;
    for (int i = 0; i < 256; i++) {
      const uint32_t t = runs[i];
      runs[i] = run;
      run += t;
    }
  }
  __syncthreads();
  uint32_t run = runs[tid];
  uint32_t* o = off + (size_t)s * (n_pieces + 1);
  for (int p = p0; p < p0 + per && p < n_pieces; p++) {
    o[p] = run;
    run += c[p];
  }
  // (the thread of the last piece) the kernel takes the batches of a slot four at a time
  if (p0 < n_pieces && p0 + per >= n_pieces) o[n_pieces] = (run + 3u) / 4u * 4u;
  if (n_pieces == 0 && tid == 0) o[0] = 0;
}

// Where entry w of the list of (slot, piece, group) lives: batch w / 8 of the piece, lane
// 8 group + w % 8.
__device__ inline int64_t nl_place(const int64_t* __restrict__ slot_base, const uint32_t* __restrict__ off,
                                   int n_pieces, int slot, int p, int g, uint32_t w) {
  return (slot_base[slot] + off[(size_t)slot * (n_pieces + 1) + p] + w / 8u) * 64 + g * 8 + (w & 7u);
}

// The entries of a row into the lists (one wave per row), in the order the row holds them: an
// entry's place in the list of (slot, piece, group) is the number of entries that the group's
// earlier rows hold in the piece plus the entries of this row in the piece before it.  Within a
// batch of 64 entries the rank among the entries of the same piece comes from ballots over the
// bits of the piece number.
__global__ void __launch_bounds__(64)
    k_nl_scatter(const int64_t* __restrict__ rowptr, const int32_t* __restrict__ colind, int32_t floor_col,
                 const float* __restrict__ vals, const int32_t* __restrict__ row_slot,
                 const int32_t* __restrict__ slot_rows, int rpw, const uint32_t* __restrict__ cnt,
                 int n_pieces, int piece_cols, int piece_bits, const int64_t* __restrict__ slot_base,
                 const uint32_t* __restrict__ off, uint2* __restrict__ pairs) {
  extern __shared__ int nl_lds[];  // next free place of the group's list, per piece
  const int64_t row = blockIdx.x;
  const int lane = threadIdx.x;
  const int rs = row_slot[row], slot = rs >> 7, lrow = rs & 127, g = lrow & 7;
  for (int p = lane; p < n_pieces; p += 64) {
    uint32_t before = 0;
    for (int lr = g; lr < lrow; lr += 8) {
      const int other = slot_rows[(size_t)slot * rpw + lr];
      if (other >= 0) before += cnt[(size_t)other * n_pieces + p];
    }
    nl_lds[p] = (int)before;
  }
  __syncthreads();
  const int64_t e0 = rowptr[row], e1 = rowptr[row + 1];
  for (int64_t base = e0; base < e1; base += 64) {
    const int64_t e = base + lane;
    bool active = e < e1;
    int p = 0, lcol = 0;
    float v = 0.0f;
    const int col = active ? colind[e] - floor_col : -1;
    active = col >= 0;
    if (active) {
      v = vals[e];
      p = col / piece_cols;
      lcol = col - p * piece_cols;
    }
    unsigned long long mask = __ballot(active);
    for (int b = 0; b < piece_bits; b++) {
      const bool bit = (p >> b) & 1;
      const unsigned long long bal = __ballot(active && bit);
      mask &= bit ? bal : ~bal;
    }
    const int rank = __popcll(mask & ((1ull << lane) - 1ull));
    int at = 0;
    if (active) at = nl_lds[p] + rank;
    __syncthreads();
    if (active) {
      if (rank == 0) nl_lds[p] += __popcll(mask);
      pairs[nl_place(slot_base, off, n_pieces, slot, p, g, (uint32_t)at)] =
          make_uint2(((unsigned)(lrow * NL_ROW_BYTES) << 16) | (unsigned)lcol, __float_as_uint(v));
    }
    __syncthreads();
  }
}

// The places of a group's list past its last entry: (row of the last entry, column 0, 0.0f), or
// the group's first row where the list is empty.
__global__ void __launch_bounds__(256)
    k_nl_fill(const uint32_t* __restrict__ cnt, const int32_t* __restrict__ slot_rows, int rpw, int n_pieces,
              int n_slots, const int64_t* __restrict__ slot_base, const uint32_t* __restrict__ off,
              uint2* __restrict__ pairs) {
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= (int64_t)n_slots * n_pieces * 8) return;
  const int g = (int)(id & 7);
  const int64_t sp = id >> 3;
  const int s = (int)(sp / n_pieces), p = (int)(sp % n_pieces);
  uint32_t len = 0;
  int last = g;
  for (int lr = g; lr < rpw; lr += 8) {
    const int row = slot_rows[(size_t)s * rpw + lr];
    const uint32_t c = row >= 0 ? cnt[(size_t)row * n_pieces + p] : 0u;
    if (c > 0) last = lr;
    len += c;
  }
  const uint32_t* o = off + (size_t)s * (n_pieces + 1);
  const uint32_t cap = 8u * (o[p + 1] - o[p]);
  const uint2 filler = make_uint2((unsigned)(last * NL_ROW_BYTES) << 16, 0u);
  for (uint32_t w = len; w < cap; w++) pairs[nl_place(slot_base, off, n_pieces, s, p, g, w)] = filler;
}

void nlists_drop(dnpeff_csr* S) {
  slot_lists& L = S->nl;
  dfree(L.pairs); dfree(L.slot_base); dfree(L.off); dfree(L.slot_rows); dfree(L.row_slot);
  dfree(L.progress);
  L = slot_lists();
}

// How many row parts rank r wants for n rows: enough for the rows of a part to fit the wave slots
// of one XCD, and at least as many as it takes to give all eight XCDs a unit when the rank has
// fewer than eight slices.
static int nlists_wgs() {
  int w = (int)tuning().nl_wgs;
  if (w < 8) w = 8;
  return w > NL_WGS_MAX ? NL_WGS_MAX : w;
}
static int nlists_parts(int64_t n_rows, int r) {
  const int n_slices = r / NL_SLICE;
  int parts = (int)ceil_div(n_rows, (int64_t)nlists_wgs() * NL_WAVES * NL_RPW_MAX);
  if (n_slices < SWEEP_XCDS && SWEEP_XCDS % n_slices == 0 && parts < SWEEP_XCDS / n_slices)
    parts = SWEEP_XCDS / n_slices;
  return parts < 1 ? 1 : parts;
}

int nlists_slots(int64_t n_rows, int r) { return nlists_parts(n_rows, r) * nlists_wgs() * NL_WAVES; }

bool nlists_supported(const dnpeff_csr* S, int r) {
  if (r < NL_SLICE || r % NL_SLICE != 0 || r > 1024) return false;
  if (S->n_rows < 1 || S->n_rows >= ((int64_t)1 << 24) || S->nnz < 1) return false;
  if (ceil_div(S->n_cols, 32768) > NL_MAX_PIECES) return false;
  return (int64_t)nlists_parts(S->n_rows, r) * nlists_wgs() * NL_WAVES <= NL_MAX_SLOTS;
}

// below[row] = entries of the row in columns < col (a row holds its entries in any order); one
// wave per row
__global__ void __launch_bounds__(256)
    k_rows_count_below(const int64_t* __restrict__ rowptr, const int32_t* __restrict__ colind, int64_t n_rows,
                       int32_t col, int* __restrict__ below) {
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= n_rows) return;
  const int lane = threadIdx.x & 63;
  const int64_t e1 = rowptr[row + 1];
  int c = 0;
  for (int64_t e = rowptr[row] + lane; e < e1; e += 64) c += colind[e] < col;
  for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off);
  if (lane == 0) below[row] = c;
}

int csr_rows_count_below(const dnpeff_csr* S, int32_t col, int* d_below) {
  DN_CHECK(has_row_major(S), "row-major copy of the matrix was released");
  if (S->n_rows == 0) return 0;
  hipLaunchKernelGGL(k_rows_count_below, dim3((unsigned)ceil_div(S->n_rows, 4)), dim3(256), 0, stream(),
                     S->rowptr, S->colind, S->n_rows, col, d_below);
  DN_LAUNCH_CHECK();
  return 0;
}

// floor_col > 0: lists of the entries in columns floor_col .. only (the far tail; the columns
// below stay with the panels and swept pieces), columns counted from floor_col.
int nlists_build(dnpeff_csr* S, int r, int32_t floor_col, double max_extra_bytes, bool* declined) {
  if (declined) *declined = false;
  const tuning_t& tn = tuning();
  int piece_cols = (int)tn.nl_piece_cols;
  if (piece_cols < 64) piece_cols = 64;
  if (piece_cols > 65536) piece_cols = 65536;
  while (piece_cols < 65536 && ceil_div(S->n_cols - floor_col, piece_cols) > NL_MAX_PIECES) piece_cols += 1024;
  const int n_parts = nlists_parts(S->n_rows, r);
  slot_lists& L = S->nl;
  const int wgs = nlists_wgs();
  if (L.pairs && L.piece_cols == piece_cols && L.n_parts == n_parts && L.wgs == wgs && L.floor_col == floor_col)
    return 0;
  nlists_drop(S);
  DN_CHECK(nlists_supported(S, r), "no slot lists for %lld rows at rank %d", (long long)S->n_rows, r);
  DN_CHECK(has_row_major(S), "slot lists are built from the row-major copy, which was released");
  hipStream_t st = stream();
  DN_CHECK(floor_col >= 0 && floor_col < S->n_cols, "slot lists: column floor %d", (int)floor_col);
  const int64_t n = S->n_rows, m = S->n_cols - floor_col;
  const int n_slots = n_parts * wgs * NL_WAVES;
  const int rpw = 8 * (int)ceil_div(n, (int64_t)n_slots * 8);
  DN_CHECK(rpw <= NL_RPW_MAX, "slot lists: %d rows per slot", rpw);
  const int n_pieces = (int)ceil_div(m, piece_cols);
  DN_CHECK(n_pieces <= NL_MAX_PIECES, "slot lists: %d pieces", n_pieces);

  // rows to (slot, lane group): longest first, dealt back and forth over the 8 n_slots groups, so
  // that the groups hold about the same number of entries (all slots of an XCD advance piece by
  // piece together, and a wave's eight groups step by step); local row = 8 * round + group
  std::vector<int64_t> rowptr((size_t)n + 1), mine((size_t)n);  // mine: the row's entries in the lists
  std::vector<int> below((size_t)n, 0);
  if (floor_col > 0) {
    dbuf<int> d_below;
    DN_TRY(d_below.alloc(n));
    DN_TRY(csr_rows_count_below(S, floor_col, d_below.p));
    DN_HIP(hipStreamSynchronize(st));
    DN_HIP(hipMemcpy(below.data(), d_below.p, sizeof(int) * n, hipMemcpyDeviceToHost));
  }
  DN_HIP(hipStreamSynchronize(st));
  DN_HIP(hipMemcpy(rowptr.data(), S->rowptr, sizeof(int64_t) * (n + 1), hipMemcpyDeviceToHost));
  int64_t z = 0;
  for (int64_t i = 0; i < n; i++) {
    mine[(size_t)i] = rowptr[(size_t)i + 1] - rowptr[(size_t)i] - below[(size_t)i];
    z += mine[(size_t)i];
  }
  std::vector<int32_t> order((size_t)n), row_slot((size_t)n), slot_rows((size_t)n_slots * rpw, -1);
  for (int64_t i = 0; i < n; i++) order[(size_t)i] = (int32_t)i;
  std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) {
    return mine[(size_t)a] > mine[(size_t)b];
  });
  const int64_t n_groups = (int64_t)n_slots * 8;
  for (int64_t t = 0; t < n; t++) {
    const int round = (int)(t / n_groups);
    const int64_t pos = t % n_groups, gs = (round & 1) ? n_groups - 1 - pos : pos;
    const int slot = (int)(gs / 8), lrow = 8 * round + (int)(gs % 8);
    row_slot[(size_t)order[(size_t)t]] = slot * 128 + lrow;
    slot_rows[(size_t)slot * rpw + lrow] = order[(size_t)t];
  }

  dbuf<uint32_t> cnt, nbat;
  DN_TRY(dmalloc(&L.row_slot, n));
  DN_TRY(dmalloc(&L.slot_rows, (int64_t)n_slots * rpw));
  DN_TRY(dmalloc(&L.off, (int64_t)n_slots * (n_pieces + 1)));
  DN_TRY(dmalloc(&L.slot_base, (int64_t)n_slots + 1));
  DN_TRY(dmalloc(&L.progress, SWEEP_XCDS * NL_SYNC_STRIDE));
  DN_TRY(cnt.alloc(n * n_pieces));
  DN_TRY(nbat.alloc((int64_t)n_slots * n_pieces));
  DN_HIP(hipMemcpy(L.row_slot, row_slot.data(), sizeof(int32_t) * n, hipMemcpyHostToDevice));
  DN_HIP(hipMemcpy(L.slot_rows, slot_rows.data(), sizeof(int32_t) * slot_rows.size(), hipMemcpyHostToDevice));
  const size_t lds = sizeof(int) * (size_t)n_pieces;
  hipLaunchKernelGGL(k_nl_row_count, dim3((unsigned)n), dim3(64), lds, st, S->rowptr, S->colind, floor_col,
                     n_pieces, piece_cols, cnt.p);
  DN_LAUNCH_CHECK();
  hipLaunchKernelGGL(k_nl_slot_batches, dim3((unsigned)ceil_div((int64_t)n_slots * n_pieces, 256)), dim3(256), 0,
                     st, cnt.p, L.slot_rows, rpw, n_pieces, n_slots, nbat.p);
  DN_LAUNCH_CHECK();
  hipLaunchKernelGGL(k_nl_slot_scan, dim3((unsigned)n_slots), dim3(256), 0, st, nbat.p, n_pieces, L.off);
  DN_LAUNCH_CHECK();
  DN_HIP(hipStreamSynchronize(st));
  if (tuning().verbose >= 2.0) {  // how far the lock step of an XCD's waves is from the mean work
    std::vector<uint32_t> hb((size_t)n_slots * n_pieces);
    DN_HIP(hipMemcpy(hb.data(), nbat.p, hb.size() * 4, hipMemcpyDeviceToHost));
    double sum = 0, sum_max = 0, sum_wgmax = 0;
    for (int p = 0; p < n_pieces; p++) {
      uint32_t mx = 0;
      double wg = 0;
      for (int s0 = 0; s0 < n_slots; s0 += NL_WAVES) {
        uint32_t m8 = 0;
        for (int w = 0; w < NL_WAVES; w++) {
          const uint32_t v = hb[(size_t)(s0 + w) * n_pieces + p];
          sum += v;
          m8 = v > m8 ? v : m8;
        }
        wg += m8;
        mx = m8 > mx ? m8 : mx;
      }
      sum_max += mx;
      sum_wgmax += wg / (n_slots / NL_WAVES);
    }
    std::fprintf(stderr, "dnpeff: slot lists: batches per slot %.0f, sum over pieces of the longest slot %.0f, of the mean over workgroups of their longest wave %.0f\n",
                 sum / n_slots, sum_max, sum_wgmax);
  }
  nbat.reset();
  // batches of the slots -> first batch of each slot
  std::vector<uint32_t> tot((size_t)n_slots);
  DN_HIP(hipMemcpy2D(tot.data(), sizeof(uint32_t), L.off + n_pieces, sizeof(uint32_t) * (size_t)(n_pieces + 1),
                     sizeof(uint32_t), (size_t)n_slots, hipMemcpyDeviceToHost));
  L.h_slot_base.assign((size_t)n_slots + 1, 0);
  for (int s = 0; s < n_slots; s++) L.h_slot_base[(size_t)s + 1] = L.h_slot_base[(size_t)s] + tot[(size_t)s];
  const int64_t n_batches = L.h_slot_base[(size_t)n_slots];
  DN_HIP(hipMemcpy(L.slot_base, L.h_slot_base.data(), sizeof(int64_t) * ((size_t)n_slots + 1),
                   hipMemcpyHostToDevice));
  if (max_extra_bytes >= 0.0 && (double)(n_batches + 8) * 512.0 - 8.0 * (double)z > max_extra_bytes) {
    if (tn.verbose != 0.0)
      fprintf(stderr, "dnpeff: slot lists of %lld entries would take %.2f GB: not built\n", (long long)z,
              (double)(n_batches + 8) * 512.0 / 1e9);
    nlists_drop(S);
    if (declined) *declined = true;
    return 0;
  }
  // (the kernel requests pairs up to seven batches past a slot's last)
  DN_TRY(dmalloc(&L.pairs, (n_batches + 8) * 64));
  DN_HIP(hipMemsetAsync(L.pairs + n_batches * 64, 0, sizeof(uint2) * 8 * 64, st));
  int piece_bits = 0;
  while ((1 << piece_bits) < n_pieces) piece_bits++;
  hipLaunchKernelGGL(k_nl_scatter, dim3((unsigned)n), dim3(64), lds, st, S->rowptr, S->colind, floor_col,
                     S->vals, L.row_slot, L.slot_rows, rpw, cnt.p, n_pieces, piece_cols, piece_bits, L.slot_base, L.off,
                     L.pairs);
  DN_LAUNCH_CHECK();
  hipLaunchKernelGGL(k_nl_fill, dim3((unsigned)ceil_div((int64_t)n_slots * n_pieces * 8, 256)), dim3(256), 0, st,
                     cnt.p, L.slot_rows, rpw, n_pieces, n_slots, L.slot_base, L.off, L.pairs);
  DN_LAUNCH_CHECK();
  DN_HIP(hipStreamSynchronize(st));
  L.piece_cols = piece_cols;
  L.floor_col = floor_col;
  L.n_entries = z;
  L.n_pieces = n_pieces;
  L.n_parts = n_parts;
  L.wgs = wgs;
  L.rpw = rpw;
  L.n_batches = n_batches;
  L.h_row_slot = std::move(row_slot);
  if (tn.verbose != 0.0)
    fprintf(stderr,
            "dnpeff: slot lists of %lld entries from column %d on: %d part(s) x %d slots of %d rows, %d pieces of "
            "%d columns, %lld batches (%.1f %% filler), %.2f GB\n",
            (long long)z, (int)floor_col, n_parts, wgs * NL_WAVES, rpw, n_pieces, piece_cols, (long long)n_batches,
            z > 0 ? 100.0 * ((double)n_batches * 64.0 / (double)z - 1.0) : 0.0,
            (double)(n_batches + 8) * 512.0 / 1e9);
  return 0;
}

__global__ void k_nl_clear(int* progress) { progress[threadIdx.x] = 0; }

// part[row * stride .. + r) = the listed entries' share of (A H^T)[row, :] (stride in floats)
int launch_spmm_n_lists(const dnpeff_csr* S, int r, const float* H_mr, float* part, int64_t stride) {
  const slot_lists& L = S->nl;
  DN_CHECK(L.pairs != nullptr, "matrix has no slot lists");
  DN_CHECK(r % NL_SLICE == 0 && ((uintptr_t)H_mr % 16) == 0 && stride >= r, "slot lists: rank %d or alignment", r);
  DN_CHECK(L.n_parts == nlists_parts(S->n_rows, r) && L.wgs == nlists_wgs(), "slot lists were built for another rank");
  static bool attr_set = false;
  const size_t lds = (size_t)NL_WAVES * L.rpw * NL_ROW_BYTES;
  if (!attr_set) {
    DN_HIP(hipFuncSetAttribute((const void*)k_spmm_n_lists, hipFuncAttributeMaxDynamicSharedMemorySize,
                               NL_WAVES * NL_RPW_MAX * NL_ROW_BYTES));
    attr_set = true;
  }
  const tuning_t& tn = tuning();
  int lag = (int)tn.nl_lag, spin_max = (int)tn.nl_spin;
  if (lag < 0) lag = 0;
  const int n_slices = r / NL_SLICE, n_units = n_slices * L.n_parts;
  for (int unit0 = 0; unit0 < n_units; unit0 += SWEEP_XCDS) {
    hipLaunchKernelGGL(k_nl_clear, dim3(1), dim3(SWEEP_XCDS * NL_SYNC_STRIDE), 0, stream(), L.progress);
    hipLaunchKernelGGL(k_spmm_n_lists, dim3(SWEEP_XCDS * L.wgs), dim3(64 * NL_WAVES), lds, stream(), L.pairs,
                       L.slot_base, L.off, L.n_pieces, L.piece_cols, L.slot_rows, L.rpw, unit0, n_units,
                       n_slices, r, H_mr + (int64_t)L.floor_col * r, part, stride, L.progress, lag, spin_max);
    DN_LAUNCH_CHECK();
    if (tn.verbose >= 2.0) {  // how the lock step went: counts past NL_GIVE_UP mean a wait ran out
      int h[SWEEP_XCDS * NL_SYNC_STRIDE];
      DN_HIP(hipStreamSynchronize(stream()));
      DN_HIP(hipMemcpy(h, L.progress, sizeof(h), hipMemcpyDeviceToHost));
      fprintf(stderr, "dnpeff: slot-list launch at unit %d: progress counters", unit0);
      for (int x = 0; x < SWEEP_XCDS; x++) fprintf(stderr, " %d", h[x * NL_SYNC_STRIDE]);
      fprintf(stderr, " (%d pieces x %d workgroups)\n", L.n_pieces, L.wgs);
    }
  }
  return 0;
}

// The sparse part's entries of one row, from the lists (by piece, in the row's own order inside a
// piece).  A filler pair is (some row, column 0 of the piece, +0.0f): an entry that holds exactly
// that is not told apart from it and is left out.
int nlists_get_row(const dnpeff_csr* S, int64_t row, std::vector<int32_t>& cols, std::vector<float>& vals) {
  const slot_lists& L = S->nl;
  DN_CHECK(L.pairs && (int64_t)L.h_row_slot.size() == S->n_rows, "matrix has no slot lists");
  const int rs = L.h_row_slot[(size_t)row], slot = rs >> 7, lrow = rs & 127;
  const int64_t b0 = L.h_slot_base[(size_t)slot], b1 = L.h_slot_base[(size_t)slot + 1];
  std::vector<uint32_t> off((size_t)L.n_pieces + 1);
  std::vector<uint2> pairs((size_t)(b1 - b0) * 64);
  DN_HIP(hipStreamSynchronize(stream()));
  DN_HIP(hipMemcpy(off.data(), L.off + (size_t)slot * (L.n_pieces + 1), sizeof(uint32_t) * off.size(),
                   hipMemcpyDeviceToHost));
  if (b1 > b0)
    DN_HIP(hipMemcpy(pairs.data(), L.pairs + b0 * 64, sizeof(uint2) * pairs.size(), hipMemcpyDeviceToHost));
  cols.clear();
  vals.clear();
  const int g = lrow & 7;
  for (int p = 0; p < L.n_pieces; p++)
    for (size_t b = off[(size_t)p]; b < off[(size_t)p + 1]; b++)
      for (int k = 0; k < 8; k++) {
        const uint2 e = pairs[b * 64 + (size_t)g * 8 + k];
        if ((int)(e.x >> 16) == lrow * NL_ROW_BYTES && !((e.x & 0xffffu) == 0u && e.y == 0u)) {
          cols.push_back((int32_t)(L.floor_col + (int64_t)p * L.piece_cols + (e.x & 0xffffu)));
          float v;
          memcpy(&v, &e.y, sizeof(float));
          vals.push_back(v);
        }
      }
  return 0;
}

// ---------------------------------------------------------------------------
// Column blocks of A^T W
// ---------------------------------------------------------------------------
constexpr int TB_ENTRIES = 2048;  // a block is closed when it holds this many entries

// blocks of one aligned group of 64 columns: whole columns, closed at TB_ENTRIES entries
__global__ void __launch_bounds__(256)
    k_tb_count(const int64_t* __restrict__ colptr, int64_t n_cols, int64_t n_groups, int* __restrict__ count) {
  const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= n_groups) return;
  const int64_t j0 = g * 64, j1 = j0 + 64 < n_cols ? j0 + 64 : n_cols;
  int blocks = 1;
  int64_t start = colptr[j0];
  for (int64_t j = j0 + 1; j < j1; j++) {
    const int64_t at = colptr[j];
    if (at - start >= TB_ENTRIES) {
      blocks++;
      start = at;
    }
  }
  count[g] = blocks;
}

__global__ void __launch_bounds__(256)
    k_tb_fill(const int64_t* __restrict__ colptr, int64_t n_cols, int64_t n_groups,
              const int64_t* __restrict__ first, int32_t* __restrict__ tb) {
  const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (g > n_groups) return;
  if (g == n_groups) {
    tb[first[n_groups]] = (int32_t)n_cols;
    return;
  }
  const int64_t j0 = g * 64, j1 = j0 + 64 < n_cols ? j0 + 64 : n_cols;
  int64_t w = first[g];
  tb[w++] = (int32_t)j0;
  int64_t start = colptr[j0];
  for (int64_t j = j0 + 1; j < j1; j++) {
    const int64_t at = colptr[j];
    if (at - start >= TB_ENTRIES) {
      tb[w++] = (int32_t)j;
      start = at;
    }
  }
}

void tblocks_drop(dnpeff_csr* S) {
  dfree(S->tb.cols);
  S->tb = col_blocks();
}

int tblocks_build(dnpeff_csr* S) {
  col_blocks& B = S->tb;
  if (B.cols) return 0;
  DN_CHECK(S->colptr != nullptr, "column blocks need the transposed copy");
  const int64_t m = S->n_cols, n_groups = ceil_div(m, 64);
  if (m == 0) return 0;
  dbuf<int> count;
  dbuf<int64_t> first;
  DN_TRY(count.alloc(n_groups));
  DN_TRY(first.alloc(n_groups + 1));
  hipLaunchKernelGGL(k_tb_count, dim3((unsigned)ceil_div(n_groups, 256)), dim3(256), 0, stream(), S->colptr, m,
                     n_groups, count.p);
  DN_LAUNCH_CHECK();
  DN_TRY(scan_counts_i64(count.p, n_groups, first.p));
  B.h_first.assign((size_t)n_groups + 1, 0);
  DN_HIP(hipStreamSynchronize(stream()));
  DN_HIP(hipMemcpy(B.h_first.data(), first.p, sizeof(int64_t) * (n_groups + 1), hipMemcpyDeviceToHost));
  B.n_blocks = B.h_first[(size_t)n_groups];
  DN_TRY(dmalloc(&B.cols, B.n_blocks + 1));
  hipLaunchKernelGGL(k_tb_fill, dim3((unsigned)ceil_div(n_groups + 1, 256)), dim3(256), 0, stream(), S->colptr,
                     m, n_groups, first.p, B.cols);
  DN_LAUNCH_CHECK();
  DN_HIP(hipStreamSynchronize(stream()));
  return 0;
}

bool tlists_supported(const dnpeff_csr* S, int r) {
  if (r < NL_SLICE || r % NL_SLICE != 0 || r > 1024) return false;
  const int n_slices = r / NL_SLICE;
  if (n_slices < SWEEP_XCDS && SWEEP_XCDS % n_slices != 0) return false;
  if (n_slices > SWEEP_XCDS && n_slices % SWEEP_XCDS != 0) return false;
  return S->n_rows < ((int64_t)1 << 24) && 4.0 * (double)S->n_rows * r < 4.0e9;
}

// Rows [col0, col1) of the sparse part's A^T W into T (row j - col0); col0 must be a multiple of 64.
int launch_spmm_t_lists(const dnpeff_csr* S, int r, const float* W_nr, float* T, int64_t col0, int64_t col1) {
  const col_blocks& B = S->tb;
  if (col1 <= col0) return 0;
  DN_CHECK(B.cols != nullptr, "matrix has no column blocks");
  DN_CHECK(col0 % 64 == 0 && (col1 % 64 == 0 || col1 == S->n_cols), "column blocks: tile [%lld, %lld)",
           (long long)col0, (long long)col1);
  DN_CHECK(((uintptr_t)W_nr % 16) == 0 && ((uintptr_t)T % 16) == 0, "column blocks: alignment");
  const int64_t blk0 = B.h_first[(size_t)(col0 / 64)], blk1 = B.h_first[(size_t)ceil_div(col1, 64)];
  if (blk1 <= blk0) return 0;
  const int n_slices = r / NL_SLICE;
  const int n_sl = n_slices < SWEEP_XCDS ? n_slices : SWEEP_XCDS;
  const int n_sub = SWEEP_XCDS / n_sl;
  const int64_t wgs = ceil_div(ceil_div(blk1 - blk0, 4), n_sub) * SWEEP_XCDS;
  DN_CHECK(wgs < ((int64_t)1 << 24), "column blocks: %lld workgroups in one launch", (long long)wgs);
  for (int slice0 = 0; slice0 < n_slices; slice0 += n_sl) {
    hipLaunchKernelGGL(k_spmm_t_lists, dim3((unsigned)wgs), dim3(256), 0, stream(), B.cols, blk0, blk1, S->colptr,
                       S->rowind, S->tvals, r, slice0, n_sl, W_nr, T, col0);
    DN_LAUNCH_CHECK();
  }
  return 0;
}

}  // namespace dn
