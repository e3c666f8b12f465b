// Component-sliced sparse products.
//
// A gathered entry of A H^T or A^T W moves a whole row of a factor (4 r bytes) into a CU, and a
// row-ordered gather finds the rows of a large factor in no cache: every entry then costs 4 r
// bytes of fabric traffic.  The kernels here cut the r components into slices of 32 (128 bytes)
// and give each XCD one slice (workgroup b runs on XCD b mod 8), so that what an XCD gathers from
// is eight times smaller and stays in its own L2:
//
//   A H^T  (k_spmm_n_lists): XCD x sums components [32 x, 32 x + 32) of every row of the result.
//     The running sums of all rows live in the LDS of the XCD's CUs (a wave slot owns up to 72
//     rows, 512 slots per XCD), and all slots walk the columns in the same order, piece by piece
//     (a piece: 16,384 columns, 2 MB of 128-byte row slices of H), so that a row slice of H is
//     fetched from HBM once and found in the L2 by the other rows that use it.  The entries are
//     kept as one stream of (local row, local column, value) per slot, ordered by piece
//     ("slot lists", built once from the transposed copy); a lane group of 8 lanes gathers one
//     128-byte slice per entry and adds its four products to the row's sums with LDS atomics, so
//     there is no per-row or per-segment bookkeeping at all.
//
//   A^T W  (k_spmm_t_lists): XCD x produces components [32 x, 32 x + 32) of every row of the
//     result from its 128-byte slices of the rows of W (n x 128 bytes: L2 resident).  A wave owns
//     a block of up to 64 consecutive columns of the transposed copy; its 8 lane groups take
//     contiguous eighths of the block's entries, sum a column's entries in registers and add the
//     sum to the column's slot of a small LDS tile when the column changes.
//
// All sums have an order fixed by the matrix structure: a wave's LDS operations execute in
// program order and lanes of one instruction that meet in an address are added in lane order.
#include "dnpeff_internal.hpp"

#include <algorithm>
#include <climits>
#include <cstring>
#include <type_traits>
#include <utility>

namespace dn {

constexpr int NL_WAVES = 8;                      // waves per workgroup of the A H^T kernel
constexpr int NL_WGS = 64;                       // its workgroups per XCD: two per CU
constexpr int NL_SLOTS = NL_WAVES * NL_WGS;      // wave slots per XCD
constexpr int NL_ROW_FLOATS = 33;                // floats between two rows of running sums in LDS
constexpr int NL_ROW_BYTES = 4 * NL_ROW_FLOATS;
constexpr int NL_RPW_MAX = 72;                   // rows per wave slot (8 x 72 x 132 bytes <= half the LDS)
constexpr int NL_SLICE = 32;                     // components per slice
constexpr int NL_CHUNK = 32768;                  // entries per chunk of the list builder
constexpr int NL_MAX_SLOTS = 4096;
constexpr int NL_SYNC_STRIDE = 32;               // ints between the progress counters of two XCDs
constexpr int NL_GIVE_UP = 1 << 22;

// Lanes 0-7 of every row of 16 lanes read lane 2 K of their row, lanes 8-15 lane 2 K + 1.
template <int K>
__device__ inline int bcast_pair(int v) {
  const int t = __builtin_amdgcn_update_dpp(0, v, 0x150 + 2 * K, 0xf, 0x3, false);
  return __builtin_amdgcn_update_dpp(t, v, 0x150 + 2 * K + 1, 0xf, 0xc, false);
}
// Lanes 0-7 of every row of 16 lanes read lane K of their row, lanes 8-15 lane 8 + K.
template <int K>
__device__ inline int bcast_octet(int v) {
  const int t = __builtin_amdgcn_update_dpp(0, v, 0x150 + K, 0xf, 0x3, false);
  return __builtin_amdgcn_update_dpp(t, v, 0x150 + 8 + K, 0xf, 0xc, false);
}
template <class F, int... I>
__device__ inline void for_steps(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}

// ---------------------------------------------------------------------------
// A H^T from the slot lists
// ---------------------------------------------------------------------------
// pairs: per slot one stream of batches of 64 (index, value) pairs; index = (132 x local row)
// << 16 | local column; the batches of piece p of slot s are off[s][p] .. off[s][p + 1] (counted
// from slot_base[s]), padded with (0, 0.0f) pairs.  Step k of a batch applies the pairs held by
// lanes 16 q + 2 k and 16 q + 2 k + 1 (q = 0 .. 3): eight entries, one per lane group.
// Unit u = part * n_slices + slice; XCD x of a launch takes unit unit0 + x.
// Running sums: fine sums in LDS ([wave][local row][33], component 4 s + k of a row at float
// 8 k + s, so that the eight lanes of a group hit eight consecutive banks), moved into per-lane
// coarse sums in registers every `flush_every` batches: two short fp32 sums instead of one of
// 10^5 terms.
template <int RPW2>
__global__ void __launch_bounds__(64 * NL_WAVES, 4)
    k_spmm_n_lists(const uint2* __restrict__ pairs, const int64_t* __restrict__ slot_base,
                   const uint32_t* __restrict__ off, int n_pieces, int piece_cols,
                   const int32_t* __restrict__ slot_rows, int rpw, int unit0, int n_units, int n_slices,
                   int r, const float* __restrict__ H, float* __restrict__ N, int* __restrict__ progress,
                   int lag, int spin_max, int flush_every) {
  extern __shared__ __align__(16) float nl_sums[];  // [NL_WAVES][rpw][NL_ROW_FLOATS]
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int x = blockIdx.x % SWEEP_XCDS, q = blockIdx.x / SWEEP_XCDS;
  const int nq = gridDim.x / SWEEP_XCDS;
  const int unit = unit0 + x;
  if (unit >= n_units) return;  // (the whole workgroup)
  const int slice = unit % n_slices, part = unit / n_slices;
  const int slot = (part * nq + q) * NL_WAVES + wave;
  int* const counter = progress + x * NL_SYNC_STRIDE;
  float* const my = nl_sums + wave * rpw * NL_ROW_FLOATS;
  for (int i = lane; i < rpw * NL_ROW_FLOATS; i += 64) my[i] = 0.0f;
  float coarse[RPW2];
#pragma unroll
  for (int i = 0; i < RPW2; i++) coarse[i] = 0.0f;
  const int sub = lane & 7;
  const unsigned r4 = 4u * (unsigned)r, sub16 = 16u * (unsigned)sub;
  char* const lds_lane = reinterpret_cast<char*>(my) + 4 * sub;

  // lane l holds component l & 31 of local rows 2 i + (l >> 5)
  auto flush = [&]() {
    const int c = lane & 31;
    float* a = my + (lane >> 5) * NL_ROW_FLOATS + ((c & 3) * 8 + (c >> 2));
#pragma unroll
    for (int i = 0; i < RPW2; i++) {
      if (2 * i + (lane >> 5) < rpw) {
        coarse[i] += a[2 * i * NL_ROW_FLOATS];
        a[2 * i * NL_ROW_FLOATS] = 0.0f;
      }
    }
  };

  const uint2* st = pairs + slot_base[slot] * 64 + lane;
  const uint32_t* of = off + (size_t)slot * (n_pieces + 1);
  const int nb = (int)of[n_pieces];
  int p = 0;
  uint32_t e1 = of[1], e2 = of[n_pieces < 2 ? n_pieces : 2];
  const char* const Hs = reinterpret_cast<const char*>(H + slice * NL_SLICE);
  const char* Hp = Hs;
  int seen = 0, since = 0;

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
          __builtin_amdgcn_s_sleep(8);
        }
        seen = c;
        if (spin == spin_max) {
          if (lane == 0)
            __hip_atomic_fetch_add(counter, NL_GIVE_UP, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          seen = INT_MAX;
        }
      }
    }
    if (since >= flush_every) {
      flush();
      since = 0;
    }
    e1 = e2;
    e2 = of[p + 2 < n_pieces ? p + 2 : n_pieces];
    Hp = Hs + (int64_t)p * piece_cols * (int64_t)r4;
  };

  if (nb > 0) {
    // Four batches of pairs are held (A: batch b, B: b + 1, C: b + 2, D: b + 3) and the loop is
    // unrolled over their four roles, so that no register is copied while its load is in flight.
    // Batch b's eight steps each add one gathered entry per lane group and then request the
    // gather of the same step of batch b + 1 into the registers just consumed: 7 or 8 gathers
    // are in flight at any time.  (nb is a multiple of 4.)
    uint2 A = st[0], B = st[64], C = st[128], D = st[192];
    while (0u >= e1) piece_done();
    float4 h[8];
    for_steps(std::make_integer_sequence<int, 8>{}, [&](auto k_tag) {
      constexpr int K = decltype(k_tag)::value;
      const int idx = bcast_pair<K>((int)A.x);
      h[K] = *reinterpret_cast<const float4*>(Hp + (__umul24((unsigned)idx & 0xffffu, r4) + sub16));
    });
    auto batch = [&](const uint2& cur, const uint2& nxt) {
      const char* const Hn = Hp;
      for_steps(std::make_integer_sequence<int, 8>{}, [&](auto k_tag) {
        constexpr int K = decltype(k_tag)::value;
        const unsigned idx = (unsigned)bcast_pair<K>((int)cur.x);
        const float v = __int_as_float(bcast_pair<K>((int)cur.y));
        float* a = reinterpret_cast<float*>(lds_lane + (idx >> 16));
        const float4 hv = h[K];
        atomicAdd(a, v * hv.x);
        atomicAdd(a + 8, v * hv.y);
        atomicAdd(a + 16, v * hv.z);
        atomicAdd(a + 24, v * hv.w);
        const int idn = bcast_pair<K>((int)nxt.x);
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

  flush();
  const int c = lane & 31;
#pragma unroll
  for (int i = 0; i < RPW2; i++) {
    const int lr = 2 * i + (lane >> 5);
    if (lr < rpw) {
      const int row = slot_rows[(size_t)slot * rpw + lr];
      if (row >= 0) N[(int64_t)row * r + slice * NL_SLICE + c] = coarse[i];
    }
  }
}

// ---------------------------------------------------------------------------
// A^T W in blocks of columns
// ---------------------------------------------------------------------------
// tb[b] = first column of block b; a block holds up to 64 consecutive columns of one aligned
// group of 64.  Workgroup w of a launch: XCD x = w mod 8 takes slice slice0 + x mod n_sl of the
// components and every (8 / n_sl)-th group of four blocks; a wave takes one block.
// T (row j - col0 for column j) receives every column of the blocks, empty ones as zeros.
__global__ void __launch_bounds__(256)
    k_spmm_t_lists(const int32_t* __restrict__ tb, int64_t blk0, int64_t blk1,
                   const int64_t* __restrict__ colptr, const int32_t* __restrict__ rowind,
                   const float* __restrict__ tvals, int r, int slice0, int n_sl,
                   const float* __restrict__ W, float* __restrict__ T, int64_t col0) {
  __shared__ __align__(16) float tiles[4][64 * NL_ROW_FLOATS];
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

  // column offsets of the block, relative to its first entry: lane l holds that of column l
  const int64_t cp = colptr[j0 + (lane < nc ? lane : nc)];
  const int64_t e0 = __shfl(cp, 0);
  const int64_t e_end = colptr[j0 + nc];
  const int L = (int)(e_end - e0);
  const int rel = lane < nc ? (int)(cp - e0) : INT_MAX;
  for (int i = lane; i < nc * NL_ROW_FLOATS; i += 64) tile[i] = 0.0f;

  if (L > 0) {
    // lane group g takes entries [g Lg, (g + 1) Lg) of the block, eight at a time (one per lane)
    const int Lg = (L + 7) / 8;
    const int g0 = grp * Lg, g1 = g0 + Lg < L ? g0 + Lg : L;
    const int nbt = (Lg + 7) / 8;
    const int32_t* ri = rowind + e0;
    const float* tv = tvals + e0;
    // (local column << 24 | row, value) of the lane's entry of batch t; lanes past the group's
    // entries hold (last column of the block, row 0, 0.0f)
    auto fetch = [&](int t, int& pk, float& v) {
      const int qe = g0 + 8 * t + sub;
      const bool ok = qe < g1;
      // (unconditional loads at a clamped position: a load under a branch would make every later
      // wait for a gather a wait for all outstanding loads)
      const int qc = qe < L ? qe : L - 1;
      const int row = ok ? ri[qc] : 0;
      v = ok ? tv[qc] : 0.0f;
      int lo = 0;  // largest column c with rel[c] <= qe
#pragma unroll
      for (int step = 32; step >= 1; step >>= 1) {
        const int mid = lo + step;
        const int rv = __shfl(rel, mid & 63);
        if (mid < 64 && rv <= qe) lo = mid;
      }
      pk = ((ok ? lo : nc - 1) << 24) | row;
    };
    int cpk, npk;
    float cv, nv;
    fetch(0, cpk, cv);
    fetch(1, npk, nv);
    float4 h[8];
    for_steps(std::make_integer_sequence<int, 8>{}, [&](auto k_tag) {
      constexpr int K = decltype(k_tag)::value;
      const unsigned pk = (unsigned)bcast_octet<K>(cpk);
      h[K] = *reinterpret_cast<const float4*>(Ws + (__umul24(pk & 0xffffffu, r4) + sub16));
    });
    float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    int cur = (int)((unsigned)bcast_octet<0>(cpk) >> 24);
    for (int t = 0; t < nbt; t++) {
      int fpk;
      float fv;
      fetch(t + 2, fpk, fv);
      for_steps(std::make_integer_sequence<int, 8>{}, [&](auto k_tag) {
        constexpr int K = decltype(k_tag)::value;
        const int c = (int)((unsigned)bcast_octet<K>(cpk) >> 24);
        const float v = __int_as_float(bcast_octet<K>(__float_as_int(cv)));
        const float4 hv = h[K];
        if (c != cur) {
          float* a = tile + cur * NL_ROW_FLOATS + sub;
          atomicAdd(a, acc.x);
          atomicAdd(a + 8, acc.y);
          atomicAdd(a + 16, acc.z);
          atomicAdd(a + 24, acc.w);
          acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
          cur = c;
        }
        acc.x = fmaf(v, hv.x, acc.x);
        acc.y = fmaf(v, hv.y, acc.y);
        acc.z = fmaf(v, hv.z, acc.z);
        acc.w = fmaf(v, hv.w, acc.w);
        const unsigned pk = (unsigned)bcast_octet<K>(npk);
        h[K] = *reinterpret_cast<const float4*>(Ws + (__umul24(pk & 0xffffffu, r4) + sub16));
      });
      cpk = npk; cv = nv;
      npk = fpk; nv = fv;
    }
    float* a = tile + cur * NL_ROW_FLOATS + sub;
    atomicAdd(a, acc.x);
    atomicAdd(a + 8, acc.y);
    atomicAdd(a + 16, acc.z);
    atomicAdd(a + 24, acc.w);
  }
  // the tile's rows to T: a lane group writes the 128 bytes of one column
  for (int c = grp; c < nc; c += 8) {
    const float* a = tile + c * NL_ROW_FLOATS + sub;
    const float4 o = make_float4(a[0], a[8], a[16], a[24]);
    *reinterpret_cast<float4*>(T + ((int64_t)(j0 + c) - col0) * r + slice * NL_SLICE + 4 * sub) = o;
  }
}

// ---------------------------------------------------------------------------
// Building the slot lists from the transposed copy
// ---------------------------------------------------------------------------
// Piece p: columns [p piece_cols, (p + 1) piece_cols), entries [pe[p], pe[p + 1]) of the
// transposed copy, cut into chunks of NL_CHUNK entries; chunk_first[p] = chunks before piece p.
__device__ inline int piece_of_chunk(const int32_t* __restrict__ chunk_first, int n_pieces, int chunk) {
  int lo = 0, hi = n_pieces;  // largest p with chunk_first[p] <= chunk
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (chunk_first[mid] <= chunk) lo = mid; else hi = mid;
  }
  return lo;
}

// hist[chunk][slot] = entries of the chunk whose row belongs to the slot (one wave per chunk)
__global__ void __launch_bounds__(64)
    k_nl_chunk_hist(const int32_t* __restrict__ rowind, const int32_t* __restrict__ row_slot,
                    const int64_t* __restrict__ pe, const int32_t* __restrict__ chunk_first, int n_pieces,
                    int n_slots, uint32_t* __restrict__ hist) {
  extern __shared__ int nl_cnt[];
  const int chunk = blockIdx.x, lane = threadIdx.x;
  const int p = piece_of_chunk(chunk_first, n_pieces, chunk);
  const int64_t e0 = pe[p] + (int64_t)(chunk - chunk_first[p]) * NL_CHUNK;
  const int64_t e1 = e0 + NL_CHUNK < pe[p + 1] ? e0 + NL_CHUNK : pe[p + 1];
  for (int s = lane; s < n_slots; s += 64) nl_cnt[s] = 0;
  __syncthreads();
  for (int64_t e = e0 + lane; e < e1; e += 64) atomicAdd(&nl_cnt[row_slot[rowind[e]] >> 7], 1);
  __syncthreads();
  for (int s = lane; s < n_slots; s += 64) hist[(size_t)chunk * n_slots + s] = (uint32_t)nl_cnt[s];
}

// hist[chunk][slot] -> entries of the slot in the earlier chunks of the same piece;
// cnt[slot][piece] = entries of (slot, piece)
__global__ void __launch_bounds__(256)
    k_nl_piece_scan(const int32_t* __restrict__ chunk_first, int n_pieces, int n_slots,
                    uint32_t* __restrict__ hist, uint32_t* __restrict__ cnt) {
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= (int64_t)n_pieces * n_slots) return;
  const int p = (int)(id / n_slots), s = (int)(id % n_slots);
  uint32_t run = 0;
  for (int c = chunk_first[p]; c < chunk_first[p + 1]; c++) {
    const uint32_t t = hist[(size_t)c * n_slots + s];
    hist[(size_t)c * n_slots + s] = run;
    run += t;
  }
  cnt[(size_t)s * n_pieces + p] = run;
}

// off[slot][p] = batches of 64 of the slot's pieces before p (one workgroup per slot)
__global__ void __launch_bounds__(256)
    k_nl_slot_scan(const uint32_t* __restrict__ cnt, int n_pieces, uint32_t* __restrict__ off) {
  __shared__ uint32_t runs[256];
  const int s = blockIdx.x, tid = threadIdx.x;
  const int per = (n_pieces + 255) / 256, p0 = tid * per;
  const uint32_t* c = cnt + (size_t)s * n_pieces;
  uint32_t sum = 0;
  for (int p = p0; p < p0 + per && p < n_pieces; p++) sum += (c[p] + 63u) / 64u;
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
    run += (c[p] + 63u) / 64u;
  }
  // (the thread of the last piece) the kernel takes the batches of a slot four at a time
  if (p0 < n_pieces && p0 + per >= n_pieces) o[n_pieces] = (run + 3u) / 4u * 4u;
  if (n_pieces == 0 && tid == 0) o[0] = 0;
}

// The entries of a chunk into the lists, in the order of the transposed copy (one wave per
// chunk): an entry's place in the list of (slot, piece) is the number of entries of that slot in
// the earlier chunks of the piece (hist) plus those before it in this chunk.  Within a batch of
// 64 entries the rank among the entries of the same slot comes from ballots over the bits of the
// slot number.
__global__ void __launch_bounds__(64)
    k_nl_scatter(const int64_t* __restrict__ colptr, const int32_t* __restrict__ rowind,
                 const float* __restrict__ tvals, const int32_t* __restrict__ row_slot,
                 const int64_t* __restrict__ pe, const int32_t* __restrict__ chunk_first, int n_pieces,
                 int piece_cols, int64_t n_cols, int n_slots, int slot_bits,
                 const uint32_t* __restrict__ hist, const int64_t* __restrict__ slot_base,
                 const uint32_t* __restrict__ off, uint2* __restrict__ pairs) {
  extern __shared__ int nl_cnt[];  // cursor[slot]
  const int chunk = blockIdx.x, lane = threadIdx.x;
  const int p = piece_of_chunk(chunk_first, n_pieces, chunk);
  const int64_t e0 = pe[p] + (int64_t)(chunk - chunk_first[p]) * NL_CHUNK;
  const int64_t e1 = e0 + NL_CHUNK < pe[p + 1] ? e0 + NL_CHUNK : pe[p + 1];
  for (int s = lane; s < n_slots; s += 64) nl_cnt[s] = (int)hist[(size_t)chunk * n_slots + s];
  __syncthreads();
  const int64_t j_lo = (int64_t)p * piece_cols;
  const int64_t j_hi = j_lo + piece_cols < n_cols ? j_lo + piece_cols : n_cols;
  for (int64_t base = e0; base < e1; base += 64) {
    const int64_t e = base + lane;
    const bool active = e < e1;
    int slot = 0, lrow = 0, lcol = 0;
    float v = 0.0f;
    if (active) {
      const int rs = row_slot[rowind[e]];
      slot = rs >> 7;
      lrow = rs & 127;
      v = tvals[e];
      int64_t lo = j_lo, hi = j_hi;  // largest column j in [j_lo, j_hi) with colptr[j] <= e
      while (hi - lo > 1) {
        const int64_t mid = (lo + hi) >> 1;
        if (colptr[mid] <= e) lo = mid; else hi = mid;
      }
      lcol = (int)(lo - j_lo);
    }
    unsigned long long mask = __ballot(active);
    for (int b = 0; b < slot_bits; b++) {
      const bool bit = (slot >> b) & 1;
      const unsigned long long bal = __ballot(active && bit);
      mask &= bit ? bal : ~bal;
    }
    const int rank = __popcll(mask & ((1ull << lane) - 1ull));
    int at = 0;
    if (active) at = nl_cnt[slot] + rank;
    __syncthreads();
    if (active) {
      if (rank == 0) nl_cnt[slot] += __popcll(mask);
      const int64_t dst = (slot_base[slot] + off[(size_t)slot * (n_pieces + 1) + p]) * 64 + at;
      pairs[dst] = make_uint2(((unsigned)(lrow * NL_ROW_BYTES) << 16) | (unsigned)lcol, __float_as_uint(v));
    }
    __syncthreads();
  }
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
static int nlists_parts(int64_t n_rows, int r) {
  const int n_slices = r / NL_SLICE;
  int parts = (int)ceil_div(n_rows, (int64_t)NL_SLOTS * NL_RPW_MAX);
  if (n_slices < SWEEP_XCDS && SWEEP_XCDS % n_slices == 0 && parts < SWEEP_XCDS / n_slices)
    parts = SWEEP_XCDS / n_slices;
  return parts < 1 ? 1 : parts;
}

bool nlists_supported(const dnpeff_csr* S, int r) {
  if (r < NL_SLICE || r % NL_SLICE != 0 || r > 1024) return false;
  if (S->n_rows < 1 || S->n_rows >= ((int64_t)1 << 24) || S->nnz < 1) return false;
  return (int64_t)nlists_parts(S->n_rows, r) * NL_SLOTS <= NL_MAX_SLOTS;
}

int nlists_build(dnpeff_csr* S, int r) {
  const tuning_t& tn = tuning();
  int piece_cols = (int)tn.nl_piece_cols;
  if (piece_cols < 64) piece_cols = 64;
  if (piece_cols > 65536) piece_cols = 65536;
  const int n_parts = nlists_parts(S->n_rows, r);
  slot_lists& L = S->nl;
  if (L.pairs && L.piece_cols == piece_cols && L.n_parts == n_parts) return 0;
  nlists_drop(S);
  DN_CHECK(nlists_supported(S, r), "no slot lists for %lld rows at rank %d", (long long)S->n_rows, r);
  DN_CHECK(S->colptr && S->rowind && S->tvals && S->rowptr, "slot lists need the transposed copy");
  hipStream_t st = stream();
  const int64_t n = S->n_rows, m = S->n_cols, z = S->nnz;
  const int n_slots = n_parts * NL_SLOTS;
  const int rpw = (int)ceil_div(n, n_slots);
  DN_CHECK(rpw <= NL_RPW_MAX, "slot lists: %d rows per slot", rpw);
  const int64_t n_pieces64 = ceil_div(m, piece_cols);
  DN_CHECK(n_pieces64 < (1 << 22), "slot lists: too many pieces");
  const int n_pieces = (int)n_pieces64;

  // rows to slots: longest first, dealt back and forth over the slots, so that the slots hold
  // about the same number of entries (all slots of an XCD advance piece by piece together)
  std::vector<int64_t> rowptr((size_t)n + 1);
  DN_HIP(hipStreamSynchronize(st));
  DN_HIP(hipMemcpy(rowptr.data(), S->rowptr, sizeof(int64_t) * (n + 1), hipMemcpyDeviceToHost));
  std::vector<int32_t> order((size_t)n), row_slot((size_t)n), slot_rows((size_t)n_slots * rpw, -1);
  for (int64_t i = 0; i < n; i++) order[(size_t)i] = (int32_t)i;
  std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) {
    return rowptr[(size_t)a + 1] - rowptr[(size_t)a] > rowptr[(size_t)b + 1] - rowptr[(size_t)b];
  });
  for (int64_t t = 0; t < n; t++) {
    const int round = (int)(t / n_slots), pos = (int)(t % n_slots);
    const int slot = (round & 1) ? n_slots - 1 - pos : pos;
    row_slot[(size_t)order[(size_t)t]] = slot * 128 + round;
    slot_rows[(size_t)slot * rpw + round] = order[(size_t)t];
  }

  // entry ranges of the pieces and their chunks
  std::vector<int64_t> pe((size_t)n_pieces + 1);
  if (n_pieces > 0)
    DN_HIP(hipMemcpy2D(pe.data(), sizeof(int64_t), S->colptr, sizeof(int64_t) * (size_t)piece_cols,
                       sizeof(int64_t), (size_t)n_pieces, hipMemcpyDeviceToHost));
  pe[(size_t)n_pieces] = z;
  std::vector<int32_t> chunk_first((size_t)n_pieces + 1);
  int64_t n_chunks = 0;
  for (int p = 0; p < n_pieces; p++) {
    chunk_first[(size_t)p] = (int32_t)n_chunks;
    n_chunks += ceil_div(pe[(size_t)p + 1] - pe[(size_t)p], NL_CHUNK);
    DN_CHECK(n_chunks < INT32_MAX, "slot lists: too many chunks");
  }
  chunk_first[(size_t)n_pieces] = (int32_t)n_chunks;

  dbuf<int64_t> d_pe;
  dbuf<int32_t> d_cf;
  dbuf<uint32_t> hist, cnt;
  DN_TRY(dmalloc(&L.row_slot, n));
  DN_TRY(dmalloc(&L.slot_rows, (int64_t)n_slots * rpw));
  DN_TRY(dmalloc(&L.off, (int64_t)n_slots * (n_pieces + 1)));
  DN_TRY(dmalloc(&L.slot_base, (int64_t)n_slots + 1));
  DN_TRY(dmalloc(&L.progress, SWEEP_XCDS * NL_SYNC_STRIDE));
  DN_TRY(d_pe.alloc(n_pieces + 1));
  DN_TRY(d_cf.alloc(n_pieces + 1));
  DN_TRY(hist.alloc(n_chunks * n_slots));
  DN_TRY(cnt.alloc((int64_t)n_slots * n_pieces));
  DN_HIP(hipMemcpy(L.row_slot, row_slot.data(), sizeof(int32_t) * n, hipMemcpyHostToDevice));
  DN_HIP(hipMemcpy(L.slot_rows, slot_rows.data(), sizeof(int32_t) * slot_rows.size(), hipMemcpyHostToDevice));
  DN_HIP(hipMemcpy(d_pe.p, pe.data(), sizeof(int64_t) * pe.size(), hipMemcpyHostToDevice));
  DN_HIP(hipMemcpy(d_cf.p, chunk_first.data(), sizeof(int32_t) * chunk_first.size(), hipMemcpyHostToDevice));
  const size_t lds = sizeof(int) * (size_t)n_slots;
  if (n_chunks > 0) {
    hipLaunchKernelGGL(k_nl_chunk_hist, dim3((unsigned)n_chunks), dim3(64), lds, st, S->rowind, L.row_slot,
                       d_pe.p, d_cf.p, n_pieces, n_slots, hist.p);
    DN_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL(k_nl_piece_scan, dim3((unsigned)ceil_div((int64_t)n_pieces * n_slots, 256)), dim3(256), 0,
                     st, d_cf.p, n_pieces, n_slots, hist.p, cnt.p);
  DN_LAUNCH_CHECK();
  hipLaunchKernelGGL(k_nl_slot_scan, dim3((unsigned)n_slots), dim3(256), 0, st, cnt.p, n_pieces, L.off);
  DN_LAUNCH_CHECK();
  DN_HIP(hipStreamSynchronize(st));
  // batches of the slots -> first batch of each slot
  std::vector<uint32_t> tot((size_t)n_slots);
  DN_HIP(hipMemcpy2D(tot.data(), sizeof(uint32_t), L.off + n_pieces, sizeof(uint32_t) * (size_t)(n_pieces + 1),
                     sizeof(uint32_t), (size_t)n_slots, hipMemcpyDeviceToHost));
  L.h_slot_base.assign((size_t)n_slots + 1, 0);
  for (int s = 0; s < n_slots; s++) L.h_slot_base[(size_t)s + 1] = L.h_slot_base[(size_t)s] + tot[(size_t)s];
  const int64_t n_batches = L.h_slot_base[(size_t)n_slots];
  DN_HIP(hipMemcpy(L.slot_base, L.h_slot_base.data(), sizeof(int64_t) * ((size_t)n_slots + 1),
                   hipMemcpyHostToDevice));
  // (the kernel requests pairs up to seven batches past a slot's last)
  DN_TRY(dmalloc(&L.pairs, (n_batches + 8) * 64));
  DN_HIP(hipMemsetAsync(L.pairs, 0, sizeof(uint2) * (size_t)(n_batches + 8) * 64, st));
  int slot_bits = 0;
  while ((1 << slot_bits) < n_slots) slot_bits++;
  if (n_chunks > 0) {
    hipLaunchKernelGGL(k_nl_scatter, dim3((unsigned)n_chunks), dim3(64), lds, st, S->colptr, S->rowind,
                       S->tvals, L.row_slot, d_pe.p, d_cf.p, n_pieces, piece_cols, m, n_slots, slot_bits,
                       hist.p, L.slot_base, L.off, L.pairs);
    DN_LAUNCH_CHECK();
  }
  DN_HIP(hipStreamSynchronize(st));
  L.piece_cols = piece_cols;
  L.n_pieces = n_pieces;
  L.n_parts = n_parts;
  L.rpw = rpw;
  L.n_batches = n_batches;
  L.h_row_slot = std::move(row_slot);
  if (tn.verbose != 0.0)
    fprintf(stderr,
            "dnpeff: slot lists: %d part(s) x %d slots of %d rows, %d pieces of %d columns, %lld batches "
            "(%.1f %% padding), %.2f GB\n",
            n_parts, NL_SLOTS, rpw, n_pieces, piece_cols, (long long)n_batches,
            z > 0 ? 100.0 * ((double)n_batches * 64.0 / (double)z - 1.0) : 0.0,
            (double)(n_batches + 8) * 512.0 / 1e9);
  return 0;
}

using nl_kernel_t = void (*)(const uint2*, const int64_t*, const uint32_t*, int, int, const int32_t*, int, int,
                             int, int, int, const float*, float*, int*, int, int, int);

__global__ void k_nl_clear(int* progress) { progress[threadIdx.x] = 0; }

// part[row, :] = the sparse part's share of (A H^T)[row, :]
int launch_spmm_n_lists(const dnpeff_csr* S, int r, const float* H_mr, float* part) {
  const slot_lists& L = S->nl;
  DN_CHECK(L.pairs != nullptr, "matrix has no slot lists");
  DN_CHECK(r % NL_SLICE == 0 && ((uintptr_t)H_mr % 16) == 0, "slot lists: rank %d or alignment", r);
  DN_CHECK(L.n_parts == nlists_parts(S->n_rows, r), "slot lists were built for another rank");
  static const nl_kernel_t kernels[6] = {k_spmm_n_lists<4>,  k_spmm_n_lists<8>,  k_spmm_n_lists<12>,
                                         k_spmm_n_lists<20>, k_spmm_n_lists<28>, k_spmm_n_lists<36>};
  static const int sizes[6] = {4, 8, 12, 20, 28, 36};
  static bool attr_set[6] = {false, false, false, false, false, false};
  int v = 0;
  while (v < 5 && 2 * sizes[v] < L.rpw) v++;
  DN_CHECK(2 * sizes[v] >= L.rpw, "slot lists: %d rows per slot", L.rpw);
  const size_t lds = (size_t)NL_WAVES * L.rpw * NL_ROW_BYTES;
  if (!attr_set[v]) {
    DN_HIP(hipFuncSetAttribute((const void*)kernels[v], hipFuncAttributeMaxDynamicSharedMemorySize,
                               NL_WAVES * NL_RPW_MAX * NL_ROW_BYTES));
    attr_set[v] = true;
  }
  const tuning_t& tn = tuning();
  int lag = (int)tn.nl_lag, spin_max = (int)tn.sweep_spin, flush_every = (int)tn.nl_flush;
  if (lag < 0) lag = 0;
  if (flush_every < 1) flush_every = 1;
  const int n_slices = r / NL_SLICE, n_units = n_slices * L.n_parts;
  for (int unit0 = 0; unit0 < n_units; unit0 += SWEEP_XCDS) {
    hipLaunchKernelGGL(k_nl_clear, dim3(1), dim3(SWEEP_XCDS * NL_SYNC_STRIDE), 0, stream(), L.progress);
    hipLaunchKernelGGL(kernels[v], dim3(SWEEP_XCDS * NL_WGS), dim3(64 * NL_WAVES), lds, stream(), L.pairs,
                       L.slot_base, L.off, L.n_pieces, L.piece_cols, L.slot_rows, L.rpw, unit0, n_units,
                       n_slices, r, H_mr, part, L.progress, lag, spin_max, flush_every);
    DN_LAUNCH_CHECK();
  }
  return 0;
}

// The sparse part's entries of one row, from the lists (column ids in ascending order).
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
  for (int p = 0; p < L.n_pieces; p++)
    for (size_t i = (size_t)off[(size_t)p] * 64; i < (size_t)off[(size_t)p + 1] * 64; i++) {
      const uint2 e = pairs[i];
      // a padding pair is all zeros: local row 0, column 0, value +0.0 (no entry holds a zero)
      if ((int)(e.x >> 16) == lrow * NL_ROW_BYTES && !(e.x == 0u && e.y == 0u)) {
        cols.push_back((int32_t)((int64_t)p * L.piece_cols + (e.x & 0xffffu)));
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
