// Per-example top-k of dense Fisher rows on the device: the sparsifier that produces the PEF
// rows the loader reads (values and indices of the k largest entries in descending order, equal
// values in ascending index order, plus the L2 norm of the whole row), i.e. what
// npeff/fishers/d_pefs_computer.py:126-129 gets from tf.math.top_k and :48-50 from the einsum.
//
// A row has ~1e8 entries and k ~ 6.5e4, so sorting the row is out of the question.  Usual case,
// two reads of the row:
//   1. a histogram of the top 11 bits of an order-preserving integer key (and the sum of
//      squares for the norm) finds the bin that holds the k-th largest entry;
//   2. every entry in that bin or above it goes to a candidate list ((key, index) pairs, any
//      order), typically k plus one bin's worth of entries;
//   3. a bitonic sort of the candidates (strides below 4096 inside LDS, the others in global
//      memory) orders them by value and index; the first k are the result.
// If the k-th entry's bin is crowded, one or two more histogram passes (11 + 10 bits) narrow
// it down first; if even the entries equal to the exact key T of the k-th entry are too many to
// sort, the entries above T and the first `need` entries equal to T in index order (a predicate
// scan) are the candidates.  Everything but the norm is integer work; nothing depends on scheduling.
#include "dnpeff_internal.hpp"
#include "scan.hpp"

#include <cstdlib>
#include <vector>

namespace dn {

// Order-preserving key of a float: larger float <=> larger unsigned key (NaNs sort above +inf).
__device__ inline uint32_t sort_key(float x) {
  const uint32_t b = __float_as_uint(x);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ inline float key_to_float(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

struct TopkState {
  uint32_t prefix;  // bits of T decided so far
  uint32_t mask;    // which bits those are
  int64_t need;     // entries still to take among those matching the prefix
  int64_t cursor;   // next free candidate slot (compaction)
  int64_t in_bin;   // entries in the bin picked last
};

constexpr int TOPK_BINS = 2048;

__global__ void __launch_bounds__(256) k_topk_init(TopkState* st, int64_t k) {
  st[blockIdx.x] = TopkState{0u, 0u, k, 0, 0};
}

// hist[row][bin] += entries of the row whose decided bits match and whose next `bits` bits are bin
template <bool VEC4>
__global__ void __launch_bounds__(256)
    k_topk_hist(const float* __restrict__ x, int64_t count, int shift, int bits,
                const TopkState* __restrict__ st, unsigned* __restrict__ hist,
                double* __restrict__ sq_partials) {
  __shared__ unsigned h[TOPK_BINS];
  __shared__ double red[256];
  double sq = 0.0;
  const int row = blockIdx.y;
  const uint32_t prefix = st[row].prefix, mask = st[row].mask;
  const unsigned nb = 1u << bits;
  for (unsigned i = threadIdx.x; i < nb; i += 256) h[i] = 0;
  __syncthreads();
  const float* xr = x + (int64_t)row * count;
  const int64_t stride = (int64_t)gridDim.x * 256;
  auto one = [&](float v) {
    const uint32_t key = sort_key(v);
    if ((key & mask) == prefix) atomicAdd(&h[(key >> shift) & (nb - 1)], 1u);
    sq += (double)v * (double)v;
  };
  if (VEC4) {  // count % 4 == 0 and x 16-byte aligned: four entries per load
    const float4* x4 = reinterpret_cast<const float4*>(xr);
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count / 4; i += stride) {
      const float4 v = x4[i];
      one(v.x); one(v.y); one(v.z); one(v.w);
    }
  } else {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += stride) one(xr[i]);
  }
  __syncthreads();
  for (unsigned i = threadIdx.x; i < nb; i += 256)
    if (h[i]) atomicAdd(&hist[(int64_t)row * TOPK_BINS + i], h[i]);
  if (sq_partials) {  // fixed tree inside the block, blocks summed in order by k_topk_norm
    red[threadIdx.x] = sq;
    __syncthreads();
    for (int off = 128; off > 0; off >>= 1) {
      if ((int)threadIdx.x < off) red[threadIdx.x] += red[threadIdx.x + off];
      __syncthreads();
    }
    if (threadIdx.x == 0) sq_partials[(int64_t)row * gridDim.x + blockIdx.x] = red[0];
  }
}

__global__ void __launch_bounds__(64)
    k_topk_norm(const double* __restrict__ sq_partials, int n_partials, float* __restrict__ norms) {
  if (threadIdx.x != 0) return;
  double s = 0.0;
  for (int i = 0; i < n_partials; i++) s += sq_partials[(int64_t)blockIdx.x * n_partials + i];
  norms[blockIdx.x] = (float)sqrt(s);
}

// Walks the bins from the top until `need` entries are covered; fixes the next bits of T.
__global__ void __launch_bounds__(64)
    k_topk_pick(unsigned* __restrict__ hist, int shift, int bits, TopkState* __restrict__ st) {
  const int row = blockIdx.x;
  unsigned* h = hist + (int64_t)row * TOPK_BINS;
  if (threadIdx.x == 0) {
    TopkState s = st[row];
    const int nb = 1 << bits;
    int64_t above = 0;
    int b = nb - 1;
    for (; b > 0; b--) {
      if (above + h[b] >= s.need) break;
      above += h[b];
    }
    s.prefix |= (uint32_t)b << shift;
    s.mask |= (uint32_t)(nb - 1) << shift;
    s.need -= above;
    s.in_bin = h[b];
    st[row] = s;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < TOPK_BINS; i += 64) h[i] = 0;
}

// Fast path: entries whose decided bits are >= the picked prefix (the k-th entry's bin and all
// bins above it) go to the candidate list; the slots past them are padded with the smallest pair.
// A workgroup collects its finds in LDS and reserves room in the list with one atomic per
// 1024+ finds: the finds are sparse (k of ~1e8), and one global atomic each on a single counter
// would serialise them.
template <bool VEC4>
__global__ void __launch_bounds__(256)
    k_topk_take_bins(const float* __restrict__ x, int64_t count, TopkState* __restrict__ st,
                     uint64_t* __restrict__ cand, int64_t kp, int64_t k) {
  __shared__ uint64_t buf[2048];
  __shared__ unsigned cnt;
  __shared__ unsigned long long gbase;
  const int row = blockIdx.y;
  const uint32_t prefix = st[row].prefix, mask = st[row].mask;
  const int64_t n_cand = k - st[row].need + st[row].in_bin;
  const float* xr = x + (int64_t)row * count;
  uint64_t* out = cand + (int64_t)row * kp;
  unsigned long long* cursor = reinterpret_cast<unsigned long long*>(&st[row].cursor);
  if (threadIdx.x == 0) cnt = 0;
  __syncthreads();
  auto one = [&](float v, int64_t i) {
    const uint32_t key = sort_key(v);
    if ((key & mask) >= prefix)
      buf[atomicAdd(&cnt, 1u)] = ((uint64_t)key << 32) | (uint32_t)(0xffffffffu - (uint32_t)i);
  };
  auto flush = [&]() {  // called by the whole workgroup
    if (threadIdx.x == 0) gbase = atomicAdd(cursor, (unsigned long long)cnt);
    __syncthreads();
    for (unsigned i = threadIdx.x; i < cnt; i += 256) out[gbase + i] = buf[i];
    __syncthreads();
    if (threadIdx.x == 0) cnt = 0;
    __syncthreads();
  };
  // every thread of the workgroup runs the same number of iterations; an iteration adds at
  // most 1024 finds
  const int64_t units = VEC4 ? count / 4 : count;
  const int per = VEC4 ? 1 : 4;  // units per thread and iteration
  const int64_t step = (int64_t)gridDim.x * 256 * per;
  for (int64_t base = (int64_t)blockIdx.x * 256 * per; base < units; base += step) {
    if (VEC4) {
      const int64_t i = base + threadIdx.x;
      if (i < units) {
        const float4 v = reinterpret_cast<const float4*>(xr)[i];
        one(v.x, 4 * i); one(v.y, 4 * i + 1); one(v.z, 4 * i + 2); one(v.w, 4 * i + 3);
      }
    } else {
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int64_t i = base + threadIdx.x + 256 * u;
        if (i < units) one(xr[i], i);
      }
    }
    __syncthreads();
    if (cnt > 1024) flush();
  }
  if (cnt > 0) flush();
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = n_cand + (int64_t)blockIdx.x * 256 + threadIdx.x; i < kp; i += stride) out[i] = 0;
}

// Entries above T go to the candidate list in any order (the sort fixes it).
__global__ void __launch_bounds__(256)
    k_topk_take_above(const float* __restrict__ x, int64_t count, TopkState* __restrict__ st,
                      uint64_t* __restrict__ cand, int64_t kp) {
  const int row = blockIdx.y;
  const uint32_t T = st[row].prefix;
  const float* xr = x + (int64_t)row * count;
  unsigned long long* cursor = reinterpret_cast<unsigned long long*>(&st[row].cursor);
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += stride) {
    const uint32_t key = sort_key(xr[i]);
    if (key > T) {
      const unsigned long long slot = atomicAdd(cursor, 1ull);
      cand[(int64_t)row * kp + slot] = ((uint64_t)key << 32) | (uint32_t)(0xffffffffu - (uint32_t)i);
    }
  }
}

// Entries equal to T, numbered in index order by `rank` (an exclusive scan of the predicate):
// the first `need` of them complete the list; the slots past k are padded with the smallest pair.
__global__ void __launch_bounds__(256)
    k_topk_take_ties(const float* __restrict__ xr, int64_t count, const TopkState* __restrict__ st_row,
                     const int64_t* __restrict__ rank, uint64_t* __restrict__ cand_row, int64_t k,
                     int64_t kp) {
  const uint32_t T = st_row->prefix;
  const int64_t need = st_row->need, base = k - need;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += stride) {
    if (sort_key(xr[i]) == T && rank[i] < need)
      cand_row[base + rank[i]] = ((uint64_t)T << 32) | (uint32_t)(0xffffffffu - (uint32_t)i);
  }
  for (int64_t i = k + (int64_t)blockIdx.x * 256 + threadIdx.x; i < kp; i += stride) cand_row[i] = 0;
}

struct TieF {
  const float* x;
  const TopkState* st;
  __device__ int64_t operator()(int64_t i) const { return sort_key(x[i]) == st->prefix ? 1 : 0; }
};

// ---- bitonic sort, descending, of kp (a power of two) pairs per row ----
constexpr int BITONIC_CHUNK = 4096;

__device__ inline void cmp_swap_desc(uint64_t& a, uint64_t& b, bool descending) {
  if ((a < b) == descending) {
    const uint64_t t = a;
    a = b;
    b = t;
  }
}

// All merge steps with stride < BITONIC_CHUNK of the stages size_lo .. size_hi, inside LDS.
__global__ void __launch_bounds__(256)
    k_bitonic_local(uint64_t* __restrict__ data, int64_t kp, int64_t size_lo, int64_t size_hi) {
  __shared__ uint64_t s[BITONIC_CHUNK];
  uint64_t* d = data + (int64_t)blockIdx.y * kp + (int64_t)blockIdx.x * BITONIC_CHUNK;
  const int64_t g0 = (int64_t)blockIdx.x * BITONIC_CHUNK;
  const int n = kp < BITONIC_CHUNK ? (int)kp : BITONIC_CHUNK;
  for (int i = threadIdx.x; i < n; i += 256) s[i] = d[i];
  __syncthreads();
  for (int64_t size = size_lo; size <= size_hi; size <<= 1) {
    int64_t j = size >> 1;
    if (j >= BITONIC_CHUNK) j = BITONIC_CHUNK >> 1;
    for (; j > 0; j >>= 1) {
      for (int t = threadIdx.x; t < n / 2; t += 256) {
        const int lo = (int)(((int64_t)t / j) * 2 * j + t % j), hi = lo + (int)j;
        const bool desc = ((g0 + lo) & size) == 0;
        cmp_swap_desc(s[lo], s[hi], desc);
      }
      __syncthreads();
    }
  }
  for (int i = threadIdx.x; i < n; i += 256) d[i] = s[i];
}

// One merge step with stride j >= BITONIC_CHUNK of stage `size`.
__global__ void __launch_bounds__(256)
    k_bitonic_global(uint64_t* __restrict__ data, int64_t kp, int64_t size, int64_t j) {
  uint64_t* d = data + (int64_t)blockIdx.y * kp;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < kp / 2; t += stride) {
    const int64_t lo = (t / j) * 2 * j + t % j, hi = lo + j;
    uint64_t a = d[lo], b = d[hi];
    cmp_swap_desc(a, b, (lo & size) == 0);
    d[lo] = a;
    d[hi] = b;
  }
}

__global__ void __launch_bounds__(256)
    k_topk_emit(const uint64_t* __restrict__ cand, int64_t k, int64_t kp, float* __restrict__ vals,
                int32_t* __restrict__ idx) {
  const int row = blockIdx.y;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < k; i += stride) {
    const uint64_t c = cand[(int64_t)row * kp + i];
    vals[(int64_t)row * k + i] = key_to_float((uint32_t)(c >> 32));
    idx[(int64_t)row * k + i] = (int32_t)(0xffffffffu - (uint32_t)c);
  }
}

}  // namespace dn

using namespace dn;

// Candidate lists longer than this (k plus the k-th entry's bin) take the exact-threshold path.
constexpr int64_t TOPK_FAST_CAP = (int64_t)1 << 21;

static int bitonic_sort_rows(uint64_t* cand, int64_t kp, int64_t n_rows) {
  hipStream_t st = stream();
  const dim3 block(256);
  const unsigned chunks = (unsigned)ceil_div(kp, BITONIC_CHUNK);
  const int64_t local_hi = kp < BITONIC_CHUNK ? kp : BITONIC_CHUNK;
  hipLaunchKernelGGL(k_bitonic_local, dim3(chunks, (unsigned)n_rows), block, 0, st, cand, kp, (int64_t)2,
                     local_hi);
  unsigned gg = (unsigned)ceil_div(kp / 2, 256);
  if (gg > 4096) gg = 4096;
  if (gg < 1) gg = 1;
  for (int64_t size = 2 * (int64_t)BITONIC_CHUNK; size <= kp; size <<= 1) {
    for (int64_t j = size >> 1; j >= BITONIC_CHUNK; j >>= 1)
      hipLaunchKernelGGL(k_bitonic_global, dim3(gg, (unsigned)n_rows), block, 0, st, cand, kp, size, j);
    hipLaunchKernelGGL(k_bitonic_local, dim3(chunks, (unsigned)n_rows), block, 0, st, cand, kp, size, size);
  }
  DN_LAUNCH_CHECK();
  return 0;
}

DN_API int dnpeff_topk_rows(int64_t n_rows, int64_t count, int64_t k, const float* x, float* vals_out,
                            int32_t* idx_out, float* norms_out) {
  clear_error();
  DN_CHECK(n_rows >= 0 && n_rows <= 65535, "n_rows %lld outside [0, 65535]", (long long)n_rows);
  DN_CHECK(count >= 1 && count <= (int64_t)INT32_MAX, "count %lld outside [1, 2^31)", (long long)count);
  DN_CHECK(k >= 1 && k <= count && k <= ((int64_t)1 << 24), "k %lld outside [1, min(count, 2^24)]",
           (long long)k);
  DN_CHECK(x && vals_out && idx_out, "NULL argument");
  if (n_rows == 0) return 0;
  hipStream_t st = stream();
  unsigned gx = (unsigned)ceil_div(count, 256 * 16);
  if (gx > 2048) gx = 2048;
  if (gx < 1) gx = 1;
  const dim3 grid(gx, (unsigned)n_rows), block(256);
  TopkState* state = nullptr;
  unsigned* hist = nullptr;
  uint64_t* cand = nullptr;
  int64_t* rank = nullptr;
  double* sq = nullptr;
  auto cleanup = [&]() {
    (void)hipStreamSynchronize(st);
    dfree(state); dfree(hist); dfree(cand); dfree(rank); dfree(sq);
  };
  int s = dmalloc(&state, n_rows) || dmalloc(&hist, n_rows * TOPK_BINS) || dmalloc(&sq, n_rows * gx);
  if (!s && hipMemsetAsync(hist, 0, sizeof(unsigned) * n_rows * TOPK_BINS, st) != hipSuccess) {
    set_error("top-k: clearing the histograms failed");
    s = 1;
  }
  if (s) { cleanup(); return s; }
  hipLaunchKernelGGL(k_topk_init, dim3((unsigned)n_rows), dim3(1), 0, st, state, k);
  const bool vec4 = count % 4 == 0 && ((uintptr_t)x % 16) == 0;
  auto launch_hist = [&](int shift, int nbits, double* sq_out) {
    if (vec4)
      hipLaunchKernelGGL(k_topk_hist<true>, grid, block, 0, st, x, count, shift, nbits, state, hist, sq_out);
    else
      hipLaunchKernelGGL(k_topk_hist<false>, grid, block, 0, st, x, count, shift, nbits, state, hist, sq_out);
  };
  launch_hist(21, 11, sq);
  hipLaunchKernelGGL(k_topk_pick, dim3((unsigned)n_rows), dim3(64), 0, st, hist, 21, 11, state);
  if (norms_out)
    hipLaunchKernelGGL(k_topk_norm, dim3((unsigned)n_rows), dim3(64), 0, st, sq, (int)gx, norms_out);
  std::vector<TopkState> host_state((size_t)n_rows);
  if (hipGetLastError() != hipSuccess || hipStreamSynchronize(st) != hipSuccess ||
      hipMemcpy(host_state.data(), state, sizeof(TopkState) * n_rows, hipMemcpyDeviceToHost) != hipSuccess) {
    set_error("top-k: the first pass failed");
    cleanup();
    return 1;
  }
  auto longest_list = [&]() {
    int64_t most = 0;
    for (const TopkState& h : host_state) {
      const int64_t n_cand = k - h.need + h.in_bin;
      if (n_cand > most) most = n_cand;
    }
    return most;
  };
  int64_t kp = 1, cap = TOPK_FAST_CAP;
  if (tuning().topk_fast_cap >= 0.0) cap = (int64_t)tuning().topk_fast_cap;  // tests: force the deeper paths
  // while the k-th entry's bin is crowded, decide the next bits of the key (one more read each)
  const int shifts[2] = {10, 0}, bits[2] = {11, 10};
  int64_t most = longest_list();
  for (int p = 0; p < 2 && most > cap; p++) {
    launch_hist(shifts[p], bits[p], nullptr);
    hipLaunchKernelGGL(k_topk_pick, dim3((unsigned)n_rows), dim3(64), 0, st, hist, shifts[p], bits[p], state);
    if (hipGetLastError() != hipSuccess || hipStreamSynchronize(st) != hipSuccess ||
        hipMemcpy(host_state.data(), state, sizeof(TopkState) * n_rows, hipMemcpyDeviceToHost) != hipSuccess) {
      set_error("top-k: a histogram pass failed");
      cleanup();
      return 1;
    }
    most = longest_list();
  }
  if (most <= cap) {
    while (kp < most) kp <<= 1;
    s = dmalloc(&cand, n_rows * kp);
    if (!s) {
      if (vec4)
        hipLaunchKernelGGL(k_topk_take_bins<true>, grid, block, 0, st, x, count, state, cand, kp, k);
      else
        hipLaunchKernelGGL(k_topk_take_bins<false>, grid, block, 0, st, x, count, state, cand, kp, k);
      s = bitonic_sort_rows(cand, kp, n_rows);
    }
  } else {
    // the whole key is decided and the entries equal to it alone are too many to sort: take
    // the first `need` of them in index order
    while (kp < k) kp <<= 1;
    s = dmalloc(&cand, n_rows * kp) || dmalloc(&rank, count + 1);
    if (!s) {
      hipLaunchKernelGGL(k_topk_take_above, grid, block, 0, st, x, count, state, cand, kp);
      if (hipGetLastError() != hipSuccess) { set_error("top-k: launch failed"); s = 1; }
    }
    for (int64_t row = 0; row < n_rows && !s; row++) {
      const float* xr = x + row * count;
      s = exclusive_scan(TieF{xr, state + row}, count, rank);
      if (!s)
        hipLaunchKernelGGL(k_topk_take_ties, dim3(gx), block, 0, st, xr, count, state + row, rank,
                           cand + row * kp, k, kp);
    }
    if (!s) s = bitonic_sort_rows(cand, kp, n_rows);
  }
  if (!s) {
    unsigned ge = (unsigned)ceil_div(k, 256);
    if (ge > 4096) ge = 4096;
    hipLaunchKernelGGL(k_topk_emit, dim3(ge, (unsigned)n_rows), block, 0, st, cand, k, kp, vals_out, idx_out);
    if (hipGetLastError() != hipSuccess) { set_error("top-k: launch failed"); s = 1; }
  }
  cleanup();
  return s;
}
