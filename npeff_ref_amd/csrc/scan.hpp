// Device-wide exclusive scan of a functor over [0, n): tile sums -> scan of the tile sums ->
// per-tile scan.  Shared by the loader and the top-k sparsifier.
#pragma once

#include "dnpeff_internal.hpp"

namespace dn {

// ---------------------------------------------------------------------------
// Exclusive scan: tile sums -> scan of tile sums -> per-tile scan
// ---------------------------------------------------------------------------
constexpr int SCAN_BLOCK = 256;
constexpr int SCAN_ITEMS = 8;
constexpr int SCAN_TILE = SCAN_BLOCK * SCAN_ITEMS;

__device__ inline int64_t block_excl_scan(int64_t v, int64_t& total) {
  __shared__ int64_t sh[SCAN_BLOCK];
  const int t = threadIdx.x;
  sh[t] = v;
  __syncthreads();
  for (int off = 1; off < SCAN_BLOCK; off <<= 1) {
    int64_t add = (t >= off) ? sh[t - off] : 0;
    __syncthreads();
    sh[t] += add;
    __syncthreads();
  }
  int64_t incl = sh[t];
  total = sh[SCAN_BLOCK - 1];
  __syncthreads();
  return incl - v;
}

template <class F>
__global__ void __launch_bounds__(SCAN_BLOCK) k_scan_tile_sums(F f, int64_t n, int64_t* tile_sums) {
  int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * SCAN_ITEMS;
  int64_t s = 0;
  for (int i = 0; i < SCAN_ITEMS; i++) {
    int64_t idx = base + i;
    if (idx < n) s += f(idx);
  }
  int64_t total;
  block_excl_scan(s, total);
  if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
}

// In-place exclusive scan of tile_sums[0..n_tiles); tile_sums[n_tiles] = total.
static __global__ void __launch_bounds__(SCAN_BLOCK) k_scan_tiles(int64_t* tile_sums, int64_t n_tiles) {
  int64_t carry = 0;
  for (int64_t base = 0; base < n_tiles; base += SCAN_BLOCK) {
    int64_t idx = base + threadIdx.x;
    int64_t v = idx < n_tiles ? tile_sums[idx] : 0;
    int64_t total;
    int64_t ex = block_excl_scan(v, total);
    if (idx < n_tiles) tile_sums[idx] = carry + ex;
    carry += total;
  }
  if (threadIdx.x == 0) tile_sums[n_tiles] = carry;
}

template <class F, class OutT>
__global__ void __launch_bounds__(SCAN_BLOCK)
    k_scan_apply(F f, int64_t n, const int64_t* tile_offsets, int64_t n_tiles, OutT* out) {
  int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * SCAN_ITEMS;
  int64_t v[SCAN_ITEMS];
  int64_t s = 0;
  for (int i = 0; i < SCAN_ITEMS; i++) {
    int64_t idx = base + i;
    v[i] = idx < n ? (int64_t)f(idx) : 0;
    s += v[i];
  }
  int64_t total;
  int64_t run = block_excl_scan(s, total) + tile_offsets[blockIdx.x];
  for (int i = 0; i < SCAN_ITEMS; i++) {
    int64_t idx = base + i;
    if (idx < n) out[idx] = (OutT)run;
    run += v[i];
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) out[n] = (OutT)tile_offsets[n_tiles];
}

static __global__ void k_set_one_i64(int64_t* p, int64_t v) { *p = v; }

template <class F, class OutT>
static int exclusive_scan(F f, int64_t n, OutT* out) {
  hipStream_t st = stream();
  int64_t n_tiles = ceil_div(n, SCAN_TILE);
  if (n_tiles == 0) {
    DN_HIP(hipMemsetAsync(out, 0, sizeof(OutT), st));
    return 0;
  }
  int64_t* tiles = nullptr;
  DN_TRY(dmalloc(&tiles, n_tiles + 1));
  hipLaunchKernelGGL((k_scan_tile_sums<F>), dim3((unsigned)n_tiles), dim3(SCAN_BLOCK), 0, st, f, n,
                     tiles);
  hipLaunchKernelGGL(k_scan_tiles, dim3(1), dim3(SCAN_BLOCK), 0, st, tiles, n_tiles);
  hipLaunchKernelGGL((k_scan_apply<F, OutT>), dim3((unsigned)n_tiles), dim3(SCAN_BLOCK), 0, st, f,
                     n, tiles, n_tiles, out);
  DN_LAUNCH_CHECK();
  DN_HIP(hipStreamSynchronize(st));
  dfree(tiles);
  return 0;
}

}  // namespace dn
