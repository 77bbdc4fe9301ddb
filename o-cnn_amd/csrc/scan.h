// Device-wide exclusive scan of a 0/1 predicate in three launches, built on
// 64-wide wavefront shuffles: tile counts -> scan of tile counts -> per-tile
// ranks.  Used for label generation and by the octree builder.
#pragma once

#include "ocnn_common.h"

namespace ocnn {

constexpr int kScanItems = 4;                       // consecutive elements per thread
constexpr int kScanTile = kBlock * kScanItems;      // elements per workgroup

inline int scan_tiles(int64_t n) { return (int)((n + kScanTile - 1) / kScanTile); }
// scratch: one int per tile (+1 spare)
inline size_t scan_scratch_bytes(int64_t n) { return sizeof(int) * (size_t)(scan_tiles(n) + 1); }

__device__ inline int wave_inclusive_scan(int v) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    int t = __shfl_up(v, d, 64);
    if (lane >= d) v += t;
  }
  return v;
}

// exclusive prefix of `v` over the 256-thread workgroup; *block_total gets the sum
__device__ inline int block_exclusive_scan(int v, int* block_total) {
  __shared__ int wave_sum[kBlock / 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int inc = wave_inclusive_scan(v);
  if (lane == 63) wave_sum[wave] = inc;
  __syncthreads();
  int base = 0, total = 0;
#pragma unroll
  for (int w = 0; w < kBlock / 64; ++w) {
    int s = wave_sum[w];
    if (w < wave) base += s;
    total += s;
  }
  __syncthreads();
  *block_total = total;
  return base + inc - v;
}

// Pred: __device__ bool operator()(int64_t i) const
template <typename Pred>
__global__ void scan_count_kernel(Pred pred, int64_t n, int* __restrict__ tile_count) {
  int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
  int c = 0;
#pragma unroll
  for (int j = 0; j < kScanItems; ++j)
    if (base + j < n && pred(base + j)) ++c;
  int total;
  block_exclusive_scan(c, &total);
  if (threadIdx.x == 0) tile_count[blockIdx.x] = total;
}

// single workgroup: tile_count[] -> exclusive offsets in place, grand total to *total_out
// (a template only so that every translation unit may hold its own copy)
template <int kUnused>
__global__ void scan_tiles_kernel(int* __restrict__ tile_count, int n_tiles, int* __restrict__ total_out) {
  __shared__ int carry;
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  for (int start = 0; start < n_tiles; start += kBlock) {
    int i = start + threadIdx.x;
    int v = i < n_tiles ? tile_count[i] : 0;
    int total;
    int ex = block_exclusive_scan(v, &total);
    int c = carry;
    if (i < n_tiles) tile_count[i] = c + ex;
    __syncthreads();
    if (threadIdx.x == 0) carry = c + total;
    __syncthreads();
  }
  if (threadIdx.x == 0 && total_out) *total_out = carry;
}

// Out: __device__ void operator()(int64_t i, bool flag, int rank) const
// rank = number of flagged elements before i
template <typename Pred, typename Out>
__global__ void scan_apply_kernel(Pred pred, Out out, int64_t n, const int* __restrict__ tile_offset) {
  int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
  bool f[kScanItems];
  int c = 0;
#pragma unroll
  for (int j = 0; j < kScanItems; ++j) {
    f[j] = base + j < n && pred(base + j);
    c += f[j] ? 1 : 0;
  }
  int total;
  int rank = tile_offset[blockIdx.x] + block_exclusive_scan(c, &total);
#pragma unroll
  for (int j = 0; j < kScanItems; ++j) {
    if (base + j < n) out(base + j, f[j], rank);
    rank += f[j] ? 1 : 0;
  }
}

// Enqueues the three launches.  scratch must hold scan_scratch_bytes(n).
template <typename Pred, typename Out>
inline hipError_t flag_scan(Pred pred, Out out, int64_t n, int* scratch, int* total_out, hipStream_t s) {
  int tiles = scan_tiles(n);
  if (tiles == 0) tiles = 1;
  scan_count_kernel<Pred><<<tiles, kBlock, 0, s>>>(pred, n, scratch);
  scan_tiles_kernel<0><<<1, kBlock, 0, s>>>(scratch, tiles, total_out);
  scan_apply_kernel<Pred, Out><<<tiles, kBlock, 0, s>>>(pred, out, n, scratch);
  return hipGetLastError();
}

}  // namespace ocnn
