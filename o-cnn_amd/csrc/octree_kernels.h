// Device code shared by the translation units that touch the octree structure:
// Morton bit interleaving and the neighbour-table kernels (the builder fills the
// tables of a fresh octree with the same kernels that the calc_neigh entry points
// launch).
#pragma once

#include "ocnn_common.h"
#include "scan.h"

namespace ocnn {

// Morton helpers: bit i of axis j lands at bit 3*i + 2 - j (x highest), the
// convention of compute_key / compute_pt (octree/octree/octree_nn.cpp:551-575).
__host__ __device__ inline uint64_t spread3(uint64_t v) {  // 16 bits -> every third bit
  v &= 0xffffull;
  v = (v | (v << 32)) & 0x00ff00000000ffffull;
  v = (v | (v << 16)) & 0x00ff0000ff0000ffull;
  v = (v | (v << 8)) & 0xf00f00f00f00f00full;
  v = (v | (v << 4)) & 0x30c30c30c30c30c3ull;
  v = (v | (v << 2)) & 0x9249249249249249ull;
  return v;
}
__host__ __device__ inline uint64_t compact3(uint64_t v) {  // inverse of spread3
  v &= 0x9249249249249249ull;
  v = (v | (v >> 2)) & 0x30c30c30c30c30c3ull;
  v = (v | (v >> 4)) & 0xf00f00f00f00f00full;
  v = (v | (v >> 8)) & 0x00ff0000ff0000ffull;
  v = (v | (v >> 16)) & 0x00ff00000000ffffull;
  v = (v | (v >> 32)) & 0xffffull;
  return v;
}
__host__ __device__ inline uint64_t morton_encode(uint32_t x, uint32_t y, uint32_t z, int depth) {
  uint64_t m = depth >= 16 ? 0xffffull : ((1ull << depth) - 1);
  return (spread3(x & m) << 2) | (spread3(y & m) << 1) | spread3(z & m);
}
__host__ __device__ inline void morton_decode(uint64_t key, int depth, uint32_t* x, uint32_t* y, uint32_t* z) {
  uint64_t m = depth >= 16 ? 0xffffull : ((1ull << depth) - 1);
  *x = (uint32_t)(compact3(key >> 2) & m);
  *y = (uint32_t)(compact3(key >> 1) & m);
  *z = (uint32_t)(compact3(key) & m);
}

// ---- neighbour tables (calc_neigh_cpu / calc_neigh_gpu, octree/octree/octree_nn.cpp:357-424,
// octree/octree/octree_nn.cu:331-413) ------------------------------------------------------
// Slot `lane` (x<<4 | y<<2 | z) of the 4x4x4 block of a non-empty parent-level node: the
// child at octant `oct` of the parent-level neighbour at offset ((x+1)>>1, ...) - 1.
// One such slot of the parent's own sibling-group block gives that neighbour.
struct NeighLane {
  int hx, hy, hz, octant;
  __device__ explicit NeighLane(int lane) {
    const int x = lane >> 4, y = (lane >> 2) & 3, z = lane & 3;
    hx = (x + 1) >> 1; hy = (y + 1) >> 1; hz = (z + 1) >> 1;
    octant = (((x + 1) & 1) << 2) | (((y + 1) & 1) << 1) | ((z + 1) & 1);
  }
  __device__ int parent_slot(int sib) const {
    return ((hx + (sib >> 2)) << 4) | ((hy + ((sib >> 1) & 1)) << 2) | (hz + (sib & 1));
  }
};

// Sparse-layer neighbour table.  The work unit is a sibling group of the parent level (8
// consecutive nodes): the 27-neighbourhoods of its non-empty members all lie in the group's
// own 4x4x4 block, so a wavefront loads that block once (one coalesced 256-byte read),
// looks up the children link of every slot some non-empty member needs (the one divergent
// gather, per group instead of per node), and every non-empty member then takes its 64
// values from the lanes of the wavefront and writes one coalesced 256-byte row.  No
// compaction pass and two dependent memory round trips, whatever the size of the level.
// A wavefront walks `iters` batches of GROUPS groups and requests the next batch's block and
// links while the current batch is gathered and written.  GROUPS = 8 keeps enough bytes in
// flight per wavefront for a large level (the kernel is bound by that, not by bandwidth);
// GROUPS = 2 gives a small level more wavefronts and each a shorter chain.
template <int GROUPS>
__global__ __launch_bounds__(kBlock) void neigh_sparse_kernel(int* __restrict__ neigh_child,
    const int* __restrict__ neigh, const int* __restrict__ children, int node_num, int iters, int child_groups) {
  const int lane = threadIdx.x & 63;
  const int wave = (int)((blockIdx.x * (unsigned)kBlock + threadIdx.x) >> 6);
  const int groups = (node_num + 7) >> 3;
  const int64_t slots = (int64_t)node_num * 8;
  const NeighLane nl(lane);
  // members (bit s = sibling s) whose 3x3x3 window of the block contains this lane's slot
  int wants = 0;
  {
    const int x = lane >> 4, y = (lane >> 2) & 3, z = lane & 3;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int dx = x - (s >> 2), dy = y - ((s >> 1) & 1), dz = z - (s & 1);
      if (dx >= 0 && dx <= 2 && dy >= 0 && dy <= 2 && dz >= 0 && dz <= 2) wants |= 1 << s;
    }
  }
  int rank8[GROUPS], slot[GROUPS];
  auto request = [&](int batch, int* r8, int* sl) {
#pragma unroll
    for (int u = 0; u < GROUPS; ++u) {
      const int g = batch * GROUPS + u;
      const int node = g * 8 + lane;
      r8[u] = (g < groups && lane < 8 && node < node_num) ? children[node] : -1;
      sl[u] = (g < groups && ((int64_t)g << 6) + lane < slots) ? neigh[((int64_t)g << 6) + lane] : -1;
    }
  };
  // batch it of wavefront w is w + it * (number of wavefronts): at any moment the wavefronts of
  // the device work on one contiguous window of the level
  const int stride = (int)(gridDim.x * (unsigned)(kBlock / 64));
  request(wave, rank8, slot);
  for (int it = 0; it < iters; ++it) {
    if ((int64_t)(wave + (int64_t)it * stride) * GROUPS >= groups) break;
    int next_rank8[GROUPS] = {}, next_slot[GROUPS] = {};
    if (it + 1 < iters) request(wave + (it + 1) * stride, next_rank8, next_slot);
    int occ[GROUPS], link[GROUPS];
#pragma unroll
    for (int u = 0; u < GROUPS; ++u) {
      occ[u] = (int)(__ballot(rank8[u] >= 0) & 0xff);
      const int t = (wants & occ[u]) ? slot[u] : -1;
      link[u] = t >= 0 ? children[t] : -1;
    }
#pragma unroll
    for (int u = 0; u < GROUPS; ++u) {
      for (int s = 0; s < 8; ++s) {
        if (!((occ[u] >> s) & 1)) continue;   // uniform over the wavefront
        const int rank = __shfl(rank8[u], s, 64);
        const int v = __shfl(link[u], nl.parent_slot(s), 64);
        if (rank >= child_groups) continue;   // a link past the child level (malformed input): no row to write
        neigh_child[((int64_t)rank << 6) + lane] = v >= 0 ? (v << 3) + nl.octant : -1;
      }
    }
#pragma unroll
    for (int u = 0; u < GROUPS; ++u) { rank8[u] = next_rank8[u]; slot[u] = next_slot[u]; }
  }
}
// `child_groups`: sibling groups of the level written, where the caller knows it (a header);
// links at or past it are skipped instead of followed.
inline void launch_neigh_sparse(int* neigh_child, const int* neigh, const int* children, int node_num,
    hipStream_t s, int child_groups = 0x7fffffff) {
  const int64_t groups = ((int64_t)node_num + 7) / 8;
  if (groups >= (1 << 16)) {
    // batches per wavefront: more than one once the wavefronts fill the device several times over
    const int64_t batches = (groups + 7) / 8;
    int64_t iters = batches / 32768;
    iters = iters < 1 ? 1 : (iters > 8 ? 8 : iters);
    neigh_sparse_kernel<8><<<blocks_for(batches, (kBlock / 64) * iters), kBlock, 0, s>>>(neigh_child, neigh, children,
        node_num, (int)iters, child_groups);
  } else {
    neigh_sparse_kernel<2><<<blocks_for((groups + 1) / 2, kBlock / 64), kBlock, 0, s>>>(neigh_child, neigh, children,
        node_num, 1, child_groups);
  }
}

// Full layer: closed form through Morton decode / encode (octree_nn.cpp:382-424).
static __global__ void neigh_full_kernel(int* __restrict__ neigh, int depth, int64_t total) {
  int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= total) return;
  const int64_t node_num = (int64_t)1 << (3 * depth);
  const int64_t groups = node_num >> 3;
  int slot = (int)(id & 63);
  int64_t g = id >> 6;
  int64_t n = g / groups;
  uint64_t i = (uint64_t)(g % groups) << 3;
  uint32_t x0, y0, z0;
  morton_decode(i, depth, &x0, &y0, &z0);
  uint32_t x1 = x0 + (slot >> 4) - 1, y1 = y0 + ((slot >> 2) & 3) - 1, z1 = z0 + (slot & 3) - 1;
  const uint32_t bound = 1u << depth;
  int v = -1;
  if (((x1 | y1 | z1) & bound) == 0) v = (int)(morton_encode(x1, y1, z1, depth) + (uint64_t)n * node_num);
  neigh[id] = v;
}

}  // namespace ocnn
