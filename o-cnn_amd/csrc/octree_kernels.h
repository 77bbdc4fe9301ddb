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
// members (bit s = sibling s) whose 3x3x3 window of the group's 4x4x4 block contains this lane's slot
__device__ inline int neigh_wanted_by(int lane) {
  int wants = 0;
  const int x = lane >> 4, y = (lane >> 2) & 3, z = lane & 3;
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    const int dx = x - (s >> 2), dy = y - ((s >> 1) & 1), dz = z - (s & 1);
    if (dx >= 0 && dx <= 2 && dy >= 0 && dy <= 2 && dz >= 0 && dz <= 2) wants |= 1 << s;
  }
  return wants;
}

// the work of wavefront `wave` out of `stride` wavefronts
template <int GROUPS>
__device__ inline void neigh_sparse_wave(int* __restrict__ neigh_child, const int* __restrict__ neigh,
    const int* __restrict__ children, int node_num, int iters, int child_groups, int wave, int stride) {
  const int lane = threadIdx.x & 63;
  const int groups = (node_num + 7) >> 3;
  const int64_t slots = (int64_t)node_num * 8;
  const NeighLane nl(lane);
  const int wants = neigh_wanted_by(lane);
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
        const int rank = __builtin_amdgcn_readlane(rank8[u], s);   // a scalar: the row's address is base + lane
        const int v = __shfl(link[u], nl.parent_slot(s), 64);
        if (rank >= child_groups) continue;   // a link past the child level (malformed input): no row to write
        (neigh_child + ((int64_t)rank << 6))[lane] = v >= 0 ? (v << 3) + nl.octant : -1;
      }
    }
#pragma unroll
    for (int u = 0; u < GROUPS; ++u) { rank8[u] = next_rank8[u]; slot[u] = next_slot[u]; }
  }
}
template <int GROUPS>
__global__ __launch_bounds__(kBlock) void neigh_sparse_kernel(int* __restrict__ neigh_child,
    const int* __restrict__ neigh, const int* __restrict__ children, int node_num, int iters, int child_groups) {
  neigh_sparse_wave<GROUPS>(neigh_child, neigh, children, node_num, iters, child_groups,
      (int)((blockIdx.x * (unsigned)kBlock + threadIdx.x) >> 6), (int)(gridDim.x * (unsigned)(kBlock / 64)));
}

// Two levels from one sibling group whose 4x4x4 block is in registers (`slot`: this lane's entry,
// `rank8`: the child link of member `lane`, lanes 0 .. 7): the rows of the non-empty members'
// children (level + 1, as above) and, from those rows while they are still in registers, the rows
// of the grandchildren (level + 2): the larger level does not wait for a launch of the smaller
// one, and the smaller one's rows are not read back.  `children` / `children_c`: the child links
// of the level and of level + 1 (consistent: every link is a sibling group of the next level).
// The loads of the eight members are requested together (an empty member reads index 0), so this
// is three dependent trips to memory.
__device__ inline void neigh_sparse2_rows(int* __restrict__ neigh_c, int* __restrict__ neigh_cc, int slot, int rank8,
    const int* __restrict__ children, const int* __restrict__ children_c) {
  const int lane = threadIdx.x & 63;
  const NeighLane nl(lane);
  const int wants = neigh_wanted_by(lane);
  const int from0 = nl.parent_slot(0);   // parent_slot(s) = from0 + the offsets of s (no carries: hx + 1 <= 3)
  const int occ = (int)(__ballot(lane < 8 && rank8 >= 0) & 0xff);
  if (occ == 0) return;
  const int t = (wants & occ) ? slot : -1;
  const int link = t >= 0 ? children[t] : -1;
  // (ranks are the same for every lane: read through readlane they stay in scalar registers and
  // the row addresses are scalar base + lane)
  int row[8], rank8_c[8];
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    const bool live = (occ >> s) & 1;
    const int rank = live ? __builtin_amdgcn_readlane(rank8, s) : 0;
    const int v = __shfl(link, from0 + ((s >> 2) << 4) + (((s >> 1) & 1) << 2) + (s & 1), 64);
    row[s] = live && v >= 0 ? (v << 3) + nl.octant : -1;
    rank8_c[s] = (children_c + rank * 8)[lane & 7];   // (every lane: lanes 8 .. 63 read the same line)
  }
  int link_c[8], occ_c[8];
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    const bool live = (occ >> s) & 1;
    occ_c[s] = live ? (int)(__ballot(lane < 8 && rank8_c[s] >= 0) & 0xff) : 0;
    const int tc = (wants & occ_c[s]) ? row[s] : -1;
    link_c[s] = children_c[max(tc, 0)];
    if (tc < 0) link_c[s] = -1;
  }
#pragma unroll
  for (int s = 0; s < 8; ++s)
    if ((occ >> s) & 1) (neigh_c + ((int64_t)__builtin_amdgcn_readlane(rank8, s) << 6))[lane] = row[s];
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    for (int m = occ_c[s]; m != 0; m &= m - 1) {   // uniform over the wavefront
      const int u = __builtin_ctz(m);
      const int r = __builtin_amdgcn_readlane(rank8_c[s], u);
      const int v = __shfl(link_c[s], from0 + ((u >> 2) << 4) + (((u >> 1) & 1) << 2) + (u & 1), 64);
      (neigh_cc + ((int64_t)r << 6))[lane] = v >= 0 ? (v << 3) + nl.octant : -1;
    }
  }
}
// levels + 1 and + 2 from sibling group `g` of a level whose table `neigh` exists
__device__ inline void neigh_sparse2_wave(int* __restrict__ neigh_c, int* __restrict__ neigh_cc,
    const int* __restrict__ neigh, const int* __restrict__ children, const int* __restrict__ children_c,
    int node_num, int g) {
  const int lane = threadIdx.x & 63;
  if (g * 8 >= node_num) return;
  const int node = g * 8 + lane;
  const int rank8 = (lane < 8 && node < node_num) ? children[node] : -1;
  const int slot = ((int64_t)g << 6) + lane < (int64_t)node_num * 8 ? neigh[((int64_t)g << 6) + lane] : -1;
  neigh_sparse2_rows(neigh_c, neigh_cc, slot, rank8, children, children_c);
}
// levels + 1, + 2 and + 3 from node `node` of a level whose table `neigh` exists: the node's own
// row of level + 1 (every member of a group reads the group's block again), then the two levels
// below from that row
__device__ inline void neigh_sparse3_wave(int* __restrict__ neigh_c, int* __restrict__ neigh_cc,
    int* __restrict__ neigh_ccc, const int* __restrict__ neigh, const int* __restrict__ children,
    const int* __restrict__ children_c, const int* __restrict__ children_cc, int node_num, int node) {
  const int lane = threadIdx.x & 63;
  if (node >= node_num) return;
  const int rank = children[node];
  if (rank < 0) return;   // uniform over the wavefront
  const NeighLane nl(lane);
  const int s = node & 7;
  const int slot = neigh[((int64_t)(node >> 3) << 6) + nl.parent_slot(s)];   // the entry this lane's value comes from
  const int v = slot >= 0 ? children[slot] : -1;
  const int row = v >= 0 ? (v << 3) + nl.octant : -1;
  neigh_c[((int64_t)rank << 6) + lane] = row;
  neigh_sparse2_rows(neigh_cc, neigh_ccc, row, children_c[rank * 8 + (lane & 7)], children_c, children_cc);
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

// The tables of `count` (1 .. kNeighLevels) consecutive sparse levels in one launch, from the level
// above the first: out[i] is the table of the i-th level written, children[i] the child links of
// the level above it (consistent links: a fresh octree's own), `neigh` / `node_num` the table and
// node count of the level above the first.  The same rows as one launch_neigh_sparse per level.
constexpr int kNeighLevels = 3;
struct NeighLevels {
  int* out[kNeighLevels];
  const int* children[kNeighLevels];
};
template <int COUNT>
__global__ __launch_bounds__(kBlock) void neigh_sparse_levels_kernel(NeighLevels a, const int* __restrict__ neigh, int node_num) {
  const int wave = (int)((blockIdx.x * (unsigned)kBlock + threadIdx.x) >> 6);
  if (COUNT == 2) neigh_sparse2_wave(a.out[0], a.out[1], neigh, a.children[0], a.children[1], node_num, wave);
  else neigh_sparse3_wave(a.out[0], a.out[1], a.out[2], neigh, a.children[0], a.children[1], a.children[2], node_num, wave);
}
inline void launch_neigh_sparse_levels(int count, int* const* out, const int* neigh, const int* const* children,
    int node_num, hipStream_t s) {
  if (count <= 1) {
    launch_neigh_sparse(out[0], neigh, children[0], node_num, s);
    return;
  }
  NeighLevels a;
  for (int i = 0; i < kNeighLevels; ++i) { a.out[i] = i < count ? out[i] : nullptr; a.children[i] = i < count ? children[i] : nullptr; }
  if (count == 2)
    neigh_sparse_levels_kernel<2><<<blocks_for(((int64_t)node_num + 7) / 8, kBlock / 64), kBlock, 0, s>>>(a, neigh, node_num);
  else
    neigh_sparse_levels_kernel<3><<<blocks_for(node_num, kBlock / 64), kBlock, 0, s>>>(a, neigh, node_num);
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
