// Integer kernels on the octree structure: neighbour tables, key generation,
// Morton <-> packed-xyz conversion, sorted-key search, label compaction.
// Everything here is bit-exact integer work bound by HBM bandwidth.
#include "octree_kernels.h"

#include <atomic>

namespace ocnn {
namespace {

// ---- keys -----------------------------------------------------------------------
__global__ void gen_key_child_kernel(uint64_t* __restrict__ key_child, const uint64_t* __restrict__ key,
    const int* __restrict__ child, int64_t total) {
  int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= total) return;
  int i = (int)(id >> 3), j = (int)(id & 7);
  int label = child[i];
  if (label < 0) return;
  uint64_t k0 = key[i];
  uint64_t x = (((k0 & 0xffffu) << 1) | ((j >> 2) & 1)) & 0xffffu;
  uint64_t y = ((((k0 >> 16) & 0xffffu) << 1) | ((j >> 1) & 1)) & 0xffffu;
  uint64_t z = ((((k0 >> 32) & 0xffffu) << 1) | (j & 1)) & 0xffffu;
  key_child[8 * (int64_t)label + j] = x | (y << 16) | (z << 32) | (k0 & 0xffff000000000000ull);
}

__global__ void gen_key_full_kernel(uint64_t* __restrict__ key, int depth, int64_t total) {
  int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= total) return;
  const int64_t node_num = (int64_t)1 << (3 * depth);
  uint32_t x, y, z;
  morton_decode((uint64_t)(id % node_num), depth, &x, &y, &z);
  key[id] = (uint64_t)x | ((uint64_t)y << 16) | ((uint64_t)z << 32) | ((uint64_t)((id / node_num) & 0xffff) << 48);
}

__global__ void xyz2key_kernel(uint64_t* __restrict__ key, const uint64_t* __restrict__ xyz, int num, int depth) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= num) return;
  uint64_t v = xyz[i];
  uint64_t k = morton_encode((uint32_t)(v & 0xffff), (uint32_t)((v >> 16) & 0xffff),
      (uint32_t)((v >> 32) & 0xffff), depth);
  key[i] = (k & 0x0000ffffffffffffull) | (v & 0xffff000000000000ull);
}

__global__ void key2xyz_kernel(uint64_t* __restrict__ xyz, const uint64_t* __restrict__ key, int num, int depth) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= num) return;
  uint64_t k = key[i];
  uint32_t x, y, z;
  morton_decode(k, depth, &x, &y, &z);
  xyz[i] = (uint64_t)x | ((uint64_t)y << 16) | ((uint64_t)z << 32) | (k & 0xffff000000000000ull);
}

__global__ void key2idx_kernel(int* __restrict__ idx, const uint64_t* __restrict__ key, int num) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < num) idx[i] = (int)(key[i] >> 48);
}

// ---- trilinear stencils between two levels (bilinear_neigh / bilinear_xyz) --------------------
// The stencil of a child: the node of the parent level in each of the 8 cells around the
// child's centre, nearest first (corner order 000, 001, 010, 100, 011, 101, 110, 111 of
// (x, y, z): weights 27, 9, 9, 9, 3, 3, 3, 1).  Seen from the 4x4x4 neighbour block of the
// parent's sibling group, child j of sibling i reads, per axis, slot (i + 1) and the slot one
// step towards the child's side; the reference tabulates that in 512 entries
// (NeighHelper, octree/octree/octree_nn.cpp:83-108), here it is computed.
__device__ inline int stencil_slot(int sib, int child, int corner) {
  // corner bits per axis in the order above: x = {0,0,0,1,0,1,1,1}, y = {0,0,1,0,1,0,1,1}, z = {0,1,0,0,1,1,0,1}
  const int cx = (0xE8 >> corner) & 1, cy = (0xD4 >> corner) & 1, cz = (0xB2 >> corner) & 1;
  const int x = ((sib >> 2) & 1) + 1 + cx * (2 * ((child >> 2) & 1) - 1);
  const int y = ((sib >> 1) & 1) + 1 + cy * (2 * ((child >> 1) & 1) - 1);
  const int z = (sib & 1) + 1 + cz * (2 * (child & 1) - 1);
  return (x << 4) | (y << 2) | z;
}

// One wavefront lane per (child, corner) of a non-empty parent: 64 table reads inside the
// parent group's 256-byte block, one 256-byte row of output per parent
// (bilinear_neigh_cpu, octree_nn.cpp:476-492).
__global__ void bilinear_neigh_kernel(int* __restrict__ bidx, const int* __restrict__ neigh,
    const int* __restrict__ child, int node_num) {
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int i = (int)(id >> 6), lane = (int)(id & 63);
  if (i >= node_num) return;
  const int cld = child[i];
  if (cld < 0) return;
  bidx[((int64_t)cld << 6) + lane] = neigh[((int64_t)(i >> 3) << 6) + stencil_slot(i & 7, lane >> 3, lane & 7)];
}

// bilinear_xyz_cpu, octree_nn.cpp:494-530: cells of level d0 around the centre of a cell of
// level d1 (packed 16-bit coordinates), and per axis the weight of the nearer cell.  Float
// steps as in the reference (the scale is a power of two: the quotient is exact).
__global__ void bilinear_xyz_kernel(uint64_t* __restrict__ xyz0, float* __restrict__ fracs,
    const uint64_t* __restrict__ xyz1, float scale, int num) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= num) return;
  const uint64_t v = xyz1[i];
  int bnd[2][3];
#pragma unroll
  for (int c = 0; c < 3; ++c) {
    const float pt = ((float)(uint32_t)((v >> (16 * c)) & 0xffff) + 0.5f) / scale - 0.5f;
    const int b = (int)pt;
    float frac = pt - (float)b;
    if (frac > 0.5f) { bnd[0][c] = b + 1; bnd[1][c] = b; }
    else { frac = 1 - frac; bnd[0][c] = b; bnd[1][c] = b + 1; }
    fracs[3 * (int64_t)i + c] = frac;
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int cx = (0xE8 >> j) & 1, cy = (0xD4 >> j) & 1, cz = (0xB2 >> j) & 1;
    xyz0[(int64_t)i * 8 + j] = (uint64_t)(uint16_t)bnd[cx][0] | ((uint64_t)(uint16_t)bnd[cy][1] << 16) |
        ((uint64_t)(uint16_t)bnd[cz][2] << 32) | (v & 0xffff000000000000ull);
  }
}

__global__ void sequence_kernel(int* __restrict__ p, int num) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < num) p[i] = i;
}

// lower_bound over the sorted key array, -1 on a miss (octree_nn.cpp:541-548)
__global__ void search_key_kernel(int* __restrict__ idx, const uint64_t* __restrict__ key, int n_key,
    const uint64_t* __restrict__ query, int n_query) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_query) return;
  uint64_t q = query[i];
  int lo = 0, hi = n_key;
  while (lo < hi) {
    int mid = lo + ((hi - lo) >> 1);
    if (key[mid] < q) lo = mid + 1; else hi = mid;
  }
  idx[i] = (lo < n_key && key[lo] == q) ? lo : -1;
}

// The same search for many queries in a large array, through two tables of samples made for the
// call: every 256th key (at most 96 KiB, held in LDS by every workgroup) and every 16th key (stays
// in the L2 cache).  A plain binary search of random queries misses the caches on its last six or
// seven probes, four or five lines a query; here a query reads one line of the second table and
// one line of keys, each line once (16 lanes read a window together).  A window starts at the
// last sample BELOW the query, so the first of several equal keys is found as lower_bound does.
constexpr int kSearchFine = 16, kSearchCoarse = 256, kSearchLdsMax = 96 * 1024;
// `shift` = elements between the 128-byte line that holds key[0] and key[0]: the windows of 16
// keys are cut at line boundaries of the array as it lies in memory, sample e is the first key of
// window e (the first window is short), so that a window is one line whatever the array's address.
__global__ void search_tables_kernel(uint64_t* __restrict__ t1, int n1, uint64_t* __restrict__ t2, int n2,
    const uint64_t* __restrict__ key, int shift) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n2) t2[i] = key[max(i * kSearchFine - shift, 0)];
  if (i < n1) t1[i] = key[max(i * kSearchCoarse - shift, 0)];
}
// number of elements below q in a[lo, hi)
__device__ inline int count_below(const uint64_t* a, int lo, int hi, uint64_t q) {
  while (lo < hi) {
    const int mid = lo + ((hi - lo) >> 1);
    if (a[mid] < q) lo = mid + 1; else hi = mid;
  }
  return lo;
}
// For every lane of the wavefront: the number of elements below the lane's q among the 16 elements
// a[base .. base + 15] (one 128-byte line; places in front of the array count as below, elements
// from n on as not below).  A wavefront's loads cost by the lines they touch, and a lane that walks its own window
// touches a line per probe; here 16 lanes read one window together, four windows a round, and the
// 16 rounds of a wavefront are independent of one another.  Every lane must call.
constexpr int kSearchBlock = 1024;
__device__ inline int window_count(const uint64_t* __restrict__ a, int base, int n, uint64_t q) {
  const int lane = threadIdx.x & 63, sub = lane & 15, grp = lane >> 4;
  const uint32_t q_lo = (uint32_t)q, q_hi = (uint32_t)(q >> 32);
  int mine = 0;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int owner = 4 * r + grp;
    const int b = __shfl(base, owner, 64);
    const uint64_t qq = ((uint64_t)(uint32_t)__shfl((int)q_hi, owner, 64) << 32) | (uint32_t)__shfl((int)q_lo, owner, 64);
    const int at = b + sub;
    const uint64_t v = a[min(max(at, 0), n - 1)];
    const unsigned long long below = __ballot(at < 0 || (at < n && v < qq));   // (places in front of the array: below)
    if ((lane >> 2) == r) mine = __popcll((below >> (16 * (lane & 3))) & 0xffffull);
  }
  return mine;
}
__global__ __launch_bounds__(kSearchBlock) void search_key_indexed_kernel(int* __restrict__ idx,
    const uint64_t* __restrict__ key, int n_key, const uint64_t* __restrict__ t1, int n1, const uint64_t* __restrict__ t2,
    int n2, const uint64_t* __restrict__ query, int n_query, int per_block, int shift) {
  extern __shared__ __attribute__((aligned(16))) uint64_t s_t1[];
  {   // the coarse table, 16 bytes a lane (its row is padded to whole units)
    const ulonglong2* src = reinterpret_cast<const ulonglong2*>(t1);
    ulonglong2* dst = reinterpret_cast<ulonglong2*>(s_t1);
    const int units = (n1 + 1) >> 1;
#pragma unroll 4
    for (int i = threadIdx.x; i < units; i += kSearchBlock) dst[i] = src[i];
  }
  __syncthreads();
  const int first = blockIdx.x * per_block, end = min(n_query, first + per_block);
  // whole wavefronts walk the block's queries (a lane past the end searches for 0 and writes nothing)
  for (int i0 = first; i0 < end; i0 += kSearchBlock) {
    const int i = i0 + threadIdx.x;
    const uint64_t q = i < end ? query[i] : 0;
    // the sample below q bounds the window from the left, the next sample (not below q) from the right
    const int e0 = max(count_below(s_t1, 0, n1, q) - 1, 0) * (kSearchCoarse / kSearchFine);
    const int e2 = max(e0 + window_count(t2, e0, n2, q) - 1, e0);
    const int k0 = e2 * kSearchFine - shift;
    const int lo = k0 + window_count(key, k0, n_key, q);
    if (i < end) idx[i] = (lo < n_key && key[lo] == q) ? lo : -1;
  }
}

struct LabelPred {
  const int* btm;
  int mask;
  __device__ bool operator()(int64_t i) const { return btm[i] == mask; }
};
struct LabelOut {
  int* label;
  __device__ void operator()(int64_t i, bool f, int rank) const { label[i] = f ? rank : -1; }
};

}  // namespace
}  // namespace ocnn

using namespace ocnn;

extern "C" {

int ocnn_calc_neigh_sparse(int* neigh_child, const int* neigh, const int* children, int node_num,
    ocnn_stream_t stream) {
  OCNN_REQUIRE(neigh_child && neigh && children, OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(node_num >= 0, OCNN_E_BADARG, "node_num %d", node_num);
  if (node_num == 0) return OCNN_OK;
  launch_neigh_sparse(neigh_child, neigh, children, node_num, as_stream(stream));
  OCNN_LAUNCH_OK("calc_neigh_sparse");
  return OCNN_OK;
}

int ocnn_calc_neigh_full(int* neigh, int depth, int batch_size, ocnn_stream_t stream) {
  OCNN_REQUIRE(neigh, OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(depth >= 1 && depth <= 9 && batch_size >= 1, OCNN_E_BADARG,
      "depth %d batch %d (a full layer deeper than 9 does not fit int32 indices)", depth, batch_size);
  int64_t total = (int64_t)batch_size << (3 * depth + 3);
  OCNN_REQUIRE(total < (1ll << 34), OCNN_E_BADARG, "full layer too large");
  neigh_full_kernel<<<blocks_for(total), kBlock, 0, as_stream(stream)>>>(neigh, depth, total);
  OCNN_LAUNCH_OK("calc_neigh_full");
  return OCNN_OK;
}

int ocnn_generate_key_child(uint64_t* key_child, const uint64_t* key, const int* child, int node_num,
    ocnn_stream_t stream) {
  OCNN_REQUIRE(key_child && key && child && node_num >= 0, OCNN_E_BADARG, "bad argument");
  if (node_num == 0) return OCNN_OK;
  int64_t total = (int64_t)node_num << 3;
  gen_key_child_kernel<<<blocks_for(total), kBlock, 0, as_stream(stream)>>>(key_child, key, child, total);
  OCNN_LAUNCH_OK("generate_key_child");
  return OCNN_OK;
}

int ocnn_generate_key_full(uint64_t* key, int depth, int batch_size, ocnn_stream_t stream) {
  OCNN_REQUIRE(key && depth >= 0 && depth <= 10 && batch_size >= 1, OCNN_E_BADARG, "bad argument");
  int64_t total = (int64_t)batch_size << (3 * depth);
  gen_key_full_kernel<<<blocks_for(total), kBlock, 0, as_stream(stream)>>>(key, depth, total);
  OCNN_LAUNCH_OK("generate_key_full");
  return OCNN_OK;
}

size_t ocnn_generate_label_scratch_bytes(int btm_h) { return scan_scratch_bytes(btm_h < 0 ? 0 : btm_h); }

int ocnn_generate_label(int* label, int* count_dev, const int* btm, int btm_h, int mask,
    void* scratch_dev, size_t scratch_bytes, ocnn_stream_t stream) {
  OCNN_REQUIRE(label && count_dev && btm && btm_h >= 0, OCNN_E_BADARG, "bad argument");
  OCNN_REQUIRE(scratch_dev && scratch_bytes >= scan_scratch_bytes(btm_h), OCNN_E_WORKSPACE,
      "scratch %zu < %zu bytes", scratch_bytes, scan_scratch_bytes(btm_h));
  LabelPred pred{btm, mask};
  LabelOut out{label};
  hipError_t e = flag_scan(pred, out, (int64_t)btm_h, (int*)scratch_dev, count_dev, as_stream(stream));
  OCNN_REQUIRE(e == hipSuccess, OCNN_E_HIP, "generate_label: %s", hipGetErrorString(e));
  return OCNN_OK;
}

int ocnn_bilinear_neigh(int* bidx, const int* neigh, const int* child, int node_num, ocnn_stream_t stream) {
  OCNN_REQUIRE(bidx && neigh && child && node_num >= 0, OCNN_E_BADARG, "bad argument");
  if (node_num > 0)
    bilinear_neigh_kernel<<<blocks_for((int64_t)node_num * 64), kBlock, 0, as_stream(stream)>>>(bidx, neigh, child, node_num);
  OCNN_LAUNCH_OK("bilinear_neigh");
  return OCNN_OK;
}

int ocnn_bilinear_xyz(uint64_t* xyz0, float* fracs, int d0, const uint64_t* xyz1, int d1, int num,
    ocnn_stream_t stream) {
  OCNN_REQUIRE(xyz0 && fracs && xyz1 && num >= 0, OCNN_E_BADARG, "bad argument");
  OCNN_REQUIRE(d0 >= 0 && d1 >= d0 && d1 - d0 < 31, OCNN_E_BADARG, "levels %d -> %d", d1, d0);
  if (num > 0)
    bilinear_xyz_kernel<<<blocks_for(num), kBlock, 0, as_stream(stream)>>>(xyz0, fracs, xyz1, (float)(1 << (d1 - d0)), num);
  OCNN_LAUNCH_OK("bilinear_xyz");
  return OCNN_OK;
}

int ocnn_sequence(int* ptr, int num, ocnn_stream_t stream) {
  OCNN_REQUIRE(ptr && num >= 0, OCNN_E_BADARG, "bad argument");
  if (num == 0) return OCNN_OK;
  sequence_kernel<<<blocks_for(num), kBlock, 0, as_stream(stream)>>>(ptr, num);
  OCNN_LAUNCH_OK("sequence");
  return OCNN_OK;
}

int ocnn_search_key(int* idx, const uint64_t* key, int n_key, const uint64_t* query, int n_query,
    ocnn_stream_t stream) {
  OCNN_REQUIRE(idx && query && (key || n_key == 0) && n_key >= 0 && n_query >= 0, OCNN_E_BADARG, "bad argument");
  if (n_query == 0) return OCNN_OK;
  search_key_kernel<<<blocks_for(n_query), kBlock, 0, as_stream(stream)>>>(idx, key, n_key, query, n_query);
  OCNN_LAUNCH_OK("search_key");
  return OCNN_OK;
}

size_t ocnn_search_key_workspace_bytes(int n_key) {
  if (n_key < 0) return 0;
  const size_t n1 = ((size_t)n_key + 15 + kSearchCoarse - 1) / kSearchCoarse, n2 = ((size_t)n_key + 15 + kSearchFine - 1) / kSearchFine;
  return (n1 + n2) * sizeof(uint64_t) + 512;
}

int ocnn_search_key_indexed(int* idx, const uint64_t* key, int n_key, const uint64_t* query, int n_query,
    void* workspace_dev, size_t workspace_bytes, ocnn_stream_t stream) {
  OCNN_REQUIRE(idx && query && (key || n_key == 0) && n_key >= 0 && n_query >= 0, OCNN_E_BADARG, "bad argument");
  if (n_query == 0) return OCNN_OK;
  const int shift = (int)((reinterpret_cast<uintptr_t>(key) & 127) / sizeof(uint64_t));
  const int n1 = (n_key + shift + kSearchCoarse - 1) / kSearchCoarse, n2 = (n_key + shift + kSearchFine - 1) / kSearchFine;
  const size_t lds = (size_t)n1 * sizeof(uint64_t);
  // few queries, few keys, or more coarse samples than a workgroup can hold: the plain search
  if (n_query < 16384 || n_key < 16384 || lds > (size_t)kSearchLdsMax)
    return ocnn_search_key(idx, key, n_key, query, n_query, stream);
  OCNN_REQUIRE(workspace_dev && workspace_bytes >= ocnn_search_key_workspace_bytes(n_key), OCNN_E_WORKSPACE,
      "workspace %zu < %zu bytes", workspace_bytes, ocnn_search_key_workspace_bytes(n_key));
  OCNN_REQUIRE((reinterpret_cast<uintptr_t>(workspace_dev) & 127) == 0, OCNN_E_WORKSPACE, "workspace not 128-byte aligned");
  hipStream_t s = as_stream(stream);
  uint64_t* t1 = static_cast<uint64_t*>(workspace_dev);
  uint64_t* t2 = t1 + ((n1 + 31) & ~31);    // on a line boundary as well
  search_tables_kernel<<<blocks_for(n2), kBlock, 0, s>>>(t1, n1, t2, n2, key, shift);
  OCNN_LAUNCH_OK("search_tables");
  static std::atomic<size_t> allowed{0};
  if (lds > 64 * 1024 && allowed.load() < lds) {
    OCNN_HIP_OK(hipFuncSetAttribute(reinterpret_cast<const void*>(&search_key_indexed_kernel),
        hipFuncAttributeMaxDynamicSharedMemorySize, kSearchLdsMax));
    allowed.store(kSearchLdsMax);
  }
  // every workgroup loads the coarse table once: enough queries each to make that cheap, enough
  // workgroups to fill the device
  int per_block = 16 * kSearchBlock;
  while (per_block > kSearchBlock && (n_query + per_block - 1) / per_block < 512) per_block >>= 1;
  const int blocks = (n_query + per_block - 1) / per_block;
  search_key_indexed_kernel<<<blocks, kSearchBlock, (lds + 15) & ~(size_t)15, s>>>(idx, key, n_key, t1, n1, t2, n2, query,
      n_query, per_block, shift);
  OCNN_LAUNCH_OK("search_key_indexed");
  return OCNN_OK;
}

int ocnn_xyz2key(uint64_t* key, const uint64_t* xyz, int num, int depth, ocnn_stream_t stream) {
  OCNN_REQUIRE(key && xyz && num >= 0 && depth >= 0 && depth <= 16, OCNN_E_BADARG, "bad argument");
  if (num == 0) return OCNN_OK;
  xyz2key_kernel<<<blocks_for(num), kBlock, 0, as_stream(stream)>>>(key, xyz, num, depth);
  OCNN_LAUNCH_OK("xyz2key");
  return OCNN_OK;
}

int ocnn_key2xyz(uint64_t* xyz, const uint64_t* key, int num, int depth, ocnn_stream_t stream) {
  OCNN_REQUIRE(key && xyz && num >= 0 && depth >= 0 && depth <= 16, OCNN_E_BADARG, "bad argument");
  if (num == 0) return OCNN_OK;
  key2xyz_kernel<<<blocks_for(num), kBlock, 0, as_stream(stream)>>>(xyz, key, num, depth);
  OCNN_LAUNCH_OK("key2xyz");
  return OCNN_OK;
}

int ocnn_key2idx(int* idx, const uint64_t* key, int num, ocnn_stream_t stream) {
  OCNN_REQUIRE(idx && key && num >= 0, OCNN_E_BADARG, "bad argument");
  if (num == 0) return OCNN_OK;
  key2idx_kernel<<<blocks_for(num), kBlock, 0, as_stream(stream)>>>(idx, key, num);
  OCNN_LAUNCH_OK("key2idx");
  return OCNN_OK;
}

}  // extern "C"
