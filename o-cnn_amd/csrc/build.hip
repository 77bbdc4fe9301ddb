// Octree construction on the device: points2octree (Octree::build,
// octree/octree/octree.cpp:74-121) fused with octree_batch (merge_octrees,
// octree/octree/merge_octrees.cpp:114-198) for a whole batch of point clouds.
//
// Design.  The reference sorts (key, index) pairs per cloud on one CPU core,
// then walks the levels bottom-up, then merges the per-cloud blobs on the host.
// Here ONE sort handles every cloud of the batch: the sort key is
// (cloud << 3*depth | morton), so the sorted order is already the node order of
// the merged batch octree, and child links are global ranks -- exactly what
// merge_octrees produces by offsetting per-cloud links.  Steps:
//   keygen -> stable LSD radix sort (8-bit digits, wavefront-ballot ranking)
//   -> unique leaves (flag scan) -> per level: parents = unique(key >> 3)
//   -> [one copy of the level sizes to the host: the caller must size the blob]
//   -> per level keys / children written straight into the blob, leaf signal
//      averaged per leaf in ascending point order (same float summation order as
//      the reference), neighbour tables level by level.
#include "ocnn_common.h"
#include "scan.h"

#include <map>
#include <mutex>
#include <vector>

namespace ocnn {

// from octree_index.hip
__host__ __device__ inline uint64_t b_spread3(uint64_t v) {
  v &= 0xffffull;
  v = (v | (v << 32)) & 0x00ff00000000ffffull;
  v = (v | (v << 16)) & 0x00ff0000ff0000ffull;
  v = (v | (v << 8)) & 0xf00f00f00f00f00full;
  v = (v | (v << 4)) & 0x30c30c30c30c30c3ull;
  v = (v | (v << 2)) & 0x9249249249249249ull;
  return v;
}
__host__ __device__ inline uint64_t b_compact3(uint64_t v) {
  v &= 0x9249249249249249ull;
  v = (v | (v >> 2)) & 0x30c30c30c30c30c3ull;
  v = (v | (v >> 4)) & 0xf00f00f00f00f00full;
  v = (v | (v >> 8)) & 0x00ff0000ff0000ffull;
  v = (v | (v >> 16)) & 0x00ff00000000ffffull;
  v = (v | (v >> 32)) & 0xffffull;
  return v;
}

namespace {

struct CloudDesc {
  const float* xyz;
  const float* normal;
  const float* feature;
  const float* label;
  int offset, count;  // position of the cloud's points in the concatenated order
};

constexpr int kMaxLevels = 17;
struct Counts {            // device-resident, copied to the host once
  int nne[kMaxLevels];     // non-empty nodes per depth (valid for depth >= full_layer)
  int pad[15];
};

struct BuildGeom {
  int depth, full_layer, n_clouds;
  int64_t n_points;
  float bbmin[3];
  float mul;               // 2^depth / bbox width, computed on the host in fp32
};

// ---- 1. keys -----------------------------------------------------------------------
__device__ inline int find_cloud(const CloudDesc* __restrict__ clouds, int n_clouds, int64_t i) {
  int lo = 0, hi = n_clouds - 1;
  while (lo < hi) {  // last cloud with offset <= i
    int mid = (lo + hi + 1) >> 1;
    if (clouds[mid].offset <= i) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// Correctly rounded fp32 square root and quotient, taken through fp64: a 53-bit
// result rounded once more to 24 bits is the correctly rounded fp32 result for both
// operations (53 >= 2*24 + 2), whatever the fp32 intrinsics of the toolchain do.
__device__ inline float sqrt_rn(float x) { return (float)sqrt((double)x); }
__device__ inline float div_rn(float a, float b) { return (float)((double)a / (double)b); }

// scaled coordinate: (p - bbmin) * mul, two separately rounded fp32 operations
// (octree.cpp:155-170); never contracted into an FMA
__device__ inline float scale_coord(float p, float bbmin, float mul) {
  return __fmul_rn(__fsub_rn(p, bbmin), mul);
}

__global__ void keygen_kernel(uint64_t* __restrict__ key, uint32_t* __restrict__ val,
    const CloudDesc* __restrict__ clouds, BuildGeom g) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= g.n_points) return;
  int b = find_cloud(clouds, g.n_clouds, i);
  const float* p = clouds[b].xyz + 3 * (i - clouds[b].offset);
  uint64_t m = (1ull << g.depth) - 1;
  uint64_t k = 0;
#pragma unroll
  for (int j = 0; j < 3; ++j) {
    // float -> unsigned truncation as static_cast<uintk> (octree.cpp:184); only the low
    // `depth` bits are interleaved (octree_nn.cpp:551-560)
    uint32_t q = (uint32_t)scale_coord(p[j], g.bbmin[j], g.mul);
    k |= b_spread3(q & m) << (2 - j);
  }
  key[i] = ((uint64_t)b << (3 * g.depth)) | k;
  val[i] = (uint32_t)i;
}

// ---- 2. radix sort (LSD, 8-bit digits, stable) ----------------------------------------
constexpr int kSortItems = 8;
constexpr int kSortTile = kBlock * kSortItems;   // 2048 elements per workgroup
constexpr int kWaves = kBlock / 64;

__global__ void radix_hist_kernel(const uint64_t* __restrict__ key, int64_t n, int shift,
    int* __restrict__ hist, int n_blocks) {
  __shared__ int h[256];
  h[threadIdx.x] = 0;
  __syncthreads();
  int64_t base = (int64_t)blockIdx.x * kSortTile;
#pragma unroll
  for (int q = 0; q < kSortItems; ++q) {
    int64_t i = base + q * kBlock + threadIdx.x;
    if (i < n) atomicAdd(&h[(int)((key[i] >> shift) & 255)], 1);
  }
  __syncthreads();
  hist[(int64_t)threadIdx.x * n_blocks + blockIdx.x] = h[threadIdx.x];  // digit-major
}

// Scan of the digit-major histogram in two levels: workgroup d turns row d (the counts of
// digit d in every tile) into exclusive offsets within the digit and records the digit
// total; the scatter kernel adds the exclusive scan of the 256 totals itself.
__global__ void radix_scan_kernel(int* __restrict__ hist, int n_blocks, int* __restrict__ digit_total) {
  __shared__ int carry;
  int* row = hist + (int64_t)blockIdx.x * n_blocks;
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  for (int start = 0; start < n_blocks; start += kBlock) {
    int i = start + threadIdx.x;
    int v = i < n_blocks ? row[i] : 0;
    int total;
    int ex = block_exclusive_scan(v, &total);
    int c = carry;
    if (i < n_blocks) row[i] = c + ex;
    __syncthreads();
    if (threadIdx.x == 0) carry = c + total;
    __syncthreads();
  }
  if (threadIdx.x == 0) digit_total[blockIdx.x] = carry;
}

// Each round places 256 consecutive elements; inside a wavefront the rank among
// equal digits comes from eight ballots (one per digit bit), across wavefronts and
// rounds from per-digit running counters in LDS.  Element order (round, wavefront,
// lane) equals the input order, which keeps the sort stable.
__global__ void radix_scatter_kernel(const uint64_t* __restrict__ key_in, const uint32_t* __restrict__ val_in,
    uint64_t* __restrict__ key_out, uint32_t* __restrict__ val_out, int64_t n, int shift,
    const int* __restrict__ hist, int n_blocks, const int* __restrict__ digit_total) {
  __shared__ int running[256];
  __shared__ int wave_cnt[kWaves][256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  {
    int total;
    int digit_base = block_exclusive_scan(digit_total[threadIdx.x], &total);
    running[threadIdx.x] = digit_base + hist[(int64_t)threadIdx.x * n_blocks + blockIdx.x];
  }
#pragma unroll
  for (int w = 0; w < kWaves; ++w) wave_cnt[w][threadIdx.x] = 0;
  __syncthreads();
  int64_t base = (int64_t)blockIdx.x * kSortTile;
  for (int q = 0; q < kSortItems; ++q) {
    int64_t i = base + q * kBlock + threadIdx.x;
    bool valid = i < n;
    uint64_t k = valid ? key_in[i] : 0;
    uint32_t v = valid ? val_in[i] : 0;
    int d = (int)((k >> shift) & 255);
    uint64_t peers = __ballot(valid);
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      uint64_t m = __ballot((d >> b) & 1);
      peers &= ((d >> b) & 1) ? m : ~m;
    }
    int rank = __popcll(peers & ((1ull << lane) - 1));
    if (valid && rank == 0) wave_cnt[wave][d] = __popcll(peers);
    __syncthreads();
    if (valid) {
      int pos = running[d] + rank;
      for (int w = 0; w < wave; ++w) pos += wave_cnt[w][d];
      key_out[pos] = k;
      val_out[pos] = v;
    }
    __syncthreads();
    {
      int t = 0;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) { t += wave_cnt[w][threadIdx.x]; wave_cnt[w][threadIdx.x] = 0; }
      running[threadIdx.x] += t;
    }
    __syncthreads();
  }
}

// ---- 3. unique leaves and parent levels ------------------------------------------------
struct LeafPred {
  const uint64_t* key; int64_t n;
  __device__ bool operator()(int64_t i) const { return i == 0 || key[i] != key[i - 1]; }
};
struct LeafOut {
  const uint64_t* key; uint64_t* ukey; int* ustart; int64_t n;
  __device__ void operator()(int64_t i, bool f, int rank) const {
    if (f) { ukey[rank] = key[i]; ustart[rank] = (int)i; }
    if (i == n - 1) ustart[rank + (f ? 1 : 0)] = (int)n;
  }
};
// list_d (size *n_dev) -> list_{d-1}: heads of runs of equal key >> 3
struct ParentPred {
  const uint64_t* list; const int* n_dev;
  __device__ bool operator()(int64_t j) const {
    return j < *n_dev && (j == 0 || (list[j] >> 3) != (list[j - 1] >> 3));
  }
};
struct ParentOut {
  const uint64_t* list; const int* n_dev; uint64_t* parent_list; int* prank;
  __device__ void operator()(int64_t j, bool f, int rank) const {
    if (j >= *n_dev) return;
    int r = rank + (f ? 1 : 0) - 1;  // rank of this element's parent
    prank[j] = r;
    if (f) parent_list[r] = list[j] >> 3;
  }
};

// ---- 4. emit: structure -------------------------------------------------------------------
struct EmitGeom {
  int depth, full_layer, n_clouds, key2xyz, key_channel;
};

__device__ inline uint64_t out_key(uint64_t morton, int d, int cloud, int key2xyz) {
  // raw Morton key, or packed (x, y, z) 16-bit fields (Octree::key_to_xyz, octree.cpp:1137-1156);
  // the cloud index goes to the top 16 bits as merge_octrees does (merge_octrees.cpp:126-131)
  uint64_t k = morton;
  if (key2xyz) {
    uint64_t m = d >= 16 ? 0xffffull : ((1ull << d) - 1);
    k = (b_compact3(morton >> 2) & m) | ((b_compact3(morton >> 1) & m) << 16) | ((b_compact3(morton) & m) << 32);
  }
  return (k & 0x0000ffffffffffffull) | ((uint64_t)(cloud & 0xffff) << 48);
}

// full layers: node t = cloud * 8^d + i, key i, child t (or -1 on the last full layer)
__global__ void emit_full_kernel(uint64_t* __restrict__ key, int* __restrict__ child, int d, int64_t total,
    EmitGeom g) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= total) return;
  int64_t per = (int64_t)1 << (3 * d);
  int cloud = (int)(t / per);
  uint64_t i = (uint64_t)(t % per);
  key[t] = out_key(i, d, cloud, g.key2xyz);
  child[t] = d < g.full_layer ? (int)t : -1;
}
// sparse layers: node t = 8 * parent_rank + octant; key from the parent's key
__global__ void emit_sparse_kernel(uint64_t* __restrict__ key, int* __restrict__ child, int d, int64_t total,
    const uint64_t* __restrict__ parent_list, EmitGeom g) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= total) return;
  uint64_t pk = parent_list[t >> 3];               // cloud << 3(d-1) | morton_{d-1}
  int cloud = (int)(pk >> (3 * (d - 1)));
  uint64_t pm = pk & ((1ull << (3 * (d - 1))) - 1);
  key[t] = out_key((pm << 3) | (uint64_t)(t & 7), d, cloud, g.key2xyz);
  child[t] = -1;
}
// child links: the j-th non-empty node of depth d points to rank j
__global__ void emit_links_kernel(int* __restrict__ child, int d, int nne, const uint64_t* __restrict__ list,
    const int* __restrict__ prank, int* __restrict__ leaf_node, EmitGeom g) {
  int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= nne) return;
  uint64_t k = list[j];
  int64_t node;
  if (d == g.full_layer) {
    int cloud = (int)(k >> (3 * d));
    node = ((int64_t)cloud << (3 * d)) + (int64_t)(k & ((1ull << (3 * d)) - 1));
  } else {
    node = ((int64_t)prank[j] << 3) + (int64_t)(k & 7);
  }
  child[node] = j;
  if (leaf_node) leaf_node[j] = (int)node;
}

struct HeaderArg { uint32_t w[OCNN_HEADER_BYTES / 4]; };
__global__ void write_header_kernel(uint32_t* __restrict__ dst, HeaderArg h) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < OCNN_HEADER_BYTES / 4) dst[i] = h.w[i];
}

__global__ void fill_f32_kernel(float* p, int64_t n, float v) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += step) p[i] = v;
}
__global__ void split_kernel(float* __restrict__ split, const int* __restrict__ child, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) split[i] = child[i] < 0 ? 0.0f : 1.0f;  // calc_split_label, octree.cpp:1158-1178
}

// ---- 5. emit: leaf signal -----------------------------------------------------------------
struct SignalGeom {
  int depth, n_clouds, nnum_d;      // nnum_d = node count of the finest level (row length)
  int ch_normal, ch_feature, has_label, has_dis, save_pts;
  float bbmin[3], mul;
};

// One thread per non-empty leaf; its points are visited in ascending original index
// (the sort is stable), so every sum is taken in the reference's order
// (octree.cpp:312-452).  All float operations are individually rounded.
__global__ void leaf_signal_kernel(float* __restrict__ feature, float* __restrict__ label_out, int n_leaf,
    const uint64_t* __restrict__ ukey, const int* __restrict__ ustart, const uint32_t* __restrict__ sorted_idx,
    const int* __restrict__ leaf_node, const CloudDesc* __restrict__ clouds, SignalGeom g) {
  int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= n_leaf) return;
  const int cloud = (int)(ukey[j] >> (3 * g.depth));
  const CloudDesc cd = clouds[cloud];
  const int s0 = ustart[j], s1 = ustart[j + 1];
  const int node = leaf_node[j];
  const int64_t H = g.nnum_d;
  float* out = feature + node;  // channel c lives at out[c * H]
  int ch = 0;
  float nrm[3] = {0.0f, 0.0f, 0.0f};
  if (cd.normal) {
    float acc[3] = {0.0f, 0.0f, 0.0f};
    for (int i = s0; i < s1; ++i) {
      const float* q = cd.normal + 3 * (int64_t)(sorted_idx[i] - cd.offset);
      for (int c = 0; c < 3; ++c) acc[c] = __fadd_rn(acc[c], q[c]);
    }
    float len = 0.0f;
    for (int c = 0; c < 3; ++c) len = __fadd_rn(len, __fmul_rn(acc[c], acc[c]));
    float factor = sqrt_rn(len);
    if (factor < 1.0e-6f) {
      const float* q = cd.normal + 3 * (int64_t)(sorted_idx[s0] - cd.offset);
      len = 0.0f;
      for (int c = 0; c < 3; ++c) { acc[c] = q[c]; len = __fadd_rn(len, __fmul_rn(acc[c], acc[c])); }
      factor = __fadd_rn(sqrt_rn(len), 1.0e-30f);
    }
    for (int c = 0; c < 3; ++c) { nrm[c] = div_rn(acc[c], factor); out[(ch + c) * H] = nrm[c]; }
    ch += 3;
  }
  const float count = __fadd_rn((float)(s1 - s0), 1.0e-30f);
  float avg_pt[3] = {0.0f, 0.0f, 0.0f};
  if (g.has_dis || g.save_pts) {
    for (int i = s0; i < s1; ++i) {
      const float* q = cd.xyz + 3 * (int64_t)(sorted_idx[i] - cd.offset);
      for (int c = 0; c < 3; ++c) avg_pt[c] = __fadd_rn(avg_pt[c], scale_coord(q[c], g.bbmin[c], g.mul));
    }
    float dis[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int c = 0; c < 3; ++c) {
      avg_pt[c] = div_rn(avg_pt[c], count);
      float fract = __fsub_rn(avg_pt[c], truncf(avg_pt[c]));  // std::modf
      dis[c] = __fsub_rn(fract, 0.5f);
      if (cd.normal) dis[3] = __fadd_rn(dis[3], __fmul_rn(dis[c], nrm[c]));
      else dis[3] = 1.0f;
    }
    if (g.has_dis) {
      const float mul = 1.1547f;  // 2 / sqrt(3), octree.cpp:405
      if (cd.normal) { out[ch * H] = __fmul_rn(dis[3], mul); ch += 1; }
      else {
        for (int c = 0; c < 3; ++c) out[(ch + c) * H] = dis[c];
        out[(ch + 3) * H] = __fmul_rn(dis[3], mul);
        ch += 4;
      }
    }
  }
  if (cd.feature) {
    for (int c = 0; c < g.ch_feature; ++c) {
      float acc = 0.0f;
      for (int i = s0; i < s1; ++i)
        acc = __fadd_rn(acc, cd.feature[(int64_t)g.ch_feature * (sorted_idx[i] - cd.offset) + c]);
      out[(ch + c) * H] = div_rn(acc, count);
    }
    ch += g.ch_feature;
  }
  if (g.save_pts) {
    for (int c = 0; c < 3; ++c) out[(ch + c) * H] = avg_pt[c];
    ch += 3;
  }
  if (g.has_label && cd.label) {
    // majority label, smallest label on a tie (std::max_element, octree.cpp:397):
    // walk the distinct labels in increasing order
    int last = -1, best = -1, best_cnt = 0;
    for (;;) {
      int m = 0x7fffffff;
      for (int i = s0; i < s1; ++i) {
        int l = (int)cd.label[sorted_idx[i] - cd.offset];
        if (l > last && l < m) m = l;
      }
      if (m == 0x7fffffff) break;
      int cnt = 0;
      for (int i = s0; i < s1; ++i) cnt += ((int)cd.label[sorted_idx[i] - cd.offset] == m) ? 1 : 0;
      if (cnt > best_cnt) { best = m; best_cnt = cnt; }
      last = m;
    }
    if (best_cnt > 0) label_out[node] = (float)best;
  }
}

// ---- neighbour kernels (same arithmetic as octree_index.hip; private copies keep this
// translation unit self-contained) ----------------------------------------------------------
// Sparse-layer neighbour table.  A workgroup takes 256 consecutive parent-level nodes,
// compacts the non-empty ones into LDS (most nodes of a deep level are empty) and then
// every wavefront writes the 64-slot blocks of the compacted nodes, four nodes per
// iteration so that four dependent load chains (neigh -> children) are in flight.
__global__ void b_neigh_sparse_kernel(int* __restrict__ neigh_child, const int* __restrict__ neigh,
    const int* __restrict__ children, int node_num) {
  __shared__ int s_node[kBlock], s_rank[kBlock], s_count;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int i = blockIdx.x * kBlock + threadIdx.x;
  const int l0 = i < node_num ? children[i] : -1;
  int total;
  const int pos = block_exclusive_scan(l0 >= 0 ? 1 : 0, &total);
  if (l0 >= 0) { s_node[pos] = i; s_rank[pos] = l0; }
  if (threadIdx.x == 0) s_count = total;
  __syncthreads();
  const int count = s_count;
  const int x = lane >> 4, y = (lane >> 2) & 3, z = lane & 3;
  const int hx = (x + 1) >> 1, hy = (y + 1) >> 1, hz = (z + 1) >> 1;
  const int octant = (((x + 1) & 1) << 2) | (((y + 1) & 1) << 1) | ((z + 1) & 1);
  for (int e = wave * 4; e < count; e += 4 * (kBlock / 64)) {
    int t[4], rank[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      t[u] = -1;
      rank[u] = -1;
      if (e + u < count) {
        const int node = s_node[e + u];
        rank[u] = s_rank[e + u];
        const int sib = node & 7;
        const int slot = ((hx + (sib >> 2)) << 4) | ((hy + ((sib >> 1) & 1)) << 2) | (hz + (sib & 1));
        t[u] = neigh[((int64_t)(node >> 3) << 6) + slot];
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      int v = -1;
      if (t[u] >= 0) {
        const int l1 = children[t[u]];
        if (l1 >= 0) v = (l1 << 3) + octant;
      }
      if (rank[u] >= 0) neigh_child[((int64_t)rank[u] << 6) + lane] = v;
    }
  }
}
__global__ void b_neigh_full_kernel(int* __restrict__ neigh, int depth, int64_t total) {
  int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= total) return;
  const int64_t node_num = (int64_t)1 << (3 * depth);
  const int64_t groups = node_num >> 3;
  int slot = (int)(id & 63);
  int64_t grp = id >> 6;
  int64_t n = grp / groups;
  uint64_t i = (uint64_t)(grp % groups) << 3;
  uint64_t m = (1ull << depth) - 1;
  uint32_t x0 = (uint32_t)(b_compact3(i >> 2) & m), y0 = (uint32_t)(b_compact3(i >> 1) & m),
           z0 = (uint32_t)(b_compact3(i) & m);
  uint32_t x1 = x0 + (slot >> 4) - 1, y1 = y0 + ((slot >> 2) & 3) - 1, z1 = z0 + (slot & 3) - 1;
  const uint32_t bound = 1u << depth;
  int v = -1;
  if (((x1 | y1 | z1) & bound) == 0)
    v = (int)(((b_spread3(x1 & m) << 2) | (b_spread3(y1 & m) << 1) | b_spread3(z1 & m)) + (uint64_t)n * node_num);
  neigh[id] = v;
}

// ---- host side -------------------------------------------------------------------------------
inline size_t al(size_t v) { return (v + 255) & ~(size_t)255; }

struct Layout {          // byte offsets inside the workspace
  size_t clouds, counts, key[2], val[2], hist, scan, ustart, leaf_node;
  size_t list[kMaxLevels], prank[kMaxLevels];
  size_t total;
  int hist_blocks;
};

Layout make_layout(int64_t N, int B, int depth) {
  Layout L;
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += al(bytes); return o; };
  L.clouds = take(sizeof(CloudDesc) * (size_t)(B > 0 ? B : 1));
  L.counts = take(sizeof(Counts));
  size_t n = (size_t)(N > 0 ? N : 1);
  for (int i = 0; i < 2; ++i) { L.key[i] = take(8 * n); L.val[i] = take(4 * n); }
  L.hist_blocks = (int)((n + kSortTile - 1) / kSortTile);
  L.hist = take(sizeof(int) * 256 * ((size_t)L.hist_blocks + 1));  // + 256 digit totals
  L.scan = take(scan_scratch_bytes((int64_t)n));
  L.ustart = take(4 * (n + 1));
  L.leaf_node = take(4 * n);
  for (int d = 0; d < kMaxLevels; ++d) {
    if (d <= depth) { L.list[d] = take(8 * n); L.prank[d] = take(4 * n); }
    else { L.list[d] = L.prank[d] = 0; }
  }
  L.total = off;
  return L;
}

struct PlanState {
  ocnn_build_params params;
  Info info;
  Layout layout;
  int64_t n_points;
  int n_clouds, sorted_buf;
  int ch_normal, ch_feature, ch_label;
  int nne[kMaxLevels];
  float mul;
};
std::mutex g_plans_mutex;
std::map<void*, PlanState> g_plans;

}  // namespace
}  // namespace ocnn

using namespace ocnn;

extern "C" {

size_t ocnn_points2octree_workspace_bytes(int64_t total_points, int n_clouds, int depth) {
  if (total_points < 0 || n_clouds < 1 || depth < 1 || depth > 16) return 0;
  return make_layout(total_points, n_clouds, depth).total;
}

int ocnn_points2octree_plan(const void* const* points_dev, const void* const* points_info, int n_clouds,
    const ocnn_build_params* params, void* workspace_dev, size_t workspace_bytes, void* info_out,
    ocnn_stream_t stream) {
  OCNN_REQUIRE(points_dev && points_info && params && workspace_dev && info_out, OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(n_clouds >= 1 && n_clouds <= 65535, OCNN_E_BADARG, "n_clouds %d", n_clouds);
  OCNN_REQUIRE(params->merged || n_clouds == 1, OCNN_E_BADARG, "a single-octree blob holds one cloud");
  OCNN_REQUIRE(!params->node_feature && !params->adaptive, OCNN_E_UNSUPPORTED,
      "node_feature / adaptive octrees are not built on the device");
  hipStream_t s = as_stream(stream);

  // ---- headers: every cloud must carry the same properties (OctreeInfo::is_consistent)
  std::vector<CloudDesc> clouds(n_clouds);
  int64_t N = 0;
  const PointsInfo* p0 = static_cast<const PointsInfo*>(points_info[0]);
  for (int i = 0; i < n_clouds; ++i) {
    const PointsInfo* pi = static_cast<const PointsInfo*>(points_info[i]);
    OCNN_REQUIRE(pi && points_dev[i], OCNN_E_BADARG, "null cloud %d", i);
    OCNN_REQUIRE(memcmp(pi->magic, "_POINTS_1.0_", 13) == 0 && pi->pt_num > 0, OCNN_E_FORMAT,
        "cloud %d: bad PointsInfo header", i);
    OCNN_REQUIRE((pi->content_flags & 1) && pi->channels[0] == 3, OCNN_E_FORMAT, "cloud %d: no xyz", i);
    OCNN_REQUIRE(pi->content_flags == p0->content_flags && pi->channels[1] == p0->channels[1] &&
        pi->channels[2] == p0->channels[2] && pi->channels[3] == p0->channels[3], OCNN_E_FORMAT,
        "cloud %d: properties differ from cloud 0", i);
    const char* base = static_cast<const char*>(points_dev[i]);
    CloudDesc& c = clouds[i];
    c.xyz = reinterpret_cast<const float*>(base + pi->ptr_dis[0]);
    c.normal = (pi->content_flags & 2) ? reinterpret_cast<const float*>(base + pi->ptr_dis[1]) : nullptr;
    c.feature = (pi->content_flags & 4) ? reinterpret_cast<const float*>(base + pi->ptr_dis[2]) : nullptr;
    c.label = (pi->content_flags & 8) ? reinterpret_cast<const float*>(base + pi->ptr_dis[3]) : nullptr;
    c.offset = (int)N;
    c.count = pi->pt_num;
    N += pi->pt_num;
    OCNN_REQUIRE(N < (1ll << 31), OCNN_E_BADARG, "more than 2^31 points");
  }
  const int ch_normal = (p0->content_flags & 2) ? p0->channels[1] : 0;
  const int ch_feature = (p0->content_flags & 4) ? p0->channels[2] : 0;
  const int ch_label = (p0->content_flags & 8) ? p0->channels[3] : 0;
  OCNN_REQUIRE(ch_normal == 0 || ch_normal == 3, OCNN_E_FORMAT, "normals must have 3 channels");

  // ---- OctreeInfo::initialize (octree_info.cpp:13-73)
  Info o;
  o.reset();
  o.set_batch_size(1);
  o.set_depth(params->depth);
  o.set_full_layer(params->full_depth);
  o.adp_layer = params->adp_depth;
  o.is_adaptive = 0;
  o.has_node_dis = params->node_dis ? 1 : 0;
  o.key2xyz = params->key2xyz ? 1 : 0;
  o.extrapolate = params->extrapolate ? 1 : 0;
  o.save_pts = params->save_pts ? 1 : 0;
  o.th_norm = params->th_normal;
  o.th_dist = params->th_distance;
  o.set_property(OCNN_KEY, (params->key2xyz && params->depth > 8) ? 2 : 1, -1);
  o.set_property(OCNN_CHILD, 1, -1);
  if (params->split_label) o.set_property(OCNN_SPLIT, 1, -1);
  int channel = ch_normal + ch_feature;
  if (params->node_dis) { channel += 1; if (ch_normal == 0) channel += 3; }
  if (params->save_pts) channel += 3;
  o.set_channel(OCNN_FEATURE, channel);
  o.set_location(OCNN_FEATURE, params->depth);
  if (ch_label == 1) o.set_property(OCNN_LABEL, 1, params->depth);
  for (int i = 0; i < 3; ++i) { o.bbmin[i] = -1.0f; o.bbmax[i] = 1.0f; }
  if (params->has_bbox) for (int i = 0; i < 3; ++i) { o.bbmin[i] = params->bbmin[i]; o.bbmax[i] = params->bbmax[i]; }
  const int depth = o.depth, fl = o.full_layer;
  OCNN_REQUIRE(depth >= 1 && depth <= 16 && fl <= depth, OCNN_E_BADARG, "depth %d full_depth %d", depth, fl);
  OCNN_REQUIRE(o.channel(OCNN_KEY) == 1 || !params->merged, OCNN_E_UNSUPPORTED,
      "octree_batch of two-channel keys (key2xyz with depth > 8)");
  OCNN_REQUIRE(3 * depth + 16 <= 64, OCNN_E_BADARG, "depth too large");
  OCNN_REQUIRE(fl <= 7, OCNN_E_BADARG, "full_depth %d too large for a dense layer", fl);
  OCNN_REQUIRE(((int64_t)n_clouds << (3 * fl)) < (1ll << 28), OCNN_E_BADARG, "full layers too large");

  Layout L = make_layout(N, n_clouds, depth);
  OCNN_REQUIRE(workspace_bytes >= L.total, OCNN_E_WORKSPACE, "workspace %zu < %zu bytes", workspace_bytes, L.total);
  OCNN_REQUIRE((reinterpret_cast<uintptr_t>(workspace_dev) & 255) == 0, OCNN_E_WORKSPACE, "workspace not 256-byte aligned");
  char* ws = static_cast<char*>(workspace_dev);
  CloudDesc* d_clouds = reinterpret_cast<CloudDesc*>(ws + L.clouds);
  Counts* d_counts = reinterpret_cast<Counts*>(ws + L.counts);
  uint64_t* d_key[2] = {reinterpret_cast<uint64_t*>(ws + L.key[0]), reinterpret_cast<uint64_t*>(ws + L.key[1])};
  uint32_t* d_val[2] = {reinterpret_cast<uint32_t*>(ws + L.val[0]), reinterpret_cast<uint32_t*>(ws + L.val[1])};
  int* d_hist = reinterpret_cast<int*>(ws + L.hist);
  int* d_digit_total = d_hist + (int64_t)256 * L.hist_blocks;
  int* d_scan = reinterpret_cast<int*>(ws + L.scan);
  int* d_ustart = reinterpret_cast<int*>(ws + L.ustart);

  OCNN_HIP_OK(hipMemcpyAsync(d_clouds, clouds.data(), sizeof(CloudDesc) * n_clouds, hipMemcpyHostToDevice, s));

  BuildGeom g;
  g.depth = depth;
  g.full_layer = fl;
  g.n_clouds = n_clouds;
  g.n_points = N;
  for (int i = 0; i < 3; ++i) g.bbmin[i] = o.bbmin[i];
  g.mul = float(1 << depth) / o.bbox_max_width();  // octree.cpp:159

  PlanState st;
  memset(&st, 0, sizeof(st));
  int cur = 0;
  if (depth > fl) {
    keygen_kernel<<<blocks_for(N), kBlock, 0, s>>>(d_key[0], d_val[0], d_clouds, g);
    OCNN_LAUNCH_OK("keygen");
    int cloud_bits = 0;
    while ((1 << cloud_bits) < n_clouds) ++cloud_bits;
    int nbits = 3 * depth + cloud_bits;
    for (int shift = 0; shift < nbits; shift += 8) {
      radix_hist_kernel<<<L.hist_blocks, kBlock, 0, s>>>(d_key[cur], N, shift, d_hist, L.hist_blocks);
      radix_scan_kernel<<<256, kBlock, 0, s>>>(d_hist, L.hist_blocks, d_digit_total);
      radix_scatter_kernel<<<L.hist_blocks, kBlock, 0, s>>>(d_key[cur], d_val[cur], d_key[cur ^ 1], d_val[cur ^ 1],
          N, shift, d_hist, L.hist_blocks, d_digit_total);
      OCNN_LAUNCH_OK("radix pass");
      cur ^= 1;
    }
    // unique leaves
    uint64_t* list_D = reinterpret_cast<uint64_t*>(ws + L.list[depth]);
    LeafPred lp{d_key[cur], N};
    LeafOut lo{d_key[cur], list_D, d_ustart, N};
    hipError_t e = flag_scan(lp, lo, N, d_scan, &d_counts->nne[depth], s);
    OCNN_REQUIRE(e == hipSuccess, OCNN_E_HIP, "leaf scan: %s", hipGetErrorString(e));
    // parents, level by level (sizes stay on the device: grids cover the upper bound N)
    for (int d = depth; d > fl; --d) {
      const uint64_t* list = reinterpret_cast<const uint64_t*>(ws + L.list[d]);
      uint64_t* plist = reinterpret_cast<uint64_t*>(ws + L.list[d - 1]);
      int* prank = reinterpret_cast<int*>(ws + L.prank[d]);
      ParentPred pp{list, &d_counts->nne[d]};
      ParentOut po{list, &d_counts->nne[d], plist, prank};
      e = flag_scan(pp, po, N, d_scan, &d_counts->nne[d - 1], s);
      OCNN_REQUIRE(e == hipSuccess, OCNN_E_HIP, "parent scan: %s", hipGetErrorString(e));
    }
    Counts h;
    OCNN_HIP_OK(hipMemcpyAsync(&h, d_counts, sizeof(Counts), hipMemcpyDeviceToHost, s));
    OCNN_HIP_OK(hipStreamSynchronize(s));
    for (int d = fl; d <= depth; ++d) st.nne[d] = h.nne[d];
  } else {
    OCNN_HIP_OK(hipStreamSynchronize(s));  // the cloud table came from host memory of this call
  }

  // ---- node counts (calc_node_num, octree.cpp:285-309; batch sums merge_octrees.cpp:39-90)
  for (int d = 0; d <= depth; ++d) {
    if (d <= fl) o.nnum[d] = n_clouds << (3 * d);
    else o.nnum[d] = st.nne[d - 1] << 3;
    if (d < fl) o.nnum_nempty[d] = o.nnum[d];
    else o.nnum_nempty[d] = depth > fl ? st.nne[d] : 0;
  }
  if (params->merged) {
    o.set_batch_size(n_clouds);
    o.set_property(OCNN_NEIGH, 8, -1);
  }
  o.set_nnum_cum();
  OCNN_REQUIRE(o.set_ptr_dis(), OCNN_E_SHAPE,
      "the octree would exceed the 2 GiB that the 32-bit offsets of the serialized format can address");
  memcpy(info_out, &o, sizeof(Info));

  st.params = *params;
  st.info = o;
  st.layout = L;
  st.n_points = N;
  st.n_clouds = n_clouds;
  st.sorted_buf = cur;
  st.ch_normal = ch_normal;
  st.ch_feature = ch_feature;
  st.ch_label = ch_label;
  st.mul = g.mul;
  {
    std::lock_guard<std::mutex> lock(g_plans_mutex);
    g_plans[workspace_dev] = st;
  }
  return OCNN_OK;
}

int ocnn_points2octree_emit(void* octree_out_dev, const void* info, void* workspace_dev, size_t workspace_bytes,
    ocnn_stream_t stream) {
  OCNN_REQUIRE(octree_out_dev && info && workspace_dev, OCNN_E_BADARG, "null pointer");
  PlanState st;
  {
    std::lock_guard<std::mutex> lock(g_plans_mutex);
    auto it = g_plans.find(workspace_dev);
    OCNN_REQUIRE(it != g_plans.end(), OCNN_E_BADARG, "no plan was made on this workspace");
    st = it->second;
    g_plans.erase(it);
  }
  OCNN_REQUIRE(memcmp(info, &st.info, sizeof(Info)) == 0, OCNN_E_BADARG, "info differs from the planned header");
  OCNN_REQUIRE(workspace_bytes >= st.layout.total, OCNN_E_WORKSPACE, "workspace shrank");
  OCNN_REQUIRE((reinterpret_cast<uintptr_t>(octree_out_dev) & 7) == 0, OCNN_E_BADARG, "blob not 8-byte aligned");
  hipStream_t s = as_stream(stream);
  const Info& o = st.info;
  const Layout& L = st.layout;
  const int depth = o.depth, fl = o.full_layer, B = st.n_clouds;
  char* ws = static_cast<char*>(workspace_dev);
  char* blob = static_cast<char*>(octree_out_dev);
  const CloudDesc* d_clouds = reinterpret_cast<const CloudDesc*>(ws + L.clouds);
  const uint32_t* d_sorted_idx = reinterpret_cast<const uint32_t*>(ws + L.val[st.sorted_buf]);
  const int* d_ustart = reinterpret_cast<const int*>(ws + L.ustart);
  int* d_leaf_node = reinterpret_cast<int*>(ws + L.leaf_node);

  // header (the tail of the 720-byte header block is padding and must be zero)
  HeaderArg hdr;
  memset(&hdr, 0, sizeof(hdr));
  memcpy(&hdr, &o, sizeof(Info));
  write_header_kernel<<<1, kBlock, 0, s>>>(reinterpret_cast<uint32_t*>(blob), hdr);
  OCNN_LAUNCH_OK("write_header");

  EmitGeom eg{depth, fl, B, o.key2xyz, o.channel(OCNN_KEY)};
  const int kch = o.channel(OCNN_KEY);
  if (kch == 2) {  // two-channel keys: the second half of each level stays zero (octree.cpp:1145)
    int64_t cnt = (int64_t)o.total_nnum() * 2 * 2;  // as 4-byte words
    fill_f32_kernel<<<blocks_for(cnt, kBlock * 4), kBlock, 0, s>>>(reinterpret_cast<float*>(blob + o.ptr_dis(OCNN_KEY, 0)), cnt, 0.0f);
  }
  for (int d = 0; d <= depth; ++d) {
    uint64_t* key = reinterpret_cast<uint64_t*>(blob + o.ptr_dis(OCNN_KEY, d));
    int* child = reinterpret_cast<int*>(blob + o.ptr_dis(OCNN_CHILD, d));
    int64_t n = o.nnum[d];
    if (n == 0) continue;
    if (d <= fl) emit_full_kernel<<<blocks_for(n), kBlock, 0, s>>>(key, child, d, n, eg);
    else emit_sparse_kernel<<<blocks_for(n), kBlock, 0, s>>>(key, child, d, n,
        reinterpret_cast<const uint64_t*>(ws + L.list[d - 1]), eg);
    if (d >= fl && depth > fl && st.nne[d] > 0)
      emit_links_kernel<<<blocks_for(st.nne[d]), kBlock, 0, s>>>(child, d, st.nne[d],
          reinterpret_cast<const uint64_t*>(ws + L.list[d]), reinterpret_cast<const int*>(ws + L.prank[d]),
          d == depth ? d_leaf_node : nullptr, eg);
    OCNN_LAUNCH_OK("emit structure");
  }
  // features / labels of the finest level
  const int64_t HD = o.nnum[depth];
  const int fch = o.channel(OCNN_FEATURE);
  float* feature = fch > 0 ? reinterpret_cast<float*>(blob + o.ptr_dis(OCNN_FEATURE, depth)) : nullptr;
  float* label = o.has(OCNN_LABEL) ? reinterpret_cast<float*>(blob + o.ptr_dis(OCNN_LABEL, depth)) : nullptr;
  if (feature && HD > 0) fill_f32_kernel<<<blocks_for(fch * HD, kBlock * 4), kBlock, 0, s>>>(feature, fch * HD, 0.0f);
  if (label && HD > 0) fill_f32_kernel<<<blocks_for(HD, kBlock * 4), kBlock, 0, s>>>(label, HD, -1.0f);
  if (depth > fl && st.nne[depth] > 0 && (feature || label)) {
    SignalGeom sg;
    sg.depth = depth;
    sg.n_clouds = B;
    sg.nnum_d = (int)HD;
    sg.ch_normal = st.ch_normal;
    sg.ch_feature = st.ch_feature;
    sg.has_label = label != nullptr;
    sg.has_dis = o.has_node_dis;
    sg.save_pts = o.save_pts;
    for (int i = 0; i < 3; ++i) sg.bbmin[i] = o.bbmin[i];
    sg.mul = st.mul;
    leaf_signal_kernel<<<blocks_for(st.nne[depth], 64), 64, 0, s>>>(feature, label, st.nne[depth],
        reinterpret_cast<const uint64_t*>(ws + L.list[depth]), d_ustart, d_sorted_idx, d_leaf_node, d_clouds, sg);
    OCNN_LAUNCH_OK("leaf_signal");
  }
  if (o.has(OCNN_SPLIT)) {
    int64_t n = o.total_nnum();
    split_kernel<<<blocks_for(n), kBlock, 0, s>>>(reinterpret_cast<float*>(blob + o.ptr_dis(OCNN_SPLIT, 0)),
        reinterpret_cast<const int*>(blob + o.ptr_dis(OCNN_CHILD, 0)), n);
    OCNN_LAUNCH_OK("split");
  }
  if (o.has(OCNN_NEIGH)) {  // merge_octrees.cpp:185-197; depth 0 holds no table (left zero)
    int64_t n0 = (int64_t)o.nnum[0] * 8;
    fill_f32_kernel<<<blocks_for(n0), kBlock, 0, s>>>(reinterpret_cast<float*>(blob + o.ptr_dis(OCNN_NEIGH, 0)), n0, 0.0f);
    for (int d = 1; d <= depth; ++d) {
      int* neigh = reinterpret_cast<int*>(blob + o.ptr_dis(OCNN_NEIGH, d));
      if (d <= fl) {
        int64_t total = (int64_t)B << (3 * d + 3);
        b_neigh_full_kernel<<<blocks_for(total), kBlock, 0, s>>>(neigh, d, total);
      } else if (o.nnum[d - 1] > 0) {
        b_neigh_sparse_kernel<<<blocks_for(o.nnum[d - 1]), kBlock, 0, s>>>(neigh,
            reinterpret_cast<const int*>(blob + o.ptr_dis(OCNN_NEIGH, d - 1)),
            reinterpret_cast<const int*>(blob + o.ptr_dis(OCNN_CHILD, d - 1)), o.nnum[d - 1]);
      }
      OCNN_LAUNCH_OK("neigh");
    }
  }
  return OCNN_OK;
}

}  // extern "C"
