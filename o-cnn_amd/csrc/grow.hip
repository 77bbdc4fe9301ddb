// Blob-level operations on serialized octrees that live on the device:
//   octree_batch  (merge_octrees, octree/octree/merge_octrees.cpp:7-198)
//   octree_new / octree_grow / octree_update (pytorch/cpp/octree_grow.cpp:13-190)
// Header arithmetic runs on the host from the caller's host copies of the
// headers; the payload never leaves the device.
#include "ocnn_common.h"
#include "octree_kernels.h"
#include "scan.h"

#include <algorithm>
#include <atomic>
#include <chrono>
#include <mutex>
#include <vector>

namespace ocnn {
namespace {

struct SplitPred {   // label == split
  const int* label;
  int split;
  __device__ bool operator()(int64_t i) const { return label[i] == split; }
};

struct HeaderArg { uint32_t w[OCNN_HEADER_BYTES / 4]; };
__global__ void g_write_header_kernel(uint32_t* __restrict__ dst, HeaderArg h) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < OCNN_HEADER_BYTES / 4) dst[i] = h.w[i];
}
int write_header(void* blob, const Info& o, hipStream_t s) {
  HeaderArg h;
  memset(&h, 0, sizeof(h));
  memcpy(&h, &o, sizeof(Info));
  g_write_header_kernel<<<1, kBlock, 0, s>>>(reinterpret_cast<uint32_t*>(blob), h);
  OCNN_LAUNCH_OK("write_header");
  return OCNN_OK;
}

__global__ void g_zero_kernel(uint32_t* p, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += step) p[i] = 0u;
}
int zero_payload(void* blob, const Info& o, hipStream_t s) {
  int64_t words = (o.sizeof_octree() - OCNN_HEADER_BYTES) / 4;
  if (words <= 0) return OCNN_OK;
  unsigned grid = blocks_for(words, kBlock * 8);
  if (grid > 65535u * 16) grid = 65535u * 16;
  g_zero_kernel<<<grid, kBlock, 0, s>>>(reinterpret_cast<uint32_t*>(static_cast<char*>(blob) + OCNN_HEADER_BYTES), words);
  OCNN_LAUNCH_OK("zero_payload");
  return OCNN_OK;
}

template <typename T>
__global__ void g_copy_kernel(T* __restrict__ dst, const T* __restrict__ src, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += step) dst[i] = src[i];
}
template <typename T>
int copy_dev(T* dst, const T* src, int64_t n, hipStream_t s) {
  if (n <= 0) return OCNN_OK;
  unsigned grid = blocks_for(n, kBlock * 4);
  if (grid > 65535u * 16) grid = 65535u * 16;
  g_copy_kernel<T><<<grid, kBlock, 0, s>>>(dst, src, n);
  OCNN_LAUNCH_OK("copy");
  return OCNN_OK;
}

__global__ void g_seq_key_child_kernel(uint64_t* __restrict__ key, int* __restrict__ child, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  if (key) key[i] = (uint64_t)i;
  child[i] = i;
}

// ---- octree_grow in one launch -------------------------------------------------------
// The grown blob is a list of byte ranges, each produced by one rule: the header, copies
// of the old properties, zeros, and the new depth's child indices 0..n-1; the new depth's
// keys are written from the side of their parents (the old deepest level), one item per
// (parent, child).  Ranges are dealt out over the workgroups of ONE launch.  A range is
// walked in 4-byte words counted from the 256-byte line its destination starts in, so
// that every wavefront stores one whole aligned line.
constexpr int kGrowRanges = 20;
constexpr int kGrowWordsPerBlock = kBlock * 16;
enum { kGrowHeader = 0, kGrowCopy, kGrowZero, kGrowSequence, kGrowKeyChild, kGrowNeigh };
struct GrowPlan {
  int n;
  int kind[kGrowRanges];
  unsigned first_block[kGrowRanges + 1];
  int64_t dst[kGrowRanges], src[kGrowRanges], words[kGrowRanges];  // byte offsets; words or items
  int64_t parent_key, parent_child, parent_neigh;                     // byte offsets in the old blob
  int parent_nodes, new_groups;                                       // nodes of the old deepest level, sibling groups of the new one
};

__global__ void __launch_bounds__(kBlock) g_grow_kernel(char* __restrict__ out,
    const char* __restrict__ in, GrowPlan p, HeaderArg h) {
  int r = 0;
  while (r + 1 < p.n && blockIdx.x >= p.first_block[r + 1]) ++r;
  const int kind = p.kind[r];
  const int64_t begin = (int64_t)(blockIdx.x - p.first_block[r]) * kGrowWordsPerBlock;
  if (kind == kGrowNeigh) {   // the new level's neighbour table from the old blob's, beside the copies (calc_neigh, octree_nn.cpp:357-380)
    const int wave = (int)((blockIdx.x - p.first_block[r]) * (kBlock / 64) + (threadIdx.x >> 6));
    neigh_sparse_wave<2>(reinterpret_cast<int*>(out + p.dst[r]), reinterpret_cast<const int*>(in + p.parent_neigh),
        reinterpret_cast<const int*>(in + p.parent_child), p.parent_nodes, 1, p.new_groups, wave, 0);
    return;
  }
  if (kind == kGrowKeyChild) {  // generate_key, octree_nn.cpp:427-463, for the children of the old level
    const uint64_t* pkey = reinterpret_cast<const uint64_t*>(in + p.parent_key);
    const int* pchild = reinterpret_cast<const int*>(in + p.parent_child);
    uint64_t* key = reinterpret_cast<uint64_t*>(out + p.dst[r]);
    const int64_t stop = min(p.words[r], begin + kGrowWordsPerBlock);
    for (int64_t id = begin + threadIdx.x; id < stop; id += kBlock) {
      int i = (int)(id >> 3), j = (int)(id & 7);
      int label = pchild[i];
      if (label < 0) continue;
      uint64_t k0 = pkey[i];
      uint64_t x = (((k0 & 0xffffu) << 1) | ((j >> 2) & 1)) & 0xffffu;
      uint64_t y = ((((k0 >> 16) & 0xffffu) << 1) | ((j >> 1) & 1)) & 0xffffu;
      uint64_t z = ((((k0 >> 32) & 0xffffu) << 1) | (j & 1)) & 0xffffu;
      key[8 * (int64_t)label + j] = x | (y << 16) | (z << 32) | (k0 & 0xffff000000000000ull);
    }
    return;
  }
  const uintptr_t dst_addr = reinterpret_cast<uintptr_t>(out) + p.dst[r];
  const int64_t lead = (int64_t)((dst_addr & 255) >> 2);  // words between the line start and the range
  uint32_t* dst = reinterpret_cast<uint32_t*>(dst_addr) - lead;
  const uint32_t* src = reinterpret_cast<const uint32_t*>(in + p.src[r]) - lead;
  const int64_t stop = min(p.words[r] + lead, begin + kGrowWordsPerBlock);
  // four words a thread and step (one 16-byte store; the source of a copy sits at another offset
  // inside its lines, so it is read as 16 bytes only when it happens to be aligned)
  const bool src16 = kind == kGrowCopy && (reinterpret_cast<uintptr_t>(src) & 15) == 0;
  for (int64_t v = begin + 4 * (int64_t)threadIdx.x; v < stop; v += 4 * kBlock) {
    if (v >= lead && v + 4 <= stop) {
      uint4 q = make_uint4(0u, 0u, 0u, 0u);
      if (src16) q = *reinterpret_cast<const uint4*>(src + v);
      else if (kind == kGrowCopy) q = make_uint4(src[v], src[v + 1], src[v + 2], src[v + 3]);
      else if (kind == kGrowSequence) q = make_uint4((uint32_t)(v - lead), (uint32_t)(v - lead + 1), (uint32_t)(v - lead + 2), (uint32_t)(v - lead + 3));
      else if (kind == kGrowHeader) q = make_uint4(h.w[v - lead], h.w[v - lead + 1], h.w[v - lead + 2], h.w[v - lead + 3]);
      *reinterpret_cast<uint4*>(dst + v) = q;
      continue;
    }
    for (int64_t u = max(v, lead); u < min(v + 4, stop); ++u) {
      uint32_t val = 0;
      if (kind == kGrowCopy) val = src[u];
      else if (kind == kGrowSequence) val = (uint32_t)(u - lead);
      else if (kind == kGrowHeader) val = h.w[u - lead];
      dst[u] = val;
    }
  }
}

struct GrowRanges {
  GrowPlan plan;
  void add(int kind, int64_t dst, int64_t src, int64_t count) {
    if (count <= 0) return;
    plan.kind[plan.n] = kind;
    plan.dst[plan.n] = dst;
    plan.src[plan.n] = src;
    plan.words[plan.n] = count;
    ++plan.n;
  }
  // blocks per range; a range that is walked from its line start has up to 63 extra words
  unsigned finish() {
    unsigned total = 0;
    for (int r = 0; r < plan.n; ++r) {
      plan.first_block[r] = total;
      int64_t span = plan.words[r] + (plan.kind[r] == kGrowKeyChild || plan.kind[r] == kGrowNeigh ? 0 : 63);
      total += (unsigned)((span + kGrowWordsPerBlock - 1) / kGrowWordsPerBlock);
    }
    plan.first_block[plan.n] = total;
    return total;
  }
};

// ---- merge ---------------------------------------------------------------------
// Per depth one launch per property over the merged node range; the source octree
// of a node is found by binary search in the per-depth cumulative node counts.
struct MergeTable {       // device layout: arrays indexed [d * (B+1) + b] / [(prop*B + b) * 17 + d]
  const int* cum;         // node offset of octree b at depth d
  const int* cum_ne;      // non-empty offset
  const int64_t* src_off; // byte offset of (prop, octree, depth) inside its blob, -1 if absent
  const char* const* src; // blob pointers
  int B;
};
__device__ inline int find_src(const int* __restrict__ cum, int B, int t) {
  int lo = 0, hi = B - 1;
  while (lo < hi) {
    int mid = (lo + hi + 1) >> 1;
    if (cum[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}
enum { kPKey = 0, kPChild = 1, kPFeature = 2, kPLabel = 3, kPSplit = 4, kPCount = 5 };

// One launch merges every property of every depth: the launch is cut into segments of whole
// workgroups (header, zero ranges, key + child of a depth, one float property of a depth).
enum { kMergeHeader = 0, kMergeZero, kMergeKeyChild, kMergeFloat };
constexpr int kMergeSegMax = 96;
struct MergeSeg {
  int kind, depth, prop, channel;
  unsigned first_block, pad;
  int64_t dst_key, dst_child;   // byte offsets in the merged blob (dst_key also: zero / float target)
  int64_t count;                // nodes of the depth, or 4-byte words to clear
};

// source octree of the workgroup's nodes: one search per workgroup when all its nodes come
// from one octree (the rule on large levels), a short search per thread otherwise
__device__ inline int block_src(const int* __restrict__ cum, int B, int t_first, int t_last, int t,
    int* s_range) {
  if (threadIdx.x == 0) {
    s_range[0] = find_src(cum, B, t_first);
    s_range[1] = find_src(cum, B, t_last);
  }
  __syncthreads();
  int lo = s_range[0], hi = s_range[1];
  while (lo < hi) {
    int mid = (lo + hi + 1) >> 1;
    if (cum[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

__global__ void __launch_bounds__(kBlock) merge_kernel(char* __restrict__ blob, MergeTable m,
    const MergeSeg* __restrict__ segs, int n_seg, HeaderArg h) {
  __shared__ int s_range[2];
  int lo = 0, hi = n_seg - 1;
  while (lo < hi) {
    int mid = (lo + hi + 1) >> 1;
    if (segs[mid].first_block <= blockIdx.x) lo = mid; else hi = mid - 1;
  }
  const MergeSeg sg = segs[lo];
  const int64_t i = (int64_t)(blockIdx.x - sg.first_block) * kBlock + threadIdx.x;
  if (sg.kind == kMergeHeader) {
    if (i < OCNN_HEADER_BYTES / 4) reinterpret_cast<uint32_t*>(blob)[i] = h.w[i];
    return;
  }
  if (sg.kind == kMergeZero) {
    uint32_t* dst = reinterpret_cast<uint32_t*>(blob + sg.dst_key);
    for (int64_t w = i * 4; w < min(sg.count, i * 4 + 4); ++w) dst[w] = 0u;
    return;
  }
  const int d = sg.depth, n = (int)sg.count;
  const int t_first = (int)((int64_t)(blockIdx.x - sg.first_block) * kBlock);
  const int t = (int)i;
  const int* cum = m.cum + d * (m.B + 1);
  const int b = block_src(cum, m.B, t_first, min(t_first + kBlock, n) - 1, min(t, n - 1), s_range);
  if (t >= n) return;
  const int j = t - cum[b];
  const char* src = m.src[b];
  if (sg.kind == kMergeKeyChild) {
    // keys get the octree's index in their top 16 bits, child links move up by the non-empty
    // nodes of the octrees before (merge_octrees.cpp:126-145)
    if (sg.dst_key >= 0) {
      uint64_t k = reinterpret_cast<const uint64_t*>(src + m.src_off[(kPKey * m.B + b) * 17 + d])[j];
      reinterpret_cast<uint64_t*>(blob + sg.dst_key)[t] = (k & 0x0000ffffffffffffull) | ((uint64_t)(b & 0xffff) << 48);
    }
    if (sg.dst_child >= 0) {
      int c = reinterpret_cast<const int*>(src + m.src_off[(kPChild * m.B + b) * 17 + d])[j];
      reinterpret_cast<int*>(blob + sg.dst_child)[t] = c == -1 ? -1 : c + m.cum_ne[d * (m.B + 1) + b];
    }
    return;
  }
  // float property with `channel` channels: dst[c, t] = src_b[c, j] (merge_octrees.cpp:147-183)
  const int nb = cum[b + 1] - cum[b];
  const float* fsrc = reinterpret_cast<const float*>(src + m.src_off[(sg.prop * m.B + b) * 17 + d]);
  float* dst = reinterpret_cast<float*>(blob + sg.dst_key);
  for (int c = 0; c < sg.channel; ++c) dst[(int64_t)c * n + t] = fsrc[(int64_t)c * nb + j];
}

// Pinned staging buffers for host tables that a stream copies asynchronously.  A buffer is
// busy until the event recorded behind its copy has completed; buffers live as long as the
// process.
struct Staging {
  void* host = nullptr;
  size_t bytes = 0;
  hipEvent_t done = nullptr;
  bool busy = false;
};
std::mutex g_staging_mutex;
std::vector<Staging*> g_staging;
Staging* take_staging(size_t bytes) {
  std::lock_guard<std::mutex> lock(g_staging_mutex);
  for (Staging* st : g_staging) {
    if (st->busy && hipEventQuery(st->done) == hipSuccess) st->busy = false;
    if (!st->busy && st->bytes >= bytes) { st->busy = true; return st; }
  }
  Staging* st = new Staging();
  size_t cap = bytes < 65536 ? 65536 : bytes;
  if (hipHostMalloc(&st->host, cap, hipHostMallocDefault) != hipSuccess ||
      hipEventCreateWithFlags(&st->done, hipEventDisableTiming) != hipSuccess) {
    if (st->host) (void)hipHostFree(st->host);
    delete st;
    return nullptr;
  }
  st->bytes = cap;
  st->busy = true;
  g_staging.push_back(st);
  return st;
}

inline size_t al(size_t v) { return (v + 255) & ~(size_t)255; }
struct MergeLayout { size_t cum, cum_ne, src_off, src, segs, total; };
MergeLayout merge_layout(int B, int depth) {
  MergeLayout L;
  size_t off = 0;
  auto take = [&](size_t b) { size_t o = off; off += al(b); return o; };
  L.cum = take(sizeof(int) * (size_t)(depth + 1) * (B + 1));
  L.cum_ne = take(sizeof(int) * (size_t)(depth + 1) * (B + 1));
  L.src_off = take(sizeof(int64_t) * (size_t)kPCount * B * 17);
  L.src = take(sizeof(char*) * (size_t)B);
  L.segs = take(sizeof(MergeSeg) * (size_t)kMergeSegMax);
  L.total = off;
  return L;
}

}  // namespace
}  // namespace ocnn

using namespace ocnn;

extern "C" {

// ---- octree_batch ------------------------------------------------------------------
int ocnn_octree_batch_info(const void* const* infos, int n, void* out_info) {
  OCNN_REQUIRE(infos && out_info && n >= 1 && n <= 65535, OCNN_E_BADARG, "bad argument");
  const Info* first = as_info(infos[0]);
  for (int i = 0; i < n; ++i) {
    OCNN_REQUIRE(infos[i], OCNN_E_BADARG, "null info %d", i);
    int e = ocnn_info_check(infos[i]);
    if (e) return e;
    OCNN_REQUIRE(first->consistent_with(*as_info(infos[i])), OCNN_E_FORMAT,
        "The formats of input octrees are not consistent (octree %d)", i);
  }
  OCNN_REQUIRE(first->depth >= 1, OCNN_E_FORMAT, "depth %d", first->depth);
  OCNN_REQUIRE(first->channel(OCNN_KEY) <= 1, OCNN_E_UNSUPPORTED, "two-channel keys cannot be merged");
  Info o = *first;  // set_batch_info, merge_octrees.cpp:92-107
  o.set_batch_size(n);
  o.set_property(OCNN_NEIGH, 8, -1);
  for (int d = 0; d <= o.depth; ++d) {
    int64_t a = 0, b = 0;
    for (int i = 0; i < n; ++i) { a += as_info(infos[i])->nnum[d]; b += as_info(infos[i])->nnum_nempty[d]; }
    OCNN_REQUIRE(a < (1ll << 28), OCNN_E_BADARG, "merged level %d too large", d);
    o.nnum[d] = (int)a;
    o.nnum_nempty[d] = (int)b;
  }
  o.set_nnum_cum();
  OCNN_REQUIRE(o.set_ptr_dis(), OCNN_E_SHAPE,
      "the octree would exceed the 2 GiB that the 32-bit offsets of the serialized format can address");
  memcpy(out_info, &o, sizeof(Info));
  return OCNN_OK;
}

size_t ocnn_octree_batch_workspace_bytes(int n, int depth) {
  if (n < 1 || depth < 0 || depth > 16) return 0;
  return merge_layout(n, depth).total;
}

int ocnn_octree_batch(void* out_dev, const void* out_info, const void* const* octrees_dev,
    const void* const* infos, int n, void* workspace_dev, size_t workspace_bytes, ocnn_stream_t stream) {
  OCNN_REQUIRE(out_dev && out_info && octrees_dev && infos && n >= 1, OCNN_E_BADARG, "bad argument");
  const Info& o = *as_info(out_info);
  const int B = n, depth = o.depth, fl = o.full_layer;
  OCNN_REQUIRE(o.batch_size == B && o.has(OCNN_NEIGH), OCNN_E_BADARG, "out_info is not the batch header");
  MergeLayout L = merge_layout(B, depth);
  OCNN_REQUIRE(workspace_dev && workspace_bytes >= L.total, OCNN_E_WORKSPACE, "workspace %zu < %zu bytes",
      workspace_bytes, L.total);
  hipStream_t s = as_stream(stream);

  // host tables, laid out as in the workspace so that one copy carries them all
  std::vector<char> tables(L.total, 0);
  int* cum = reinterpret_cast<int*>(tables.data() + L.cum);
  int* cum_ne = reinterpret_cast<int*>(tables.data() + L.cum_ne);
  int64_t* src_off = reinterpret_cast<int64_t*>(tables.data() + L.src_off);
  const char** src = reinterpret_cast<const char**>(tables.data() + L.src);
  MergeSeg* segs = reinterpret_cast<MergeSeg*>(tables.data() + L.segs);
  const int props[kPCount] = {OCNN_KEY, OCNN_CHILD, OCNN_FEATURE, OCNN_LABEL, OCNN_SPLIT};
  for (int b = 0; b < B; ++b) {
    const Info* oi = as_info(infos[b]);
    OCNN_REQUIRE(octrees_dev[b], OCNN_E_BADARG, "null octree %d", b);
    src[b] = static_cast<const char*>(octrees_dev[b]);
    for (int d = 0; d <= depth; ++d) {
      cum[d * (B + 1) + b + 1] = cum[d * (B + 1) + b] + oi->nnum[d];
      cum_ne[d * (B + 1) + b + 1] = cum_ne[d * (B + 1) + b] + oi->nnum_nempty[d];
      for (int p = 0; p < kPCount; ++p) src_off[((size_t)p * B + b) * 17 + d] = oi->ptr_dis(props[p], d);
    }
  }
  for (int d = 0; d <= depth; ++d)
    OCNN_REQUIRE(cum[d * (B + 1) + B] == o.nnum[d], OCNN_E_BADARG, "out_info disagrees with the inputs at depth %d", d);

  // segments of the merge launch; what no segment and no neighbour kernel writes is cleared
  // (the reference starts from a zeroed buffer, merge_octrees.cpp:109-113)
  struct Span { int64_t at, bytes; };
  std::vector<Span> written;
  int n_seg = 0;
  unsigned blocks = 0;
  auto add_seg = [&](int kind, int d, int prop, int channel, int64_t dst_key, int64_t dst_child, int64_t count,
                     int64_t items) {
    if (items <= 0 || n_seg >= kMergeSegMax) return;
    MergeSeg& g = segs[n_seg++];
    g.kind = kind; g.depth = d; g.prop = prop; g.channel = channel;
    g.first_block = blocks; g.dst_key = dst_key; g.dst_child = dst_child; g.count = count;
    blocks += blocks_for(items);
  };
  add_seg(kMergeHeader, 0, 0, 0, 0, 0, 0, OCNN_HEADER_BYTES / 4);
  const int fprops[3] = {OCNN_FEATURE, OCNN_LABEL, OCNN_SPLIT};
  const int findex[3] = {kPFeature, kPLabel, kPSplit};
  for (int d = depth; d >= 0; --d) {  // the large levels first
    const int n_d = o.nnum[d];
    if (n_d == 0) continue;
    const int64_t k_off = o.has(OCNN_KEY) ? o.ptr_dis(OCNN_KEY, d) : -1;
    const int64_t c_off = o.has(OCNN_CHILD) ? o.ptr_dis(OCNN_CHILD, d) : -1;
    add_seg(kMergeKeyChild, d, 0, 0, k_off, c_off, n_d, n_d);
    if (k_off >= 0) written.push_back({k_off, (int64_t)n_d * 8});
    if (c_off >= 0) written.push_back({c_off, (int64_t)n_d * 4});
    for (int q = 0; q < 3; ++q) {
      if (!o.has(fprops[q])) continue;
      if (o.location(fprops[q]) == depth && d != depth) continue;
      const int ch = o.channel(fprops[q]);
      add_seg(kMergeFloat, d, findex[q], ch, o.ptr_dis(fprops[q], d), -1, n_d, n_d);
      written.push_back({o.ptr_dis(fprops[q], d), (int64_t)n_d * ch * 4});
    }
    if (d >= 1) written.push_back({o.ptr_dis(OCNN_NEIGH, d), (int64_t)n_d * 32});
  }
  std::sort(written.begin(), written.end(), [](const Span& x, const Span& y) { return x.at < y.at; });
  {
    int64_t at = OCNN_HEADER_BYTES;
    const int64_t blob_end = o.sizeof_octree();
    for (size_t i = 0; i <= written.size(); ++i) {
      const int64_t next = i < written.size() ? written[i].at : blob_end;
      if (next > at) add_seg(kMergeZero, 0, 0, 0, at, -1, (next - at) / 4, (next - at + 15) / 16);
      if (i < written.size()) at = std::max(at, written[i].at + written[i].bytes);
    }
  }
  OCNN_REQUIRE(n_seg < kMergeSegMax, OCNN_E_UNSUPPORTED, "too many segments to merge");
  char* ws = static_cast<char*>(workspace_dev);
  // The tables travel through a pinned staging buffer that is handed back when the stream has
  // passed the copy, so the call does not wait for the device.
  Staging* stage = take_staging(L.total);
  OCNN_REQUIRE(stage, OCNN_E_HIP, "no pinned host memory for the merge tables");
  memcpy(stage->host, tables.data(), L.total);
  hipError_t ce = hipMemcpyAsync(ws, stage->host, L.total, hipMemcpyHostToDevice, s);
  if (ce == hipSuccess) ce = hipEventRecord(stage->done, s);
  if (ce != hipSuccess) {
    (void)hipStreamSynchronize(s);
    stage->busy = false;
    return fail(OCNN_E_HIP, "merge tables: %s", hipGetErrorString(ce));
  }
  MergeTable m;
  m.cum = reinterpret_cast<const int*>(ws + L.cum);
  m.cum_ne = reinterpret_cast<const int*>(ws + L.cum_ne);
  m.src_off = reinterpret_cast<const int64_t*>(ws + L.src_off);
  m.src = reinterpret_cast<const char* const*>(ws + L.src);
  m.B = B;

  char* blob = static_cast<char*>(out_dev);
  HeaderArg h;
  memset(&h, 0, sizeof(h));
  memcpy(&h, &o, sizeof(Info));
  merge_kernel<<<blocks, kBlock, 0, s>>>(blob, m, reinterpret_cast<const MergeSeg*>(ws + L.segs), n_seg, h);
  OCNN_LAUNCH_OK("merge");
  int e = OCNN_OK;
  OCNN_REQUIRE(o.has(OCNN_CHILD), OCNN_E_FORMAT, "octrees without child links cannot get neighbour tables");
  for (int d = 1; d <= depth;) {
    int* neigh = reinterpret_cast<int*>(blob + o.ptr_dis(OCNN_NEIGH, d));
    if (d <= fl) {
      e = ocnn_calc_neigh_full(neigh, d, B, stream);
      if (e) return e;
      ++d;
      continue;
    }
    if (o.nnum[d - 1] <= 0) { ++d; continue; }
    // the last levels in one launch, their rows handed down in registers (levels of up to two
    // million nodes: beyond that a launch per level is as fast)
    int count = 1;
    if (depth - d < kNeighLevels && o.nnum[depth] <= (1 << 21)) while (d + count <= depth && o.nnum[d + count - 1] > 0) ++count;
    int* tables[kNeighLevels] = {nullptr, nullptr, nullptr};
    const int* links[kNeighLevels] = {nullptr, nullptr, nullptr};
    for (int i = 0; i < count; ++i) {
      tables[i] = reinterpret_cast<int*>(blob + o.ptr_dis(OCNN_NEIGH, d + i));
      links[i] = reinterpret_cast<const int*>(blob + o.ptr_dis(OCNN_CHILD, d + i - 1));
    }
    launch_neigh_sparse_levels(count, tables, reinterpret_cast<const int*>(blob + o.ptr_dis(OCNN_NEIGH, d - 1)), links,
        o.nnum[d - 1], s);
    OCNN_LAUNCH_OK("calc_neigh_sparse");
    d += count;
  }
  return OCNN_OK;
}

// ---- octree_new / octree_grow / octree_update -------------------------------------------
int ocnn_octree_new_info(int batch_size, int channel, int node_dis, int adaptive_layer, void* out_info) {
  OCNN_REQUIRE(out_info && batch_size >= 1 && channel >= 0, OCNN_E_BADARG, "bad argument");
  Info o;  // pytorch/cpp/octree_grow.cpp:110-140
  o.reset();
  o.set_batch_size(batch_size);
  o.set_depth(0);
  o.set_full_layer(0);
  o.has_node_dis = node_dis ? 1 : 0;
  if (adaptive_layer > 1) { o.is_adaptive = 1; o.adp_layer = adaptive_layer; }
  o.key2xyz = 1;
  o.set_property(OCNN_KEY, 1, -1);
  o.set_property(OCNN_CHILD, 1, -1);
  o.set_property(OCNN_NEIGH, 8, -1);
  o.set_property(OCNN_FEATURE, channel, -1);
  for (int i = 0; i < 3; ++i) { o.bbmin[i] = 0.0f; o.bbmax[i] = 2.0f; }
  o.nnum[0] = batch_size;
  o.set_nnum_cum();
  o.nnum_nempty[0] = batch_size;
  OCNN_REQUIRE(o.set_ptr_dis(), OCNN_E_SHAPE,
      "the octree would exceed the 2 GiB that the 32-bit offsets of the serialized format can address");
  memcpy(out_info, &o, sizeof(Info));
  return OCNN_OK;
}

int ocnn_octree_new(void* out_dev, const void* out_info, ocnn_stream_t stream) {
  OCNN_REQUIRE(out_dev && out_info, OCNN_E_BADARG, "null pointer");
  const Info& o = *as_info(out_info);
  hipStream_t s = as_stream(stream);
  char* blob = static_cast<char*>(out_dev);
  int e = zero_payload(blob, o, s);
  if (e) return e;
  e = write_header(blob, o, s);
  if (e) return e;
  int n = o.nnum[0];
  g_seq_key_child_kernel<<<blocks_for(n), kBlock, 0, s>>>(reinterpret_cast<uint64_t*>(blob + o.ptr_dis(OCNN_KEY, 0)),
      reinterpret_cast<int*>(blob + o.ptr_dis(OCNN_CHILD, 0)), n);
  OCNN_LAUNCH_OK("octree_new");
  return OCNN_OK;
}

int ocnn_octree_grow_info(const void* in_info, int target_depth, int full_octree, void* out_info) {
  OCNN_REQUIRE(in_info && out_info, OCNN_E_BADARG, "null pointer");
  const Info* oi = as_info(in_info);
  OCNN_REQUIRE(target_depth >= 1 && target_depth <= 13, OCNN_E_BADARG, "target_depth %d", target_depth);
  OCNN_REQUIRE(target_depth == oi->depth + 1 || (oi->depth == 0 && oi->full_layer == 1 && target_depth == 1),
      OCNN_E_BADARG, "octree_grow adds depth %d to an octree of depth %d", target_depth, oi->depth);
  OCNN_REQUIRE(oi->has(OCNN_KEY) && oi->has(OCNN_CHILD) && oi->has(OCNN_NEIGH), OCNN_E_FORMAT,
      "octree_grow needs key, child and neigh properties");
  int64_t node_num = (int64_t)oi->nnum_nempty[target_depth - 1] << 3;
  OCNN_REQUIRE(node_num < (1ll << 28), OCNN_E_BADARG, "grown level too large");
  Info o = *oi;  // update_octreeinfo, octree_grow.cpp:57-73
  o.set_depth(target_depth);
  if (full_octree) o.set_full_layer(target_depth);
  float width = (float)(1 << target_depth);
  for (int i = 0; i < 3; ++i) { o.bbmin[i] = 0.0f; o.bbmax[i] = width; }
  o.nnum[target_depth] = (int)node_num;
  o.nnum_nempty[target_depth] = (int)node_num;
  o.set_nnum_cum();
  OCNN_REQUIRE(o.set_ptr_dis(), OCNN_E_SHAPE,
      "the octree would exceed the 2 GiB that the 32-bit offsets of the serialized format can address");
  memcpy(out_info, &o, sizeof(Info));
  return OCNN_OK;
}

int ocnn_octree_grow(void* out_dev, const void* out_info, const void* in_dev, const void* in_info,
    int target_depth, int full_octree, ocnn_stream_t stream) {
  OCNN_REQUIRE(out_dev && out_info && in_dev && in_info, OCNN_E_BADARG, "null pointer");
  Info check;
  int e = ocnn_octree_grow_info(in_info, target_depth, full_octree, &check);
  if (e) return e;
  OCNN_REQUIRE(memcmp(&check, out_info, sizeof(Info)) == 0, OCNN_E_BADARG, "out_info is not the grown header");
  const Info& o = *as_info(out_info);
  const Info& oi = *as_info(in_info);
  hipStream_t s = as_stream(stream);
  char* blob = static_cast<char*>(out_dev);
  const char* in = static_cast<const char*>(in_dev);
  // copy_octree_gpu, octree_grow.cpp:75-87: everything below the new depth is copied, the
  // rest of the payload starts as zeros (the reference allocates the blob with torch::zeros)
  const int64_t ncum = oi.nnum_cum[target_depth];
  const int node_num = o.nnum[target_depth];
  const int64_t key_new = o.ptr_dis(OCNN_KEY, target_depth);
  const int64_t child_new = o.ptr_dis(OCNN_CHILD, target_depth);
  const int64_t neigh_new = o.ptr_dis(OCNN_NEIGH, target_depth);
  struct Span { int64_t at, bytes; };
  std::vector<Span> written;  // payload bytes that some rule or a later kernel writes
  GrowRanges g;
  memset(&g.plan, 0, sizeof(g.plan));
  if (!full_octree && o.nnum[target_depth - 1] > 0) {   // first: its wavefronts wait longest
    const int64_t groups = ((int64_t)o.nnum[target_depth - 1] + 7) / 8;
    g.add(kGrowNeigh, neigh_new, 0, (int64_t)blocks_for((groups + 1) / 2, kBlock / 64) * kGrowWordsPerBlock);
    g.plan.parent_neigh = oi.ptr_dis(OCNN_NEIGH, target_depth - 1);
    g.plan.parent_child = oi.ptr_dis(OCNN_CHILD, target_depth - 1);
    g.plan.parent_nodes = o.nnum[target_depth - 1];
    g.plan.new_groups = node_num / 8;
  }
  g.add(kGrowHeader, 0, 0, OCNN_HEADER_BYTES / 4);
  const int props[4] = {OCNN_KEY, OCNN_CHILD, OCNN_NEIGH, OCNN_FEATURE};
  const int elem[4] = {8, 4, 4, 4};
  for (int i = 0; i < 4; ++i) {
    if (!oi.has(props[i])) continue;
    int64_t bytes = ncum * oi.channel(props[i]) * elem[i];
    g.add(kGrowCopy, o.ptr_dis(props[i], 0), oi.ptr_dis(props[i], 0), bytes / 4);
    written.push_back({o.ptr_dis(props[i], 0), bytes});
  }
  written.push_back({key_new, (int64_t)node_num * 8});
  written.push_back({child_new, (int64_t)node_num * 4});
  written.push_back({neigh_new, (int64_t)node_num * 32});
  std::sort(written.begin(), written.end(), [](const Span& x, const Span& y) { return x.at < y.at; });
  int64_t at = OCNN_HEADER_BYTES;
  const int64_t blob_end = o.sizeof_octree();
  for (size_t i = 0; i <= written.size(); ++i) {
    int64_t next = i < written.size() ? written[i].at : blob_end;
    if (next > at) g.add(kGrowZero, at, 0, (next - at) / 4);
    if (i < written.size()) at = std::max(at, written[i].at + written[i].bytes);
  }
  g.add(kGrowSequence, child_new, 0, node_num);
  if (!full_octree) {
    g.add(kGrowKeyChild, key_new, 0, (int64_t)o.nnum[target_depth - 1] << 3);
    g.plan.parent_key = oi.ptr_dis(OCNN_KEY, target_depth - 1);
    g.plan.parent_child = oi.ptr_dis(OCNN_CHILD, target_depth - 1);
  }
  HeaderArg h;
  memset(&h, 0, sizeof(h));
  memcpy(&h, &o, sizeof(Info));
  unsigned blocks = g.finish();
  g_grow_kernel<<<blocks, kBlock, 0, s>>>(blob, in, g.plan, h);
  OCNN_LAUNCH_OK("octree_grow");
  // the new level's neighbours (and, for a full level, its keys) come from the old blob's tables
  int* neigh = reinterpret_cast<int*>(blob + neigh_new);
  if (full_octree) {
    e = ocnn_calc_neigh_full(neigh, target_depth, o.batch_size, stream);
    if (e) return e;
    e = ocnn_generate_key_full(reinterpret_cast<uint64_t*>(blob + key_new), target_depth, o.batch_size, stream);
    if (e) return e;
  }
  return OCNN_OK;
}

// pinned words for counts that a call waits for; kept for the life of the process
struct UpdateSlot { int count; int seq; };
static std::mutex g_pinned_mutex;
static std::vector<UpdateSlot*> g_pinned_free;
static std::atomic<int> g_update_seq{1};
static UpdateSlot* take_slot() {
  {
    std::lock_guard<std::mutex> lock(g_pinned_mutex);
    if (!g_pinned_free.empty()) { UpdateSlot* p = g_pinned_free.back(); g_pinned_free.pop_back(); return p; }
  }
  void* p = nullptr;
  if (hipHostMalloc(&p, 64, hipHostMallocCoherent) != hipSuccess) return nullptr;
  memset(p, 0, 64);
  return static_cast<UpdateSlot*>(p);
}
static void give_slot(UpdateSlot* p) {
  std::lock_guard<std::mutex> lock(g_pinned_mutex);
  g_pinned_free.push_back(p);
}

// Scan of the tile counts (one workgroup, as scan_tiles_kernel) that also settles the split count:
// nothing splits -> one node is kept (octree_grow.cpp:180-185; result[1] says so).  The count goes
// to the device words and, `seq` last, to the pinned host slot that the caller polls: the launches
// behind this one (the ranks, the copy of the blob) then run while the host already sizes the next
// level.
static __global__ void g_update_tiles_kernel(int* __restrict__ tile_count, int n_tiles, int* __restrict__ result,
    UpdateSlot* __restrict__ host, int seq) {
  __shared__ int carry;
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  for (int start = 0; start < n_tiles; start += kBlock) {
    const int i = start + threadIdx.x;
    const int v = i < n_tiles ? tile_count[i] : 0;
    int total;
    const int ex = block_exclusive_scan(v, &total);
    const int c = carry;
    if (i < n_tiles) tile_count[i] = c + ex;
    __syncthreads();
    if (threadIdx.x == 0) carry = c + total;
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    const int none = carry == 0 ? 1 : 0;
    const int count = none ? 1 : carry;
    result[0] = count;
    result[1] = none;
    __hip_atomic_store(&host->count, count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    __threadfence_system();
    __hip_atomic_store(&host->seq, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

// Workgroups 0 .. tiles-1: children[i] = rank among the labels equal to `split`, -1 for the others
// (generate_label, octree_nn.h:176-177).  Workgroups from `tiles` on: the words of the source blob
// outside the child array go to the result, the header word nnum_nempty[depth] replaced by the
// count; in place (`src` null) the first workgroup patches that word.
static __global__ void __launch_bounds__(kBlock) g_update_apply_kernel(uint32_t* __restrict__ dst, const uint32_t* __restrict__ src,
    const int* __restrict__ label, int split, int n, const int* __restrict__ tile_offset, const int* __restrict__ result,
    int tiles, int64_t child_word, int64_t count_word, int64_t blob_words) {
  if ((int)blockIdx.x < tiles) {
    int* children = reinterpret_cast<int*>(dst + child_word);
    const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
    bool f[kScanItems];
    int c = 0;
#pragma unroll
    for (int j = 0; j < kScanItems; ++j) {
      f[j] = base + j < n && label[base + j] == split;
      c += f[j] ? 1 : 0;
    }
    int total;
    int rank = tile_offset[blockIdx.x] + block_exclusive_scan(c, &total);
    const bool none = result[1] != 0;
#pragma unroll
    for (int j = 0; j < kScanItems; ++j) {
      if (base + j < n) children[base + j] = f[j] ? rank : ((none && base + j == 0) ? 0 : -1);
      rank += f[j] ? 1 : 0;
    }
    if (!src && blockIdx.x == 0 && threadIdx.x == 0) dst[count_word] = (uint32_t)result[0];
    return;
  }
  // four words a thread; a piece that touches the child array or lies at the end goes word by word
  const int64_t w0 = ((int64_t)(blockIdx.x - tiles) * kBlock + threadIdx.x) * 4;
  if (w0 >= blob_words) return;
  const uint32_t count = (uint32_t)result[0];
  if (w0 + 4 <= blob_words && (w0 + 4 <= child_word || w0 >= child_word + n)) {
    uint4 v = *reinterpret_cast<const uint4*>(src + w0);
    if (count_word >= w0 && count_word < w0 + 4) (&v.x)[count_word - w0] = count;
    *reinterpret_cast<uint4*>(dst + w0) = v;
    return;
  }
  for (int64_t w = w0; w < w0 + 4 && w < blob_words; ++w)
    if (w < child_word || w >= child_word + n) dst[w] = w == count_word ? count : src[w];
}

// children[depth] from the labels into `out` (the rest of `in` copied along when `in` is given),
// the split count to *split_num
static int update_impl(char* out, const char* in, const Info& o, const int* label, int n_label, int depth, int split,
    void* scratch_dev, size_t scratch_bytes, hipStream_t s, int* split_num) {
  const size_t need = scan_scratch_bytes(n_label) + 256;
  OCNN_REQUIRE(scratch_dev && scratch_bytes >= need, OCNN_E_WORKSPACE, "scratch %zu < %zu bytes", scratch_bytes, need);
  OCNN_REQUIRE((reinterpret_cast<uintptr_t>(out) & 15) == 0 && (reinterpret_cast<uintptr_t>(in) & 15) == 0, OCNN_E_BADARG,
      "octree blobs must be 16-byte aligned");
  int* result = reinterpret_cast<int*>(scratch_dev);
  int* tile_count = reinterpret_cast<int*>(static_cast<char*>(scratch_dev) + 256);
  int tiles = scan_tiles(n_label);
  if (tiles == 0) tiles = 1;
  UpdateSlot* slot = take_slot();
  OCNN_REQUIRE(slot, OCNN_E_HIP, "no pinned host memory for the split count");
  const int seq = g_update_seq.fetch_add(1) & 0x3fffffff;
  SplitPred pred{label, split};
  scan_count_kernel<SplitPred><<<tiles, kBlock, 0, s>>>(pred, n_label, tile_count);
  g_update_tiles_kernel<<<1, kBlock, 0, s>>>(tile_count, tiles, result, slot, seq);
  const int64_t blob_words = o.sizeof_octree() / 4;
  const unsigned copy_blocks = in ? blocks_for(blob_words, kBlock * 4) : 0;
  g_update_apply_kernel<<<tiles + copy_blocks, kBlock, 0, s>>>(reinterpret_cast<uint32_t*>(out),
      reinterpret_cast<const uint32_t*>(in), label, split, n_label, tile_count, result, tiles,
      o.ptr_dis(OCNN_CHILD, depth) / 4, (int64_t)(offsetof(Info, nnum_nempty) / 4) + depth, blob_words);
  if (hipGetLastError() != hipSuccess) { give_slot(slot); return fail(OCNN_E_HIP, "launch of octree_update failed"); }
  // the count is a few microseconds away; after 20 ms of polling the stream is asked (which also
  // reports a launch that failed)
  const auto t0 = std::chrono::steady_clock::now();
  bool seen = false;
  for (int spins = 0;; ++spins) {
    if (__atomic_load_n(&slot->seq, __ATOMIC_ACQUIRE) == seq) { seen = true; break; }
    if ((spins & 1023) == 1023 && std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(20)) break;
  }
  if (!seen) {
    const hipError_t err = hipStreamSynchronize(s);
    seen = err == hipSuccess && __atomic_load_n(&slot->seq, __ATOMIC_ACQUIRE) == seq;
    if (!seen) { give_slot(slot); return fail(OCNN_E_HIP, "split count: %s", hipGetErrorString(err)); }
  }
  *split_num = slot->count;
  give_slot(slot);
  return OCNN_OK;
}

int ocnn_octree_update(void* octree_dev, void* info, const int* label, int n_label, int depth, int split,
    void* scratch_dev, size_t scratch_bytes, ocnn_stream_t stream) {
  OCNN_REQUIRE(octree_dev && info && label, OCNN_E_BADARG, "null pointer");
  Info* o = static_cast<Info*>(info);
  OCNN_REQUIRE(depth >= 0 && depth <= o->depth, OCNN_E_BADARG, "depth %d", depth);
  OCNN_REQUIRE(n_label == o->nnum[depth], OCNN_E_SHAPE, "label has %d entries, depth %d has %d nodes", n_label,
      depth, o->nnum[depth]);
  int split_num = 0;
  const int e = update_impl(static_cast<char*>(octree_dev), nullptr, *o, label, n_label, depth, split, scratch_dev,
      scratch_bytes, as_stream(stream), &split_num);
  if (e) return e;
  o->nnum_nempty[depth] = split_num;
  return OCNN_OK;
}

int ocnn_octree_update_copy(void* out_dev, const void* in_dev, void* info, const int* label, int n_label, int depth,
    int split, void* scratch_dev, size_t scratch_bytes, ocnn_stream_t stream) {
  OCNN_REQUIRE(out_dev && in_dev && info && label, OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(out_dev != in_dev, OCNN_E_BADARG, "ocnn_octree_update_copy writes a second blob: use ocnn_octree_update in place");
  Info* o = static_cast<Info*>(info);
  OCNN_REQUIRE(depth >= 0 && depth <= o->depth, OCNN_E_BADARG, "depth %d", depth);
  OCNN_REQUIRE(n_label == o->nnum[depth], OCNN_E_SHAPE, "label has %d entries, depth %d has %d nodes", n_label,
      depth, o->nnum[depth]);
  int split_num = 0;
  const int e = update_impl(static_cast<char*>(out_dev), static_cast<const char*>(in_dev), *o, label, n_label, depth,
      split, scratch_dev, scratch_bytes, as_stream(stream), &split_num);
  if (e) return e;
  o->nnum_nempty[depth] = split_num;
  return OCNN_OK;
}

size_t ocnn_octree_update_scratch_bytes(int n_label) {
  return scan_scratch_bytes(n_label < 0 ? 0 : n_label) + 256;
}

}  // extern "C"
