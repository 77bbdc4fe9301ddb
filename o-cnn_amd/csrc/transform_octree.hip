// octree_scan on the device: ScanOctree (octree/octree/transform_octree.cpp:11-297) driven
// as pytorch/cpp/transform_octree.cpp:5-22 does.  The octree is looked at from a number of
// directions; a finest-level node survives iff it is non-empty, faces one of the views and
// is the nearest node of its pixel in that view's z-buffer; the levels above keep what has a
// surviving child, and the octree is rebuilt from the survivors.
//
// The reference fills the z-buffer node by node ("nearer than the current one wins"), i.e.
// every pixel ends with its nearest node, the first of equals.  Here that is one 64-bit
// atomic minimum per node over (depth as an ordered integer, node index).  The view frame is
// computed on the host with the reference's operations (libm included); everything after
// the buffer is integer work: flags bottom-up, ranks by prefix scans, a gather per level.
#include "octree_kernels.h"

#include <cfloat>
#include <cmath>
#include <vector>

namespace ocnn {
namespace {

constexpr int kMaxD = 17;

struct ViewFrame {
  float x[3], y[3], z[3], bbmin[3];
  int width;
};

inline float dot3(const float* a, const float* b) { return a[0] * b[0] + a[1] * b[1] + a[2] * b[2]; }

// set_axis + bbox_xy (transform_octree.cpp:13-92, math_functions.cpp:130-208)
ViewFrame view_frame(const float* z, int depth, float scale_) {
  ViewFrame f;
  const float z0[3] = {0, 0, 1};
  float angle = dot3(z0, z);
  if (angle < -1) angle = -1;
  if (angle > 1) angle = 1;
  angle = (float)acos((double)angle);
  float axis[3];
  axis[0] = z0[1] * z[2] - z0[2] * z[1];
  axis[1] = z0[2] * z[0] - z0[0] * z[2];
  axis[2] = z0[0] * z[1] - z0[1] * z[0];
  float len = 0.0f;
  for (int i = 0; i < 3; ++i) len += axis[i] * axis[i];
  len = sqrtf(len);
  const float ilen = (float)(1.0 / ((double)len + 1.0e-10));
  for (int i = 0; i < 3; ++i) axis[i] *= ilen;
  const float cosa = (float)cos((double)angle), cosa1 = 1 - cosa, sina = (float)sin((double)angle);
  float rot[9];
  rot[0] = cosa + axis[0] * axis[0] * cosa1;
  rot[1] = axis[0] * axis[1] * cosa1 + axis[2] * sina;
  rot[2] = axis[0] * axis[2] * cosa1 - axis[1] * sina;
  rot[3] = axis[0] * axis[1] * cosa1 - axis[2] * sina;
  rot[4] = cosa + axis[1] * axis[1] * cosa1;
  rot[5] = axis[1] * axis[2] * cosa1 + axis[0] * sina;
  for (int i = 0; i < 3; ++i) { f.x[i] = rot[i]; f.y[i] = rot[3 + i]; f.z[i] = z[i]; }
  float bbmax[3];
  for (int i = 0; i < 3; ++i) { f.bbmin[i] = FLT_MAX; bbmax[i] = -FLT_MAX; }
  for (int i = 0; i < 8; ++i) {
    const float pt[3] = {float(i / 4), float((i / 2) % 2), float(i % 2)};
    const float v[3] = {dot3(pt, f.x), dot3(pt, f.y), dot3(pt, f.z)};
    for (int c = 0; c < 3; ++c) {
      if (v[c] < f.bbmin[c]) f.bbmin[c] = v[c];
      if (v[c] > bbmax[c]) bbmax[c] = v[c];
    }
  }
  float width = -1;
  const float scale = (float)(1 << depth);
  for (int i = 0; i < 3; ++i) {
    bbmax[i] *= scale;
    f.bbmin[i] *= scale;
    const float dis = bbmax[i] - f.bbmin[i];
    if (dis > width) width = dis;
  }
  f.width = static_cast<int>(width * scale_) + 2;
  return f;
}

__global__ void fill_u64_kernel(unsigned long long* __restrict__ p, int64_t n, unsigned long long v) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}
__global__ void fill_i32_kernel(int* __restrict__ p, int64_t n, int v) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

__device__ inline float ddot(const float* a, float b0, float b1, float b2) {
  return __fadd_rn(__fadd_rn(__fmul_rn(a[0], b0), __fmul_rn(a[1], b1)), __fmul_rn(a[2], b2));
}

// z_buffer (transform_octree.cpp:99-138): nearest node per pixel, the first one among equals
__global__ void zbuffer_kernel(unsigned long long* __restrict__ buf, const uint64_t* __restrict__ key,
    const int* __restrict__ child, const float* __restrict__ normal /* channel-major rows of num, or null */,
    int num, int depth, int key2xyz, ViewFrame f, float scale_) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= num || child[i] < 0) return;
  float n0 = 0.0f, n1 = 0.0f, n2 = 0.0f;
  if (normal) { n0 = normal[i]; n1 = normal[(int64_t)num + i]; n2 = normal[2 * (int64_t)num + i]; }
  // dot_prod(normal, z_) >= 0: invisible
  if (__fadd_rn(__fadd_rn(__fmul_rn(n0, f.z[0]), __fmul_rn(n1, f.z[1])), __fmul_rn(n2, f.z[2])) >= 0) return;
  float p0, p1, p2;
  const uint64_t k = key[i];
  if (key2xyz) {
    p0 = (float)(k & 0xffff); p1 = (float)((k >> 16) & 0xffff); p2 = (float)((k >> 32) & 0xffff);
  } else {
    uint32_t x, y, z;
    morton_decode(k, depth, &x, &y, &z);
    p0 = (float)x; p1 = (float)y; p2 = (float)z;
  }
  const float x = __fmul_rn(__fsub_rn(ddot(f.x, p0, p1, p2), f.bbmin[0]), scale_);
  const float y = __fmul_rn(__fsub_rn(ddot(f.y, p0, p1, p2), f.bbmin[1]), scale_);
  const float z = ddot(f.z, p0, p1, p2);
  const int64_t pix = (int64_t)static_cast<int>(__fadd_rn(x, 0.5f)) * f.width + static_cast<int>(__fadd_rn(y, 0.5f));
  if (pix < 0 || pix >= (int64_t)f.width * f.width) return;   // cannot happen: the grid covers the cube
  uint32_t u = __float_as_uint(z);
  u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);             // float order -> unsigned order
  atomicMin(&buf[pix], ((unsigned long long)u << 32) | (unsigned long long)(unsigned)i);
}
__global__ void zbuffer_mark_kernel(int* __restrict__ drop, const unsigned long long* __restrict__ buf, int64_t pixels) {
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= pixels) return;
  const unsigned long long v = buf[p];
  if (v != ~0ull) drop[(unsigned)(v & 0xffffffffull)] = 0;
}
// generate_flags (transform_octree.cpp:140-170): a node is kept iff one of its children is
__global__ void parent_flag_kernel(int* __restrict__ drop, const int* __restrict__ drop_c, const int* __restrict__ child,
    int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int j = child[i];
  int dr = 1;
  if (j >= 0)
    for (int k = 0; k < 8; ++k) dr = drop_c[j * 8 + k] == 0 ? 0 : dr;
  drop[i] = dr;
}

struct KeptPred {
  const int* drop;
  __device__ bool operator()(int64_t i) const { return drop[i] == 0; }
};
struct KeptOut {
  int* rank;
  __device__ void operator()(int64_t i, bool, int r) const { rank[i] = r; }
};

// trim_octree (transform_octree.cpp:172-297): the children of every kept node of level d-1
struct TrimArgs {
  int n_parent, n_in, n_out, fch, has_label, has_split;
  const int *drop_p, *rank_p;      // level d-1 (null: every node kept, rank = index)
  const int *drop_d, *rank_d;      // level d
  const int* child_p;
  const uint64_t* key_in; const float *f_in, *l_in, *s_in;
  uint64_t* key_out; int* child_out; float *f_out, *l_out, *s_out;
};
__global__ void trim_kernel(TrimArgs a) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  const int i = t >> 3, o = t & 7;
  if (i >= a.n_parent) return;
  if (a.drop_p && a.drop_p[i] != 0) return;
  const int c = a.child_p[i];
  if (c < 0) return;
  const int64_t k = (int64_t)c * 8 + o, j = (int64_t)(a.rank_p ? a.rank_p[i] : i) * 8 + o;
  const bool kept = a.drop_d[k] == 0;
  a.key_out[j] = a.key_in[k];
  a.child_out[j] = kept ? a.rank_d[k] : -1;
  if (a.f_out)
    for (int ch = 0; ch < a.fch; ++ch) a.f_out[(int64_t)ch * a.n_out + j] = kept ? a.f_in[(int64_t)ch * a.n_in + k] : 0.0f;
  if (a.l_out) a.l_out[j] = kept ? a.l_in[k] : -1.0f;
  if (a.s_out) a.s_out[j] = kept ? a.s_in[k] : 0.0f;
}
__global__ void copy_words_kernel(uint32_t* __restrict__ dst, const uint32_t* __restrict__ src, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

inline size_t al(size_t v) { return (v + 255) & ~(size_t)255; }

// ---- octree_dropout (octree/octree/transform_octree.cpp:286-431)
__global__ void drop_flags_kernel(int* __restrict__ drop, const unsigned char* __restrict__ flags, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) drop[i] = flags[i] != 0;
}
// a dropped node takes its children along (:301-314)
__global__ void drop_children_kernel(int* __restrict__ drop_c, const int* __restrict__ drop_p,
    const int* __restrict__ child_p, int n_parent) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  const int i = t >> 3;
  if (i >= n_parent) return;
  const int c = child_p[i];
  if (c >= 0) drop_c[(int64_t)c * 8 + (t & 7)] = drop_p[i];
}
struct LivePred {   // kept and non-empty: the nodes whose children are renumbered
  const int* drop; const int* child;
  __device__ bool operator()(int64_t i) const { return drop[i] == 0 && child[i] >= 0; }
};
// the kept nodes of one level below the dropout level, compacted (:365-416)
struct DropArgs {
  int n_in, n_out, fch;
  const int *drop, *rank, *live_rank, *child_in;
  const uint64_t* key_in; const float *f_in, *l_in, *s_in;
  uint64_t* key_out; int* child_out; float *f_out, *l_out, *s_out;
};
__global__ void drop_gather_kernel(DropArgs a) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= a.n_in || a.drop[i] != 0) return;
  const int j = a.rank[i];
  a.key_out[j] = a.key_in[i];
  const int c = a.child_in[i];
  a.child_out[j] = c < 0 ? c : a.live_rank[i];
  if (a.f_out)
    for (int ch = 0; ch < a.fch; ++ch) a.f_out[(int64_t)ch * a.n_out + j] = a.f_in[(int64_t)ch * a.n_in + i];
  if (a.l_out) a.l_out[j] = a.l_in[i];
  if (a.s_out) a.s_out[j] = a.s_in[i];
}
// the dropout level itself (:419-425): a dropped node keeps its old child entry
__global__ void drop_level_children_kernel(int* __restrict__ child_out, const int* __restrict__ child_in,
    const int* __restrict__ drop, const int* __restrict__ live_rank, int n, int clear_dropped) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int c = child_in[i];
  child_out[i] = (drop[i] != 0 || c < 0) ? (clear_dropped ? -1 : c) : live_rank[i];
}
__global__ void copy_words64_kernel(uint32_t* __restrict__ dst, const uint32_t* __restrict__ src, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

}  // namespace
}  // namespace ocnn

using namespace ocnn;

extern "C" int ocnn_octree_scan(const void* octree_dev, const void* info, const float* axis, int n_axis, float scale,
    ocnn_alloc_fn alloc, void* alloc_ctx, void* info_out, void** octree_out_dev, ocnn_stream_t stream) {
  OCNN_REQUIRE(octree_dev && info && axis && alloc && info_out && octree_out_dev, OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(n_axis >= 1 && scale > 0.0f, OCNN_E_BADARG, "n_axis %d scale %g", n_axis, (double)scale);
  const Info& oi = *as_info(info);
  OCNN_REQUIRE(oi.batch_size == 1 && oi.channel(OCNN_KEY) == 1 && !oi.has(OCNN_NEIGH), OCNN_E_UNSUPPORTED,
      "octree_scan takes a single octree with one-channel keys (scan first, batch afterwards)");
  const int D = oi.depth, fl = oi.full_layer;
  OCNN_REQUIRE(D >= 1 && D <= 16 && fl >= 1 && fl <= D, OCNN_E_FORMAT, "depth %d full_depth %d", D, fl);
  hipStream_t s = as_stream(stream);
  const char* in = static_cast<const char*>(octree_dev);

  // ---- view frames (host) and scratch
  std::vector<ViewFrame> frames(n_axis);
  int64_t max_pix = 1;
  for (int a = 0; a < n_axis; ++a) {
    frames[a] = view_frame(axis + 3 * a, D, scale);
    OCNN_REQUIRE(frames[a].width >= 1 && frames[a].width <= 32768, OCNN_E_BADARG, "z-buffer of width %d", frames[a].width);
    const int64_t pix = (int64_t)frames[a].width * frames[a].width;
    if (pix > max_pix) max_pix = pix;
  }
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t v = off; off += al(bytes); return v; };
  size_t o_drop[kMaxD], o_rank[kMaxD];
  int max_n = 1;
  for (int d = 0; d <= D; ++d) {
    o_drop[d] = take(4 * ((size_t)oi.nnum[d] + 1));
    o_rank[d] = take(4 * ((size_t)oi.nnum[d] + 1));
    if (oi.nnum[d] > max_n) max_n = oi.nnum[d];
  }
  const size_t o_buf = take(8 * (size_t)max_pix);
  const size_t o_scan = take(scan_scratch_bytes(max_n));
  const size_t o_counts = take(sizeof(int) * 32);
  const size_t o_hdr = take(OCNN_HEADER_BYTES);
  char* ws = static_cast<char*>(alloc(off, alloc_ctx));
  OCNN_REQUIRE(ws, OCNN_E_BADARG, "the allocator returned no memory for %zu bytes of scratch", off);
  OCNN_REQUIRE((reinterpret_cast<uintptr_t>(ws) & 7) == 0, OCNN_E_BADARG, "scratch not 8-byte aligned");
  int *drop[kMaxD], *rank[kMaxD];
  for (int d = 0; d <= D; ++d) { drop[d] = reinterpret_cast<int*>(ws + o_drop[d]); rank[d] = reinterpret_cast<int*>(ws + o_rank[d]); }
  unsigned long long* buf = reinterpret_cast<unsigned long long*>(ws + o_buf);
  int* d_counts = reinterpret_cast<int*>(ws + o_counts);

  // ---- z-buffers over the finest level
  const int num = oi.nnum[D];
  const int fch = oi.channel(OCNN_FEATURE), floc = oi.location(OCNN_FEATURE);
  const float* normal = (fch >= 3 && (floc == -1 || floc == D))
      ? reinterpret_cast<const float*>(in + oi.ptr_dis(OCNN_FEATURE, D)) : nullptr;
  fill_i32_kernel<<<blocks_for(num), kBlock, 0, s>>>(drop[D], num, 1);
  for (int a = 0; a < n_axis; ++a) {
    const int64_t pix = (int64_t)frames[a].width * frames[a].width;
    fill_u64_kernel<<<blocks_for(pix), kBlock, 0, s>>>(buf, pix, ~0ull);
    zbuffer_kernel<<<blocks_for(num), kBlock, 0, s>>>(buf, reinterpret_cast<const uint64_t*>(in + oi.ptr_dis(OCNN_KEY, D)),
        reinterpret_cast<const int*>(in + oi.ptr_dis(OCNN_CHILD, D)), normal, num, D, oi.key2xyz, frames[a], scale);
    zbuffer_mark_kernel<<<blocks_for(pix), kBlock, 0, s>>>(drop[D], buf, pix);
  }
  OCNN_LAUNCH_OK("z-buffer");
  // ---- flags of the levels above, ranks of the survivors
  for (int d = D - 1; d >= fl; --d)
    parent_flag_kernel<<<blocks_for(oi.nnum[d]), kBlock, 0, s>>>(drop[d], drop[d + 1],
        reinterpret_cast<const int*>(in + oi.ptr_dis(OCNN_CHILD, d)), oi.nnum[d]);
  for (int d = fl; d <= D; ++d) {
    KeptPred kp{drop[d]};
    KeptOut ko{rank[d]};
    hipError_t e = flag_scan(kp, ko, (int64_t)oi.nnum[d], reinterpret_cast<int*>(ws + o_scan), d_counts + d, s);
    OCNN_REQUIRE(e == hipSuccess, OCNN_E_HIP, "scan: %s", hipGetErrorString(e));
  }
  int h[32];
  {
    const int e = fetch_words(h, d_counts, 32, s);
    if (e) return e;
  }

  Info o = oi;
  for (int d = 0; d <= D; ++d) o.nnum_nempty[d] = d < fl ? (1 << (3 * d)) : h[d];
  o.nnum[0] = 1;
  for (int d = 1; d <= D; ++d) o.nnum[d] = 8 * o.nnum_nempty[d - 1];
  o.set_nnum_cum();
  OCNN_REQUIRE(o.set_ptr_dis(), OCNN_E_SHAPE, "the octree would exceed 2 GiB");
  memcpy(info_out, &o, sizeof(Info));

  // ---- the new octree: zeros (level 0 stays so, as in the reference), header, a gather per level
  const size_t bytes = (size_t)o.sizeof_octree();
  char* out = static_cast<char*>(alloc(bytes, alloc_ctx));
  OCNN_REQUIRE(out, OCNN_E_BADARG, "the allocator returned no memory for the octree");
  OCNN_REQUIRE((reinterpret_cast<uintptr_t>(out) & 7) == 0, OCNN_E_BADARG, "blob not 8-byte aligned");
  *octree_out_dev = out;
  fill_i32_kernel<<<blocks_for((int64_t)(bytes / 4)), kBlock, 0, s>>>(reinterpret_cast<int*>(out), (int64_t)(bytes / 4), 0);
  {
    uint32_t hdr[OCNN_HEADER_BYTES / 4];
    memset(hdr, 0, sizeof(hdr));
    memcpy(hdr, &o, sizeof(Info));
    OCNN_HIP_OK(hipMemcpyAsync(ws + o_hdr, hdr, sizeof(hdr), hipMemcpyHostToDevice, s));
    OCNN_HIP_OK(hipStreamSynchronize(s));   // `hdr` lives on this stack frame
    copy_words_kernel<<<1, kBlock, 0, s>>>(reinterpret_cast<uint32_t*>(out), reinterpret_cast<const uint32_t*>(ws + o_hdr),
        OCNN_HEADER_BYTES / 4);
  }
  const int lch = oi.channel(OCNN_LABEL), lloc = oi.location(OCNN_LABEL);
  const int sch = oi.channel(OCNN_SPLIT), sloc = oi.location(OCNN_SPLIT);
  for (int d = 1; d <= D; ++d) {
    TrimArgs a;
    memset(&a, 0, sizeof(a));
    a.n_parent = oi.nnum[d - 1]; a.n_in = oi.nnum[d]; a.n_out = o.nnum[d]; a.fch = fch;
    a.drop_p = d - 1 >= fl ? drop[d - 1] : nullptr;
    a.rank_p = d - 1 >= fl ? rank[d - 1] : nullptr;
    a.drop_d = drop[d]; a.rank_d = rank[d];
    if (d < fl) {   // full levels below the last one: every node kept, rank = index
      fill_i32_kernel<<<blocks_for(oi.nnum[d]), kBlock, 0, s>>>(drop[d], oi.nnum[d], 0);
      // rank[d][k] = k
      KeptPred kp{drop[d]};
      KeptOut ko{rank[d]};
      hipError_t e = flag_scan(kp, ko, (int64_t)oi.nnum[d], reinterpret_cast<int*>(ws + o_scan), d_counts + 20, s);
      OCNN_REQUIRE(e == hipSuccess, OCNN_E_HIP, "scan: %s", hipGetErrorString(e));
    }
    a.child_p = reinterpret_cast<const int*>(in + oi.ptr_dis(OCNN_CHILD, d - 1));
    a.key_in = reinterpret_cast<const uint64_t*>(in + oi.ptr_dis(OCNN_KEY, d));
    a.key_out = reinterpret_cast<uint64_t*>(out + o.ptr_dis(OCNN_KEY, d));
    a.child_out = reinterpret_cast<int*>(out + o.ptr_dis(OCNN_CHILD, d));
    if (fch && (floc == -1 || d == D)) {
      a.f_in = reinterpret_cast<const float*>(in + oi.ptr_dis(OCNN_FEATURE, d));
      a.f_out = reinterpret_cast<float*>(out + o.ptr_dis(OCNN_FEATURE, d));
    }
    if (lch && (lloc == -1 || d == D)) {
      a.l_in = reinterpret_cast<const float*>(in + oi.ptr_dis(OCNN_LABEL, d));
      a.l_out = reinterpret_cast<float*>(out + o.ptr_dis(OCNN_LABEL, d));
    }
    if (sch && (sloc == -1 || d == D)) {
      a.s_in = reinterpret_cast<const float*>(in + oi.ptr_dis(OCNN_SPLIT, d));
      a.s_out = reinterpret_cast<float*>(out + o.ptr_dis(OCNN_SPLIT, d));
    }
    if (a.n_parent > 0) trim_kernel<<<blocks_for((int64_t)a.n_parent * 8), kBlock, 0, s>>>(a);
  }
  OCNN_LAUNCH_OK("trim");
  return OCNN_OK;
}

extern "C" int ocnn_octree_dropout(const void* octree_dev, const void* info, const unsigned char* flags_dev,
    int depth_dropout, int clear_dropped, ocnn_alloc_fn alloc, void* alloc_ctx, void* info_out, void** octree_out_dev,
    ocnn_stream_t stream) {
  OCNN_REQUIRE(octree_dev && info && flags_dev && alloc && info_out && octree_out_dev, OCNN_E_BADARG, "null pointer");
  const Info& oi = *as_info(info);
  const int D = oi.depth, dd = depth_dropout;
  OCNN_REQUIRE(D >= 1 && D <= 16, OCNN_E_FORMAT, "depth %d", D);
  OCNN_REQUIRE(dd >= 0 && dd <= D, OCNN_E_BADARG, "depth_dropout %d outside [0, %d]", dd, D);
  OCNN_REQUIRE(oi.channel(OCNN_KEY) == 1, OCNN_E_UNSUPPORTED, "octree_dropout takes one-channel keys");
  hipStream_t s = as_stream(stream);
  const char* in = static_cast<const char*>(octree_dev);

  size_t off = 0;
  auto take = [&](size_t bytes) { size_t v = off; off += al(bytes); return v; };
  size_t o_drop[kMaxD], o_rank[kMaxD], o_live[kMaxD];
  int max_n = 1;
  for (int d = dd; d <= D; ++d) {
    o_drop[d] = take(4 * ((size_t)oi.nnum[d] + 1));
    o_rank[d] = take(4 * ((size_t)oi.nnum[d] + 1));
    o_live[d] = take(4 * ((size_t)oi.nnum[d] + 1));
    if (oi.nnum[d] > max_n) max_n = oi.nnum[d];
  }
  const size_t o_scan = take(scan_scratch_bytes(max_n));
  const size_t o_counts = take(sizeof(int) * 2 * kMaxD);
  const size_t o_hdr = take(OCNN_HEADER_BYTES);
  char* ws = static_cast<char*>(alloc(off, alloc_ctx));
  OCNN_REQUIRE(ws, OCNN_E_BADARG, "the allocator returned no memory for %zu bytes of scratch", off);
  OCNN_REQUIRE((reinterpret_cast<uintptr_t>(ws) & 7) == 0, OCNN_E_BADARG, "scratch not 8-byte aligned");
  auto drop = [&](int d) { return reinterpret_cast<int*>(ws + o_drop[d]); };
  auto rank = [&](int d) { return reinterpret_cast<int*>(ws + o_rank[d]); };
  auto live = [&](int d) { return reinterpret_cast<int*>(ws + o_live[d]); };
  auto child_in = [&](int d) { return reinterpret_cast<const int*>(in + oi.ptr_dis(OCNN_CHILD, d)); };
  int* d_counts = reinterpret_cast<int*>(ws + o_counts);   // [d]: kept nodes, [kMaxD + d]: kept non-empty nodes

  // ---- flags top-down, ranks of the kept nodes and of the kept non-empty nodes
  if (oi.nnum[dd] > 0) drop_flags_kernel<<<blocks_for(oi.nnum[dd]), kBlock, 0, s>>>(drop(dd), flags_dev, oi.nnum[dd]);
  for (int d = dd + 1; d <= D; ++d)
    if (oi.nnum[d - 1] > 0)
      drop_children_kernel<<<blocks_for((int64_t)oi.nnum[d - 1] * 8), kBlock, 0, s>>>(drop(d), drop(d - 1), child_in(d - 1),
          oi.nnum[d - 1]);
  for (int d = dd; d <= D; ++d) {
    hipError_t e = hipSuccess;
    if (d > dd) {
      KeptPred kp{drop(d)};
      KeptOut ko{rank(d)};
      e = flag_scan(kp, ko, (int64_t)oi.nnum[d], reinterpret_cast<int*>(ws + o_scan), d_counts + d, s);
      OCNN_REQUIRE(e == hipSuccess, OCNN_E_HIP, "scan: %s", hipGetErrorString(e));
    }
    LivePred lp{drop(d), child_in(d)};
    KeptOut lo{live(d)};
    e = flag_scan(lp, lo, (int64_t)oi.nnum[d], reinterpret_cast<int*>(ws + o_scan), d_counts + kMaxD + d, s);
    OCNN_REQUIRE(e == hipSuccess, OCNN_E_HIP, "scan: %s", hipGetErrorString(e));
  }
  int h[2 * kMaxD];
  {
    static_assert(2 * kMaxD <= kFetchWords, "counts of both scans in one fetch");
    const int e = fetch_words(h, d_counts, 2 * kMaxD, s);
    if (e) return e;
  }

  Info o = oi;
  for (int d = dd + 1; d <= D; ++d) o.nnum[d] = h[d];
  for (int d = dd; d <= D; ++d) o.nnum_nempty[d] = h[kMaxD + d];
  o.set_nnum_cum();
  OCNN_REQUIRE(o.set_ptr_dis(), OCNN_E_SHAPE, "the octree would exceed 2 GiB");
  memcpy(info_out, &o, sizeof(Info));

  // ---- the new octree: zeros, header, levels 0..depth_dropout as they are, a gather per level below
  const size_t bytes = (size_t)o.sizeof_octree();
  char* out = static_cast<char*>(alloc(bytes, alloc_ctx));
  OCNN_REQUIRE(out, OCNN_E_BADARG, "the allocator returned no memory for the octree");
  OCNN_REQUIRE((reinterpret_cast<uintptr_t>(out) & 7) == 0, OCNN_E_BADARG, "blob not 8-byte aligned");
  *octree_out_dev = out;
  fill_i32_kernel<<<blocks_for((int64_t)(bytes / 4)), kBlock, 0, s>>>(reinterpret_cast<int*>(out), (int64_t)(bytes / 4), 0);
  {
    uint32_t hdr[OCNN_HEADER_BYTES / 4];
    memset(hdr, 0, sizeof(hdr));
    memcpy(hdr, &o, sizeof(Info));
    OCNN_HIP_OK(hipMemcpyAsync(ws + o_hdr, hdr, sizeof(hdr), hipMemcpyHostToDevice, s));
    OCNN_HIP_OK(hipStreamSynchronize(s));   // `hdr` lives on this stack frame
    copy_words_kernel<<<1, kBlock, 0, s>>>(reinterpret_cast<uint32_t*>(out), reinterpret_cast<const uint32_t*>(ws + o_hdr),
        OCNN_HEADER_BYTES / 4);
  }
  const int fch = oi.channel(OCNN_FEATURE), floc = oi.location(OCNN_FEATURE);
  const int lch = oi.channel(OCNN_LABEL), lloc = oi.location(OCNN_LABEL);
  const int sch = oi.channel(OCNN_SPLIT), sloc = oi.location(OCNN_SPLIT);
  const int64_t num = oi.nnum_cum[dd + 1];
  auto copy_prefix = [&](int prop, int64_t words) {
    if (words > 0)
      copy_words64_kernel<<<blocks_for(words), kBlock, 0, s>>>(reinterpret_cast<uint32_t*>(out + o.ptr_dis(prop, 0)),
          reinterpret_cast<const uint32_t*>(in + oi.ptr_dis(prop, 0)), words);
  };
  copy_prefix(OCNN_KEY, 2 * num);
  copy_prefix(OCNN_CHILD, num);
  if (oi.has(OCNN_FEATURE) && floc == -1) copy_prefix(OCNN_FEATURE, num * fch);
  if (oi.has(OCNN_LABEL) && lloc == -1) copy_prefix(OCNN_LABEL, num * lch);
  if (oi.has(OCNN_SPLIT) && sloc == -1) copy_prefix(OCNN_SPLIT, num * sch);
  for (int d = dd + 1; d <= D; ++d) {
    if (oi.nnum[d] == 0) continue;
    DropArgs a;
    memset(&a, 0, sizeof(a));
    a.n_in = oi.nnum[d]; a.n_out = o.nnum[d]; a.fch = fch;
    a.drop = drop(d); a.rank = rank(d); a.live_rank = live(d); a.child_in = child_in(d);
    a.key_in = reinterpret_cast<const uint64_t*>(in + oi.ptr_dis(OCNN_KEY, d));
    a.key_out = reinterpret_cast<uint64_t*>(out + o.ptr_dis(OCNN_KEY, d));
    a.child_out = reinterpret_cast<int*>(out + o.ptr_dis(OCNN_CHILD, d));
    if (oi.has(OCNN_FEATURE) && fch && (floc == -1 || d == D)) {
      a.f_in = reinterpret_cast<const float*>(in + oi.ptr_dis(OCNN_FEATURE, d));
      a.f_out = reinterpret_cast<float*>(out + o.ptr_dis(OCNN_FEATURE, d));
    }
    if (lch && (lloc == -1 || d == D)) {
      a.l_in = reinterpret_cast<const float*>(in + oi.ptr_dis(OCNN_LABEL, d));
      a.l_out = reinterpret_cast<float*>(out + o.ptr_dis(OCNN_LABEL, d));
    }
    if (sch && (sloc == -1 || d == D)) {
      a.s_in = reinterpret_cast<const float*>(in + oi.ptr_dis(OCNN_SPLIT, d));
      a.s_out = reinterpret_cast<float*>(out + o.ptr_dis(OCNN_SPLIT, d));
    }
    drop_gather_kernel<<<blocks_for(a.n_in), kBlock, 0, s>>>(a);
  }
  if (oi.nnum[dd] > 0)
    drop_level_children_kernel<<<blocks_for(oi.nnum[dd]), kBlock, 0, s>>>(reinterpret_cast<int*>(out + o.ptr_dis(OCNN_CHILD, dd)),
        child_in(dd), drop(dd), live(dd), oi.nnum[dd], clear_dropped);
  OCNN_LAUNCH_OK("octree_dropout");
  return OCNN_OK;
}
