// Point-cloud transforms on the device: bounding sphere, normalisation, rotation / scale /
// jitter / normal orientation and clipping of a serialized point cloud.  Replaces the host
// loops of pytorch/cpp/transform_points.cpp:7-125 (PointsParser, octree/octree/
// points_parser.cpp:42-260) so that normalise -> transform -> clip -> points2octree runs
// without the cloud leaving the device.  Every floating-point operation is rounded
// individually in the reference's order (the file is compiled without contraction and
// square roots / quotients go through fp64), so results are bit-identical to the host path.
#include "ocnn_common.h"
#include "scan.h"

#include <cfloat>
#include <cmath>
#include <cstring>

namespace ocnn {
namespace {

__device__ inline float sqrt_rn(float x) { return (float)sqrt((double)x); }
__device__ inline float div_rn(float a, float b) { return (float)((double)a / (double)b); }

int check_points(const void* points_info, const PointsInfo** out) {
  OCNN_REQUIRE(points_info, OCNN_E_BADARG, "null points header");
  const PointsInfo* pi = static_cast<const PointsInfo*>(points_info);
  OCNN_REQUIRE(strcmp(pi->magic, "_POINTS_1.0_") == 0, OCNN_E_FORMAT, "not a _POINTS_1.0_ blob");
  OCNN_REQUIRE(pi->pt_num > 0, OCNN_E_FORMAT, "The pt_num_ should be larger than 0.");
  OCNN_REQUIRE(pi->content_flags & 1, OCNN_E_FORMAT, "the cloud holds no coordinates");
  *out = pi;
  return OCNN_OK;
}
inline size_t blob_bytes(const PointsInfo* pi) { return (size_t)pi->ptr_dis[4]; }

// ---- bounding box / bounding sphere --------------------------------------------------------
// Extremes per axis with the index of their FIRST occurrence (the host loop compares with
// strict < and >), as (value, point index) pairs: slot 2a = min of axis a, 2a+1 = max.
struct Extreme { float v[6]; int id[6]; };

__device__ inline void merge_extreme(Extreme& a, const Extreme& b) {
#pragma unroll
  for (int s = 0; s < 6; ++s) {
    const bool is_min = (s & 1) == 0;
    const bool better = is_min ? (b.v[s] < a.v[s]) : (b.v[s] > a.v[s]);
    if (better || (b.v[s] == a.v[s] && b.id[s] < a.id[s])) { a.v[s] = b.v[s]; a.id[s] = b.id[s]; }
  }
}

__global__ void extremes_kernel(Extreme* __restrict__ partial, const float* __restrict__ pt, int npt) {
  __shared__ Extreme sh[kBlock];
  Extreme e;
#pragma unroll
  for (int s = 0; s < 6; ++s) { e.v[s] = (s & 1) ? -FLT_MAX : FLT_MAX; e.id[s] = 0x7fffffff; }
  for (int i = blockIdx.x * kBlock + threadIdx.x; i < npt; i += gridDim.x * kBlock) {
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const float v = pt[3 * (int64_t)i + a];
      if (v < e.v[2 * a]) { e.v[2 * a] = v; e.id[2 * a] = i; }
      if (v > e.v[2 * a + 1]) { e.v[2 * a + 1] = v; e.id[2 * a + 1] = i; }
    }
  }
  sh[threadIdx.x] = e;
  __syncthreads();
  for (int step = kBlock / 2; step > 0; step >>= 1) {
    if (threadIdx.x < step) merge_extreme(sh[threadIdx.x], sh[threadIdx.x + step]);
    __syncthreads();
  }
  if (threadIdx.x == 0) partial[blockIdx.x] = sh[0];
}

// One workgroup finishes the sphere of math_functions.cpp:49-108 (the build without Miniball):
// the widest of the three extreme pairs gives the first sphere, then every point outside grows
// it, IN POINT ORDER.  The order is kept exactly: a chunk of points is tested in parallel
// against the current sphere, the first violating point updates it, and the rest of the chunk
// is tested again.
constexpr int kSphereThreads = 1024;
__global__ __launch_bounds__(kSphereThreads) void sphere_kernel(float* __restrict__ out4,
    const Extreme* __restrict__ partial, int n_partial, const float* __restrict__ pt, int npt, int method_box) {
  __shared__ Extreme sh[kBlock];
  __shared__ float s_center[3], s_radius, s_radius2;
  __shared__ int s_first;
  const int tid = threadIdx.x;
  if (tid < kBlock) {
    Extreme e;
#pragma unroll
    for (int s = 0; s < 6; ++s) { e.v[s] = (s & 1) ? -FLT_MAX : FLT_MAX; e.id[s] = 0x7fffffff; }
    for (int i = tid; i < n_partial; i += kBlock) merge_extreme(e, partial[i]);
    sh[tid] = e;
  }
  __syncthreads();
  for (int step = kBlock / 2; step > 0; step >>= 1) {
    if (tid < step) merge_extreme(sh[tid], sh[tid + step]);
    __syncthreads();
  }
  if (method_box) {  // pytorch/cpp/transform_points.cpp:22-30
    if (tid == 0) {
      float radius = 0.0f;
      for (int j = 0; j < 3; ++j) {
        const float bbmin = sh[0].v[2 * j], bbmax = sh[0].v[2 * j + 1];
        out4[1 + j] = (bbmax + bbmin) / 2.0f;
        const float width = (bbmax - bbmin) / 2.0f;
        radius += width * width;
      }
      out4[0] = sqrt_rn(radius + 1.0e-20f);
    }
    return;
  }
  if (tid == 0) {
    const int* id = sh[0].id;
    float radius = 0.0f;
    int choose = 0;
    for (int i = 0; i < 3; i++) {
      const float* p = pt + 3 * (int64_t)id[2 * i];
      const float* q = pt + 3 * (int64_t)id[2 * i + 1];
      const float dx = p[0] - q[0], dy = p[1] - q[1], dz = p[2] - q[2];
      const float r2 = dx * dx + dy * dy + dz * dz;
      if (r2 > radius) { radius = r2; choose = 2 * i; }
    }
    const float* p = pt + 3 * (int64_t)id[choose];
    const float* q = pt + 3 * (int64_t)id[choose + 1];
    for (int c = 0; c < 3; ++c) s_center[c] = 0.5f * (p[c] + q[c]);
    s_radius2 = radius * 0.25f;
    s_radius = sqrt_rn(s_radius2);
  }
  __syncthreads();
  for (int base = 0; base < npt; base += kSphereThreads) {
    const int i = base + tid;
    float x = 0.0f, y = 0.0f, z = 0.0f;
    if (i < npt) { x = pt[3 * (int64_t)i]; y = pt[3 * (int64_t)i + 1]; z = pt[3 * (int64_t)i + 2]; }
    int from = base;  // points of the chunk before `from` already passed
    while (true) {
      if (tid == 0) s_first = 0x7fffffff;
      __syncthreads();
      float dis2 = 0.0f;
      if (i < npt && i >= from) {
        const float dx = x - s_center[0], dy = y - s_center[1], dz = z - s_center[2];
        dis2 = dx * dx + dy * dy + dz * dz;
        if (dis2 > s_radius2) atomicMin(&s_first, i);
      }
      __syncthreads();
      const int first = s_first;
      if (first == 0x7fffffff) break;
      if (i == first) {
        const float old_to_p = sqrt_rn(dis2);
        const float radius = (s_radius + old_to_p) * 0.5f;
        const float old_to_new = old_to_p - radius;
        const float c0 = div_rn(radius * s_center[0] + old_to_new * x, old_to_p);
        const float c1 = div_rn(radius * s_center[1] + old_to_new * y, old_to_p);
        const float c2 = div_rn(radius * s_center[2] + old_to_new * z, old_to_p);
        s_radius = radius;
        s_radius2 = radius * radius;
        s_center[0] = c0; s_center[1] = c1; s_center[2] = c2;
      }
      from = first + 1;
      __syncthreads();
    }
  }
  if (tid == 0) { out4[0] = s_radius; out4[1] = s_center[0]; out4[2] = s_center[1]; out4[3] = s_center[2]; }
}

// ---- normalise / transform ---------------------------------------------------------------
// The steps of transform_points (and normalize_points, which is translate + scale) applied to
// one point in the reference's order; a step that the host code skips is skipped here.
struct Affine {
  int displace, rotate, translate, scale, scale_normals, orient;  // orient: 0 none, 1..3 = x y z, 4 = xyz
  float offset, rot[9], shift[3], s[3], t[3];
};

__device__ inline void rotate3(float* v, const float* rot) {  // matrix_prod, math_functions.cpp:185-196
  float r[3];
#pragma unroll
  for (int m = 0; m < 3; ++m) {
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < 3; ++k) acc += rot[k * 3 + m] * v[k];
    r[m] = acc;
  }
  v[0] = r[0]; v[1] = r[1]; v[2] = r[2];
}

__global__ void affine_kernel(float* __restrict__ pt, float* __restrict__ nm, int npt, Affine a) {
  const int i = blockIdx.x * kBlock + threadIdx.x;
  if (i >= npt) return;
  float p[3] = {pt[3 * (int64_t)i], pt[3 * (int64_t)i + 1], pt[3 * (int64_t)i + 2]};
  float n[3] = {0.0f, 0.0f, 0.0f};
  if (nm) { n[0] = nm[3 * (int64_t)i]; n[1] = nm[3 * (int64_t)i + 1]; n[2] = nm[3 * (int64_t)i + 2]; }
  if (a.displace && nm)
    for (int m = 0; m < 3; ++m) p[m] += n[m] * a.offset;
  if (a.rotate) { rotate3(p, a.rot); if (nm) rotate3(n, a.rot); }
  if (a.translate)
    for (int m = 0; m < 3; ++m) p[m] += a.shift[m];
  if (a.scale) {
    for (int m = 0; m < 3; ++m) p[m] *= a.s[m];
    if (a.scale_normals && nm) {
      for (int m = 0; m < 3; ++m) n[m] *= a.t[m];
      float len = 0.0f;
      for (int m = 0; m < 3; ++m) len += n[m] * n[m];
      const float inv = div_rn(1.0f, sqrt_rn(len) + 1.0e-15f);
      for (int m = 0; m < 3; ++m) n[m] = n[m] * inv;
    }
  }
  if (a.orient && nm) {
    if (a.orient <= 3) {
      if (n[a.orient - 1] < 0) for (int m = 0; m < 3; ++m) n[m] = -n[m];
    } else {
      for (int m = 0; m < 3; ++m) if (n[m] < 0) n[m] = -n[m];
    }
  }
  for (int m = 0; m < 3; ++m) pt[3 * (int64_t)i + m] = p[m];
  if (nm) for (int m = 0; m < 3; ++m) nm[3 * (int64_t)i + m] = n[m];
}

void host_matrix_prod(float* Cm, const float* A, const float* B, int M, int N, int K) {
  for (int n = 0; n < N; ++n)
    for (int m = 0; m < M; ++m) {
      Cm[n * M + m] = 0;
      for (int k = 0; k < K; ++k) Cm[n * M + m] += A[k * M + m] * B[n * K + k];
    }
}
void host_rotation_matrix(float* rot, const float* angle) {  // math_functions.cpp:148-158
  const float cosx = (float)cos((double)angle[0]), sinx = (float)sin((double)angle[0]);
  const float cosy = (float)cos((double)angle[1]), siny = (float)sin((double)angle[1]);
  const float cosz = (float)cos((double)angle[2]), sinz = (float)sin((double)angle[2]);
  const float rotx[9] = {1.0f, 0, 0, 0, cosx, sinx, 0, -sinx, cosx};
  const float roty[9] = {cosy, 0, -siny, 0, 1.0f, 0, siny, 0, cosy};
  const float rotz[9] = {cosz, sinz, 0, -sinz, cosz, 0, 0, 0, 1.0f};
  float tmp[9];
  host_matrix_prod(tmp, rotx, roty, 3, 3, 3);
  host_matrix_prod(rot, tmp, rotz, 3, 3, 3);
}
// PointsParser::scale (points_parser.cpp:75-101): no-op for unit or zero factors; the normals
// change (and are renormalised) only under a non-uniform scale
void set_scale(Affine* a, const float* s) {
  a->scale = !((s[0] == 1.0f && s[1] == 1.0f && s[2] == 1.0f) || s[0] == 0.0f || s[1] == 0.0f || s[2] == 0.0f);
  a->scale_normals = a->scale && !(s[0] == s[1] && s[0] == s[2]);
  for (int j = 0; j < 3; ++j) { a->s[j] = s[j]; a->t[j] = a->scale ? 1.0f / s[j] : 1.0f; }
}

int run_affine(void* out_dev, const void* in_dev, const PointsInfo* pi, const Affine& a, hipStream_t s) {
  if (out_dev != in_dev)
    OCNN_HIP_OK(hipMemcpyAsync(out_dev, in_dev, blob_bytes(pi), hipMemcpyDeviceToDevice, s));
  if (!(a.displace || a.rotate || a.translate || a.scale || a.orient)) return OCNN_OK;
  char* b = static_cast<char*>(out_dev);
  float* pt = reinterpret_cast<float*>(b + pi->ptr_dis[0]);
  float* nm = (pi->content_flags & 2) ? reinterpret_cast<float*>(b + pi->ptr_dis[1]) : nullptr;
  affine_kernel<<<blocks_for(pi->pt_num), kBlock, 0, s>>>(pt, nm, pi->pt_num, a);
  OCNN_LAUNCH_OK("points_affine");
  return OCNN_OK;
}

// ---- clip -----------------------------------------------------------------------------------
struct InBox {
  const float* pt; float lo[3], hi[3];
  __device__ bool operator()(int64_t i) const {
    const float x = pt[3 * i], y = pt[3 * i + 1], z = pt[3 * i + 2];
    return lo[0] < x && x < hi[0] && lo[1] < y && y < hi[1] && lo[2] < z && z < hi[2];
  }
};
struct ClipOut {
  int* mask;
  const float* src[4]; float* dst[4]; int ch[4];
  __device__ void operator()(int64_t i, bool flag, int rank) const {
    mask[i] = flag ? 1 : 0;
    if (!flag) return;
#pragma unroll
    for (int t = 0; t < 4; ++t)
      for (int c = 0; c < ch[t]; ++c) dst[t][(int64_t)rank * ch[t] + c] = src[t][i * ch[t] + c];
  }
};
// header with the new point count; with no point inside, the reference keeps point 0 and moves
// it to the box corner (points_parser.cpp:169-176)
__global__ void clip_finish_kernel(char* out, PointsInfo hdr, int* mask, float lo0, float lo1, float lo2, int none_inside) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    *reinterpret_cast<PointsInfo*>(out) = hdr;
    if (none_inside) {
      float* p = reinterpret_cast<float*>(out + hdr.ptr_dis[0]);
      p[0] = lo0; p[1] = lo1; p[2] = lo2;
      mask[0] = 1;
    }
  }
}

}  // namespace
}  // namespace ocnn

using namespace ocnn;

extern "C" {

size_t ocnn_points_workspace_bytes(int pt_num) {
  size_t extremes = sizeof(Extreme) * 1024 + 256;
  size_t scan = scan_scratch_bytes(pt_num) + 256;
  return (extremes > scan ? extremes : scan) + 256;
}

int ocnn_bounding_sphere(const void* points_dev, const void* points_info, int method_box, float* out4,
    void* workspace_dev, size_t workspace_bytes, ocnn_stream_t stream) {
  const PointsInfo* pi;
  int e = check_points(points_info, &pi);
  if (e) return e;
  OCNN_REQUIRE(points_dev && out4, OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(workspace_dev && workspace_bytes >= ocnn_points_workspace_bytes(pi->pt_num), OCNN_E_WORKSPACE,
      "workspace %zu < %zu bytes", workspace_bytes, ocnn_points_workspace_bytes(pi->pt_num));
  hipStream_t s = as_stream(stream);
  const float* pt = reinterpret_cast<const float*>(static_cast<const char*>(points_dev) + pi->ptr_dis[0]);
  float* out_dev = static_cast<float*>(workspace_dev);
  Extreme* partial = reinterpret_cast<Extreme*>(static_cast<char*>(workspace_dev) + 256);
  int blocks = blocks_for(pi->pt_num);
  if (blocks > 1024) blocks = 1024;
  extremes_kernel<<<blocks, kBlock, 0, s>>>(partial, pt, pi->pt_num);
  OCNN_LAUNCH_OK("extremes");
  sphere_kernel<<<1, kSphereThreads, 0, s>>>(out_dev, partial, blocks, pt, pi->pt_num, method_box ? 1 : 0);
  OCNN_LAUNCH_OK("sphere");
  return fetch_words(out4, out_dev, 4, s);
}

int ocnn_normalize_points(void* out_dev, const void* in_dev, const void* points_info, float radius,
    const float* center, ocnn_stream_t stream) {
  const PointsInfo* pi;
  int e = check_points(points_info, &pi);
  if (e) return e;
  OCNN_REQUIRE(out_dev && in_dev && center, OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(radius >= 0.0f, OCNN_E_BADARG, "radius %g < 0", radius);
  Affine a;
  memset(&a, 0, sizeof(a));
  for (int j = 0; j < 3; ++j) a.shift[j] = -center[j];
  a.translate = a.shift[0] != 0.0f || a.shift[1] != 0.0f || a.shift[2] != 0.0f;
  const float inv = 1.0f / radius;
  const float sc[3] = {inv, inv, inv};
  set_scale(&a, sc);
  return run_affine(out_dev, in_dev, pi, a, as_stream(stream));
}

int ocnn_transform_points(void* out_dev, const void* in_dev, const void* points_info, const float* angle,
    const float* scale, const float* jitter, float offset, const char* normal_axis, ocnn_stream_t stream) {
  const PointsInfo* pi;
  int e = check_points(points_info, &pi);
  if (e) return e;
  OCNN_REQUIRE(out_dev && in_dev && angle && scale && jitter, OCNN_E_BADARG, "null pointer");
  const float kEPS = 1.0e-10f;
  Affine a;
  memset(&a, 0, sizeof(a));
  a.displace = offset > kEPS;
  a.offset = offset;
  a.rotate = fabs(angle[0]) > kEPS || fabs(angle[1]) > kEPS || fabs(angle[2]) > kEPS;
  if (a.rotate) host_rotation_matrix(a.rot, angle);
  a.translate = fabs(jitter[0]) > kEPS || fabs(jitter[1]) > kEPS || fabs(jitter[2]) > kEPS;
  for (int j = 0; j < 3; ++j) a.shift[j] = jitter[j];
  if (scale[0] != 1.0f || scale[1] != 1.0f || scale[2] != 1.0f) set_scale(&a, scale);
  if (normal_axis && normal_axis[0]) {
    if (!strcmp(normal_axis, "x")) a.orient = 1;
    else if (!strcmp(normal_axis, "y")) a.orient = 2;
    else if (!strcmp(normal_axis, "z")) a.orient = 3;
    else if (!strcmp(normal_axis, "xyz")) a.orient = 4;
  }
  return run_affine(out_dev, in_dev, pi, a, as_stream(stream));
}

int ocnn_clip_points(void* out_dev, void* out_info, int* inbox_mask_dev, const void* in_dev,
    const void* points_info, const float* bbmin, const float* bbmax, void* workspace_dev,
    size_t workspace_bytes, ocnn_stream_t stream) {
  const PointsInfo* pi;
  int e = check_points(points_info, &pi);
  if (e) return e;
  OCNN_REQUIRE(out_dev && out_info && inbox_mask_dev && in_dev && bbmin && bbmax, OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(out_dev != in_dev, OCNN_E_BADARG, "clip_points does not run in place");
  OCNN_REQUIRE(workspace_dev && workspace_bytes >= ocnn_points_workspace_bytes(pi->pt_num), OCNN_E_WORKSPACE,
      "workspace %zu < %zu bytes", workspace_bytes, ocnn_points_workspace_bytes(pi->pt_num));
  hipStream_t s = as_stream(stream);
  const int npt = pi->pt_num;
  OCNN_HIP_OK(hipMemcpyAsync(out_dev, in_dev, blob_bytes(pi), hipMemcpyDeviceToDevice, s));
  const char* in = static_cast<const char*>(in_dev);
  char* out = static_cast<char*>(out_dev);
  InBox pred;
  pred.pt = reinterpret_cast<const float*>(in + pi->ptr_dis[0]);
  for (int j = 0; j < 3; ++j) { pred.lo[j] = bbmin[j]; pred.hi[j] = bbmax[j]; }
  ClipOut co;
  co.mask = inbox_mask_dev;
  for (int t = 0; t < 4; ++t) {
    const bool has = (pi->content_flags & (1 << t)) && pi->channels[t] > 0;
    co.ch[t] = has ? pi->channels[t] : 0;
    co.src[t] = has ? reinterpret_cast<const float*>(in + pi->ptr_dis[t]) : nullptr;
    co.dst[t] = has ? reinterpret_cast<float*>(out + pi->ptr_dis[t]) : nullptr;
  }
  int* total_dev = static_cast<int*>(workspace_dev);
  int* scratch = reinterpret_cast<int*>(static_cast<char*>(workspace_dev) + 256);
  OCNN_HIP_OK(flag_scan(pred, co, npt, scratch, total_dev, s));
  int inside = 0;
  {
    const int e = fetch_words(&inside, total_dev, 1, s);
    if (e) return e;
  }
  PointsInfo hdr = *pi;
  const int none = inside == 0;
  hdr.pt_num = none ? 1 : inside;
  clip_finish_kernel<<<1, 64, 0, s>>>(out, hdr, inbox_mask_dev, bbmin[0], bbmin[1], bbmin[2], none);
  OCNN_LAUNCH_OK("clip_finish");
  memcpy(out_info, &hdr, sizeof(hdr));
  return OCNN_OK;
}

}  // extern "C"
