// Feature transfer between octrees and to free points:
//   * octree_align: the features of one octree scattered to the nodes of another with the same
//     keys (align_forward_gpu / align_backward_gpu, octree/octree/octree_nn.cu:710-752, driven as
//     in pytorch/cpp/octree_align.cpp:9-83);
//   * nearest / trilinear interpolation at free points (octree_nearest_pts, octree_trilinear_pts,
//     pytorch/ocnn/modules.py:209-275), fused: the reference builds eight keys per point, searches
//     them, assembles a sparse matrix and multiplies twice; here one kernel does key arithmetic,
//     the eight binary searches and the weights, and a second one the weighted gather.
#include "ocnn_common.h"

namespace ocnn {
namespace {

// ---- align -----------------------------------------------------------------------------------
__global__ void align_forward_kernel(float* __restrict__ top, int top_h, const float* __restrict__ btm, int btm_h,
    const int* __restrict__ index, int channel) {
  const int h = blockIdx.x * kBlock + threadIdx.x;
  if (h >= btm_h) return;
  const int j = index[h];
  if (j < 0 || j >= top_h) return;
  for (int c = 0; c < channel; ++c) top[(int64_t)c * top_h + j] = btm[(int64_t)c * btm_h + h];
}
__global__ void align_backward_kernel(const float* __restrict__ top, int top_h, float* __restrict__ btm, int btm_h,
    const int* __restrict__ index, int channel) {
  const int h = blockIdx.x * kBlock + threadIdx.x;
  if (h >= btm_h) return;
  const int j = index[h];
  const bool ok = j >= 0 && j < top_h;
  for (int c = 0; c < channel; ++c) btm[(int64_t)c * btm_h + h] = ok ? top[(int64_t)c * top_h + j] : 0.0f;
}
__global__ void zero_kernel(float* __restrict__ p, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < n) p[i] = 0.0f;
}

// ---- interpolation ---------------------------------------------------------------------------
// Morton key of a packed (x, y, z, id) key, as octree_search_key does for key_is_xyz
// (pytorch/cpp/octree_key.cpp:83-132 -> xyz2key): bit i of axis j goes to bit 3i + 2 - j.
__device__ inline uint64_t packed_to_morton(uint64_t v, int depth) {
  const uint32_t x = (uint32_t)(v & 0xffff), y = (uint32_t)((v >> 16) & 0xffff), z = (uint32_t)((v >> 32) & 0xffff);
  uint64_t k = 0;
  for (int i = 0; i < depth; ++i) {
    k |= (uint64_t)((x >> i) & 1u) << (3 * i + 2);
    k |= (uint64_t)((y >> i) & 1u) << (3 * i + 1);
    k |= (uint64_t)((z >> i) & 1u) << (3 * i);
  }
  return (k & 0x0000ffffffffffffull) | (v & 0xffff000000000000ull);
}
__device__ inline int search(const uint64_t* __restrict__ key, int n_key, uint64_t q) {
  int lo = 0, hi = n_key;
  while (lo < hi) {
    const int mid = lo + ((hi - lo) >> 1);
    if (key[mid] < q) lo = mid + 1; else hi = mid;
  }
  return (lo < n_key && key[lo] == q) ? lo : -1;
}
// float -> int16 as torch's .short(): truncation toward zero, then the low 16 bits
__device__ inline uint64_t as_short(float v) { return (uint64_t)(uint16_t)(int16_t)(int)v; }

// one thread per (point, corner): index and weight.  K = 1 (nearest) or 8 (trilinear).
__global__ void interp_index_kernel(int* __restrict__ idx, float* __restrict__ weight, const float* __restrict__ pts,
    int n_pts, const uint64_t* __restrict__ key, int n_key, int depth, int K) {
  const int t = blockIdx.x * kBlock + threadIdx.x;
  if (t >= n_pts * K) return;
  const int p = t / K, m = t % K;
  const float* q = pts + 4 * (int64_t)p;
  if (K == 1) {  // modules.py:209-221
    const uint64_t packed = as_short(q[0]) | (as_short(q[1]) << 16) | (as_short(q[2]) << 32) | (as_short(q[3]) << 48);
    idx[t] = search(key, n_key, packed_to_morton(packed, depth));
    weight[t] = 1.0f;
    return;
  }
  // modules.py:224-268: values live at voxel centres; corner m = (m >> 2, m >> 1, m) & 1 along x, y, z
  float frac[3];
  uint64_t packed = 0;
  for (int c = 0; c < 3; ++c) {
    const float f = q[c] - 0.5f;
    const float i = floorf(f);
    frac[c] = f - i;
    packed |= as_short(i) << (16 * c);
  }
  packed |= as_short(q[3]) << 48;
  // the corner offset is ADDED to the packed 64-bit key, carries included, as the reference does
  const uint64_t off = (uint64_t)((m >> 2) & 1) | ((uint64_t)((m >> 1) & 1) << 16) | ((uint64_t)(m & 1) << 32);
  idx[t] = search(key, n_key, packed_to_morton(packed + off, depth));
  const float fx = (float)(1 - ((m >> 2) & 1)) - frac[0];
  const float fy = (float)(1 - ((m >> 1) & 1)) - frac[1];
  const float fz = (float)(1 - (m & 1)) - frac[2];
  weight[t] = fabsf(fx * fy * fz);
}

// out[c, p] = sum_m w_m data[c, idx_m] / (sum_m w_m + 1e-10) over the corners that exist;
// nearest: data[c, idx] or 0.  One thread per point, channels in the inner loop.
__global__ void interp_gather_kernel(float* __restrict__ out, const float* __restrict__ data, int channel, int H,
    const int* __restrict__ idx, const float* __restrict__ weight, int n_pts, int K, int normalise) {
  const int p = blockIdx.x * kBlock + threadIdx.x;
  if (p >= n_pts) return;
  int id[8];
  float w[8];
  float norm = 0.0f;
  for (int m = 0; m < K; ++m) {
    id[m] = idx[(int64_t)p * K + m];
    w[m] = (id[m] >= 0 && id[m] < H) ? weight[(int64_t)p * K + m] : 0.0f;
    if (id[m] < 0 || id[m] >= H) id[m] = -1;
    norm += w[m];
  }
  const float inv = normalise ? 1.0f / (norm + 1e-10f) : 1.0f;
  for (int c = 0; c < channel; ++c) {
    float acc = 0.0f;
    for (int m = 0; m < K; ++m)
      if (id[m] >= 0) acc += w[m] * data[(int64_t)c * H + id[m]];
    out[(int64_t)c * n_pts + p] = acc * inv;
  }
}
// the adjoint: grad_data[c, idx_m] += w_m / (norm + 1e-10) * grad_out[c, p]
__global__ void interp_scatter_kernel(float* __restrict__ grad_data, const float* __restrict__ grad_out, int channel,
    int H, const int* __restrict__ idx, const float* __restrict__ weight, int n_pts, int K, int normalise) {
  const int p = blockIdx.x * kBlock + threadIdx.x;
  if (p >= n_pts) return;
  int id[8];
  float w[8];
  float norm = 0.0f;
  for (int m = 0; m < K; ++m) {
    id[m] = idx[(int64_t)p * K + m];
    const bool ok = id[m] >= 0 && id[m] < H;
    w[m] = ok ? weight[(int64_t)p * K + m] : 0.0f;
    if (!ok) id[m] = -1;
    norm += w[m];
  }
  const float inv = normalise ? 1.0f / (norm + 1e-10f) : 1.0f;
  for (int c = 0; c < channel; ++c) {
    const float g = grad_out[(int64_t)c * n_pts + p] * inv;
    for (int m = 0; m < K; ++m)
      if (id[m] >= 0) unsafeAtomicAdd(grad_data + (int64_t)c * H + id[m], w[m] * g);
  }
}

}  // namespace
}  // namespace ocnn

using namespace ocnn;

extern "C" {

int ocnn_align_forward(float* top, int top_h, int channel, const float* btm, int btm_h, const int* idx,
    ocnn_stream_t stream) {
  OCNN_REQUIRE(top && btm && idx && top_h >= 0 && btm_h >= 0 && channel > 0, OCNN_E_BADARG, "bad argument");
  hipStream_t s = as_stream(stream);
  const int64_t n = (int64_t)top_h * channel;
  if (n > 0) zero_kernel<<<blocks_for(n), kBlock, 0, s>>>(top, n);
  if (btm_h > 0) align_forward_kernel<<<blocks_for(btm_h), kBlock, 0, s>>>(top, top_h, btm, btm_h, idx, channel);
  OCNN_LAUNCH_OK("align_forward");
  return OCNN_OK;
}

int ocnn_align_backward(const float* top, int top_h, int channel, float* btm, int btm_h, const int* idx,
    ocnn_stream_t stream) {
  OCNN_REQUIRE(top && btm && idx && top_h >= 0 && btm_h >= 0 && channel > 0, OCNN_E_BADARG, "bad argument");
  if (btm_h > 0)
    align_backward_kernel<<<blocks_for(btm_h), kBlock, 0, as_stream(stream)>>>(top, top_h, btm, btm_h, idx, channel);
  OCNN_LAUNCH_OK("align_backward");
  return OCNN_OK;
}

int ocnn_octree_interp(float* out, const float* data, int channel, int H, const uint64_t* key, int n_key,
    const float* pts, int n_pts, int depth, int method, int* idx, float* weight, ocnn_stream_t stream) {
  OCNN_REQUIRE(out && data && pts && idx && weight && (key || n_key == 0), OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(channel > 0 && H >= 0 && n_key >= 0 && n_pts >= 0 && depth >= 0 && depth <= 16, OCNN_E_BADARG,
      "bad argument");
  OCNN_REQUIRE(method == 0 || method == 1, OCNN_E_BADARG, "method %d is neither nearest (0) nor linear (1)", method);
  if (n_pts == 0) return OCNN_OK;
  hipStream_t s = as_stream(stream);
  const int K = method == 0 ? 1 : 8;
  interp_index_kernel<<<blocks_for((int64_t)n_pts * K), kBlock, 0, s>>>(idx, weight, pts, n_pts, key, n_key, depth, K);
  OCNN_LAUNCH_OK("interp_index");
  interp_gather_kernel<<<blocks_for(n_pts), kBlock, 0, s>>>(out, data, channel, H, idx, weight, n_pts, K, method);
  OCNN_LAUNCH_OK("interp_gather");
  return OCNN_OK;
}

int ocnn_octree_interp_backward(float* grad_data, const float* grad_out, int channel, int H, int n_pts, int method,
    const int* idx, const float* weight, ocnn_stream_t stream) {
  OCNN_REQUIRE(grad_data && grad_out && idx && weight && channel > 0 && H >= 0 && n_pts >= 0, OCNN_E_BADARG,
      "bad argument");
  OCNN_REQUIRE(method == 0 || method == 1, OCNN_E_BADARG, "method %d", method);
  hipStream_t s = as_stream(stream);
  const int64_t n = (int64_t)H * channel;
  if (n > 0) zero_kernel<<<blocks_for(n), kBlock, 0, s>>>(grad_data, n);
  if (n_pts > 0)
    interp_scatter_kernel<<<blocks_for(n_pts), kBlock, 0, s>>>(grad_data, grad_out, channel, H, idx, weight, n_pts,
        method == 0 ? 1 : 8, method);
  OCNN_LAUNCH_OK("interp_scatter");
  return OCNN_OK;
}

}  // extern "C"
