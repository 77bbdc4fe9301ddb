// Bandwidth-bound gather/scatter ops of the octree hot path: pad / depad,
// octree2col / col2octree (API ops; the convolution itself never builds a
// column buffer), max-pool / unpool / mask-pool.
//
// All tensors are channel-major [C, H]; one thread handles one row index h so
// that a wavefront touches 64 consecutive h (256 B of fp32) per channel, and
// index arrays (label / neigh / mask) are read once and reused over a chunk
// of channels.
#include "ocnn_common.h"

namespace ocnn {
namespace {

constexpr int kChanChunk = 8;  // channels handled per thread in the gather ops

template <typename T> __device__ inline T zero_of();
template <> __device__ inline float zero_of<float>() { return 0.0f; }
template <> __device__ inline uint16_t zero_of<uint16_t>() { return 0; }
template <typename T> __device__ inline T from_f32(float v);
template <> __device__ inline float from_f32<float>(float v) { return v; }
template <> __device__ inline uint16_t from_f32<uint16_t>(float v) { return f32_to_bf16(v); }
template <typename T> __device__ inline float to_f32(T v);
template <> __device__ inline float to_f32<float>(float v) { return v; }
template <> __device__ inline float to_f32<uint16_t>(uint16_t v) { return bf16_to_f32(v); }

template <typename T>
__global__ void fill_kernel(T* p, int64_t n, T v) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += step) p[i] = v;
}

// ---- pad / depad -----------------------------------------------------------
template <typename T>
__global__ void pad_forward_kernel(T* __restrict__ Y, int Hy, int C, const T* __restrict__ X,
    int Hx, const int* __restrict__ label, T dval) {
  int h = blockIdx.x * blockDim.x + threadIdx.x;
  if (h >= Hy) return;
  int l = label[h];
  int c0 = blockIdx.y * kChanChunk, c1 = min(C, c0 + kChanChunk);
  for (int c = c0; c < c1; ++c)
    Y[(int64_t)c * Hy + h] = (l < 0 || l >= Hx) ? dval : X[(int64_t)c * Hx + l];
}

template <typename T>
__global__ void pad_backward_kernel(T* __restrict__ X, int Hx, int C, const T* __restrict__ Y,
    int Hy, const int* __restrict__ label) {
  int h = blockIdx.x * blockDim.x + threadIdx.x;
  if (h >= Hy) return;
  int l = label[h];
  if (l < 0 || l >= Hx) return;  // rows outside X are ignored rather than written
  int c0 = blockIdx.y * kChanChunk, c1 = min(C, c0 + kChanChunk);
  for (int c = c0; c < c1; ++c) X[(int64_t)c * Hx + l] = Y[(int64_t)c * Hy + h];
}

__global__ void make_ichild_kernel(int* __restrict__ ichild, int n_nempty,
    const int* __restrict__ child, int n) {
  int h = blockIdx.x * blockDim.x + threadIdx.x;
  if (h >= n) return;
  int l = child[h];
  if (l >= 0 && l < n_nempty) ichild[l] = h;
}

// ---- octree2col / col2octree -------------------------------------------------
struct ColArgs {
  int channel, height, octree_h, K, stride, height_col, n;
  int slot[27];  // neighbour slot of each tap for sibling 0
};

// neighbour row of column h for tap k, -1 when absent.  P = non-empty variant.
template <bool P>
__device__ inline int col_source(const ColArgs& a, int h, int k, const int* __restrict__ neigh,
    const int* __restrict__ child, const int* __restrict__ ichild) {
  int64_t index;
  if (a.stride == 2) {
    index = ((int64_t)h << 6) + a.slot[k];
  } else {
    int hp = P ? ichild[h] : h;
    index = ((int64_t)(hp >> 3) << 6) + sibling_slot(hp & 7) + a.slot[k];
  }
  int p = neigh[index];
  if (P && p >= 0) p = child[p];
  return p;
}

template <typename T, bool P>
__global__ void octree2col_kernel(T* __restrict__ col, const T* __restrict__ data, ColArgs a,
    const int* __restrict__ neigh, const int* __restrict__ child, const int* __restrict__ ichild) {
  int hl = blockIdx.x * blockDim.x + threadIdx.x;  // column inside the chunk
  if (hl >= a.height_col) return;
  int k = blockIdx.y;
  int h = a.n * a.height_col + hl;
  int p = h < a.height ? col_source<P>(a, h, k, neigh, child, ichild) : -1;
  int c0 = blockIdx.z * kChanChunk, c1 = min(a.channel, c0 + kChanChunk);
  for (int c = c0; c < c1; ++c)
    col[((int64_t)c * a.K + k) * a.height_col + hl] =
        (p < 0 || p >= a.octree_h) ? zero_of<T>() : data[(int64_t)c * a.octree_h + p];
}

template <bool P>
__global__ void col2octree_kernel(const float* __restrict__ col, float* __restrict__ data, ColArgs a,
    const int* __restrict__ neigh, const int* __restrict__ child, const int* __restrict__ ichild) {
  int hl = blockIdx.x * blockDim.x + threadIdx.x;
  if (hl >= a.height_col) return;
  int k = blockIdx.y;
  int h = a.n * a.height_col + hl;
  if (h >= a.height) return;
  int p = col_source<P>(a, h, k, neigh, child, ichild);
  if (p < 0 || p >= a.octree_h) return;
  int c0 = blockIdx.z * kChanChunk, c1 = min(a.channel, c0 + kChanChunk);
  for (int c = c0; c < c1; ++c)
    unsafeAtomicAdd(&data[(int64_t)c * a.octree_h + p],
        col[((int64_t)c * a.K + k) * a.height_col + hl]);
}

// ---- pooling -------------------------------------------------------------------
// One thread reduces one sibling group (8 consecutive rows = 32 B of fp32).
template <typename T>
__global__ void max_pool_kernel(T* __restrict__ top, int top_h, int* __restrict__ mask,
    const T* __restrict__ btm, int btm_h, int64_t total) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  int c = (int)(i / top_h), h = (int)(i % top_h);
  const T* src = btm + (int64_t)c * btm_h + 8 * (int64_t)h;
  T v[8];
  if ((reinterpret_cast<uintptr_t>(src) & (8 * sizeof(T) - 1)) == 0) {
    if (sizeof(T) == 4) {
      float4 a = reinterpret_cast<const float4*>(src)[0], b = reinterpret_cast<const float4*>(src)[1];
      memcpy(v, &a, 16);
      memcpy(v + 4, &b, 16);
    } else {
      uint4 a = reinterpret_cast<const uint4*>(src)[0];
      memcpy(v, &a, 16);
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = src[j];
  }
  T best = v[0];
  float bestf = to_f32(best);
  int arg = 0;
#pragma unroll
  for (int j = 1; j < 8; ++j) {
    float f = to_f32(v[j]);
    if (f > bestf) { bestf = f; best = v[j]; arg = j; }
  }
  top[i] = best;
  mask[i] = 8 * h + arg;
}

// Writes every row of the sibling group: the pooled value where the mask points,
// zero elsewhere, so no separate zero fill is needed.  A mask that points outside
// its own group (never produced by max_pool) is left to unpool_foreign_kernel.
template <typename T>
__global__ void max_unpool_kernel(const T* __restrict__ top, int top_h, const int* __restrict__ mask,
    T* __restrict__ btm, int btm_h, int64_t total) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  int c = (int)(i / top_h), h = (int)(i % top_h);
  int m = mask[i] - 8 * h;
  T val = top[i];
  T v[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = (j == m) ? val : zero_of<T>();
  T* dst = btm + (int64_t)c * btm_h + 8 * (int64_t)h;
  if ((reinterpret_cast<uintptr_t>(dst) & (8 * sizeof(T) - 1)) == 0) {
    if (sizeof(T) == 4) {
      float4 a, b;
      memcpy(&a, v, 16);
      memcpy(&b, v + 4, 16);
      reinterpret_cast<float4*>(dst)[0] = a;
      reinterpret_cast<float4*>(dst)[1] = b;
    } else {
      uint4 a;
      memcpy(&a, v, 16);
      reinterpret_cast<uint4*>(dst)[0] = a;
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) dst[j] = v[j];
  }
}

template <typename T>
__global__ void unpool_foreign_kernel(const T* __restrict__ top, int top_h,
    const int* __restrict__ mask, T* __restrict__ btm, int btm_h, int64_t total) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  int c = (int)(i / top_h), h = (int)(i % top_h);
  int m = mask[i];
  if ((m >> 3) == h || m < 0 || m >= btm_h) return;
  btm[(int64_t)c * btm_h + m] = top[i];
}

template <typename T>
__global__ void mask_pool_kernel(T* __restrict__ top, int top_h, const int* __restrict__ mask,
    const T* __restrict__ btm, int btm_h, int64_t total) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  int c = (int)(i / top_h);
  int m = mask[i];
  top[i] = (m < 0 || m >= btm_h) ? zero_of<T>() : btm[(int64_t)c * btm_h + m];
}

bool fill_col_args(ColArgs* a, int channel, int height, int octree_h, const int* ks, int stride,
    int height_col, int n) {
  KernelTaps t;
  if (!kernel_taps(ks, &t)) return false;
  a->channel = channel;
  a->height = height;
  a->octree_h = octree_h;
  a->K = t.count;
  a->stride = stride;
  a->height_col = height_col;
  a->n = n;
  for (int k = 0; k < 27; ++k) a->slot[k] = k < t.count ? tap_slot(t.tap[k]) : 0;
  return true;
}

int check_col(const void* col, const void* data, int channel, int height, const int* ks, int stride,
    const int* neigh, int height_col, int n, int dtype) {
  OCNN_REQUIRE(col && data && neigh && ks, OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(channel > 0 && height >= 0 && height_col > 0 && n >= 0, OCNN_E_BADARG,
      "channel %d height %d height_col %d n %d", channel, height, height_col, n);
  OCNN_REQUIRE(stride == 1 || stride == 2, OCNN_E_BADARG, "stride %d", stride);
  OCNN_REQUIRE(dtype == OCNN_F32 || dtype == OCNN_BF16, OCNN_E_BADARG, "dtype %d", dtype);
  return OCNN_OK;
}

template <bool P>
int run_octree2col(void* col, const void* data, int channel, int height, int octree_h, const int* ks,
    int stride, const int* neigh, const int* child, const int* ichild, int height_col, int n,
    int dtype, hipStream_t s) {
  int e = check_col(col, data, channel, height, ks, stride, neigh, height_col, n, dtype);
  if (e) return e;
  ColArgs a;
  OCNN_REQUIRE(fill_col_args(&a, channel, height, octree_h, ks, stride, height_col, n),
      OCNN_E_UNSUPPORTED, "kernel size %d%d%d", ks[0], ks[1], ks[2]);
  dim3 grid(blocks_for(height_col), a.K, (channel + kChanChunk - 1) / kChanChunk);
  if (dtype == OCNN_F32)
    octree2col_kernel<float, P><<<grid, kBlock, 0, s>>>((float*)col, (const float*)data, a, neigh, child, ichild);
  else
    octree2col_kernel<uint16_t, P><<<grid, kBlock, 0, s>>>((uint16_t*)col, (const uint16_t*)data, a, neigh, child, ichild);
  OCNN_LAUNCH_OK("octree2col");
  return OCNN_OK;
}

template <bool P>
int run_col2octree(const void* col, void* data, int channel, int height, int octree_h, const int* ks,
    int stride, const int* neigh, const int* child, const int* ichild, int height_col, int n,
    int dtype, hipStream_t s) {
  int e = check_col(col, data, channel, height, ks, stride, neigh, height_col, n, dtype);
  if (e) return e;
  OCNN_REQUIRE(dtype == OCNN_F32, OCNN_E_UNSUPPORTED, "col2octree accumulates in fp32 only");
  ColArgs a;
  OCNN_REQUIRE(fill_col_args(&a, channel, height, octree_h, ks, stride, height_col, n),
      OCNN_E_UNSUPPORTED, "kernel size %d%d%d", ks[0], ks[1], ks[2]);
  if (n == 0) {  // the output is cleared once, by the first chunk (octree_nn.cpp:226)
    int64_t cnt = (int64_t)channel * octree_h;
    fill_kernel<float><<<blocks_for(cnt, kBlock * 4), kBlock, 0, s>>>((float*)data, cnt, 0.0f);
    OCNN_LAUNCH_OK("fill");
  }
  if (height == 0) return OCNN_OK;
  dim3 grid(blocks_for(height_col), a.K, (channel + kChanChunk - 1) / kChanChunk);
  col2octree_kernel<P><<<grid, kBlock, 0, s>>>((const float*)col, (float*)data, a, neigh, child, ichild);
  OCNN_LAUNCH_OK("col2octree");
  return OCNN_OK;
}

int check_pool(const void* top, int top_h, const void* mask, const void* btm, int btm_h, int channel,
    int dtype) {
  OCNN_REQUIRE(top && mask && btm, OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(channel > 0 && top_h >= 0 && btm_h >= 0, OCNN_E_BADARG, "channel %d top_h %d btm_h %d",
      channel, top_h, btm_h);
  OCNN_REQUIRE(dtype == OCNN_F32 || dtype == OCNN_BF16, OCNN_E_BADARG, "dtype %d", dtype);
  return OCNN_OK;
}

}  // namespace
}  // namespace ocnn

using namespace ocnn;

extern "C" {

int ocnn_pad_forward(void* Y, int Hy, int C, const void* X, int Hx, const int* label, float dval,
    int dtype, ocnn_stream_t stream) {
  OCNN_REQUIRE(Y && label && (X || Hx == 0), OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(Hy >= 0 && Hx >= 0 && C > 0, OCNN_E_BADARG, "Hy %d Hx %d C %d", Hy, Hx, C);
  if (Hy == 0) return OCNN_OK;
  dim3 grid(blocks_for(Hy), (C + kChanChunk - 1) / kChanChunk);
  hipStream_t s = as_stream(stream);
  if (dtype == OCNN_F32)
    pad_forward_kernel<float><<<grid, kBlock, 0, s>>>((float*)Y, Hy, C, (const float*)X, Hx, label, dval);
  else if (dtype == OCNN_BF16) {
    // the pad value is rounded to bf16 on the host side of the launch
    uint32_t u;
    memcpy(&u, &dval, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    pad_forward_kernel<uint16_t><<<grid, kBlock, 0, s>>>((uint16_t*)Y, Hy, C, (const uint16_t*)X, Hx,
        label, (uint16_t)(u >> 16));
  } else
    return fail(OCNN_E_BADARG, "dtype %d", dtype);
  OCNN_LAUNCH_OK("pad_forward");
  return OCNN_OK;
}

int ocnn_pad_backward(void* X, int Hx, int C, const void* Y, int Hy, const int* label, int dtype,
    ocnn_stream_t stream) {
  OCNN_REQUIRE(label && (X || Hx == 0) && (Y || Hy == 0), OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(Hy >= 0 && Hx >= 0 && C > 0, OCNN_E_BADARG, "Hy %d Hx %d C %d", Hy, Hx, C);
  if (Hy == 0 || Hx == 0) return OCNN_OK;
  dim3 grid(blocks_for(Hy), (C + kChanChunk - 1) / kChanChunk);
  hipStream_t s = as_stream(stream);
  if (dtype == OCNN_F32)
    pad_backward_kernel<float><<<grid, kBlock, 0, s>>>((float*)X, Hx, C, (const float*)Y, Hy, label);
  else if (dtype == OCNN_BF16)
    pad_backward_kernel<uint16_t><<<grid, kBlock, 0, s>>>((uint16_t*)X, Hx, C, (const uint16_t*)Y, Hy, label);
  else
    return fail(OCNN_E_BADARG, "dtype %d", dtype);
  OCNN_LAUNCH_OK("pad_backward");
  return OCNN_OK;
}

int ocnn_make_ichild(int* ichild, int n_nempty, const int* child, int n_node, ocnn_stream_t stream) {
  OCNN_REQUIRE(child && (ichild || n_nempty == 0), OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(n_nempty >= 0 && n_node >= 0, OCNN_E_BADARG, "n_nempty %d n_node %d", n_nempty, n_node);
  if (n_node == 0) return OCNN_OK;
  make_ichild_kernel<<<blocks_for(n_node), kBlock, 0, as_stream(stream)>>>(ichild, n_nempty, child, n_node);
  OCNN_LAUNCH_OK("make_ichild");
  return OCNN_OK;
}

int ocnn_octree2col(void* col, const void* data, int channel, int height, const int* kernel_size,
    int stride, const int* neigh, int height_col, int n, int dtype, ocnn_stream_t stream) {
  int octree_h = height << (3 * (stride - 1));
  return run_octree2col<false>(col, data, channel, height, octree_h, kernel_size, stride, neigh,
      nullptr, nullptr, height_col, n, dtype, as_stream(stream));
}
int ocnn_col2octree(const void* col, void* data, int channel, int height, const int* kernel_size,
    int stride, const int* neigh, int height_col, int n, int dtype, ocnn_stream_t stream) {
  int octree_h = height << (3 * (stride - 1));
  return run_col2octree<false>(col, data, channel, height, octree_h, kernel_size, stride, neigh,
      nullptr, nullptr, height_col, n, dtype, as_stream(stream));
}
int ocnn_octree2colP(void* col, const void* data, int channel, int height, int octree_h,
    const int* kernel_size, int stride, const int* neigh, const int* child, const int* ichild,
    int height_col, int n, int dtype, ocnn_stream_t stream) {
  OCNN_REQUIRE(child && (ichild || stride == 2), OCNN_E_BADARG, "null child/ichild");
  return run_octree2col<true>(col, data, channel, height, octree_h, kernel_size, stride, neigh, child,
      ichild, height_col, n, dtype, as_stream(stream));
}
int ocnn_col2octreeP(const void* col, void* data, int channel, int height, int octree_h,
    const int* kernel_size, int stride, const int* neigh, const int* child, const int* ichild,
    int height_col, int n, int dtype, ocnn_stream_t stream) {
  OCNN_REQUIRE(child && (ichild || stride == 2), OCNN_E_BADARG, "null child/ichild");
  return run_col2octree<true>(col, data, channel, height, octree_h, kernel_size, stride, neigh, child,
      ichild, height_col, n, dtype, as_stream(stream));
}

int ocnn_octree_max_pool(void* top, int top_h, int* mask, const void* btm, int btm_h, int channel,
    int dtype, ocnn_stream_t stream) {
  int e = check_pool(top, top_h, mask, btm, btm_h, channel, dtype);
  if (e) return e;
  OCNN_REQUIRE((int64_t)top_h * 8 <= btm_h, OCNN_E_SHAPE, "top_h %d * 8 > btm_h %d", top_h, btm_h);
  int64_t total = (int64_t)channel * top_h;
  if (total == 0) return OCNN_OK;
  hipStream_t s = as_stream(stream);
  if (dtype == OCNN_F32)
    max_pool_kernel<float><<<blocks_for(total), kBlock, 0, s>>>((float*)top, top_h, mask, (const float*)btm, btm_h, total);
  else
    max_pool_kernel<uint16_t><<<blocks_for(total), kBlock, 0, s>>>((uint16_t*)top, top_h, mask, (const uint16_t*)btm, btm_h, total);
  OCNN_LAUNCH_OK("max_pool");
  return OCNN_OK;
}

int ocnn_octree_max_unpool(const void* top, int top_h, const int* mask, void* btm, int btm_h,
    int channel, int dtype, ocnn_stream_t stream) {
  int e = check_pool(top, top_h, mask, btm, btm_h, channel, dtype);
  if (e) return e;
  OCNN_REQUIRE((int64_t)top_h * 8 == btm_h, OCNN_E_SHAPE, "btm_h %d != 8 * top_h %d", btm_h, top_h);
  int64_t total = (int64_t)channel * top_h;
  if (total == 0) return OCNN_OK;
  hipStream_t s = as_stream(stream);
  if (dtype == OCNN_F32) {
    max_unpool_kernel<float><<<blocks_for(total), kBlock, 0, s>>>((const float*)top, top_h, mask, (float*)btm, btm_h, total);
    unpool_foreign_kernel<float><<<blocks_for(total), kBlock, 0, s>>>((const float*)top, top_h, mask, (float*)btm, btm_h, total);
  } else {
    max_unpool_kernel<uint16_t><<<blocks_for(total), kBlock, 0, s>>>((const uint16_t*)top, top_h, mask, (uint16_t*)btm, btm_h, total);
    unpool_foreign_kernel<uint16_t><<<blocks_for(total), kBlock, 0, s>>>((const uint16_t*)top, top_h, mask, (uint16_t*)btm, btm_h, total);
  }
  OCNN_LAUNCH_OK("max_unpool");
  return OCNN_OK;
}

int ocnn_octree_mask_pool(void* top, int top_h, const int* mask, const void* btm, int btm_h,
    int channel, int dtype, ocnn_stream_t stream) {
  int e = check_pool(top, top_h, mask, btm, btm_h, channel, dtype);
  if (e) return e;
  int64_t total = (int64_t)channel * top_h;
  if (total == 0) return OCNN_OK;
  hipStream_t s = as_stream(stream);
  if (dtype == OCNN_F32)
    mask_pool_kernel<float><<<blocks_for(total), kBlock, 0, s>>>((float*)top, top_h, mask, (const float*)btm, btm_h, total);
  else
    mask_pool_kernel<uint16_t><<<blocks_for(total), kBlock, 0, s>>>((uint16_t*)top, top_h, mask, (const uint16_t*)btm, btm_h, total);
  OCNN_LAUNCH_OK("mask_pool");
  return OCNN_OK;
}

}  // extern "C"
