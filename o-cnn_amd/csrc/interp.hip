// Feature transfer between octrees and to free points:
//   * octree_align: the features of one octree scattered to the nodes of another with the same
//     keys (align_forward_gpu / align_backward_gpu, octree/octree/octree_nn.cu:710-752, driven as
//     in pytorch/cpp/octree_align.cpp:9-83);
//   * nearest / trilinear interpolation at free points (octree_nearest_pts, octree_trilinear_pts,
//     pytorch/ocnn/modules.py:209-275), fused: the reference builds eight keys per point, searches
//     them, assembles a sparse matrix and multiplies twice; here one kernel does key arithmetic,
//     the eight binary searches and the weights, and a second one the weighted gather.
#include "ocnn_common.h"
#include "scan.h"

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
// btm[c][h] = top[c][index[h]], or zero where the index names no row.  A thread serves one row in
// kAlignChunk channels (blockIdx.y): their loads are issued together and outside any per-lane
// branch (a row without a source reads row 0 and stores zero), so they are all in flight at once.
constexpr int kAlignChunk = 8;
__global__ void align_backward_kernel(const float* __restrict__ top, int top_h, float* __restrict__ btm, int btm_h,
    const int* __restrict__ index, int channel) {
  const int h = blockIdx.x * kBlock + threadIdx.x;
  if (h >= btm_h) return;
  const int c0 = blockIdx.y * kAlignChunk;
  const int j = index[h];
  const bool ok = j >= 0 && j < top_h;
  const int from = ok ? j : 0;
  float v[kAlignChunk];
#pragma unroll
  for (int i = 0; i < kAlignChunk; ++i)
    v[i] = (top_h > 0 && c0 + i < channel) ? top[(int64_t)(c0 + i) * top_h + from] : 0.0f;  // the same for the whole grid row
#pragma unroll
  for (int i = 0; i < kAlignChunk; ++i)
    if (c0 + i < channel) btm[(int64_t)(c0 + i) * btm_h + h] = ok ? v[i] : 0.0f;
}
// top[c][index[h]] += btm[c][h] where the index names a row: the transfer and the sum behind it
// (a skip connection) in one pass.  The rows of top that nothing is moved to are not touched.
__global__ void align_add_kernel(float* __restrict__ top, int top_h, const float* __restrict__ btm, int btm_h,
    const int* __restrict__ index, int channel) {
  const int h = blockIdx.x * kBlock + threadIdx.x;
  if (h >= btm_h) return;
  const int c0 = blockIdx.y * kAlignChunk;
  const int j = index[h];
  const bool ok = j >= 0 && j < top_h;
  const int to = ok ? j : 0;
  float v[kAlignChunk], t[kAlignChunk];
#pragma unroll
  for (int i = 0; i < kAlignChunk; ++i) {
    const bool live = c0 + i < channel;
    v[i] = live ? btm[(int64_t)(c0 + i) * btm_h + h] : 0.0f;
    t[i] = live ? top[(int64_t)(c0 + i) * top_h + to] : 0.0f;
  }
#pragma unroll
  for (int i = 0; i < kAlignChunk; ++i)
    if (ok && c0 + i < channel) top[(int64_t)(c0 + i) * top_h + to] = t[i] + v[i];
}
__global__ void fill_i32_kernel(int* __restrict__ p, int n, int v) {
  const int i = blockIdx.x * kBlock + threadIdx.x;
  if (i < n) p[i] = v;
}
// inverse[index[h]] = h over the valid entries of index; inverse was filled with -1 first
__global__ void align_invert_kernel(int* __restrict__ inverse, int top_h, const int* __restrict__ index, int btm_h) {
  const int h = blockIdx.x * kBlock + threadIdx.x;
  if (h >= btm_h) return;
  const int j = index[h];
  if (j >= 0 && j < top_h) inverse[j] = h;
}
// octree_mask (octree_nn.cu:805-818): the rows whose label equals `mask` become zero.
// One thread per four consecutive rows of one channel where the row count allows.
__global__ void mask_rows_kernel(float* __restrict__ out, const float* __restrict__ in,
    const int* __restrict__ label, int height, int mask, int64_t num) {
  const int h = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
  const int64_t base = (int64_t)blockIdx.y * height + h;
  if (h >= height || base >= num) return;
  if ((height & 3) == 0 && base + 3 < num) {
    const int4 l = *reinterpret_cast<const int4*>(label + h);
    float4 v = *reinterpret_cast<const float4*>(in + base);
    if (l.x == mask) v.x = 0.0f;
    if (l.y == mask) v.y = 0.0f;
    if (l.z == mask) v.z = 0.0f;
    if (l.w == mask) v.w = 0.0f;
    *reinterpret_cast<float4*>(out + base) = v;
  } else {
    for (int j = 0; j < 4 && h + j < height && base + j < num; ++j)
      out[base + j] = label[h + j] == mask ? 0.0f : in[base + j];
  }
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
// nearest: data[c, idx] or 0.  One thread per point, channels in the inner loop.  K is a
// template parameter so that the corner arrays stay in registers (with a run-time bound they
// are indexed dynamically and live in scratch memory: 10x slower).
template <int K>
__global__ void interp_gather_kernel(float* __restrict__ out, const float* __restrict__ data, int channel, int H,
    const int* __restrict__ idx, const float* __restrict__ weight, int n_pts, int normalise) {
  const int p = blockIdx.x * kBlock + threadIdx.x;
  if (p >= n_pts) return;
  int id[K];
  float w[K];
  float norm = 0.0f;
#pragma unroll
  for (int m = 0; m < K; ++m) {
    id[m] = idx[(int64_t)p * K + m];
    w[m] = (id[m] >= 0 && id[m] < H) ? weight[(int64_t)p * K + m] : 0.0f;
    if (id[m] < 0 || id[m] >= H) id[m] = -1;
    norm += w[m];
  }
  const float inv = normalise ? 1.0f / (norm + 1e-10f) : 1.0f;
  for (int c = 0; c < channel; ++c) {
    float acc = 0.0f;
#pragma unroll
    for (int m = 0; m < K; ++m)
      if (id[m] >= 0) acc += w[m] * data[(int64_t)c * H + id[m]];
    out[(int64_t)c * n_pts + p] = acc * inv;
  }
}
// ---- the same gather through a row-major copy of the features ----------------------------------
// In the channel-major tensor the C values of a node are C cache lines apart, so the kernel
// above asks for 8 x C lines per point.  With a workspace the features are first copied
// row-major ([H, Cpad], Cpad = C rounded up to 4): a corner is then one contiguous row, read by
// 16 lanes as 16-byte vectors (two line requests per 64 channels).  The results of 64 points go
// through an LDS tile so that the channel-major output leaves in 256-byte rows.
__global__ void __launch_bounds__(kBlock) rows_copy_kernel(float* __restrict__ xt, const float* __restrict__ data,
    int channel, int H, int cpad) {
  __shared__ float tile[64][65];
  const int h0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    const int c = c0 + i, h = h0 + tx;
    tile[i][tx] = (c < channel && h < H) ? data[(int64_t)c * H + h] : 0.0f;
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int h = h0 + i, c = c0 + tx;
    if (h < H && c < cpad) xt[(int64_t)h * cpad + c] = tile[tx][i];
  }
}

constexpr int kInterpPts = 64;  // points per workgroup
template <int K>
__global__ void __launch_bounds__(kBlock) interp_gather_rows_kernel(float* __restrict__ out,
    const float4* __restrict__ xt, int channel, int cpad4, const int* __restrict__ idx,
    const float* __restrict__ weight, int n_pts, int normalise) {
  __shared__ float tile[64][kInterpPts + 1];  // [channel of the chunk][point]
  const int tid = threadIdx.x;
  const int pl = tid >> 4, cq = tid & 15;     // point inside a pass of 16, 4-channel group
  const int p0 = blockIdx.x * kInterpPts;
  int id[kInterpPts / 16][K];
  float w[kInterpPts / 16][K], inv[kInterpPts / 16];
#pragma unroll
  for (int pass = 0; pass < kInterpPts / 16; ++pass) {
    const int p = p0 + pass * 16 + pl;
    float norm = 0.0f;
#pragma unroll
    for (int m = 0; m < K; ++m) {
      const int v = p < n_pts ? idx[(int64_t)p * K + m] : -1;
      id[pass][m] = v;
      w[pass][m] = v >= 0 ? weight[(int64_t)p * K + m] : 0.0f;
      norm += w[pass][m];
    }
    inv[pass] = normalise ? 1.0f / (norm + 1e-10f) : 1.0f;
  }
  for (int chunk = 0; chunk * 16 < cpad4; ++chunk) {  // 64 channels at a time
    const int q = chunk * 16 + cq;
#pragma unroll
    for (int pass = 0; pass < kInterpPts / 16; ++pass) {
      float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
      if (q < cpad4) {
#pragma unroll
        for (int m = 0; m < K; ++m)
          if (id[pass][m] >= 0) {
            const float4 v = xt[(int64_t)id[pass][m] * cpad4 + q];
            acc.x += w[pass][m] * v.x; acc.y += w[pass][m] * v.y; acc.z += w[pass][m] * v.z; acc.w += w[pass][m] * v.w;
          }
      }
      const int pt = pass * 16 + pl;
      // the sum first, the normalisation once at the end, as the per-channel kernel does
      tile[4 * cq + 0][pt] = acc.x * inv[pass]; tile[4 * cq + 1][pt] = acc.y * inv[pass];
      tile[4 * cq + 2][pt] = acc.z * inv[pass]; tile[4 * cq + 3][pt] = acc.w * inv[pass];
    }
    __syncthreads();
    const int lane = tid & 63, row = tid >> 6;
    for (int c = row; c < 64; c += 4) {
      const int ch = chunk * 64 + c;
      if (ch < channel && p0 + lane < n_pts) out[(int64_t)ch * n_pts + p0 + lane] = tile[c][lane];
    }
    __syncthreads();
  }
}

// The adjoint as a gather.  The (point, corner) pairs are binned by node with a counting sort
// (histogram, prefix sum, fill through a cursor per node), the output gradient is copied
// row-major ([point][channel]: a pair then reads one contiguous row), and every node sums its
// pairs in registers and writes its row once, through an LDS tile so that the channel-major
// result leaves in 256-byte rows.  No floating-point atomics; the order of the pairs of a node
// (and with it the rounding of its sum) follows the order in which the cursor was taken.
__global__ void interp_hist_kernel(int* __restrict__ count, const int* __restrict__ idx, int64_t n, int H) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int id = idx[i];
  if ((unsigned)id < (unsigned)H) atomicAdd(&count[id], 1);
}
__global__ void __launch_bounds__(kBlock) seg_tile_sum_kernel(const int* __restrict__ v, int64_t n, int* __restrict__ tile_sum) {
  const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
  int c = 0;
#pragma unroll
  for (int j = 0; j < kScanItems; ++j) c += base + j < n ? v[base + j] : 0;
  int total;
  block_exclusive_scan(c, &total);
  if (threadIdx.x == 0) tile_sum[blockIdx.x] = total;
}
// v[i] <- sum of v[0..i) (in place)
__global__ void __launch_bounds__(kBlock) seg_exclusive_kernel(int* __restrict__ v, int64_t n, const int* __restrict__ tile_offset) {
  const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
  int x[kScanItems];
  int c = 0;
#pragma unroll
  for (int j = 0; j < kScanItems; ++j) { x[j] = base + j < n ? v[base + j] : 0; c += x[j]; }
  int total;
  int run = tile_offset[blockIdx.x] + block_exclusive_scan(c, &total);
#pragma unroll
  for (int j = 0; j < kScanItems; ++j) {
    if (base + j < n) v[base + j] = run;
    run += x[j];
  }
}
// cursor[id] starts at the first slot of node id and ends at the first slot of node id + 1
template <int K>
__global__ void interp_fill_kernel(int2* __restrict__ pairs, int* __restrict__ cursor, const int* __restrict__ idx,
    const float* __restrict__ weight, int n_pts, int H, int normalise) {
  const int p = blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= n_pts) return;
  int id[K];
  float w[K];
  float norm = 0.0f;
#pragma unroll
  for (int m = 0; m < K; ++m) {
    id[m] = idx[(int64_t)p * K + m];
    w[m] = id[m] >= 0 ? (weight ? weight[(int64_t)p * K + m] : 1.0f) : 0.0f;   // no weights: a plain scatter-add
    norm += w[m];
  }
  const float inv = normalise ? 1.0f / (norm + 1e-10f) : 1.0f;
#pragma unroll
  for (int m = 0; m < K; ++m)
    if ((unsigned)id[m] < (unsigned)H) pairs[atomicAdd(&cursor[id[m]], 1)] = make_int2(p, __float_as_int(w[m] * inv));
}
__global__ void __launch_bounds__(kBlock) interp_reduce_kernel(float* __restrict__ grad_data,
    const float4* __restrict__ rows, const int2* __restrict__ pairs, const int* __restrict__ ends, int channel, int cpad4,
    int H) {
  __shared__ float tile[64][65];   // [node][channel of the chunk]
  const int tid = threadIdx.x;
  const int nl = tid >> 4, cq = tid & 15;
  const int n0 = blockIdx.x * 64;
  const int lane = tid & 63, row = tid >> 6;
  int b[4], e[4];
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    const int node = n0 + pass * 16 + nl;
    b[pass] = (node < H && node > 0) ? ends[node - 1] : 0;
    e[pass] = node < H ? ends[node] : 0;
  }
  for (int chunk = 0; chunk * 16 < cpad4; ++chunk) {
    const int c4 = chunk * 16 + cq;
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
      float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      if (c4 < cpad4) {
        int j = b[pass];
        for (; j + 1 < e[pass]; j += 2) {
          const int2 p0 = pairs[j], p1 = pairs[j + 1];
          const float4 g0 = rows[(int64_t)p0.x * cpad4 + c4], g1 = rows[(int64_t)p1.x * cpad4 + c4];
          const float w0 = __int_as_float(p0.y), w1 = __int_as_float(p1.y);
          acc.x += w0 * g0.x; acc.y += w0 * g0.y; acc.z += w0 * g0.z; acc.w += w0 * g0.w;
          acc.x += w1 * g1.x; acc.y += w1 * g1.y; acc.z += w1 * g1.z; acc.w += w1 * g1.w;
        }
        if (j < e[pass]) {
          const int2 p0 = pairs[j];
          const float4 g0 = rows[(int64_t)p0.x * cpad4 + c4];
          const float w0 = __int_as_float(p0.y);
          acc.x += w0 * g0.x; acc.y += w0 * g0.y; acc.z += w0 * g0.z; acc.w += w0 * g0.w;
        }
      }
      float* t = &tile[pass * 16 + nl][4 * cq];
      t[0] = acc.x; t[1] = acc.y; t[2] = acc.z; t[3] = acc.w;
    }
    __syncthreads();
    for (int c = row; c < 64; c += 4) {
      const int ch = chunk * 64 + c, node = n0 + lane;
      if (ch < channel && node < H) grad_data[(int64_t)ch * H + node] = tile[lane][c];
    }
    __syncthreads();
  }
}

// the adjoint: grad_data[c, idx_m] += w_m / (norm + 1e-10) * grad_out[c, p]
template <int K>
__global__ void interp_scatter_kernel(float* __restrict__ grad_data, const float* __restrict__ grad_out, int channel,
    int H, const int* __restrict__ idx, const float* __restrict__ weight, int n_pts, int normalise) {
  const int p = blockIdx.x * kBlock + threadIdx.x;
  if (p >= n_pts) return;
  int id[K];
  float w[K];
  float norm = 0.0f;
#pragma unroll
  for (int m = 0; m < K; ++m) {
    id[m] = idx[(int64_t)p * K + m];
    const bool ok = id[m] >= 0 && id[m] < H;
    w[m] = ok ? (weight ? weight[(int64_t)p * K + m] : 1.0f) : 0.0f;
    if (!ok) id[m] = -1;
    norm += w[m];
  }
  const float inv = normalise ? 1.0f / (norm + 1e-10f) : 1.0f;
  for (int c = 0; c < channel; ++c) {
    const float g = grad_out[(int64_t)c * n_pts + p] * inv;
#pragma unroll
    for (int m = 0; m < K; ++m)
      if (id[m] >= 0) unsafeAtomicAdd(grad_data + (int64_t)c * H + id[m], w[m] * g);
  }
}

// workspace of the gathered adjoint: segment ends, (point, weight) pairs, row-major output
// gradient, tile sums of the prefix scan
struct InterpBackLayout {
  size_t ends, pairs, rows, scan, total;
  InterpBackLayout(int channel, int H, int n_pts, int K) {
    auto al = [](size_t v) { return (v + 255) & ~(size_t)255; };
    size_t off = 0;
    ends = off; off += al(sizeof(int) * ((size_t)H + 1));
    pairs = off; off += al(sizeof(int2) * (size_t)n_pts * K);
    rows = off; off += al(sizeof(float) * (size_t)n_pts * ((channel + 3) / 4 * 4));
    scan = off; off += al(scan_scratch_bytes(H));
    total = off;
  }
};

}  // namespace
}  // namespace ocnn

namespace ocnn {
namespace {
int scatter_add_rows(float* grad_data, const float* grad_out, int channel, int H, int n_pts, int method,
    const int* idx, const float* weight, void* workspace_dev, size_t workspace_bytes, hipStream_t s);
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

int ocnn_align_forward_ws(float* top, int top_h, int channel, const float* btm, int btm_h, const int* idx,
    int* inverse_ws, ocnn_stream_t stream) {
  OCNN_REQUIRE(top && btm && idx && inverse_ws && top_h >= 0 && btm_h >= 0 && channel > 0, OCNN_E_BADARG,
      "bad argument");
  hipStream_t s = as_stream(stream);
  if (top_h == 0) return OCNN_OK;
  // Every row of top is written once, by the thread of that row: its source row through the
  // inverted index, or zero.  (The scatter form writes top twice, the zeros and the rows.)
  fill_i32_kernel<<<blocks_for(top_h), kBlock, 0, s>>>(inverse_ws, top_h, -1);
  if (btm_h > 0) align_invert_kernel<<<blocks_for(btm_h), kBlock, 0, s>>>(inverse_ws, top_h, idx, btm_h);
  align_backward_kernel<<<dim3(blocks_for(top_h), (channel + kAlignChunk - 1) / kAlignChunk), kBlock, 0, s>>>(
      btm, btm_h, top, top_h, inverse_ws, channel);
  OCNN_LAUNCH_OK("align_forward_ws");
  return OCNN_OK;
}

int ocnn_align_forward_add(float* top, int top_h, int channel, const float* btm, int btm_h, const int* idx,
    ocnn_stream_t stream) {
  OCNN_REQUIRE(top && btm && idx && top_h >= 0 && btm_h >= 0 && channel > 0, OCNN_E_BADARG, "bad argument");
  if (top_h > 0 && btm_h > 0)
    align_add_kernel<<<dim3(blocks_for(btm_h), (channel + kAlignChunk - 1) / kAlignChunk), kBlock, 0,
        as_stream(stream)>>>(top, top_h, btm, btm_h, idx, channel);
  OCNN_LAUNCH_OK("align_forward_add");
  return OCNN_OK;
}

int ocnn_align_backward(const float* top, int top_h, int channel, float* btm, int btm_h, const int* idx,
    ocnn_stream_t stream) {
  OCNN_REQUIRE(top && btm && idx && top_h >= 0 && btm_h >= 0 && channel > 0, OCNN_E_BADARG, "bad argument");
  if (btm_h > 0)
    align_backward_kernel<<<dim3(blocks_for(btm_h), (channel + kAlignChunk - 1) / kAlignChunk), kBlock, 0,
        as_stream(stream)>>>(top, top_h, btm, btm_h, idx, channel);
  OCNN_LAUNCH_OK("align_backward");
  return OCNN_OK;
}

size_t ocnn_octree_interp_workspace_bytes(int channel, int H) {
  if (channel <= 0 || H <= 0) return 0;
  return ((size_t)H * (size_t)((channel + 3) / 4 * 4) * sizeof(float) + 255) & ~(size_t)255;
}

size_t ocnn_octree_interp_backward_workspace_bytes(int channel, int H, int n_pts, int method) {
  if (channel <= 0 || H <= 0 || n_pts <= 0 || (method != 0 && method != 1)) return 0;
  return InterpBackLayout(channel, H, n_pts, method == 0 ? 1 : 8).total;
}

int ocnn_octree_interp(float* out, const float* data, int channel, int H, const uint64_t* key, int n_key,
    const float* pts, int n_pts, int depth, int method, int* idx, float* weight, ocnn_stream_t stream) {
  return ocnn_octree_interp_ws(out, data, channel, H, key, n_key, pts, n_pts, depth, method, idx, weight, nullptr, 0,
      stream);
}

int ocnn_octree_interp_ws(float* out, const float* data, int channel, int H, const uint64_t* key, int n_key,
    const float* pts, int n_pts, int depth, int method, int* idx, float* weight, void* workspace_dev,
    size_t workspace_bytes, ocnn_stream_t stream) {
  OCNN_REQUIRE(out && data && pts && idx && weight && (key || n_key == 0), OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(channel > 0 && H >= 0 && n_key >= 0 && n_pts >= 0 && depth >= 0 && depth <= 16, OCNN_E_BADARG,
      "bad argument");
  OCNN_REQUIRE(method == 0 || method == 1, OCNN_E_BADARG, "method %d is neither nearest (0) nor linear (1)", method);
  if (n_pts == 0) return OCNN_OK;
  hipStream_t s = as_stream(stream);
  const int K = method == 0 ? 1 : 8;
  interp_index_kernel<<<blocks_for((int64_t)n_pts * K), kBlock, 0, s>>>(idx, weight, pts, n_pts, key, n_key, depth, K);
  OCNN_LAUNCH_OK("interp_index");
  // the row-major copy pays once the points ask for more rows than the level has
  const bool rows = workspace_dev && H > 0 && workspace_bytes >= ocnn_octree_interp_workspace_bytes(channel, H) &&
      (reinterpret_cast<uintptr_t>(workspace_dev) & 15) == 0 && (int64_t)n_pts * K >= H / 2;
  if (rows) {
    const int cpad = (channel + 3) / 4 * 4;
    float* xt = static_cast<float*>(workspace_dev);
    rows_copy_kernel<<<dim3(blocks_for(H, 64), blocks_for(cpad, 64)), kBlock, 0, s>>>(xt, data, channel, H, cpad);
    OCNN_LAUNCH_OK("rows_copy");
    if (K == 1)
      interp_gather_rows_kernel<1><<<blocks_for(n_pts, kInterpPts), kBlock, 0, s>>>(out, (const float4*)xt, channel,
          cpad / 4, idx, weight, n_pts, method);
    else
      interp_gather_rows_kernel<8><<<blocks_for(n_pts, kInterpPts), kBlock, 0, s>>>(out, (const float4*)xt, channel,
          cpad / 4, idx, weight, n_pts, method);
  } else if (K == 1) {
    interp_gather_kernel<1><<<blocks_for(n_pts), kBlock, 0, s>>>(out, data, channel, H, idx, weight, n_pts, method);
  } else {
    interp_gather_kernel<8><<<blocks_for(n_pts), kBlock, 0, s>>>(out, data, channel, H, idx, weight, n_pts, method);
  }
  OCNN_LAUNCH_OK("interp_gather");
  return OCNN_OK;
}

int ocnn_octree_interp_backward(float* grad_data, const float* grad_out, int channel, int H, int n_pts, int method,
    const int* idx, const float* weight, ocnn_stream_t stream) {
  return ocnn_octree_interp_backward_ws(grad_data, grad_out, channel, H, n_pts, method, idx, weight, nullptr, 0, stream);
}

int ocnn_octree_interp_backward_ws(float* grad_data, const float* grad_out, int channel, int H, int n_pts, int method,
    const int* idx, const float* weight, void* workspace_dev, size_t workspace_bytes, ocnn_stream_t stream) {
  OCNN_REQUIRE(weight, OCNN_E_BADARG, "null weights");
  return scatter_add_rows(grad_data, grad_out, channel, H, n_pts, method, idx, weight, workspace_dev, workspace_bytes,
      as_stream(stream));
}

// ---- octree_gather / octree_gatherbk / octree_mask (octree/octree/octree_nn.h:204-218) -------
int ocnn_octree_gather(void* top, int top_h, int channel, const void* btm, int btm_h, const int* idx, int dtype,
    ocnn_stream_t stream) {
  // the reference's own definition: pad_forward with the value 0 (octree_nn.cu:770-773)
  return ocnn_pad_forward(top, top_h, channel, btm, btm_h, idx, 0.0f, dtype, stream);
}

size_t ocnn_octree_gatherbk_workspace_bytes(int channel, int btm_h, int top_h) {
  return ocnn_octree_interp_backward_workspace_bytes(channel, btm_h, top_h, 0);
}

int ocnn_octree_gatherbk(const float* top, int top_h, int channel, float* btm, int btm_h, const int* idx,
    void* workspace_dev, size_t workspace_bytes, ocnn_stream_t stream) {
  // btm[c, idx[h]] += top[c, h] over all h with idx[h] != -1, btm zero-filled first
  // (octree_nn.cu:782-801).  With a workspace the rows are binned by target and every target sums
  // its sources (no floating-point atomics); without one, or for few rows, an atomic scatter.
  return scatter_add_rows(btm, top, channel, btm_h, top_h, 0, idx, nullptr, workspace_dev, workspace_bytes,
      as_stream(stream));
}

int ocnn_octree_mask(float* out, const float* in, const int* label, int height, int mask, int64_t num,
    ocnn_stream_t stream) {
  OCNN_REQUIRE(out && in && label && height > 0 && num >= 0, OCNN_E_BADARG, "bad argument");
  if (num > 0) {
    const int64_t rows = (num + height - 1) / height;
    OCNN_REQUIRE(rows <= 65535, OCNN_E_BADARG, "more than 65535 channels");
    mask_rows_kernel<<<dim3(blocks_for((height + 3) / 4), (unsigned)rows), kBlock, 0, as_stream(stream)>>>(out, in, label,
        height, mask, num);
  }
  OCNN_LAUNCH_OK("octree_mask");
  return OCNN_OK;
}

}  // extern "C"

namespace ocnn {
namespace {

// grad_data[c, idx[p, m]] += w[p, m] * grad_out[c, p] (grad_data zero-filled first): the adjoint
// of the interpolation and, with unit weights (weight == nullptr), of octree_gather.
int scatter_add_rows(float* grad_data, const float* grad_out, int channel, int H, int n_pts, int method,
    const int* idx, const float* weight, void* workspace_dev, size_t workspace_bytes, hipStream_t s) {
  OCNN_REQUIRE(grad_data && grad_out && idx && channel > 0 && H >= 0 && n_pts >= 0, OCNN_E_BADARG,
      "bad argument");
  OCNN_REQUIRE(method == 0 || method == 1, OCNN_E_BADARG, "method %d", method);
  const int Kc = method == 0 ? 1 : 8;
  const size_t need = ocnn_octree_interp_backward_workspace_bytes(channel, H, n_pts, method);
  if (workspace_dev && H > 0 && n_pts > 0 && need > 0 && workspace_bytes >= need &&
      (reinterpret_cast<uintptr_t>(workspace_dev) & 15) == 0 && (int64_t)n_pts * Kc >= H / 2) {
    const int cpad = (channel + 3) / 4 * 4;
    const InterpBackLayout L(channel, H, n_pts, Kc);
    char* ws = static_cast<char*>(workspace_dev);
    int* ends = reinterpret_cast<int*>(ws + L.ends);
    int2* pairs = reinterpret_cast<int2*>(ws + L.pairs);
    float* rows = reinterpret_cast<float*>(ws + L.rows);
    int* tiles = reinterpret_cast<int*>(ws + L.scan);
    const int64_t n_pairs = (int64_t)n_pts * Kc;
    zero_kernel<<<blocks_for(H), kBlock, 0, s>>>(reinterpret_cast<float*>(ends), H);
    interp_hist_kernel<<<blocks_for(n_pairs), kBlock, 0, s>>>(ends, idx, n_pairs, H);
    const int n_tiles = scan_tiles(H);
    seg_tile_sum_kernel<<<n_tiles, kBlock, 0, s>>>(ends, H, tiles);
    scan_tiles_kernel<0><<<1, kBlock, 0, s>>>(tiles, n_tiles, nullptr);
    seg_exclusive_kernel<<<n_tiles, kBlock, 0, s>>>(ends, H, tiles);
    if (Kc == 1) interp_fill_kernel<1><<<blocks_for(n_pts), kBlock, 0, s>>>(pairs, ends, idx, weight, n_pts, H, method);
    else interp_fill_kernel<8><<<blocks_for(n_pts), kBlock, 0, s>>>(pairs, ends, idx, weight, n_pts, H, method);
    rows_copy_kernel<<<dim3(blocks_for(n_pts, 64), blocks_for(cpad, 64)), kBlock, 0, s>>>(rows, grad_out, channel, n_pts, cpad);
    interp_reduce_kernel<<<blocks_for(H, 64), kBlock, 0, s>>>(grad_data, reinterpret_cast<const float4*>(rows), pairs, ends,
        channel, cpad / 4, H);
    OCNN_LAUNCH_OK("interp_reduce");
    return OCNN_OK;
  }
  const int64_t n = (int64_t)H * channel;
  if (n > 0) zero_kernel<<<blocks_for(n), kBlock, 0, s>>>(grad_data, n);
  if (n_pts > 0) {
    if (method == 0)
      interp_scatter_kernel<1><<<blocks_for(n_pts), kBlock, 0, s>>>(grad_data, grad_out, channel, H, idx, weight, n_pts, method);
    else
      interp_scatter_kernel<8><<<blocks_for(n_pts), kBlock, 0, s>>>(grad_data, grad_out, channel, H, idx, weight, n_pts, method);
  }
  OCNN_LAUNCH_OK("interp_scatter");
  return OCNN_OK;
}

}  // namespace
}  // namespace ocnn
