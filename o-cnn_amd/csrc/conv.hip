// Octree convolution / deconvolution as an implicit GEMM on the CDNA4 matrix
// cores.  The reference computes  top = W[Co, Ci*K] x octree2col(btm)[Ci*K, H]
// through a column buffer in HBM (octree/octree/octree_conv.cpp:276-325); here
// the gather through the neighbour table feeds MFMA operands directly:
//
//   out[m, n] = sum_{tap k} sum_{c}  A[k][m][c] * in[c, src(n, k)]
//
// One wavefront owns 64 output columns (two 32-wide MFMA column tiles) and all
// output channels (MT row tiles of 32 per pass).  For every tap it looks up the
// source row of its columns once, then walks the input channels feeding
// v_mfma_f32_32x32x2_f32 (fp32) or v_mfma_f32_32x32x16_bf16 (bf16 storage, fp32
// accumulate).  Weights are re-laid out once per call into MFMA A-fragment
// order so that each fragment is one coalesced 256-byte (fp32) or 1-KiB (bf16)
// load shared by all wavefronts through the vector L1.
#include "ocnn_common.h"

#include <atomic>
#include <mutex>
#include <type_traits>

namespace ocnn {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));  // one 16-byte LDS / global unit

enum { kModeS1 = 0, kModeS2Conv = 1, kModeS2Deconv = 2, kModeS2DeconvAny = 3 };

struct ConvArgs {
  int M, Cin, N, K;     // output channels, input channels, output columns, taps
  int Hin, Hout;        // row lengths of the input / output tensors
  int mode, nempty;
  int mtiles;           // ceil(M / 32)
  int csteps;           // channel steps per tap: ceil(Cin/2) fp32, ceil(Cin/16) bf16
  int slot[27];         // neighbour slot of tap k for sibling 0
  const int* neigh;
  const int* child;
  const int* ichild;
  const float* bias;    // optional per-output-channel bias (fp32), added before the store
  int relu;             // optional max(., 0) before the store
  // optional: the source rows of every (tap, column), made ahead of the convolution by
  // conv_sources_kernel: table[k * src_pitch + column] = row, -1 for none
  const int* src_table = nullptr;
  int src_pitch = 0;
};

// epilogue shared by every kernel: bias and ReLU are applied to the fp32 accumulator
__device__ inline float finish(const ConvArgs& a, float v, int m) {
  if (a.bias) v += a.bias[m];
  if (a.relu) v = fmaxf(v, 0.0f);
  return v;
}

constexpr int kWaveCols = 64;                 // output columns per wavefront
constexpr int kConvWaves = 4;                 // wavefronts per workgroup
constexpr int kTileCols = kWaveCols * kConvWaves;

// Stride-2 deconvolution with any tap set, seen from an output node.  Column h (a sibling
// group of the output level, i.e. a non-empty node of the input level) scatters through tap
// t to the node at offset t - 1 from its first sibling (col2octree, octree_nn.cpp:216-241).
// Per axis a node with sibling bit s is reached from its own group by tap s + 1, and, when
// s = 1, from the group two cells further by tap 0; any other tap does not reach it.  The
// first sibling of that other group sits in the node's own 4x4x4 block at coordinate 3.
__device__ inline int deconv_s2_source(const int* __restrict__ neigh, int node, int tap_slot_k) {
  const int s = node & 7;
  int slot = 0;
#pragma unroll
  for (int axis = 0; axis < 3; ++axis) {
    const int t = (tap_slot_k >> (4 - 2 * axis)) & 3, sb = (s >> (2 - axis)) & 1;
    int c;
    if (t == sb + 1) c = 1;
    else if (sb == 1 && t == 0) c = 3;
    else return -1;
    slot = (slot << 2) | c;
  }
  const int q = neigh[((int64_t)(node >> 3) << 6) + slot];
  return q >= 0 ? q >> 3 : -1;
}

// source row of output column n for tap k (-1: contributes zero)
__device__ inline int conv_src(const ConvArgs& a, int n, int k) {
  if (n >= a.N) return -1;
  int p;
  if (a.mode == kModeS2DeconvAny) {
    p = deconv_s2_source(a.neigh, a.nempty ? a.ichild[n] : n, a.slot[k]);
  } else if (a.mode == kModeS1) {
    int node = a.nempty ? a.ichild[n] : n;
    p = a.neigh[((int64_t)(node >> 3) << 6) + sibling_slot(node & 7) + a.slot[k]];
    if (a.nempty && p >= 0) p = a.child[p];
  } else if (a.mode == kModeS2Conv) {
    p = a.neigh[((int64_t)n << 6) + a.slot[k]];
    if (a.nempty && p >= 0) p = a.child[p];
  } else {
    int node = a.nempty ? a.ichild[n] : n;
    p = (k == (node & 7)) ? (node >> 3) : -1;
  }
  return (p >= 0 && p < a.Hin) ? p : -1;
}

// XCD-aware tile order: consecutive workgroup ids land on different XCDs, so give
// each XCD one contiguous range of column tiles (neighbouring tiles share
// neighbour rows, which then stay in that XCD's L2).
__device__ inline int xcd_tile(int bid, int n_tiles) {
  constexpr int kXcd = 8;
  int per = (n_tiles + kXcd - 1) / kXcd;
  return (bid % kXcd) * per + bid / kXcd;
}

// A level with few column tiles cannot fill the device by tiles alone: the passes over the
// output channels (independent of one another) are then dealt out over blockIdx.y, enough of them
// for 768 workgroups (two or three on each of 256 CUs).  That choice stands unless another split
// leaves the most loaded compute unit with strictly less work: with `split` workgroups a tile, each
// doing ceil(npass / split) passes, a unit holds ceil(n_tiles * split / 256) of them.  773 tiles
// of two passes (depth 7 of the scene, 128 output channels in fp32): some units hold 4 workgroups
// of 2 passes (8) against 7 of one pass: 256 -> 128 channels 3.49 -> 2.99 ms, 128 -> 128 1.74 ->
// 1.50 ms.
inline int pass_split(int n_tiles, int npass) {
  constexpr int kWanted = 768, kUnits = 256;
  if (npass <= 1) return 1;
  auto load = [&](int split) {
    return (((int64_t)n_tiles * split + kUnits - 1) / kUnits) * ((npass + split - 1) / split);
  };
  int best = 1;
  if (n_tiles < kWanted) {
    const int p = (kWanted + n_tiles - 1) / n_tiles;
    best = p < npass ? p : npass;
  }
  int64_t best_load = load(best);
  for (int split = 1; split <= npass; ++split)
    if (load(split) < best_load) { best_load = load(split); best = split; }
  return best;
}

// For a kernel that keeps its input columns in registers over all passes (every further workgroup of
// a tile reads them again): more workgroups a tile only where that takes a tenth or more off the
// most loaded unit's work.
inline int pass_split_costly(int n_tiles, int npass) {
  constexpr int kUnits = 256;
  auto load = [&](int split) {
    return (((int64_t)n_tiles * split + kUnits - 1) / kUnits) * ((npass + split - 1) / split);
  };
  int best = 1;
  for (int split = 2; split <= npass; ++split)
    if (load(split) * 10 <= load(best) * 9) best = split;
  return best;
}

// Wavefronts per workgroup (64 columns each) of a kernel whose wavefronts share nothing but a table:
// a level of a few hundred 256-column tiles leaves some compute units with two workgroups and others
// with one (363 tiles on 256 units: the launch lasts as long as two), and smaller workgroups spread
// evenly.  The pick is the size whose most loaded unit holds the fewest wavefronts' work; on a tie
// the larger (neighbouring columns share rows and the weights in the L1).  Measured at depth 7 of
// the scene (92 723 columns): 256 -> 128 channels 0.248 -> 0.202 ms, 128 -> 128 0.131 -> 0.107 ms.
inline int direct_waves(int cols, int npass) {
  constexpr int kUnits = 256;   // compute units of the device
  int best = kConvWaves;
  int64_t best_load = INT64_MAX;
  for (int w = kConvWaves; w >= 1; w >>= 1) {
    const int tiles = (cols + kWaveCols * w - 1) / (kWaveCols * w);
    const int split = pass_split(tiles, npass);
    const int64_t load = (((int64_t)tiles * split + kUnits - 1) / kUnits) * w * ((npass + split - 1) / split);
    if (load < best_load) { best_load = load; best = w; }
  }
  return best;
}

// ---- main kernels ----------------------------------------------------------------
// Accumulator layout of the 32x32 MFMA: lane l, register i holds
// D[row = 8*(i/4) + 4*(l>>5) + (i%4)][col = l&31].
template <typename OutT, int MT>
__device__ inline void store_tiles(const ConvArgs& a, OutT* __restrict__ out, floatx16 (&acc)[MT][2],
    int mt0, int n0, int lane) {
  const int r = lane & 31, kh = lane >> 5;
  if (sizeof(OutT) == 2 && (a.Hout & 1) == 0 && (a.N & 1) == 0 && (reinterpret_cast<uintptr_t>(out) & 3) == 0) {
    // bf16 with an even row length: neighbouring lanes (columns n, n + 1) swap one value of each
    // channel pair (m, m + 1), so the even lane stores both columns of channel m and the odd lane
    // both columns of channel m + 1 as one aligned word: half the store instructions
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        const int n = n0 + nt * 32 + r;           // N is even: a column and its partner exist together
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          const int m = (mt0 + mt) * 32 + 8 * (i / 4) + 4 * kh + (i % 4);
          const float v0 = finish(a, acc[mt][nt][i], min(m, a.M - 1));
          const float v1 = finish(a, acc[mt][nt][i + 1], min(m + 1, a.M - 1));
          const uint32_t mine = (r & 1) ? f32_to_bf16(v1) : f32_to_bf16(v0);
          const uint32_t send = (r & 1) ? f32_to_bf16(v0) : f32_to_bf16(v1);
          const uint32_t got = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send, 0xB1, 0xf, 0xf, true);  // lane ^ 1
          const int mm = m + (r & 1);
          if (n < a.N && mm < a.M)
            *reinterpret_cast<uint32_t*>(reinterpret_cast<uint16_t*>(out) + (int64_t)mm * a.Hout + (n & ~1)) =
                (r & 1) ? (got | (mine << 16)) : (mine | (got << 16));
        }
      }
    return;
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      int n = n0 + nt * 32 + r;
      if (n >= a.N) continue;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        int m = (mt0 + mt) * 32 + 8 * (i / 4) + 4 * kh + (i % 4);
        if (m < a.M) {
          const float v = finish(a, acc[mt][nt][i], m);
          if (sizeof(OutT) == 4) reinterpret_cast<float*>(out)[(int64_t)m * a.Hout + n] = v;
          else reinterpret_cast<uint16_t*>(out)[(int64_t)m * a.Hout + n] = f32_to_bf16(v);
        }
      }
    }
}

// ---- one tap, stride 1 (1x1x1): no neighbours --------------------------------------------------
// out[m][n] = sum over c of W(m, c) x[c][n]: the product of two matrices on the channel-major
// tensor as it lies (lanes 0 .. 31 read 32 consecutive columns of channel c, lanes 32 .. 63 of
// channel c + 1: the B operand of one k-step), bound by the bytes of x and out.  The weights of a
// chunk of channels wait in LDS in A-fragment order.
constexpr int kOneTapChunk = 128;   // channels per LDS stage
template <int MT>
__global__ __launch_bounds__(256) void conv_one_tap_f32_kernel(ConvArgs a, float* __restrict__ out,
    const float* __restrict__ in, const float* __restrict__ W, int64_t sm, int64_t sc, int n_tiles) {
  __shared__ float sW[(kOneTapChunk / 2) * MT * 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = xcd_tile(blockIdx.x, n_tiles);
  if (tile >= n_tiles) return;
  const int n0 = tile * kTileCols + wave * kWaveCols;
  const int r = lane & 31, kh = lane >> 5;
  const int npass = (a.mtiles + MT - 1) / MT;
  // columns past the end read the last column (their results are not stored)
  const float* x0 = in + min(n0 + r, a.N - 1);
  const float* x1 = in + min(n0 + 32 + r, a.N - 1);
  for (int pass = blockIdx.y; pass < npass; pass += gridDim.y) {
    floatx16 acc[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.0f;
    for (int c0 = 0; c0 < a.Cin; c0 += kOneTapChunk) {
      const int nks = (min(kOneTapChunk, a.Cin - c0) + 1) >> 1;
      __syncthreads();   // the previous chunk's fragments are no longer read
      for (int e = threadIdx.x; e < nks * MT * 64; e += 256) {
        const int l = e & 63, mt = (e >> 6) % MT, ks = (e >> 6) / MT;
        const int m = (pass * MT + mt) * 32 + (l & 31), c = c0 + 2 * ks + (l >> 5);
        sW[e] = (m < a.M && c < a.Cin) ? W[m * sm + c * sc] : 0.0f;
      }
      __syncthreads();
      constexpr int kAhead = 8;   // k-steps whose operands are requested together
      for (int k0 = 0; k0 < nks; k0 += kAhead) {
        float b0[kAhead], b1[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
          const int c = c0 + 2 * (k0 + u) + kh;
          const int64_t row = (int64_t)min(c, a.Cin - 1) * a.Hin;
          b0[u] = x0[row];
          b1[u] = x1[row];
          if (c >= a.Cin || k0 + u >= nks) { b0[u] = 0.0f; b1[u] = 0.0f; }   // (an odd channel count: the weight there is zero too)
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
          if (k0 + u >= nks) break;   // uniform
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            const float av = sW[((k0 + u) * MT + mt) * 64 + lane];
            acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, b0[u], acc[mt][0], 0, 0, 0);
            acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, b1[u], acc[mt][1], 0, 0, 0);
          }
        }
      }
    }
    if (n0 < a.N) store_tiles<float, MT>(a, out, acc, pass * MT, n0, lane);
  }
}

// ---- two 1x1x1 convolutions in a row (a prediction head) ----------------------------------------
// hidden = relu(W1 x + b1) (at most 32 channels: one accumulator tile per 32 columns), out = W2 hidden
// + b2 (at most kPairMaxOut channels), optionally label = argmax over the channels of out.  The
// first product is the kernel above; the hidden channels never leave the registers: a lane holds
// 16 of the 32 hidden values of its column, multiplies them with the matching 16 weights of every
// output channel and adds the other half from its partner lane.  Bound by the bytes of x.
constexpr int kPairMaxOut = 8;
__global__ __launch_bounds__(256) void conv_one_tap_pair_f32_kernel(float* __restrict__ out, int* __restrict__ label,
    const float* __restrict__ in, const float* __restrict__ W1, const float* __restrict__ b1,
    const float* __restrict__ W2, const float* __restrict__ b2, int C, int H, int hidden, int relu1, int M2,
    int n_tiles) {
  __shared__ float sW[(kOneTapChunk / 2) * 64];
  __shared__ float sW2[kPairMaxOut][32];
  __shared__ float sB1[32];
  __shared__ float sB2[kPairMaxOut];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = xcd_tile(blockIdx.x, n_tiles);
  if (tile >= n_tiles) return;
  const int n0 = tile * kTileCols + wave * kWaveCols;
  const int r = lane & 31, kh = lane >> 5;
  const float* x0 = in + min(n0 + r, H - 1);
  const float* x1 = in + min(n0 + 32 + r, H - 1);
  {  // (read behind the first barrier of the chunk loop)
    const int j = threadIdx.x >> 5, m = threadIdx.x & 31;
    sW2[j][m] = (j < M2 && m < hidden) ? W2[j * hidden + m] : 0.0f;
    if (threadIdx.x < 32) sB1[threadIdx.x] = (b1 && (int)threadIdx.x < hidden) ? b1[threadIdx.x] : 0.0f;
    if (threadIdx.x < kPairMaxOut) sB2[threadIdx.x] = (b2 && (int)threadIdx.x < M2) ? b2[threadIdx.x] : 0.0f;
  }
  floatx16 acc[2];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[nt][i] = 0.0f;
  for (int c0 = 0; c0 < C; c0 += kOneTapChunk) {
    const int nks = (min(kOneTapChunk, C - c0) + 1) >> 1;
    __syncthreads();   // the previous chunk's fragments are no longer read
    for (int e = threadIdx.x; e < nks * 64; e += 256) {
      const int l = e & 63, ks = e >> 6;
      const int m = l & 31, c = c0 + 2 * ks + (l >> 5);
      sW[e] = (m < hidden && c < C) ? W1[(int64_t)m * C + c] : 0.0f;
    }
    __syncthreads();
    constexpr int kAhead = 8;   // k-steps whose operands are requested together
    for (int k0 = 0; k0 < nks; k0 += kAhead) {
      float v0[kAhead], v1[kAhead];
#pragma unroll
      for (int u = 0; u < kAhead; ++u) {
        const int c = c0 + 2 * (k0 + u) + kh;
        const int64_t row = (int64_t)min(c, C - 1) * H;
        v0[u] = x0[row];
        v1[u] = x1[row];
        if (c >= C || k0 + u >= nks) { v0[u] = 0.0f; v1[u] = 0.0f; }
      }
#pragma unroll
      for (int u = 0; u < kAhead; ++u) {
        if (k0 + u >= nks) break;   // uniform
        const float av = sW[(k0 + u) * 64 + lane];
        acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, v0[u], acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, v1[u], acc[1], 0, 0, 0);
      }
    }
  }
  const float floor = relu1 ? 0.0f : -__builtin_inff();
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
    const int col = n0 + nt * 32 + r;
    float hval[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int m = 8 * (i / 4) + 4 * kh + (i % 4);   // the hidden channel of accumulator element i
      hval[i] = fmaxf(acc[nt][i] + sB1[m], floor);
    }
    float best = 0.0f;
    int arg = 0;
#pragma unroll
    for (int j = 0; j < kPairMaxOut; ++j) {
      if (j >= M2) break;   // uniform
      float p = 0.0f;
#pragma unroll
      for (int i = 0; i < 16; ++i) p += sW2[j][8 * (i / 4) + 4 * kh + (i % 4)] * hval[i];
      p += __shfl_xor(p, 32, 64);
      p += sB2[j];
      if (col < H && kh == (j & 1)) out[(int64_t)j * H + col] = p;
      if (j == 0 || p > best) { best = p; arg = j; }   // the first of equal maxima, as torch.argmax
    }
    if (label && kh == 0 && col < H) label[col] = arg;
  }
}

// ---- general gather kernel over a row-major copy of the input -------------------------------
// Every case without a dedicated kernel (non-empty-node convolutions, the small kernel shapes,
// stride-2 cases other than 2x2x2 over all nodes) runs here.  The input is first copied
// row-major ([H + 1, Cpad], row H zero = missing neighbour), so that the source row of a column
// is contiguous over channels and one 16-byte load per lane brings 4 (fp32) or 8 (bf16) input
// channels: 4x / 8x fewer gather instructions than per-channel gathers from the channel-major
// tensor, which is what bounds this kernel.  Lane (n, kh) loads channels 4kh..4kh+3 of an
// 8-channel group and the four values feed four MFMA k-steps with k-pairs (j, 4+j).
// Loop nest: pass over 32*MT output rows -> tap -> 64-channel slab (its weights staged in LDS
// in A-fragment order, next slab prefetched) -> 8-channel group.
constexpr int kRowSlab = 64;    // channels per stage of the bf16 row kernel
constexpr int kRowSlabF = 32;   // ... of the fp32 row kernel: with 64 the weights on their way to LDS no longer fit the
                                // register file next to the gathers of the next stage and travel through scratch memory
                                // (a wait for every weight load as soon as it is issued, every stage)

__global__ __launch_bounds__(256) void transpose_rows_f32_kernel(float* __restrict__ dst,
    const float* __restrict__ src, int C, int H, int Cpad) {
  __shared__ float tile[64][65];
  const int h0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    int c = c0 + i, h = h0 + tx;
    tile[i][tx] = (c < C && h < H) ? src[(int64_t)c * H + h] : 0.0f;
  }
  __syncthreads();
  const int cq = threadIdx.x & 15, hh = threadIdx.x >> 4;  // 16 lanes x float4 = one 64-channel row
  if (c0 + cq * 4 >= Cpad) return;
  for (int i = hh; i < 64; i += 16) {
    int h = h0 + i;
    if (h > H) continue;
    float4 v = h < H ? make_float4(tile[cq * 4][i], tile[cq * 4 + 1][i], tile[cq * 4 + 2][i], tile[cq * 4 + 3][i])
                     : make_float4(0.f, 0.f, 0.f, 0.f);
    *reinterpret_cast<float4*>(dst + (int64_t)h * Cpad + c0 + cq * 4) = v;
  }
}

// Source rows of one output column for all taps (-1: contributes zero), handed to `put(tap, row)`.
// Stride-1 modes: three dependent trips for all taps together -- the node, its neighbours (all in
// the 256-byte block of the node's sibling group), their ranks among the non-empty nodes.
template <class Put>
__device__ inline void lookup_sources(const ConvArgs& a, int col, Put put) {
  if (a.mode == kModeS1) {
    const bool mine = col < a.N;
    const int node = mine ? (a.nempty ? a.ichild[col] : col) : 0;
    const int* __restrict__ block = a.neigh + ((int64_t)(node >> 3) << 6) + sibling_slot(node & 7);
    int nb[27];
#pragma unroll
    for (int k = 0; k < 27; ++k) nb[k] = (mine && k < a.K) ? block[a.slot[k]] : -1;
    if (a.nempty) {
      int rank[27];
#pragma unroll
      for (int k = 0; k < 27; ++k) rank[k] = a.child[max(nb[k], 0)];
#pragma unroll
      for (int k = 0; k < 27; ++k) nb[k] = nb[k] >= 0 ? rank[k] : -1;
    }
#pragma unroll
    for (int k = 0; k < 27; ++k) put(k, (nb[k] >= 0 && nb[k] < a.Hin) ? nb[k] : -1);
  } else {
#pragma unroll
    for (int k = 0; k < 27; ++k) put(k, k < a.K ? conv_src(a, col, k) : -1);
  }
}

// The source rows of all taps of all columns, one thread a column, into table[27][pitch].  Inside
// a convolution kernel the look-up is two or three dependent trips to memory per tile in front of
// everything else, run by the two or three workgroups that fit a compute unit beside their
// accumulators (about 10 of the 40 microseconds a 256-column tile of a 64 -> 64 bf16 convolution over
// the non-empty nodes lives).  The table depends on the octree level and the kernel shape only: a
// caller that convolves the same level again (the other layers of that depth) makes it once.
__global__ __launch_bounds__(kBlock) void conv_sources_kernel(ConvArgs a, int* __restrict__ table, int pitch) {
  const int col = blockIdx.x * kBlock + threadIdx.x;
  if (col >= pitch) return;
  lookup_sources(a, col, [&](int k, int row) { table[(int64_t)k * pitch + col] = row; });
}
// a tile's part of the table, or the look-up itself: put(k, row) for the 27 taps of column `col`
template <class Put>
__device__ inline void tile_sources(const ConvArgs& a, int col, Put put) {
  if (a.src_table) {
    int row[27];
#pragma unroll
    for (int k = 0; k < 27; ++k) row[k] = a.src_table[(int64_t)k * a.src_pitch + col];
#pragma unroll
    for (int k = 0; k < 27; ++k) put(k, row[k]);
  } else {
    lookup_sources(a, col, put);
  }
}

template <int MT>
__global__ __launch_bounds__(256) void conv_rows_f32_kernel(ConvArgs a, float* __restrict__ out,
    const float4* __restrict__ xt, const float* __restrict__ Wt, int n_tiles, int cpad) {
  constexpr int kWWords = (kRowSlabF / 8) * 4 * MT * 64;  // weights of one (tap, slab)
  constexpr int kWVec = kWWords / 4 / 256;               // float4 per thread (4 for MT = 2)
  __shared__ __attribute__((aligned(16))) float sW[2 * kWWords];  // double buffered: one barrier per stage
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = xcd_tile(blockIdx.x, n_tiles);
  if (tile >= n_tiles) return;
  const int n0 = tile * kTileCols + wave * kWaveCols;
  const int r = lane & 31, kh = lane >> 5;
  const int nslab = (cpad + kRowSlabF - 1) / kRowSlabF;
  const int npass = (a.mtiles + MT - 1) / MT;
  const int cpad4 = cpad >> 2;
  const int nstage = a.K * nslab;
  // source rows of all taps of the workgroup's 256 columns, looked up once and all together
  // (inside the tap loop a look-up is a chain of two or three trips to memory per tap)
  __shared__ int sSrc[27][kTileCols];
  tile_sources(a, tile * kTileCols + (int)threadIdx.x, [&](int k, int row) { sSrc[k][threadIdx.x] = row; });
  __syncthreads();
  for (int pass = blockIdx.y; pass < npass; pass += gridDim.y) {  // passes may be dealt out over workgroups
    floatx16 acc[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.0f;
    // weights on their way to LDS: a value type, so that they stay in registers
    struct WRegs { float4 v[kWVec > 0 ? kWVec : 1]; };
    WRegs wr;
    auto fetch_w = [&](int stage) {
      const float4* wsrc = reinterpret_cast<const float4*>(Wt + ((int64_t)pass * nstage + stage) * kWWords);
      WRegs w;
#pragma unroll
      for (int v = 0; v < kWVec; ++v) w.v[v] = wsrc[v * 256 + threadIdx.x];
      return w;
    };
    // Software pipeline over the stages (tap, 64-channel slab): while the MFMAs of one stage run,
    // the weights AND all gathers of the next stage (8 channel groups x 2 columns, 16 bytes each)
    // are in flight; the source rows of a tap are looked up two taps ahead.
    float4 nx0[kRowSlabF / 8], nx1[kRowSlabF / 8];
    auto src_of = [&](int k, int half) { return k < a.K ? sSrc[k][wave * kWaveCols + half * 32 + r] : -1; };
    auto fetch_x = [&](int s0, int s1, int slab) {
      const float4* row0 = xt + (int64_t)(s0 < 0 ? a.Hin : s0) * cpad4 + kh;
      const float4* row1 = xt + (int64_t)(s1 < 0 ? a.Hin : s1) * cpad4 + kh;
      const int ngroup = min(kRowSlabF, cpad - slab * kRowSlabF) >> 3;
#pragma unroll
      for (int c8 = 0; c8 < kRowSlabF / 8; ++c8)
        if (c8 < ngroup) {
          nx0[c8] = row0[(slab * kRowSlabF + c8 * 8) >> 2];
          nx1[c8] = row1[(slab * kRowSlabF + c8 * 8) >> 2];
        }
    };
    int s0c = src_of(0, 0), s1c = src_of(0, 1);      // rows of the current tap
    int s0n = src_of(1, 0), s1n = src_of(1, 1);      // ... of the next one
    // A tap whose neighbour is missing for all 64 columns of the wavefront adds nothing: its
    // products are not formed (over the non-empty nodes of a surface that is about half of the
    // (wavefront, tap) pairs).  Uniform over the wavefront.
    auto any_row = [](int src) { return __ballot(src >= 0) != 0; };
    bool l0c = any_row(s0c), l1c = any_row(s1c), l0n = any_row(s0n), l1n = any_row(s1n);
    wr = fetch_w(0);
    fetch_x(s0c, s1c, 0);
    __syncthreads();  // the last stage of the previous pass may still be reading the weights
#pragma unroll
    for (int v = 0; v < kWVec; ++v) reinterpret_cast<float4*>(sW)[v * 256 + threadIdx.x] = wr.v[v];
    if (1 < nstage) wr = fetch_w(1);
    int stage = 0;
    for (int k = 0; k < a.K; ++k) {
      const int s0n2 = src_of(k + 2, 0), s1n2 = src_of(k + 2, 1);
      const bool l0n2 = any_row(s0n2), l1n2 = any_row(s1n2);
      for (int slab = 0; slab < nslab; ++slab, ++stage) {
        // stage - 1 is over everywhere and the weights of this stage are in place; the weights
        // of the next stage (requested a stage ago) go into the other buffer while this one is
        // read, those of the stage after that are requested
        __syncthreads();
        const float* wcur = sW + (stage & 1) * kWWords;
        if (stage + 1 < nstage) {
#pragma unroll
          for (int v = 0; v < kWVec; ++v)
            reinterpret_cast<float4*>(sW + ((stage + 1) & 1) * kWWords)[v * 256 + threadIdx.x] = wr.v[v];
        }
        // group c8 of the NEXT stage is requested right after group c8 of this one has been read
        // out of its registers, so every gather has seven eighths of a stage to arrive
        const bool more = stage + 1 < nstage;
        const bool same_tap = slab + 1 < nslab;
        const int nslab_next = same_tap ? slab + 1 : 0;
        const int s0x = same_tap ? s0c : s0n, s1x = same_tap ? s1c : s1n;
        const float4* nrow0 = xt + (int64_t)(s0x < 0 ? a.Hin : s0x) * cpad4 + kh + ((nslab_next * kRowSlabF) >> 2);
        const float4* nrow1 = xt + (int64_t)(s1x < 0 ? a.Hin : s1x) * cpad4 + kh + ((nslab_next * kRowSlabF) >> 2);
        const int ngroup_next = more ? (min(kRowSlabF, cpad - nslab_next * kRowSlabF) >> 3) : 0;
        if (stage + 2 < nstage) wr = fetch_w(stage + 2);
        const int ngroup = min(kRowSlabF, cpad - slab * kRowSlabF) >> 3;
        // Both column tiles or none: the test is made once per stage and the MFMAs stay one
        // straight-line block (a body per case of (tile 0 live, tile 1 live) made the compiler
        // move the 64 accumulator registers at every join; a branch per MFMA breaks up their issue).
        const bool live = l0c || l1c;
#pragma unroll
        for (int c8 = 0; c8 < kRowSlabF / 8; ++c8) {
          const float4 b0 = nx0[c8], b1 = nx1[c8];
          if (c8 < ngroup_next) {   // requested whether live or not (a dead tile reads the zero row, which
            nx0[c8] = nrow0[c8 * 2];  // stays in the L1): a branch per request would cost the waits their order
            nx1[c8] = nrow1[c8 * 2];
          }
          if (c8 >= ngroup || !live) continue;  // uniform
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float v0 = j == 0 ? b0.x : j == 1 ? b0.y : j == 2 ? b0.z : b0.w;
            const float v1 = j == 0 ? b1.x : j == 1 ? b1.y : j == 2 ? b1.z : b1.w;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
              const float av = wcur[((c8 * 4 + j) * MT + mt) * 64 + lane];
              acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, v0, acc[mt][0], 0, 0, 0);
              acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, v1, acc[mt][1], 0, 0, 0);
            }
          }
        }
      }
      s0c = s0n; s1c = s1n; s0n = s0n2; s1n = s1n2;
      l0c = l0n; l1c = l1n; l0n = l0n2; l1n = l1n2;
    }
    if (n0 < a.N) store_tiles<float, MT>(a, out, acc, pass * MT, n0, lane);
  }
}
// The same operator without LDS for the weights and without barriers (the fp32 form of
// conv_rows_bf16_direct_kernel below): a wavefront walks the (tap, 32-channel slab) stages of
// the taps that are live for its own 64 columns, reads the A fragments of a stage straight from
// the packed weights (16 bytes a lane: the four k-steps of an 8-channel group) and gathers the
// rows of the column halves that have the neighbour, with the next stage's weights and rows in
// flight (two register sets).  The staged kernel above takes every workgroup through all
// K x slabs barriers and moves the weights of all taps through LDS whether a tap is live or not;
// over the non-empty nodes of a surface about half of the (wavefront, tap) pairs are dead.
// Stages in the same order as the staged kernel (tap, then slab), a dead half adds nothing:
// the same sums.
template <int MT, int WPS = 2, int WAVES = kConvWaves>
__global__ __launch_bounds__(64 * WAVES, WPS) void conv_rows_f32_direct_kernel(ConvArgs a, float* __restrict__ out,
    const float4* __restrict__ xt, const float4* __restrict__ Wt, int n_tiles, int cpad) {
  constexpr int kG = kRowSlabF / 8;                    // 8-channel groups of a slab
  constexpr int kWVecs = kG * MT * 64;                 // 16-byte units of one (tap, slab)
  constexpr int kCols = kWaveCols * WAVES;             // columns of a workgroup
  __shared__ int sSrc[27][kCols];                      // source row of (tap, column), in 16-byte units of the copy
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = xcd_tile(blockIdx.x, n_tiles);
  if (tile >= n_tiles) return;
  const int n0 = tile * kCols + wave * kWaveCols;
  const int r = lane & 31, kh = lane >> 5;
  const int nslab = (cpad + kRowSlabF - 1) / kRowSlabF;
  const int npass = (a.mtiles + MT - 1) / MT;
  const int cpad4 = cpad >> 2;
  tile_sources(a, tile * kCols + (int)threadIdx.x,
      [&](int k, int row) { sSrc[k][threadIdx.x] = (row < 0 ? a.Hin : row) * cpad4; });
  const int c0 = wave * kWaveCols + r;
  unsigned live[2] = {0, 0};
  __syncthreads();                                     // source rows written
  {
    const int none = a.Hin * cpad4;
#pragma unroll
    for (int k = 0; k < 27; ++k) {
      if (k >= a.K) break;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
        if (__ballot(sSrc[k][c0 + 32 * nt] != none) != 0) live[nt] |= 1u << k;
    }
    live[0] = __builtin_amdgcn_readfirstlane(live[0]);
    live[1] = __builtin_amdgcn_readfirstlane(live[1]);
  }
  const unsigned live_any = live[0] | live[1];
  for (int pass = blockIdx.y; pass < npass; pass += gridDim.y) {
    floatx16 acc[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.0f;
    float4 wa[2][kG][MT], x[2][kG][2];                 // two register sets: [set][group][row tile / column half]
    auto fetch = [&](int tap, int slab, auto set) {
      constexpr int S = decltype(set)::value;
      if (tap < 0) return;                             // uniform
      const int ngroup = min(kRowSlabF, cpad - slab * kRowSlabF) >> 3;
      const float4* wsrc = Wt + (((int64_t)pass * a.K + tap) * nslab + slab) * kWVecs + lane;
#pragma unroll
      for (int c8 = 0; c8 < kG; ++c8)
        if (c8 < ngroup) {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) wa[S][c8][mt] = wsrc[(c8 * MT + mt) * 64];
        }
      const int s0 = sSrc[tap][c0], s1 = sSrc[tap][c0 + 32];
      const int off = ((slab * kRowSlabF) >> 2) + kh;
      if ((live[0] >> tap) & 1) {                      // uniform over the wavefront
#pragma unroll
        for (int c8 = 0; c8 < kG; ++c8)
          if (c8 < ngroup) x[S][c8][0] = xt[(int64_t)s0 + off + 2 * c8];
      }
      if ((live[1] >> tap) & 1) {
#pragma unroll
        for (int c8 = 0; c8 < kG; ++c8)
          if (c8 < ngroup) x[S][c8][1] = xt[(int64_t)s1 + off + 2 * c8];
      }
    };
    auto part = [](const float4& v, int j) { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; };
    auto compute = [&](int tap, int slab, auto set) {
      constexpr int S = decltype(set)::value;
      const bool l0 = (live[0] >> tap) & 1, l1 = (live[1] >> tap) & 1;   // uniform over the wavefront
      const int ngroup = min(kRowSlabF, cpad - slab * kRowSlabF) >> 3;
#pragma unroll
      for (int c8 = 0; c8 < kG; ++c8) {
        if (c8 >= ngroup) continue;                    // uniform
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            const float av = part(wa[S][c8][mt], j);
            if (l0) acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, part(x[S][c8][0], j), acc[mt][0], 0, 0, 0);
            if (l1) acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, part(x[S][c8][1], j), acc[mt][1], 0, 0, 0);
          }
        }
      }
    };
    unsigned todo = live_any;                          // live taps not yet requested (uniform)
    auto next_tap = [&]() {
      if (todo == 0) return -1;
      const int t = __builtin_ctz(todo);
      todo &= todo - 1;
      return t;
    };
    // the stages (live tap, slab) in order, two in flight
    int t0 = next_tap(), s0 = 0;
    fetch(t0, s0, std::integral_constant<int, 0>());
    while (t0 >= 0) {
      int t1 = t0, s1 = s0 + 1;
      if (s1 == nslab) { s1 = 0; t1 = next_tap(); }
      fetch(t1, s1, std::integral_constant<int, 1>());
      compute(t0, s0, std::integral_constant<int, 0>());
      if (t1 < 0) break;
      t0 = t1; s0 = s1 + 1;
      if (s0 == nslab) { s0 = 0; t0 = next_tap(); }
      fetch(t0, s0, std::integral_constant<int, 0>());
      compute(t1, s1, std::integral_constant<int, 1>());
    }
    if (n0 < a.N) store_tiles<float, MT>(a, out, acc, pass * MT, n0, lane);
  }
}
// [pass][tap][slab][c8][j][mt][lane]: lane (m, kh) <- W'(m, slab*64 + c8*8 + 4kh + j, tap)
// (direct: [pass][tap][slab][c8][mt][lane][j], the four k-steps of a group as one 16-byte unit a lane)
__global__ void pack_weights_rows_f32(float* __restrict__ Wt, const float* __restrict__ W, int M, int Cin, int K,
    int MT, int npass, int nslab, int64_t sm, int64_t sc, int direct) {
  int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = (int64_t)npass * K * nslab * (kRowSlabF / 8) * 4 * MT * 64;
  if (id >= total) return;
  int l, j, mt;
  int64_t f;
  if (direct) {
    j = (int)(id & 3);
    l = (int)((id >> 2) & 63);
    f = id >> 8;
    mt = (int)(f % MT); f /= MT;
  } else {
    l = (int)(id & 63);
    f = id >> 6;
    mt = (int)(f % MT); f /= MT;
    j = (int)(f % 4); f /= 4;
  }
  int c8 = (int)(f % (kRowSlabF / 8)); f /= (kRowSlabF / 8);
  int slab = (int)(f % nslab); f /= nslab;
  int k = (int)(f % K);
  int pass = (int)(f / K);
  int m = (pass * MT + mt) * 32 + (l & 31), c = slab * kRowSlabF + c8 * 8 + 4 * (l >> 5) + j;
  Wt[id] = (m < M && c < Cin) ? W[m * sm + c * sc + k] : 0.0f;
}

template <int MT>
__global__ __launch_bounds__(256) void conv_rows_bf16_kernel(ConvArgs a, uint16_t* __restrict__ out,
    const u32x4* __restrict__ xt, const u32x4* __restrict__ Wt, int n_tiles, int cpad) {
  constexpr int kWUnits = (kRowSlab / 16) * MT * 64;  // 16-byte units of one (tap, slab)
  __shared__ u32x4 sW[kWUnits];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = xcd_tile(blockIdx.x, n_tiles);
  if (tile >= n_tiles) return;
  const int n0 = tile * kTileCols + wave * kWaveCols;
  const int r = lane & 31, kh = lane >> 5;
  const int nslab = (cpad + kRowSlab - 1) / kRowSlab;
  const int npass = (a.mtiles + MT - 1) / MT;
  const int cpad8 = cpad >> 3;
  const int nstage = a.K * nslab;
  for (int pass = blockIdx.y; pass < npass; pass += gridDim.y) {  // passes may be dealt out over workgroups
    floatx16 acc[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.0f;
    u32x4 wr[2];
    auto fetch_w = [&](int stage) {
      const u32x4* wsrc = Wt + ((int64_t)pass * nstage + stage) * kWUnits;
#pragma unroll
      for (int v = 0; v < 2; ++v) {
        int idx = v * 256 + threadIdx.x;
        wr[v] = idx < kWUnits ? wsrc[idx] : (u32x4)(0u);
      }
    };
    // same pipeline as the fp32 kernel: weights and all gathers of the next stage (4 groups of 16
    // channels x 2 columns) are requested before the MFMAs of the current one
    u32x4 nx0[kRowSlab / 16], nx1[kRowSlab / 16];
    auto src_of = [&](int k, int half) { return k < a.K ? conv_src(a, n0 + half * 32 + r, k) : -1; };
    auto fetch_x = [&](int s0, int s1, int slab) {
      const u32x4* row0 = xt + (int64_t)(s0 < 0 ? a.Hin : s0) * cpad8 + kh;
      const u32x4* row1 = xt + (int64_t)(s1 < 0 ? a.Hin : s1) * cpad8 + kh;
      const int ngroup = min(kRowSlab, cpad - slab * kRowSlab) >> 4;
#pragma unroll
      for (int c16 = 0; c16 < kRowSlab / 16; ++c16)
        if (c16 < ngroup) {
          nx0[c16] = row0[(slab * kRowSlab + c16 * 16) >> 3];
          nx1[c16] = row1[(slab * kRowSlab + c16 * 16) >> 3];
        }
    };
    int s0c = src_of(0, 0), s1c = src_of(0, 1);
    int s0n = src_of(1, 0), s1n = src_of(1, 1);
    fetch_w(0);
    fetch_x(s0c, s1c, 0);
    int stage = 0;
    for (int k = 0; k < a.K; ++k) {
      const int s0n2 = src_of(k + 2, 0), s1n2 = src_of(k + 2, 1);
      for (int slab = 0; slab < nslab; ++slab, ++stage) {
        __syncthreads();
#pragma unroll
        for (int v = 0; v < 2; ++v) {
          int idx = v * 256 + threadIdx.x;
          if (idx < kWUnits) sW[idx] = wr[v];
        }
        __syncthreads();
        const bool more = stage + 1 < nstage;
        const bool same_tap = slab + 1 < nslab;
        const int nslab_next = same_tap ? slab + 1 : 0;
        const int s0x = same_tap ? s0c : s0n, s1x = same_tap ? s1c : s1n;
        const u32x4* nrow0 = xt + (int64_t)(s0x < 0 ? a.Hin : s0x) * cpad8 + kh + ((nslab_next * kRowSlab) >> 3);
        const u32x4* nrow1 = xt + (int64_t)(s1x < 0 ? a.Hin : s1x) * cpad8 + kh + ((nslab_next * kRowSlab) >> 3);
        const int ngroup_next = more ? (min(kRowSlab, cpad - nslab_next * kRowSlab) >> 4) : 0;
        if (more) fetch_w(stage + 1);
        const int ngroup = min(kRowSlab, cpad - slab * kRowSlab) >> 4;
#pragma unroll
        for (int c16 = 0; c16 < kRowSlab / 16; ++c16) {
          union { u32x4 q; bf16x8 v; } b0, b1;
          b0.q = nx0[c16];
          b1.q = nx1[c16];
          if (c16 < ngroup_next) {
            nx0[c16] = nrow0[c16 * 2];
            nx1[c16] = nrow1[c16 * 2];
          }
          if (c16 >= ngroup) continue;  // uniform
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            union { u32x4 q; bf16x8 v; } av;
            av.q = sW[(c16 * MT + mt) * 64 + lane];
            acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av.v, b0.v, acc[mt][0], 0, 0, 0);
            acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av.v, b1.v, acc[mt][1], 0, 0, 0);
          }
        }
      }
      s0c = s0n; s1c = s1n; s0n = s0n2; s1n = s1n2;
    }
    if (n0 < a.N) store_tiles<uint16_t, MT>(a, out, acc, pass * MT, n0, lane);
  }
}
// Every 16-byte store of the row-major epilogues goes through this one function.  At depth 9 a
// few words per million outputs held the value computed for the NEXT store, different from run to
// run, while these stores sat in conditional blocks of their own (channel piece inside the pitch or
// not) with nothing between them and the next writer of their data registers; two wait states
// behind each store cured it.  The cause is established by that experiment, not by a rule of the
// instruction set that could be relied on elsewhere, so the cure is applied to every such store:
//   * the store is unconditional: a piece outside the pitch (`inside` false, uniform) gets the
//     out-of-range offset that columns behind the level use, and the hardware drops it, so no
//     store stands alone in a block;
//   * the wait states are tied to the store's data registers: the asm statement takes the four
//     registers as read-write operands, so the register allocator keeps them (and nothing else
//     in them) until the two wait states have passed.
// tests/test_gpu_rows.py::test_rows_operators_full_size is the regression test (equal bits
// over repeated runs at full size).
typedef uint32_t store16_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store16_then_wait(store16_t v, __amdgpu_buffer_rsrc_t buf, int voffset, int soffset,
    bool inside) {
  __builtin_amdgcn_raw_buffer_store_b128(v, buf, inside ? voffset : 0x7fffff00, soffset, 0);
  asm volatile("s_nop 1" : "+v"(v) : : "memory");
}

// Row-major epilogue of the 32x32 accumulator tiles acc[MT][2] of a wavefront (columns n0 .. n0 + 63,
// channels cb + 32 mt ..): lane (r, kh) holds channels cb + 32 mt + 8 q + 4 kh + e of its two
// columns; the lanes r and r + 32 swap halves, so that each ends up with 8 consecutive channels and
// stores 16 bytes (32 contiguous bytes per row and store).  A column behind the level gets an
// offset past the end of the buffer and the hardware drops its store.
template <int MT>
__device__ inline void rows_out_tiles(const ConvArgs& a, uint16_t* __restrict__ out, int out_pitch, int out_cpad,
    floatx16 (&acc)[MT][2], int cb, int n0, int lane) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  typedef float floatx2_t __attribute__((ext_vector_type(2)));
  const int r = lane & 31, kh = lane >> 5;
  const __amdgpu_buffer_rsrc_t obuf = __builtin_amdgcn_make_buffer_rsrc(
      out, 0, (int)(((int64_t)a.Hout + 1) * out_pitch * 2), 0x00020000);
  const float floor = a.relu ? 0.0f : -__builtin_inff();
  auto pack = [](float lo, float hi) {
    floatx2_t f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
  };
  auto clamp = [&](float v) { return v < floor ? floor : v; };   // keeps a NaN
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    float bias[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int ch = cb + 32 * mt + 8 * (i / 4) + 4 * kh + (i % 4);
      bias[i] = a.bias ? a.bias[min(ch, a.M - 1)] : 0.0f;
      if (ch >= a.M) bias[i] = 0.0f;   // the padding channels of a row stay zero
    }
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const int n = n0 + nt * 32 + r;
      const int ooff = n < a.N ? (n * out_pitch + 8 * kh) * 2 : 0x7fffff00;
      uint32_t w[4][2];
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int i = 4 * q + 2 * h;
          w[q][h] = pack(clamp(acc[mt][nt][i] + bias[i]), clamp(acc[mt][nt][i + 1] + bias[i + 1]));
        }
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        const auto s0 = __builtin_amdgcn_permlane32_swap(w[2 * jj][0], w[2 * jj + 1][0], false, false);
        const auto s1 = __builtin_amdgcn_permlane32_swap(w[2 * jj][1], w[2 * jj + 1][1], false, false);
        store16_then_wait(store16_t{s0[0], s1[0], s0[1], s1[1]}, obuf, ooff, (cb + 32 * mt + 16 * jj) * 2,
            cb + 32 * mt + 16 * jj < out_cpad);
      }
    }
  }
}

// The same operator with a deeper pipeline, for tap sets of three taps or more.  The kernel
// above pays two barriers per (tap, 64-channel slab) for 16 MFMAs per wavefront and has one
// stage of gathers in flight; with 27 rows to fetch per column from the L2 that leaves the
// matrix pipe idle seven cycles in eight.  Here
//   * the source rows of all taps of the workgroup's 256 columns are looked up once, up front and
//     all together (two dependent trips to memory for the whole tile), and wait in LDS;
//   * the weights come in groups of three taps (24 KiB for 64 output channels, two buffers):
//     one barrier per three taps;
//   * a tap's operands (64 channels x 2 column tiles = 8 loads per lane, which read each source
//     row in full) are requested two taps ahead into a ring of three register sets;
//   * the register budget allows two workgroups per CU, so that a second wavefront per SIMD
//     multiplies while the first waits.
// Non-empty 3x3x3 64 -> 64 at depth 9 (232 158 columns): 0.162 -> 0.132 ms for the operator, the
// kernel itself 0.11 ms.  What bounds it now is the volume of the gathers: 27 rows of 128 bytes
// per column from the L2, 0.8 GB per launch, where the matrix work is 20 microseconds; neighbouring
// columns share most of their rows, which only a per-tile list of distinct rows staged in LDS
// would exploit.
// SLAB: input channels per stage.  MT = 4 (128 output channels a pass) with 32-channel stages halves the
// operand bytes per MFMA against MT = 2 with 64-channel stages at the same LDS and register budget: two
// row tiles share a gathered operand at MT = 2, four at MT = 4, and the L1 delivers 64 bytes a cycle.
// ROWS_OUT: row-major output ([Hout + 1][out_pitch], channels below out_cpad and the zero row written),
// as the row-major kernels further down write it.
template <int MT, int SLAB, bool ROWS_OUT>
__global__ __launch_bounds__(256, 2) void conv_rows_bf16_deep_kernel(ConvArgs a, uint16_t* __restrict__ out,
    const u32x4* __restrict__ xt, const u32x4* __restrict__ Wt, int n_tiles, int cpad, int in_pitch, int out_pitch, int out_cpad) {
  constexpr int kG = 3;                                 // taps per weight group
  constexpr int kKs = SLAB / 16;                    // k-steps per slab
  constexpr int kWUnits = kKs * MT * 64;                // 16-byte units of one (tap, slab)
  constexpr int kWVec = kG * kWUnits / 256;             // per thread and group
  __shared__ u32x4 sW[2][kG * kWUnits];
  __shared__ int sSrc[27][kTileCols];                   // source row of (tap, column), in 16-byte units of the copy
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = xcd_tile(blockIdx.x, n_tiles);
  if (tile >= n_tiles) return;
  const int n0 = tile * kTileCols + wave * kWaveCols;
  const int r = lane & 31, kh = lane >> 5;
  const int nslab = (cpad + SLAB - 1) / SLAB;
  const int npass = (a.mtiles + MT - 1) / MT;
  const int cpad8 = in_pitch >> 3;   // 16-byte units per input row (the pitch; the channels read are below cpad)
  const int ngroup = (a.K + kG - 1) / kG;
  {
    tile_sources(a, tile * kTileCols + (int)threadIdx.x,
        [&](int k, int row) { sSrc[k][threadIdx.x] = (row < 0 ? a.Hin : row) * cpad8; });
  }
  const int c0 = wave * kWaveCols + r;                  // my column of the first column tile, inside the workgroup's tile
  union Frag { u32x4 q; bf16x8 v; };
  // Taps whose neighbour is missing for all 32 columns of a column tile add nothing: their
  // operands are not requested and their products not formed.  Over the non-empty nodes of a
  // surface that is most taps (the columns of a wavefront lie on one patch of the surface, and
  // the nodes off that patch are empty for all of them).  live[nt]: bit k = tap k has a
  // neighbour in column tile nt of this wavefront.
  unsigned live[2] = {0, 0};
  __syncthreads();                                       // source rows written
  {
    const int none = a.Hin * cpad8;
#pragma unroll
    for (int k = 0; k < 27; ++k) {
      if (k >= a.K) break;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
        if (__ballot(sSrc[k][c0 + 32 * nt] != none) != 0) live[nt] |= 1u << k;
    }
    live[0] = __builtin_amdgcn_readfirstlane(live[0]);
    live[1] = __builtin_amdgcn_readfirstlane(live[1]);
  }
  for (int pass = blockIdx.y; pass < npass; pass += gridDim.y) {  // passes may be dealt out over workgroups
    floatx16 acc[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.0f;
    for (int slab = 0; slab < nslab; ++slab) {
      const int nks = min(SLAB, cpad - slab * SLAB) >> 4;    // k-steps of this slab (uniform)
      const int col16 = ((slab * SLAB) >> 3) + kh;               // my 16-byte unit inside a row
      u32x4 wr[kWVec];
      // group g of this (pass, slab): taps 3g .. 3g+2, each kWUnits units at ((pass K + tap) nslab + slab) kWUnits
      auto fetch_w = [&](int g) {
#pragma unroll
        for (int v = 0; v < kWVec; ++v) {
          const int idx = v * 256 + (int)threadIdx.x;
          const int tap = min(g * kG + idx / kWUnits, a.K - 1);
          wr[v] = Wt[(((int64_t)pass * a.K + tap) * nslab + slab) * kWUnits + idx % kWUnits];
        }
      };
      Frag x[3][kKs][2];                                 // ring of three taps: [tap % 3][k-step][column tile]
      auto fetch_x = [&](int tap, auto set) {
        constexpr int S = decltype(set)::value;
        if (tap >= a.K) return;                          // uniform
        const int s0 = sSrc[tap][c0], s1 = sSrc[tap][c0 + 32];
        if ((live[0] >> tap) & 1) {                      // uniform over the wavefront
#pragma unroll
          for (int ks = 0; ks < kKs; ++ks)
            if (ks < nks) x[S][ks][0].q = xt[(int64_t)s0 + col16 + 2 * ks];
        }
        if ((live[1] >> tap) & 1) {
#pragma unroll
          for (int ks = 0; ks < kKs; ++ks)
            if (ks < nks) x[S][ks][1].q = xt[(int64_t)s1 + col16 + 2 * ks];
        }
      };
      __syncthreads();                                   // source rows written (first time); weight buffers free
      fetch_w(0);
      fetch_x(0, std::integral_constant<int, 0>());
      fetch_x(1, std::integral_constant<int, 1>());
#pragma unroll
      for (int v = 0; v < kWVec; ++v) sW[0][v * 256 + threadIdx.x] = wr[v];
      for (int g = 0; g < ngroup; ++g) {
        __syncthreads();                                 // group g's weights are in LDS; the other buffer is free
        const u32x4* wcur = sW[g & 1];
        if (g + 1 < ngroup) fetch_w(g + 1);
        auto tap_step = [&](auto jc) {
          constexpr int J = decltype(jc)::value;
          const int tap = g * kG + J;
          if (tap >= a.K) return;                        // uniform
          fetch_x(tap + 2, std::integral_constant<int, (J + 2) % 3>());
          const bool l0 = (live[0] >> tap) & 1, l1 = (live[1] >> tap) & 1;   // uniform over the wavefront
          if (!l0 && !l1) return;
#pragma unroll
          for (int ks = 0; ks < kKs; ++ks) {
            if (ks >= nks) continue;                     // uniform
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
              Frag av;
              av.q = wcur[J * kWUnits + (ks * MT + mt) * 64 + lane];
              if (l0) acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av.v, x[J][ks][0].v, acc[mt][0], 0, 0, 0);
              if (l1) acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av.v, x[J][ks][1].v, acc[mt][1], 0, 0, 0);
            }
          }
        };
        tap_step(std::integral_constant<int, 0>());
        tap_step(std::integral_constant<int, 1>());
        tap_step(std::integral_constant<int, 2>());
        if (g + 1 < ngroup) {
#pragma unroll
          for (int v = 0; v < kWVec; ++v) sW[(g + 1) & 1][v * 256 + threadIdx.x] = wr[v];
        }
      }
    }
    if constexpr (ROWS_OUT) {
      rows_out_tiles<MT>(a, out, out_pitch, out_cpad, acc, pass * MT * 32, n0, lane);
      if (tile == 0 && wave == 0 && lane * 8 >= pass * MT * 32 && lane * 8 < min((pass + 1) * MT * 32, out_cpad))
        *reinterpret_cast<uint4*>(out + (int64_t)a.Hout * out_pitch + lane * 8) = make_uint4(0, 0, 0, 0);
    } else {
      if (n0 < a.N) store_tiles<uint16_t, MT>(a, out, acc, pass * MT, n0, lane);
    }
  }
}

// The same operator without LDS for the weights and without barriers: a wavefront reads the A
// fragments of a tap straight from the packed weights (1 KiB coalesced per fragment, served by the
// L1 / L2: the four wavefronts of a workgroup and the workgroups of a compute unit read the same
// bytes) and only for the taps that are live for its own 64 columns.  Over the non-empty nodes of
// a surface most (wavefront, tap) pairs are dead (12 of 27 taps live per 32 columns at depth 9 of
// the scene), but the LDS-staged kernel moves the weights of all 27 taps through LDS for every
// tile, 216 KiB for 64 -> 64, more than the rows it gathers, and synchronises its wavefronts nine
// times a slab.  Here a wavefront walks its live taps in ascending order with the next live tap's
// weights and rows in flight (two register sets), at its own pace.  Same products in the same order
// as conv_rows_bf16_deep_kernel: the results are bit-identical.
template <int MT, int SLAB, bool ROWS_OUT, int WPS = 2, int WAVES = kConvWaves>
__global__ __launch_bounds__(64 * WAVES, WPS) void conv_rows_bf16_direct_kernel(ConvArgs a, uint16_t* __restrict__ out,
    const u32x4* __restrict__ xt, const u32x4* __restrict__ Wt, int n_tiles, int cpad, int in_pitch, int out_pitch, int out_cpad) {
  constexpr int kKs = SLAB / 16;                        // k-steps per slab
  constexpr int kWUnits = kKs * MT * 64;                // 16-byte units of one (tap, slab)
  constexpr int kCols = kWaveCols * WAVES;              // columns of a workgroup
  __shared__ int sSrc[27][kCols];                   // source row of (tap, column), in 16-byte units of the copy
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = xcd_tile(blockIdx.x, n_tiles);
  if (tile >= n_tiles) return;
  const int n0 = tile * kCols + wave * kWaveCols;
  const int r = lane & 31, kh = lane >> 5;
  const int nslab = (cpad + SLAB - 1) / SLAB;
  const int npass = (a.mtiles + MT - 1) / MT;
  const int cpad8 = in_pitch >> 3;
  tile_sources(a, tile * kCols + (int)threadIdx.x,
      [&](int k, int row) { sSrc[k][threadIdx.x] = (row < 0 ? a.Hin : row) * cpad8; });
  const int c0 = wave * kWaveCols + r;
  union Frag { u32x4 q; bf16x8 v; };
  unsigned live[2] = {0, 0};
  __syncthreads();                                       // source rows written
  {
    const int none = a.Hin * cpad8;
#pragma unroll
    for (int k = 0; k < 27; ++k) {
      if (k >= a.K) break;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
        if (__ballot(sSrc[k][c0 + 32 * nt] != none) != 0) live[nt] |= 1u << k;
    }
    live[0] = __builtin_amdgcn_readfirstlane(live[0]);
    live[1] = __builtin_amdgcn_readfirstlane(live[1]);
  }
  const unsigned live_any = live[0] | live[1];
  for (int pass = blockIdx.y; pass < npass; pass += gridDim.y) {
    floatx16 acc[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.0f;
    for (int slab = 0; slab < nslab; ++slab) {
      const int nks = min(SLAB, cpad - slab * SLAB) >> 4;    // k-steps of this slab (uniform)
      const int col16 = ((slab * SLAB) >> 3) + kh;               // my 16-byte unit inside a row
      Frag wa[2][kKs][MT], x[2][kKs][2];                     // two register sets: [set][k-step][row tile / column tile]
      auto fetch = [&](int tap, auto set) {
        constexpr int S = decltype(set)::value;
        if (tap < 0) return;                              // uniform
        const u32x4* wsrc = Wt + (((int64_t)pass * a.K + tap) * nslab + slab) * kWUnits + lane;
#pragma unroll
        for (int ks = 0; ks < kKs; ++ks)
          if (ks < nks) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) wa[S][ks][mt].q = wsrc[(ks * MT + mt) * 64];
          }
        const int s0 = sSrc[tap][c0], s1 = sSrc[tap][c0 + 32];
        if ((live[0] >> tap) & 1) {                      // uniform over the wavefront
#pragma unroll
          for (int ks = 0; ks < kKs; ++ks)
            if (ks < nks) x[S][ks][0].q = xt[(int64_t)s0 + col16 + 2 * ks];
        }
        if ((live[1] >> tap) & 1) {
#pragma unroll
          for (int ks = 0; ks < kKs; ++ks)
            if (ks < nks) x[S][ks][1].q = xt[(int64_t)s1 + col16 + 2 * ks];
        }
      };
      auto compute = [&](int tap, auto set) {
        constexpr int S = decltype(set)::value;
        const bool l0 = (live[0] >> tap) & 1, l1 = (live[1] >> tap) & 1;   // uniform over the wavefront
#pragma unroll
        for (int ks = 0; ks < kKs; ++ks) {
          if (ks >= nks) continue;                       // uniform
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            if (l0) acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wa[S][ks][mt].v, x[S][ks][0].v, acc[mt][0], 0, 0, 0);
            if (l1) acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wa[S][ks][mt].v, x[S][ks][1].v, acc[mt][1], 0, 0, 0);
          }
        }
      };
      unsigned todo = live_any;                          // live taps not yet requested (uniform)
      auto next_tap = [&]() {
        if (todo == 0) return -1;
        const int t = __builtin_ctz(todo);
        todo &= todo - 1;
        return t;
      };
      int t0 = next_tap();
      fetch(t0, std::integral_constant<int, 0>());
      while (t0 >= 0) {
        const int t1 = next_tap();
        fetch(t1, std::integral_constant<int, 1>());
        compute(t0, std::integral_constant<int, 0>());
        if (t1 < 0) break;
        t0 = next_tap();
        fetch(t0, std::integral_constant<int, 0>());
        compute(t1, std::integral_constant<int, 1>());
      }
    }
    if constexpr (ROWS_OUT) {
      rows_out_tiles<MT>(a, out, out_pitch, out_cpad, acc, pass * MT * 32, n0, lane);
      if (tile == 0 && wave == 0 && lane * 8 >= pass * MT * 32 && lane * 8 < min((pass + 1) * MT * 32, out_cpad))
        *reinterpret_cast<uint4*>(out + (int64_t)a.Hout * out_pitch + lane * 8) = make_uint4(0, 0, 0, 0);
    } else {
      if (n0 < a.N) store_tiles<uint16_t, MT>(a, out, acc, pass * MT, n0, lane);
    }
  }
}

// [pass][tap][slab][c16][mt][lane][j]: lane (m, kh), j <- W'(m, slab*64 + c16*16 + 8kh + j, tap)
__global__ void pack_weights_rows_bf16(uint16_t* __restrict__ Wt, const uint16_t* __restrict__ W, int M, int Cin,
    int K, int MT, int npass, int nslab, int64_t sm, int64_t sc, int slab_ch) {
  int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = (int64_t)npass * K * nslab * (slab_ch / 16) * MT * 64 * 8;
  if (id >= total) return;
  int j = (int)(id & 7);
  int l = (int)((id >> 3) & 63);
  int64_t f = id >> 9;
  int mt = (int)(f % MT); f /= MT;
  int c16 = (int)(f % (slab_ch / 16)); f /= (slab_ch / 16);
  int slab = (int)(f % nslab); f /= nslab;
  int k = (int)(f % K);
  int pass = (int)(f / K);
  int m = (pass * MT + mt) * 32 + (l & 31), c = slab * slab_ch + c16 * 16 + 8 * (l >> 5) + j;
  Wt[id] = (m < M && c < Cin) ? W[m * sm + c * sc + k] : (uint16_t)0;
}

// ---- LDS-staged kernel for stride-1 convolutions over all nodes -----------------------
// The eight siblings of a group read their taps from ONE 4x4x4 block of neighbour slots,
// so the block is gathered once per group and channel (64 values) and then serves all
// 8 x K (sibling, tap) pairs from LDS: 3.4x fewer global gathers than per-tap gathering
// for the 27-tap kernel, and every operand of the MFMA loop comes out of LDS.
//
// Workgroup = 4 wavefronts = 256 columns = 32 sibling groups; wavefront w owns groups
// 8w .. 8w+7 (its own 64 columns), stages only those, and computes all output channels of
// a pass (MT row tiles).  The channel loop runs in slabs of kSlab = 2 input channels (one MFMA
// k-step per tap; short slabs keep a workgroup at 34 KiB of LDS, and with buffer loads (scalar
// base, one 32-bit offset a lane, nothing to mask) the kernel fits 128 VGPRs, so that four
// workgroups share a CU and fill one another's barrier gaps; with 64-bit addresses in registers
// it took 164 VGPRs and three workgroups, 6 % slower):
//   LDS X [kSlab][32 groups][80]  fp32: the neighbour blocks (wavefront-private parts)
//   LDS W [K][kSlab/2][MT][64]    fp32: the slab's weights in A-fragment order (shared)
// Group g sits at word 80*g + {0,2,8,10}[g&3]: with that skew the 32 lanes of a half
// wavefront (4 groups x 8 siblings, sibling offsets {0,1,4,5,16,17,20,21}) hit 32
// different banks for every tap.
// The next slab's gathers and weights are issued before the MFMA loop of the current
// slab and land in LDS after it, so their latency hides behind ~14k cycles of MFMA.
constexpr int kSlab = 2;
constexpr int kKSteps = kSlab / 2;  // MFMA k-steps (two channels each) per slab
constexpr int kGroupStride = 80;
constexpr int kPlane = 32 * kGroupStride;   // words per channel plane

__device__ inline int group_base(int g) {
  return g * kGroupStride + ((g & 1) << 1) + ((g & 2) << 2);
}

template <int MT, int K>
__global__ __launch_bounds__(256, 4) void conv_s1_f32_lds_kernel(ConvArgs a, float* __restrict__ out,
    const float* __restrict__ in, const float* __restrict__ Wt, int n_tiles) {
  constexpr int kWWords = K * kKSteps * MT * 64;          // weight words per (pass, slab)
  constexpr int kWVec = (kWWords / 4 + 255) / 256;  // float4 loads per thread
  __shared__ float sX[kSlab * kPlane];
  __shared__ __attribute__((aligned(16))) float sW[kWWords];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = xcd_tile(blockIdx.x, n_tiles);
  if (tile >= n_tiles) return;
  const int n0 = tile * kTileCols + wave * kWaveCols;
  const int r = lane & 31, kh = lane >> 5;
  const int nslab = (a.Cin + kSlab - 1) / kSlab;
  const int npass = (a.mtiles + MT - 1) / MT;
  const bool mirrored = a.slot[0] != 0;  // deconvolution walks the taps through the opposite offsets

  // neighbour rows of slot `lane` of my eight groups (kept for all slabs and passes), as byte
  // offsets into a channel of the input; a missing neighbour lies past any channel and reads as zero
  int nb[8];
  const int group0 = (tile * kTileCols) / 8 + wave * 8;
  const int n_groups = a.N >> 3;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    int g = group0 + j;
    int v = g < n_groups ? a.neigh[((int64_t)g << 6) + lane] : -1;
    nb[j] = (v >= 0 && v < a.Hin) ? v * 4 : (int)0x80000000u;
  }
  // LDS word offsets of my two B columns (channel plane and tap slot are added per read)
  int boff[2];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
    boff[nt] = group_base(wave * 8 + nt * 4 + (r >> 3)) + sibling_slot(r & 7) + kh * kPlane;

  for (int pass = blockIdx.y; pass < npass; pass += gridDim.y) {  // passes may be dealt out over workgroups
    floatx16 acc[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.0f;

    float xr[8][kSlab];
    float4 wr[kWVec];
    // Buffer loads: a scalar base and one 32-bit offset a lane, no 64-bit addresses in registers;
    // what lies past a buffer (a piece behind the slab's weights, a channel behind the last) reads as zero.
    auto fetch = [&](int slab) {
      const __amdgpu_buffer_rsrc_t wsrc = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<float*>(Wt) + ((int64_t)pass * nslab + slab) * kWWords, 0, kWWords * 4, 0x00020000);
#pragma unroll
      for (int v = 0; v < kWVec; ++v) {
        const u32x4 w4 = __builtin_amdgcn_raw_buffer_load_b128(wsrc, (v * 256 + (int)threadIdx.x) * 16, 0, 0);
        wr[v] = make_float4(__uint_as_float(w4[0]), __uint_as_float(w4[1]), __uint_as_float(w4[2]), __uint_as_float(w4[3]));
      }
#pragma unroll
      for (int cc = 0; cc < kSlab; ++cc) {
        const int c = slab * kSlab + cc;
        const __amdgpu_buffer_rsrc_t plane = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float*>(in) + (int64_t)c * a.Hin, 0, c < a.Cin ? a.Hin * 4 : 0, 0x00020000);
#pragma unroll
        for (int j = 0; j < 8; ++j)
          xr[j][cc] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(plane, nb[j], 0, 0));
      }
    };
    fetch(0);
    for (int slab = 0; slab < nslab; ++slab) {
      __syncthreads();  // everyone is done reading the previous slab
#pragma unroll
      for (int v = 0; v < kWVec; ++v) {
        int idx = v * 256 + threadIdx.x;
        if (idx < kWWords / 4) reinterpret_cast<float4*>(sW)[idx] = wr[v];
      }
#pragma unroll
      for (int cc = 0; cc < kSlab; ++cc)
#pragma unroll
        for (int j = 0; j < 8; ++j)
          sX[cc * kPlane + group_base(wave * 8 + j) + lane] = xr[j][cc];
      __syncthreads();
      if (slab + 1 < nslab) fetch(slab + 1);
      // taps in (dx, dy) pairs of three dz each: the slot of tap (dx, dy, dz) is dx<<4 | dy<<2 | dz
      // (mirrored: 42 minus that), computed instead of read from the argument block, so the loop
      // holds no scalar load to wait for
      static_assert(K == 27, "slot arithmetic below is the 3x3x3 kernel's");
#pragma unroll 1
      for (int kxy = 0; kxy < 9; ++kxy) {
        const int s3 = ((kxy / 3) << 4) | ((kxy % 3) << 2);
#pragma unroll
        for (int kz = 0; kz < 3; ++kz) {
          const int k = kxy * 3 + kz;
          const int slot = mirrored ? 42 - (s3 | kz) : (s3 | kz);
#pragma unroll
          for (int ks = 0; ks < kKSteps; ++ks) {
            float b0 = sX[boff[0] + ks * 2 * kPlane + slot];
            float b1 = sX[boff[1] + ks * 2 * kPlane + slot];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
              float av = sW[((k * kKSteps + ks) * MT + mt) * 64 + lane];
              acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, b0, acc[mt][0], 0, 0, 0);
              acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, b1, acc[mt][1], 0, 0, 0);
            }
          }
        }
      }
    }
    if (n0 < a.N) store_tiles<float, MT>(a, out, acc, pass * MT, n0, lane);
  }
}

// weights in the order the LDS kernel copies them: [pass][slab][tap][kstep][mt][lane]
__global__ void pack_weights_lds_f32(float* __restrict__ Wt, const float* __restrict__ W, int M, int Cin, int K,
    int MT, int npass, int nslab, int64_t sm, int64_t sc) {
  int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = (int64_t)npass * nslab * K * kKSteps * MT * 64;
  if (id >= total) return;
  int l = (int)(id & 63);
  int64_t f = id >> 6;
  int mt = (int)(f % MT); f /= MT;
  int ks = (int)(f % kKSteps); f /= kKSteps;
  int k = (int)(f % K); f /= K;
  int slab = (int)(f % nslab);
  int pass = (int)(f / nslab);
  int m = (pass * MT + mt) * 32 + (l & 31), c = slab * kSlab + 2 * ks + (l >> 5);
  Wt[id] = (m < M && c < Cin) ? W[m * sm + c * sc + k] : 0.0f;
}


// ---- LDS-staged bf16 kernel (3x3x3, stride 1, all nodes) ----------------------------------
// v_mfma_f32_32x32x16_bf16 wants 8 consecutive input channels of one column per lane, which
// the channel-major [C, H] tensor cannot deliver without eight 2-byte gathers.  So the input
// is first transposed to row-major [H + 1, Cpad] bf16 (row H is all zero and stands for a
// missing neighbour, Cpad = Cin rounded up to 16): a neighbour is then one contiguous row
// and every staged element moves as a 16-byte vector.
//
// Slab = 16 channels (one MFMA k-step per tap).  Per sibling group only two x-layers of the
// 4x4x4 block are resident (taps with offset dx read layers dx and dx+1): layer x lives in
// the units with bit0 == x&1 and layer x+2 overwrites layer x, so every slot is still
// gathered exactly once per slab.  The weights of the 9 taps of one dx sit next to it.
//   LDS X [2 halves of 8 channels][32 groups][32 units] x 16 B = 32 KiB
//   LDS W [9 taps][MT][64 lanes] x 16 B                        = 18 KiB (MT = 2)
// 50 KiB per workgroup: three workgroups per CU.  Unit index of slot (x,y,z):
//   (x&1) | (y&1)<<1 | (z&1)<<2 | (y>>1)<<3 | (z>>1)<<4
// so the 8 siblings of a group (consecutive lanes) always read 8 different 16-byte units;
// odd groups store unit u at u ^ 8 and the second channel half at u ^ 1 (see the kernel):
// with that, and the staging lanes ordered by the unit bits, no read or write of the kernel
// meets a bank conflict (SQ_LDS_BANK_CONFLICT = 0 on the depth-9 scene).
constexpr int kB16Half = 32 * 32;  // 16-byte units per 8-channel half

__device__ inline int b16_unit(int x, int y, int z) {
  return (x & 1) | ((y & 1) << 1) | ((z & 1) << 2) | ((y >> 1) << 3) | ((z >> 1) << 4);
}

// Row-major copy of a channel-major bf16 tensor: src [C, H] -> dst [H + 1, Cpad], row H zero.
// 64 channels x 128 rows per workgroup; reads are 4-byte (two rows of one
// channel) and coalesced per channel row, writes are 16-byte (8 channels of one row) and,
// for Cpad = 64, contiguous over the whole tile.
__global__ __launch_bounds__(256) void transpose_rows_bf16_kernel(uint16_t* __restrict__ dst,
    const uint16_t* __restrict__ src, int C, int H, int Cpad) {
  constexpr int kPitch = 130;  // halfwords; 8 channel rows apart = 8 banks apart
  __shared__ __attribute__((aligned(16))) uint16_t tile[64 * kPitch];
  const int h0 = blockIdx.x * 128, c0 = blockIdx.y * 64;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const bool even = (H & 1) == 0;
#pragma unroll 4
  for (int pass = 0; pass < 16; ++pass) {
    const int cl = pass * 4 + wave, c = c0 + cl, h = h0 + 2 * lane;
    uint32_t v = 0;
    if (c < C) {
      const uint16_t* p = src + (int64_t)c * H + h;
      if (even && h + 1 < H) v = *reinterpret_cast<const uint32_t*>(p);
      else {
        if (h < H) v = p[0];
        if (h + 1 < H) v |= (uint32_t)p[1] << 16;
      }
    }
    *reinterpret_cast<uint32_t*>(&tile[cl * kPitch + 2 * lane]) = v;
  }
  __syncthreads();
  const int cg = threadIdx.x & 7, hh = threadIdx.x >> 3;
  if (c0 + cg * 8 >= Cpad) return;
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    const int hl = pass * 32 + hh, h = h0 + hl;
    if (h > H) continue;
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      w[j] = (uint32_t)tile[(cg * 8 + 2 * j) * kPitch + hl] | ((uint32_t)tile[(cg * 8 + 2 * j + 1) * kPitch + hl] << 16);
    uint4 o = h < H ? make_uint4(w[0], w[1], w[2], w[3]) : make_uint4(0, 0, 0, 0);
    *reinterpret_cast<uint4*>(dst + (int64_t)h * Cpad + c0 + cg * 8) = o;
  }
}

// The inverse copy: row-major src [H + 1, pitch] -> channel-major dst [C, H] (64 rows x 64
// channels per workgroup; 16-byte reads of 8 channels of a row, 4-byte writes of two rows of a
// channel, coalesced per channel row).
__global__ __launch_bounds__(256) void transpose_channels_bf16_kernel(uint16_t* __restrict__ dst,
    const uint16_t* __restrict__ src, int C, int H, int pitch) {
  constexpr int kPitch = 66;  // halfwords per channel row of the tile
  __shared__ uint16_t tile[64 * kPitch];
  const int h0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
  const int t = threadIdx.x;
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int hl = pass * 32 + (t >> 3), cg = t & 7;
    const int h = h0 + hl, c = c0 + cg * 8;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (h < H && c < pitch) v = *reinterpret_cast<const uint4*>(src + (int64_t)h * pitch + c);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      tile[(cg * 8 + 2 * j) * kPitch + hl] = (uint16_t)(w[j] & 0xffff);
      tile[(cg * 8 + 2 * j + 1) * kPitch + hl] = (uint16_t)(w[j] >> 16);
    }
  }
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 16; ++pass) {
    const int cl = pass * 4 + (t >> 6), c = c0 + cl, h = h0 + (t & 63);
    if (c < C && h < H) dst[(int64_t)c * H + h] = tile[cl * kPitch + (t & 63)];
  }
}

// ROWS_OUT: the output is written row-major as well ([Hout + 1][out_pitch] bf16, row Hout zero); the
// input rows may be a slice of a wider tensor (pitch8: 16-byte units a row).
template <int MT, bool ROWS_OUT = false>
__global__ __launch_bounds__(256, 2) void conv_s1_bf16_lds_kernel(ConvArgs a, uint16_t* __restrict__ out,
    const u32x4* __restrict__ xt, const u32x4* __restrict__ Wt, int n_tiles, int cpad8, int pitch8 = 0,
    int out_pitch = 0, int out_cpad = 0) {
  if (pitch8 == 0) pitch8 = cpad8;
  constexpr int kWUnits = 9 * MT * 64;               // 16-byte units per weight chunk
  constexpr int kWVec = (kWUnits + 255) / 256;
  __shared__ u32x4 sX[2 * kB16Half];
  __shared__ u32x4 sW[kWUnits];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = xcd_tile(blockIdx.x, n_tiles);
  if (tile >= n_tiles) return;
  const int n0 = tile * kTileCols + wave * kWaveCols;
  const int r = lane & 31, kh = lane >> 5;
  const int nslab = cpad8 >> 1;                       // 16-channel slabs
  const int npass = (a.mtiles + MT - 1) / MT;

  // staging role of this lane: half s_kh, (y,z) = s_yz, groups 8*wave + 2*j + s_g (j = 0..3)
  // lane bits 1..4 are (y&1, z&1, y>>1, z>>1): sixteen consecutive lanes then write sixteen
  // different 16-byte units of one 256-byte row of banks (see the unit index above; the
  // second channel half keeps its units with bit 0 flipped)
  const int s_kh = lane & 1, s_g = lane >> 5;
  const int s_y = ((lane >> 1) & 1) | (((lane >> 3) & 1) << 1), s_z = ((lane >> 2) & 1) | (((lane >> 4) & 1) << 1);
  const int s_yz = (s_y << 2) | s_z;
  int nb[4][4];  // [j][x-layer] neighbour row (H = the zero row)
  const int group0 = (tile * kTileCols) / 8 + wave * 8;
  const int n_groups = a.N >> 3;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    int g = group0 + 2 * j + s_g;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      int v = g < n_groups ? a.neigh[((int64_t)g << 6) + (x << 4) + s_yz] : -1;
      nb[j][x] = (v >= 0 && v < a.Hin) ? v : a.Hin;
    }
  }
  // compute role: column r of each of the two column tiles, channel half kh
  const int sib = r & 7, si = sib >> 2, sj = (sib >> 1) & 1, sk = sib & 1;
  int cbase[2];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) cbase[nt] = kh * kB16Half + (wave * 8 + nt * 4 + (r >> 3)) * 32;
  // Odd groups keep their units with bit 3 flipped: a 16-byte LDS read is served sixteen lanes
  // (two sibling groups) at a time, and the blocks of two groups, 512 bytes apart, would meet in
  // the same banks.
  const int gswz = (((r >> 3) & 1) << 3) ^ kh;

  for (int pass = blockIdx.y; pass < npass; pass += gridDim.y) {  // passes may be dealt out over workgroups
    floatx16 acc[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.0f;

    // Phases: a slab has four, phase L stages x-layer L (into the units with bit0 == L&1;
    // layer L overwrites layer L-2, whose last readers finished before the phase's first
    // barrier) and, for L >= 1, the weights of the 9 taps with dx = L-1, then computes them.
    // Layer L of a later phase is requested two phases ahead into register set L&1, the
    // weights one phase ahead, so the requests have one or two compute phases to land.
    u32x4 xr[2][4];
    u32x4 wr[kWVec];
#define OCNN_FETCH_W(SLAB, DX)                                                                 \
    do {                                                                                       \
      const u32x4* wsrc = Wt + (((int64_t)pass * nslab + (SLAB)) * 3 + (DX)) * kWUnits;        \
      _Pragma("unroll") for (int v = 0; v < kWVec; ++v) {                                      \
        int idx = v * 256 + threadIdx.x;                                                       \
        wr[v] = idx < kWUnits ? wsrc[idx] : (u32x4)(0u);                                       \
      }                                                                                        \
    } while (0)
#define OCNN_FETCH_X(SLAB, L)                                                                  \
    do {                                                                                       \
      const int col = (SLAB) * 2 + s_kh;                                                       \
      _Pragma("unroll") for (int j = 0; j < 4; ++j)                                            \
        xr[(L) & 1][j] = xt[(int64_t)nb[j][L] * pitch8 + col];                                 \
    } while (0)
#define OCNN_PHASE(SLAB, L)                                                                    \
    do {                                                                                       \
      __syncthreads();                                                                         \
      if ((L) >= 1) {                                                                          \
        _Pragma("unroll") for (int v = 0; v < kWVec; ++v) {                                    \
          int idx = v * 256 + threadIdx.x;                                                     \
          if (idx < kWUnits) sW[idx] = wr[v];                                                  \
        }                                                                                      \
      }                                                                                        \
      _Pragma("unroll") for (int j = 0; j < 4; ++j)                                            \
        sX[s_kh * kB16Half + (wave * 8 + 2 * j + s_g) * 32 + (b16_unit(L, s_y, s_z) ^ (s_g << 3) ^ s_kh)] = xr[(L) & 1][j]; \
      __syncthreads();                                                                         \
      /* weights of the next computing phase: phase L requests those of dx = L */            \
      if ((L) <= 2) OCNN_FETCH_W(SLAB, L);                                                     \
      /* x-layer two phases ahead */                                                           \
      if ((L) <= 1) OCNN_FETCH_X(SLAB, (L) + 2);                                               \
      else if ((SLAB) + 1 < nslab) OCNN_FETCH_X((SLAB) + 1, (L) - 2);                          \
      if ((L) >= 1) {                                                                          \
        const int ux = ((L) - 1 + si) & 1;                                                     \
        _Pragma("unroll") for (int dy = 0; dy < 3; ++dy)                                       \
        _Pragma("unroll") for (int dz = 0; dz < 3; ++dz) {                                     \
          const int y = dy + sj, z = dz + sk;                                                  \
          const int unit = (ux | ((y & 1) << 1) | ((z & 1) << 2) | ((y >> 1) << 3) | ((z >> 1) << 4)) ^ gswz; \
          union { u32x4 q; bf16x8 v; } b0, b1;                                                 \
          b0.q = sX[cbase[0] + unit];                                                          \
          b1.q = sX[cbase[1] + unit];                                                          \
          _Pragma("unroll") for (int mt = 0; mt < MT; ++mt) {                                  \
            union { u32x4 q; bf16x8 v; } av;                                                   \
            av.q = sW[((dy * 3 + dz) * MT + mt) * 64 + lane];                                  \
            acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av.v, b0.v, acc[mt][0], 0, 0, 0); \
            acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av.v, b1.v, acc[mt][1], 0, 0, 0); \
          }                                                                                    \
        }                                                                                      \
      }                                                                                        \
    } while (0)
    OCNN_FETCH_X(0, 0);
    OCNN_FETCH_X(0, 1);
    for (int slab = 0; slab < nslab; ++slab) {
      OCNN_PHASE(slab, 0);
      OCNN_PHASE(slab, 1);
      OCNN_PHASE(slab, 2);
      OCNN_PHASE(slab, 3);
    }
#undef OCNN_FETCH_W
#undef OCNN_FETCH_X
#undef OCNN_PHASE
    if constexpr (ROWS_OUT) {
      rows_out_tiles<MT>(a, out, out_pitch, out_cpad, acc, pass * MT * 32, n0, lane);
      if (tile == 0 && wave == 0 && lane * 8 >= pass * MT * 32 && lane * 8 < min((pass + 1) * MT * 32, out_cpad))
        *reinterpret_cast<uint4*>(out + (int64_t)a.Hout * out_pitch + lane * 8) = make_uint4(0, 0, 0, 0);
    } else {
      if (n0 < a.N) store_tiles<uint16_t, MT>(a, out, acc, pass * MT, n0, lane);
    }
  }
}

// ---- register-fed bf16 kernel (3x3x3, stride 1, all nodes, large levels) ---------------------
// The LDS kernel above serves every (tap, sibling) pair with its own operand read, and its phases
// (gather -> LDS -> barrier -> compute) of two workgroups per CU do not hide one another.  Here a
// wavefront owns 32 sibling groups and ALL 8 siblings of each: its accumulators are 8 siblings x
// MT row tiles of 32x32 (256 registers for 64 output channels, the accumulation half of the
// register file at one wavefront per SIMD), MFMA column n is GROUP n, and the B operand of slot
// (x, y, z) -- lane (n, kh) holds 8 channels of the row found in that slot of group n's 4x4x4
// neighbour block -- serves every sibling (i, j, k) whose tap (x - i, y - j, z - k) exists: 6.75
// MFMAs per operand on average instead of 2.  So the operands come straight from the row-major
// copy into registers: every slot row is requested once per k-step, exactly as often as the LDS
// kernel stages it, nothing of the input passes through LDS and no barrier sits between a
// gather and its use.  The block is walked x-layer by x-layer (16 slots = 64 registers, the next
// layer in flight in a second set): layer L feeds the siblings with i = 0 through the taps
// dx = L and those with i = 1 through dx = L - 1.
// Weights: all 27 taps of one 16-channel k-step sit in LDS in A-fragment order (54 KiB for 64
// output channels), the next k-step's are copied in during the current one (two buffers, one
// barrier per k-step); a wavefront reads each tap's fragment twice per k-step, 0.25 KiB of LDS
// operands per MFMA.  The neighbour rows of a wavefront's groups wait in LDS too (68 words per
// group: 16-byte reads of 32 lanes then meet no bank twice).
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

// two fp32 values -> two bf16 in one word (round to nearest even, the conversion instruction of
// this GPU; the same values as f32_to_bf16 for everything that is not a NaN)
__device__ inline uint32_t pack_bf16x2(float lo, float hi) {
  floatx2 f = {lo, hi};
  bf16x2 h = __builtin_convertvector(f, bf16x2);
  return __builtin_bit_cast(uint32_t, h);
}
// max(v, floor) that keeps a NaN (floor = 0 for a ReLU, -inf for none)
__device__ inline float relu_floor(float v, float floor) { return v < floor ? floor : v; }

constexpr int kRegGroups = 32;               // sibling groups (MFMA columns) per wavefront
constexpr int kRegTileGroups = 4 * kRegGroups;
constexpr int kNbPitch = 68;

// ROWS_OUT: the output is written row-major as well ([Hout + 1][out_pitch] bf16, row Hout zero,
// channels from M up to the pitch zero), the layout the next convolution of a chain gathers
// from: 32 contiguous bytes per row and store instead of 16 bytes per channel and group.
template <int MT, bool ROWS_OUT>
__global__ __launch_bounds__(256, 1) void conv_s1_bf16_reg_kernel(ConvArgs a, uint16_t* __restrict__ out,
    const u32x4* __restrict__ xt, const u32x4* __restrict__ Wt, int n_tiles, int cpad8, int out_pitch, int out_cpad) {
  constexpr int kWUnits = 27 * MT * 64;        // 16-byte units of one k-step's weights
  constexpr int kWPiece = kWUnits / 4;         // copied per layer phase
  constexpr int kWVec = (kWPiece + 255) / 256;
  constexpr int kWVec0 = (kWUnits + 255) / 256;
  __shared__ u32x4 sW[2][kWUnits];
  __shared__ __attribute__((aligned(16))) int sNb[4][kRegGroups * kNbPitch];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = xcd_tile(blockIdx.x, n_tiles);
  if (tile >= n_tiles) return;
  const int n = lane & 31, kh = lane >> 5;
  const int nks = cpad8 >> 1;                  // 16-channel k-steps
  const int npass = (a.mtiles + MT - 1) / MT;
  const int n_groups = a.N >> 3;
  const int g0 = tile * kRegTileGroups + wave * kRegGroups;
  const int row_bytes = cpad8 * 16;
  const int half = kh * 16;

  // the row-major copy and the packed weights as buffers: 32-bit offsets per lane, the k-step's
  // column / the piece of the weights as the scalar offset (the host sends levels beyond 2 GiB
  // to the other kernel)
  const int xrows_bytes = (int)(((int64_t)a.Hin + 1) * row_bytes);
  const __amdgpu_buffer_rsrc_t xrows = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<u32x4*>(xt), 0, xrows_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t wbuf = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<u32x4*>(Wt), 0, npass * nks * kWUnits * 16, 0x00020000);

  // Set-up, all requests in flight before the first is looked at: the neighbour tables of my
  // 32 groups (8 KiB in one piece, eight 16-byte loads per lane) and the first k-step's weights
  // of the first pass.  The tables go to LDS as byte offsets of the rows (a missing neighbour and
  // anything beyond the level = row Hin, which is all zero).
  int pass = blockIdx.y;
  {
    const int u0 = g0 * 16;                       // my first 16-byte unit of the level's table
    const int4* nsrc = reinterpret_cast<const int4*>(a.neigh);
    const int last = n_groups * 16 - 1;
    int4 nv[8];
    u32x4 w0[kWVec0];
#pragma unroll
    for (int j = 0; j < 8; ++j) nv[j] = nsrc[min(u0 + j * 64 + lane, last)];
#pragma unroll
    for (int v = 0; v < kWVec0; ++v)
      w0[v] = __builtin_amdgcn_raw_buffer_load_b128(wbuf, min(v * 256 + (int)threadIdx.x, kWUnits - 1) * 16,
          pass * nks * kWUnits * 16, 0);
    const unsigned hin = (unsigned)a.Hin;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int u = j * 64 + lane;               // group u >> 4, slots 4 (u & 15) ...
      const unsigned gone = (unsigned)((last - (u0 + u)) >> 31);   // all ones past the end of the table
      int4 o;
      o.x = (int)(min((unsigned)nv[j].x | gone, hin) * (unsigned)row_bytes);
      o.y = (int)(min((unsigned)nv[j].y | gone, hin) * (unsigned)row_bytes);
      o.z = (int)(min((unsigned)nv[j].z | gone, hin) * (unsigned)row_bytes);
      o.w = (int)(min((unsigned)nv[j].w | gone, hin) * (unsigned)row_bytes);
      *reinterpret_cast<int4*>(&sNb[wave][(u >> 4) * kNbPitch + 4 * (u & 15)]) = o;
    }
#pragma unroll
    for (int v = 0; v < kWVec0; ++v) sW[0][min(v * 256 + (int)threadIdx.x, kWUnits - 1)] = w0[v];
  }

  u32x4 bl[2][16];   // two x-layers of operands: [buffer][y*4 + z]
  u32x4 wr[kWVec];
  // requests the 4 slot rows (Y, 0..3) of layer L at k-step KS into buffer L & 1
#define OCNN_REQ_ROW(BUF, KS, L, Y)                                                             \
  do {                                                                                          \
    const int4 rows = *reinterpret_cast<const int4*>(&sNb[wave][n * kNbPitch + (L) * 16 + (Y) * 4]); \
    const int col = (KS) * 32;                                                                  \
    bl[(L) & 1][(Y) * 4 + 0] = __builtin_amdgcn_raw_buffer_load_b128(BUF, rows.x + half, col, 0); \
    bl[(L) & 1][(Y) * 4 + 1] = __builtin_amdgcn_raw_buffer_load_b128(BUF, rows.y + half, col, 0); \
    bl[(L) & 1][(Y) * 4 + 2] = __builtin_amdgcn_raw_buffer_load_b128(BUF, rows.z + half, col, 0); \
    bl[(L) & 1][(Y) * 4 + 3] = __builtin_amdgcn_raw_buffer_load_b128(BUF, rows.w + half, col, 0); \
  } while (0)
  // Layer L + 2 (of this k-step, or layer L - 2 of the next) takes over the registers of layer L
  // row by row as the rows die: row y is last used by the taps with dy = min(y, 2).  Its first
  // rows are then under way for a phase and two thirds before the phase that multiplies them
  // starts, the last ones for a phase and a third.
#define OCNN_REFILL(KS, L, Y)                                                                   \
  do {                                                                                          \
    if ((L) < 2) OCNN_REQ_ROW(xrows, KS, (L) + 2, Y);                                           \
    else OCNN_REQ_ROW(xnext, ks_next, (L) - 2, Y);                                              \
    /* the requests stay where they are (the scheduler would sink them to their first use    \
       to save registers) */                                                                   \
    __builtin_amdgcn_sched_barrier(0);                                                          \
  } while (0)
  // One layer phase: a quarter of the next k-step's weights on their way, the layer multiplied
  // into the siblings it reaches, the weights parked in LDS.  No branches (a thread past the end
  // of the piece copies its last unit once more; the last k-step copies the first weights of the
  // next pass, or its own, and its requests for "the next k-step" go through a buffer of size
  // zero: they cost an issue slot, touch no memory and return at once): one basic block per
  // phase, so the waits the compiler places count exactly the requests that must have landed.
#define OCNN_LAYER_PHASE(KS, L)                                                                 \
  do {                                                                                          \
    {                                                                                           \
      /* a thread's units inside a piece: computed here every time, four registers are worth   \
         more than eight additions */                                                          \
      int tid = threadIdx.x;                                                                    \
      asm volatile("" : "+v"(tid));                                                             \
      _Pragma("unroll") for (int v = 0; v < kWVec; ++v)                                         \
        wr[v] = __builtin_amdgcn_raw_buffer_load_b128(wbuf, min(v * 256 + tid, kWPiece - 1) * 16, \
            wsrc + (L) * kWPiece * 16, 0);                                                      \
    }                                                                                           \
    __builtin_amdgcn_sched_barrier(0);                                                          \
    /* work items of the layer: (dy, dz) x the sibling halves it reaches; the weights of      \
       item t + 1 are read from LDS before the multiplications of item t are issued */          \
    {                                                                                           \
      constexpr int kBoth = ((L) == 1 || (L) == 2) ? 1 : 0;                                     \
      constexpr int kItems = kBoth ? 18 : 9;                                                    \
      union { u32x4 q; bf16x8 v; } av[2][MT];                                                   \
      _Pragma("unroll") for (int mt = 0; mt < MT; ++mt)                                         \
        av[0][mt].q = wcur[(((L) == 3 ? 2 : (L)) * 9 * MT + mt) * 64 + lane];                   \
      __builtin_amdgcn_sched_group_barrier(0x100, MT, 0);                                       \
      _Pragma("unroll") for (int it = 0; it < kItems; ++it) {                                   \
        /* issue order: the reads of the next item, then this item's multiplications */       \
        __builtin_amdgcn_sched_group_barrier(0x100, MT, 0);                                     \
        __builtin_amdgcn_sched_group_barrier(0x008, 4 * MT, 0);                                 \
        if (it + 1 < kItems) {                                                                  \
          const int nyz = kBoth ? (it + 1) >> 1 : it + 1;                                       \
          const int nsi = kBoth ? (it + 1) & 1 : ((L) == 3 ? 1 : 0);                            \
          _Pragma("unroll") for (int mt = 0; mt < MT; ++mt)                                     \
            av[(it + 1) & 1][mt].q = wcur[((((L) - nsi) * 9 + nyz) * MT + mt) * 64 + lane];     \
        }                                                                                       \
        const int yz = kBoth ? it >> 1 : it, si = kBoth ? it & 1 : ((L) == 3 ? 1 : 0);          \
        const int dy = yz / 3, dz = yz % 3;                                                     \
        _Pragma("unroll") for (int sj = 0; sj < 2; ++sj)                                        \
        _Pragma("unroll") for (int sk = 0; sk < 2; ++sk) {                                      \
          union { u32x4 q; bf16x8 v; } bv;                                                      \
          bv.q = bl[(L) & 1][(dy + sj) * 4 + (dz + sk)];                                        \
          _Pragma("unroll") for (int mt = 0; mt < MT; ++mt)                                     \
            acc[si * 4 + sj * 2 + sk][mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(            \
                av[it & 1][mt].v, bv.v, acc[si * 4 + sj * 2 + sk][mt], 0, 0, 0);                \
        }                                                                                       \
        if (it + 1 == kItems / 3) OCNN_REFILL(KS, L, 0);                                        \
        if (it + 1 == 2 * kItems / 3) OCNN_REFILL(KS, L, 1);                                    \
      }                                                                                         \
      OCNN_REFILL(KS, L, 2);                                                                    \
      OCNN_REFILL(KS, L, 3);                                                                    \
    }                                                                                           \
    _Pragma("unroll") for (int v = 0; v < kWVec; ++v)                                           \
      wnext[(L) * kWPiece + min(v * 256 + (int)threadIdx.x, kWPiece - 1)] = wr[v];              \
  } while (0)

  int wbase = 0;   // LDS buffer of a pass's first k-step
  for (; pass < npass; pass += gridDim.y) {   // passes may be dealt out over workgroups
#pragma unroll
    for (int y = 0; y < 4; ++y) { OCNN_REQ_ROW(xrows, 0, 0, y); }
#pragma unroll
    for (int y = 0; y < 4; ++y) { OCNN_REQ_ROW(xrows, 0, 1, y); }

    // lane (n, kh) holds rows m0 + 32 mt + 8 (i / 4) + i % 4 of columns 8 (g0 + n) .. + 7
    const int m0 = pass * MT * 32 + 4 * kh;
    floatx16 acc[8][MT];
#pragma unroll
    for (int sb = 0; sb < 8; ++sb)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[sb][mt][i] = 0.0f;

    const int wpass = pass * nks * kWUnits * 16;   // byte offsets into the packed weights
    const int wfirst = (pass + (int)gridDim.y < npass ? pass + (int)gridDim.y : pass) * nks * kWUnits * 16;
    for (int ks = 0; ks < nks; ++ks) {
      __syncthreads();   // this k-step's weights are in LDS; the other buffer is free
      const u32x4* wcur = sW[(wbase + ks) & 1];
      u32x4* wnext = sW[(wbase + ks + 1) & 1];
      const int ks_next = min(ks + 1, nks - 1);
      const __amdgpu_buffer_rsrc_t xnext = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<u32x4*>(xt), 0, ks + 1 < nks ? xrows_bytes : 0, 0x00020000);
      const int wsrc = ks + 1 < nks ? wpass + (ks + 1) * kWUnits * 16 : wfirst;
      OCNN_LAYER_PHASE(ks, 0);
      OCNN_LAYER_PHASE(ks, 1);
      OCNN_LAYER_PHASE(ks, 2);
      OCNN_LAYER_PHASE(ks, 3);
    }
    wbase = (wbase + nks) & 1;

    const int g = g0 + n;
    if constexpr (ROWS_OUT) {
      // Lane (n, kh) holds channels cb + 32 mt + 8 q + 4 kh + r (q, r = 0..3) of the 8 rows of its
      // group.  The two lanes of a group swap halves (lanes 0-31 against 32-63), so that kh = 0 ends
      // up with channels 16 j .. + 7 and kh = 1 with 16 j + 8 .. + 15 of (mt, j): one 16-byte store
      // each, 32 contiguous bytes per row.
      const int cb = pass * MT * 32;
      // stores through a buffer: a lane whose group lies behind the level gets an offset past the
      // end and the hardware drops its store (no branch per store); the offsets have 32 bits (the
      // host sends larger outputs elsewhere)
      const __amdgpu_buffer_rsrc_t obuf = __builtin_amdgcn_make_buffer_rsrc(
          out, 0, (int)(((int64_t)a.Hout + 1) * out_pitch * 2), 0x00020000);
      const int obase = g < n_groups ? (g * 8 * out_pitch + cb + 8 * kh) * 2 : 0x7fffff00;
      auto store_rows = [&](auto value) {   // value(sb, mt, i): what goes out for accumulator i
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int sb = 0; sb < 8; ++sb) {
            uint32_t w[4][2];
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
              for (int h = 0; h < 2; ++h)
                w[q][h] = pack_bf16x2(value(sb, mt, 4 * q + 2 * h), value(sb, mt, 4 * q + 2 * h + 1));
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              const auto s0 = __builtin_amdgcn_permlane32_swap(w[2 * j][0], w[2 * j + 1][0], false, false);
              const auto s1 = __builtin_amdgcn_permlane32_swap(w[2 * j][1], w[2 * j + 1][1], false, false);
              // channels cb + 32 mt + 16 j .. + 15 (8 in each lane of the pair): inside the pitch or not
              // for the whole wavefront
              store16_then_wait(store16_t{s0[0], s1[0], s0[1], s1[1]}, obuf, obase,
                  (sb * out_pitch + 32 * mt + 16 * j) * 2, cb + 32 * mt + 16 * j < out_cpad);
            }
          }
      };
      if (!a.bias && !a.relu) {
        store_rows([&](int sb, int mt, int i) { return acc[sb][mt][i]; });
      } else {
        const float floor = a.relu ? 0.0f : -__builtin_inff();
        float bias[MT][16];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int ch = m0 + 32 * mt + 8 * (i / 4) + (i % 4);
            bias[mt][i] = a.bias ? a.bias[min(ch, a.M - 1)] : 0.0f;
            if (ch >= a.M) bias[mt][i] = 0.0f;   // the padding channels of a row stay zero
          }
        store_rows([&](int sb, int mt, int i) { return relu_floor(acc[sb][mt][i] + bias[mt][i], floor); });
      }
      // the all-zero row behind the last one (what a missing neighbour reads): once per pass range
      if (tile == 0 && wave == 0 && lane * 8 < out_cpad && lane * 8 >= cb && lane * 8 < cb + MT * 32)
        *reinterpret_cast<uint4*>(out + (int64_t)a.Hout * out_pitch + lane * 8) = make_uint4(0, 0, 0, 0);
      continue;
    }
    // one 16-byte store per output channel: the 8 columns of a group are contiguous
    uint16_t* orow = out + (int64_t)g * 8 + (int64_t)m0 * a.Hout;
    const int m_left = g < n_groups ? a.M - m0 : 0;   // rows of mine that exist
    // Straight-line code; the conversion is the hardware's (round to nearest even).  The plain
    // operator (no bias, no ReLU: what the reference's octree_conv is) only converts and stores.
    if (!a.bias && !a.relu) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int dm = 32 * mt + 8 * (i / 4) + (i % 4);
          uint32_t w[4];
#pragma unroll
          for (int sp = 0; sp < 4; ++sp) w[sp] = pack_bf16x2(acc[2 * sp][mt][i], acc[2 * sp + 1][mt][i]);
          if (dm < m_left)
            *reinterpret_cast<uint4*>(orow + (int64_t)dm * a.Hout) = make_uint4(w[0], w[1], w[2], w[3]);
        }
      continue;
    }
    // the biases of my rows are fetched together, the ReLU is a maximum with 0 or -inf
    const float floor = a.relu ? 0.0f : -__builtin_inff();
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      float bias[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) bias[i] = 0.0f;
      if (a.bias) {
#pragma unroll
        for (int i = 0; i < 16; ++i) bias[i] = a.bias[min(m0 + 32 * mt + 8 * (i / 4) + (i % 4), a.M - 1)];
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int dm = 32 * mt + 8 * (i / 4) + (i % 4);
        uint32_t w[4];
#pragma unroll
        for (int sp = 0; sp < 4; ++sp)
          w[sp] = pack_bf16x2(relu_floor(acc[2 * sp][mt][i] + bias[i], floor),
                              relu_floor(acc[2 * sp + 1][mt][i] + bias[i], floor));
        if (dm < m_left)
          *reinterpret_cast<uint4*>(orow + (int64_t)dm * a.Hout) = make_uint4(w[0], w[1], w[2], w[3]);
      }
    }
  }
#undef OCNN_REQ_ROW
#undef OCNN_REFILL
#undef OCNN_LAYER_PHASE
}

// weights for the bf16 LDS kernel: [pass][slab][dx][dy*3+dz][mt][lane][8 channels]; the tap
// index counts geometric offsets, so a deconvolution (which gathers through the mirrored
// offset) reads weight tap 26 - k
__global__ void pack_weights_lds_bf16(uint16_t* __restrict__ Wt, const uint16_t* __restrict__ W, int M, int Cin,
    int MT, int npass, int nslab, int64_t sm, int64_t sc, int mirror) {
  int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = (int64_t)npass * nslab * 27 * MT * 64 * 8;
  if (id >= total) return;
  int j = (int)(id & 7);
  int l = (int)((id >> 3) & 63);
  int64_t f = id >> 9;
  int mt = (int)(f % MT); f /= MT;
  int k = (int)(f % 27); f /= 27;
  int slab = (int)(f % nslab);
  int pass = (int)(f / nslab);
  int m = (pass * MT + mt) * 32 + (l & 31), c = slab * 16 + 8 * (l >> 5) + j;
  int kw = mirror ? 26 - k : k;
  Wt[id] = (m < M && c < Cin) ? W[m * sm + c * sc + kw] : (uint16_t)0;
}


// ---- 2x2x2 stride-2 convolution over all nodes ----------------------------------------------
//   out[co, h] = sum_ci sum_s W[co, ci*8 + s] * x[ci, 8h + s]
// The 8 taps of column h are the 8 children of parent h: 32 contiguous bytes (fp32) per
// channel.  Lane (n, kh) of a column tile loads ONE float4 = taps 4kh .. 4kh+3 of column n, so
// a wavefront load is a fully coalesced 1-KiB read and every input element is read exactly
// once; the four values feed four MFMA k-steps whose k-pairs are (tap j, tap 4+j) -- the
// weights are packed in that order.  HBM-bound at Cin = Cout = 64 (28 flop/byte).
constexpr int kS2Slab = 4;  // input channels per weight slab (fp32): with 8 the kernel needs 160 registers beside 84 of
                            // the second file (two wavefronts a SIMD); with 4 and three asked for, 148 in all: 9 % faster

template <int MT>
__global__ __launch_bounds__(256, 3) void conv_s2_f32_kernel(ConvArgs a, float* __restrict__ out,
    const float* __restrict__ in, const float* __restrict__ Wt, int n_tiles) {
  constexpr int kWWords = kS2Slab * 4 * MT * 64;
  constexpr int kWVec = (kWWords / 4 + 255) / 256;
  __shared__ __attribute__((aligned(16))) float sW[kWWords];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = xcd_tile(blockIdx.x, n_tiles);
  if (tile >= n_tiles) return;
  const int n0 = tile * kTileCols + wave * kWaveCols;
  const int r = lane & 31, kh = lane >> 5;
  const int nslab = (a.Cin + kS2Slab - 1) / kS2Slab;
  const int npass = (a.mtiles + MT - 1) / MT;
  // my float4 inside a channel row, per column tile.  Columns beyond N are clamped (computed, never
  // stored) and channels beyond Cin read channel Cin - 1 (their weights are zero), so the loads
  // carry no branch and stay in flight across the MFMAs.
  const float* xbase[2];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) xbase[nt] = in + (int64_t)min(n0 + nt * 32 + r, a.N - 1) * 8 + 4 * kh;
  float4 b[kS2Slab][2];
  auto load_x = [&](int slab, int cc) {
    const int c = min(slab * kS2Slab + cc, a.Cin - 1);
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) b[cc][nt] = *reinterpret_cast<const float4*>(xbase[nt] + (int64_t)c * a.Hin);
  };
  // my passes: blockIdx.y, + gridDim.y, ... (a level of few tiles deals its passes out over workgroups);
  // stages are counted over those
  const int my_passes = ((int)blockIdx.y < npass) ? (npass - (int)blockIdx.y + (int)gridDim.y - 1) / (int)gridDim.y : 0;
  const int nstage = my_passes * nslab;
  float4 wr[kWVec];
  auto fetch_w = [&](int stage) {   // stage of my own count -> (pass, slab) of the packed weights
    const int at = ((int)blockIdx.y + (stage / nslab) * (int)gridDim.y) * nslab + stage % nslab;
    const float4* wsrc = reinterpret_cast<const float4*>(Wt + (int64_t)at * kWWords);
#pragma unroll
    for (int v = 0; v < kWVec; ++v) {
      int idx = v * 256 + threadIdx.x;
      wr[v] = idx < kWWords / 4 ? wsrc[idx] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  };
  if (my_passes == 0) return;
  fetch_w(0);
#pragma unroll
  for (int cc = 0; cc < kS2Slab; ++cc) load_x(0, cc);
  for (int mine = 0; mine < my_passes; ++mine) {
    const int pass = (int)blockIdx.y + mine * (int)gridDim.y;
    floatx16 acc[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.0f;
    for (int slab = 0; slab < nslab; ++slab) {
      const int stage = mine * nslab + slab;
      __syncthreads();
#pragma unroll
      for (int v = 0; v < kWVec; ++v) {
        int idx = v * 256 + threadIdx.x;
        if (idx < kWWords / 4) reinterpret_cast<float4*>(sW)[idx] = wr[v];
      }
      __syncthreads();
      const bool more = stage + 1 < nstage;
      if (more) fetch_w(stage + 1);
      const int next_slab = slab + 1 < nslab ? slab + 1 : 0;
#pragma unroll
      for (int cc = 0; cc < kS2Slab; ++cc) {
        const float4 c0 = b[cc][0], c1 = b[cc][1];
        if (more) load_x(next_slab, cc);  // the next slab's channel takes the registers just read
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float b0 = j == 0 ? c0.x : j == 1 ? c0.y : j == 2 ? c0.z : c0.w;
          const float b1 = j == 0 ? c1.x : j == 1 ? c1.y : j == 2 ? c1.z : c1.w;
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            float av = sW[((cc * 4 + j) * MT + mt) * 64 + lane];
            acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, b0, acc[mt][0], 0, 0, 0);
            acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, b1, acc[mt][1], 0, 0, 0);
          }
        }
      }
    }
    if (n0 < a.N) store_tiles<float, MT>(a, out, acc, pass * MT, n0, lane);
  }
}
// [pass][slab][cc][j][mt][lane]: lane (m, kh) <- W[m][(slab*kS2Slab+cc)*8 + 4kh + j]
__global__ void pack_weights_s2_f32(float* __restrict__ Wt, const float* __restrict__ W, int M, int Cin, int MT,
    int npass, int nslab) {
  int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = (int64_t)npass * nslab * kS2Slab * 4 * MT * 64;
  if (id >= total) return;
  int l = (int)(id & 63);
  int64_t f = id >> 6;
  int mt = (int)(f % MT); f /= MT;
  int j = (int)(f % 4); f /= 4;
  int cc = (int)(f % kS2Slab); f /= kS2Slab;
  int slab = (int)(f % nslab);
  int pass = (int)(f / nslab);
  int m = (pass * MT + mt) * 32 + (l & 31), c = slab * kS2Slab + cc;
  Wt[id] = (m < M && c < Cin) ? W[(int64_t)m * Cin * 8 + c * 8 + 4 * (l >> 5) + j] : 0.0f;
}

// bf16: one 16-byte load = all 8 taps of (channel ci0 + kh, column n); an MFMA k-step of 16
// covers two input channels.  Slab = 8 channels = 4 k-steps.
// (The occupancy asked for in the launch bounds matters: left to itself the compiler puts the
// accumulators into the second register file beside 114 registers of the first and two wavefronts
// fit a SIMD; asked for three it keeps everything in 114 registers, four fit, and the kernel is a
// quarter faster.  The same holds for the wide-channel stride-2 deconvolution below.)
template <int MT>
__global__ __launch_bounds__(256, 3) void conv_s2_bf16_kernel(ConvArgs a, uint16_t* __restrict__ out,
    const uint16_t* __restrict__ in, const uint4* __restrict__ Wt, int n_tiles) {
  constexpr int kWUnits = 4 * MT * 64;
  __shared__ uint4 sW[kWUnits];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = xcd_tile(blockIdx.x, n_tiles);
  if (tile >= n_tiles) return;
  const int n0 = tile * kTileCols + wave * kWaveCols;
  const int r = lane & 31, kh = lane >> 5;
  const int nslab = (a.Cin + 7) / 8;
  const int npass = (a.mtiles + MT - 1) / MT;
  int64_t xoff[2];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
    int n = n0 + nt * 32 + r;
    xoff[nt] = n < a.N ? (int64_t)n * 8 : -1;
  }
  for (int pass = blockIdx.y; pass < npass; pass += gridDim.y) {   // passes may be dealt out over workgroups
    floatx16 acc[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.0f;
    for (int slab = 0; slab < nslab; ++slab) {
      __syncthreads();
      for (int idx = threadIdx.x; idx < kWUnits; idx += 256)
        sW[idx] = Wt[((int64_t)pass * nslab + slab) * kWUnits + idx];
      __syncthreads();
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int c = slab * 8 + 2 * q + kh;
        union { uint4 v4; bf16x8 v; } b0, b1;
        b0.v4 = (c < a.Cin && xoff[0] >= 0) ? *reinterpret_cast<const uint4*>(in + (int64_t)c * a.Hin + xoff[0])
                                            : make_uint4(0, 0, 0, 0);
        b1.v4 = (c < a.Cin && xoff[1] >= 0) ? *reinterpret_cast<const uint4*>(in + (int64_t)c * a.Hin + xoff[1])
                                            : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          union { uint4 v4; bf16x8 v; } av;
          av.v4 = sW[(q * MT + mt) * 64 + lane];
          acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av.v, b0.v, acc[mt][0], 0, 0, 0);
          acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av.v, b1.v, acc[mt][1], 0, 0, 0);
        }
      }
    }
    if (n0 < a.N) store_tiles<uint16_t, MT>(a, out, acc, pass * MT, n0, lane);
  }
}
// [pass][slab][q][mt][lane][j]: lane (m, kh), tap j <- W[m][(slab*8 + 2q + kh)*8 + j]
__global__ void pack_weights_s2_bf16(uint16_t* __restrict__ Wt, const uint16_t* __restrict__ W, int M, int Cin,
    int MT, int npass, int nslab) {
  int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = (int64_t)npass * nslab * 4 * MT * 64 * 8;
  if (id >= total) return;
  int j = (int)(id & 7);
  int l = (int)((id >> 3) & 63);
  int64_t f = id >> 9;
  int mt = (int)(f % MT); f /= MT;
  int q = (int)(f % 4); f /= 4;
  int slab = (int)(f % nslab);
  int pass = (int)(f / nslab);
  int m = (pass * MT + mt) * 32 + (l & 31), c = slab * 8 + 2 * q + (l >> 5);
  Wt[id] = (m < M && c < Cin) ? W[(int64_t)m * Cin * 8 + c * 8 + j] : (uint16_t)0;
}

// ---- 2x2x2 stride-2 convolution, row-major bf16 on both sides, padded ---------------------------
// Column = node t of the coarser level, ALL of them: the pad that the reference's modules apply
// after a stride-2 convolution (pytorch/ocnn/octree_conv.py:102-127) is part of the operator.
// The operand of a column is the 8 rows of the node's children, which are consecutive rows of the
// input: y[t] = sum_j W_j x[8 child[t] + j]; an empty node has no children, reads zeros and ends up
// with the bias alone.  An MFMA k-step is (child j, 16 channels): lane (n, kh) loads 16 contiguous
// bytes of row 8 child + j.  The k-steps are numbered j * ksteps + ks and staged eight at a time:
// their weights wait in LDS (two buffers, one barrier per stage), the next stage's are on their
// way meanwhile.  Output rows as the 3x3x3 row-major kernel writes them.
constexpr int kS2Stage = 8;   // k-steps per weight stage
template <int MT>
__global__ __launch_bounds__(256, 3) void conv_s2_rows_bf16_kernel(ConvArgs a, uint16_t* __restrict__ out,
    int out_pitch, int out_cpad, const u32x4* __restrict__ xt, int in_pitch, int in_cpad,
    const u32x4* __restrict__ Wt, int n_tiles) {
  constexpr int kStageUnits = kS2Stage * MT * 64;
  constexpr int kWVec = kStageUnits / 256;
  __shared__ u32x4 sW[2][kStageUnits];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = xcd_tile(blockIdx.x, n_tiles);
  if (tile >= n_tiles) return;
  const int n0 = tile * kTileCols + wave * kWaveCols;
  const int r = lane & 31, kh = lane >> 5;
  const int row_bytes = in_pitch * 2;
  const int ksteps = in_cpad >> 4;           // 16-channel k-steps per child = stages (8 children)
  const int npass = (a.mtiles + MT - 1) / MT;
  const __amdgpu_buffer_rsrc_t xrows = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<u32x4*>(xt), 0, (int)(((int64_t)a.Hin + 1) * row_bytes), 0x00020000);
  const __amdgpu_buffer_rsrc_t obuf = __builtin_amdgcn_make_buffer_rsrc(
      out, 0, (int)(((int64_t)a.Hout + 1) * out_pitch * 2), 0x00020000);
  // byte offset of the first child's row; a column without children (or behind the level) reads
  // past the end of the buffer, which yields zeros
  int xoff[2], ooff[2];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
    const int n = n0 + nt * 32 + r;
    const int c = n < a.N ? a.child[n] : -1;
    xoff[nt] = c >= 0 ? c * 8 * row_bytes + kh * 16 : 0x7fffff00;
    ooff[nt] = n < a.N ? (n * out_pitch + 8 * kh) * 2 : 0x7fffff00;
  }
  for (int pass = blockIdx.y; pass < npass; pass += gridDim.y) {
    floatx16 acc[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.0f;
    const u32x4* wpass = Wt + (int64_t)pass * ksteps * kStageUnits;
    u32x4 wr[kWVec];
#pragma unroll
    for (int v = 0; v < kWVec; ++v) wr[v] = wpass[v * 256 + threadIdx.x];
    __syncthreads();   // the previous pass has left the buffers
#pragma unroll
    for (int v = 0; v < kWVec; ++v) sW[0][v * 256 + threadIdx.x] = wr[v];
    int j = 0, ks = 0;   // child and channel step of the stage's first k-step
    for (int st = 0; st < ksteps; ++st) {
      __syncthreads();   // this stage's weights are in LDS; the other buffer is free
      const u32x4* wnext = wpass + (int64_t)min(st + 1, ksteps - 1) * kStageUnits;
#pragma unroll
      for (int v = 0; v < kWVec; ++v) wr[v] = wnext[v * 256 + threadIdx.x];
      union { u32x4 q; bf16x8 v; } b[kS2Stage][2];
#pragma unroll
      for (int t = 0; t < kS2Stage; ++t) {
        const int so = j * row_bytes + ks * 32;
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) b[t][nt].q = __builtin_amdgcn_raw_buffer_load_b128(xrows, xoff[nt], so, 0);
        if (++ks == ksteps) { ks = 0; ++j; }
      }
      const u32x4* wcur = sW[st & 1];
#pragma unroll
      for (int t = 0; t < kS2Stage; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          union { u32x4 q; bf16x8 v; } av;
          av.q = wcur[(t * MT + mt) * 64 + lane];
          acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av.v, b[t][0].v, acc[mt][0], 0, 0, 0);
          acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av.v, b[t][1].v, acc[mt][1], 0, 0, 0);
        }
#pragma unroll
      for (int v = 0; v < kWVec; ++v) sW[(st + 1) & 1][v * 256 + threadIdx.x] = wr[v];
    }
    // rows out: lane (r, kh) holds channels cb + 32 mt + 8 q + 4 kh + e of its two nodes; the lanes
    // of a pair swap halves and store 16 bytes each (see conv_s1_bf16_reg_kernel)
    const int cb = pass * MT * 32;
    const float floor = a.relu ? 0.0f : -__builtin_inff();
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      float bias[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int ch = cb + 32 * mt + 8 * (i / 4) + 4 * kh + (i % 4);
        bias[i] = a.bias ? a.bias[min(ch, a.M - 1)] : 0.0f;
        if (ch >= a.M) bias[i] = 0.0f;
      }
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        uint32_t w[4][2];
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const int i = 4 * q + 2 * h;
            w[q][h] = pack_bf16x2(relu_floor(acc[mt][nt][i] + bias[i], floor),
                                  relu_floor(acc[mt][nt][i + 1] + bias[i + 1], floor));
          }
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
          const auto s0 = __builtin_amdgcn_permlane32_swap(w[2 * jj][0], w[2 * jj + 1][0], false, false);
          const auto s1 = __builtin_amdgcn_permlane32_swap(w[2 * jj][1], w[2 * jj + 1][1], false, false);
          store16_then_wait(store16_t{s0[0], s1[0], s0[1], s1[1]}, obuf, ooff[nt], (cb + 32 * mt + 16 * jj) * 2,
              cb + 32 * mt + 16 * jj < out_cpad);
        }
      }
    }
    if (tile == 0 && wave == 0 && lane * 8 >= cb && lane * 8 < min(cb + MT * 32, out_cpad))
      *reinterpret_cast<uint4*>(out + (int64_t)a.Hout * out_pitch + lane * 8) = make_uint4(0, 0, 0, 0);
  }
}
// [pass][t = j * ksteps + ks][mt][lane][e]: lane (m, kh) <- W[m][(16 ks + 8 kh + e) * 8 + j]
__global__ void pack_weights_s2_rows_bf16(uint16_t* __restrict__ Wt, const uint16_t* __restrict__ W, int M, int Cin,
    int MT, int npass, int ksteps) {
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = (int64_t)npass * 8 * ksteps * MT * 64 * 8;
  if (id >= total) return;
  const int e = (int)(id & 7);
  const int l = (int)((id >> 3) & 63);
  int64_t f = id >> 9;
  const int mt = (int)(f % MT); f /= MT;
  const int t = (int)(f % (8 * ksteps));
  const int pass = (int)(f / (8 * ksteps));
  const int j = t / ksteps, ks = t % ksteps;
  const int m = (pass * MT + mt) * 32 + (l & 31), c = 16 * ks + 8 * (l >> 5) + e;
  Wt[id] = (m < M && c < Cin) ? W[(int64_t)m * Cin * 8 + c * 8 + j] : (uint16_t)0;
}

// ---- 2x2x2 stride-2 deconvolution over all nodes ----------------------------------------------
//   out[co, 8h + s] = sum_ci W[ci, co*8 + s] * in[ci, h]
// A GEMM with rows m' = co*8 + s (the weight matrix transposed, no re-layout needed for fp32:
// row ci of W is contiguous over m'), K = Cin, columns = parents h.  In the 32x32 accumulator
// a lane holds 4 consecutive rows = 4 consecutive children of one (co, h): one 16-byte store;
// the two half wavefronts complete the 32-byte sibling group, consecutive lanes are consecutive
// parents, so stores are coalesced and every child is written exactly once (no atomics, no
// zero fill -- the reference scatters with atomicAdd, octree/octree/octree_nn.cu:130-174).
template <typename OutT>
__device__ inline void store_children(const ConvArgs& a, OutT* __restrict__ out, const floatx16& acc,
    int row0, int n, int kh) {
  // rows row0 + 8q + 4kh + (0..3), q = 0..3  ->  co = (row0 >> 3) + q, children 4kh .. 4kh+3
  if (n >= a.N) return;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    int co = (row0 >> 3) + q;
    if (co >= a.M) continue;
    int64_t o = (int64_t)co * a.Hout + (int64_t)n * 8 + 4 * kh;
    const float v0 = finish(a, acc[4 * q], co), v1 = finish(a, acc[4 * q + 1], co);
    const float v2 = finish(a, acc[4 * q + 2], co), v3 = finish(a, acc[4 * q + 3], co);
    if (sizeof(OutT) == 4) {
      *reinterpret_cast<float4*>(reinterpret_cast<float*>(out) + o) = make_float4(v0, v1, v2, v3);
    } else {
      uint2 v;
      v.x = (uint32_t)f32_to_bf16(v0) | ((uint32_t)f32_to_bf16(v1) << 16);
      v.y = (uint32_t)f32_to_bf16(v2) | ((uint32_t)f32_to_bf16(v3) << 16);
      *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(out) + o) = v;
    }
  }
}

// bf16: lane (n, kh) holds children 4kh .. 4kh + 3 (8 bytes) of four output channels.  The two
// lanes of a parent swap halves (lanes 0-31 against 32-63) for a pair of channels, so that kh = 0
// ends up with all eight children of the pair's first channel and kh = 1 with those of the second:
// one 16-byte store a lane, 512 contiguous bytes per half wavefront, half the store instructions
// and twice the bytes per request of the 8-byte form.
__device__ inline void store_children_bf16(const ConvArgs& a, uint16_t* __restrict__ out, const floatx16& acc,
    int row0, int n, int kh) {
  if (n >= a.N) return;          // both lanes of a parent leave together
  const int co0 = row0 >> 3;
#pragma unroll
  for (int qp = 0; qp < 2; ++qp) {
    uint32_t w[2][2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int q = 2 * qp + h, co = min(co0 + q, a.M - 1);
      w[h][0] = pack_bf16x2(finish(a, acc[4 * q], co), finish(a, acc[4 * q + 1], co));
      w[h][1] = pack_bf16x2(finish(a, acc[4 * q + 2], co), finish(a, acc[4 * q + 3], co));
    }
    const auto s0 = __builtin_amdgcn_permlane32_swap(w[0][0], w[1][0], false, false);
    const auto s1 = __builtin_amdgcn_permlane32_swap(w[0][1], w[1][1], false, false);
    const int co = co0 + 2 * qp + kh;
    if (co < a.M)
      *reinterpret_cast<uint4*>(out + (int64_t)co * a.Hout + (int64_t)n * 8) = make_uint4(s0[0], s1[0], s0[1], s1[1]);
  }
}

// Over the non-empty nodes the row of a child is its rank among the non-empty nodes of the finer
// level (a.child: that level's child links); an empty child has no row and is not stored.
__device__ inline void store_children_nempty_f32(const ConvArgs& a, float* __restrict__ out, const floatx16& acc,
    int row0, int n, int kh) {
  if (n >= a.N) return;
  int link[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) link[j] = a.child[(int64_t)n * 8 + 4 * kh + j];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int co = (row0 >> 3) + q;
    if (co >= a.M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (link[j] >= 0 && link[j] < a.Hout) out[(int64_t)co * a.Hout + link[j]] = finish(a, acc[4 * q + j], co);
  }
}

constexpr int kD2MT = 4;  // row tiles per pass: 128 rows = 16 output channels x 8 children

// fp32: a wavefront keeps its 64 columns x 64 input channels in registers (read once, coalesced,
// reused by every pass), a pass is 64 rows = 8 output channels x 8 children whose weights
// [64 channels][64 rows] are staged in LDS (the next pass's are in flight meanwhile), and the MFMA
// loop reads A from LDS and B from registers.  With more than 64 input channels the register
// block is refilled for the next chunk right after each k-step has consumed its pair.
constexpr int kD2fMT = 2;
constexpr int kD2fChunk = 64;

// HALF: a layer of 32 input channels or fewer fills the first half of its one chunk only, and the
// k-steps of the other half (zero weights) are left out at compile time (a test inside the loop
// costs the schedule of every k-step).
// NE: over the non-empty nodes (the columns are the non-empty parents either way; a child goes to
// its rank among the non-empty nodes of the finer level or nowhere).
template <bool HALF, bool NE = false>
__global__ __launch_bounds__(256, 3) void deconv_s2_f32_kernel(ConvArgs a, float* __restrict__ out,
    const float* __restrict__ in, const float* __restrict__ W, int n_tiles) {
  constexpr int kSteps = HALF ? kD2fChunk / 4 : kD2fChunk / 2;   // k-steps (channel pairs) of a stage
  __shared__ __attribute__((aligned(16))) float sW[kD2fChunk * 32 * kD2fMT];
  constexpr int kWVec = kD2fChunk * 32 * kD2fMT / 4 / 256;  // float4 per thread and stage
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = xcd_tile(blockIdx.x, n_tiles);
  if (tile >= n_tiles) return;
  const int n0 = tile * kTileCols + wave * kWaveCols;
  const int r = lane & 31, kh = lane >> 5;
  const int rows = a.M * 8;
  const int npass = (rows + 32 * kD2fMT - 1) / (32 * kD2fMT);
  const int nchunk = (a.Cin + kD2fChunk - 1) / kD2fChunk;
  // my passes: blockIdx.y, + gridDim.y, ... (a level of few tiles deals its passes out over workgroups)
  const int my_passes = ((int)blockIdx.y < npass) ? (npass - (int)blockIdx.y + (int)gridDim.y - 1) / (int)gridDim.y : 0;
  if (my_passes == 0) return;
  const int nstage = my_passes * nchunk;
  int ncol[2];
  const float* xcol[2];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
    ncol[nt] = n0 + nt * 32 + r;
    xcol[nt] = in + min(ncol[nt], a.N - 1);  // columns beyond N are computed but never stored
  }
  // channel 2ks + kh of a chunk; channels beyond Cin read channel Cin - 1 and meet zero weights
  float xb[kD2fChunk / 2][2];
  auto load_x = [&](int chunk, int ks) {
    const int c = min(chunk * kD2fChunk + 2 * ks + kh, a.Cin - 1);
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) xb[ks][nt] = xcol[nt][(int64_t)c * a.Hin];
  };
  float4 wr[kWVec];
  auto fetch_w = [&](int stage) {
    const int pass = (int)blockIdx.y + (stage / nchunk) * (int)gridDim.y, chunk = stage % nchunk;
#pragma unroll
    for (int v = 0; v < kWVec; ++v) {
      const int idx = v * 256 + threadIdx.x;              // [channel][16 row quads]
      const int c = chunk * kD2fChunk + idx / (8 * kD2fMT);
      const int row = pass * 32 * kD2fMT + 4 * (idx % (8 * kD2fMT));
      wr[v] = (c < a.Cin && row < rows) ? *reinterpret_cast<const float4*>(W + (int64_t)c * rows + row)
                                        : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  };
#pragma unroll
  for (int ks = 0; ks < kSteps; ++ks) load_x(0, ks);
  fetch_w(0);
  floatx16 acc[kD2fMT][2];
  for (int stage = 0; stage < nstage; ++stage) {
    const int pass = (int)blockIdx.y + (stage / nchunk) * (int)gridDim.y, chunk = stage % nchunk;
    if (chunk == 0) {
#pragma unroll
      for (int mt = 0; mt < kD2fMT; ++mt)
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int v = 0; v < kWVec; ++v) reinterpret_cast<float4*>(sW)[v * 256 + threadIdx.x] = wr[v];
    __syncthreads();
    if (stage + 1 < nstage) fetch_w(stage + 1);
    const int next_chunk = (chunk + 1) % nchunk;
    const bool refill = nchunk > 1 && stage + 1 < nstage;
#pragma unroll
    for (int ks = 0; ks < kSteps; ++ks) {
      const float b0 = xb[ks][0], b1 = xb[ks][1];
      if (refill) load_x(next_chunk, ks);
#pragma unroll
      for (int mt = 0; mt < kD2fMT; ++mt) {
        const float av = sW[(2 * ks + kh) * 32 * kD2fMT + mt * 32 + r];
        acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, b0, acc[mt][0], 0, 0, 0);
        acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, b1, acc[mt][1], 0, 0, 0);
      }
    }
    if (chunk == nchunk - 1) {
      const int row_base = pass * 32 * kD2fMT;
#pragma unroll
      for (int mt = 0; mt < kD2fMT; ++mt)
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
          if constexpr (NE) store_children_nempty_f32(a, out, acc[mt][nt], row_base + mt * 32, ncol[nt], kh);
          else store_children<float>(a, out, acc[mt][nt], row_base + mt * 32, ncol[nt], kh);
        }
    }
  }
}

// bf16: activations come from the row-major copy [H + 1, Cpad] (16-byte operand loads); weights
// packed [pass][kstep][mt][lane][8]: lane (m', kh), j <- W[16*kstep + 8kh + j][m']
__global__ __launch_bounds__(256, 2) void deconv_s2_bf16_kernel(ConvArgs a, uint16_t* __restrict__ out,
    const uint4* __restrict__ xt, const uint4* __restrict__ Wt, int n_tiles, int cpad8) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = xcd_tile(blockIdx.x, n_tiles);
  if (tile >= n_tiles) return;
  const int n0 = tile * kTileCols + wave * kWaveCols;
  if (n0 >= a.N) return;
  const int r = lane & 31, kh = lane >> 5;
  const int rows = a.M * 8;
  const int npass = (rows + 32 * kD2MT - 1) / (32 * kD2MT);
  const int ksteps = cpad8 >> 1;
  int ncol[2];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) ncol[nt] = n0 + nt * 32 + r;
  for (int pass = blockIdx.y; pass < npass; pass += gridDim.y) {  // passes may be dealt out over workgroups
    floatx16 acc[kD2MT][2];
#pragma unroll
    for (int mt = 0; mt < kD2MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.0f;
    const int row_base = pass * 32 * kD2MT;
#pragma unroll 2
    for (int ks = 0; ks < ksteps; ++ks) {
      union { uint4 v4; bf16x8 v; } b0, b1;
      b0.v4 = xt[(int64_t)min(ncol[0], a.Hin) * cpad8 + 2 * ks + kh];
      b1.v4 = xt[(int64_t)min(ncol[1], a.Hin) * cpad8 + 2 * ks + kh];
#pragma unroll
      for (int mt = 0; mt < kD2MT; ++mt) {
        union { uint4 v4; bf16x8 v; } av;
        av.v4 = Wt[(((int64_t)pass * ksteps + ks) * kD2MT + mt) * 64 + lane];
        acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av.v, b0.v, acc[mt][0], 0, 0, 0);
        acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av.v, b1.v, acc[mt][1], 0, 0, 0);
      }
    }
#pragma unroll
    for (int mt = 0; mt < kD2MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) store_children_bf16(a, out, acc[mt][nt], row_base + mt * 32, ncol[nt], kh);
  }
}
// The same for at most 64 input channels (KS k-steps of 16): a wavefront's 64 columns x all
// channels stay in registers for every pass (read once, all requests in flight together), the
// packed weights of a pass (128 rows) are staged in LDS for the four wavefronts, the next pass's
// in flight meanwhile (two buffers, one barrier per pass), and the loop only reads LDS and
// multiplies.  What is left is the store of the children: the kernel is bound by its output.
template <int KS>
__global__ __launch_bounds__(256, 2) void deconv_s2_bf16_reg_kernel(ConvArgs a, uint16_t* __restrict__ out,
    const uint4* __restrict__ xt, const uint4* __restrict__ Wt, int n_tiles) {
  constexpr int kUnits = KS * kD2MT * 64;            // 16-byte units of one pass's weights
  constexpr int kVec = kUnits / 256;                 // per thread
  __shared__ uint4 sW[2][kUnits];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = xcd_tile(blockIdx.x, n_tiles);
  if (tile >= n_tiles) return;
  const int n0 = tile * kTileCols + wave * kWaveCols;
  const int r = lane & 31, kh = lane >> 5;
  const int rows = a.M * 8;
  const int npass = (rows + 32 * kD2MT - 1) / (32 * kD2MT);
  int ncol[2];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) ncol[nt] = n0 + nt * 32 + r;
  union Frag { uint4 v4; bf16x8 v; };
  Frag b[KS][2];
  uint4 wr[kVec];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) b[ks][nt].v4 = xt[(int64_t)min(ncol[nt], a.Hin) * (2 * KS) + 2 * ks + kh];
  // passes may be dealt out over workgroups (blockIdx.y) where the level has few column tiles
  const int pass0 = blockIdx.y, pstep = gridDim.y;
  if (pass0 >= npass) return;
#pragma unroll
  for (int v = 0; v < kVec; ++v) wr[v] = Wt[(int64_t)pass0 * kUnits + v * 256 + threadIdx.x];
#pragma unroll
  for (int v = 0; v < kVec; ++v) sW[0][v * 256 + threadIdx.x] = wr[v];
  int buf = 0;
  for (int pass = pass0; pass < npass; pass += pstep, buf ^= 1) {
    __syncthreads();   // this pass's weights are in LDS; the other buffer is free
    const uint4* wcur = sW[buf];
    const int nxt = pass + pstep < npass ? pass + pstep : pass;
#pragma unroll
    for (int v = 0; v < kVec; ++v) wr[v] = Wt[(int64_t)nxt * kUnits + v * 256 + threadIdx.x];
    floatx16 acc[kD2MT][2];
#pragma unroll
    for (int mt = 0; mt < kD2MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.0f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int mt = 0; mt < kD2MT; ++mt) {
        Frag av;
        av.v4 = wcur[(ks * kD2MT + mt) * 64 + lane];
        acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av.v, b[ks][0].v, acc[mt][0], 0, 0, 0);
        acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av.v, b[ks][1].v, acc[mt][1], 0, 0, 0);
      }
#pragma unroll
    for (int v = 0; v < kVec; ++v) sW[buf ^ 1][v * 256 + threadIdx.x] = wr[v];
    if (n0 < a.N) {
      const int row_base = pass * 32 * kD2MT;
#pragma unroll
      for (int mt = 0; mt < kD2MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) store_children_bf16(a, out, acc[mt][nt], row_base + mt * 32, ncol[nt], kh);
    }
  }
}

__global__ void pack_weights_d2_bf16(uint16_t* __restrict__ Wt, const uint16_t* __restrict__ W, int rows, int Cin,
    int npass, int ksteps) {
  int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = (int64_t)npass * ksteps * kD2MT * 64 * 8;
  if (id >= total) return;
  int j = (int)(id & 7);
  int l = (int)((id >> 3) & 63);
  int64_t f = id >> 9;
  int mt = (int)(f % kD2MT); f /= kD2MT;
  int ks = (int)(f % ksteps);
  int pass = (int)(f / ksteps);
  int m = (pass * kD2MT + mt) * 32 + (l & 31), c = 16 * ks + 8 * (l >> 5) + j;
  Wt[id] = (m < rows && c < Cin) ? W[(int64_t)c * rows + m] : (uint16_t)0;
}

// ---- 2x2x2 stride-2 deconvolution, row-major bf16 on both sides, depad folded in -------------------
// Column = p-th non-empty node of the level; its operand is that node's row of the input (all
// nodes of the level, row ichild[p]: the depad the reference's modules apply before a stride-2
// deconvolution, pytorch/ocnn/octree_conv.py:102-127, is part of the operator).  GEMM rows are
// ordered (child s, output channel): a 32-row tile is 32 channels of one child and goes out as
// 16-byte pieces of row 8 p + s, like the convolutions above.  The columns' operands stay in
// registers for every pass, the packed weights of a pass are staged in LDS (two buffers, one
// barrier per pass).
// NE: the operator over the non-empty nodes.  The columns are then the rows of the input as they
// come (rank p of the non-empty nodes of the level), and child s of column p goes to the row that
// the child links of the finer level name for node 8 p + s, or nowhere when that node is empty.
// (The general row kernel serves this operator too, one live tap in eight per column and the
// weights of all eight taps read by every tile: 0.074 ms for 256 -> 128 from 24 730 nodes, where
// this kernel takes the time of its stores.)
template <int KS, int MT2, bool NE = false>
__global__ __launch_bounds__(256) void deconv_s2_rows_bf16_kernel(ConvArgs a, uint16_t* __restrict__ out,
    int out_pitch, int out_cpad, const u32x4* __restrict__ xt, int in_pitch, const u32x4* __restrict__ Wt, int n_tiles) {
  constexpr int kUnits = KS * MT2 * 64;
  constexpr int kVec = (kUnits + 255) / 256;          // (an odd KS above four leaves the last round half used)
  constexpr bool kWhole = kUnits % 256 == 0;
  __shared__ u32x4 sW[2][kVec * 256];
  __shared__ int sRow[NE ? kTileCols * 8 : 1];        // NE: byte offset of the output row of (column, child)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = xcd_tile(blockIdx.x, n_tiles);
  if (tile >= n_tiles) return;
  const int n0 = tile * kTileCols + wave * kWaveCols;
  const int r = lane & 31, kh = lane >> 5;
  const int ctiles = (a.M + 31) / 32;                 // 32-channel tiles per child
  const int npass = (8 * ctiles + MT2 - 1) / MT2;
  const __amdgpu_buffer_rsrc_t xrows = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<u32x4*>(xt), 0, (int)(((int64_t)a.Hin + 1) * in_pitch * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t obuf = __builtin_amdgcn_make_buffer_rsrc(
      out, 0, (int)(((int64_t)a.Hout + 1) * out_pitch * 2), 0x00020000);
  union Frag { u32x4 q; bf16x8 v; };
  Frag b[KS][2];
  int ooff[2];
  if constexpr (NE) {
    // the ranks of the children of the tile's columns: eight child links a column, contiguous
    for (int i = threadIdx.x; i < kTileCols * 8; i += 256) {
      const int node = tile * kTileCols * 8 + i;         // node 8 p + s of the finer level
      const int rank = (node >> 3) < a.N ? a.child[node] : -1;
      sRow[i] = rank >= 0 && rank < a.Hout ? rank * out_pitch * 2 : 0x7fffff00;
    }
  }
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
    const int n = n0 + nt * 32 + r;
    const int src = n < a.N ? (NE ? n : a.ichild[n]) : -1;
    const int xoff = src >= 0 ? src * in_pitch * 2 + kh * 16 : 0x7fffff00;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) b[ks][nt].q = __builtin_amdgcn_raw_buffer_load_b128(xrows, xoff, ks * 32, 0);
    ooff[nt] = n < a.N ? (n * 8 * out_pitch + 8 * kh) * 2 : 0x7fffff00;
  }
  u32x4 wr[kVec];
  // passes may be dealt out over workgroups (blockIdx.y) where the level has few column tiles
  const int pass0 = blockIdx.y, pstep = gridDim.y;
  if (pass0 >= npass) return;
#pragma unroll
  for (int v = 0; v < kVec; ++v)
    wr[v] = Wt[(int64_t)pass0 * kUnits + (kWhole ? v * 256 + (int)threadIdx.x : min(v * 256 + (int)threadIdx.x, kUnits - 1))];
#pragma unroll
  for (int v = 0; v < kVec; ++v) sW[0][v * 256 + threadIdx.x] = wr[v];
  const float floor = a.relu ? 0.0f : -__builtin_inff();
  int buf = 0;
  for (int pass = pass0; pass < npass; pass += pstep, buf ^= 1) {
    __syncthreads();   // this pass's weights are in LDS; the other buffer is free
    const u32x4* wcur = sW[buf];
    const int nxt = pass + pstep < npass ? pass + pstep : pass;
#pragma unroll
    for (int v = 0; v < kVec; ++v)
      wr[v] = Wt[(int64_t)nxt * kUnits + (kWhole ? v * 256 + (int)threadIdx.x : min(v * 256 + (int)threadIdx.x, kUnits - 1))];
    floatx16 acc[MT2][2];
#pragma unroll
    for (int mt = 0; mt < MT2; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.0f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int mt = 0; mt < MT2; ++mt) {
        Frag av;
        av.q = wcur[(ks * MT2 + mt) * 64 + lane];
        acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av.v, b[ks][0].v, acc[mt][0], 0, 0, 0);
        acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av.v, b[ks][1].v, acc[mt][1], 0, 0, 0);
      }
#pragma unroll
    for (int v = 0; v < kVec; ++v) sW[buf ^ 1][v * 256 + threadIdx.x] = wr[v];
#pragma unroll
    for (int mt = 0; mt < MT2; ++mt) {
      const int t = pass * MT2 + mt;                  // tile = (child, 32-channel block)
      if (t >= 8 * ctiles) break;
      const int child = t / ctiles, cb = (t % ctiles) * 32;
      float bias[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int ch = cb + 8 * (i / 4) + 4 * kh + (i % 4);
        bias[i] = a.bias ? a.bias[min(ch, a.M - 1)] : 0.0f;
        if (ch >= a.M) bias[i] = 0.0f;
      }
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        uint32_t w[4][2];
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const int i = 4 * q + 2 * h;
            w[q][h] = pack_bf16x2(relu_floor(acc[mt][nt][i] + bias[i], floor),
                                  relu_floor(acc[mt][nt][i + 1] + bias[i + 1], floor));
          }
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
          const auto s0 = __builtin_amdgcn_permlane32_swap(w[2 * jj][0], w[2 * jj + 1][0], false, false);
          const auto s1 = __builtin_amdgcn_permlane32_swap(w[2 * jj][1], w[2 * jj + 1][1], false, false);
          if constexpr (NE) {
            const int row = sRow[(wave * kWaveCols + nt * 32 + r) * 8 + child];   // written before the first barrier
            store16_then_wait(store16_t{s0[0], s1[0], s0[1], s1[1]}, obuf, row == 0x7fffff00 ? row : row + 16 * kh,
                (cb + 16 * jj) * 2, cb + 16 * jj < out_cpad);
          } else {
            store16_then_wait(store16_t{s0[0], s1[0], s0[1], s1[1]}, obuf, ooff[nt],
                (child * out_pitch + cb + 16 * jj) * 2, cb + 16 * jj < out_cpad);
          }
        }
      }
      if (tile == 0 && wave == 0 && child == 0 && lane * 8 >= cb && lane * 8 < min(cb + 32, out_cpad))
        *reinterpret_cast<uint4*>(out + (int64_t)a.Hout * out_pitch + lane * 8) = make_uint4(0, 0, 0, 0);
    }
  }
}
// [pass][ks][mt][lane][e]: tile t = pass * MT2 + mt = (child s, channel block cbk); lane (m, kh) <-
// W[16 ks + 8 kh + e][(32 cbk + m) * 8 + s]   (deconvolution weights are [Cin, Cout * 8])
__global__ void pack_weights_d2_rows_bf16(uint16_t* __restrict__ Wt, const uint16_t* __restrict__ W, int Cout, int Cin,
    int MT2, int npass, int ksteps) {
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = (int64_t)npass * ksteps * MT2 * 64 * 8;
  if (id >= total) return;
  const int e = (int)(id & 7);
  const int l = (int)((id >> 3) & 63);
  int64_t f = id >> 9;
  const int mt = (int)(f % MT2); f /= MT2;
  const int ks = (int)(f % ksteps);
  const int pass = (int)(f / ksteps);
  const int ctiles = (Cout + 31) / 32;
  const int t = pass * MT2 + mt;
  const int child = t / ctiles, co = (t % ctiles) * 32 + (l & 31), c = 16 * ks + 8 * (l >> 5) + e;
  Wt[id] = (t < 8 * ctiles && co < Cout && c < Cin) ? W[(int64_t)c * Cout * 8 + co * 8 + child] : (uint16_t)0;
}

template <typename T>
__global__ void zero_rows_kernel(T* p, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += step) p[i] = (T)0;
}

__global__ void ichild_kernel(int* __restrict__ ichild, int n_nempty, const int* __restrict__ child, int n) {
  int h = blockIdx.x * blockDim.x + threadIdx.x;
  if (h >= n) return;
  int l = child[h];
  if (l >= 0 && l < n_nempty) ichild[l] = h;
}

// Shape rules of OctreeBaseConv::reshape (octree/octree/octree_conv.cpp:48-104)
// and the input-height check of pytorch/cpp/octree_conv.cpp:72-78.
// The register-fed bf16 kernel keeps one workgroup per CU busy with 1024 columns each; below
// this many such tiles the LDS kernel (256 columns per workgroup, three workgroups per CU) fills
// the device better.  Measured crossover on 256 CUs: between 110 and 215 tiles.
std::atomic<int> g_bf16_reg_min_tiles{192};
std::atomic<int> g_rows_direct_f32{1};   // fp32 row kernel over the non-empty nodes: the same choice
std::atomic<int> g_rows_direct{1};   // bf16 row kernels with three taps or more: 1 = weights straight from memory per live tap

struct ConvPlan {
  int top_depth, workspace_depth, top_h, btm_h, workspace_h;
  int child_h, ichild_h;
  int mode;
  KernelTaps taps;
  int mtiles, csteps;
  size_t wt_bytes, ichild_bytes, xt_bytes, xt_general, total_bytes;
};

inline size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

int make_plan(const Info* o, int depth, int channel_in, int num_output, const int* ks, int stride,
    int nempty, int deconv, int dtype, ConvPlan* p) {
  OCNN_REQUIRE(o && ks, OCNN_E_BADARG, "null pointer");
  int e = ocnn_info_check(o);
  if (e) return e;
  OCNN_REQUIRE(depth > 0 && depth <= o->depth, OCNN_E_BADARG, "depth %d not in [1,%d]", depth, o->depth);
  OCNN_REQUIRE(num_output > 0 && channel_in > 0, OCNN_E_BADARG, "channels %d -> %d", channel_in, num_output);
  OCNN_REQUIRE(stride == 1 || stride == 2, OCNN_E_BADARG, "stride %d", stride);
  OCNN_REQUIRE(dtype == OCNN_F32 || dtype == OCNN_BF16, OCNN_E_BADARG, "dtype %d", dtype);
  OCNN_REQUIRE(kernel_taps(ks, &p->taps), OCNN_E_UNSUPPORTED, "kernel size %d%d%d", ks[0], ks[1], ks[2]);
  OCNN_REQUIRE(o->has(OCNN_NEIGH) && o->has(OCNN_CHILD), OCNN_E_FORMAT,
      "the octree holds no neighbour table (not an octree_batch result)");
  p->top_depth = p->workspace_depth = depth;
  if (stride == 2) {
    if (deconv) p->top_depth = p->workspace_depth = depth + 1;
    else p->top_depth = depth - 1;
    OCNN_REQUIRE(p->top_depth >= 0 && p->top_depth <= o->depth, OCNN_E_BADARG,
        "output depth %d outside the octree", p->top_depth);
  }
  int top_h;
  if (!nempty) {
    top_h = o->nnum[p->top_depth];
    if (stride == 2 && !deconv) top_h = o->nnum_nempty[p->top_depth];
  } else {
    top_h = o->nnum_nempty[p->top_depth];
  }
  if (top_h == 0) top_h = 1;
  p->top_h = top_h;
  p->workspace_h = top_h;
  if (stride == 2) p->workspace_h = deconv ? o->nnum[p->top_depth] / 8 : o->nnum[depth] / 8;
  p->btm_h = ((stride == 2 && deconv) || nempty) ? o->nnum_nempty[depth] : o->nnum[depth];
  p->child_h = o->nnum[p->workspace_depth];
  p->ichild_h = o->nnum_nempty[p->workspace_depth];
  if (stride == 1) p->mode = kModeS1;
  else if (!deconv) p->mode = kModeS2Conv;
  else p->mode = (ks[0] == 2 && ks[1] == 2 && ks[2] == 2) ? kModeS2Deconv : kModeS2DeconvAny;
  p->mtiles = (num_output + 31) / 32;
  p->csteps = 0;
  {  // general row-major gather path: padded weights + the row-major copy of the input
    size_t cpad = dtype == OCNN_F32 ? ((size_t)channel_in + 7) / 8 * 8 : ((size_t)channel_in + 15) / 16 * 16;
    const size_t slab = dtype == OCNN_F32 ? kRowSlabF : kRowSlab;
    size_t nslab = (cpad + slab - 1) / slab, npass = (size_t)(p->mtiles + 1) / 2;
    size_t per_stage = dtype == OCNN_F32 ? (kRowSlabF / 8) * 4 * 2 * 64 * sizeof(float)
                                         : (kRowSlab / 16) * 2 * 64 * 8 * sizeof(uint16_t);
    p->wt_bytes = align256(npass * p->taps.count * nslab * per_stage);
    p->xt_general = align256(((size_t)p->btm_h + 1) * cpad * (dtype == OCNN_F32 ? 4 : 2));
  }
  if (dtype == OCNN_F32) {  // the LDS kernel pads channels to slabs of 4 and row tiles to passes
    size_t lds_words = (size_t)((p->mtiles + 1) / 2) * ((channel_in + kSlab - 1) / kSlab) * p->taps.count * kKSteps * 2 * 64;
    p->wt_bytes = align256(lds_words * sizeof(float) > p->wt_bytes ? lds_words * sizeof(float) : p->wt_bytes);
  }
  p->ichild_bytes = nempty ? align256(sizeof(int) * (size_t)(p->ichild_h + 1)) : 0;
  p->xt_bytes = 0;
  if (dtype == OCNN_BF16 && stride == 1 && !nempty && p->taps.count == 27) {
    // LDS kernel: weights padded to passes of 2 row tiles and slabs of 16 channels, plus the
    // row-major copy of the input ([H + 1, Cpad] bf16)
    size_t cpad = (size_t)(channel_in + 15) / 16 * 16;
    size_t w = (size_t)((p->mtiles + 1) / 2) * (cpad / 16) * 27 * 2 * 64 * 8 * sizeof(uint16_t);
    if (w > p->wt_bytes) p->wt_bytes = align256(w);
    p->xt_bytes = align256(((size_t)p->btm_h + 1) * cpad * sizeof(uint16_t));
  }
  const bool is222 = ks[0] == 2 && ks[1] == 2 && ks[2] == 2;
  if (stride == 2 && !nempty && is222 && !deconv) {  // dedicated stride-2 kernels: padded packing
    size_t npass = (size_t)(p->mtiles + 1) / 2;
    size_t w = dtype == OCNN_F32 ? npass * ((channel_in + kS2Slab - 1) / kS2Slab) * kS2Slab * 4 * 2 * 64 * sizeof(float)
                                 : npass * ((channel_in + 7) / 8) * 4 * 2 * 64 * 8 * sizeof(uint16_t);
    if (w > p->wt_bytes) p->wt_bytes = align256(w);
  }
  if (stride == 2 && !nempty && is222 && deconv && dtype == OCNN_BF16) {
    size_t cpad = (size_t)(channel_in + 15) / 16 * 16;
    size_t npass = ((size_t)num_output * 8 + 32 * kD2MT - 1) / (32 * kD2MT);
    size_t w = npass * (cpad / 16) * kD2MT * 64 * 8 * sizeof(uint16_t);
    if (w > p->wt_bytes) p->wt_bytes = align256(w);
    p->xt_bytes = align256(((size_t)p->btm_h + 1) * cpad * sizeof(uint16_t));
  }
  if (p->xt_general > p->xt_bytes) p->xt_bytes = p->xt_general;  // one buffer serves whichever path runs
  p->total_bytes = p->wt_bytes + p->ichild_bytes + p->xt_bytes;
  return OCNN_OK;
}

int run_conv(int deconv, void* top, const void* btm, int channel_in, int btm_h, const void* weights,
    const void* octree_dev, const void* info, int depth, int num_output, const int* ks, int stride,
    int nempty, int dtype, void* ws, size_t ws_bytes, hipStream_t s, const float* bias = nullptr,
    int relu = 0, bool builtin_scratch = false, const int* sources = nullptr, size_t sources_bytes = 0) {
  OCNN_REQUIRE(top && btm && weights && octree_dev && info, OCNN_E_BADARG, "null pointer");
  const Info* o = as_info(info);
  ConvPlan p;
  int e = make_plan(o, depth, channel_in, num_output, ks, stride, nempty, deconv, dtype, &p);
  if (e) return e;
  OCNN_REQUIRE(btm_h == p.btm_h, OCNN_E_SHAPE, "input height %d, the octree has %d rows at depth %d",
      btm_h, p.btm_h, depth);
  OCNN_REQUIRE(ws && (builtin_scratch || ws_bytes >= p.total_bytes), OCNN_E_WORKSPACE,
      "workspace %zu < %zu bytes", ws_bytes, p.total_bytes);
  OCNN_REQUIRE((reinterpret_cast<uintptr_t>(ws) & 15) == 0, OCNN_E_WORKSPACE, "workspace not 16-byte aligned");

  const char* blob = static_cast<const char*>(octree_dev);
  ConvArgs a;
  a.M = num_output;
  a.Cin = channel_in;
  a.N = p.top_h;
  a.K = p.taps.count;
  a.Hin = btm_h;
  a.Hout = p.top_h;
  a.mode = p.mode;
  a.nempty = nempty ? 1 : 0;
  a.mtiles = p.mtiles;
  a.csteps = p.csteps;
  for (int k = 0; k < 27; ++k) {
    int tap = k < p.taps.count ? p.taps.tap[k] : 13;
    // deconvolution gathers through the mirrored offset: the rows h that scatter
    // to p through tap k are exactly the neighbours of p at the opposite offset
    a.slot[k] = tap_slot(deconv && stride == 1 ? 26 - tap : tap);
  }
  a.neigh = reinterpret_cast<const int*>(blob + o->ptr_dis(OCNN_NEIGH, p.workspace_depth));
  a.child = reinterpret_cast<const int*>(blob + o->ptr_dis(OCNN_CHILD, p.workspace_depth));
  a.ichild = nullptr;
  a.bias = bias;
  a.relu = relu ? 1 : 0;
  // degenerate layer without nodes: the reference emits one zero column
  // (octree_conv.cpp:82) -- nothing to gather
  bool empty_layer = (nempty ? o->nnum_nempty[p.top_depth] : (stride == 2 && !deconv
      ? o->nnum_nempty[p.top_depth] : o->nnum[p.top_depth])) == 0;
  if (empty_layer) {
    int64_t cnt = (int64_t)num_output * p.top_h;
    if (dtype == OCNN_F32) zero_rows_kernel<float><<<blocks_for(cnt), kBlock, 0, s>>>((float*)top, cnt);
    else zero_rows_kernel<uint16_t><<<blocks_for(cnt), kBlock, 0, s>>>((uint16_t*)top, cnt);
    OCNN_LAUNCH_OK("zero_rows");
    return OCNN_OK;
  }

  char* wsb = static_cast<char*>(ws);
  // conv: W[num_output, channel_in*K]; deconv: W[channel_in, num_output*K]
  int64_t sm = deconv ? a.K : (int64_t)channel_in * a.K;
  int64_t sc = deconv ? (int64_t)num_output * a.K : a.K;
  int n_tiles = (a.N + kTileCols - 1) / kTileCols;
  int grid = ((n_tiles + 7) / 8) * 8;
  const bool k222 = ks[0] == 2 && ks[1] == 2 && ks[2] == 2;
  // which kernel runs, and how much of the workspace it touches: the weights in their packed
  // order always come first, the inverted child links of the non-empty mode second, the
  // row-major copy of the input (only some kernels read one) last
  enum { kPathS2Conv, kPathS2Deconv, kPathS1LdsF32, kPathRowsF32, kPathS1LdsBf16, kPathRowsBf16, kPathOneTapF32 } path;
  bool copies_input = true;
  if (dtype == OCNN_F32 && a.mode == kModeS1 && a.K == 1 && a.Hin == a.N && a.Hin > 0) {
    // 1x1x1: every column reads its own row, over all nodes and over the non-empty ones alike
    path = kPathOneTapF32;
    copies_input = false;
  } else if (a.mode == kModeS2Conv && !a.nempty && k222 && (a.Hin & 7) == 0 &&
      (reinterpret_cast<uintptr_t>(btm) & 15) == 0) {
    path = kPathS2Conv;
    copies_input = false;
  } else if (a.mode == kModeS2Deconv && (!a.nempty || dtype == OCNN_F32) && (reinterpret_cast<uintptr_t>(top) & 15) == 0 &&
             (dtype != OCNN_F32 || (reinterpret_cast<uintptr_t>(weights) & 15) == 0) &&
             (!a.nempty || o->nnum[p.top_depth] == 8 * a.Hin)) {
    // (fp32 also over the non-empty nodes: the same columns, the children stored by rank)
    path = kPathS2Deconv;
    copies_input = dtype != OCNN_F32;
  } else if (dtype == OCNN_F32 && a.mode == kModeS1 && !a.nempty && a.K == 27 &&
             a.Hin < (1 << 29)) {  // its gathers address a channel with 32-bit byte offsets
    path = kPathS1LdsF32;
    copies_input = false;
  } else if (dtype == OCNN_F32) {
    path = kPathRowsF32;
  } else if (a.mode == kModeS1 && !a.nempty && a.K == 27) {
    path = kPathS1LdsBf16;
  } else {
    path = kPathRowsBf16;
  }
  if (builtin_scratch) {
    const size_t used = p.wt_bytes + p.ichild_bytes + (copies_input ? p.xt_bytes : 0);
    OCNN_REQUIRE(used <= ws_bytes, OCNN_E_WORKSPACE,
        "this call needs %zu bytes of scratch memory, the built-in array holds %zu: "
        "use ocnn_octree_conv_fused with a workspace of your own", used, ws_bytes);
  }
  a.src_table = nullptr;
  a.src_pitch = 0;
  if (nempty && sources && (path == kPathRowsF32 || path == kPathRowsBf16)) {
    // the caller's table of source rows (ocnn_conv_rows_sources): no look-up in the kernel, and the
    // inverted child links, which only the look-up reads, are not made
    const int pitch = (a.N + kTileCols - 1) / kTileCols * kTileCols;
    OCNN_REQUIRE(sources_bytes >= sizeof(int) * 27 * (size_t)pitch, OCNN_E_WORKSPACE,
        "the table of source rows takes %zu bytes, the buffer holds %zu", sizeof(int) * 27 * (size_t)pitch, sources_bytes);
    a.src_table = sources;
    a.src_pitch = pitch;
  } else if (nempty && path != kPathOneTapF32 && path != kPathS2Deconv) {
    int* ichild = reinterpret_cast<int*>(wsb + p.wt_bytes);
    ichild_kernel<<<blocks_for(p.child_h), kBlock, 0, s>>>(ichild, p.ichild_h, a.child, p.child_h);
    OCNN_LAUNCH_OK("ichild");
    a.ichild = ichild;
  }
  if (path == kPathS2Conv) {
    const int MT = a.mtiles == 1 ? 1 : 2;
    const int npass = (a.mtiles + MT - 1) / MT;
    if (dtype == OCNN_F32) {
      const int nslab = (a.Cin + kS2Slab - 1) / kS2Slab;
      int64_t total = (int64_t)npass * nslab * kS2Slab * 4 * MT * 64;
      pack_weights_s2_f32<<<blocks_for(total), kBlock, 0, s>>>((float*)wsb, (const float*)weights, a.M, a.Cin, MT, npass, nslab);
      const dim3 g2(grid, pass_split(n_tiles, npass));
      if (MT == 1) conv_s2_f32_kernel<1><<<g2, 256, 0, s>>>(a, (float*)top, (const float*)btm, (const float*)wsb, n_tiles);
      else conv_s2_f32_kernel<2><<<g2, 256, 0, s>>>(a, (float*)top, (const float*)btm, (const float*)wsb, n_tiles);
    } else {
      const int nslab = (a.Cin + 7) / 8;
      int64_t total = (int64_t)npass * nslab * 4 * MT * 64 * 8;
      pack_weights_s2_bf16<<<blocks_for(total), kBlock, 0, s>>>((uint16_t*)wsb, (const uint16_t*)weights, a.M, a.Cin, MT, npass, nslab);
      const dim3 g2(grid, pass_split(n_tiles, npass));
      if (MT == 1) conv_s2_bf16_kernel<1><<<g2, 256, 0, s>>>(a, (uint16_t*)top, (const uint16_t*)btm, (const uint4*)wsb, n_tiles);
      else conv_s2_bf16_kernel<2><<<g2, 256, 0, s>>>(a, (uint16_t*)top, (const uint16_t*)btm, (const uint4*)wsb, n_tiles);
    }
  } else if (path == kPathS2Deconv) {
    // columns are the parents here: one column tile writes the 8 children of 256 parents
    ConvArgs d = a;
    d.N = a.Hin;
    int d_tiles = (d.N + kTileCols - 1) / kTileCols;
    int d_grid = ((d_tiles + 7) / 8) * 8;
    if (dtype == OCNN_F32) {
      const dim3 g2(d_grid, pass_split_costly(d_tiles, (d.M * 8 + 32 * kD2fMT - 1) / (32 * kD2fMT)));
      if (d.nempty && d.Cin <= kD2fChunk / 2)
        deconv_s2_f32_kernel<true, true><<<g2, 256, 0, s>>>(d, (float*)top, (const float*)btm, (const float*)weights, d_tiles);
      else if (d.nempty)
        deconv_s2_f32_kernel<false, true><<<g2, 256, 0, s>>>(d, (float*)top, (const float*)btm, (const float*)weights, d_tiles);
      else if (d.Cin <= kD2fChunk / 2)
        deconv_s2_f32_kernel<true><<<g2, 256, 0, s>>>(d, (float*)top, (const float*)btm, (const float*)weights, d_tiles);
      else
        deconv_s2_f32_kernel<false><<<g2, 256, 0, s>>>(d, (float*)top, (const float*)btm, (const float*)weights, d_tiles);
    } else {
      const int cpad = (a.Cin + 15) / 16 * 16;
      const int rows = a.M * 8, npass = (rows + 32 * kD2MT - 1) / (32 * kD2MT), ksteps = cpad / 16;
      int64_t total = (int64_t)npass * ksteps * kD2MT * 64 * 8;
      pack_weights_d2_bf16<<<blocks_for(total), kBlock, 0, s>>>((uint16_t*)wsb, (const uint16_t*)weights, rows, a.Cin, npass, ksteps);
      uint16_t* xt = reinterpret_cast<uint16_t*>(wsb + p.wt_bytes + p.ichild_bytes);
      dim3 tgrid((a.Hin + 1 + 127) / 128, (cpad + 63) / 64);
      transpose_rows_bf16_kernel<<<tgrid, 256, 0, s>>>(xt, (const uint16_t*)btm, a.Cin, a.Hin, cpad);
      // (bound by its stores: dealt out only where the tiles alone leave compute units empty)
      const dim3 g2(d_grid, d_tiles < 256 ? pass_split_costly(d_tiles, npass) : 1);
      if (ksteps == 1)
        deconv_s2_bf16_reg_kernel<1><<<g2, 256, 0, s>>>(d, (uint16_t*)top, (const uint4*)xt, (const uint4*)wsb, d_tiles);
      else if (ksteps == 2)
        deconv_s2_bf16_reg_kernel<2><<<g2, 256, 0, s>>>(d, (uint16_t*)top, (const uint4*)xt, (const uint4*)wsb, d_tiles);
      else if (ksteps == 4)
        deconv_s2_bf16_reg_kernel<4><<<g2, 256, 0, s>>>(d, (uint16_t*)top, (const uint4*)xt, (const uint4*)wsb, d_tiles);
      else if (ksteps == 8)
        deconv_s2_bf16_reg_kernel<8><<<g2, 256, 0, s>>>(d, (uint16_t*)top, (const uint4*)xt, (const uint4*)wsb, d_tiles);
      else
        deconv_s2_bf16_kernel<<<dim3(d_grid, pass_split(d_tiles, (d.M * 8 + 32 * kD2MT - 1) / (32 * kD2MT))), 256, 0, s>>>(d, (uint16_t*)top, (const uint4*)xt, (const uint4*)wsb, d_tiles, cpad / 8);
    }
  } else if (path == kPathOneTapF32) {
    const int MT = a.mtiles == 1 ? 1 : 2;
    const int npass = (a.mtiles + MT - 1) / MT;
    if (MT == 1)
      conv_one_tap_f32_kernel<1><<<dim3(grid, pass_split(n_tiles, npass)), 256, 0, s>>>(a, (float*)top, (const float*)btm, (const float*)weights, sm, sc, n_tiles);
    else
      conv_one_tap_f32_kernel<2><<<dim3(grid, pass_split(n_tiles, npass)), 256, 0, s>>>(a, (float*)top, (const float*)btm, (const float*)weights, sm, sc, n_tiles);
  } else if (path == kPathS1LdsF32) {
    // Two row tiles a workgroup halve the gathers per product, one row tile doubles the number of
    // workgroups: the latter where a level is so small that the former leaves the CUs short of work
    // (12 824 columns, 128 -> 256 channels: 0.31 -> 0.285 ms).
    const int MT = (a.mtiles == 1 || (int64_t)n_tiles * ((a.mtiles + 1) / 2) < 512) ? 1 : 2;
    const int npass = (a.mtiles + MT - 1) / MT, nslab = (a.Cin + kSlab - 1) / kSlab;
    int64_t total = (int64_t)npass * nslab * a.K * kKSteps * MT * 64;
    pack_weights_lds_f32<<<blocks_for(total), kBlock, 0, s>>>((float*)wsb, (const float*)weights, a.M, a.Cin, a.K,
        MT, npass, nslab, sm, sc);
    OCNN_LAUNCH_OK("pack_weights_lds");
    const int split = pass_split(n_tiles, npass);
    if (MT == 1)
      conv_s1_f32_lds_kernel<1, 27><<<dim3(grid, split), 256, 0, s>>>(a, (float*)top, (const float*)btm, (const float*)wsb, n_tiles);
    else
      conv_s1_f32_lds_kernel<2, 27><<<dim3(grid, split), 256, 0, s>>>(a, (float*)top, (const float*)btm, (const float*)wsb, n_tiles);
  } else if (path == kPathRowsF32) {
    const int MT = a.mtiles == 1 ? 1 : 2;
    const int cpad = (a.Cin + 7) / 8 * 8;
    const int npass = (a.mtiles + MT - 1) / MT, nslab = (cpad + kRowSlabF - 1) / kRowSlabF;
    int64_t total = (int64_t)npass * a.K * nslab * (kRowSlabF / 8) * 4 * MT * 64;
    // Stride 1 over the non-empty nodes of a sparse level (fewer than one node in five non-empty: the
    // finest levels of a surface), three taps or more: weights straight from memory per live tap.
    // Depth 9 of the scene (one in six), 64 -> 64: 0.476 -> 0.383 ms, 64 -> 32: 0.358 -> 0.246 ms,
    // 6 -> 32: 0.107 -> 0.074 ms.  On denser levels most taps are live and the staged kernel, which
    // shares a stage's weights between its four wavefronts through LDS, is ahead (depth 7, one in
    // two, 128 -> 128: 0.87 against 1.03 ms); stride 2 gains nothing either way.
    const int direct_rule = g_rows_direct_f32.load();   // 2 (tests): whatever the level
    const bool direct = nempty && a.mode == kModeS1 && a.K >= 3 && direct_rule != 0 &&
        (direct_rule == 2 || (int64_t)o->nnum_nempty[p.top_depth] * 5 < o->nnum[p.top_depth]);
    pack_weights_rows_f32<<<blocks_for(total), kBlock, 0, s>>>((float*)wsb, (const float*)weights, a.M, a.Cin, a.K,
        MT, npass, nslab, sm, sc, direct ? 1 : 0);
    OCNN_LAUNCH_OK("pack_weights_rows");
    float* xt = (float*)(wsb + p.wt_bytes + p.ichild_bytes);
    dim3 tg((a.Hin + 64) / 64, (cpad + 63) / 64);
    transpose_rows_f32_kernel<<<tg, 256, 0, s>>>(xt, (const float*)btm, a.Cin, a.Hin, cpad);
    OCNN_LAUNCH_OK("transpose_rows");
    if (direct) {
      const int waves = direct_waves(a.N, npass);
      const int tiles = (a.N + kWaveCols * waves - 1) / (kWaveCols * waves);
      const dim3 g(((tiles + 7) / 8) * 8, pass_split(tiles, npass));
#define OCNN_ROWS_F32_DIRECT(MT_)                                                                                \
      if (waves == 4) conv_rows_f32_direct_kernel<MT_, 2, 4><<<g, 256, 0, s>>>(a, (float*)top, (const float4*)xt, (const float4*)wsb, tiles, cpad); \
      else if (waves == 2) conv_rows_f32_direct_kernel<MT_, 2, 2><<<g, 128, 0, s>>>(a, (float*)top, (const float4*)xt, (const float4*)wsb, tiles, cpad); \
      else conv_rows_f32_direct_kernel<MT_, 2, 1><<<g, 64, 0, s>>>(a, (float*)top, (const float4*)xt, (const float4*)wsb, tiles, cpad)
      if (MT == 1) { OCNN_ROWS_F32_DIRECT(1); } else { OCNN_ROWS_F32_DIRECT(2); }
#undef OCNN_ROWS_F32_DIRECT
    } else if (MT == 1)
      conv_rows_f32_kernel<1><<<dim3(grid, pass_split(n_tiles, npass)), 256, 0, s>>>(a, (float*)top, (const float4*)xt, (const float*)wsb, n_tiles, cpad);
    else
      conv_rows_f32_kernel<2><<<dim3(grid, pass_split(n_tiles, npass)), 256, 0, s>>>(a, (float*)top, (const float4*)xt, (const float*)wsb, n_tiles, cpad);
  } else if (path == kPathS1LdsBf16) {
    const int MT = a.mtiles == 1 ? 1 : 2;
    const int cpad = (a.Cin + 15) / 16 * 16;
    const int npass = (a.mtiles + MT - 1) / MT, nslab = cpad / 16;
    int64_t total = (int64_t)npass * nslab * 27 * MT * 64 * 8;
    pack_weights_lds_bf16<<<blocks_for(total), kBlock, 0, s>>>((uint16_t*)wsb, (const uint16_t*)weights, a.M, a.Cin,
        MT, npass, nslab, sm, sc, deconv);
    uint16_t* xt = reinterpret_cast<uint16_t*>(wsb + p.wt_bytes + p.ichild_bytes);
    dim3 tgrid((a.Hin + 1 + 127) / 128, (cpad + 63) / 64);
    transpose_rows_bf16_kernel<<<tgrid, 256, 0, s>>>(xt, (const uint16_t*)btm, a.Cin, a.Hin, cpad);
    OCNN_LAUNCH_OK("pack/transpose");
    // the kernels walk geometric offsets in natural order (the packer mirrored the weights)
    const int r_tiles = ((a.N >> 3) + kRegTileGroups - 1) / kRegTileGroups;
    const bool fits32 = ((int64_t)a.Hin + 1) * cpad * 2 < ((int64_t)1 << 31);   // the kernel addresses rows with 32-bit byte offsets
    const bool use_reg = fits32 && r_tiles >= g_bf16_reg_min_tiles.load(std::memory_order_relaxed);
    if (use_reg) {
      const int r_grid = ((r_tiles + 7) / 8) * 8;
      if (MT == 1)
        conv_s1_bf16_reg_kernel<1, false><<<dim3(r_grid, pass_split(r_tiles, npass)), 256, 0, s>>>(a, (uint16_t*)top, (const u32x4*)xt, (const u32x4*)wsb, r_tiles, cpad / 8, 0, 0);
      else
        conv_s1_bf16_reg_kernel<2, false><<<dim3(r_grid, pass_split(r_tiles, npass)), 256, 0, s>>>(a, (uint16_t*)top, (const u32x4*)xt, (const u32x4*)wsb, r_tiles, cpad / 8, 0, 0);
    } else if (MT == 1)
      conv_s1_bf16_lds_kernel<1><<<dim3(grid, pass_split(n_tiles, npass)), 256, 0, s>>>(a, (uint16_t*)top, (const u32x4*)xt, (const u32x4*)wsb, n_tiles, cpad / 8);
    else
      conv_s1_bf16_lds_kernel<2><<<dim3(grid, pass_split(n_tiles, npass)), 256, 0, s>>>(a, (uint16_t*)top, (const u32x4*)xt, (const u32x4*)wsb, n_tiles, cpad / 8);
  } else {
    const bool deep = a.K >= 3;   // fewer taps than a weight group: the shallow kernel
    // 128 output channels a pass where the operator has whole blocks of them (see the kernel)
    const bool wide = deep && a.mtiles % 4 == 0;
    const int MT = a.mtiles == 1 ? 1 : (wide ? 4 : 2);
    // (the rule of make_rows_plan: 32-channel stages at three wavefronts a SIMD on a level where one
    // node in five or more is non-empty)
    const bool dense_level = nempty && deep && MT == 2 && (int64_t)o->nnum_nempty[p.top_depth] * 5 >= o->nnum[p.top_depth];
    const int slab_ch = wide || dense_level ? 32 : kRowSlab;
    const int cpad = (a.Cin + 15) / 16 * 16;
    const int npass = (a.mtiles + MT - 1) / MT, nslab = (cpad + slab_ch - 1) / slab_ch;
    int64_t total = (int64_t)npass * a.K * nslab * (slab_ch / 16) * MT * 64 * 8;
    pack_weights_rows_bf16<<<blocks_for(total), kBlock, 0, s>>>((uint16_t*)wsb, (const uint16_t*)weights, a.M,
        a.Cin, a.K, MT, npass, nslab, sm, sc, slab_ch);
    OCNN_LAUNCH_OK("pack_weights_rows");
    uint16_t* xt = (uint16_t*)(wsb + p.wt_bytes + p.ichild_bytes);
    dim3 tg((a.Hin + 1 + 127) / 128, (cpad + 63) / 64);
    transpose_rows_bf16_kernel<<<tg, 256, 0, s>>>(xt, (const uint16_t*)btm, a.Cin, a.Hin, cpad);
    OCNN_LAUNCH_OK("transpose_rows");
    const dim3 rgrid(grid, pass_split(n_tiles, npass));
    // (with whole blocks of 128 output channels and a channel-major store the staged kernel is ahead,
    // unless the level is one that smaller workgroups spread better over the device: direct_waves)
    const int waves = deep ? direct_waves(a.N, npass) : kConvWaves;
    const bool direct = deep && (!wide || waves < kConvWaves) && g_rows_direct.load() != 0;
    const bool staged = dense_level && (int64_t)o->nnum_nempty[p.top_depth] * 5 >= (int64_t)o->nnum[p.top_depth] * 2;
    auto launch_direct = [&](auto mt, auto slab, auto wps) {
      constexpr int MT_ = decltype(mt)::value, SLAB_ = decltype(slab)::value, WPS_ = decltype(wps)::value;
      const int tiles = (a.N + kWaveCols * waves - 1) / (kWaveCols * waves);
      const dim3 g(((tiles + 7) / 8) * 8, pass_split(tiles, npass));
      if (waves == 4)
        conv_rows_bf16_direct_kernel<MT_, SLAB_, false, WPS_, 4><<<g, 256, 0, s>>>(a, (uint16_t*)top, (const u32x4*)xt, (const u32x4*)wsb, tiles, cpad, cpad, 0, 0);
      else if (waves == 2)
        conv_rows_bf16_direct_kernel<MT_, SLAB_, false, WPS_, 2><<<g, 128, 0, s>>>(a, (uint16_t*)top, (const u32x4*)xt, (const u32x4*)wsb, tiles, cpad, cpad, 0, 0);
      else
        conv_rows_bf16_direct_kernel<MT_, SLAB_, false, WPS_, 1><<<g, 64, 0, s>>>(a, (uint16_t*)top, (const u32x4*)xt, (const u32x4*)wsb, tiles, cpad, cpad, 0, 0);
    };
    using std::integral_constant;
    if (dense_level && direct && !staged)
      launch_direct(integral_constant<int, 2>(), integral_constant<int, 32>(), integral_constant<int, 3>());
    else if (dense_level)
      conv_rows_bf16_deep_kernel<2, 32, false><<<rgrid, 256, 0, s>>>(a, (uint16_t*)top, (const u32x4*)xt, (const u32x4*)wsb, n_tiles, cpad, cpad, 0, 0);
    else if (direct && wide)
      launch_direct(integral_constant<int, 4>(), integral_constant<int, 32>(), integral_constant<int, 2>());
    else if (direct && MT == 1)
      launch_direct(integral_constant<int, 1>(), integral_constant<int, kRowSlab>(), integral_constant<int, 2>());
    else if (direct)
      launch_direct(integral_constant<int, 2>(), integral_constant<int, kRowSlab>(), integral_constant<int, 2>());
    else if (wide)
      conv_rows_bf16_deep_kernel<4, 32, false><<<rgrid, 256, 0, s>>>(a, (uint16_t*)top, (const u32x4*)xt, (const u32x4*)wsb, n_tiles, cpad, cpad, 0, 0);
    else if (deep && MT == 1)
      conv_rows_bf16_deep_kernel<1, kRowSlab, false><<<rgrid, 256, 0, s>>>(a, (uint16_t*)top, (const u32x4*)xt, (const u32x4*)wsb, n_tiles, cpad, cpad, 0, 0);
    else if (deep)
      conv_rows_bf16_deep_kernel<2, kRowSlab, false><<<rgrid, 256, 0, s>>>(a, (uint16_t*)top, (const u32x4*)xt, (const u32x4*)wsb, n_tiles, cpad, cpad, 0, 0);
    else if (MT == 1)
      conv_rows_bf16_kernel<1><<<rgrid, 256, 0, s>>>(a, (uint16_t*)top, (const u32x4*)xt, (const u32x4*)wsb, n_tiles, cpad);
    else
      conv_rows_bf16_kernel<2><<<rgrid, 256, 0, s>>>(a, (uint16_t*)top, (const u32x4*)xt, (const u32x4*)wsb, n_tiles, cpad);
  }
  OCNN_LAUNCH_OK("octree_conv");
  return OCNN_OK;
}


// ---- weight gradient ----------------------------------------------------------------------
// G[m, c*K + k] = sum_n A[m, n] * X[c, src(n, k)]   (weight_gpu_gemm, octree_conv.cpp:327-356,
// without the column buffer).  A is the operand on the column side of the convolution geometry
// ([M, N]), X the gathered side, read from its row-major copy xt[Hin + 1][cpad] (row Hin zero).
// The reduction runs over the columns, so the MFMA k dimension is n: lane (m, kh) loads one
// float4 of A = columns n0 + 4kh .. + 3, and step j multiplies the column pair (n0 + j,
// n0 + 4 + j); lane (c, kh) gathers xt[src(n0 + 4kh + j, tap)][c], 128 contiguous bytes per half
// wavefront.  A wavefront is one slice: it walks a contiguous range of blocks of 8 columns with its
// own accumulators for 3 taps x (MT x NT) 32x32 tiles and writes them to partial[slice]; a second
// kernel adds the slices in a fixed order, so the result is reproducible (no atomics).
// Source row for the weight gradient, without branches so that the index loads of all
// (tap, column) pairs of a block are in flight together; a missing neighbour, a column or a
// tap out of range all map to row Hin of the row-major copy, which is zero.
__device__ inline int wgrad_src(const ConvArgs& a, int n, int k) {
  const bool live = n < a.N && k < a.K;
  const int nn = min(n, a.N - 1), kk = min(k, a.K - 1);
  int p;
  if (a.mode == kModeS2Deconv) {
    const int node = a.nempty ? a.ichild[nn] : nn;
    p = (kk == (node & 7)) ? (node >> 3) : -1;
  } else {
    int64_t at;
    if (a.mode == kModeS1) {
      const int node = a.nempty ? a.ichild[nn] : nn;
      at = ((int64_t)(node >> 3) << 6) + sibling_slot(node & 7) + a.slot[kk];
    } else {
      at = ((int64_t)nn << 6) + a.slot[kk];
    }
    p = a.neigh[at];
    if (a.nempty) {
      const int c = a.child[max(p, 0)];
      p = p >= 0 ? c : -1;
    }
  }
  return (live && p >= 0 && p < a.Hin) ? p : a.Hin;
}

// aq[n / 4][mpad][4] <- A[M][N]: four consecutive columns of a row become one 16-byte unit, rows
// are contiguous within a column quad; zero beyond M and N (N is padded to whole 8-column blocks).
__global__ __launch_bounds__(256) void interleave_quads_kernel(float* __restrict__ aq, const float* __restrict__ A,
    int M, int N, int mpad, int n_quads) {
  __shared__ float tile[64][65];
  const int n0 = blockIdx.x * 64, m0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    const int m = m0 + i, n = n0 + tx;
    tile[i][tx] = (m < M && n < N) ? A[(int64_t)m * N + n] : 0.0f;
  }
  __syncthreads();
  // 16 column quads x 64 rows: consecutive threads take consecutive rows of one quad
  for (int u = threadIdx.x; u < 16 * 64; u += 256) {
    const int q = u >> 6, i = u & 63;
    const int quad = (n0 >> 2) + q, m = m0 + i;
    if (quad < n_quads && m < mpad)
      *reinterpret_cast<float4*>(aq + ((int64_t)quad * mpad + m) * 4) =
          make_float4(tile[i][4 * q], tile[i][4 * q + 1], tile[i][4 * q + 2], tile[i][4 * q + 3]);
  }
}

constexpr int kWgTaps = 3;

template <int MT, int NT, bool FAST>
__global__ __launch_bounds__(256, 2) void conv_wgrad_f32_kernel(ConvArgs a, const float* __restrict__ A,
    const float* __restrict__ xt, float* __restrict__ partial, int cpad, int mpad, int n_slices, int cpasses) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int slice = blockIdx.x * 4 + wave;
  const int tap0 = blockIdx.y * kWgTaps;
  const int mpass = blockIdx.z / cpasses, cpass = blockIdx.z % cpasses;
  const int r = lane & 31, kh = lane >> 5;
  floatx16 acc[kWgTaps][MT][NT];
#pragma unroll
  for (int t = 0; t < kWgTaps; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[t][mt][nt][i] = 0.0f;
  const int nblocks = (a.N + 7) >> 3;
  // a slice is a contiguous range of column blocks: the 128-byte lines of A a wavefront touches
  // (one per row, 16 bytes used per block) and the neighbour rows of xt are reused from L1
  const int per_slice = (nblocks + n_slices - 1) / n_slices;
  const int b_end = min(nblocks, (slice + 1) * per_slice);
  // with two column tiles, tile nt holds the channels 2n + nt, so that one 8-byte load per lane
  // feeds both tiles and a half wavefront reads 256 contiguous bytes of a row
  const float* xcol = xt + (NT == 2 ? cpass * 64 + 2 * r : cpass * 32 + r);
  // software pipeline: the source rows and the A values of block b + 1 are requested before the
  // MFMAs of block b, and all gathers of a block are in flight together
  // FAST = stride 1 over all nodes with whole sibling groups: the index load then carries no
  // branches, so the compiler keeps it in flight across the MFMAs
  const int my_tap = min(tap0 + min(lane >> 3, kWgTaps - 1), a.K - 1);
  const bool tap_live = tap0 + min(lane >> 3, kWgTaps - 1) < a.K;
  const int my_slot = sibling_slot(lane & 7) + a.slot[my_tap];
  auto load_src = [&](int b) {
    // all source rows of a block with one load: lane (t, column) = (lane >> 3, lane & 7)
    if (FAST) return a.neigh[((int64_t)b << 6) + my_slot];  // range-checked when it is used
    return wgrad_src(a, b * 8 + (lane & 7), tap0 + min(lane >> 3, kWgTaps - 1));
  };
  // A comes from its quad-interleaved copy aq[n / 4][mpad][4] (zero beyond M and N): the 32 lanes of
  // a half wavefront read 512 contiguous bytes, every byte of a cache line is used, and the load
  // needs no bounds check.  (Read in place, [M, N] row-major, a wavefront touches one 128-byte line
  // per row and block and uses 16 bytes of it; eight wavefronts then overflow the L1 and A is
  // fetched eight times.)
  auto load_a = [&](int b, float (&av)[MT][4]) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = (mpass * MT + mt) * 32 + r;
      const float4 v = *reinterpret_cast<const float4*>(A + (((int64_t)b * 2 + kh) * mpad + m) * 4);
      av[mt][0] = v.x; av[mt][1] = v.y; av[mt][2] = v.z; av[mt][3] = v.w;
    }
  };
  // gathers of one tap of a block: 4 column pairs x NT tiles
  auto load_b = [&](int srcv, int t, float (&bv)[4][NT]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int lo = __builtin_amdgcn_readlane(srcv, t * 8 + j);
      const int hi = __builtin_amdgcn_readlane(srcv, t * 8 + 4 + j);
      const float* row = xcol + (int64_t)(kh ? hi : lo) * cpad;
      if (NT == 2) {
        const float2 v = *reinterpret_cast<const float2*>(row);
        bv[j][0] = v.x; bv[j][NT - 1] = v.y;
      } else {
        bv[j][0] = *row;
      }
    }
  };
  auto mfma_tap = [&](int t, const float (&av)[MT][4], const float (&bv)[4][NT]) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          acc[t][mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[mt][j], bv[j][nt], acc[t][mt][nt], 0, 0, 0);
  };
  auto checked = [&](int v) { return FAST ? ((tap_live && v >= 0 && v < a.Hin) ? v : a.Hin) : v; };
  // Software pipeline at tap granularity: while the 4 * MT * NT MFMAs of one tap run, the gathers
  // of the next tap are in flight, and the source rows and A values of the NEXT block are
  // requested a whole block ahead.
  static_assert(kWgTaps == 3, "the pipeline below is written for three taps per wavefront");
  const int b_begin = slice * per_slice;
  if (b_begin < b_end) {
    int srcv = checked(load_src(b_begin));
    float av[MT][4], bv0[4][NT], bv1[4][NT];
    load_a(b_begin, av);
    load_b(srcv, 0, bv0);
    for (int b = b_begin; b < b_end; ++b) {
      const int bn = min(b + 1, b_end - 1);  // the last block is requested twice: no branch
      float av_cur[MT][4];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          av_cur[mt][j] = av[mt][j];
      int srcv_next = load_src(bn);
      load_a(bn, av);
      load_b(srcv, 1, bv1);
      __builtin_amdgcn_sched_barrier(0);
      mfma_tap(0, av_cur, bv0);
      __builtin_amdgcn_sched_barrier(0);
      load_b(srcv, 2, bv0);
      __builtin_amdgcn_sched_barrier(0);
      mfma_tap(1, av_cur, bv1);
      __builtin_amdgcn_sched_barrier(0);
      srcv = checked(srcv_next);
      load_b(srcv, 0, bv1);
      __builtin_amdgcn_sched_barrier(0);
      mfma_tap(2, av_cur, bv0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) bv0[j][nt] = bv1[j][nt];
    }
  }
  // partial[slice][tap][m][c]: a half wavefront writes 128 (256) contiguous bytes
#pragma unroll
  for (int t = 0; t < kWgTaps; ++t) {
    const int tap = tap0 + t;
    if (tap >= a.K) continue;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = (mpass * MT + mt) * 32 + 8 * (i / 4) + 4 * kh + (i % 4);
        float* dst = partial + (((int64_t)slice * a.K + tap) * mpad + m) * cpad;
        if (NT == 2) {
          *reinterpret_cast<float2*>(dst + cpass * 64 + 2 * r) = make_float2(acc[t][mt][0][i], acc[t][mt][NT - 1][i]);
        } else {
          dst[cpass * 32 + r] = acc[t][mt][0][i];
        }
      }
  }
}
// Weight gradient of the 3x3x3 stride-1 operator over all nodes, through LDS.  All 27 taps of the
// 8 columns of a block read their source rows from the block's own 64 neighbour slots, so a
// workgroup stages those 64 rows (32 channels each, 8 KiB) once per block, two blocks ahead of
// their use (index -> row -> LDS, each one block apart: memory latency never meets the matrix
// pipe), and eight wavefronts multiply from LDS: wavefront (g, h) owns the taps 7g .. 7g + 6 and
// the 32 rows of A of half h, i.e. 7 accumulator tiles; the two wavefronts of a tap group share
// a SIMD.  A workgroup is one slice of column blocks for one 32-channel chunk and 64 rows of A;
// the partial sums have the layout of the kernel above and go through the same reduction.
constexpr int kWgLdsTaps = 7;
constexpr int kWgLdsRow = 36;   // words per staged row: 32 channels + 4, so that the 16-byte stores of 8 lanes spread over all banks
template <int HALVES>   // 2: 64 rows of A per workgroup (eight wavefronts); 1: 32 rows (four, two workgroups per unit)
__global__ __launch_bounds__(256 * HALVES) void conv_wgrad_f32_lds_kernel(ConvArgs a, const float* __restrict__ A,
    const float* __restrict__ X, float* __restrict__ partial, int cpad, int mpad, int n_slices, int cpasses) {
  __shared__ __attribute__((aligned(16))) float s_rows[3][64 * kWgLdsRow];
  constexpr int kVec = 2 / HALVES;   // 16-byte units a thread stages per block
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int tapgroup = wave & 3, mhalf = wave >> 2;
  const int slice = blockIdx.x;
  const int cpass = blockIdx.y % cpasses, mpass = blockIdx.y / cpasses;
  const int r = lane & 31, kh = lane >> 5;
  const int tap0 = tapgroup * kWgLdsTaps;
  floatx16 acc[kWgLdsTaps];
#pragma unroll
  for (int t = 0; t < kWgLdsTaps; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[t][i] = 0.0f;
  const int nblocks = a.N >> 3;
  const int per_slice = (nblocks + n_slices - 1) / n_slices;
  const int b_begin = slice * per_slice, b_end = min(nblocks, b_begin + per_slice);
  // staging: thread (slot, part) moves 16 * kVec bytes of the 128-byte row of a slot's node in
  // the row-major copy of the input
  struct Units { float4 v[kVec]; };
  const int st_slot = tid / (8 / kVec), st_part = tid % (8 / kVec);
  const float* xcol = X + cpass * 32 + st_part * 4 * kVec;
  // neighbour of this thread's slot in block b, as stored: it is looked at only when the row is
  // requested, one block later, so that the wavefront never waits for the index it just asked for
  auto index_of = [&](int b) { return a.neigh[((int64_t)b << 6) + st_slot]; };
  auto load_row = [&](int p) {   // the zero row if there is no neighbour
    p = (p >= 0 && p < a.Hin) ? p : a.Hin;
    Units u;
#pragma unroll
    for (int v = 0; v < kVec; ++v) u.v[v] = *reinterpret_cast<const float4*>(xcol + (int64_t)p * cpad + 4 * v);
    return u;
  };
  auto store_row = [&](int buf, const Units& u) {
#pragma unroll
    for (int v = 0; v < kVec; ++v)
      *reinterpret_cast<float4*>(&s_rows[buf][st_slot * kWgLdsRow + st_part * 4 * kVec + 4 * v]) = u.v[v];
  };
  // A in place: lane (row, kh) takes the four columns 4 kh .. 4 kh + 3 of block b of its row
  const int m = (mpass * HALVES + mhalf) * 32 + r;
  const float* arow = A + (int64_t)m * a.N + 4 * kh;
  auto load_a = [&](int b) { return *reinterpret_cast<const float4*>(arow + ((int64_t)b << 3)); };
  // LDS word of this lane's B value for k-step j of tap t: row slot(sibling j + 4 kh, tap), channel r
  int boff[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) boff[j] = sibling_slot(j + 4 * kh) * kWgLdsRow + r;
  int tslot[kWgLdsTaps];
#pragma unroll
  for (int t = 0; t < kWgLdsTaps; ++t) tslot[t] = a.slot[min(tap0 + t, a.K - 1)] * kWgLdsRow;
  if (b_begin < b_end) {
    const int last = b_end - 1;
    // Three LDS buffers: while block b is multiplied from registers, the B values of block b + 1
    // are read from LDS and the rows of block b + 2 are written to it; the rows of block b + 3
    // and the index of block b + 4 are in flight from memory.
    auto read_b = [&](int buf, float (&bv)[4][kWgLdsTaps]) {
      const float* src = s_rows[buf];
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int t = 0; t < kWgLdsTaps; ++t) bv[j][t] = src[boff[j] + tslot[t]];
    };
    store_row(0, load_row(index_of(b_begin)));
    store_row(1, load_row(index_of(min(b_begin + 1, last))));
    Units rows_next = load_row(index_of(min(b_begin + 2, last)));
    int idx_next = index_of(min(b_begin + 3, last));
    float4 av = load_a(b_begin);
    __syncthreads();
    float bv[4][kWgLdsTaps];
    read_b(0, bv);
    int nxt = 1;                       // buffer of block b + 1
    for (int b = b_begin; b < b_end; ++b) {
      const float4 av_next = load_a(min(b + 1, last));
      const float aj[4] = {av.x, av.y, av.z, av.w};
      float bv_next[4][kWgLdsTaps];
      read_b(nxt, bv_next);
      // consecutive MFMAs go to different accumulators (k-step outside, tap inside); a tap past
      // the 27th reads the slot of the last one and its tile is never written
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int t = 0; t < kWgLdsTaps; ++t)
          acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(aj[j], bv[j][t], acc[t], 0, 0, 0);
      const int wr = nxt == 2 ? 0 : nxt + 1;   // buffer of block b + 2
      store_row(wr, rows_next);
      rows_next = load_row(idx_next);
      idx_next = index_of(min(b + 4, last));
      av = av_next;
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int t = 0; t < kWgLdsTaps; ++t) bv[j][t] = bv_next[j][t];
      __syncthreads();
      nxt = wr;
    }
  }
  // partial[slice][tap][m][c]
#pragma unroll
  for (int t = 0; t < kWgLdsTaps; ++t) {
    const int tap = tap0 + t;
    if (tap >= a.K) continue;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int mm = (mpass * HALVES + mhalf) * 32 + 8 * (i / 4) + 4 * kh + (i % 4);
      partial[(((int64_t)slice * a.K + tap) * mpad + mm) * cpad + cpass * 32 + r] = acc[t][i];
    }
  }
}

// The LDS-staged weight gradient for every other shape (non-empty nodes, stride 2, the smaller tap
// sets, the deconvolution's geometry): a block of 8 columns reads 8 K source rows, one per
// (tap, column), whose numbers a small launch writes down beforehand (src[block][tap][column],
// wgrad_src: the zero row where there is nothing).  A workgroup stages these rows (32 channels
// each) two blocks ahead of their use, as the kernel above does with the 64 rows of a sibling
// group, and wavefront (g, h) multiplies the taps T g .. T g + T - 1 with the 32 rows of A of
// half h.  A comes from its quad-interleaved copy (any number of columns, zero past the end).
__global__ void wgrad_sources_kernel(ConvArgs a, int* __restrict__ src, int nblocks, int row_bytes) {
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= (int64_t)nblocks * a.K * 8) return;
  const int j = (int)(id & 7), k = (int)((id >> 3) % a.K), b = (int)((id >> 3) / a.K);
  src[id] = wgrad_src(a, b * 8 + j, k) * row_bytes;   // where the row starts in the row-major copy
}
// Blocks of 8 columns a turn of the kernel below takes at once: a turn ends in a barrier, so a tap
// set with few taps per wavefront takes several blocks to keep the matrix pipe fed between two.
__host__ __device__ constexpr int wgrad_src_blocks(int T) { return T >= 7 ? 1 : T == 1 ? 4 : 2; }
// LDS rows of the kernel below: three buffers of a turn's rows, the rows that the taps past the K-th
// of the last wavefront read behind the third buffer (never used), and a spare row
__host__ __device__ inline int wgrad_src_lds_rows(int K, int T) {
  return 3 * K * 8 * wgrad_src_blocks(T) + (32 * T - 8 * K) + 1;
}
// DIRECT: the 2x2x2 stride-2 operator over all nodes.  The eight source rows of column n are the
// eight children 8 n .. 8 n + 7 (tap k = child k), so a block's 64 rows are 64 consecutive rows of
// the finer level and X is read as it lies, channel-major [C][hin]: thread (channel, quad) moves
// four consecutive rows of a channel (16 bytes, a channel's 64 rows are 256 contiguous bytes) and
// scatters them over the staged rows.  No row-major copy of X, no table of row numbers.
// `nturns` turns of wgrad_src_blocks(T) blocks each; aq and src cover whole turns (zero columns /
// the zero row past the last column).
template <int HALVES, int T, bool DIRECT>
__global__ __launch_bounds__(256 * HALVES) void conv_wgrad_f32_lds_src_kernel(int K, int nturns,
    const float* __restrict__ aq, const float* __restrict__ X, int x_bytes, int hin, const int* __restrict__ src,
    float* __restrict__ partial, int cpad, int mpad, int n_slices, int cpasses) {
  static_assert(!DIRECT || (HALVES == 2 && T == 2), "the direct form stages 32 channels x 16 quads a block with 512 threads");
  extern __shared__ __attribute__((aligned(16))) float s_dyn[];
  constexpr int kThreads = 256 * HALVES;
  constexpr int BPT = wgrad_src_blocks(T);
  constexpr int kUnits = DIRECT ? BPT : (T * BPT + HALVES - 1) / HALVES;   // 16-byte units a thread stages per turn (K <= 4 T)
  const int rows8 = K * 8, rows = rows8 * BPT, buf_words = rows * kWgLdsRow;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int tapgroup = wave & 3, mhalf = wave >> 2;
  const int slice = blockIdx.x;
  const int cpass = blockIdx.y % cpasses, mpass = blockIdx.y / cpasses;
  const int r = lane & 31, kh = lane >> 5;
  const int tap0 = tapgroup * T;
  floatx16 acc[T];
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[t][i] = 0.0f;
  const int per_slice = (nturns + n_slices - 1) / n_slices;
  const int b_begin = slice * per_slice, b_end = min(nturns, b_begin + per_slice);
  // Everything the loop reads from memory goes through buffers with 32-bit offsets: a lane's part
  // of the offset is fixed, the turn's part is a scalar, so that a turn of the loop spends next
  // to no vector instructions on addresses (they share the issue port with the MFMAs).
  const __amdgpu_buffer_rsrc_t xbuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(X), 0, x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t sbuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<int*>(DIRECT ? (const int*)X : src), 0,
      DIRECT ? 0 : nturns * rows * 4, 0x00020000);
  const __amdgpu_buffer_rsrc_t abuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(aq), 0,
      nturns * BPT * 2 * mpad * 16, 0x00020000);
  // staging: unit u of a turn = 16 bytes `part` of row u / 8; a thread takes the units
  // tid, tid + kThreads, ... (a unit past the turn's rows repeats the last row and lands in the
  // spare row: no branch in the loop, which the instruction order below relies on)
  const int spare = (wgrad_src_lds_rows(K, T) - 1) * kWgLdsRow;
  int st_src[kUnits], st_lds[kUnits], st_step[kUnits], st_col[kUnits];
#pragma unroll
  for (int v = 0; v < kUnits; ++v) {
    const bool real = tid + v * kThreads < rows * 8;
    const int u = min(tid + v * kThreads, rows * 8 - 1);
    st_src[v] = (u >> 3) * 4;
    st_lds[v] = real ? (u >> 3) * kWgLdsRow + (u & 7) * 4 : spare + (u & 7) * 4;
    st_step[v] = real ? buf_words : 0;
    st_col[v] = (cpass * 32 + (u & 7) * 4) * 4;
  }
  struct Idx { int p[kUnits]; };
  struct Units { u32x4 v[kUnits]; };
  // direct form: thread (channel, quad) = (tid >> 4, tid & 15) of every block of the turn; fine row
  // 4 quad + i of a block is child (row & 7) of column (row >> 3), i.e. staged row
  // (row & 7) * 8 + (row >> 3)
  const int d_off = ((cpass * 32 + (tid >> 4)) * hin + 4 * (tid & 15)) * 4;
  int d_lds[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = 4 * (tid & 15) + i;
    d_lds[i] = ((row & 7) * 8 + (row >> 3)) * kWgLdsRow + (tid >> 4);
  }
  auto index_of = [&](int b) {
    Idx x;
#pragma unroll
    for (int v = 0; v < kUnits; ++v)
      x.p[v] = DIRECT ? b * BPT + v : (int)__builtin_amdgcn_raw_buffer_load_b32(sbuf, st_src[v], b * rows * 4, 0);
    return x;
  };
  auto load_rows = [&](const Idx& x) {
    Units u;
#pragma unroll
    for (int v = 0; v < kUnits; ++v) {
      if (DIRECT) {
        u32x4 q = __builtin_amdgcn_raw_buffer_load_b128(xbuf, d_off, x.p[v] * 256, 0);
        const bool inside = x.p[v] * 64 + 4 * (tid & 15) < hin;   // whole quads: the level has a multiple of 8 rows
        q.x = inside ? q.x : 0u; q.y = inside ? q.y : 0u; q.z = inside ? q.z : 0u; q.w = inside ? q.w : 0u;
        u.v[v] = q;
      } else {
        u.v[v] = __builtin_amdgcn_raw_buffer_load_b128(xbuf, x.p[v] + st_col[v], 0, 0);
      }
    }
    return u;
  };
  auto store_rows = [&](int buf, const Units& u) {
#pragma unroll
    for (int v = 0; v < kUnits; ++v) {
      if (DIRECT) {
        float* base = s_dyn + buf * buf_words + v * rows8 * kWgLdsRow;
        base[d_lds[0]] = __uint_as_float(u.v[v].x); base[d_lds[1]] = __uint_as_float(u.v[v].y);
        base[d_lds[2]] = __uint_as_float(u.v[v].z); base[d_lds[3]] = __uint_as_float(u.v[v].w);
      } else {
        *reinterpret_cast<u32x4*>(&s_dyn[buf * st_step[v] + st_lds[v]]) = u.v[v];
      }
    }
  };
  const int m = (mpass * HALVES + mhalf) * 32 + r;
  const int a_lane = (kh * mpad + m) * 16;
  struct AVals { u32x4 v[BPT]; };
  auto load_a = [&](int b) {
    AVals a4;
#pragma unroll
    for (int bb = 0; bb < BPT; ++bb)
      a4.v[bb] = __builtin_amdgcn_raw_buffer_load_b128(abuf, a_lane, (b * BPT + bb) * 2 * mpad * 16, 0);
    return a4;
  };
  // LDS word of this lane's B value for k-step j of tap t: row (tap, column j + 4 kh), channel r;
  // the block of the turn, the tap and the k-step are constant offsets from the lane's own word
  const int lane_word = (tap0 * 8 + 4 * kh) * kWgLdsRow + r;
  if (b_begin < b_end) {
    const int last = b_end - 1;
    auto read_b = [&](int buf, float (&bv)[BPT][4][T]) {
      const float* base = s_dyn + buf * buf_words + lane_word;
#pragma unroll
      for (int bb = 0; bb < BPT; ++bb) {
        const float* sub = base + bb * rows8 * kWgLdsRow;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int t = 0; t < T; ++t) bv[bb][j][t] = sub[(t * 8 + j) * kWgLdsRow];
      }
    };
    store_rows(0, load_rows(index_of(b_begin)));
    store_rows(1, load_rows(index_of(min(b_begin + 1, last))));
    Units rows_next = load_rows(index_of(min(b_begin + 2, last)));
    Idx idx_next = index_of(min(b_begin + 3, last));
    AVals av = load_a(b_begin);
    __syncthreads();
    // One turn: the MFMAs of turn b from registers, with everything else of the turn spread
    // between them (the two wavefronts of a SIMD meet at the barrier every turn, so work that
    // follows the last MFMA of one finds the matrix pipe idle in the other as well): B values of
    // turn b + 1 out of LDS, rows of turn b + 2 into LDS, rows of turn b + 3 and the numbers of
    // turn b + 4 requested.
    auto turn = [&](int b, int rd, int wr, const float (&cur)[BPT][4][T], float (&nxtv)[BPT][4][T]) {
      const AVals av_next = load_a(min(b + 1, last));
      read_b(rd, nxtv);
#pragma unroll
      for (int bb = 0; bb < BPT; ++bb) {
        const float aj[4] = {__uint_as_float(av.v[bb].x), __uint_as_float(av.v[bb].y), __uint_as_float(av.v[bb].z),
            __uint_as_float(av.v[bb].w)};
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int t = 0; t < T; ++t)
            acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(aj[j], cur[bb][j][t], acc[t], 0, 0, 0);
      }
      store_rows(wr, rows_next);
      rows_next = load_rows(idx_next);
      idx_next = index_of(min(b + 4, last));
      av = av_next;
      constexpr int kMfma = 4 * T * BPT;
      constexpr int kLoads = (DIRECT ? kUnits : 2 * kUnits) + BPT, kWrites = DIRECT ? 4 * kUnits : kUnits;
#pragma unroll
      for (int i = 0; i < kMfma; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
        if ((i * kLoads) / kMfma != ((i + 1) * kLoads) / kMfma) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // a load from memory
        if ((i * kWrites) / kMfma != ((i + 1) * kWrites) / kMfma) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);   // an LDS write
        __builtin_amdgcn_sched_group_barrier(0x006, 2, 0);   // what is left of address arithmetic
      }
      __syncthreads();
    };
    float bva[BPT][4][T], bvb[BPT][4][T];
    read_b(0, bva);
    int rd = 1;                        // buffer of turn b + 1
    for (int b = b_begin; b < b_end; b += 2) {
      int wr = rd == 2 ? 0 : rd + 1;   // buffer of turn b + 2
      turn(b, rd, wr, bva, bvb);
      rd = wr;
      if (b + 1 < b_end) {
        wr = rd == 2 ? 0 : rd + 1;
        turn(b + 1, rd, wr, bvb, bva);
        rd = wr;
      }
    }
  }
  // partial[slice][tap][m][c]
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const int tap = tap0 + t;
    if (tap >= K) continue;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int mm = (mpass * HALVES + mhalf) * 32 + 8 * (i / 4) + 4 * kh + (i % 4);
      partial[(((int64_t)slice * K + tap) * mpad + mm) * cpad + cpass * 32 + r] = acc[t][i];
    }
  }
}

// G <- the slices added up in a fixed order: eight groups of consecutive slices side by side (one
// per 32 threads of a workgroup, each adding its slices in order), then the eight sums in order.
__global__ __launch_bounds__(256) void conv_wgrad_reduce_kernel(float* __restrict__ G, const float* __restrict__ partial,
    int n_slices, int M, int Cin, int K, int mpad, int cpad) {
  __shared__ float s_sum[8][32];
  const int64_t per = (int64_t)K * mpad * cpad;
  const int e = threadIdx.x & 31, grp = threadIdx.x >> 5;
  const int64_t id = (int64_t)blockIdx.x * 32 + e;
  const int per_group = (n_slices + 7) / 8;
  const int s0 = grp * per_group, s1 = min(n_slices, s0 + per_group);
  float sum = 0.0f;
  if (id < per)
    for (int sl = s0; sl < s1; ++sl) sum += partial[sl * per + id];
  s_sum[grp][e] = sum;
  __syncthreads();
  if (grp != 0 || id >= per) return;
  float total = 0.0f;
#pragma unroll
  for (int g = 0; g < 8; ++g) total += s_sum[g][e];
  const int c = (int)(id % cpad), m = (int)((id / cpad) % mpad), k = (int)(id / ((int64_t)cpad * mpad));
  if (m >= M || c >= Cin) return;
  G[((int64_t)m * Cin + c) * K + k] = total;
}

// The staging buffers of the larger tap sets pass the 64 KiB a kernel may use without asking.
template <int HALVES, int T, bool DIRECT = false>
int launch_wgrad_src(dim3 grid, size_t lds, hipStream_t s, int K, int nturns, const float* aq, const float* xt,
    int x_bytes, int hin, const int* src, float* partial, int cpad, int mpad, int n_slices, int cpasses) {
  static std::atomic<size_t> allowed{0};
  if (lds > 64 * 1024 && allowed.load() < lds) {
    OCNN_HIP_OK(hipFuncSetAttribute(reinterpret_cast<const void*>(&conv_wgrad_f32_lds_src_kernel<HALVES, T, DIRECT>),
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    allowed.store(lds);
  }
  conv_wgrad_f32_lds_src_kernel<HALVES, T, DIRECT><<<grid, 256 * HALVES, lds, s>>>(K, nturns, aq, xt, x_bytes, hin, src,
      partial, cpad, mpad, n_slices, cpasses);
  OCNN_LAUNCH_OK("conv_wgrad_lds_src");
  return OCNN_OK;
}
std::atomic<int> g_wgrad_lds{1};   // test hook: 0 sends every shape but 3x3x3 stride 1 over all nodes to the register-fed kernel

struct WgradPlan {
  int MT, NT, mpasses, cpasses, mpad, cpad, n_slices, tapgroups;
  int lds_slices;   // slices of the LDS-staged kernel, 0 if the shape does not qualify for it
  int src_taps;     // taps per wavefront of the LDS-staged kernel with a source table, 0 if the shape does not qualify
  int src_slices;
  size_t xt_bytes, partial_bytes, ichild_bytes, aq_bytes, src_bytes, total_bytes;
};
// `p` is the plan of the underlying convolution geometry (deconv = 0): M rows on the column side,
// channel_in channels on the gathered side.
void make_wgrad_plan(const ConvPlan& p, int M, int channel_in, int nempty, WgradPlan* w) {
  const int mtiles = (M + 31) / 32, ctiles = (channel_in + 31) / 32;
  w->MT = mtiles == 1 ? 1 : 2;
  w->NT = ctiles == 1 ? 1 : 2;
  w->mpasses = (mtiles + w->MT - 1) / w->MT;
  w->cpasses = (ctiles + w->NT - 1) / w->NT;
  w->mpad = w->mpasses * w->MT * 32;
  w->cpad = w->cpasses * w->NT * 32;
  w->tapgroups = (p.taps.count + kWgTaps - 1) / kWgTaps;
  // one round of resident workgroups (two per compute unit at this register budget), so that
  // no second, half-empty round trails; never more slices than column blocks
  const int nblocks = (p.top_h + 7) / 8;
  int per_launch = w->tapgroups * w->mpasses * w->cpasses;
  int groups = 512 / per_launch;
  int max_groups = (nblocks + 3) / 4;
  if (groups > max_groups) groups = max_groups;
  if (groups < 1) groups = 1;
  w->n_slices = groups * 4;
  // the LDS-staged kernel wants one slice per resident workgroup and tile (run_wgrad)
  w->lds_slices = 0;
  if (p.taps.count == 27 && ((M & 63) == 0 || M == 32) && (channel_in & 31) == 0) {
    const int halves = M == 32 ? 1 : 2;
    const int tiles = (channel_in / 32) * (M / (32 * halves));
    w->lds_slices = (halves == 1 ? 512 : 256) / tiles;
    if (w->lds_slices < 1) w->lds_slices = 1;
  }
  // every other shape with whole 32-channel chunks and 32 / 64-row tiles of A: the LDS-staged kernel
  // with a source table (a single tap is a plain product, left to the register-fed kernel)
  w->src_taps = 0; w->src_slices = 0; w->src_bytes = 0;
  const int K = p.taps.count;
  if (K >= 2 && K <= 28 && ((M & 63) == 0 || M == 32) && (channel_in & 31) == 0) {
    const int halves = M == 32 ? 1 : 2;
    w->src_taps = K > 12 ? 7 : K > 8 ? 3 : K > 4 ? 2 : 1;
    const int tiles = (channel_in / 32) * (M / (32 * halves));
    const size_t lds = (size_t)wgrad_src_lds_rows(K, w->src_taps) * kWgLdsRow * sizeof(float);
    const int per_cu = (lds > 80 * 1024 ? 1 : 2) * (halves == 1 ? 2 : 1);
    w->src_slices = 256 * per_cu / tiles;
    if (w->src_slices < 1) w->src_slices = 1;
    if (w->src_slices > nblocks) w->src_slices = nblocks;
    w->src_bytes = align256((size_t)(nblocks + 3) * K * 8 * sizeof(int));   // whole turns of up to four blocks
  }
  w->xt_bytes = align256(((size_t)p.btm_h + 1) * w->cpad * sizeof(float));
  int most_slices = w->n_slices > w->lds_slices ? w->n_slices : w->lds_slices;
  if (w->src_slices > most_slices) most_slices = w->src_slices;
  w->partial_bytes = align256((size_t)most_slices * p.taps.count * w->mpad * w->cpad * sizeof(float));
  w->ichild_bytes = nempty ? align256(sizeof(int) * (size_t)(p.ichild_h + 1)) : 0;
  w->aq_bytes = align256((size_t)(nblocks + 3) * 2 * w->mpad * 4 * sizeof(float));   // zero columns up to a whole turn
  w->total_bytes = w->xt_bytes + w->partial_bytes + w->ichild_bytes + w->aq_bytes + w->src_bytes;
}

// grad_w[M, channel_in * K] from A [M, top_h] (column side) and X [channel_in, btm_h] (gathered side)
int run_wgrad(float* grad_w, const float* A, int M, const float* X, int channel_in, const Info* o,
    const void* octree_dev, const ConvPlan& p, int nempty, void* ws, size_t ws_bytes, hipStream_t s) {
  WgradPlan w;
  make_wgrad_plan(p, M, channel_in, nempty, &w);
  OCNN_REQUIRE(ws && ws_bytes >= w.total_bytes, OCNN_E_WORKSPACE, "workspace %zu < %zu bytes", ws_bytes, w.total_bytes);
  const char* blob = static_cast<const char*>(octree_dev);
  char* wsb = static_cast<char*>(ws);
  ConvArgs a;
  a.M = M; a.Cin = channel_in; a.N = p.top_h; a.K = p.taps.count; a.Hin = p.btm_h; a.Hout = p.top_h;
  a.mode = p.mode; a.nempty = nempty ? 1 : 0; a.mtiles = (M + 31) / 32; a.csteps = 0;
  for (int k = 0; k < 27; ++k) a.slot[k] = tap_slot(k < p.taps.count ? p.taps.tap[k] : 13);
  a.neigh = reinterpret_cast<const int*>(blob + o->ptr_dis(OCNN_NEIGH, p.workspace_depth));
  a.child = reinterpret_cast<const int*>(blob + o->ptr_dis(OCNN_CHILD, p.workspace_depth));
  a.ichild = nullptr; a.bias = nullptr; a.relu = 0;
  float* xt = reinterpret_cast<float*>(wsb);
  float* partial = reinterpret_cast<float*>(wsb + w.xt_bytes);
  if (nempty) {
    int* ichild = reinterpret_cast<int*>(wsb + w.xt_bytes + w.partial_bytes);
    ichild_kernel<<<blocks_for(p.child_h), kBlock, 0, s>>>(ichild, p.ichild_h, a.child, p.child_h);
    OCNN_LAUNCH_OK("ichild");
    a.ichild = ichild;
  }
  // whole sibling groups (N % 8 == 0), every column a node
  const bool fast = a.mode == kModeS1 && !a.nempty && (a.N & 7) == 0;
  if (fast && w.lds_slices > 0 && w.mpad == M && w.cpad == channel_in && (reinterpret_cast<uintptr_t>(A) & 15) == 0) {
    // the output gradient is read in place; every workgroup is a slice of blocks for one tile of
    // 32 channels and 64 rows (one workgroup per compute unit) or 32 rows (two)
    const int halves = M == 32 ? 1 : 2;
    const int tiles = (w.cpad / 32) * (w.mpad / (32 * halves));
    const int n_slices = w.lds_slices;
    dim3 tg((a.Hin + 64) / 64, (w.cpad + 63) / 64);
    transpose_rows_f32_kernel<<<tg, 256, 0, s>>>(xt, X, channel_in, a.Hin, w.cpad);
    OCNN_LAUNCH_OK("transpose_rows");
    if (halves == 1)
      conv_wgrad_f32_lds_kernel<1><<<dim3(n_slices, tiles), 256, 0, s>>>(a, A, xt, partial, w.cpad, w.mpad, n_slices,
          w.cpad / 32);
    else
      conv_wgrad_f32_lds_kernel<2><<<dim3(n_slices, tiles), 512, 0, s>>>(a, A, xt, partial, w.cpad, w.mpad, n_slices,
          w.cpad / 32);
    OCNN_LAUNCH_OK("conv_wgrad_lds");
    const int64_t per = (int64_t)a.K * w.mpad * w.cpad;
    conv_wgrad_reduce_kernel<<<blocks_for(per, 32), 256, 0, s>>>(grad_w, partial, n_slices, M, channel_in, a.K, w.mpad,
        w.cpad);
    OCNN_LAUNCH_OK("conv_wgrad_reduce");
    return OCNN_OK;
  }
  float* aq = reinterpret_cast<float*>(wsb + w.xt_bytes + w.partial_bytes + w.ichild_bytes);
  // whole turns of the LDS-staged kernel (columns past the last one are zero)
  const int bpt = w.src_taps > 0 ? wgrad_src_blocks(w.src_taps) : 1;
  const int nturns = ((a.N + 7) / 8 + bpt - 1) / bpt, nblocks_pad = nturns * bpt;
  const int n_quads = nblocks_pad * 2;
  dim3 qg((n_quads * 4 + 63) / 64, (w.mpad + 63) / 64);
  interleave_quads_kernel<<<qg, 256, 0, s>>>(aq, A, M, a.N, w.mpad, n_quads);
  OCNN_LAUNCH_OK("interleave_quads");
  // 2x2x2 stride 2 over all nodes: the children of column n are the rows 8 n .. 8 n + 7, X is read in place
  if (a.mode == kModeS2Conv && a.K == 8 && !a.nempty && w.src_taps == 2 && (M & 63) == 0 && w.mpad == M &&
      w.cpad == channel_in && a.Hin == 8 * a.N && (int64_t)channel_in * a.Hin * 4 < (1ll << 31) &&
      (int64_t)n_quads * w.mpad * 16 < (1ll << 31) && (reinterpret_cast<uintptr_t>(X) & 15) == 0 && g_wgrad_lds.load()) {
    const int tiles = (w.cpad / 32) * (w.mpad / 64);
    const size_t lds = (size_t)wgrad_src_lds_rows(a.K, 2) * kWgLdsRow * sizeof(float);
    const int slices = std::min(w.src_slices, nturns);
    int e = launch_wgrad_src<2, 2, true>(dim3(slices, tiles), lds, s, a.K, nturns, aq, X, channel_in * a.Hin * 4,
        a.Hin, nullptr, partial, w.cpad, w.mpad, slices, w.cpad / 32);
    if (e) return e;
    const int64_t per = (int64_t)a.K * w.mpad * w.cpad;
    conv_wgrad_reduce_kernel<<<blocks_for(per, 32), 256, 0, s>>>(grad_w, partial, slices, M, channel_in, a.K,
        w.mpad, w.cpad);
    OCNN_LAUNCH_OK("conv_wgrad_reduce");
    return OCNN_OK;
  }
  dim3 tg((a.Hin + 64) / 64, (w.cpad + 63) / 64);
  transpose_rows_f32_kernel<<<tg, 256, 0, s>>>(xt, X, channel_in, a.Hin, w.cpad);
  OCNN_LAUNCH_OK("transpose_rows");
  const int64_t x_bytes = ((int64_t)a.Hin + 1) * w.cpad * 4;
  const int64_t most_bytes = std::max(x_bytes, std::max((int64_t)nblocks_pad * a.K * 32, (int64_t)nblocks_pad * 2 * w.mpad * 16));
  if (w.src_taps > 0 && w.mpad == M && w.cpad == channel_in && most_bytes < (1ll << 31) && g_wgrad_lds.load()) {
    int* src = reinterpret_cast<int*>(wsb + w.xt_bytes + w.partial_bytes + w.ichild_bytes + w.aq_bytes);
    const int slices = std::min(w.src_slices, nturns);
    wgrad_sources_kernel<<<blocks_for((int64_t)nblocks_pad * a.K * 8), kBlock, 0, s>>>(a, src, nblocks_pad, w.cpad * 4);
    OCNN_LAUNCH_OK("wgrad_sources");
    const int halves = M == 32 ? 1 : 2;
    const int tiles = (w.cpad / 32) * (w.mpad / (32 * halves));
    const size_t lds = (size_t)wgrad_src_lds_rows(a.K, w.src_taps) * kWgLdsRow * sizeof(float);
    int e = OCNN_OK;
#define OCNN_WGRAD_SRC(H_, T_)                                                                                    \
    e = launch_wgrad_src<H_, T_>(dim3(slices, tiles), lds, s, a.K, nturns, aq, xt, (int)x_bytes, a.Hin,           \
        src, partial, w.cpad, w.mpad, slices, w.cpad / 32)
    if (halves == 2) {
      if (w.src_taps == 7) OCNN_WGRAD_SRC(2, 7); else if (w.src_taps == 3) OCNN_WGRAD_SRC(2, 3);
      else if (w.src_taps == 2) OCNN_WGRAD_SRC(2, 2); else OCNN_WGRAD_SRC(2, 1);
    } else {
      if (w.src_taps == 7) OCNN_WGRAD_SRC(1, 7); else if (w.src_taps == 3) OCNN_WGRAD_SRC(1, 3);
      else if (w.src_taps == 2) OCNN_WGRAD_SRC(1, 2); else OCNN_WGRAD_SRC(1, 1);
    }
#undef OCNN_WGRAD_SRC
    if (e) return e;
    const int64_t per = (int64_t)a.K * w.mpad * w.cpad;
    conv_wgrad_reduce_kernel<<<blocks_for(per, 32), 256, 0, s>>>(grad_w, partial, slices, M, channel_in, a.K,
        w.mpad, w.cpad);
    OCNN_LAUNCH_OK("conv_wgrad_reduce");
    return OCNN_OK;
  }
  dim3 grid(w.n_slices / 4, w.tapgroups, w.mpasses * w.cpasses);
#define OCNN_WGRAD(MT_, NT_)                                                                                     \
  do {                                                                                                           \
    if (fast) conv_wgrad_f32_kernel<MT_, NT_, true><<<grid, 256, 0, s>>>(a, aq, xt, partial, w.cpad, w.mpad,     \
        w.n_slices, w.cpasses);                                                                                  \
    else conv_wgrad_f32_kernel<MT_, NT_, false><<<grid, 256, 0, s>>>(a, aq, xt, partial, w.cpad, w.mpad,         \
        w.n_slices, w.cpasses);                                                                                  \
  } while (0)
  if (w.MT == 1 && w.NT == 1) OCNN_WGRAD(1, 1);
  else if (w.MT == 1) OCNN_WGRAD(1, 2);
  else if (w.NT == 1) OCNN_WGRAD(2, 1);
  else OCNN_WGRAD(2, 2);
#undef OCNN_WGRAD
  OCNN_LAUNCH_OK("conv_wgrad");
  int64_t per = (int64_t)a.K * w.mpad * w.cpad;
  conv_wgrad_reduce_kernel<<<blocks_for(per, 32), 256, 0, s>>>(grad_w, partial, w.n_slices, M, channel_in, a.K,
      w.mpad, w.cpad);
  OCNN_LAUNCH_OK("conv_wgrad_reduce");
  return OCNN_OK;
}

// Plans of the three pieces of a gradient call: the weight-gradient geometry (always a
// convolution), and the operator that computes the data gradient (the transposed operator).
struct GradPlan {
  ConvPlan geom, data;
  WgradPlan w;
  int geom_depth, data_depth, data_cin, data_cout, wg_M, wg_C;
  size_t total_bytes;
};
int make_grad_plan(const Info* o, int is_deconv, int depth, int channel_in, int num_output, const int* ks,
    int stride, int nempty, int dtype, GradPlan* g) {
  OCNN_REQUIRE(dtype == OCNN_F32, OCNN_E_UNSUPPORTED, "gradients are computed in fp32 only");
  int e;
  if (!is_deconv) {
    // forward conv: X[Cin] at depth -> Y[Cout].  grad_w = dY * col(X)^T; grad_X = deconv(dY; W).
    g->geom_depth = depth;
    g->wg_M = num_output; g->wg_C = channel_in;
    e = make_plan(o, depth, channel_in, num_output, ks, stride, nempty, 0, dtype, &g->geom);
    if (e) return e;
    g->data_depth = stride == 2 ? depth - 1 : depth;
    g->data_cin = num_output; g->data_cout = channel_in;
    e = make_plan(o, g->data_depth, num_output, channel_in, ks, stride, nempty, 1, dtype, &g->data);
    if (e) return e;
  } else {
    // forward deconv: X[Cin] at depth -> Y[Cout] at depth (+1).  grad_w = X * col(dY)^T;
    // grad_X = conv(dY; W).
    g->geom_depth = stride == 2 ? depth + 1 : depth;
    g->wg_M = channel_in; g->wg_C = num_output;
    e = make_plan(o, g->geom_depth, num_output, channel_in, ks, stride, nempty, 0, dtype, &g->geom);
    if (e) return e;
    g->data_depth = g->geom_depth;
    g->data_cin = num_output; g->data_cout = channel_in;
    g->data = g->geom;
  }
  if (e) return e;
  make_wgrad_plan(g->geom, g->wg_M, g->wg_C, nempty, &g->w);
  g->total_bytes = g->w.total_bytes > g->data.total_bytes ? g->w.total_bytes : g->data.total_bytes;
  return OCNN_OK;
}

int run_grad(int is_deconv, void* grad_data, void* grad_w, const void* data_in, int channel_in, int btm_h,
    const void* weights, const void* grad_out, const void* octree_dev, const void* info, int depth,
    int num_output, const int* ks, int stride, int nempty, int dtype, void* ws, size_t ws_bytes, hipStream_t s) {
  OCNN_REQUIRE(data_in && weights && grad_out && octree_dev && info, OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(grad_data || grad_w, OCNN_E_BADARG, "nothing to compute");
  const Info* o = as_info(info);
  GradPlan g;
  int e = make_grad_plan(o, is_deconv, depth, channel_in, num_output, ks, stride, nempty, dtype, &g);
  if (e) return e;
  const int in_h = is_deconv ? g.geom.top_h : g.geom.btm_h;    // rows of data_in
  const int out_h = is_deconv ? g.geom.btm_h : g.geom.top_h;   // rows of grad_out
  OCNN_REQUIRE(btm_h == in_h, OCNN_E_SHAPE, "input height %d, the octree has %d rows at depth %d", btm_h, in_h, depth);
  OCNN_REQUIRE(ws && ws_bytes >= g.total_bytes, OCNN_E_WORKSPACE, "workspace %zu < %zu bytes", ws_bytes, g.total_bytes);
  if (grad_w) {
    const float* A = static_cast<const float*>(is_deconv ? data_in : grad_out);
    const float* X = static_cast<const float*>(is_deconv ? grad_out : data_in);
    e = run_wgrad(static_cast<float*>(grad_w), A, g.wg_M, X, g.wg_C, o, octree_dev, g.geom, nempty, ws, ws_bytes, s);
    if (e) return e;
  }
  if (grad_data) {
    // the transposed operator with the same weight buffer; its workspace use starts after the
    // weight-gradient kernels on the same stream have finished
    e = run_conv(is_deconv ? 0 : 1, grad_data, grad_out, g.data_cin, out_h, weights, octree_dev, info, g.data_depth,
        g.data_cout, ks, stride, nempty, dtype, ws, ws_bytes, s);
    if (e) return e;
  }
  return OCNN_OK;
}

}  // namespace

// ---- scratch memory that belongs to the library ------------------------------------------
// ocnn_octree_conv_static serves callers that cannot allocate (code under HIP graph capture,
// serving loops, harnesses that forbid it): its workspace is this array.  Every GPU the
// library runs on holds its own copy at its own address for the life of the process; the name
// below is only the host-side handle of the symbol, the address kernels may use comes from
// hipGetSymbolAddress with that GPU current.
constexpr size_t kBuiltinScratchBytes = (size_t)OCNN_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kBuiltinScratchBytes];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices];

// The array's address on the current device (looked up once per device), or a negative code.
int builtin_scratch(void** out) {
  int dev = -1;
  OCNN_HIP_OK(hipGetDevice(&dev));
  OCNN_REQUIRE(dev >= 0 && dev < kMaxDevices, OCNN_E_UNSUPPORTED, "device %d beyond the %d this library tracks",
      dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    OCNN_HIP_OK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    OCNN_REQUIRE(ptr != nullptr, OCNN_E_HIP, "the scratch array has no address on device %d", dev);
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return OCNN_OK;
}

// Row-major bf16 operators over all nodes of a level: what a chain of convolutions keeps between
// its members instead of copying every input row-major first.
//   3x3x3 stride 1 (conv / deconv): rows of depth d in, rows of depth d out
//   2x2x2 stride 2 conv:   rows of depth d in, rows of ALL nodes of depth d-1 out (pad folded in)
//   2x2x2 stride 2 deconv: rows of ALL nodes of depth d in (depad folded in), rows of depth d+1 out
struct RowsPlan {
  int kind;            // 0: 3x3x3 s1, 1: 2x2x2 s2 conv, 2: 2x2x2 s2 deconv
  int btm_h, top_h, cols, cpad, out_cpad;
  int MT, npass, ksteps;
  size_t wt_bytes, ichild_bytes, src_bytes, total_bytes;
  int src_pitch;       // columns of the source table (kind 3): the column tiles, whole
  int slab_ch;         // input channels per stage of the row kernels (kind 3)
  bool staged;         // 64 output channels a pass on a level where most taps of a tile are live: weights through LDS
};
int make_rows_plan(const Info* o, int depth, int channel_in, int num_output, const int* ks, int stride, int nempty,
    int deconv, int dtype, RowsPlan* r) {
  OCNN_REQUIRE(o && ks, OCNN_E_BADARG, "null pointer");
  int e = ocnn_info_check(o);
  if (e) return e;
  OCNN_REQUIRE(dtype == OCNN_BF16, OCNN_E_UNSUPPORTED, "row-major operators: bf16");
  OCNN_REQUIRE(depth > 0 && depth <= o->depth, OCNN_E_BADARG, "depth %d not in [1,%d]", depth, o->depth);
  OCNN_REQUIRE(num_output > 0 && channel_in > 0, OCNN_E_BADARG, "channels %d -> %d", channel_in, num_output);
  OCNN_REQUIRE(o->has(OCNN_NEIGH) && o->has(OCNN_CHILD), OCNN_E_FORMAT,
      "the octree holds no neighbour table (not an octree_batch result)");
  const bool k333 = ks[0] == 3 && ks[1] == 3 && ks[2] == 3, k222 = ks[0] == 2 && ks[1] == 2 && ks[2] == 2;
  r->cpad = (channel_in + 15) / 16 * 16;
  r->out_cpad = (num_output + 15) / 16 * 16;
  r->ksteps = r->cpad / 16;
  r->ichild_bytes = 0;
  r->src_bytes = 0;
  r->src_pitch = 0;
  r->slab_ch = kRowSlab;
  r->staged = false;
  const int mtiles = (num_output + 31) / 32;
  if (nempty && stride == 2 && k222 && deconv && depth < o->depth && r->ksteps >= 1 && r->ksteps <= 16 &&
      (int64_t)o->nnum_nempty[depth + 1] * 5 >= (int64_t)o->nnum[depth + 1] * 2) {
    // 2x2x2 stride-2 deconvolution over the non-empty nodes: the all-nodes kernel with the rows of
    // the input as its columns and the child links of the finer level as the map of its output rows.
    // It forms all eight children of a column and drops the empty ones, so it pays where two
    // children in five or more exist (256 -> 128 from depth 6 of the scene: 0.074 -> 0.05 ms); on a
    // sparser level the general row kernel, which forms the non-empty rows only, is ahead (64 -> 32
    // onto depth 9, one child in six: 0.023 against 0.031 ms)
    r->kind = 4;
    r->btm_h = r->cols = o->nnum_nempty[depth];
    r->top_h = o->nnum_nempty[depth + 1];
    r->MT = r->ksteps <= 4 ? 4 : 2;
    r->npass = (8 * mtiles + r->MT - 1) / r->MT;
    r->wt_bytes = align256((size_t)r->npass * r->ksteps * r->MT * 64 * 16);
  } else if (nempty) {
    // over the non-empty nodes: the general row kernel (rows = ranks of the non-empty nodes on
    // both sides, exactly the operator of the channel-major entry points)
    OCNN_REQUIRE((stride == 1 && k333) || (stride == 2 && k222), OCNN_E_UNSUPPORTED,
        "row-major operators: 3x3x3 stride 1, 2x2x2 stride 2");
    ConvPlan p;
    e = make_plan(o, depth, channel_in, num_output, ks, stride, 1, deconv, dtype, &p);
    if (e) return e;
    r->kind = 3;
    r->btm_h = p.btm_h;
    r->top_h = r->cols = p.top_h;
    const bool wide = mtiles % 4 == 0;
    r->MT = mtiles == 1 ? 1 : (wide ? 4 : 2);
    r->npass = (mtiles + r->MT - 1) / r->MT;
    {
      // 64 output channels a pass: on a level where one node in five or more is non-empty (about
      // five neighbours a column and up) 32-channel stages, whose two register sets leave room for
      // three wavefronts a SIMD; on a sparser level (2.2 neighbours a column at depth 9 of a scanned
      // room) 64-channel stages at two wavefronts.  Measured, 64 -> 64 with kept tables: depth 8
      // 0.075 -> 0.060 ms with the first, depth 9 0.062 -> 0.067 ms.
      // Where two nodes in five or more are non-empty (about ten neighbours a column) most taps are
      // live for every wavefront, and weights staged once in LDS for the four wavefronts win again:
      // depth 7, 64 -> 64: 0.050 ms staged against 0.054 ms.
      const bool dense_level = (int64_t)o->nnum_nempty[p.top_depth] * 5 >= o->nnum[p.top_depth];
      const int slab_ch = r->MT == 4 || (r->MT == 2 && dense_level) ? 32 : kRowSlab;
      r->slab_ch = slab_ch;
      r->staged = r->MT == 2 && (int64_t)o->nnum_nempty[p.top_depth] * 5 >= (int64_t)o->nnum[p.top_depth] * 2;
      const int nslab = (r->cpad + slab_ch - 1) / slab_ch;
      r->wt_bytes = align256((size_t)r->npass * p.taps.count * nslab * (slab_ch / 16) * r->MT * 64 * 16);
      // the two orders of a 64-channel pass take the same room: one more line tells them apart, so
      // that weights packed for one are refused by a call that would read them in the other
      if (r->MT == 2 && slab_ch == 32) r->wt_bytes += 256;
    }
    r->ichild_bytes = p.ichild_bytes;
    r->src_pitch = (r->cols + kTileCols - 1) / kTileCols * kTileCols;
    r->src_bytes = align256(sizeof(int) * 27 * (size_t)(r->src_pitch > 0 ? r->src_pitch : kTileCols));
  } else if (stride == 1 && k333) {
    r->kind = 0;
    r->btm_h = r->top_h = r->cols = o->nnum[depth];
    r->MT = mtiles == 1 ? 1 : 2;
    r->npass = (mtiles + r->MT - 1) / r->MT;
    r->wt_bytes = align256((size_t)r->npass * r->ksteps * 27 * r->MT * 64 * 16);
  } else if (stride == 2 && k222 && !deconv) {
    r->kind = 1;
    r->btm_h = o->nnum[depth];
    r->top_h = r->cols = o->nnum[depth - 1];
    r->MT = mtiles == 1 ? 1 : 2;
    r->npass = (mtiles + r->MT - 1) / r->MT;
    r->wt_bytes = align256((size_t)r->npass * 8 * r->ksteps * r->MT * 64 * 16);
  } else if (stride == 2 && k222 && deconv) {
    OCNN_REQUIRE(depth < o->depth, OCNN_E_BADARG, "output depth %d outside the octree", depth + 1);
    OCNN_REQUIRE(r->ksteps >= 1 && r->ksteps <= 16, OCNN_E_UNSUPPORTED,
        "row-major stride-2 deconvolution: at most 256 input channels");
    r->kind = 2;
    r->btm_h = o->nnum[depth];
    r->cols = o->nnum_nempty[depth];
    r->top_h = o->nnum[depth + 1];
    r->MT = r->ksteps <= 4 ? 4 : 2;
    r->npass = (8 * mtiles + r->MT - 1) / r->MT;
    r->wt_bytes = align256((size_t)r->npass * r->ksteps * r->MT * 64 * 16);
    r->ichild_bytes = align256(sizeof(int) * (size_t)(r->cols + 1));
  } else {
    return fail(OCNN_E_UNSUPPORTED, "row-major operators: 3x3x3 stride 1, 2x2x2 stride 2");
  }
  r->total_bytes = r->wt_bytes + r->ichild_bytes;   // (the table of sources is the caller's, see ocnn_conv_rows_sources)
  return OCNN_OK;
}

// `packed` (optional): the weights as ocnn_conv_rows_pack left them -- then `weights` is not read and no
// packing kernel runs; `ichild_in` (optional): the inverted child links the operator needs -- then
// none are computed.  With both (or with `packed` for an operator that needs no links) the call needs
// no workspace.  `only_pack`: pack `weights` into `ws` and return.
int run_conv_rows(int deconv, void* top_rows, int top_pitch, const void* btm_rows, int btm_pitch, int channel_in,
    int btm_h, const void* weights, const float* bias, int relu, const void* octree_dev, const void* info,
    int depth, int num_output, const int* ks, int stride, int nempty, int dtype, void* ws, size_t ws_bytes,
    hipStream_t s, const void* packed = nullptr, const int* ichild_in = nullptr, bool only_pack = false,
    const int* sources_in = nullptr, int* sources_out = nullptr) {
  OCNN_REQUIRE((only_pack || sources_out || (top_rows && btm_rows)) && (weights || packed || sources_out) && octree_dev &&
      info && ks, OCNN_E_BADARG, "null pointer");
  const Info* o = as_info(info);
  RowsPlan r;
  int e = make_rows_plan(o, depth, channel_in, num_output, ks, stride, nempty, deconv, dtype, &r);
  if (e) return e;
  // the inverted child links serve the look-up of the source rows only: a caller that brings the
  // table of sources needs none
  const bool need_links = r.ichild_bytes > 0 && !ichild_in && !only_pack && !(sources_in && r.kind == 3);
  const size_t ws_need = (packed || sources_out ? 0 : r.wt_bytes) + (need_links ? r.ichild_bytes : 0);
  OCNN_REQUIRE(ws_need == 0 || (ws && ws_bytes >= ws_need), OCNN_E_WORKSPACE, "workspace %zu < %zu bytes", ws_bytes, ws_need);
  OCNN_REQUIRE(ws_need == 0 || (reinterpret_cast<uintptr_t>(ws) & 15) == 0, OCNN_E_WORKSPACE, "workspace not 16-byte aligned");
  OCNN_REQUIRE(!packed || (reinterpret_cast<uintptr_t>(packed) & 15) == 0, OCNN_E_BADARG, "packed weights not 16-byte aligned");
  char* wsb = static_cast<char*>(ws);
  if (!packed && !sources_out) {   // the weights in the order the kernel of this operator reads them
    const int mtiles_w = (num_output + 31) / 32;
    if (r.kind == 0) {
      const int64_t sm = deconv ? 27 : (int64_t)channel_in * 27, sc = deconv ? (int64_t)num_output * 27 : 27;
      const int64_t total = (int64_t)r.npass * r.ksteps * 27 * r.MT * 64 * 8;
      pack_weights_lds_bf16<<<blocks_for(total), kBlock, 0, s>>>((uint16_t*)ws, (const uint16_t*)weights, num_output,
          channel_in, r.MT, r.npass, r.ksteps, sm, sc, deconv);
    } else if (r.kind == 1) {
      const int64_t total = (int64_t)r.npass * 8 * r.ksteps * r.MT * 64 * 8;
      pack_weights_s2_rows_bf16<<<blocks_for(total), kBlock, 0, s>>>((uint16_t*)ws, (const uint16_t*)weights, num_output,
          channel_in, r.MT, r.npass, r.ksteps);
    } else if (r.kind == 2 || r.kind == 4) {
      const int64_t total = (int64_t)r.npass * r.ksteps * r.MT * 64 * 8;
      pack_weights_d2_rows_bf16<<<blocks_for(total), kBlock, 0, s>>>((uint16_t*)ws, (const uint16_t*)weights, num_output,
          channel_in, r.MT, r.npass, r.ksteps);
    } else {
      const int K = stride == 1 ? 27 : 8;
      const int64_t sm = deconv ? K : (int64_t)channel_in * K, sc = deconv ? (int64_t)num_output * K : K;
      const int slab_ch = r.slab_ch;
      const int nslab = (r.cpad + slab_ch - 1) / slab_ch;
      const int64_t total = (int64_t)r.npass * K * nslab * (slab_ch / 16) * r.MT * 64 * 8;
      pack_weights_rows_bf16<<<blocks_for(total), kBlock, 0, s>>>((uint16_t*)ws, (const uint16_t*)weights, num_output,
          channel_in, K, r.MT, r.npass, nslab, sm, sc, slab_ch);
    }
    (void)mtiles_w;
    OCNN_LAUNCH_OK("pack_weights");
    if (only_pack) return OCNN_OK;
  }
  const void* wpk = packed ? packed : ws;
  int* links_ws = reinterpret_cast<int*>(wsb + (packed || sources_out ? 0 : r.wt_bytes));
  OCNN_REQUIRE(sources_out || btm_h == r.btm_h, OCNN_E_SHAPE, "input height %d, the octree has %d rows at depth %d", btm_h,
      r.btm_h, depth);
  // the stride-2 convolution also reads a channel slice of a wider tensor (an encoder feature that
  // sits in the tensor the decoder reads as a concatenation)
  OCNN_REQUIRE(btm_pitch == r.cpad || ((r.kind == 1 || r.kind == 3 || r.kind == 4) && btm_pitch > r.cpad && btm_pitch % 8 == 0), OCNN_E_SHAPE,
      "input pitch %d: rows of %d channels are padded to %d", btm_pitch, channel_in, r.cpad);
  OCNN_REQUIRE(top_pitch >= r.out_cpad && top_pitch % 8 == 0, OCNN_E_SHAPE, "output pitch %d for %d channels",
      top_pitch, num_output);
  OCNN_REQUIRE(((reinterpret_cast<uintptr_t>(top_rows) | reinterpret_cast<uintptr_t>(btm_rows)) & 15) == 0,
      OCNN_E_BADARG, "rows not 16-byte aligned");
  OCNN_REQUIRE(((int64_t)btm_h + 1) * btm_pitch * 2 < ((int64_t)1 << 31) - (1 << 20) &&
      ((int64_t)r.top_h + 1) * top_pitch * 2 < ((int64_t)1 << 31) - (1 << 20), OCNN_E_UNSUPPORTED,
      "level too large for 32-bit row offsets");
  const char* blob = static_cast<const char*>(octree_dev);
  ConvArgs a;
  a.M = num_output;
  a.Cin = channel_in;
  a.N = r.cols;
  a.Hin = btm_h;
  a.Hout = r.top_h;
  a.nempty = 0;
  a.mtiles = (num_output + 31) / 32;
  a.csteps = 0;
  a.ichild = nullptr;
  a.bias = bias;
  a.relu = relu ? 1 : 0;
  for (int k = 0; k < 27; ++k) a.slot[k] = 0;
  if (r.kind == 3) {
    ConvPlan p;
    e = make_plan(o, depth, channel_in, num_output, ks, stride, 1, deconv, dtype, &p);
    if (e) return e;
    const bool empty_level = o->nnum_nempty[p.top_depth] == 0;
    if (empty_level) {   // one zero row (octree_conv.cpp:82) and the zero row behind it
      OCNN_REQUIRE(top_pitch == r.out_cpad, OCNN_E_UNSUPPORTED, "empty level into a channel slice");
      const int64_t cnt = ((int64_t)r.top_h + 1) * top_pitch;
      zero_rows_kernel<uint16_t><<<blocks_for(cnt), kBlock, 0, s>>>((uint16_t*)top_rows, cnt);
      OCNN_LAUNCH_OK("zero_rows");
      return OCNN_OK;
    }
    a.K = p.taps.count;
    a.mode = p.mode;
    a.nempty = 1;
    for (int k = 0; k < 27; ++k) {
      const int tap = k < p.taps.count ? p.taps.tap[k] : 13;
      a.slot[k] = tap_slot(deconv && stride == 1 ? 26 - tap : tap);
    }
    a.neigh = reinterpret_cast<const int*>(blob + o->ptr_dis(OCNN_NEIGH, p.workspace_depth));
    a.child = reinterpret_cast<const int*>(blob + o->ptr_dis(OCNN_CHILD, p.workspace_depth));
    if (ichild_in) {
      a.ichild = ichild_in;
    } else if (need_links) {
      ichild_kernel<<<blocks_for(p.child_h), kBlock, 0, s>>>(links_ws, p.ichild_h, a.child, p.child_h);
      a.ichild = links_ws;
    }
    // the source rows of every (tap, column): the caller's table, or looked up per tile inside the
    // kernel (a table made for one call costs more than it saves: 0.087 -> 0.095 ms at depth 9)
    if (sources_out) {
      a.Hin = r.btm_h;
      conv_sources_kernel<<<blocks_for(r.src_pitch), kBlock, 0, s>>>(a, sources_out, r.src_pitch);
      OCNN_LAUNCH_OK("conv_sources");
      return OCNN_OK;
    }
    if (sources_in) {
      a.src_table = sources_in;
      a.src_pitch = r.src_pitch;
    }
    const int n_tiles = (a.N + kTileCols - 1) / kTileCols;
    const dim3 grid(((n_tiles + 7) / 8) * 8, pass_split(n_tiles, r.npass));
    const bool direct = a.K >= 3 && g_rows_direct.load() != 0;
    // the barrier-free kernel in workgroups of four, two or one wavefront (direct_waves)
    auto launch_direct = [&](auto mt, auto slab, auto wps) {
      constexpr int MT_ = decltype(mt)::value, SLAB_ = decltype(slab)::value, WPS_ = decltype(wps)::value;
      const int waves = direct_waves(a.N, r.npass);
      const int tiles = (a.N + kWaveCols * waves - 1) / (kWaveCols * waves);
      const dim3 g(((tiles + 7) / 8) * 8, pass_split(tiles, r.npass));
      if (waves == 4)
        conv_rows_bf16_direct_kernel<MT_, SLAB_, true, WPS_, 4><<<g, 256, 0, s>>>(a, (uint16_t*)top_rows, (const u32x4*)btm_rows,
            (const u32x4*)wpk, tiles, r.cpad, btm_pitch, top_pitch, r.out_cpad);
      else if (waves == 2)
        conv_rows_bf16_direct_kernel<MT_, SLAB_, true, WPS_, 2><<<g, 128, 0, s>>>(a, (uint16_t*)top_rows, (const u32x4*)btm_rows,
            (const u32x4*)wpk, tiles, r.cpad, btm_pitch, top_pitch, r.out_cpad);
      else
        conv_rows_bf16_direct_kernel<MT_, SLAB_, true, WPS_, 1><<<g, 64, 0, s>>>(a, (uint16_t*)top_rows, (const u32x4*)btm_rows,
            (const u32x4*)wpk, tiles, r.cpad, btm_pitch, top_pitch, r.out_cpad);
    };
    using std::integral_constant;
    if (r.slab_ch == 32 && r.MT == 2 && direct && !r.staged)
      launch_direct(integral_constant<int, 2>(), integral_constant<int, 32>(), integral_constant<int, 3>());
    else if (r.slab_ch == 32 && r.MT == 2)
      conv_rows_bf16_deep_kernel<2, 32, true><<<grid, 256, 0, s>>>(a, (uint16_t*)top_rows, (const u32x4*)btm_rows,
          (const u32x4*)wpk, n_tiles, r.cpad, btm_pitch, top_pitch, r.out_cpad);
    else if (direct && r.MT == 4)
      launch_direct(integral_constant<int, 4>(), integral_constant<int, 32>(), integral_constant<int, 2>());
    else if (direct && r.MT == 2)
      launch_direct(integral_constant<int, 2>(), integral_constant<int, kRowSlab>(), integral_constant<int, 2>());
    else if (direct)
      launch_direct(integral_constant<int, 1>(), integral_constant<int, kRowSlab>(), integral_constant<int, 2>());
    else if (r.MT == 4)
      conv_rows_bf16_deep_kernel<4, 32, true><<<grid, 256, 0, s>>>(a, (uint16_t*)top_rows, (const u32x4*)btm_rows,
          (const u32x4*)wpk, n_tiles, r.cpad, btm_pitch, top_pitch, r.out_cpad);
    else if (r.MT == 2)
      conv_rows_bf16_deep_kernel<2, kRowSlab, true><<<grid, 256, 0, s>>>(a, (uint16_t*)top_rows, (const u32x4*)btm_rows,
          (const u32x4*)wpk, n_tiles, r.cpad, btm_pitch, top_pitch, r.out_cpad);
    else
      conv_rows_bf16_deep_kernel<1, kRowSlab, true><<<grid, 256, 0, s>>>(a, (uint16_t*)top_rows, (const u32x4*)btm_rows,
          (const u32x4*)wpk, n_tiles, r.cpad, btm_pitch, top_pitch, r.out_cpad);
    OCNN_LAUNCH_OK("octree_conv_rows");
    return OCNN_OK;
  }
  if (r.top_h == 0 || r.cols == 0) {   // nothing to convolve: zero rows (one data row at least, and the zero row)
    const int64_t cnt = ((int64_t)r.top_h + 1) * top_pitch;
    OCNN_REQUIRE(top_pitch == r.out_cpad, OCNN_E_UNSUPPORTED, "empty level into a channel slice");
    zero_rows_kernel<uint16_t><<<blocks_for(cnt), kBlock, 0, s>>>((uint16_t*)top_rows, cnt);
    OCNN_LAUNCH_OK("zero_rows");
    return OCNN_OK;
  }
  if (r.kind == 0) {
    KernelTaps taps;
    kernel_taps(ks, &taps);
    a.K = 27;
    a.mode = kModeS1;
    for (int k = 0; k < 27; ++k) a.slot[k] = tap_slot(deconv ? 26 - taps.tap[k] : taps.tap[k]);
    a.neigh = reinterpret_cast<const int*>(blob + o->ptr_dis(OCNN_NEIGH, depth));
    a.child = reinterpret_cast<const int*>(blob + o->ptr_dis(OCNN_CHILD, depth));
    const int r_tiles = ((a.N >> 3) + kRegTileGroups - 1) / kRegTileGroups;
    if (r_tiles * pass_split(r_tiles, r.npass) < 128 && g_bf16_reg_min_tiles.load(std::memory_order_relaxed) > 1) {
      // a level that gives the 1024-column workgroups of the register-fed kernel fewer than 128
      // (tiles x passes): the LDS kernel's 256-column workgroups, three a compute unit, fill the
      // device better (same weights, same products in the same order).  Measured: 12 824 columns,
      // 128 -> 256: 73 -> 48 us; 44 512 columns, 256 -> 256 (176 workgroups): 152 us against 163.
      const int n_tiles = (a.N + kTileCols - 1) / kTileCols;
      const dim3 lgrid(((n_tiles + 7) / 8) * 8, pass_split(n_tiles, r.npass));
      if (r.MT == 1)
        conv_s1_bf16_lds_kernel<1, true><<<lgrid, 256, 0, s>>>(a, (uint16_t*)top_rows, (const u32x4*)btm_rows,
            (const u32x4*)wpk, n_tiles, r.cpad / 8, btm_pitch / 8, top_pitch, r.out_cpad);
      else
        conv_s1_bf16_lds_kernel<2, true><<<lgrid, 256, 0, s>>>(a, (uint16_t*)top_rows, (const u32x4*)btm_rows,
            (const u32x4*)wpk, n_tiles, r.cpad / 8, btm_pitch / 8, top_pitch, r.out_cpad);
      OCNN_LAUNCH_OK("octree_conv_rows");
      return OCNN_OK;
    }
    const dim3 grid(((r_tiles + 7) / 8) * 8, pass_split(r_tiles, r.npass));
    if (r.MT == 1)
      conv_s1_bf16_reg_kernel<1, true><<<grid, 256, 0, s>>>(a, (uint16_t*)top_rows, (const u32x4*)btm_rows,
          (const u32x4*)wpk, r_tiles, r.cpad / 8, top_pitch, r.out_cpad);
    else
      conv_s1_bf16_reg_kernel<2, true><<<grid, 256, 0, s>>>(a, (uint16_t*)top_rows, (const u32x4*)btm_rows,
          (const u32x4*)wpk, r_tiles, r.cpad / 8, top_pitch, r.out_cpad);
  } else if (r.kind == 1) {
    a.K = 8;
    a.mode = kModeS2Conv;
    a.neigh = nullptr;
    a.child = reinterpret_cast<const int*>(blob + o->ptr_dis(OCNN_CHILD, depth - 1));
    const int n_tiles = (a.N + kTileCols - 1) / kTileCols;
    const dim3 grid(((n_tiles + 7) / 8) * 8, pass_split(n_tiles, r.npass));
    if (r.MT == 1)
      conv_s2_rows_bf16_kernel<1><<<grid, 256, 0, s>>>(a, (uint16_t*)top_rows, top_pitch, r.out_cpad,
          (const u32x4*)btm_rows, btm_pitch, r.cpad, (const u32x4*)wpk, n_tiles);
    else
      conv_s2_rows_bf16_kernel<2><<<grid, 256, 0, s>>>(a, (uint16_t*)top_rows, top_pitch, r.out_cpad,
          (const u32x4*)btm_rows, btm_pitch, r.cpad, (const u32x4*)wpk, n_tiles);
  } else if (r.kind == 4) {
    a.K = 8;
    a.mode = kModeS2Deconv;
    a.neigh = nullptr;
    a.child = reinterpret_cast<const int*>(blob + o->ptr_dis(OCNN_CHILD, depth + 1));
    OCNN_REQUIRE(o->nnum[depth + 1] == 8 * r.cols, OCNN_E_FORMAT, "depth %d holds %d nodes for %d non-empty parents",
        depth + 1, o->nnum[depth + 1], r.cols);
    if (r.top_h == 0 || r.cols == 0) {
      OCNN_REQUIRE(top_pitch == r.out_cpad, OCNN_E_UNSUPPORTED, "empty level into a channel slice");
      const int64_t cnt = ((int64_t)r.top_h + 1) * top_pitch;
      zero_rows_kernel<uint16_t><<<blocks_for(cnt), kBlock, 0, s>>>((uint16_t*)top_rows, cnt);
      OCNN_LAUNCH_OK("zero_rows");
      return OCNN_OK;
    }
    const int n_tiles = (a.N + kTileCols - 1) / kTileCols;
    const dim3 grid(((n_tiles + 7) / 8) * 8, pass_split(n_tiles, r.npass));
#define OCNN_D2_ROWS_NE(KS, MT2)                                                                      \
    deconv_s2_rows_bf16_kernel<KS, MT2, true><<<grid, 256, 0, s>>>(a, (uint16_t*)top_rows, top_pitch, r.out_cpad, \
        (const u32x4*)btm_rows, btm_pitch, (const u32x4*)wpk, n_tiles)
    switch (r.ksteps) {
      case 1: OCNN_D2_ROWS_NE(1, 4); break;
      case 2: OCNN_D2_ROWS_NE(2, 4); break;
      case 3: OCNN_D2_ROWS_NE(3, 4); break;
      case 4: OCNN_D2_ROWS_NE(4, 4); break;
      case 5: OCNN_D2_ROWS_NE(5, 2); break;
      case 6: OCNN_D2_ROWS_NE(6, 2); break;
      case 7: OCNN_D2_ROWS_NE(7, 2); break;
      case 8: OCNN_D2_ROWS_NE(8, 2); break;
      case 9: OCNN_D2_ROWS_NE(9, 2); break;
      case 10: OCNN_D2_ROWS_NE(10, 2); break;
      case 11: OCNN_D2_ROWS_NE(11, 2); break;
      case 12: OCNN_D2_ROWS_NE(12, 2); break;
      case 13: OCNN_D2_ROWS_NE(13, 2); break;
      case 14: OCNN_D2_ROWS_NE(14, 2); break;
      case 15: OCNN_D2_ROWS_NE(15, 2); break;
      default: OCNN_D2_ROWS_NE(16, 2); break;
    }
#undef OCNN_D2_ROWS_NE
  } else {
    a.K = 8;
    a.mode = kModeS2Deconv;
    a.neigh = nullptr;
    a.child = reinterpret_cast<const int*>(blob + o->ptr_dis(OCNN_CHILD, depth));
    if (ichild_in) {
      a.ichild = ichild_in;
    } else {
      ichild_kernel<<<blocks_for(btm_h), kBlock, 0, s>>>(links_ws, r.cols, a.child, btm_h);
      a.ichild = links_ws;
    }
    const int n_tiles = (a.N + kTileCols - 1) / kTileCols;
    const dim3 grid(((n_tiles + 7) / 8) * 8, pass_split(n_tiles, r.npass));
#define OCNN_D2_ROWS(KS, MT2)                                                                         \
    deconv_s2_rows_bf16_kernel<KS, MT2><<<grid, 256, 0, s>>>(a, (uint16_t*)top_rows, top_pitch, r.out_cpad, \
        (const u32x4*)btm_rows, btm_pitch, (const u32x4*)wpk, n_tiles)
    switch (r.ksteps) {
      case 1: OCNN_D2_ROWS(1, 4); break;
      case 2: OCNN_D2_ROWS(2, 4); break;
      case 3: OCNN_D2_ROWS(3, 4); break;
      case 4: OCNN_D2_ROWS(4, 4); break;
      case 5: OCNN_D2_ROWS(5, 2); break;
      case 6: OCNN_D2_ROWS(6, 2); break;
      case 7: OCNN_D2_ROWS(7, 2); break;
      case 8: OCNN_D2_ROWS(8, 2); break;
      case 9: OCNN_D2_ROWS(9, 2); break;
      case 10: OCNN_D2_ROWS(10, 2); break;
      case 11: OCNN_D2_ROWS(11, 2); break;
      case 12: OCNN_D2_ROWS(12, 2); break;
      case 13: OCNN_D2_ROWS(13, 2); break;
      case 14: OCNN_D2_ROWS(14, 2); break;
      case 15: OCNN_D2_ROWS(15, 2); break;
      default: OCNN_D2_ROWS(16, 2); break;
    }
#undef OCNN_D2_ROWS
  }
  OCNN_LAUNCH_OK("octree_conv_rows");
  return OCNN_OK;
}

// called by ocnn_device_check so that set-up code can resolve the address ahead of the first call
int prepare_builtin_scratch() {
  void* ptr = nullptr;
  return builtin_scratch(&ptr);
}

}  // namespace ocnn

using namespace ocnn;

extern "C" {

int ocnn_octree_conv_static(void* top, const void* btm, int channel_in, int btm_h, const void* weights,
    const float* bias, int relu, int is_deconv, const void* octree_dev, const void* info, int depth,
    int num_output, const int* kernel_size, int stride, int nempty, int dtype, ocnn_stream_t stream) {
  void* ptr = nullptr;
  int e = builtin_scratch(&ptr);
  if (e) return e;
  return run_conv(is_deconv ? 1 : 0, top, btm, channel_in, btm_h, weights, octree_dev, info, depth, num_output,
      kernel_size, stride, nempty, dtype, ptr, kBuiltinScratchBytes, as_stream(stream), bias, relu, true);
}

int ocnn_conv_rows_direct(int on) {
  g_rows_direct_f32.store(on == 2 ? 2 : (on ? 1 : 0));
  return g_rows_direct.exchange(on ? 1 : 0);
}
int ocnn_conv_wgrad_staged(int on) { return g_wgrad_lds.exchange(on ? 1 : 0); }

int ocnn_conv_bf16_tile_threshold(int tiles) {
  const int old = g_bf16_reg_min_tiles.load();
  g_bf16_reg_min_tiles.store(tiles > 0 ? tiles : (tiles == 0 ? 192 : 1));
  return old;
}

int ocnn_conv_shape(const void* info, int depth, int channel_in, int num_output, const int* kernel_size,
    int stride, int nempty, int is_deconv, int dtype, int* top_h, int* btm_h, size_t* workspace_bytes) {
  ConvPlan p;
  int e = make_plan(as_info(info), depth, channel_in, num_output, kernel_size, stride, nempty, is_deconv,
      dtype, &p);
  if (e) return e;
  if (top_h) *top_h = p.top_h;
  if (btm_h) *btm_h = p.btm_h;
  if (workspace_bytes) *workspace_bytes = p.total_bytes;
  return OCNN_OK;
}

int ocnn_octree_conv(void* top, const void* btm, int channel_in, int btm_h, const void* weights,
    const void* octree_dev, const void* info, int depth, int num_output, const int* kernel_size, int stride,
    int nempty, int dtype, void* workspace_dev, size_t workspace_bytes, ocnn_stream_t stream) {
  return run_conv(0, top, btm, channel_in, btm_h, weights, octree_dev, info, depth, num_output, kernel_size,
      stride, nempty, dtype, workspace_dev, workspace_bytes, as_stream(stream));
}

int ocnn_octree_deconv(void* top, const void* btm, int channel_in, int btm_h, const void* weights,
    const void* octree_dev, const void* info, int depth, int num_output, const int* kernel_size, int stride,
    int nempty, int dtype, void* workspace_dev, size_t workspace_bytes, ocnn_stream_t stream) {
  return run_conv(1, top, btm, channel_in, btm_h, weights, octree_dev, info, depth, num_output, kernel_size,
      stride, nempty, dtype, workspace_dev, workspace_bytes, as_stream(stream));
}

int ocnn_conv1x1_pair(float* out, int* label, const float* data, int channel_in, int height, const float* w1,
    const float* b1, int hidden, int relu1, const float* w2, const float* b2, int num_output, ocnn_stream_t stream) {
  OCNN_REQUIRE(out && data && w1 && w2, OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(channel_in > 0 && height >= 0 && hidden > 0 && num_output > 0, OCNN_E_BADARG, "bad argument");
  OCNN_REQUIRE(hidden <= 32 && num_output <= kPairMaxOut, OCNN_E_UNSUPPORTED,
      "two 1x1x1 convolutions in one pass: at most 32 hidden and %d output channels", kPairMaxOut);
  if (height == 0) return OCNN_OK;
  const int n_tiles = (height + kTileCols - 1) / kTileCols;
  conv_one_tap_pair_f32_kernel<<<((n_tiles + 7) / 8) * 8, 256, 0, as_stream(stream)>>>(out, label, data, w1, b1, w2, b2,
      channel_in, height, hidden, relu1, num_output, n_tiles);
  OCNN_LAUNCH_OK("conv1x1_pair");
  return OCNN_OK;
}

int ocnn_octree_conv_fused(void* top, const void* btm, int channel_in, int btm_h, const void* weights,
    const float* bias, int relu, int is_deconv, const void* octree_dev, const void* info, int depth,
    int num_output, const int* kernel_size, int stride, int nempty, int dtype, void* workspace_dev,
    size_t workspace_bytes, ocnn_stream_t stream) {
  return run_conv(is_deconv ? 1 : 0, top, btm, channel_in, btm_h, weights, octree_dev, info, depth, num_output,
      kernel_size, stride, nempty, dtype, workspace_dev, workspace_bytes, as_stream(stream), bias, relu);
}

int ocnn_octree_conv_fused_sources(void* top, const void* btm, int channel_in, int btm_h, const void* weights,
    const float* bias, int relu, int is_deconv, const int* sources_dev, size_t sources_bytes, const void* octree_dev,
    const void* info, int depth, int num_output, const int* kernel_size, int stride, int nempty, int dtype,
    void* workspace_dev, size_t workspace_bytes, ocnn_stream_t stream) {
  return run_conv(is_deconv ? 1 : 0, top, btm, channel_in, btm_h, weights, octree_dev, info, depth, num_output,
      kernel_size, stride, nempty, dtype, workspace_dev, workspace_bytes, as_stream(stream), bias, relu, false,
      sources_dev, sources_bytes);
}

int ocnn_octree_conv_rows(void* top_rows, int top_pitch, const void* btm_rows, int btm_pitch, int channel_in,
    int btm_h, const void* weights, const float* bias, int relu, int is_deconv, const void* octree_dev,
    const void* info, int depth, int num_output, const int* kernel_size, int stride, int nempty, int dtype,
    void* workspace_dev, size_t workspace_bytes, ocnn_stream_t stream) {
  return run_conv_rows(is_deconv ? 1 : 0, top_rows, top_pitch, btm_rows, btm_pitch, channel_in, btm_h, weights, bias,
      relu, octree_dev, info, depth, num_output, kernel_size, stride, nempty, dtype, workspace_dev, workspace_bytes,
      as_stream(stream));
}

int ocnn_conv_rows_shape(const void* info, int depth, int channel_in, int num_output, const int* kernel_size,
    int stride, int nempty, int is_deconv, int dtype, int* top_h, int* btm_h, size_t* workspace_bytes) {
  RowsPlan r;
  int e = make_rows_plan(as_info(info), depth, channel_in, num_output, kernel_size, stride, nempty, is_deconv, dtype, &r);
  if (e) return e;
  if (top_h) *top_h = r.top_h;
  if (btm_h) *btm_h = r.btm_h;
  if (workspace_bytes) *workspace_bytes = r.total_bytes;
  return OCNN_OK;
}

int ocnn_conv_rows_packed_bytes(const void* info, int depth, int channel_in, int num_output, const int* kernel_size,
    int stride, int nempty, int is_deconv, int dtype, size_t* packed_bytes) {
  RowsPlan r;
  int e = make_rows_plan(as_info(info), depth, channel_in, num_output, kernel_size, stride, nempty, is_deconv, dtype, &r);
  if (e) return e;
  if (packed_bytes) *packed_bytes = r.wt_bytes;
  return OCNN_OK;
}

int ocnn_conv_rows_pack(void* packed_dev, size_t packed_bytes, const void* weights, const void* octree_dev,
    const void* info, int depth, int channel_in, int num_output, const int* kernel_size, int stride, int nempty,
    int is_deconv, int dtype, ocnn_stream_t stream) {
  OCNN_REQUIRE(packed_dev && weights, OCNN_E_BADARG, "null pointer");
  return run_conv_rows(is_deconv ? 1 : 0, nullptr, 0, nullptr, 0, channel_in, 0, weights, nullptr, 0, octree_dev, info,
      depth, num_output, kernel_size, stride, nempty, dtype, packed_dev, packed_bytes, as_stream(stream), nullptr, nullptr,
      true);
}

int ocnn_conv_rows_sources_bytes(const void* info, int depth, const int* kernel_size, int stride, int nempty,
    int is_deconv, size_t* sources_bytes) {
  RowsPlan r;
  int e = make_rows_plan(as_info(info), depth, 16, 16, kernel_size, stride, nempty, is_deconv, OCNN_BF16, &r);
  if (e) return e;
  if (sources_bytes) *sources_bytes = r.src_bytes;
  return OCNN_OK;
}

int ocnn_conv_rows_sources(int* sources_dev, size_t sources_bytes, const int* ichild_dev, const void* octree_dev,
    const void* info, int depth, const int* kernel_size, int stride, int nempty, int is_deconv, void* workspace_dev,
    size_t workspace_bytes, ocnn_stream_t stream) {
  OCNN_REQUIRE(sources_dev, OCNN_E_BADARG, "null pointer");
  RowsPlan r;
  int e = make_rows_plan(as_info(info), depth, 16, 16, kernel_size, stride, nempty, is_deconv, OCNN_BF16, &r);
  if (e) return e;
  OCNN_REQUIRE(r.src_bytes > 0, OCNN_E_UNSUPPORTED, "this operator looks no source rows up (nempty operators do)");
  OCNN_REQUIRE(sources_bytes >= r.src_bytes, OCNN_E_WORKSPACE, "the table takes %zu bytes, the buffer holds %zu",
      (size_t)r.src_bytes, sources_bytes);
  return run_conv_rows(is_deconv ? 1 : 0, nullptr, 16, nullptr, 16, 16, r.btm_h, nullptr, nullptr, 0, octree_dev, info,
      depth, 16, kernel_size, stride, nempty, OCNN_BF16, workspace_dev, workspace_bytes, as_stream(stream), nullptr,
      ichild_dev, false, nullptr, sources_dev);   // (pitches of 16 channels: only the look-up runs)
}

int ocnn_octree_conv_rows_packed(void* top_rows, int top_pitch, const void* btm_rows, int btm_pitch, int channel_in,
    int btm_h, const void* packed_weights, size_t packed_bytes, const int* ichild_dev, const int* sources_dev,
    const float* bias, int relu, int is_deconv, const void* octree_dev, const void* info, int depth, int num_output,
    const int* kernel_size, int stride, int nempty, int dtype, void* workspace_dev, size_t workspace_bytes,
    ocnn_stream_t stream) {
  OCNN_REQUIRE(packed_weights, OCNN_E_BADARG, "null pointer");
  {   // a buffer packed for another operator has another size: refused, not read out of bounds
    RowsPlan r;
    int e = make_rows_plan(as_info(info), depth, channel_in, num_output, kernel_size, stride, nempty, is_deconv, dtype, &r);
    if (e) return e;
    OCNN_REQUIRE(packed_bytes == r.wt_bytes, OCNN_E_WORKSPACE,
        "the packed weights hold %zu bytes, this operator reads %zu (packed for another shape?)", packed_bytes, (size_t)r.wt_bytes);
  }
  return run_conv_rows(is_deconv ? 1 : 0, top_rows, top_pitch, btm_rows, btm_pitch, channel_in, btm_h, nullptr, bias,
      relu, octree_dev, info, depth, num_output, kernel_size, stride, nempty, dtype, workspace_dev, workspace_bytes,
      as_stream(stream), packed_weights, ichild_dev, false, sources_dev);
}

int ocnn_rows_from_channels(void* rows, int pitch, const void* data, int channel, int height, int dtype,
    ocnn_stream_t stream) {
  OCNN_REQUIRE(rows && data, OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(dtype == OCNN_BF16, OCNN_E_UNSUPPORTED, "row-major copies: bf16");
  OCNN_REQUIRE(channel > 0 && height >= 0 && pitch == (channel + 15) / 16 * 16, OCNN_E_SHAPE,
      "pitch %d for %d channels", pitch, channel);
  OCNN_REQUIRE((reinterpret_cast<uintptr_t>(rows) & 15) == 0, OCNN_E_BADARG, "rows not 16-byte aligned");
  dim3 grid((height + 1 + 127) / 128, (pitch + 63) / 64);
  transpose_rows_bf16_kernel<<<grid, 256, 0, as_stream(stream)>>>((uint16_t*)rows, (const uint16_t*)data, channel,
      height, pitch);
  OCNN_LAUNCH_OK("rows_from_channels");
  return OCNN_OK;
}

int ocnn_channels_from_rows(void* data, const void* rows, int pitch, int channel, int height, int dtype,
    ocnn_stream_t stream) {
  OCNN_REQUIRE(rows && data, OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(dtype == OCNN_BF16, OCNN_E_UNSUPPORTED, "row-major copies: bf16");
  OCNN_REQUIRE(channel > 0 && height >= 0 && pitch >= channel && pitch % 8 == 0, OCNN_E_SHAPE,
      "pitch %d for %d channels", pitch, channel);
  OCNN_REQUIRE((reinterpret_cast<uintptr_t>(rows) & 15) == 0, OCNN_E_BADARG, "rows not 16-byte aligned");
  if (height == 0) return OCNN_OK;
  dim3 grid((height + 63) / 64, (channel + 63) / 64);
  transpose_channels_bf16_kernel<<<grid, 256, 0, as_stream(stream)>>>((uint16_t*)data, (const uint16_t*)rows, channel,
      height, pitch);
  OCNN_LAUNCH_OK("channels_from_rows");
  return OCNN_OK;
}

int ocnn_conv_grad_workspace_bytes(const void* info, int depth, int channel_in, int num_output,
    const int* kernel_size, int stride, int nempty, int is_deconv, int dtype, size_t* workspace_bytes) {
  GradPlan g;
  int e = make_grad_plan(as_info(info), is_deconv, depth, channel_in, num_output, kernel_size, stride, nempty,
      dtype, &g);
  if (e) return e;
  if (workspace_bytes) *workspace_bytes = g.total_bytes;
  return OCNN_OK;
}

int ocnn_octree_conv_grad(void* grad_data, void* grad_weights, const void* data_in, int channel_in, int btm_h,
    const void* weights, const void* grad_out, const void* octree_dev, const void* info, int depth,
    int num_output, const int* kernel_size, int stride, int nempty, int dtype, void* workspace_dev,
    size_t workspace_bytes, ocnn_stream_t stream) {
  return run_grad(0, grad_data, grad_weights, data_in, channel_in, btm_h, weights, grad_out, octree_dev, info,
      depth, num_output, kernel_size, stride, nempty, dtype, workspace_dev, workspace_bytes, as_stream(stream));
}

int ocnn_octree_deconv_grad(void* grad_data, void* grad_weights, const void* data_in, int channel_in, int btm_h,
    const void* weights, const void* grad_out, const void* octree_dev, const void* info, int depth,
    int num_output, const int* kernel_size, int stride, int nempty, int dtype, void* workspace_dev,
    size_t workspace_bytes, ocnn_stream_t stream) {
  return run_grad(1, grad_data, grad_weights, data_in, channel_in, btm_h, weights, grad_out, octree_dev, info,
      depth, num_output, kernel_size, stride, nempty, dtype, workspace_dev, workspace_bytes, as_stream(stream));
}


}  // extern "C"
