// Bandwidth-bound gather/scatter ops of the octree hot path: pad / depad,
// octree2col / col2octree (API ops; the convolution itself never builds a
// column buffer), max-pool / unpool / mask-pool.
//
// All tensors are channel-major [C, H]; one thread handles one row index h so
// that a wavefront touches 64 consecutive h (256 B of fp32) per channel, and
// index arrays (label / neigh / mask) are read once and reused over a chunk
// of channels.
#include "ocnn_common.h"

#include <algorithm>
#include <atomic>

namespace ocnn {
namespace {

constexpr int kChanChunk = 8;  // channels handled per thread in the gather ops
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));  // one 16-byte LDS / global unit

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
// A workgroup takes kPadTile rows of the padded side and kChanChunk channels; the labels of
// the tile sit in LDS.  A feature row starts anywhere inside a 256-byte line, and a
// wavefront store that straddles a line boundary costs almost twice an aligned one, so
// every channel walks the tile rotated by its own amount: wavefronts store whole lines and
// only the two ends of the tile are partial.
constexpr int kPadTile = 1024;

template <typename T>
__device__ inline int line_rotation(const T* row) {  // elements up to the next 64-element boundary
  return (int)((0 - (reinterpret_cast<uintptr_t>(row) / sizeof(T))) & 63);
}

// fill: optional fp32 value per channel for the rows without a source (rounded to T), instead of dval
template <typename T>
__global__ void __launch_bounds__(kBlock) pad_forward_kernel(T* __restrict__ Y, int Hy, int C,
    const T* __restrict__ X, int Hx, const int* __restrict__ label, T dval, const float* __restrict__ fill) {
  __shared__ int s_l[kPadTile];
  const int tid = threadIdx.x;
  const int tile0 = blockIdx.x * kPadTile;
  const int rows = min(kPadTile, Hy - tile0);
#pragma unroll
  for (int q = 0; q < kPadTile / kBlock; ++q) {
    const int r = q * kBlock + tid;
    const int l = r < rows ? label[tile0 + r] : -1;
    s_l[r] = (l < 0 || l >= Hx) ? -1 : l;
  }
  __syncthreads();
  for (int c = blockIdx.y; c < C; c += gridDim.y) {  // channels dealt out over blockIdx.y
    T* row = Y + (int64_t)c * Hy + tile0;
    const T* xin = X + (int64_t)c * Hx;
    const int rot = line_rotation(row);
    T v[kPadTile / kBlock];
    int at[kPadTile / kBlock];
    T none = dval;
    if (fill) {
      if constexpr (sizeof(T) == 4) none = fill[c];
      else none = f32_to_bf16(fill[c]);
    }
#pragma unroll
    for (int q = 0; q < kPadTile / kBlock; ++q) {
      const int r = (q * kBlock + tid + rot) & (kPadTile - 1);
      at[q] = r < rows ? r : -1;
      const int l = r < rows ? s_l[r] : -1;
      v[q] = l < 0 ? none : xin[l];
    }
#pragma unroll
    for (int q = 0; q < kPadTile / kBlock; ++q)
      if (at[q] >= 0) row[at[q]] = v[q];
  }
}

// X[c, label[h]] = Y[c, h].  The labels of a tile normally are consecutive numbers in
// ascending order (they are ranks of non-empty nodes), so the tile owns one contiguous piece
// of X: the workgroup inverts the labels in LDS and stores that piece densely.  A tile whose
// labels are anything else (gaps, repeats, a wide spread) is scattered row by row instead.
template <typename T>
__global__ void __launch_bounds__(kBlock) pad_backward_kernel(T* __restrict__ X, int Hx, int C,
    const T* __restrict__ Y, int Hy, const int* __restrict__ label) {
  __shared__ int s_l[kPadTile];
  __shared__ int s_h[kPadTile];
  __shared__ int s_lo[kBlock / 64], s_hi[kBlock / 64];
  const int tid = threadIdx.x;
  const int tile0 = blockIdx.x * kPadTile;
  const int rows = min(kPadTile, Hy - tile0);
  int lo = 0x7fffffff, hi = -1;
#pragma unroll
  for (int q = 0; q < kPadTile / kBlock; ++q) {
    const int r = q * kBlock + tid;
    int l = r < rows ? label[tile0 + r] : -1;
    if (l < 0 || l >= Hx) l = -1;  // rows outside X are ignored rather than written
    s_l[r] = l;
    s_h[r] = -1;
    if (l >= 0) { lo = min(lo, l); hi = max(hi, l); }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    lo = min(lo, __shfl_xor(lo, off));
    hi = max(hi, __shfl_xor(hi, off));
  }
  if ((tid & 63) == 0) { s_lo[tid >> 6] = lo; s_hi[tid >> 6] = hi; }
  __syncthreads();
#pragma unroll
  for (int w = 0; w < kBlock / 64; ++w) { lo = min(lo, s_lo[w]); hi = max(hi, s_hi[w]); }
  if (hi < 0) return;  // nothing of this tile lands in X
  const int span = hi - lo + 1;
  bool dense = span <= kPadTile;
  if (dense) {
#pragma unroll
    for (int q = 0; q < kPadTile / kBlock; ++q) {
      const int r = q * kBlock + tid;
      if (s_l[r] >= 0) s_h[s_l[r] - lo] = r;
    }
    __syncthreads();
    bool all_set = true;
#pragma unroll
    for (int q = 0; q < kPadTile / kBlock; ++q) {
      const int i = q * kBlock + tid;
      if (i < span && s_h[i] < 0) all_set = false;
    }
    dense = __syncthreads_and(all_set) != 0;
    // a label named twice leaves a gap elsewhere, so `dense` also means: no repeats
  }
  for (int c0 = blockIdx.y * kChanChunk; c0 < C; c0 += gridDim.y * kChanChunk) {  // chunks dealt out
  const int c1 = min(C, c0 + kChanChunk);
  if (dense) {
    // the piece of X is a quarter of the tile or less on a sparse level, so the loads that
    // can be in flight are the channels' rather than the rows': all channels of a row first
    const T* yin = Y + (int64_t)c0 * Hy + tile0;
    T* row0 = X + (int64_t)c0 * Hx + lo;
    for (int q = 0; q * kBlock < span + 64; ++q) {
      T v[kChanChunk];
      int at[kChanChunk];
#pragma unroll
      for (int j = 0; j < kChanChunk; ++j) {
        const int rot = line_rotation(row0 + (int64_t)j * Hx);
        const int i = q * kBlock + tid - ((64 - rot) & 63);  // wavefronts start on line boundaries
        at[j] = (c0 + j < c1 && i >= 0 && i < span) ? i : -1;
        if (at[j] >= 0) v[j] = yin[(int64_t)j * Hy + s_h[i]];
      }
#pragma unroll
      for (int j = 0; j < kChanChunk; ++j)
        if (at[j] >= 0) row0[(int64_t)j * Hx + at[j]] = v[j];
    }
  } else {
    for (int c = c0; c < c1; ++c) {
      const T* yin = Y + (int64_t)c * Hy + tile0;
      T* xout = X + (int64_t)c * Hx;
#pragma unroll
      for (int q = 0; q < kPadTile / kBlock; ++q) {
        const int r = q * kBlock + tid;
        if (s_l[r] >= 0) xout[s_l[r]] = yin[r];
      }
    }
  }
  }
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
  int slot[27];   // neighbour slot of each tap for sibling 0
  int rslot[27];  // slot of the opposite offset (the tap seen from the neighbour's side)
};

// neighbour row of column h for tap k, -1 when absent.  P = non-empty variant.
template <bool P>
__device__ inline int64_t col_base(const ColArgs& a, int h, const int* __restrict__ ichild) {
  if (a.stride == 2) return (int64_t)h << 6;
  int hp = P ? ichild[h] : h;
  return ((int64_t)(hp >> 3) << 6) + sibling_slot(hp & 7);
}
template <bool P>
__device__ inline int col_source(const ColArgs& a, int64_t base, int k, const int* __restrict__ neigh,
    const int* __restrict__ child) {
  int p = neigh[base + a.slot[k]];
  if (P && p >= 0) p = child[p];
  return (p >= 0 && p < a.octree_h) ? p : -1;
}

// column whose tap k reads row p, -1 when there is none: the neighbour of p at the
// opposite offset (a stride-2 column is a sibling group, named by its first node).
// Equal to the inverse of col_source whenever the table is a neighbour table of an
// octree, which col_check_kernel verifies.
template <bool P>
__device__ inline int col_target(const ColArgs& a, int p, int k, const int* __restrict__ neigh,
    const int* __restrict__ child, const int* __restrict__ ichild) {
  int pp = P ? ichild[p] : p;
  int q = neigh[((int64_t)(pp >> 3) << 6) + sibling_slot(pp & 7) + a.rslot[k]];
  if (q < 0) return -1;
  int h;
  if (a.stride == 2) {
    if (q & 7) return -1;
    h = q >> 3;
  } else {
    h = P ? child[q] : q;
  }
  return (h >= 0 && h < a.height) ? h : -1;
}

// A workgroup covers kColTile columns.  The rows of col are height_col elements apart,
// so a row starts anywhere inside a 256-byte line, and a wavefront storing 64
// consecutive elements that straddle a line boundary costs almost twice one that
// does not.  Each row (channel, tap) is therefore shifted by its own 0..63 columns so
// that its stores are aligned; the neighbour rows of the tile plus a 64-column apron
// are staged in LDS per tap, where every row finds them under its own shift.
constexpr int kColTile = 256, kColApron = 64;

template <typename T, bool P>
__global__ void __launch_bounds__(kColTile) octree2col_kernel(T* __restrict__ col,
    const T* __restrict__ data, ColArgs a, const int* __restrict__ neigh,
    const int* __restrict__ child, const int* __restrict__ ichild) {
  __shared__ int s_src[2][kColTile + kColApron];
  const int tid = threadIdx.x;
  const int first = blockIdx.x * kColTile - kColApron;  // column staged at s_src[.][0]
  const int lo = a.n * a.height_col;
  // staged columns of this thread: first + tid, and first + kColTile + tid for tid < kColApron
  int hl0 = first + tid, hl1 = first + kColTile + tid;
  bool live0 = hl0 >= 0 && hl0 < a.height_col && lo + hl0 < a.height;
  bool live1 = tid < kColApron && hl1 < a.height_col && lo + hl1 < a.height;
  int64_t base0 = live0 ? col_base<P>(a, lo + hl0, ichild) : 0;
  int64_t base1 = live1 ? col_base<P>(a, lo + hl1, ichild) : 0;
  const int c0 = blockIdx.y * kChanChunk, c1 = min(a.channel, c0 + kChanChunk);
  const uint64_t col_elem = reinterpret_cast<uintptr_t>(col) / sizeof(T);
  // Tap k + 1 is looked up and its values are loaded before tap k is stored, so the
  // loads of one tap fly while the stores of the previous one drain.
  T v[kChanChunk], vn[kChanChunk];
  int64_t at[kChanChunk], atn[kChanChunk];
  auto stage = [&](int k) {
    int* src = s_src[k & 1];
    src[tid] = live0 ? col_source<P>(a, base0, k, neigh, child) : -1;
    if (tid < kColApron) src[kColTile + tid] = live1 ? col_source<P>(a, base1, k, neigh, child) : -1;
  };
  auto load = [&](int k, T* val, int64_t* where) {
    const int* src = s_src[k & 1];
#pragma unroll
    for (int j = 0; j < kChanChunk; ++j) {
      int c = c0 + j;
      int64_t row = ((int64_t)c * a.K + k) * a.height_col;
      int shift = (int)((col_elem + (uint64_t)row) & (kColApron - 1));
      int hl = first + kColApron + tid - shift;
      bool ok = c < c1 && hl >= 0 && hl < a.height_col;
      where[j] = ok ? row + hl : -1;
      int p = ok ? src[kColApron + tid - shift] : -1;
      val[j] = p < 0 ? zero_of<T>() : data[(int64_t)c * a.octree_h + p];
    }
  };
  stage(0);
  __syncthreads();
  load(0, v, at);
  for (int k = 0; k < a.K; ++k) {
    if (k + 1 < a.K) stage(k + 1);
    __syncthreads();  // one barrier per tap: the buffer written here was last read two taps ago
    if (k + 1 < a.K) load(k + 1, vn, atn);
#pragma unroll
    for (int j = 0; j < kChanChunk; ++j)
      if (at[j] >= 0) col[at[j]] = v[j];
#pragma unroll
    for (int j = 0; j < kChanChunk; ++j) { v[j] = vn[j]; at[j] = atn[j]; }
  }
}

// Stride 1 over all nodes: the 27 taps of the 8 columns of a sibling group all lie in
// the group's 64-entry block, so a workgroup stages the blocks of its tile once per
// channel in LDS (64 values per group instead of 8 x 27) and serves every tap from
// there, with the same per-row shift for aligned stores.  Entry s of staged group g
// sits at g * 64 + (s ^ spread(g)), spread() moving the low bits of g to bits 1, 3, 5:
// the 8 columns of a group differ in bits 0, 2, 4 of s, so a wavefront's 64 reads hit
// 64 different banks.
constexpr int kBlockTile = 256;  // columns and threads of a workgroup
constexpr int kStageGroups = (kBlockTile + kColApron) / 8 + 1;  // + 1: a chunk may start inside a group
constexpr int kStageSlots = kStageGroups * 64;
constexpr int kStagePerThread = (kStageSlots + kBlockTile - 1) / kBlockTile;
constexpr int kOctCap = 128;  // octets a tile may copy (a tile of the scenes measured names 66 on average, 132 at most)
constexpr int kOctTab = 512;  // slots of the hash table that finds them (a quarter full at most)

__device__ inline int stage_index(int g, int s) {
  return g * 64 + (s ^ (((g & 1) << 1) | ((g & 2) << 2) | ((g & 4) << 3)));
}

template <typename T, int KC>  // KC: the taps when known (27), which lets the waits count the stores; 0: a.K
__global__ void __launch_bounds__(kBlockTile) octree2col_block_kernel(T* __restrict__ col,
    const T* __restrict__ data, ColArgs a, const int* __restrict__ neigh) {
  __shared__ T s_val[2][kStageSlots];
  const int tid = threadIdx.x;
  const int lo = a.n * a.height_col;
  const int first = blockIdx.x * kBlockTile - kColApron;  // first column the tile may store
  const int g0 = (lo + first) >> 3;                      // first staged group (may be negative)
  // Loads and stores go through buffers (a channel of the input, a row of col): what is not there
  // gets an offset past the end, reads as zero and is not stored, so that neither sits in a branch
  // and the waits are exact: the gathers of the next channel are waited for while the stores of
  // this one are still on their way (with branches the compiler waits for everything in flight).
  constexpr int kNone = (int)0x80000000u;
  int src[kStagePerThread];  // byte offsets of the rows behind this thread's staged entries, the same for every channel
#pragma unroll
  for (int j = 0; j < kStagePerThread; ++j) {
    int i = tid + j * kBlockTile, g = g0 + (i >> 6);
    int p = -1;
    if (i < kStageSlots && g >= 0 && (int64_t)g * 8 < a.height) p = neigh[((int64_t)g << 6) + (i & 63)];
    src[j] = (p >= 0 && p < a.octree_h) ? p * (int)sizeof(T) : kNone;
  }
  const uint64_t col_elem = reinterpret_cast<uintptr_t>(col) / sizeof(T);
  // The rows of the next channel are gathered into registers while the taps of this
  // one are stored.
  T next[kStagePerThread];
  auto gather = [&](int c) {
    const __amdgpu_buffer_rsrc_t plane = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<T*>(data) + (int64_t)c * a.octree_h, 0, a.octree_h * (int)sizeof(T), 0x00020000);
#pragma unroll
    for (int j = 0; j < kStagePerThread; ++j) {
      if constexpr (sizeof(T) == 4) next[j] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(plane, src[j], 0, 0));
      else next[j] = (T)__builtin_amdgcn_raw_buffer_load_b16(plane, src[j], 0, 0);
    }
  };
  auto pass = [&](int c, int turn) __attribute__((always_inline)) {
    T* val = s_val[turn];
#pragma unroll
    for (int j = 0; j < kStagePerThread; ++j) {
      int i = tid + j * kBlockTile;
      if (i < kStageSlots) val[stage_index(i >> 6, i & 63)] = next[j];
    }
    __syncthreads();  // one barrier per channel: the other buffer is still being read
    if (c + (int)gridDim.y < a.channel) gather(c + gridDim.y);
    auto put = [&](int k) {
      int64_t row = ((int64_t)c * a.K + k) * a.height_col;
      int shift = (int)((col_elem + (uint64_t)row) & (kColApron - 1));
      int hl = first + kColApron + tid - shift;
      const bool inside = hl >= 0 && hl < a.height_col;
      int h = lo + hl;
      T v = zero_of<T>();
      if (inside && h < a.height) v = val[stage_index((h >> 3) - g0, sibling_slot(h & 7) + a.slot[k])];
      const __amdgpu_buffer_rsrc_t out_row = __builtin_amdgcn_make_buffer_rsrc(
          col + row, 0, a.height_col * (int)sizeof(T), 0x00020000);
      const int at = inside ? hl * (int)sizeof(T) : kNone;
      if constexpr (sizeof(T) == 4) __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), out_row, at, 0, 0);
      else __builtin_amdgcn_raw_buffer_store_b16((short)v, out_row, at, 0, 0);
    };
    if constexpr (KC > 0) {
#pragma unroll
      for (int k = 0; k < KC; ++k) put(k);
    } else {
#pragma unroll 9
      for (int k = 0; k < a.K; ++k) put(k);
    }
  };
  // Few tiles: channels dealt out over blockIdx.y.  The first channel stands outside the loop so
  // that every turn of the loop starts in the same state (a gather under way and, after it, the
  // stores of the channel before): the wait for the gather can then leave those stores in flight.
  int c = blockIdx.y;
  if (c >= a.channel) return;
  gather(c);
  pass(c, 0);
  int turn = 1;
  for (c += gridDim.y; c < a.channel; c += gridDim.y, turn ^= 1) pass(c, turn);
}

// The same with each value loaded once.  The blocks of neighbouring groups overlap: the 64
// entries of a block lie in 27 sibling octets (rows p with the same p >> 3, 32 contiguous
// bytes of a float channel), and the 41 blocks of a tile name about 70 different octets of a
// scene, not 41 x 27.  A load instruction costs by the cache lines its lanes touch, so the
// tile finds its octets once (a hash table in LDS), loads each of them once per channel in
// 16-byte units, and fills the blocks from that copy.  A tile with more octets than the copy
// holds gathers every entry from memory as above (same results).  Finding the octets costs
// about as much as two channels, and the units need channels that start on 16-byte
// boundaries: other calls go to the kernel above.
template <typename T, int KC>
__global__ void __launch_bounds__(kBlockTile) octree2col_octet_kernel(T* __restrict__ col,
    const T* __restrict__ data, ColArgs a, const int* __restrict__ neigh) {
  constexpr int kUnitElems = 16 / (int)sizeof(T);       // elements of a 16-byte unit
  constexpr int kOctUnits = 8 / kUnitElems;             // units of an octet
  constexpr int kUnits = kOctCap * kOctUnits;           // units of a copy
  constexpr int kUnitLoads = (kUnits + kBlockTile - 1) / kBlockTile;  // units a thread loads per channel
  constexpr int kZeroOct = kOctCap * 8;                 // an octet of zeros behind the copy
  static_assert(kStageSlots % kUnitElems == 0, "the copies start on a 16-byte boundary");
  __shared__ __align__(16) T s_mem[kStageSlots + 2 * (kZeroOct + 8)];
  __shared__ int s_count, s_over;
  T* const val = s_mem;                // the staged blocks
  T* const oct = s_mem + kStageSlots;  // two copies of the octets (this channel's, the next one's), each followed by the zeros
  // The tables of the set-up lie over both and are dead before the first channel.
  int* const s_key = reinterpret_cast<int*>(s_mem);                                  // octet in a slot, or -1
  unsigned short* const s_id = reinterpret_cast<unsigned short*>(s_key + kOctTab);   // its place in the copy
  int* const s_list = reinterpret_cast<int*>(s_id + kOctTab);                        // octet at a place
  static_assert(kOctTab * 6 + kOctCap * 4 <= (int)sizeof(s_mem), "set-up tables");
  const int tid = threadIdx.x;
  const int lo = a.n * a.height_col;
  const int first = blockIdx.x * kBlockTile - kColApron;  // first column the tile may store
  const int g0 = (lo + first) >> 3;                      // first staged group (may be negative)
  // Loads and stores go through buffers (a channel of the input, a row of col): what is not there
  // gets an offset past the end, reads as zero and is not stored, so that neither sits in a branch
  // and the waits are exact: the loads of the next channel are waited for while the stores of
  // this one are still on their way (with branches the compiler waits for everything in flight).
  constexpr int kNone = (int)0x80000000u;
  for (int i = tid; i < kOctTab; i += kBlockTile) s_key[i] = -1;
  if (tid == 0) { s_count = 0; s_over = 0; }
  __syncthreads();
  auto slot_of = [&](int o, bool insert) {  // linear probing; -1: no room (insert) or not there
    const unsigned at = ((unsigned)o * 2654435761u) >> 23;
    for (int probe = 0; probe < 32; ++probe) {
      const int slot = (at + probe) & (kOctTab - 1);
      const int old = insert ? atomicCAS(&s_key[slot], -1, o) : s_key[slot];
      if (old == o || (insert && old == -1)) return slot;
      if (old == -1) return -1;
    }
    return -1;
  };
  // Per staged entry of this thread: first its row, then where its value comes from, the same
  // for every channel (an index into oct, or a byte offset into the channel when gathering).
  int from[kStagePerThread];
#pragma unroll
  for (int j = 0; j < kStagePerThread; ++j) {
    int i = tid + j * kBlockTile, g = g0 + (i >> 6);
    int p = -1;
    if (i < kStageSlots && g >= 0 && (int64_t)g * 8 < a.height) p = neigh[((int64_t)g << 6) + (i & 63)];
    from[j] = (p >= 0 && p < a.octree_h) ? p : -1;
    if (from[j] >= 0 && slot_of(p >> 3, true) < 0) s_over = 1;
  }
  __syncthreads();
  for (int i = tid; i < kOctTab; i += kBlockTile) {
    const int o = s_key[i];
    if (o < 0) continue;
    const int id = atomicAdd(&s_count, 1);  // any order: the places only say where a value waits
    if (id < kOctCap) { s_list[id] = o; s_id[i] = (unsigned short)id; }
  }
  __syncthreads();
  const int n_oct = s_count;
  const bool gathers = s_over != 0 || n_oct > kOctCap;  // the same for the whole workgroup
  int unit_at[kUnitLoads];  // byte offsets, within a channel, of the units this thread copies
#pragma unroll
  for (int l = 0; l < kUnitLoads; ++l) {
    const int u = tid + l * kBlockTile, o = u / kOctUnits;
    unit_at[l] = (!gathers && o < n_oct) ? (s_list[o] * 8 + (u % kOctUnits) * kUnitElems) * (int)sizeof(T) : kNone;
  }
#pragma unroll
  for (int j = 0; j < kStagePerThread; ++j) {
    const int p = from[j];
    if (gathers) from[j] = p >= 0 ? p * (int)sizeof(T) : kNone;
    else from[j] = p >= 0 ? s_id[slot_of(p >> 3, false)] * 8 + (p & 7) : kZeroOct;
  }
  __syncthreads();  // the tables have been read
  if (tid < 16) oct[(tid >> 3) * (kZeroOct + 8) + kZeroOct + (tid & 7)] = zero_of<T>();
  const uint64_t col_elem = reinterpret_cast<uintptr_t>(col) / sizeof(T);
  // What the next channel needs is loaded into registers while the taps of this one are stored.
  u32x4 unit[kUnitLoads];
  T next[kStagePerThread];
  auto fetch = [&](int c) {
    const __amdgpu_buffer_rsrc_t plane = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<T*>(data) + (int64_t)c * a.octree_h, 0, a.octree_h * (int)sizeof(T), 0x00020000);
    if (gathers) {
#pragma unroll
      for (int j = 0; j < kStagePerThread; ++j) {
        if constexpr (sizeof(T) == 4) next[j] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(plane, from[j], 0, 0));
        else next[j] = (T)__builtin_amdgcn_raw_buffer_load_b16(plane, from[j], 0, 0);
      }
    } else {
#pragma unroll
      for (int l = 0; l < kUnitLoads; ++l) unit[l] = __builtin_amdgcn_raw_buffer_load_b128(plane, unit_at[l], 0, 0);
    }
  };
  // Copy b holds the octets of the channel being stored; those of the next channel are written
  // into the other copy at the top of a pass, a whole pass after their loads were issued, and the
  // loads of the channel after that are issued right behind.
  auto land = [&](int b) {
#pragma unroll
    for (int l = 0; l < kUnitLoads; ++l)
      if (tid + l * kBlockTile < kUnits) reinterpret_cast<u32x4*>(oct + b * (kZeroOct + 8))[tid + l * kBlockTile] = unit[l];
  };
  auto pass = [&](int c, int b) __attribute__((always_inline)) {
    const int step = gridDim.y;
    if (!gathers) {
      if (c + step < a.channel) land(b ^ 1);
      if (c + 2 * step < a.channel) fetch(c + 2 * step);
    }
    __syncthreads();  // the octets are in place, and nobody reads the blocks of the channel before
    const T* const here = oct + b * (kZeroOct + 8);
#pragma unroll
    for (int j = 0; j < kStagePerThread; ++j) {
      int i = tid + j * kBlockTile;
      T v = gathers ? next[j] : here[from[j]];
      if (i < kStageSlots) val[stage_index(i >> 6, i & 63)] = v;
    }
    if (gathers && c + step < a.channel) fetch(c + step);
    __syncthreads();  // the blocks are in place
    auto put = [&](int k) {
      int64_t row = ((int64_t)c * a.K + k) * a.height_col;
      int shift = (int)((col_elem + (uint64_t)row) & (kColApron - 1));
      int hl = first + kColApron + tid - shift;
      const bool inside = hl >= 0 && hl < a.height_col;
      int h = lo + hl;
      T v = zero_of<T>();
      if (inside && h < a.height) v = val[stage_index((h >> 3) - g0, sibling_slot(h & 7) + a.slot[k])];
      const __amdgpu_buffer_rsrc_t out_row = __builtin_amdgcn_make_buffer_rsrc(
          col + row, 0, a.height_col * (int)sizeof(T), 0x00020000);
      const int at = inside ? hl * (int)sizeof(T) : kNone;
      if constexpr (sizeof(T) == 4) __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), out_row, at, 0, 0);
      else __builtin_amdgcn_raw_buffer_store_b16((short)v, out_row, at, 0, 0);
    };
    if constexpr (KC > 0) {
#pragma unroll
      for (int k = 0; k < KC; ++k) put(k);
    } else {
#pragma unroll 9
      for (int k = 0; k < a.K; ++k) put(k);
    }
  };
  // Few tiles: channels dealt out over blockIdx.y.  The first channel stands outside the loop so
  // that every turn of the loop starts in the same state (loads under way and, after them, the
  // stores of the channel before): the wait for the loads can then leave those stores in flight.
  int c = blockIdx.y;
  if (c >= a.channel) return;
  fetch(c);
  if (!gathers) {
    land(0);
    if (c + (int)gridDim.y < a.channel) fetch(c + gridDim.y);
  }
  pass(c, 0);
  int b = 1;
  for (c += gridDim.y; c < a.channel; c += gridDim.y, b ^= 1) pass(c, b);
}

// Where a call records that its table is not symmetric.  Either a word the caller owns
// (ocnn_col2octree_cached: the verdict then outlives the call and later calls with the same
// table skip the check), or, for the reference's plain signature, a slot of a ring: a call owns
// slot id % kColSlots and the value id, which no other call ever writes, so slots need no
// clearing; calls overlapping on other streams only collide kColSlots calls apart.
constexpr unsigned long long kColMarkOwned = 0xC01A5E7715BADull;   // "not symmetric" in a caller's word
constexpr int kColSlots = 1024;
__device__ unsigned long long g_col_asymmetric[kColSlots];
std::atomic<unsigned long long> g_col_calls{0};
// the ring's address on the current device (asked once per device)
unsigned long long* col_ring() {
  static std::atomic<unsigned long long*> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  unsigned long long* p = cached[dev].load(std::memory_order_acquire);
  if (p) return p;
  void* q = nullptr;
  if (hipGetSymbolAddress(&q, HIP_SYMBOL(g_col_asymmetric)) != hipSuccess) return nullptr;
  p = static_cast<unsigned long long*>(q);
  cached[dev].store(p, std::memory_order_release);
  return p;
}

// The gather form of col2octree below is exact when (column h, tap k) -> row p and
// (row p, tap k) -> column h are inverse maps.  y = 0 walks the columns of the chunk,
// y = 1 the rows; any pair that does not map back marks the call.
template <bool P>
__global__ void col_check_kernel(ColArgs a, const int* __restrict__ neigh,
    const int* __restrict__ child, const int* __restrict__ ichild, unsigned long long* __restrict__ mark,
    unsigned long long id, bool no_inverse) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (no_inverse) {  // the caller gave no inverse child table: always scatter
    if (i == 0 && blockIdx.y == 0) *mark = id;
    return;
  }
  int lo = a.n * a.height_col, hi = min(a.height, lo + a.height_col);
  bool bad = false;
  if (blockIdx.y == 0) {
    int h = lo + i;
    if (h >= hi) return;
    int64_t base = col_base<P>(a, h, ichild);
    for (int k = 0; k < a.K; ++k) {
      int p = col_source<P>(a, base, k, neigh, child);
      if (p >= 0 && col_target<P>(a, p, k, neigh, child, ichild) != h) bad = true;
    }
  } else {
    int p = i;
    if (p >= a.octree_h) return;
    for (int k = 0; k < a.K; ++k) {
      int h = col_target<P>(a, p, k, neigh, child, ichild);
      if (h >= lo && h < hi &&
          col_source<P>(a, col_base<P>(a, h, ichild), k, neigh, child) != p) bad = true;
    }
  }
  if (bad) *mark = id;
}

// Gather form: one thread per row sums its taps in ascending order, no atomics.
// Leaves the work to col2octree_atomic_kernel when the call is marked (and then only
// clears the rows if this is the first chunk).
template <bool P>
__global__ void col2octree_kernel(const float* __restrict__ col, float* __restrict__ data, ColArgs a,
    const int* __restrict__ neigh, const int* __restrict__ child, const int* __restrict__ ichild,
    const unsigned long long* __restrict__ mark, unsigned long long id) {
  int p = blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= a.octree_h) return;
  bool marked = *mark == id;
  int c0 = blockIdx.y * kChanChunk, c1 = min(a.channel, c0 + kChanChunk);
  float acc[kChanChunk];
#pragma unroll
  for (int j = 0; j < kChanChunk; ++j) acc[j] = 0.0f;
  if (!marked) {
    int lo = a.n * a.height_col, hi = min(a.height, lo + a.height_col);
    int hl[27];  // column of every tap inside the chunk, -1 when there is none
#pragma unroll
    for (int k = 0; k < 27; ++k) {
      int h = k < a.K ? col_target<P>(a, p, k, neigh, child, ichild) : -1;
      hl[k] = (h >= lo && h < hi) ? h - lo : -1;
    }
#pragma unroll
    for (int k = 0; k < 27; ++k) {
      if (hl[k] < 0) continue;
#pragma unroll
      for (int j = 0; j < kChanChunk; ++j)
        if (c0 + j < c1) acc[j] += col[((int64_t)(c0 + j) * a.K + k) * a.height_col + hl[k]];
    }
  } else if (a.n != 0) {
    return;
  }
#pragma unroll
  for (int j = 0; j < kChanChunk; ++j)
    if (c0 + j < c1) {
      float* dst = &data[(int64_t)(c0 + j) * a.octree_h + p];
      *dst = a.n == 0 ? acc[j] : *dst + acc[j];
    }
}

// Gather form for the 27 taps at stride 1 over all nodes, where columns and rows are the same
// nodes: a workgroup owns kGatherTile consecutive rows and streams the same range of the 27
// col rows of a channel through LDS with coalesced 16-byte loads, the next channel flying
// while this one is summed.  A row finds the column of a tap in LDS when that column lies
// inside the tile (19 of 20 do in a depth-9 scene, neighbours being close in z-order); for the
// others the thread asks global memory (a load under a lane mask) before the tile is written to
// LDS.  Taps are summed in ascending order as above.
constexpr int kGatherTile = 1024, kGatherUnits = kGatherTile / 4;  // rows of a tile, 16-byte units of a staged row
constexpr int kGatherLoads = (27 * kGatherUnits + kGatherTile - 1) / kGatherTile;  // 16-byte loads a thread and channel

__global__ void __launch_bounds__(kGatherTile, 4) col2octree_tile_kernel(const float* __restrict__ col,
    float* __restrict__ data, ColArgs a, const int* __restrict__ neigh,
    const unsigned long long* __restrict__ mark, unsigned long long id) {
  extern __shared__ __attribute__((aligned(16))) float s_col[];  // [27][kGatherTile] and one word that stays zero
  const int tid = threadIdx.x;
  const int r0 = blockIdx.x * kGatherTile, p = r0 + tid;
  const int c0 = blockIdx.y * kChanChunk, c1 = min(a.channel, c0 + kChanChunk);
  const int lo = a.n * a.height_col, hi = min(a.height, lo + a.height_col);  // lo is a multiple of 4 (host)
  // The col rows of a channel are one buffer (the host checks that they fit 2 GiB), a tap is a
  // scalar offset into it, and a column is a 32-bit offset; an offset past any buffer reads as
  // zero, and so does each word of a 16-byte load that lies past the end.
  constexpr int kNoColumn = (int)0x80000000u;
  const int row_bytes = a.height_col * 4;
  auto rows_of = [&](int c) {
    return __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(col) + (int64_t)c * 27 * a.height_col, 0, 27 * row_bytes, 0x00020000);
  };
  // staging: load j of the thread is tap tid / kGatherUnits + 4 j, columns 4 (tid % kGatherUnits) .. + 3 of the tile
  const int tap0 = __builtin_amdgcn_readfirstlane(tid / kGatherUnits);
  const int group = (tid % kGatherUnits) * 4;
  const int mine = (r0 + group >= lo && r0 + group < hi) ? (r0 + group - lo) * 4 : kNoColumn;
  u32x4 next[kGatherLoads];
  auto fetch = [&](int c) {
    if (c >= c1) return;
    const __amdgpu_buffer_rsrc_t rows = rows_of(c);
#pragma unroll
    for (int j = 0; j < kGatherLoads; ++j) {
      const int k = tap0 + 4 * j;
      next[j] = __builtin_amdgcn_raw_buffer_load_b128(rows, k < 27 ? mine : kNoColumn, min(k, 26) * row_bytes, 0);
    }
  };
  // Set-up, everything asked for at once: the first tile, the neighbour blocks of the tile's
  // sibling groups (one contiguous piece of the table, read in 16-byte units and laid out in
  // LDS as octree2col_block_kernel does, so that the 8 siblings of 8 groups hit 64 banks) and
  // the mark of the call.
  fetch(c0);
  constexpr int kBlockUnits = kGatherTile / 8 * 64 / 4;  // 16-byte units of the tile's neighbour blocks
  const int table_units = (int)(((int64_t)a.octree_h + 7) / 8 * 16);  // units of the whole table
  const u32x4* table = reinterpret_cast<const u32x4*>(neigh) + (int64_t)(r0 >> 3) * 16;
  u32x4 block[kBlockUnits / kGatherTile];
#pragma unroll
  for (int j = 0; j < kBlockUnits / kGatherTile; ++j) {
    const int u = tid + j * kGatherTile;
    block[j] = (int64_t)(r0 >> 3) * 16 + u < table_units ? table[u] : u32x4{~0u, ~0u, ~0u, ~0u};
  }
  if (*mark == id) {  // the scatter kernel does the work; the first chunk clears the rows for it
    if (a.n == 0 && p < a.octree_h)
      for (int c = c0; c < c1; ++c) data[(int64_t)c * a.octree_h + p] = 0.0f;
    return;
  }
  int* s_block = reinterpret_cast<int*>(s_col);
#pragma unroll
  for (int j = 0; j < kBlockUnits / kGatherTile; ++j) {
    const int u = tid + j * kGatherTile;
#pragma unroll
    for (int e = 0; e < 4; ++e) s_block[stage_index(u >> 4, (u & 15) * 4 + e)] = (int)block[j][e];
  }
  __syncthreads();
  // per tap: the column's place in the staged tile, or kFar + its place in the chunk when it
  // lies outside the tile, or -1 when there is no column
  constexpr int kFar = 1 << 30;
  int where[27];
#pragma unroll
  for (int k = 0; k < 27; ++k) {
    int h = s_block[stage_index(tid >> 3, sibling_slot(tid & 7) + a.rslot[k])];
    bool have = p < a.octree_h && h >= lo && h < hi;  // h < height = octree_h here
    bool inside = have && h >= r0 && h < r0 + kGatherTile;
    where[k] = inside ? h - r0 : (have ? kFar + (h - lo) : -1);
  }
  __syncthreads();  // the blocks make room for the first tile
  auto fetch_far = [&](int c, float (&ask)[27]) {
    if (c >= c1) return;
    const __amdgpu_buffer_rsrc_t rows = rows_of(c);
#pragma unroll
    for (int k = 0; k < 27; ++k) {
      ask[k] = 0.0f;
      if (where[k] >= kFar)  // only the lanes that ask take part in the load
        ask[k] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rows, (where[k] - kFar) * 4, k * row_bytes, 0));
    }
  };
  // One channel: the far columns are asked for, the tile goes from registers to LDS, the loads of
  // the next channel's tile start, then the taps are summed.
  float ask[27];
  if (tid == 0) s_col[27 * kGatherTile] = 0.0f;
  for (int c = c0; c < c1; ++c) {
    fetch_far(c, ask);
    if (c > c0) __syncthreads();  // every wavefront has summed the previous channel
#pragma unroll
    for (int j = 0; j < kGatherLoads; ++j) {
      const int k = tap0 + 4 * j;
      if (k < 27) *reinterpret_cast<u32x4*>(&s_col[k * kGatherTile + group]) = next[j];
    }
    // The far loads sit in branches, where the compiler cannot count them: without this wait for
    // all loads it waits for all of them at the first far value below, when the next tile flies.
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    fetch(c + 1);  // before the barrier: a wavefront whose part of the tile has arrived early asks early
    __syncthreads();
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < 27; ++k) {
      // Every lane reads LDS (the zero word when its column is not in the tile) and takes the bits
      // of the far value on top, which are zero when it did not ask.  A select between the two
      // the compiler turns into an LDS read under a lane mask into the register of the far value,
      // with a wait for every load in flight before each read.
      const unsigned near = __float_as_uint(s_col[(unsigned)where[k] < (unsigned)kGatherTile
                                                      ? k * kGatherTile + where[k] : 27 * kGatherTile]);
      const float v = __uint_as_float(near | __float_as_uint(ask[k]));
      acc = where[k] < 0 ? acc : acc + v;
    }
    if (p < a.octree_h) {
      float* dst = &data[(int64_t)c * a.octree_h + p];
      *dst = a.n == 0 ? acc : *dst + acc;
    }
  }
}

// Scatter form, for any table (octree_nn.cu:130-174); runs only for a marked call.
template <bool P>
__global__ void col2octree_atomic_kernel(const float* __restrict__ col, float* __restrict__ data,
    ColArgs a, const int* __restrict__ neigh, const int* __restrict__ child,
    const int* __restrict__ ichild, const unsigned long long* __restrict__ mark, unsigned long long id) {
  if (*mark != id) return;
  int hl = blockIdx.x * blockDim.x + threadIdx.x;
  if (hl >= a.height_col) return;
  int h = a.n * a.height_col + hl;
  if (h >= a.height) return;
  int64_t base = col_base<P>(a, h, ichild);
  int c0 = blockIdx.y * kChanChunk, c1 = min(a.channel, c0 + kChanChunk);
  for (int k = 0; k < a.K; ++k) {
    int p = col_source<P>(a, base, k, neigh, child);
    if (p < 0) continue;
    for (int c = c0; c < c1; ++c)
      unsafeAtomicAdd(&data[(int64_t)c * a.octree_h + p],
          col[((int64_t)c * a.K + k) * a.height_col + hl]);
  }
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

// Row-major activations ([H + 1][pitch] bf16, row H zero): max pooling with the pad behind it.
// Thread = (node p of the coarser level, 8-channel piece): the node's child link c names the rows
// 8c .. 8c + 7 of the finer level; the eight 16-byte pieces are requested together, the maximum is
// taken channel by channel in row order (the first maximum wins, as in max_pool_kernel), and an
// empty node writes zeros.  Row `top_h` (what a missing neighbour reads) is written as zeros too.
// mask (optional, [top_h + 1][pitch] int32): the absolute row of the maximum, -1 for an empty node.
__global__ __launch_bounds__(kBlock) void max_pool_rows_kernel(uint16_t* __restrict__ top, int top_pitch,
    int* __restrict__ mask, const uint16_t* __restrict__ btm, int btm_pitch, int pieces, const int* __restrict__ child,
    int top_h, int btm_h) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int p = (int)(i / pieces), j = (int)(i % pieces);
  if (p > top_h) return;
  const int c = p < top_h ? child[p] : -1;
  uint4 v[8];
  if (c >= 0 && 8 * (int64_t)c + 7 < btm_h) {
#pragma unroll
    for (int r = 0; r < 8; ++r)
      v[r] = *reinterpret_cast<const uint4*>(btm + (8 * (int64_t)c + r) * btm_pitch + 8 * j);
  } else {
#pragma unroll
    for (int r = 0; r < 8; ++r) v[r] = make_uint4(0, 0, 0, 0);
  }
  uint16_t best[8];
  int arg[8];
  {
    uint16_t h[8];
    memcpy(h, &v[0], 16);
#pragma unroll
    for (int e = 0; e < 8; ++e) { best[e] = h[e]; arg[e] = 0; }
  }
#pragma unroll
  for (int r = 1; r < 8; ++r) {
    uint16_t h[8];
    memcpy(h, &v[r], 16);
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (bf16_to_f32(h[e]) > bf16_to_f32(best[e])) { best[e] = h[e]; arg[e] = r; }
  }
  uint4 o;
  memcpy(&o, best, 16);
  *reinterpret_cast<uint4*>(top + (int64_t)p * top_pitch + 8 * j) = o;
  if (mask) {
    int m[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) m[e] = c >= 0 ? 8 * c + arg[e] : -1;
    int4* dst = reinterpret_cast<int4*>(mask + (int64_t)p * top_pitch + 8 * j);
    dst[0] = make_int4(m[0], m[1], m[2], m[3]);
    dst[1] = make_int4(m[4], m[5], m[6], m[7]);
  }
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
  for (int k = 0; k < 27; ++k) {
    a->slot[k] = k < t.count ? tap_slot(t.tap[k]) : 0;
    a->rslot[k] = k < t.count ? tap_slot(26 - t.tap[k]) : 0;
  }
  return true;
}

int check_col(const void* col, const void* data, int channel, int height, const int* ks, int stride,
    const int* neigh, int height_col, int n, int dtype) {
  OCNN_REQUIRE(col && data && neigh && ks, OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(channel > 0 && height >= 0 && height_col > 0 && n >= 0, OCNN_E_BADARG,
      "channel %d height %d height_col %d n %d", channel, height, height_col, n);
  OCNN_REQUIRE(((int64_t)n + 1) * height_col <= INT32_MAX, OCNN_E_BADARG,
      "chunk %d of %d columns is out of range", n, height_col);
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
  if (!P && stride == 1 && (int64_t)octree_h * 4 < (int64_t(1) << 31) && (int64_t)height_col * 4 < (int64_t(1) << 31)) {
    unsigned tiles = blocks_for((int64_t)height_col + kColApron - 1, kBlockTile);
    dim3 grid(tiles, std::min<unsigned>(channel, std::max(1u, 2048u / tiles)));
    // The octet kernel loads 16-byte units, so every channel must start on a 16-byte boundary,
    // and it pays from about 5 channels per workgroup on.
    const size_t esize = dtype == OCNN_F32 ? 4 : 2;
    const bool octets = reinterpret_cast<uintptr_t>(data) % 16 == 0 && (size_t)octree_h * esize % 16 == 0 &&
        channel / grid.y >= 5;
#define OCNN_O2C(kernel, T, KC) kernel<T, KC><<<grid, kBlockTile, 0, s>>>((T*)col, (const T*)data, a, neigh)
#define OCNN_O2C_TAPS(kernel, T) do { if (a.K == 27) OCNN_O2C(kernel, T, 27); else OCNN_O2C(kernel, T, 0); } while (0)
    if (dtype == OCNN_F32) {
      if (octets) OCNN_O2C_TAPS(octree2col_octet_kernel, float); else OCNN_O2C_TAPS(octree2col_block_kernel, float);
    } else {
      if (octets) OCNN_O2C_TAPS(octree2col_octet_kernel, uint16_t); else OCNN_O2C_TAPS(octree2col_block_kernel, uint16_t);
    }
#undef OCNN_O2C_TAPS
#undef OCNN_O2C
    OCNN_LAUNCH_OK("octree2col");
    return OCNN_OK;
  }
  unsigned tiles = blocks_for((int64_t)height_col + kColApron - 1, kColTile);
  dim3 grid(tiles, (channel + kChanChunk - 1) / kChanChunk);
  if (dtype == OCNN_F32)
    octree2col_kernel<float, P><<<grid, kColTile, 0, s>>>((float*)col, (const float*)data, a, neigh, child, ichild);
  else
    octree2col_kernel<uint16_t, P><<<grid, kColTile, 0, s>>>((uint16_t*)col, (const uint16_t*)data, a, neigh, child, ichild);
  OCNN_LAUNCH_OK("octree2col");
  return OCNN_OK;
}

template <bool P>
int run_col2octree(const void* col, void* data, int channel, int height, int octree_h, const int* ks,
    int stride, const int* neigh, const int* child, const int* ichild, int height_col, int n,
    int dtype, hipStream_t s, unsigned long long* owned_mark = nullptr, bool check_now = true) {
  int e = check_col(col, data, channel, height, ks, stride, neigh, height_col, n, dtype);
  if (e) return e;
  OCNN_REQUIRE(dtype == OCNN_F32, OCNN_E_UNSUPPORTED, "col2octree accumulates in fp32 only");
  ColArgs a;
  OCNN_REQUIRE(fill_col_args(&a, channel, height, octree_h, ks, stride, height_col, n),
      OCNN_E_UNSUPPORTED, "kernel size %d%d%d", ks[0], ks[1], ks[2]);
  if (octree_h == 0) return OCNN_OK;
  // The first chunk (n == 0) overwrites the rows, later ones add to them
  // (octree_nn.cpp:226 clears the output before the first chunk).
  unsigned long long id = owned_mark ? kColMarkOwned : ++g_col_calls;
  unsigned long long* mark = owned_mark ? owned_mark : nullptr;
  if (!mark) {
    unsigned long long* ring = col_ring();
    OCNN_REQUIRE(ring, OCNN_E_HIP, "no address for the table marks of this device");
    mark = ring + id % kColSlots;
  }
  bool can_invert = !P || ichild != nullptr;
  int chunk_cols = (int)std::max<int64_t>(0,
      std::min<int64_t>(height, ((int64_t)n + 1) * height_col) - (int64_t)n * height_col);
  int chans = (channel + kChanChunk - 1) / kChanChunk;
  // At stride 1 with a tap set that holds the opposite of each of its taps, a row's
  // columns are found the way a column's rows are (tap k one way is the opposite tap
  // the other way), so over the whole range one direction of the check says it all.
  bool one_way = stride == 1 && ks[0] != 2 && n == 0 && chunk_cols == height && height == octree_h;
  if (check_now) {
    dim3 check_grid(blocks_for(std::max(std::max(chunk_cols, octree_h), 1)), one_way ? 1 : 2);
    col_check_kernel<P><<<check_grid, kBlock, 0, s>>>(a, neigh, child, ichild, mark, id, !can_invert);
    OCNN_LAUNCH_OK("col_check");
  }
  if (!P && stride == 1 && a.K == 27 && height == octree_h && ((int64_t)n * height_col) % 4 == 0 &&
      (int64_t)27 * height_col * 4 < (int64_t(1) << 31)) {
    col2octree_tile_kernel<<<dim3(blocks_for(octree_h, kGatherTile), chans), kGatherTile,
        (27 * kGatherTile + 1) * sizeof(float), s>>>(
        (const float*)col, (float*)data, a, neigh, mark, id);
  } else {
    col2octree_kernel<P><<<dim3(blocks_for(octree_h), chans), kBlock, 0, s>>>((const float*)col,
        (float*)data, a, neigh, child, ichild, mark, id);
  }
  OCNN_LAUNCH_OK("col2octree");
  if (chunk_cols > 0) {
    col2octree_atomic_kernel<P><<<dim3(blocks_for(height_col), chans), kBlock, 0, s>>>(
        (const float*)col, (float*)data, a, neigh, child, ichild, mark, id);
    OCNN_LAUNCH_OK("col2octree_atomic");
  }
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

static int run_pad_forward(void* Y, int Hy, int C, const void* X, int Hx, const int* label, float dval,
    const float* fill, int dtype, ocnn_stream_t stream);

int ocnn_pad_forward(void* Y, int Hy, int C, const void* X, int Hx, const int* label, float dval,
    int dtype, ocnn_stream_t stream) {
  return run_pad_forward(Y, Hy, C, X, Hx, label, dval, nullptr, dtype, stream);
}

int ocnn_pad_forward_fill(void* Y, int Hy, int C, const void* X, int Hx, const int* label, const float* fill,
    int dtype, ocnn_stream_t stream) {
  OCNN_REQUIRE(fill, OCNN_E_BADARG, "null pointer");
  return run_pad_forward(Y, Hy, C, X, Hx, label, 0.0f, fill, dtype, stream);
}

static int run_pad_forward(void* Y, int Hy, int C, const void* X, int Hx, const int* label, float dval,
    const float* fill, int dtype, ocnn_stream_t stream) {
  OCNN_REQUIRE(Y && label && (X || Hx == 0), OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(Hy >= 0 && Hx >= 0 && C > 0, OCNN_E_BADARG, "Hy %d Hx %d C %d", Hy, Hx, C);
  if (Hy == 0) return OCNN_OK;
  // the labels of a tile are staged once per workgroup: few workgroups per tile when there
  // are many tiles
  const unsigned tiles = blocks_for(Hy, kPadTile);
  dim3 grid(tiles, std::min<unsigned>(C, std::max(1u, 4096u / tiles)));
  hipStream_t s = as_stream(stream);
  if (dtype == OCNN_F32)
    pad_forward_kernel<float><<<grid, kBlock, 0, s>>>((float*)Y, Hy, C, (const float*)X, Hx, label, dval, fill);
  else if (dtype == OCNN_BF16) {
    // the pad value is rounded to bf16 on the host side of the launch
    uint32_t u;
    memcpy(&u, &dval, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    pad_forward_kernel<uint16_t><<<grid, kBlock, 0, s>>>((uint16_t*)Y, Hy, C, (const uint16_t*)X, Hx,
        label, (uint16_t)(u >> 16), fill);
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
  const unsigned tiles = blocks_for(Hy, kPadTile), chunks = (C + kChanChunk - 1) / kChanChunk;
  dim3 grid(tiles, std::min(chunks, std::max(1u, 2048u / tiles)));
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

int ocnn_col2octree_cached(const void* col, void* data, int channel, int height, int octree_h,
    const int* kernel_size, int stride, const int* neigh, const int* child, const int* ichild,
    int height_col, int n, int dtype, unsigned long long* table_mark_dev, int check_now,
    ocnn_stream_t stream) {
  OCNN_REQUIRE(table_mark_dev, OCNN_E_BADARG, "null table mark");
  OCNN_REQUIRE((reinterpret_cast<uintptr_t>(table_mark_dev) & 7) == 0, OCNN_E_BADARG, "table mark not 8-byte aligned");
  if (child)
    return run_col2octree<true>(col, data, channel, height, octree_h, kernel_size, stride, neigh, child,
        ichild, height_col, n, dtype, as_stream(stream), table_mark_dev, check_now != 0);
  return run_col2octree<false>(col, data, channel, height, octree_h, kernel_size, stride, neigh,
      nullptr, nullptr, height_col, n, dtype, as_stream(stream), table_mark_dev, check_now != 0);
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

int ocnn_octree_max_pool_rows(void* top_rows, int top_pitch, int* mask_rows, const void* btm_rows, int btm_pitch,
    int channel, const void* octree_dev, const void* info, int depth, int dtype, ocnn_stream_t stream) {
  OCNN_REQUIRE(top_rows && btm_rows && octree_dev && info, OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(dtype == OCNN_BF16, OCNN_E_UNSUPPORTED, "row-major activations: bf16");
  const Info* o = as_info(info);
  int e = ocnn_info_check(o);
  if (e) return e;
  OCNN_REQUIRE(depth > 1 && depth <= o->depth, OCNN_E_BADARG, "depth %d not in [2,%d]", depth, o->depth);
  const int pitch = (channel + 15) / 16 * 16;
  OCNN_REQUIRE(channel > 0 && top_pitch >= pitch && btm_pitch >= pitch && top_pitch % 8 == 0 && btm_pitch % 8 == 0,
      OCNN_E_SHAPE, "pitches %d / %d for %d channels", top_pitch, btm_pitch, channel);
  OCNN_REQUIRE(((reinterpret_cast<uintptr_t>(top_rows) | reinterpret_cast<uintptr_t>(btm_rows) |
      reinterpret_cast<uintptr_t>(mask_rows)) & 15) == 0, OCNN_E_BADARG, "rows not 16-byte aligned");
  const int top_h = o->nnum[depth - 1], btm_h = o->nnum[depth];
  const int pieces = pitch / 8;
  const int* child = reinterpret_cast<const int*>(static_cast<const char*>(octree_dev) + o->ptr_dis(OCNN_CHILD, depth - 1));
  const int64_t total = ((int64_t)top_h + 1) * pieces;
  max_pool_rows_kernel<<<blocks_for(total), kBlock, 0, as_stream(stream)>>>((uint16_t*)top_rows, top_pitch, mask_rows,
      (const uint16_t*)btm_rows, btm_pitch, pieces, child, top_h, btm_h);
  OCNN_LAUNCH_OK("max_pool_rows");
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
