// Octree construction on the device: points2octree (Octree::build,
// octree/octree/octree.cpp:74-121) fused with octree_batch (merge_octrees,
// octree/octree/merge_octrees.cpp:114-198) for a whole batch of point clouds.
//
// Design.  The reference sorts (key, index) pairs per cloud on one CPU core,
// then walks the levels bottom-up, then merges the per-cloud blobs on the host.
// Here ONE sort handles every cloud of the batch: the sort key is
// (cloud << 3*depth | morton), so the sorted order is already the node order of
// the merged batch octree, and child links are global ranks -- exactly what
// merge_octrees produces by offsetting per-cloud links.  A small octree is bound
// by the number of dependent launches and memory round trips, so the work is
// packed into few launches with short dependency chains:
//
//   plan:  init (control words, cloud table)
//          keys + the digit histograms of every sort pass
//          one launch per sort pass: stable LSD radix sort; each tile publishes
//            its digit counts and looks back over the tiles before it for its
//            global offsets (no separate scan launches)
//          ONE scan for every level at once: element i starts a new node at level
//            d iff it differs from element i-1 above bit 3*(depth-d); the
//            per-level counts travel as 16-bit fields of four 64-bit words
//          [the level sizes reach the host through pinned memory that the scan's last
//           workgroup writes and the host polls: the caller must size the blob]
//   emit:  one launch writes header, keys, children, split labels and full-layer
//            neighbour tables of every level (the children of a sibling group
//            are found by position, nothing is scattered) and, in workgroups of
//            their own, the signal of the finest level (tiles of 1024 nodes staged
//            in LDS, full rows out, zeros for empty nodes);
//          one launch per sparse level for the neighbour tables (each needs the
//            level above).
#include "build_adaptive.h"
#include "octree_kernels.h"

#include <atomic>
#include <chrono>
#include <type_traits>
#include <map>
#include <mutex>
#include <vector>

namespace ocnn {
namespace {

struct CloudDesc {
  const float* xyz;
  const float* normal;
  const float* feature;
  const float* label;
  int offset, count;  // position of the cloud's points in the concatenated order
};

constexpr int kMaxLevels = 17;
constexpr int kMergedNoNeigh = 2;   // ocnn_build_params::merged: batch layout, no neighbour tables (first stage of a two-stage build)
constexpr int kMaxPasses = 8;
constexpr uint32_t kFlagSum = 1u << 30;    // status word: published (the count is in the low bits)
constexpr uint32_t kCountMask = (1u << 30) - 1;

struct Control {                 // device-resident, zeroed by init_kernel
  int nne[kMaxLevels];           // non-empty nodes per depth (valid for depth >= full_layer)
  int error;                     // a bounded wait ran out (never expected)
  unsigned ticket[kMaxPasses + 1];  // tile tickets: one per sort pass, the last for the level scan
  unsigned done;                 // workgroups of the level scan that have finished
  int pad[4];
};
static_assert(sizeof(Control) == 128, "Control layout");

// What the host needs before it can size the blob, in pinned host memory: the workgroup of the
// level scan that finishes last writes it there, `seq` last (the host polls that word instead of
// waiting for the stream, which costs a device-to-host copy and the wake-up of a blocked thread).
struct HostCounts {
  int nne[kMaxLevels];
  int error;
  int seq;
};

struct BuildGeom {
  int depth, full_layer, n_clouds;
  int passes, bits;            // sort: `passes` digits of `bits` bits each
  int64_t n_points;
  float bbmin[3];
  float mul;                   // 2^depth / bbox width, computed on the host in fp32
};

// ---- 0. control words and the cloud table ---------------------------------------------
constexpr int kArgClouds = 48;
struct CloudChunk { CloudDesc c[kArgClouds]; };

__global__ void init_kernel(uint32_t* __restrict__ zero, int64_t zero_words, CloudDesc* __restrict__ clouds,
    CloudChunk chunk, int first, int count) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) clouds[first + i] = chunk.c[i];
  const int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (; i < zero_words; i += step) zero[i] = 0;
}

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

// Sort keys and, on the way, the digit histogram of every sort pass (the passes
// themselves then need no counting launch).  Neighbouring points mostly share their high
// digits: a wavefront whose lanes all hold the same digit adds its count once instead of
// serialising 64 LDS atomics on one address.
constexpr int kKeyItems = 4;   // points per thread: 250 k points then make 244 workgroups (with 8, half the CUs had none)
constexpr int kKeyGrid = 512;   // workgroups at most: each adds its histograms to the global ones once
constexpr int kHistCopies = 16; // global histogram copies: atomics on one address are served one by one
__global__ __launch_bounds__(kBlock) void keygen_kernel(uint64_t* __restrict__ key, uint32_t* __restrict__ val,
    const CloudDesc* __restrict__ clouds, int* __restrict__ hist, BuildGeom g) {
  __shared__ int h[kMaxPasses][256];
  __shared__ int s_off[kBlock + 1];     // offsets of the clouds a chunk touches
  for (int p = 0; p < g.passes; ++p) h[p][threadIdx.x] = 0;
  const uint64_t m = (1ull << g.depth) - 1;
  const uint32_t dmask = (1u << g.bits) - 1;
  const int lane = threadIdx.x & 63;
  const int64_t chunks = (g.n_points + kBlock * kKeyItems - 1) / (kBlock * kKeyItems);
  for (int64_t chunk = blockIdx.x; chunk < chunks; chunk += gridDim.x) {
    const int64_t base = chunk * (kBlock * kKeyItems);
    const int64_t last = min(base + kBlock * kKeyItems, g.n_points) - 1;
    // clouds of the first and last point of the chunk; the table between them goes to LDS
    const int b_lo = find_cloud(clouds, g.n_clouds, base);
    const int b_hi = find_cloud(clouds, g.n_clouds, last);
    const int span = min(b_hi - b_lo + 1, kBlock);
    __syncthreads();
    if ((int)threadIdx.x < span) s_off[threadIdx.x] = clouds[b_lo + threadIdx.x].offset;
    __syncthreads();
    int cloud[kKeyItems];
    float xyz[kKeyItems][3];
#pragma unroll
    for (int q = 0; q < kKeyItems; ++q) {
      const int64_t i = base + q * kBlock + threadIdx.x;
      cloud[q] = 0;
      xyz[q][0] = xyz[q][1] = xyz[q][2] = 0.0f;
      if (i < g.n_points) {
        int b = b_lo;
        if (b_hi - b_lo < kBlock) {  // last cloud of the span with offset <= i
          int lo = 0, hi = span - 1;
          while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (s_off[mid] <= i) lo = mid; else hi = mid - 1;
          }
          b += lo;
        } else {
          b = find_cloud(clouds, g.n_clouds, i);
        }
        cloud[q] = b;
        const float* p = clouds[b].xyz + 3 * (i - clouds[b].offset);
        xyz[q][0] = p[0]; xyz[q][1] = p[1]; xyz[q][2] = p[2];
      }
    }
#pragma unroll
    for (int q = 0; q < kKeyItems; ++q) {
      const int64_t i = base + q * kBlock + threadIdx.x;
      const bool valid = i < g.n_points;
      uint64_t k = 0;
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        // float -> unsigned truncation as static_cast<uintk> (octree.cpp:184); only the low
        // `depth` bits are interleaved (octree_nn.cpp:551-560)
        uint32_t c = (uint32_t)scale_coord(xyz[q][j], g.bbmin[j], g.mul);
        k |= spread3(c & m) << (2 - j);
      }
      k |= (uint64_t)cloud[q] << (3 * g.depth);
      if (valid) {
        key[i] = k;
        val[i] = (uint32_t)i;
      }
      const uint64_t active = __ballot(valid);
      if (active != 0) {
        const int leader = __ffsll((long long)active) - 1;
        for (int ps = 0; ps < g.passes; ++ps) {
          const int d = (int)((uint32_t)(k >> (ps * g.bits)) & dmask);
          const int d0 = __shfl(d, leader, 64);
          if (__ballot(valid && d != d0) == 0) {
            if (lane == leader) atomicAdd(&h[ps][d0], __popcll(active));
          } else if (valid) {
            atomicAdd(&h[ps][d], 1);
          }
        }
      }
    }
  }
  __syncthreads();
  for (int p = 0; p < g.passes; ++p) {
    const int c = h[p][threadIdx.x];
    if (c) atomicAdd(&hist[((blockIdx.x % kHistCopies) * kMaxPasses + p) * 256 + threadIdx.x], c);
  }
}

// ---- 2. radix sort (LSD, stable), one launch per digit ------------------------------------
__device__ inline uint32_t status_load(const uint32_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline void status_store(uint32_t* p, uint32_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Sum of the counts of tiles 0 .. tile-1 for one scan lane (a digit / a level), in two levels:
// tiles form groups of 32.  Every tile publishes its count; the last tile of a group adds the
// group up and publishes the group's count; a tile then needs the counts of the groups before
// its own and of the tiles before it inside its group.  All tiles start together, so a chain
// that walks back tile by tile would take as many round trips as there are tiles; here it is
// two hand-offs whatever the number of tiles.
//
// A tile only ever waits for tiles before it.  First try: tile = workgroup index, which ends
// as long as the device starts workgroups in index order (a thousand same-address ticket
// atomics cost more than the pass itself).  Every wait is bounded; if one ever runs out, the
// host repeats the plan with tile ids drawn from a ticket counter, where every earlier tile
// is running by construction.
constexpr int kGroupTiles = 32;

// sum of `count` (<= 32) status words of one scan lane from tile / group `first` on, waiting
// until all of them are published; `stride` = scan lanes per tile (the words of one tile are
// contiguous, so a workgroup reads and writes whole rows).  All words are requested together.
__device__ inline int wait_sum(const uint32_t* __restrict__ status, int stride, int lane_id, int first, int count,
    int spin_limit, int* __restrict__ error) {
  const uint32_t* p = status + (int64_t)first * stride + lane_id;
  int spins = 0;
  for (;;) {
    uint32_t s[kGroupTiles];
#pragma unroll
    for (int j = 0; j < kGroupTiles; ++j) s[j] = j < count ? status_load(p + (int64_t)j * stride) : kFlagSum;
    uint32_t all = kFlagSum;
    int sum = 0;
#pragma unroll
    for (int j = 0; j < kGroupTiles; ++j) { all &= s[j]; sum += (int)(s[j] & kCountMask); }
    if (all & kFlagSum) return sum;
    if (++spins > spin_limit) {
      __hip_atomic_store(error, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      return sum;
    }
    __builtin_amdgcn_s_sleep(1);
  }
}

// publish the count of (tile, lane)
__device__ inline void tile_publish(uint32_t* __restrict__ tile_status, int stride, int lane_id, int tile, int cnt) {
  status_store(&tile_status[(int64_t)tile * stride + lane_id], (uint32_t)cnt | kFlagSum);
}
// counts of all tiles before `tile` (after tile_publish)
__device__ inline int tile_prefix(const uint32_t* __restrict__ tile_status, uint32_t* __restrict__ group_status,
    int stride, int lane_id, int tile, int cnt, int spin_limit, int* __restrict__ error) {
  const int g = tile / kGroupTiles, j = tile % kGroupTiles;
  const int within = j > 0 ? wait_sum(tile_status, stride, lane_id, g * kGroupTiles, j, spin_limit, error) : 0;
  if (j == kGroupTiles - 1) status_store(&group_status[(int64_t)g * stride + lane_id], (uint32_t)(within + cnt) | kFlagSum);
  int before = within;
  for (int g0 = 0; g0 < g; g0 += kGroupTiles)
    before += wait_sum(group_status, stride, lane_id, g0, min(kGroupTiles, g - g0), spin_limit, error);
  return before;
}

// A tile is 256 * ITEMS consecutive elements; wavefront w owns the w-th quarter and ranks it
// 64 elements at a time: the rank among equal digits inside a round comes from ballots (one
// per digit bit), across rounds from the wavefront's own running counters in LDS, so the
// order (wavefront, round, lane) equals the input order and the sort is stable.  The tile is
// then reordered in LDS so that equal digits leave as contiguous runs.
template <int ITEMS, bool TICKETS>
__global__ __launch_bounds__(kBlock) void sort_pass_kernel(const uint64_t* __restrict__ key_in,
    const uint32_t* __restrict__ val_in, uint64_t* __restrict__ key_out, uint32_t* __restrict__ val_out, int n,
    int shift, int bits, const int* __restrict__ hist, uint32_t* __restrict__ status,
    uint32_t* __restrict__ group_status, Control* __restrict__ ctl, int pass, int spin_limit) {
  constexpr int kTile = kBlock * ITEMS;
  __shared__ int s_tile;
  __shared__ int wave_cnt[kBlock / 64][256];
  __shared__ int s_gbase[256];
  __shared__ uint64_t s_key[kTile];
  __shared__ uint32_t s_val[kTile];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (TICKETS) {
    if (tid == 0) s_tile = (int)atomicAdd(&ctl->ticket[pass], 1u);
    __syncthreads();
  }
  if (spin_limit < 0 && tid == 0 && blockIdx.x == 0) ctl->error = 1;  // a forced failure (tests)
  const int tile = TICKETS ? s_tile : (int)blockIdx.x;
  const int tile_n = min(kTile, n - tile * kTile);
  const int wbase = tile * kTile + wave * 64 * ITEMS;
  const uint32_t dmask = (1u << bits) - 1;

  uint64_t k[ITEMS];
  uint32_t v[ITEMS];
  int loc[ITEMS];
#pragma unroll
  for (int q = 0; q < ITEMS; ++q) {
    const int i = wbase + q * 64 + lane;
    k[q] = i < n ? key_in[i] : 0;
    v[q] = i < n ? val_in[i] : 0;
  }
  int digit_total = 0;
#pragma unroll
  for (int c = 0; c < kHistCopies; ++c) digit_total += hist[c * kMaxPasses * 256 + tid];
#pragma unroll
  for (int w = 0; w < kBlock / 64; ++w) wave_cnt[w][tid] = 0;
  int unused;
  const int digit_base = block_exclusive_scan(digit_total, &unused);  // elements with a smaller digit
  // Rank of an element among the lanes of its round with the same digit: from ballots.  The
  // first lane of each digit group then adds the group to the wavefront's counter; the LDS
  // unit applies the atomics of a wavefront in program order, so the returned values are the
  // counts of the earlier rounds and the rounds need not wait for one another.
  int leader[ITEMS], earlier[ITEMS];
#pragma unroll
  for (int q = 0; q < ITEMS; ++q) {
    const bool valid = wbase + q * 64 + lane < n;
    const int d = (int)((uint32_t)(k[q] >> shift) & dmask);
    uint64_t peers = __ballot(valid);
    for (int b = 0; b < bits; ++b) {
      const uint64_t m = __ballot((d >> b) & 1);
      peers &= ((d >> b) & 1) ? m : ~m;
    }
    loc[q] = __popcll(peers & ((1ull << lane) - 1));
    leader[q] = valid ? __ffsll((long long)peers) - 1 : lane;
    earlier[q] = 0;
    if (valid && leader[q] == lane) earlier[q] = atomicAdd(&wave_cnt[wave][d], __popcll(peers));
  }
#pragma unroll
  for (int q = 0; q < ITEMS; ++q) loc[q] += __shfl(earlier[q], leader[q], 64);
  __syncthreads();
  // thread = digit: count of the tile (published at once: later tiles wait for it), position of
  // the digit's run inside the tile, offsets of the wavefronts inside the run
  int cnt = 0, local;
  {
    int c[kBlock / 64];
#pragma unroll
    for (int w = 0; w < kBlock / 64; ++w) { c[w] = wave_cnt[w][tid]; cnt += c[w]; }
    tile_publish(status, 256, tid, tile, cnt);
    local = block_exclusive_scan(cnt, &unused);
    int run = local;
#pragma unroll
    for (int w = 0; w < kBlock / 64; ++w) { wave_cnt[w][tid] = run; run += c[w]; }
  }
  __syncthreads();
  // reorder the tile in LDS (this needs nothing from other tiles and frees the registers)
#pragma unroll
  for (int q = 0; q < ITEMS; ++q) {
    if (wbase + q * 64 + lane < n) {
      const int d = (int)((uint32_t)(k[q] >> shift) & dmask);
      const int p = wave_cnt[wave][d] + loc[q];
      s_key[p] = k[q];
      s_val[p] = v[q];
    }
  }
  s_gbase[tid] = digit_base - local + tile_prefix(status, group_status, 256, tid, tile, cnt, spin_limit, &ctl->error);
  __syncthreads();
#pragma unroll
  for (int q = 0; q < ITEMS; ++q) {
    const int t = q * kBlock + tid;
    if (t < tile_n) {
      const uint64_t kk = s_key[t];
      const int pos = s_gbase[(uint32_t)(kk >> shift) & dmask] + t;
      key_out[pos] = kk;
      val_out[pos] = s_val[t];
    }
  }
}

// ---- 3. all levels in one scan -------------------------------------------------------------
// Element i of the sorted keys is the first point of a new node at level d iff it differs
// from element i-1 in a bit at or above 3*(depth-d).  Its `first level` a (relative to the
// full layer) says it heads a node at every level >= a.  The number of heads at level
// full_layer + f up to an element is carried in field f (16 bits) of four 64-bit words, so
// one scan serves every level.
// (named members, not an array: a run-time choice between array elements would be turned into
// indexed addressing and move the whole struct out of the registers)
struct Packed4 {
  uint64_t w0, w1, w2, w3;
};
template <int N, class F>
__device__ inline void static_for(F&& f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}
__device__ inline uint64_t heads_word(int s) {  // fields >= s of one word set to 1
  constexpr uint64_t kOnes = 0x0001000100010001ull;
  return s <= 0 ? kOnes : (s >= 4 ? 0ull : kOnes << (16 * s));
}
__device__ inline Packed4 heads_from(int a) {  // one count in every field f >= a
  return Packed4{heads_word(a), heads_word(a - 4), heads_word(a - 8), heads_word(a - 12)};
}
__device__ inline void add_to(Packed4& a, const Packed4& b) {
  a.w0 += b.w0; a.w1 += b.w1; a.w2 += b.w2; a.w3 += b.w3;
}
__device__ inline int field_of(const Packed4& p, int f) {
  const uint64_t lo = f < 4 ? p.w0 : p.w1, hi = f < 12 ? p.w2 : p.w3;
  const uint64_t w = f < 8 ? lo : hi;
  return (int)((w >> (16 * (f & 3))) & 0xffff);
}
__device__ inline uint64_t wave_inclusive_scan_u64(uint64_t v) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const uint64_t t = __shfl_up((unsigned long long)v, d, 64);
    if (lane >= d) v += t;
  }
  return v;
}
__device__ inline Packed4 block_exclusive_scan_p4(Packed4 v, Packed4* block_total) {
  __shared__ uint64_t wave_sum[kBlock / 64][4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const Packed4 inc = {wave_inclusive_scan_u64(v.w0), wave_inclusive_scan_u64(v.w1), wave_inclusive_scan_u64(v.w2),
      wave_inclusive_scan_u64(v.w3)};
  if (lane == 63) {
    wave_sum[wave][0] = inc.w0; wave_sum[wave][1] = inc.w1; wave_sum[wave][2] = inc.w2; wave_sum[wave][3] = inc.w3;
  }
  __syncthreads();
  uint64_t base[4] = {0, 0, 0, 0}, tot[4] = {0, 0, 0, 0};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
#pragma unroll
    for (int w = 0; w < kBlock / 64; ++w) {
      const uint64_t s = wave_sum[w][j];
      if (w < wave) base[j] += s;
      tot[j] += s;
    }
  }
  __syncthreads();
  *block_total = Packed4{tot[0], tot[1], tot[2], tot[3]};
  return Packed4{base[0] + inc.w0 - v.w0, base[1] + inc.w1 - v.w1, base[2] + inc.w2 - v.w2, base[3] + inc.w3 - v.w3};
}

struct LevelOut {
  uint64_t* list[kMaxLevels];   // list[d][r]: key (cloud << 3d | morton) of the r-th non-empty node of level d
  int* first[kMaxLevels];       // first[d][r]: rank at level d+1 of that node's first child; [nne_d] = nne_{d+1}
  int* ustart;                  // first sorted point of each leaf; [n_leaf] = n_points
};

constexpr int kLevelItems = 4;   // keys per thread (8 left half the CUs without a workgroup on a 250 k cloud)
constexpr int kLevelTile = kBlock * kLevelItems;

template <bool TICKETS>
__global__ __launch_bounds__(kBlock) void levels_kernel(const uint64_t* __restrict__ key, int n, int depth,
    int full_layer, LevelOut out, uint32_t* __restrict__ status, uint32_t* __restrict__ group_status,
    Control* __restrict__ ctl, int spin_limit, HostCounts* __restrict__ host, int seq) {
  __shared__ int s_tile;
  __shared__ int s_before[16];
  const int tid = threadIdx.x;
  if (TICKETS) {
    if (tid == 0) s_tile = (int)atomicAdd(&ctl->ticket[kMaxPasses], 1u);
    __syncthreads();
  }
  const int tile = TICKETS ? s_tile : (int)blockIdx.x;
  const int L = depth - full_layer + 1;  // levels full_layer .. depth
  const int i0 = tile * kLevelTile + tid * kLevelItems;

  uint64_t k[kLevelItems];
  int a[kLevelItems];
  const uint64_t before_first = i0 > 0 && i0 - 1 < n ? key[i0 - 1] : 0;
  static_for<kLevelItems>([&](auto J) {   // compile-time indices keep k[] and a[] in registers
    constexpr int j = decltype(J)::value;
    k[j] = i0 + j < n ? key[i0 + j] : 0;
  });
  Packed4 mine = {0, 0, 0, 0};
  static_for<kLevelItems>([&](auto J) {
    constexpr int j = decltype(J)::value;
    const int i = i0 + j;
    a[j] = 64;  // heads nothing (also: beyond the end)
    if (i < n) {
      if (i == 0) a[j] = 0;
      else {
        uint64_t prev = before_first;
        if constexpr (j > 0) prev = k[j - 1];
        const uint64_t x = k[j] ^ prev;
        if (x != 0) {
          const int t = (63 - __clzll((long long)x)) / 3;   // differs at level depth - t
          a[j] = max(0, depth - t - full_layer);
        }
      }
      if (a[j] < L) add_to(mine, heads_from(a[j]));
    }
  });
  Packed4 total;
  const Packed4 run = block_exclusive_scan_p4(mine, &total);  // heads of this tile before this thread
  if (tid < 16) {
    tile_publish(status, 16, tid, tile, field_of(total, tid));
    s_before[tid] = tile_prefix(status, group_status, 16, tid, tile, field_of(total, tid), spin_limit, &ctl->error);
  }
  __syncthreads();
  // level by level (uniform over the workgroup, so the output pointers are scalars): b_* =
  // heads before this thread at level f / f+1, c_* = the same among its own elements
  const bool has_last = i0 <= n - 1 && n - 1 < i0 + kLevelItems;
  for (int f = 0; f < L; ++f) {
    const int d = full_layer + f;
    const int shift = 3 * (depth - d);
    const int b0 = s_before[f] + field_of(run, f);
    const int b1 = f + 1 < L ? s_before[f + 1] + field_of(run, f + 1) : 0;
    uint64_t* __restrict__ list = out.list[d];
    int* __restrict__ first = out.first[d];
    int c0 = 0, c1 = 0;
    static_for<kLevelItems>([&](auto J) {   // compile-time indices keep k[] and a[] in registers
      constexpr int j = decltype(J)::value;
      c1 += a[j] <= f + 1 ? 1 : 0;
      if (a[j] <= f) {
        const int r = b0 + c0;
        ++c0;
        list[r] = k[j] >> shift;
        if (f + 1 < L) first[r] = b1 + c1 - 1;
        else out.ustart[r] = i0 + j;
      }
    });
    if (has_last) {
      status_store(reinterpret_cast<uint32_t*>(&ctl->nne[d]), (uint32_t)(b0 + c0));
      if (f + 1 < L) first[b0 + c0] = b1 + c1;
      else out.ustart[b0 + c0] = n;
    }
  }
  // the workgroup that finishes last hands the counts (and whether any wait ran out, in this
  // launch or in a sort pass before it) to the host
  // (counts and error word are written and read with device-scope atomic accesses, which do not
  // linger in an XCD's L2; the wait below is for their acknowledgement.  A device-wide fence
  // here would have every workgroup write back its XCD's whole L2.)
  __shared__ int s_last_one;
  if (has_last) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  if (tid == 0) s_last_one = atomicAdd(&ctl->done, 1u) == gridDim.x - 1;
  __syncthreads();
  if (s_last_one && tid < 64) {   // one wavefront: a lane per word, then the sequence number
    static_assert(kMaxLevels + 1 <= 64, "one lane per word");
    const int* src = tid < kMaxLevels ? &ctl->nne[tid] : &ctl->error;
    int* dst = tid < kMaxLevels ? &host->nne[tid] : &host->error;
    if (tid <= kMaxLevels)
      __hip_atomic_store(dst, __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT),
          __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    __threadfence_system();
    if (tid == 0) __hip_atomic_store(&host->seq, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

// ---- 4. emit -------------------------------------------------------------------------------
__device__ inline uint64_t out_key(uint64_t morton, int d, int cloud, int key2xyz) {
  // raw Morton key, or packed (x, y, z) 16-bit fields (Octree::key_to_xyz, octree.cpp:1137-1156);
  // the cloud index goes to the top 16 bits as merge_octrees does (merge_octrees.cpp:126-131)
  uint64_t k = morton;
  if (key2xyz) {
    uint64_t m = d >= 16 ? 0xffffull : ((1ull << d) - 1);
    k = (compact3(morton >> 2) & m) | ((compact3(morton >> 1) & m) << 16) | ((compact3(morton) & m) << 32);
  }
  return (k & 0x0000ffffffffffffull) | ((uint64_t)(cloud & 0xffff) << 48);
}

struct SignalGeom {
  int depth, nnum_d;      // nnum_d = node count of the finest level (row length)
  int ch_feature, channels, has_label, has_dis, save_pts;
  float bbmin[3], mul;
};

// Signal of one non-empty leaf: its points are visited in ascending original index (the
// sort is stable), so every sum is taken in the reference's order (octree.cpp:312-452).
// All float operations are individually rounded.
__device__ inline void leaf_signal(float* __restrict__ feature, float* __restrict__ label_out, int node,
    int cloud, int s0, int s1, const uint32_t* __restrict__ sorted_idx, const CloudDesc* __restrict__ clouds,
    const SignalGeom& g) {
  const CloudDesc cd = clouds[cloud];
  const int64_t H = g.nnum_d;
  float* out = feature + node;  // channel c lives at out[c * H]
  // one pass over the points: every attribute of a point is requested together
  constexpr int kRegFeatures = 4;
  const int F = cd.feature ? g.ch_feature : 0;
  const bool need_pt = g.has_dis || g.save_pts;
  float acc[3] = {0.0f, 0.0f, 0.0f}, avg_pt[3] = {0.0f, 0.0f, 0.0f}, facc[kRegFeatures];
#pragma unroll
  for (int c = 0; c < kRegFeatures; ++c) facc[c] = 0.0f;
  // two points at a time: all their loads are requested before the first sum, the sums
  // themselves stay in ascending point order
  constexpr int kChunk = 2;
  for (int i0 = s0; i0 < s1; i0 += kChunk) {
    int64_t idx[kChunk];
    float nv[kChunk][3], pv[kChunk][3], fv[kChunk][kRegFeatures];
#pragma unroll
    for (int u = 0; u < kChunk; ++u) idx[u] = i0 + u < s1 ? (int64_t)(sorted_idx[i0 + u] - cd.offset) : -1;
#pragma unroll
    for (int u = 0; u < kChunk; ++u) {
      if (idx[u] < 0) continue;
      if (cd.normal) {
        const float* q = cd.normal + 3 * idx[u];
        for (int c = 0; c < 3; ++c) nv[u][c] = q[c];
      }
      if (need_pt) {
        const float* q = cd.xyz + 3 * idx[u];
        for (int c = 0; c < 3; ++c) pv[u][c] = q[c];
      }
      const float* q = cd.feature + F * idx[u];
#pragma unroll
      for (int c = 0; c < kRegFeatures; ++c)
        if (c < F) fv[u][c] = q[c];
    }
#pragma unroll
    for (int u = 0; u < kChunk; ++u) {
      if (idx[u] < 0) continue;
      if (cd.normal)
        for (int c = 0; c < 3; ++c) acc[c] = __fadd_rn(acc[c], nv[u][c]);
      if (need_pt)
        for (int c = 0; c < 3; ++c) avg_pt[c] = __fadd_rn(avg_pt[c], scale_coord(pv[u][c], g.bbmin[c], g.mul));
#pragma unroll
      for (int c = 0; c < kRegFeatures; ++c)
        if (c < F) facc[c] = __fadd_rn(facc[c], fv[u][c]);
    }
  }
  int ch = 0;
  float nrm[3] = {0.0f, 0.0f, 0.0f};
  if (cd.normal) {
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
  if (need_pt) {
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
  if (F > 0) {
#pragma unroll
    for (int c = 0; c < kRegFeatures; ++c)
      if (c < F) out[(ch + c) * H] = div_rn(facc[c], count);
    for (int c = kRegFeatures; c < F; ++c) {   // channels beyond the register budget: one more pass each
      float sum = 0.0f;
      for (int i = s0; i < s1; ++i)
        sum = __fadd_rn(sum, cd.feature[(int64_t)F * (sorted_idx[i] - cd.offset) + c]);
      out[(ch + c) * H] = div_rn(sum, count);
    }
    ch += F;
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

// The emit launch is cut into segments of whole workgroups; each segment is one kind of
// work on one level.
enum SegKind { kSegHeader = 0, kSegFull = 1, kSegFullNeigh = 2, kSegSparse = 3, kSegNeighSearch = 4, kSegLeafSignal = 5 };
// sparse levels with at most this many sibling groups get their neighbour table inside the emit
// launch (by key search); larger ones from the table of the level above, one launch each
constexpr int kSearchGroups = 8192;   // measured on the depth-9 scene: 2048 and 32768 are 2-4 % slower, 100000 18 %
constexpr int kSearchPerWave = 4;
constexpr int kMaxSeg = 56;
struct HeaderArg { uint32_t w[OCNN_HEADER_BYTES / 4]; };

struct EmitArgs {
  HeaderArg hdr;
  int depth, full_layer, n_clouds, key2xyz, key_channel;
  int n_seg;
  int seg_begin[kMaxSeg + 1];          // first workgroup of each segment
  unsigned char seg_kind[kMaxSeg], seg_level[kMaxSeg];
  int nnum[kMaxLevels], nne[kMaxLevels];
  int64_t off_key[kMaxLevels], off_child[kMaxLevels], off_split[kMaxLevels], off_neigh[kMaxLevels];
  int64_t off_feature, off_label;      // of the finest level; -1: absent
  const uint64_t* list[kMaxLevels];
  const int* first[kMaxLevels];
  const int* ustart;
  const uint32_t* sorted_idx;
  const CloudDesc* clouds;
  SignalGeom sg;
};
static_assert(sizeof(EmitArgs) <= 3800, "kernel arguments must stay below 4 KiB");

// Signal of the finest level for a tile of kSignalTile consecutive nodes.  The non-empty nodes
// of the tile are consecutive leaves (ranks grow with the node index), so threads 0 .. count-1
// take one leaf each -- dense wavefronts for the point gathers, where one thread per node keeps
// one lane in seven busy at depth 9 -- and leave the result in a compact LDS table (one column
// per leaf, kBlock leaves a round; a tile with more leaves takes more rounds).  The rows are then
// written out in full: every node looks up its leaf (or writes zeros, label -1), so every row of
// the block is written exactly once.  Which leaf sits in which node is read off the level lists
// (node 8 p + octant for the leaves first[p] .. first[p + 1] of the p-th sibling group), not off
// the child links: the tile waits for no other part of the blob and runs inside the launch that
// writes those.  Needs channels <= kSignalStage.  LDS per tile: 1 KiB per channel + 8-10 KiB --
// the launch is bound by how many workgroups are resident, not by bytes.
// (Tried and dropped: an LDS image of the tile's full rows, 4 KiB per channel: five workgroups
// per CU; tiles of 512 nodes, 3-5 % slower; one thread per non-empty leaf writing a compact
// table that a second launch expands into the rows, 15 % slower on eight scenes.)
constexpr int kSignalTile = 1024, kSignalStage = 8;
constexpr int kSignalRounds = kSignalTile / kBlock;
__host__ __device__ inline size_t signal_lds_bytes(int channels, bool has_label, bool batch) {
  return sizeof(float) * kBlock * (size_t)(channels + (has_label ? 1 : 0)) + sizeof(int) * (kSignalTile + 2) +
      sizeof(int) * (kSignalRounds + 2) + sizeof(unsigned short) * kSignalTile * (batch ? 2 : 1);
}
__device__ inline void leaf_signal_tile(char* __restrict__ blob, const EmitArgs& a, int block, unsigned char* s_raw) {
  const SignalGeom& g = a.sg;
  float* feature = a.off_feature >= 0 ? reinterpret_cast<float*>(blob + a.off_feature) : nullptr;
  float* label = a.off_label >= 0 ? reinterpret_cast<float*>(blob + a.off_label) : nullptr;
  const bool batch = a.n_clouds > 1;
  // [channels (+ label)][kBlock] values of a round's leaves; per leaf its first point (one more
  // entry closes the last leaf); the node of every kBlock-th leaf; per node its leaf (0xffff:
  // none); per leaf its cloud (batches only)
  float* s_val = reinterpret_cast<float*>(s_raw);
  float* s_lab = s_val + (size_t)g.channels * kBlock;
  int* s_start = reinterpret_cast<int*>(s_lab + (label ? kBlock : 0));
  int* s_bound = s_start + kSignalTile + 2;
  unsigned short* s_leaf = reinterpret_cast<unsigned short*>(s_bound + kSignalRounds + 2);
  unsigned short* s_cloud = s_leaf + kSignalTile;
  const int tid = threadIdx.x;
  const int node0 = block * kSignalTile;
  const int rows = min(kSignalTile, g.nnum_d - node0);
  const int p0 = node0 >> 3, n_groups = rows >> 3;          // a level holds whole sibling groups
  const int* __restrict__ first = a.first[g.depth - 1];
  const uint64_t* __restrict__ leaf_key = a.list[g.depth];
  const int j0 = first[p0], count = first[p0 + n_groups] - j0;
  for (int t = tid; t < n_groups; t += kBlock) {
    const int c0 = first[p0 + t], c1 = first[p0 + t + 1];
    int oct[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      oct[u] = 8;
      if (c0 + u < c1) {
        const uint64_t lk = leaf_key[c0 + u];
        oct[u] = (int)(lk & 7);
        const int l = c0 + u - j0;
        if (batch) s_cloud[l] = (unsigned short)(lk >> (3 * g.depth));
        if ((l & (kBlock - 1)) == 0) s_bound[l / kBlock] = t * 8 + oct[u];
      }
    }
#pragma unroll
    for (int o = 0; o < 8; ++o) {
      int l = 0xffff;
#pragma unroll
      for (int u = 0; u < 8; ++u) l = oct[u] == o ? c0 + u - j0 : l;
      s_leaf[t * 8 + o] = (unsigned short)l;
    }
  }
  // the leaves' point ranges, requested with the keys above: a leaf then starts with its points'
  // indices instead of with one more trip to memory
  for (int t = tid; t <= count; t += kBlock) s_start[t] = a.ustart[j0 + t];
  __syncthreads();
  SignalGeom lg = g;
  lg.nnum_d = kBlock;   // row length of the LDS table
  for (int r0 = 0; r0 == 0 || r0 < count; r0 += kBlock) {
    const int t = r0 + tid;
    if (label) s_lab[tid] = -1.0f;
    if (t < count)
      leaf_signal(s_val, label ? s_lab : nullptr, tid, batch ? (int)s_cloud[t] : 0, s_start[t], s_start[t + 1],
          a.sorted_idx, a.clouds, lg);
    __syncthreads();
    // nodes of this round: from the node of its first leaf (the tile's first node in round 0) up to
    // the node of the next round's first leaf (the end of the tile after the last round)
    const int n_lo = r0 == 0 ? 0 : s_bound[r0 / kBlock];
    const int n_hi = r0 + kBlock < count ? s_bound[r0 / kBlock + 1] : rows;
    for (int r = n_lo + tid; r < n_hi; r += kBlock) {
      const int l = (int)s_leaf[r] - r0;          // 0xffff - r0 >= kBlock: an empty node
      const bool leaf = l < kBlock;
      for (int ch = 0; ch < g.channels; ++ch)
        feature[(int64_t)ch * g.nnum_d + node0 + r] = leaf ? s_val[ch * kBlock + l] : 0.0f;
      if (label) label[node0 + r] = leaf ? s_lab[l] : -1.0f;
    }
    if (r0 + kBlock < count) __syncthreads();     // the table is reused
  }
}

// a sparse segment stages the parent key of each of its kBlock sibling groups and the child links
constexpr size_t kEmitLdsBytes = (size_t)kBlock * (sizeof(uint64_t) + 8 * sizeof(int));

__global__ __launch_bounds__(kBlock, 8) void emit_kernel(char* __restrict__ blob, const EmitArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char s_raw[];   // max(kEmitLdsBytes, a signal tile)
  uint64_t* s_parent = reinterpret_cast<uint64_t*>(s_raw);
  int* s_child = reinterpret_cast<int*>(s_raw + sizeof(uint64_t) * kBlock);
  int seg = 0;
  while (seg + 1 < a.n_seg && (int)blockIdx.x >= a.seg_begin[seg + 1]) ++seg;
  const int kind = a.seg_kind[seg], d = a.seg_level[seg];
  const int block = blockIdx.x - a.seg_begin[seg];
  const int tid = threadIdx.x;

  if (kind == kSegLeafSignal) {
    leaf_signal_tile(blob, a, block, s_raw);
    return;
  }

  if (kind == kSegHeader) {
    // header (the tail of the 720-byte block is padding, zero); depth 0 holds no neighbour table
    uint32_t* dst = reinterpret_cast<uint32_t*>(blob);
    for (int i = tid; i < OCNN_HEADER_BYTES / 4; i += kBlock) dst[i] = a.hdr.w[i];
    if (a.off_neigh[0] >= 0) {
      int* n0 = reinterpret_cast<int*>(blob + a.off_neigh[0]);
      for (int i = tid; i < a.nnum[0] * 8; i += kBlock) n0[i] = 0;
    }
    return;
  }
  if (kind == kSegFullNeigh) {  // closed form (octree_nn.cpp:382-424)
    const int64_t id = (int64_t)block * kBlock + tid;
    const int64_t node_num = (int64_t)1 << (3 * d);
    if (id >= ((int64_t)a.n_clouds * node_num) << 3) return;
    const int64_t groups = node_num >> 3;
    const int slot = (int)(id & 63);
    const int64_t g = id >> 6;
    const int64_t cloud = g / groups;
    uint32_t x0, y0, z0;
    morton_decode((uint64_t)(g % groups) << 3, d, &x0, &y0, &z0);
    const uint32_t x1 = x0 + (slot >> 4) - 1, y1 = y0 + ((slot >> 2) & 3) - 1, z1 = z0 + (slot & 3) - 1;
    int v = -1;
    if (((x1 | y1 | z1) & (1u << d)) == 0) v = (int)(morton_encode(x1, y1, z1, d) + (uint64_t)cloud * node_num);
    reinterpret_cast<int*>(blob + a.off_neigh[d])[id] = v;
    return;
  }
  if (kind == kSegNeighSearch) {
    // Neighbour table of a small sparse level straight from the geometry, so that it waits for
    // no other level: wavefront = sibling group g (children of the g-th non-empty node of level
    // d-1), lane = slot (x<<4 | y<<2 | z) = the node at offset (x-1, y-1, z-1) from sibling 0.
    // That node exists iff it lies inside the cube and its parent is a non-empty node of the
    // same cloud: the parent's rank r in the sorted list gives the index 8r + octant.  Equal to
    // what calc_neigh derives level by level (octree_nn.cpp:357-380).
    // The 64 slots of a group have only 27 different parents (the 3x3x3 nodes around the group's
    // own parent), so 27 lanes search and the slots pick their parent's rank up by a shuffle; a
    // wavefront takes four groups, two in each half of its lanes, and walks the two searches of a
    // lane side by side (the divergent loads of the search are what this segment costs).
    const int n_par = a.nne[d - 1];
    const int g0 = (block * (kBlock / 64) + (tid >> 6)) * kSearchPerWave;
    if (g0 >= n_par) return;
    const int lane = tid & 63, half = lane >> 5, pl = lane & 31;
    const int bits = 3 * (d - 1);
    const uint64_t* __restrict__ list = a.list[d - 1];
    const int ox = pl / 9 - 1, oy = (pl / 3) % 3 - 1, oz = pl % 3 - 1;   // pl < 27
    uint64_t want[2];
    int lo[2], hi[2];
    bool inside[2];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const uint64_t pk = list[min(g0 + 2 * q + half, n_par - 1)];
      const uint64_t cloud_bits = (pk >> bits) << bits;
      uint32_t px, py, pz;
      morton_decode(pk - cloud_bits, d - 1, &px, &py, &pz);
      const int nx = (int)px + ox, ny = (int)py + oy, nz = (int)pz + oz;
      inside[q] = pl < 27 && nx >= 0 && ny >= 0 && nz >= 0 && ((nx | ny | nz) >> (d - 1)) == 0;
      want[q] = cloud_bits | morton_encode((uint32_t)max(nx, 0), (uint32_t)max(ny, 0), (uint32_t)max(nz, 0), d - 1);
      lo[q] = 0;
      hi[q] = inside[q] ? n_par : 0;   // an empty range: nothing is looked up
    }
    for (int span = n_par; span > 0; span >>= 1) {   // enough halvings for every search
      uint64_t v[2];
#pragma unroll
      for (int q = 0; q < 2; ++q) v[q] = lo[q] < hi[q] ? list[(lo[q] + hi[q]) >> 1] : 0;
#pragma unroll
      for (int q = 0; q < 2; ++q)
        if (lo[q] < hi[q]) {
          const int mid = (lo[q] + hi[q]) >> 1;
          if (v[q] < want[q]) lo[q] = mid + 1; else hi[q] = mid;
        }
    }
    int rank[2];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const uint64_t at = list[min(lo[q], n_par - 1)];
      rank[q] = inside[q] && lo[q] < n_par && at == want[q] ? lo[q] : -1;
    }
    // slot (x, y, z) of a group = the node at (x - 1, y - 1, z - 1) from sibling 0: its parent is
    // the one at ((x + 1) >> 1) - 1 ... from the group's parent, its octant the low bits of x + 1 ...
    const int sx = lane >> 4, sy = (lane >> 2) & 3, sz = lane & 3;
    const int from = ((sx + 1) >> 1) * 9 + ((sy + 1) >> 1) * 3 + ((sz + 1) >> 1);
    const int oct = (((sx + 1) & 1) << 2) | (((sy + 1) & 1) << 1) | ((sz + 1) & 1);
#pragma unroll
    for (int q = 0; q < 2; ++q)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int r = __shfl(rank[q], from + 32 * h, 64);
        const int g = g0 + 2 * q + h;
        if (g < n_par) reinterpret_cast<int*>(blob + a.off_neigh[d])[((int64_t)g << 6) + lane] = r < 0 ? -1 : 8 * r + oct;
      }
    return;
  }
  uint64_t* key = reinterpret_cast<uint64_t*>(blob + a.off_key[d]);
  int* child = reinterpret_cast<int*>(blob + a.off_child[d]);
  float* split = a.off_split[d] >= 0 ? reinterpret_cast<float*>(blob + a.off_split[d]) : nullptr;
  const int n_d = a.nnum[d];
  if (kind == kSegFull) {
    // full layers: node t = cloud * 8^d + i, key i; child t, or on the last full layer the
    // rank among the non-empty nodes
    const int64_t t = (int64_t)block * kBlock + tid;
    if (t >= n_d) return;
    const int64_t per = (int64_t)1 << (3 * d);
    const int cloud = (int)(t / per);
    const uint64_t i = (uint64_t)(t % per);
    key[t] = out_key(i, d, cloud, a.key2xyz);
    if (a.key_channel == 2) key[n_d + t] = 0;
    int c = (int)t;
    if (d == a.full_layer) {
      c = -1;
      if (a.depth > a.full_layer) {
        const uint64_t want = ((uint64_t)cloud << (3 * d)) | i;
        const uint64_t* __restrict__ list = a.list[d];
        int lo = 0, hi = a.nne[d];
        while (lo < hi) {
          const int mid = (lo + hi) >> 1;
          if (list[mid] < want) lo = mid + 1; else hi = mid;
        }
        if (lo < a.nne[d] && list[lo] == want) c = lo;
      }
    }
    child[t] = c;
    if (split) split[t] = c < 0 ? 0.0f : 1.0f;  // calc_split_label, octree.cpp:1158-1178
    return;
  }
  // sparse layers: thread = sibling group p (the children of the p-th non-empty node of level
  // d-1): node 8p + octant, key from the parent's key; the non-empty ones are consecutive in
  // list[d] from first[d-1][p].  Parent keys and child links are staged in LDS so that the nodes
  // leave in full rows.
  const int groups = a.nne[d - 1];
  const int p = block * kBlock + tid;
  if (p < groups) {
    s_parent[tid] = a.list[d - 1][p];     // cloud << 3(d-1) | morton_{d-1}
    const int c0 = a.first[d - 1][p], c1 = a.first[d - 1][p + 1];
    int oct[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) oct[u] = c0 + u < c1 ? (int)(a.list[d][c0 + u] & 7) : 8;
#pragma unroll
    for (int o = 0; o < 8; ++o) {
      int c = -1;
#pragma unroll
      for (int u = 0; u < 8; ++u) c = oct[u] == o ? c0 + u : c;
      s_child[tid * 8 + o] = c;
    }
  }
  __syncthreads();
  const int64_t node0 = (int64_t)block * kBlock * 8;
  const int rows = min(kBlock * 8, n_d - (int)node0);  // nodes of this workgroup
  const uint64_t pmask = (1ull << (3 * (d - 1))) - 1;
  for (int r = tid; r < rows; r += kBlock) {
    const uint64_t pk = s_parent[r >> 3];
    key[node0 + r] = out_key(((pk & pmask) << 3) | (uint64_t)(r & 7), d, (int)(pk >> (3 * (d - 1))), a.key2xyz);
    if (a.key_channel == 2) key[n_d + node0 + r] = 0;
    const int c = s_child[r];
    child[node0 + r] = c;
    if (split) split[node0 + r] = c < 0 ? 0.0f : 1.0f;
  }
}

// Signal of the finest level, one thread per node: empty nodes get zeros (label -1), so every
// row of the feature block is written exactly once, in full wavefront-wide rows.
__global__ __launch_bounds__(kBlock) void leaf_signal_kernel(float* __restrict__ feature,
    float* __restrict__ label, const int* __restrict__ child, const uint64_t* __restrict__ leaf_key,
    const int* __restrict__ ustart, const uint32_t* __restrict__ sorted_idx, const CloudDesc* __restrict__ clouds,
    SignalGeom g) {
  const int node = blockIdx.x * blockDim.x + threadIdx.x;
  if (node >= g.nnum_d) return;
  const int j = child[node];
  if (label) label[node] = -1.0f;
  if (j < 0) {
    for (int c = 0; c < g.channels; ++c) feature[(int64_t)c * g.nnum_d + node] = 0.0f;
    return;
  }
  leaf_signal(feature, label, node, (int)(leaf_key[j] >> (3 * g.depth)), ustart[j], ustart[j + 1], sorted_idx,
      clouds, g);
}

__global__ void fill_f32_kernel(float* p, int64_t n, float v) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += step) p[i] = v;
}

// ---- host side -------------------------------------------------------------------------------
inline size_t al(size_t v) { return (v + 255) & ~(size_t)255; }
inline int sort_items(int64_t n) { return n <= (1 << 19) ? 4 : 8; }
// status rows (one per tile / per group of tiles) of a pass
inline size_t status_words(int tiles) { return (size_t)tiles; }
inline size_t group_words(int tiles) { return (size_t)(tiles / kGroupTiles + 1); }

struct Layout {          // byte offsets inside the workspace
  size_t clouds, control, hist, sort_status, sort_groups, level_status, level_groups, zero_end;
  size_t key[2], val[2], ustart;
  size_t list[kMaxLevels], first[kMaxLevels];
  size_t total;
  int sort_tiles, level_tiles;
};

Layout make_layout(int64_t N, int B, int depth) {
  Layout L;
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += al(bytes); return o; };
  size_t n = (size_t)(N > 0 ? N : 1);
  L.clouds = take(sizeof(CloudDesc) * (size_t)(B > 0 ? B : 1));
  L.sort_tiles = (int)((n + kBlock * sort_items(N) - 1) / (kBlock * sort_items(N)));
  L.level_tiles = (int)((n + kLevelTile - 1) / kLevelTile);
  // one zeroed region: control words, histograms, look-back status of every pass
  L.control = take(sizeof(Control));
  L.hist = take(sizeof(int) * 256 * kMaxPasses * kHistCopies);
  L.sort_status = take(sizeof(uint32_t) * 256 * status_words(L.sort_tiles) * kMaxPasses);
  L.sort_groups = take(sizeof(uint32_t) * 256 * group_words(L.sort_tiles) * kMaxPasses);
  L.level_status = take(sizeof(uint32_t) * 16 * status_words(L.level_tiles));
  L.level_groups = take(sizeof(uint32_t) * 16 * group_words(L.level_tiles));
  L.zero_end = off;
  for (int i = 0; i < 2; ++i) { L.key[i] = take(8 * n); L.val[i] = take(4 * n); }
  L.ustart = take(4 * (n + 1));
  for (int d = 0; d < kMaxLevels; ++d) {
    if (d <= depth) { L.list[d] = take(8 * n); L.first[d] = take(4 * (n + 1)); }
    else { L.list[d] = L.first[d] = 0; }
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

// bounded waits of the look-back (polls of one status window, each followed by a short sleep)
constexpr int kFirstWaitLimit = 1 << 16, kTicketWaitLimit = 1 << 22;
std::atomic<int> g_first_wait_limit{kFirstWaitLimit};
std::atomic<int> g_ticket_reruns{0};

// Pinned host slots that the level scan writes the node counts into (coherent host memory:
// the device writes it in place, the host reads it in place).
std::mutex g_slots_mutex;
std::vector<HostCounts*> g_free_slots;
HostCounts* take_slot() {
  {
    std::lock_guard<std::mutex> lock(g_slots_mutex);
    if (!g_free_slots.empty()) { HostCounts* s = g_free_slots.back(); g_free_slots.pop_back(); return s; }
  }
  void* p = nullptr;
  if (hipHostMalloc(&p, 256, hipHostMallocCoherent) != hipSuccess) return nullptr;
  memset(p, 0, 256);
  return static_cast<HostCounts*>(p);
}
void give_slot(HostCounts* s) {
  std::lock_guard<std::mutex> lock(g_slots_mutex);
  g_free_slots.push_back(s);
}
std::atomic<int> g_plan_seq{1};

// Waits until the device has written `seq` into the slot.  The host polls the word for a while
// (the answer is a few microseconds away when the stream was idle), then falls back on the
// stream, which also reports a launch that failed.
int await_counts(HostCounts* h, int seq, hipStream_t s) {
  const auto t0 = std::chrono::steady_clock::now();
  for (int spins = 0;; ++spins) {
    if (__atomic_load_n(&h->seq, __ATOMIC_ACQUIRE) == seq) return OCNN_OK;
    if ((spins & 1023) == 1023 &&
        std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(20)) break;
  }
  hipError_t e = hipStreamSynchronize(s);
  OCNN_REQUIRE(e == hipSuccess, OCNN_E_HIP, "node counts: %s", hipGetErrorString(e));
  OCNN_REQUIRE(__atomic_load_n(&h->seq, __ATOMIC_ACQUIRE) == seq, OCNN_E_HIP,
      "the level scan finished without handing over the node counts");
  return OCNN_OK;
}

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
      "node_feature / adaptive octrees take two rounds of allocation: use ocnn_points2octree");
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
    OCNN_REQUIRE(N < (1ll << 30), OCNN_E_BADARG, "more than 2^30 points");
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
  Control* d_ctl = reinterpret_cast<Control*>(ws + L.control);
  uint64_t* d_key[2] = {reinterpret_cast<uint64_t*>(ws + L.key[0]), reinterpret_cast<uint64_t*>(ws + L.key[1])};
  uint32_t* d_val[2] = {reinterpret_cast<uint32_t*>(ws + L.val[0]), reinterpret_cast<uint32_t*>(ws + L.val[1])};
  int* d_hist = reinterpret_cast<int*>(ws + L.hist);
  uint32_t* d_sort_status = reinterpret_cast<uint32_t*>(ws + L.sort_status);

  BuildGeom g;
  g.depth = depth;
  g.full_layer = fl;
  g.n_clouds = n_clouds;
  g.n_points = N;
  for (int i = 0; i < 3; ++i) g.bbmin[i] = o.bbmin[i];
  g.mul = float(1 << depth) / o.bbox_max_width();  // octree.cpp:159
  int cloud_bits = 0;
  while ((1 << cloud_bits) < n_clouds) ++cloud_bits;
  const int nbits = 3 * depth + cloud_bits;
  g.passes = (nbits + 7) / 8;
  g.bits = (nbits + g.passes - 1) / g.passes;

  // control words + the cloud table (passed as kernel arguments, 48 clouds a launch: no
  // staged host-to-device copy)
  auto init = [&]() -> int {
    const int64_t zero_words = depth > fl ? (int64_t)((L.zero_end - L.control) / 4) : (int64_t)(sizeof(Control) / 4);
    for (int first = 0; first < n_clouds; first += kArgClouds) {
      CloudChunk chunk;
      memset(&chunk, 0, sizeof(chunk));
      const int count = n_clouds - first < kArgClouds ? n_clouds - first : kArgClouds;
      memcpy(chunk.c, clouds.data() + first, sizeof(CloudDesc) * count);
      const int64_t zw = first == 0 ? zero_words : 0;
      int64_t blocks = (zw + kBlock * 4 - 1) / (kBlock * 4);
      if (blocks < 1) blocks = 1;
      if (blocks > 1024) blocks = 1024;
      init_kernel<<<(unsigned)blocks, kBlock, 0, s>>>(reinterpret_cast<uint32_t*>(ws + L.control), zw, d_clouds,
          chunk, first, count);
    }
    OCNN_LAUNCH_OK("init");
    return OCNN_OK;
  };

  PlanState st;
  memset(&st, 0, sizeof(st));
  int cur = 0;
  // keys, sort, level scan, counts to the host; *wait_error: a bounded wait ran out
  auto sort_and_scan = [&](bool tickets, int spin_limit, int* wait_error) -> int {
    cur = 0;
    keygen_kernel<<<min(blocks_for(N, kBlock * kKeyItems), (unsigned)kKeyGrid), kBlock, 0, s>>>(d_key[0], d_val[0],
        d_clouds, d_hist, g);
    OCNN_LAUNCH_OK("keygen");
    for (int p = 0; p < g.passes; ++p) {
      uint32_t* status = d_sort_status + (size_t)p * 256 * status_words(L.sort_tiles);
      uint32_t* groups = reinterpret_cast<uint32_t*>(ws + L.sort_groups) + (size_t)p * 256 * group_words(L.sort_tiles);
      auto launch = [&](auto kernel) {
        kernel<<<L.sort_tiles, kBlock, 0, s>>>(d_key[cur], d_val[cur], d_key[cur ^ 1], d_val[cur ^ 1], (int)N,
            p * g.bits, g.bits, d_hist + p * 256, status, groups, d_ctl, p, spin_limit);
      };
      if (sort_items(N) == 4) { if (tickets) launch(sort_pass_kernel<4, true>); else launch(sort_pass_kernel<4, false>); }
      else { if (tickets) launch(sort_pass_kernel<8, true>); else launch(sort_pass_kernel<8, false>); }
      OCNN_LAUNCH_OK("sort pass");
      cur ^= 1;
    }
    LevelOut lo;
    memset(&lo, 0, sizeof(lo));
    for (int d = fl; d <= depth; ++d) {
      lo.list[d] = reinterpret_cast<uint64_t*>(ws + L.list[d]);
      lo.first[d] = reinterpret_cast<int*>(ws + L.first[d]);
    }
    lo.ustart = reinterpret_cast<int*>(ws + L.ustart);
    uint32_t* level_status = reinterpret_cast<uint32_t*>(ws + L.level_status);
    uint32_t* level_groups = reinterpret_cast<uint32_t*>(ws + L.level_groups);
    HostCounts* h = take_slot();
    OCNN_REQUIRE(h, OCNN_E_HIP, "no pinned host memory for the node counts");
    const int seq = g_plan_seq.fetch_add(1) & 0x3fffffff;
    if (tickets) levels_kernel<true><<<L.level_tiles, kBlock, 0, s>>>(d_key[cur], (int)N, depth, fl, lo, level_status, level_groups, d_ctl, spin_limit, h, seq);
    else levels_kernel<false><<<L.level_tiles, kBlock, 0, s>>>(d_key[cur], (int)N, depth, fl, lo, level_status, level_groups, d_ctl, spin_limit, h, seq);
    if (hipGetLastError() != hipSuccess) { give_slot(h); return fail(OCNN_E_HIP, "launch of levels failed"); }
    const int rc = await_counts(h, seq, s);
    for (int d = fl; d <= depth; ++d) st.nne[d] = h->nne[d];
    *wait_error = h->error;
    give_slot(h);
    return rc;
  };

  int rc = init();
  if (rc != OCNN_OK) return rc;
  if (depth > fl) {
    int wait_error = 0;
    rc = sort_and_scan(false, g_first_wait_limit.load(), &wait_error);
    if (rc != OCNN_OK) return rc;
    if (wait_error) {  // tiles did not start in index order: once more, with ticket order
      g_ticket_reruns.fetch_add(1);
      rc = init();
      if (rc == OCNN_OK) rc = sort_and_scan(true, kTicketWaitLimit, &wait_error);
      if (rc != OCNN_OK) return rc;
      OCNN_REQUIRE(wait_error == 0, OCNN_E_HIP, "a tile waited too long for the tiles before it");
    }
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
    if (params->merged != kMergedNoNeigh) o.set_property(OCNN_NEIGH, 8, -1);
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

  EmitArgs a;
  memset(&a, 0, sizeof(a));
  memcpy(&a.hdr, &o, sizeof(Info));
  a.depth = depth;
  a.full_layer = fl;
  a.n_clouds = B;
  a.key2xyz = o.key2xyz;
  a.key_channel = o.channel(OCNN_KEY);
  for (int d = 0; d < kMaxLevels; ++d) {
    a.off_key[d] = a.off_child[d] = a.off_split[d] = a.off_neigh[d] = -1;
    if (d > depth) continue;
    a.nnum[d] = o.nnum[d];
    a.nne[d] = st.nne[d];
    a.off_key[d] = o.ptr_dis(OCNN_KEY, d);
    a.off_child[d] = o.ptr_dis(OCNN_CHILD, d);
    a.off_split[d] = o.ptr_dis(OCNN_SPLIT, d);
    a.off_neigh[d] = o.ptr_dis(OCNN_NEIGH, d);
    a.list[d] = reinterpret_cast<const uint64_t*>(ws + L.list[d]);
    a.first[d] = reinterpret_cast<const int*>(ws + L.first[d]);
  }
  const int64_t HD = o.nnum[depth];
  const int fch = o.channel(OCNN_FEATURE);
  a.off_feature = fch > 0 ? o.ptr_dis(OCNN_FEATURE, depth) : -1;
  a.off_label = o.has(OCNN_LABEL) ? o.ptr_dis(OCNN_LABEL, depth) : -1;
  a.ustart = reinterpret_cast<const int*>(ws + L.ustart);
  a.sorted_idx = reinterpret_cast<const uint32_t*>(ws + L.val[st.sorted_buf]);
  a.clouds = reinterpret_cast<const CloudDesc*>(ws + L.clouds);
  a.sg.depth = depth;
  a.sg.nnum_d = (int)HD;
  a.sg.ch_feature = st.ch_feature;
  a.sg.channels = fch;
  a.sg.has_label = a.off_label >= 0;
  a.sg.has_dis = o.has_node_dis;
  a.sg.save_pts = o.save_pts;
  for (int i = 0; i < 3; ++i) a.sg.bbmin[i] = o.bbmin[i];
  a.sg.mul = st.mul;

  int n_seg = 0, blocks = 0;
  auto add_seg = [&](int kind, int level, int64_t nblocks) {
    if (nblocks <= 0) return;
    a.seg_begin[n_seg] = blocks;
    a.seg_kind[n_seg] = (unsigned char)kind;
    a.seg_level[n_seg] = (unsigned char)level;
    ++n_seg;
    blocks += (int)nblocks;
  };
  add_seg(kSegHeader, 0, 1);
  // the searched neighbour tables first (their divergent loads then run beside the workgroups
  // below, which mostly wait for memory), then the signal of the finest level: its workgroups
  // take longest
  int searched_to = fl;  // sparse levels up to here have their neighbour table after this launch
  if (o.has(OCNN_NEIGH))
    for (int d = fl + 1; d <= depth && st.nne[d - 1] > 0 && st.nne[d - 1] <= kSearchGroups; ++d) {
      add_seg(kSegNeighSearch, d, blocks_for(st.nne[d - 1], (kBlock / 64) * kSearchPerWave));
      searched_to = d;
    }
  const bool has_signal = depth > fl && HD > 0 && (a.off_feature >= 0 || a.off_label >= 0);
  const bool signal_inside = has_signal && fch <= kSignalStage;
  size_t lds = kEmitLdsBytes;
  if (signal_inside) {
    add_seg(kSegLeafSignal, depth, blocks_for(HD, kSignalTile));
    const size_t need = signal_lds_bytes(fch, a.off_label >= 0, B > 1);
    if (need > lds) lds = need;
  }
  for (int d = depth; d > fl; --d) add_seg(kSegSparse, d, blocks_for(st.nne[d - 1]) * (st.nne[d - 1] > 0 ? 1 : 0));
  for (int d = 0; d <= fl; ++d) {
    add_seg(kSegFull, d, blocks_for(o.nnum[d]));
    if (o.has(OCNN_NEIGH) && d >= 1) add_seg(kSegFullNeigh, d, blocks_for((int64_t)B << (3 * d + 3)));
  }
  a.seg_begin[n_seg] = blocks;
  a.n_seg = n_seg;
  emit_kernel<<<blocks, kBlock, lds, s>>>(blob, a);
  OCNN_LAUNCH_OK("emit");

  if (has_signal && !signal_inside) {   // more channels than a tile stages: one thread per node, after the child links
    float* f_ptr = a.off_feature >= 0 ? reinterpret_cast<float*>(blob + a.off_feature) : nullptr;
    float* l_ptr = a.off_label >= 0 ? reinterpret_cast<float*>(blob + a.off_label) : nullptr;
    const int* c_ptr = reinterpret_cast<const int*>(blob + a.off_child[depth]);
    leaf_signal_kernel<<<blocks_for(HD), kBlock, 0, s>>>(f_ptr, l_ptr, c_ptr, a.list[depth], a.ustart,
        a.sorted_idx, a.clouds, a.sg);
    OCNN_LAUNCH_OK("leaf_signal");
  }
  if (depth == fl && HD > 0) {  // no sparse level: the finest level carries no signal
    if (a.off_feature >= 0)
      fill_f32_kernel<<<blocks_for(fch * HD, kBlock * 4), kBlock, 0, s>>>(reinterpret_cast<float*>(blob + a.off_feature), fch * HD, 0.0f);
    if (a.off_label >= 0)
      fill_f32_kernel<<<blocks_for(HD, kBlock * 4), kBlock, 0, s>>>(reinterpret_cast<float*>(blob + a.off_label), HD, -1.0f);
    OCNN_LAUNCH_OK("fill");
  }
  if (o.has(OCNN_NEIGH)) {
    // merge_octrees.cpp:185-197: the remaining sparse levels, each from the level above; the last
    // (and largest) two or three in one launch while the tables are bound by the chain of dependent
    // trips to memory rather than by their bytes (measured on depth-9 scenes of 250 k points, levels
    // fused 1 / 2 / 3: one scene 0.121 / 0.113 / 0.112 ms, four 0.310 / 0.290 / 0.295, eight 0.575 /
    // 0.579 / 0.608)
    const int fuse = o.nnum[depth] <= (1 << 21) ? 3 : (o.nnum[depth] <= (1 << 23) ? 2 : 1);
    for (int d = searched_to + 1; d <= depth;) {
      if (o.nnum[d - 1] <= 0) { ++d; continue; }
      int count = 1;
      if (depth - d < fuse) while (d + count <= depth && o.nnum[d + count - 1] > 0) ++count;
      int* out[kNeighLevels] = {nullptr, nullptr, nullptr};
      const int* children[kNeighLevels] = {nullptr, nullptr, nullptr};
      for (int i = 0; i < count; ++i) {
        out[i] = reinterpret_cast<int*>(blob + o.ptr_dis(OCNN_NEIGH, d + i));
        children[i] = reinterpret_cast<const int*>(blob + o.ptr_dis(OCNN_CHILD, d + i - 1));
      }
      launch_neigh_sparse_levels(count, out, reinterpret_cast<const int*>(blob + o.ptr_dis(OCNN_NEIGH, d - 1)), children,
          o.nnum[d - 1], s);
      OCNN_LAUNCH_OK("neigh");
      d += count;
    }
  }
  return OCNN_OK;
}

int ocnn_points2octree_into(const void* const* points_dev, const void* const* points_info, int n_clouds,
    const ocnn_build_params* params, void* workspace_dev, size_t workspace_bytes, void* octree_buf_dev,
    size_t capacity, void* info_out, ocnn_stream_t stream) {
  OCNN_REQUIRE(octree_buf_dev && info_out, OCNN_E_BADARG, "null pointer");
  int e = ocnn_points2octree_plan(points_dev, points_info, n_clouds, params, workspace_dev, workspace_bytes,
      info_out, stream);
  if (e != OCNN_OK) return e;
  const int64_t need = static_cast<const Info*>(info_out)->sizeof_octree();
  // too small: the plan stays on the workspace for ocnn_points2octree_emit
  OCNN_REQUIRE((size_t)need <= capacity, OCNN_E_WORKSPACE, "the octree takes %lld bytes, the buffer holds %zu",
      (long long)need, capacity);
  return ocnn_points2octree_emit(octree_buf_dev, info_out, workspace_dev, workspace_bytes, stream);
}

int ocnn_points2octree_wait_limit(int polls) {
  const int before = g_first_wait_limit.load();
  g_first_wait_limit.store(polls == 0 ? kFirstWaitLimit : polls);
  return before;
}
int ocnn_points2octree_ticket_reruns(void) { return g_ticket_reruns.load(); }

int ocnn_points2octree(const void* const* points_dev, const void* const* points_info, int n_clouds,
    const ocnn_build_params* params, void* workspace_dev, size_t workspace_bytes, ocnn_alloc_fn alloc,
    void* alloc_ctx, void* info_out, void** octree_out_dev, ocnn_stream_t stream) {
  OCNN_REQUIRE(alloc && octree_out_dev && params && points_info && points_dev, OCNN_E_BADARG, "null pointer");
  if (params->node_feature || params->adaptive) {
    // Signals at every depth / trimming: a plain octree first (raw Morton keys, average points
    // kept whenever the displacement is), then the second stage on top of it.  A batch goes
    // through both stages as ONE octree in merged layout: every step of the second stage works
    // within a sibling group or over a node's own leaves, except the trimming rule that keeps
    // one node per level, which is applied per octree (the index in the top bits of the keys).
    OCNN_REQUIRE(params->merged == 0 || params->merged == 1, OCNN_E_BADARG, "merged %d", params->merged);
    OCNN_REQUIRE(n_clouds == 1 || params->merged, OCNN_E_BADARG, "a single-octree blob holds one cloud");
    const PointsInfo* pi = static_cast<const PointsInfo*>(points_info[0]);
    OCNN_REQUIRE(pi, OCNN_E_BADARG, "null cloud header");
    const bool has_normal = (pi->content_flags & 2) != 0;
    // trim_octree reads the normal error (exists only with normals) and leaves the average
    // points untrimmed (octree.cpp:1004-1135): the reference cannot build these either
    OCNN_REQUIRE(!params->adaptive || (has_normal && !params->save_pts && params->adp_depth >= 1),
        OCNN_E_UNSUPPORTED, "adaptive octrees need normals, no save_pts and adp_depth >= 1");
    ocnn_build_params p0 = *params;
    p0.node_feature = p0.adaptive = p0.key2xyz = p0.split_label = p0.extrapolate = 0;
    p0.save_pts = (params->node_dis || params->save_pts) ? 1 : 0;
    p0.merged = params->merged ? kMergedNoNeigh : 0;   // the first stage's neighbour tables would be thrown away
    AdaptiveInput in;
    in.merged = params->merged ? 1 : 0;
    int e = ocnn_points2octree_plan(points_dev, points_info, n_clouds, &p0, workspace_dev, workspace_bytes, &in.info0, stream);
    if (e != OCNN_OK) return e;
    in.blob0 = static_cast<char*>(alloc((size_t)in.info0.sizeof_octree(), alloc_ctx));
    if (!in.blob0) {
      std::lock_guard<std::mutex> lock(g_plans_mutex);
      g_plans.erase(workspace_dev);
      return fail(OCNN_E_BADARG, "the allocator returned no memory for the first-stage octree");
    }
    e = ocnn_points2octree_emit(in.blob0, &in.info0, workspace_dev, workspace_bytes, stream);
    if (e != OCNN_OK) return e;
    in.ch_normal = has_normal ? pi->channels[1] : 0;
    in.ch_feature = (pi->content_flags & 4) ? pi->channels[2] : 0;
    in.ch_dis = params->node_dis ? (has_normal ? 1 : 4) : 0;
    in.has_pt = p0.save_pts;
    in.has_label = (pi->content_flags & 8) && pi->channels[3] == 1;
    in.params = *params;
    return adaptive_finish(in, alloc, alloc_ctx, info_out, octree_out_dev, as_stream(stream));
  }
  int e = ocnn_points2octree_plan(points_dev, points_info, n_clouds, params, workspace_dev, workspace_bytes,
      info_out, stream);
  if (e != OCNN_OK) return e;
  void* blob = alloc((size_t)static_cast<const Info*>(info_out)->sizeof_octree(), alloc_ctx);
  if (!blob) {
    std::lock_guard<std::mutex> lock(g_plans_mutex);
    g_plans.erase(workspace_dev);
    return fail(OCNN_E_BADARG, "the allocator returned no memory for %lld bytes",
        (long long)static_cast<const Info*>(info_out)->sizeof_octree());
  }
  *octree_out_dev = blob;
  return ocnn_points2octree_emit(blob, info_out, workspace_dev, workspace_bytes, stream);
}

}  // extern "C"
