// Second stage of the octree builder for node_feature / adaptive octrees
// (Octree::build, octree/octree/octree.cpp:96-120): signals at every depth with the
// normal and distance errors of the planar approximation (calc_signal, :454-664, over
// the leaf ranges of covered_depth_nodes, :958-1002), extrapolation into empty nodes
// (:666-806), split labels (:1158-1178) and trimming (trim_octree, :1004-1135), then
// serialization (:907-956).
//
// Every float result must equal the sequential CPU result bit for bit (the trimming
// thresholds decide the STRUCTURE of the octree), so a sum is taken by one wavefront in
// the reference's order: 64 lanes fetch 64 consecutive leaf nodes, the values of the
// non-empty ones are read lane by lane (v_readlane) and added one after the other.  Maxima,
// minima and counts do not depend on the order and are reduced across the lanes.
#include "build_adaptive.h"
#include "octree_kernels.h"

#include <algorithm>
#include <vector>

namespace ocnn {
namespace {

constexpr int kMaxD = 17;

__device__ inline float sqrt_rn(float x) { return (float)sqrt((double)x); }
__device__ inline float div_rn(float a, float b) { return (float)((double)a / (double)b); }
__device__ inline float read_lane(float v, int src) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src));
}
__device__ inline float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ inline float wave_min(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ inline int wave_min_i(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = min(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ inline int wave_max_i(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = max(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ inline int wave_sum_i(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ inline float norm3(const float* v) {  // math_functions.cpp:257-263
  float len = 0.0f;
  for (int c = 0; c < 3; ++c) len = __fadd_rn(len, __fmul_rn(v[c], v[c]));
  return sqrt_rn(len);
}

// ---- covered_depth_nodes (octree.cpp:958-1002): range of finest-level nodes under a node.
// The finest level itself needs no table (a node covers itself).  The level above it covers
// its eight children, and every node of the finest level is such a child: its error terms start
// "infinite" here (calc_signal leaves them at 1.0e20f, octree.cpp:456-470).
__global__ void cover_first_kernel(int* __restrict__ dnum, int* __restrict__ didx, const int* __restrict__ child,
    float* __restrict__ nerr_c, float* __restrict__ derr_c, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int c = child[i];
  dnum[i] = c >= 0 ? 8 : 0;
  didx[i] = c >= 0 ? c * 8 : -1;
  if (c >= 0) {
    const float4 big = make_float4(1.0e20f, 1.0e20f, 1.0e20f, 1.0e20f);
    float4* e0 = reinterpret_cast<float4*>(nerr_c + c * 8);
    float4* e1 = reinterpret_cast<float4*>(derr_c + c * 8);
    e0[0] = big; e0[1] = big; e1[0] = big; e1[1] = big;
  }
}
__device__ inline void cover_node(int* __restrict__ dnum, int* __restrict__ didx, const int* __restrict__ child,
    const int* dnum_c, const int* didx_c, int i) {
  int num = 0, idx = -1;
  const int c = child[i];
  if (c >= 0) {
    for (int j = 0; j < 8; ++j) num += dnum_c[c * 8 + j];
    for (int j = 0; j < 8; ++j)
      if (didx_c[c * 8 + j] != -1) { idx = didx_c[c * 8 + j]; break; }
  }
  dnum[i] = num;
  didx[i] = idx;
}
__global__ void cover_kernel(int* __restrict__ dnum, int* __restrict__ didx, const int* __restrict__ child,
    const int* __restrict__ dnum_c, const int* __restrict__ didx_c, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) cover_node(dnum, didx, child, dnum_c, didx_c, i);
}
// the small levels at the top, one after the other in one workgroup
struct CoverTop {
  int d_top;   // levels d_top .. 0; level d_top + 1 is complete
  int n[kMaxD];
  int* dnum[kMaxD]; int* didx[kMaxD]; const int* child[kMaxD];
};
__global__ __launch_bounds__(1024) void cover_top_kernel(const CoverTop t) {
  for (int d = t.d_top; d >= 0; --d) {
    for (int i = threadIdx.x; i < t.n[d]; i += 1024) cover_node(t.dnum[d], t.didx[d], t.child[d], t.dnum[d + 1], t.didx[d + 1], i);
    __syncthreads();   // the level's tables are read by the next one (same workgroup: its writes are visible after the barrier)
  }
}

__global__ void fill_kernel(float* __restrict__ p, int64_t n, float v) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

// ---- calc_signal (octree.cpp:454-664) -------------------------------------------------------
// corner and edge conventions of the marching-cube tables the reference intersects with
// (octree/octree/marching_cube_table.cpp:312-321)
__constant__ float kCorner[8][3] = {{0, 0, 0}, {0, 0, 1}, {0, 1, 1}, {0, 1, 0}, {1, 0, 0}, {1, 0, 1}, {1, 1, 1}, {1, 1, 0}};
__constant__ int kEdgeVert[12][2] = {{0, 1}, {1, 2}, {2, 3}, {3, 0}, {4, 5}, {5, 6}, {6, 7}, {7, 4}, {0, 4}, {1, 5}, {2, 6}, {3, 7}};

// vertices where the plane (pt, normal) cuts the edges of the unit cube at pt_base
// (intersect_cube, marching_cube.cpp:83-98 with contouring :40-65)
__device__ inline int intersect_cube(float* V, const float* pt, const float* pt_base, const float* normal) {
  float fval[8];
  unsigned cube_case = 0;
  for (int k = 0; k < 8; ++k) {
    float f = 0.0f;
    for (int j = 0; j < 3; ++j)
      f = __fadd_rn(f, __fmul_rn(__fsub_rn(__fadd_rn(kCorner[k][j], pt_base[j]), pt[j]), normal[j]));
    fval[k] = f;
    if (f < 0.0f) cube_case |= 1u << k;
  }
  int nv = 0;
  for (int e = 0; e < 12; ++e) {
    const int v1 = kEdgeVert[e][0], v2 = kEdgeVert[e][1];
    if ((((cube_case >> v1) ^ (cube_case >> v2)) & 1u) == 0) continue;
    float f1 = 0.0f, f2 = 0.0f;
    for (int k = 0; k < 8; ++k) { f1 = k == v1 ? fval[k] : f1; f2 = k == v2 ? fval[k] : f2; }
    float df = __fsub_rn(f2, f1);
    if (df == 0) df = __fadd_rn(df, 1.0e-10f);
    const float t = div_rn(-f1, df);
    for (int j = 0; j < 3; ++j) {
      const float pj = __fadd_rn(kCorner[v1][j], __fmul_rn(t, __fsub_rn(kCorner[v2][j], kCorner[v1][j])));
      V[3 * nv + j] = __fadd_rn(pj, pt_base[j]);
    }
    nv++;
  }
  return nv;
}

// Ordered sums over the non-empty leaves of a range.  The non-empty leaves of the finest level
// are packed once, in leaf order (LeafPack below; rows padded to whole 16-byte units), so a
// node's leaves are the packed range k0 <= k < k1 of every row.  row[c] is the packed row of
// value c (null: absent, sums to zero).  256 leaves at a time go through the wavefront's LDS
// block (a lane moves four consecutive leaves of a value with one 16-byte load and store), and
// lane c adds up value c leaf after leaf: the channels run side by side, each in the
// reference's order.  Leaves outside the range enter as +0, which changes no partial sum (a
// partial sum is never -0: the chain starts at +0).  Three blocks of 256 leaves are requested
// ahead of the one being added (the chain of a node high up in the tree covers the whole finest
// level, adding a block takes less time than a load from memory: the latency must not be paid
// per block).  sum[c] / last[c] get the sum and the
// last value of channel c on every lane.
constexpr int kPassValues = 8, kPassLeaves = 256;
template <int NV>
__device__ inline void ordered_sums(int k0, int k1, int lane, float* __restrict__ lds, const float* const (&row)[NV],
    const float* __restrict__ any_row, int64_t row_len, float* sum, float* last) {
  static_assert(NV <= kPassValues, "LDS block too small");
  float acc = 0.0f;
  constexpr int kAhead = 3;      // blocks requested before they are needed
  float4 vals[kAhead][NV];
  // Every request issues the same NV loads whatever the range (an absent row reads `any_row`,
  // a block past the end reads the last four values of the row, both become zeros): the number
  // of loads in flight behind a block is then a constant, and waiting for one block does not
  // wait for the blocks requested after it.
  const int k_last = (int)row_len - 4;
  auto request = [&](float4 (&dst)[NV], int base) {   // loads only: nothing here waits for them
    const int kk = min(base + 4 * lane, k_last);
#pragma unroll
    for (int c = 0; c < NV; ++c) dst[c] = *reinterpret_cast<const float4*>((row[c] ? row[c] : any_row) + kk);
  };
  auto stage = [&](const float4 (&raw)[NV], int base) {   // a block's values, zeros outside the range, to LDS
    const int k = base + 4 * lane;
#pragma unroll
    for (int c = 0; c < NV; ++c) {
      const bool have = row[c] != nullptr;
      float4 v = raw[c];
      v.x = (have && k >= k0 && k < k1) ? v.x : 0.0f;
      v.y = (have && k + 1 >= k0 && k + 1 < k1) ? v.y : 0.0f;
      v.z = (have && k + 2 >= k0 && k + 2 < k1) ? v.z : 0.0f;
      v.w = (have && k + 3 >= k0 && k + 3 < k1) ? v.w : 0.0f;
      *reinterpret_cast<float4*>(lds + c * kPassLeaves + 4 * lane) = v;
    }
    __builtin_amdgcn_wave_barrier();   // same wavefront: the LDS unit keeps its accesses in order
  };
  auto chain = [&](int base) {
    const int total = min(kPassLeaves, k1 - base);
    if (lane < NV) {
      // the adds form one dependent chain, and one wavefront issues an instruction every few
      // cycles: nothing but the adds and the LDS reads may sit in the loop.  Two register sets
      // take turns (the reads of the next 32 leaves are in flight while the current 32 are
      // added, an LDS read takes longer than 16 adds; the scheduler is told to keep that
      // order), every offset is a constant.
      constexpr int kStep = 32, kChunks = kPassLeaves / kStep;
      const float4* src = reinterpret_cast<const float4*>(lds + lane * kPassLeaves);
      float4 ra[kStep / 4], rb[kStep / 4];
      auto read = [&](float4 (&r)[kStep / 4], int chunk) {
#pragma unroll
        for (int i = 0; i < kStep / 4; ++i) r[i] = src[chunk * (kStep / 4) + i];
      };
      auto add = [&](const float4 (&r)[kStep / 4]) {
#pragma unroll
        for (int i = 0; i < kStep / 4; ++i) {
          acc = __fadd_rn(acc, r[i].x); acc = __fadd_rn(acc, r[i].y);
          acc = __fadd_rn(acc, r[i].z); acc = __fadd_rn(acc, r[i].w);
        }
      };
      read(ra, 0);
#pragma unroll
      for (int ch = 0; ch < kChunks; ch += 2) {
        if (ch * kStep >= total) break;
        read(rb, ch + 1);
        __builtin_amdgcn_sched_barrier(0);
        add(ra);
        __builtin_amdgcn_sched_barrier(0);
        if ((ch + 1) * kStep >= total) break;
        if (ch + 2 < kChunks) read(ra, ch + 2);
        __builtin_amdgcn_sched_barrier(0);
        add(rb);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __builtin_amdgcn_wave_barrier();
  };
  if (k0 < k1) {
    const int kb = k0 & ~3;
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      request(vals[u], kb + u * kPassLeaves);
      __builtin_amdgcn_sched_barrier(0);   // block after block, as in the loop: the wait below counts on the order
    }
    // kAhead blocks a turn, without a way out in between (a block past the end adds nothing):
    // straight-line code keeps the count of loads in flight a constant
    for (int base = kb; base < k1; base += kAhead * kPassLeaves) {
#pragma unroll
      for (int u = 0; u < kAhead; ++u) {
        const int b = base + u * kPassLeaves;
        stage(vals[u], b);
        request(vals[u], b + kAhead * kPassLeaves);   // its registers are free once the block sits in LDS
        __builtin_amdgcn_sched_barrier(0);
        chain(b);
      }
    }
  }
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    sum[c] = read_lane(acc, c);
    last[c] = (row[c] && k0 < k1) ? row[c][k1 - 1] : 0.0f;
  }
}
// The same walk for a sum whose terms interleave the channels (the normal error): every lane
// takes the same walk over the packed leaves, `term(vals)` gives the leaf's terms in order.
template <int NV, class Load, class Terms>
__device__ inline void ordered_terms(int k0, int k1, int lane, float* __restrict__ lds, Load load, Terms terms) {
  constexpr int kPassRounds = kPassLeaves / 64;
  for (int base = k0; base < k1; base += 64 * kPassRounds) {
#pragma unroll
    for (int u = 0; u < kPassRounds; ++u) {
      float vals[NV];
#pragma unroll
      for (int c = 0; c < NV; ++c) vals[c] = 0.0f;
      const int k = base + u * 64 + lane;
      if (k < k1) load(k, vals);
#pragma unroll
      for (int c = 0; c < NV; ++c) lds[(u * 64 + lane) * NV + c] = vals[c];
    }
    __builtin_amdgcn_wave_barrier();
    const int total = min(64 * kPassRounds, k1 - base);
#pragma unroll 4
    for (int t = 0; t < total; ++t) {
      float one[NV];
#pragma unroll
      for (int c = 0; c < NV; ++c) one[c] = lds[t * NV + c];
      terms(one);
    }
    __builtin_amdgcn_wave_barrier();
  }
}

// The non-empty leaves in leaf order: rank[j] = non-empty leaves before leaf j (rank[nD] = their
// number), and their normals / points / features side by side, channel-major rows of nD.
struct LeafPred {
  const int* child_D;
  __device__ bool operator()(int64_t j) const { return child_D[j] != -1; }
};
struct LeafPack {
  int* rank;
  int64_t nD, nP;   // leaves; row stride of the packed arrays
  int cf;
  const float *nrm_D, *pt_D, *feat_D, *lab_D;
  float *nrm_P, *pt_P, *feat_P, *lab_P;
  __device__ void operator()(int64_t j, bool f, int r) const {
    rank[j] = r;
    if (!f) return;
    if (nrm_D) for (int c = 0; c < 3; ++c) nrm_P[c * nP + r] = nrm_D[c * nD + j];
    if (pt_D) for (int c = 0; c < 3; ++c) pt_P[c * nP + r] = pt_D[c * nD + j];
    for (int c = 0; c < cf; ++c) feat_P[c * nP + r] = feat_D[c * nD + j];
    if (lab_D) lab_P[r] = lab_D[j];
  }
};

// what a node's signal is computed from: the level's own rows and the finest level
struct SignalArgs {
  int d, depth, n, nD, cf, ch_dis, adp_layer, calc_nerr, calc_derr;
  float imul;
  const uint64_t* key;        // level d
  const int* child;           // level d
  const int *dnum, *didx;     // level d
  const int* child_D;         // finest level: structure and signal, channel-major rows of nD
  const float *nrm_D, *pt_D, *feat_D, *lab_D;
  const int* rank_D;          // non-empty leaves before a leaf; [nD] = their number
  const float *nrm_P, *pt_P, *feat_P, *lab_P;   // the non-empty leaves packed in leaf order, rows of nP
  const float* any_P;         // nP floats that may be read (whatever they hold)
  int64_t nP;
  float *normal, *pt, *feature, *label, *dis, *nerr, *derr;   // level d (null: absent)
};
struct SignalLevel {   // the part of SignalArgs that differs from level to level
  int n;
  const uint64_t* key;
  const int *child, *dnum, *didx;
  float *normal, *pt, *feature, *label, *dis, *nerr, *derr;
};

// One wavefront per node; every level above the finest in one launch, the root first (its
// chain is the longest, the others run beside it).
// The two levels above the finest (at most 8 and 64 leaves to a node, and nine nodes in ten of
// the levels above the finest) go one THREAD per node in a launch of their own: a wavefront
// per node spends its time on the fixed cost of a node there, not on leaves.
// The table travels as a kernel argument (under 2 KB): no copy, no wait.
struct SignalLevels {
  int first_wave[kMaxD + 1];     // of level d among the levels that go one wavefront per node; [depth] = total
  int first_thread[kMaxD + 1];   // of level d among the levels that go one thread per node; [depth] = total
  SignalArgs common;             // the level fields are filled per node from `level`
  SignalLevel level[kMaxD - 1];
};
__device__ inline SignalArgs signal_args(const SignalLevels& L, int d) {
  SignalArgs a = L.common;
  const SignalLevel& l = L.level[d];
  a.d = d; a.n = l.n; a.key = l.key; a.child = l.child; a.dnum = l.dnum; a.didx = l.didx;
  a.normal = l.normal; a.pt = l.pt; a.feature = l.feature; a.label = l.label; a.dis = l.dis;
  a.nerr = l.nerr; a.derr = l.derr;
  return a;
}
__global__ __launch_bounds__(kBlock) void signal_kernel(const SignalLevels levels, int depth) {
  const int lane = threadIdx.x & 63;
  const int w = (int)((blockIdx.x * (unsigned)kBlock + threadIdx.x) >> 6);
  if (w >= levels.first_wave[depth]) return;
  int d = 0;
  while (w >= levels.first_wave[d + 1]) ++d;
  const SignalArgs a = signal_args(levels, d);
  const int i = w - levels.first_wave[d];
  __shared__ __attribute__((aligned(16))) float s_pass[kBlock / 64][kPassLeaves * kPassValues];
  float* lds = s_pass[threadIdx.x >> 6];
  const int64_t n = a.n;
  const bool has_normal = a.nrm_D != nullptr, has_pt = a.pt_D != nullptr;
  if (a.child[i] == -1) {   // empty: zero signal, no label, errors "infinite"
    if (lane == 0) {
      if (a.normal) for (int c = 0; c < 3; ++c) a.normal[c * n + i] = 0.0f;
      if (a.pt) for (int c = 0; c < 3; ++c) a.pt[c * n + i] = 0.0f;
      for (int c = 0; c < a.cf; ++c) a.feature[c * n + i] = 0.0f;
      if (a.label) a.label[i] = -1.0f;
      if (a.dis) for (int c = 0; c < a.ch_dis; ++c) a.dis[c * n + i] = 0.0f;
      if (a.nerr) a.nerr[i] = 1.0e20f;
      if (a.derr) a.derr[i] = 1.0e20f;
    }
    return;
  }
  const int j0 = a.didx[i], j1 = j0 + a.dnum[i];
  const float scale = (float)(1 << (a.depth - a.d));

  // sums of normals and points over the non-empty leaves, in leaf order
  float n_avg[3] = {0.0f, 0.0f, 0.0f}, last_n[3] = {0.0f, 0.0f, 0.0f}, pt_avg[3] = {0.0f, 0.0f, 0.0f};
  float sum6[6], last6[6];
  const int k0 = a.rank_D[j0], k1 = a.rank_D[j1];
  const int leaves = k1 - k0;
  const int64_t nP = a.nP;
  {
    const float* const rows6[6] = {has_normal ? a.nrm_P : nullptr, has_normal ? a.nrm_P + nP : nullptr,
        has_normal ? a.nrm_P + 2 * nP : nullptr, has_pt ? a.pt_P : nullptr, has_pt ? a.pt_P + nP : nullptr,
        has_pt ? a.pt_P + 2 * nP : nullptr};
    ordered_sums<6>(k0, k1, lane, lds, rows6, a.any_P, nP, sum6, last6);
  }
  for (int c = 0; c < 3; ++c) { n_avg[c] = sum6[c]; last_n[c] = last6[c]; pt_avg[c] = sum6[3 + c]; }
  if (has_normal) {
    float len = norm3(n_avg);
    if (len < 1.0e-6f) {
      for (int c = 0; c < 3; ++c) n_avg[c] = last_n[c];
      len = __fadd_rn(norm3(n_avg), 1.0e-30f);
    }
    for (int c = 0; c < 3; ++c) n_avg[c] = div_rn(n_avg[c], len);
    if (lane == 0) for (int c = 0; c < 3; ++c) a.normal[c * n + i] = n_avg[c];
  }
  const float count = leaves > 0 ? (float)leaves : 1.0e-30f;   // 1e-30f + 1 + 1 + ... in float
  if (has_pt) {
    const float div = __fmul_rn(count, scale);
    for (int c = 0; c < 3; ++c) pt_avg[c] = div_rn(pt_avg[c], div);
    if (lane == 0) for (int c = 0; c < 3; ++c) a.pt[c * n + i] = pt_avg[c];
  }
  for (int c0 = 0; c0 < a.cf; c0 += kPassValues) {   // features: eight channels per ordered pass
    float fsum[kPassValues], flast[kPassValues];
    const int nc = min(kPassValues, a.cf - c0);
    const float* rows8[kPassValues];
    for (int c = 0; c < kPassValues; ++c) rows8[c] = c < nc ? a.feat_P + (c0 + c) * nP : nullptr;
    ordered_sums<kPassValues>(k0, k1, lane, lds, rows8, a.any_P, nP, fsum, flast);
    if (lane == 0)
      for (int c = 0; c < kPassValues; ++c) if (c < nc) a.feature[(c0 + c) * n + i] = div_rn(fsum[c], count);
  }
  if (a.label) {
    // most frequent label (>= 0) of the non-empty leaves, the smallest one on a tie
    int mx = -1;
    for (int k = k0 + lane; k < k1; k += 64) mx = max(mx, (int)a.lab_P[k]);
    mx = wave_max_i(mx);
    int best = -1, best_cnt = 0;
    if (mx >= 0 && mx < kPassLeaves * kPassValues) {
      // the labels fit the wavefront's LDS block: one counting pass
      int* bins = reinterpret_cast<int*>(lds);
      for (int b = lane; b <= mx; b += 64) bins[b] = 0;
      __builtin_amdgcn_wave_barrier();
      for (int k = k0 + lane; k < k1; k += 64) {
        const int l = (int)a.lab_P[k];
        if (l >= 0) atomicAdd(&bins[l], 1);
      }
      __builtin_amdgcn_wave_barrier();
      for (int b = lane; b <= mx; b += 64) {   // ascending: a lane keeps the smallest label of its best count
        const int c = bins[b];
        if (c > best_cnt) { best_cnt = c; best = b; }
      }
      const int m = wave_max_i(best_cnt);
      best = wave_min_i((m > 0 && best_cnt == m) ? best : 0x7fffffff);
      best_cnt = m;
      __builtin_amdgcn_wave_barrier();
    } else if (mx >= 0) {
      // any label values: walk the distinct labels upwards
      int last = -1;
      for (;;) {
        int m = 0x7fffffff;
        for (int k = k0 + lane; k < k1; k += 64) {
          const int l = (int)a.lab_P[k];
          if (l > last && l < m) m = l;
        }
        m = wave_min_i(m);
        if (m == 0x7fffffff) break;
        int cnt = 0;
        for (int k = k0 + lane; k < k1; k += 64) cnt += ((int)a.lab_P[k] == m) ? 1 : 0;
        cnt = wave_sum_i(cnt);
        if (cnt > best_cnt) { best = m; best_cnt = cnt; }
        last = m;
      }
    }
    if (lane == 0) a.label[i] = best_cnt > 0 ? (float)best : -1.0f;
  }
  uint32_t bx, by, bz;
  morton_decode(a.key[i], a.d, &bx, &by, &bz);
  const float pt_base[3] = {(float)bx, (float)by, (float)bz};
  if (a.dis) {
    float dis_avg[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int c = 0; c < 3; ++c) {
      const float fract = __fsub_rn(pt_avg[c], pt_base[c]);
      dis_avg[c] = __fsub_rn(fract, 0.5f);
      if (has_normal) dis_avg[3] = __fadd_rn(dis_avg[3], __fmul_rn(dis_avg[c], n_avg[c]));
      else dis_avg[3] = 1.0f;
    }
    if (lane == 0) {
      if (!has_normal) {
        for (int c = 0; c < 3; ++c) a.dis[c * n + i] = dis_avg[c];
        a.dis[3 * n + i] = __fmul_rn(dis_avg[3], a.imul);
      } else {
        a.dis[i] = __fmul_rn(dis_avg[3], a.imul);
      }
    }
  }
  if (a.nerr) {
    float nm_err = 1.0e20f;
    if (a.calc_nerr && has_normal && a.d >= a.adp_layer) {
      nm_err = 0.0f;
      ordered_terms<3>(k0, k1, lane, lds,
          [&](int k, float* v) { for (int c = 0; c < 3; ++c) v[c] = a.nrm_P[c * nP + k]; },
          [&](const float* v) {
            for (int c = 0; c < 3; ++c) {
              const float tmp = __fsub_rn(v[c], n_avg[c]);
              nm_err = __fadd_rn(nm_err, __fmul_rn(tmp, tmp));
            }
          });
      nm_err = div_rn(nm_err, count);
    }
    if (lane == 0) a.nerr[i] = nm_err;
  }
  if (a.derr) {
    float err = 1.0e20f;
    if (a.calc_derr && has_pt && a.d >= a.adp_layer) {
      // largest distance of a leaf point from the plane ...
      float pt_avg1[3];
      for (int c = 0; c < 3; ++c) pt_avg1[c] = __fmul_rn(pt_avg[c], scale);
      float distance_max1 = -1.0f;
      for (int k = k0 + lane; k < k1; k += 64) {
        float dis = 0.0f;
        for (int c = 0; c < 3; ++c) dis = __fadd_rn(dis, __fmul_rn(__fsub_rn(a.pt_P[c * nP + k], pt_avg1[c]), n_avg[c]));
        distance_max1 = fmaxf(distance_max1, fabsf(dis));
      }
      distance_max1 = wave_max(distance_max1);
      // ... and of a vertex of the plane's polygon inside the node from its nearest leaf point
      float vtx[36];
      const int nv = intersect_cube(vtx, pt_avg, pt_base, n_avg);
      float distance_max2 = nv == 0 ? 5.0e10f : -1.0f;
      for (int k = 0; k < nv; ++k) {
        float vk[3];
        for (int c = 0; c < 3; ++c) vk[c] = __fmul_rn(vtx[3 * k + c], scale);
        // the correctly rounded root is monotonic: the smallest root is the root of the smallest square
        float sq_min = __builtin_inff();   // (no leaf, or only infinite squares: 1.0e30f as before)
        for (int k = k0 + lane; k < k1; k += 64) {
          float dis = 0.0f;
          for (int c = 0; c < 3; ++c) {
            const float ptc = __fsub_rn(a.pt_P[c * nP + k], vk[c]);
            dis = __fadd_rn(dis, __fmul_rn(ptc, ptc));
          }
          sq_min = fminf(sq_min, dis);
        }
        sq_min = wave_min(sq_min);
        const float distance_min = fminf(1.0e30f, sqrt_rn(sq_min));
        if (distance_min > distance_max2) distance_max2 = distance_min;
      }
      err = distance_max2 > distance_max1 ? distance_max2 : distance_max1;
    }
    if (lane == 0) a.derr[i] = err;
  }
}

// intersect_cube for one thread: the same vertices in the same order, kept in registers (every
// index below is a constant once the loops are unrolled; a vertex goes to slot `nv` through
// selects).  At most six edges of a cube are cut by a plane.
__device__ inline int intersect_cube_regs(float (&vx)[6], float (&vy)[6], float (&vz)[6], const float* pt,
    const float* pt_base, const float* normal) {
  constexpr float kC[8][3] = {{0, 0, 0}, {0, 0, 1}, {0, 1, 1}, {0, 1, 0}, {1, 0, 0}, {1, 0, 1}, {1, 1, 1}, {1, 1, 0}};
  constexpr int kE[12][2] = {{0, 1}, {1, 2}, {2, 3}, {3, 0}, {4, 5}, {5, 6}, {6, 7}, {7, 4}, {0, 4}, {1, 5}, {2, 6}, {3, 7}};
  float fval[8];
  unsigned cube_case = 0;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    float f = 0.0f;
#pragma unroll
    for (int j = 0; j < 3; ++j)
      f = __fadd_rn(f, __fmul_rn(__fsub_rn(__fadd_rn(kC[k][j], pt_base[j]), pt[j]), normal[j]));
    fval[k] = f;
    if (f < 0.0f) cube_case |= 1u << k;
  }
#pragma unroll
  for (int q = 0; q < 6; ++q) { vx[q] = 0.0f; vy[q] = 0.0f; vz[q] = 0.0f; }
  int nv = 0;
#pragma unroll
  for (int e = 0; e < 12; ++e) {
    const int v1 = kE[e][0], v2 = kE[e][1];
    if ((((cube_case >> v1) ^ (cube_case >> v2)) & 1u) == 0) continue;
    const float f1 = fval[v1], f2 = fval[v2];
    float df = __fsub_rn(f2, f1);
    if (df == 0) df = __fadd_rn(df, 1.0e-10f);
    const float t = div_rn(-f1, df);
    float p[3];
#pragma unroll
    for (int j = 0; j < 3; ++j)
      p[j] = __fadd_rn(__fadd_rn(kC[v1][j], __fmul_rn(t, __fsub_rn(kC[v2][j], kC[v1][j]))), pt_base[j]);
#pragma unroll
    for (int q = 0; q < 6; ++q)
      if (nv == q) { vx[q] = p[0]; vy[q] = p[1]; vz[q] = p[2]; }
    nv++;
  }
  return nv;
}

// One thread per node: calc_signal as the reference writes it, leaf after leaf (the sums are
// the same chains as in signal_kernel, so both forms give the same bits).
__global__ __launch_bounds__(kBlock) void signal_small_kernel(const SignalLevels levels, int depth) {
  const int t = blockIdx.x * kBlock + threadIdx.x;
  if (t >= levels.first_thread[depth]) return;
  int d = 0;
  while (t >= levels.first_thread[d + 1]) ++d;
  const SignalArgs a = signal_args(levels, d);
  const int i = t - levels.first_thread[d];
  const int64_t n = a.n;
  const bool has_normal = a.nrm_D != nullptr, has_pt = a.pt_D != nullptr;
  if (a.child[i] == -1) {   // empty: zero signal, no label, errors "infinite"
    if (a.normal) for (int c = 0; c < 3; ++c) a.normal[c * n + i] = 0.0f;
    if (a.pt) for (int c = 0; c < 3; ++c) a.pt[c * n + i] = 0.0f;
    for (int c = 0; c < a.cf; ++c) a.feature[c * n + i] = 0.0f;
    if (a.label) a.label[i] = -1.0f;
    if (a.dis) for (int c = 0; c < a.ch_dis; ++c) a.dis[c * n + i] = 0.0f;
    if (a.nerr) a.nerr[i] = 1.0e20f;
    if (a.derr) a.derr[i] = 1.0e20f;
    return;
  }
  const int j0 = a.didx[i], j1 = j0 + a.dnum[i];
  const float scale = (float)(1 << (a.depth - a.d));
  const int k0 = a.rank_D[j0], k1 = a.rank_D[j1];
  const int leaves = k1 - k0;
  const int64_t nP = a.nP;
  // A sweep over the node's leaves takes them eight at a time: the loads of a group are issued
  // together (the adds of a chain wait for one another, the loads need not), `leaf(nrm, pt)`
  // then sees the leaves in order.  An absent row reads a row that exists; its values are unused.
  const float* nrm_row = has_normal ? a.nrm_P : a.any_P;
  const float* pt_row = has_pt ? a.pt_P : a.any_P;
  const int64_t nrm_step = has_normal ? nP : 0, pt_step = has_pt ? nP : 0;
  auto sweep = [&](auto leaf) {
    for (int k = k0; k < k1; k += 8) {
      float vn[8][3], vp[8][3];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int kk = min(k + j, k1 - 1);
#pragma unroll
        for (int c = 0; c < 3; ++c) { vn[j][c] = nrm_row[c * nrm_step + kk]; vp[j][c] = pt_row[c * pt_step + kk]; }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (k + j < k1) leaf(vn[j], vp[j]);
    }
  };
  float n_avg[3] = {0.0f, 0.0f, 0.0f}, last_n[3] = {0.0f, 0.0f, 0.0f}, pt_avg[3] = {0.0f, 0.0f, 0.0f};
  sweep([&](const float* vn, const float* vp) {
    if (has_normal) for (int c = 0; c < 3; ++c) { n_avg[c] = __fadd_rn(n_avg[c], vn[c]); last_n[c] = vn[c]; }
    if (has_pt) for (int c = 0; c < 3; ++c) pt_avg[c] = __fadd_rn(pt_avg[c], vp[c]);
  });
  if (has_normal) {
    float len = norm3(n_avg);
    if (len < 1.0e-6f) {
      for (int c = 0; c < 3; ++c) n_avg[c] = last_n[c];
      len = __fadd_rn(norm3(n_avg), 1.0e-30f);
    }
    for (int c = 0; c < 3; ++c) n_avg[c] = div_rn(n_avg[c], len);
    for (int c = 0; c < 3; ++c) a.normal[c * n + i] = n_avg[c];
  }
  const float count = leaves > 0 ? (float)leaves : 1.0e-30f;   // 1e-30f + 1 + 1 + ... in float
  if (has_pt) {
    const float div = __fmul_rn(count, scale);
    for (int c = 0; c < 3; ++c) pt_avg[c] = div_rn(pt_avg[c], div);
    for (int c = 0; c < 3; ++c) a.pt[c * n + i] = pt_avg[c];
  }
  for (int c = 0; c < a.cf; ++c) {
    float f = 0.0f;
    for (int k = k0; k < k1; ++k) f = __fadd_rn(f, a.feat_P[c * nP + k]);
    a.feature[c * n + i] = div_rn(f, count);
  }
  if (a.label) {
    // most frequent label (>= 0) of the non-empty leaves, the smallest one on a tie
    int best = -1, best_cnt = 0;
    for (int u = k0; u < k1; ++u) {
      const int l = (int)a.lab_P[u];
      if (l < 0) continue;
      int cnt = 0;
      for (int k = k0; k < k1; ++k) cnt += ((int)a.lab_P[k] == l) ? 1 : 0;
      if (cnt > best_cnt || (cnt == best_cnt && l < best)) { best = l; best_cnt = cnt; }
    }
    a.label[i] = best_cnt > 0 ? (float)best : -1.0f;
  }
  uint32_t bx, by, bz;
  morton_decode(a.key[i], a.d, &bx, &by, &bz);
  const float pt_base[3] = {(float)bx, (float)by, (float)bz};
  if (a.dis) {
    float dis_avg[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int c = 0; c < 3; ++c) {
      const float fract = __fsub_rn(pt_avg[c], pt_base[c]);
      dis_avg[c] = __fsub_rn(fract, 0.5f);
      if (has_normal) dis_avg[3] = __fadd_rn(dis_avg[3], __fmul_rn(dis_avg[c], n_avg[c]));
      else dis_avg[3] = 1.0f;
    }
    if (!has_normal) {
      for (int c = 0; c < 3; ++c) a.dis[c * n + i] = dis_avg[c];
      a.dis[3 * n + i] = __fmul_rn(dis_avg[3], a.imul);
    } else {
      a.dis[i] = __fmul_rn(dis_avg[3], a.imul);
    }
  }
  const bool do_nerr = a.nerr && a.calc_nerr && has_normal && a.d >= a.adp_layer;
  const bool do_derr = a.derr && a.calc_derr && has_pt && a.d >= a.adp_layer;
  float nm_err = 0.0f, distance_max1 = -1.0f;
  float pt_avg1[3];
  for (int c = 0; c < 3; ++c) pt_avg1[c] = __fmul_rn(pt_avg[c], scale);
  if (do_nerr || do_derr) {
    // one sweep for both: the chain of the normal error, and the largest distance of a leaf
    // point from the plane
    sweep([&](const float* vn, const float* vp) {
      if (do_nerr)
        for (int c = 0; c < 3; ++c) {
          const float tmp = __fsub_rn(vn[c], n_avg[c]);
          nm_err = __fadd_rn(nm_err, __fmul_rn(tmp, tmp));
        }
      if (do_derr) {
        float dis = 0.0f;
        for (int c = 0; c < 3; ++c) dis = __fadd_rn(dis, __fmul_rn(__fsub_rn(vp[c], pt_avg1[c]), n_avg[c]));
        distance_max1 = fmaxf(distance_max1, fabsf(dis));
      }
    });
  }
  if (a.nerr) a.nerr[i] = do_nerr ? div_rn(nm_err, count) : 1.0e20f;
  if (a.derr) {
    float err = 1.0e20f;
    if (do_derr) {
      // ... and of a vertex of the plane's polygon inside the node from its nearest leaf point:
      // every vertex in the same sweep.  The correctly rounded root is monotonic: the smallest
      // root is the root of the smallest square.
      float vx[6], vy[6], vz[6], sq_min[6];
      const int nv = intersect_cube_regs(vx, vy, vz, pt_avg, pt_base, n_avg);
#pragma unroll
      for (int q = 0; q < 6; ++q) {
        vx[q] = __fmul_rn(vx[q], scale); vy[q] = __fmul_rn(vy[q], scale); vz[q] = __fmul_rn(vz[q], scale);
        sq_min[q] = __builtin_inff();   // (no leaf, or only infinite squares: 1.0e30f as the reference starts from)
      }
      if (nv > 0)
        sweep([&](const float*, const float* vp) {
#pragma unroll
          for (int q = 0; q < 6; ++q) {
            const float px = __fsub_rn(vp[0], vx[q]), py = __fsub_rn(vp[1], vy[q]), pz = __fsub_rn(vp[2], vz[q]);
            const float dis = __fadd_rn(__fadd_rn(__fadd_rn(0.0f, __fmul_rn(px, px)), __fmul_rn(py, py)), __fmul_rn(pz, pz));
            sq_min[q] = fminf(sq_min[q], dis);
          }
        });
      float distance_max2 = nv == 0 ? 5.0e10f : -1.0f;
#pragma unroll
      for (int q = 0; q < 6; ++q) {
        const float distance_min = fminf(1.0e30f, sqrt_rn(sq_min[q]));
        if (q < nv && distance_min > distance_max2) distance_max2 = distance_min;
      }
      err = distance_max2 > distance_max1 ? distance_max2 : distance_max1;
    }
    a.derr[i] = err;
  }
}

// ---- extrapolate_signal (octree.cpp:666-806): one thread per sibling group ------------------
// OctreeParser::key2xyz<float> (octree_parser.cpp:151-165) on the builder's keys: they are still
// Morton codes at this point, and with the key2xyz option the reference reads them as packed
// 16-bit fields all the same -- reproduced as it is.
__device__ inline void node_xyz(float* xyz, uint64_t key, int depth, int packed) {
  if (packed) {
    for (int c = 0; c < 3; ++c) xyz[c] = (float)((key >> (16 * c)) & 0xffff);
  } else {
    uint32_t x, y, z;
    morton_decode(key, depth, &x, &y, &z);
    xyz[0] = (float)x; xyz[1] = (float)y; xyz[2] = (float)z;
  }
}

struct ExtrapolateArgs {
  int n, cf, has_dis, d, key2xyz;
  int per_octree;     // nodes of one octree on this level where the level is full (else n)
  float imul;
  const uint64_t* key;
  const int* child;
  float *normal, *feature, *label, *dis;   // level d, null: absent
};
__global__ void extrapolate_kernel(ExtrapolateArgs a) {
  const int g = blockIdx.x * blockDim.x + threadIdx.x;
  const int i_base = g * 8;
  if (i_base >= a.n) return;
  const int64_t n = a.n;
  int occ = 0, cnt = 0;
  for (int j = 0; j < 8; ++j)
    if (a.child[i_base + j] != -1) { occ |= 1 << j; ++cnt; }
  if (occ == 255) return;   // nothing empty
  if (cnt == 0) {
    // No non-empty sibling (happens on the last full layer only): normals, features and labels
    // stay as they are; the displacement comes from the nearest non-empty node of the level
    // (L1 distance, the first one on a tie), octree.cpp:776-803.  In a batch "the level" is
    // the level of the node's own octree: on a full layer its nodes are one block of the row.
    if (!(a.has_dis && a.dis)) return;
    const int j_first = (i_base / a.per_octree) * a.per_octree, j_end = min(a.n, j_first + a.per_octree);
    for (int id = 0; id < 8; ++id) {
      const int i = i_base + id;
      float pti[3], ptj[3], dis_min = 1.0e30f;
      node_xyz(pti, a.key[i], a.d, a.key2xyz);
      int j_min = -1;
      for (int j = j_first; j < j_end; ++j) {
        if (a.child[j] == -1) continue;
        node_xyz(ptj, a.key[j], a.d, a.key2xyz);
        const float dd = __fadd_rn(__fadd_rn(fabsf(__fsub_rn(pti[0], ptj[0])), fabsf(__fsub_rn(pti[1], ptj[1]))),
            fabsf(__fsub_rn(pti[2], ptj[2])));
        if (dd < dis_min) { dis_min = dd; j_min = j; }
      }
      if (j_min < 0) continue;
      float dis = a.dis[j_min];
      node_xyz(ptj, a.key[j_min], a.d, a.key2xyz);
      if (a.normal)
        for (int c = 0; c < 3; ++c)
          dis = __fadd_rn(dis, __fmul_rn(__fmul_rn(a.normal[c * n + j_min], __fsub_rn(ptj[c], pti[c])), a.imul));
      if (dis > 0.0f) dis = 2.0f;
      if (dis < 0.0f) dis = -2.0f;
      a.dis[i] = dis;
    }
    return;
  }
  const float count = (float)cnt;       // 1e-30f + 1 + 1 + ...
  float n_avg[3] = {0.0f, 0.0f, 0.0f};
  if (a.normal) {
    for (int j = 0; j < 8; ++j) {
      if (!((occ >> j) & 1)) continue;
      for (int c = 0; c < 3; ++c) n_avg[c] = __fadd_rn(n_avg[c], a.normal[c * n + i_base + j]);
    }
    const float ilen = div_rn(1.0f, __fadd_rn(norm3(n_avg), 1.0e-30f));
    for (int c = 0; c < 3; ++c) n_avg[c] = __fmul_rn(n_avg[c], ilen);
    for (int j = 0; j < 8; ++j)
      if (!((occ >> j) & 1))
        for (int c = 0; c < 3; ++c) a.normal[c * n + i_base + j] = n_avg[c];
  }
  for (int c = 0; c < a.cf; ++c) {
    float f_avg = 0.0f;
    for (int j = 0; j < 8; ++j)
      if ((occ >> j) & 1) f_avg = __fadd_rn(f_avg, a.feature[c * n + i_base + j]);
    f_avg = div_rn(f_avg, count);
    for (int j = 0; j < 8; ++j)
      if (!((occ >> j) & 1)) a.feature[c * n + i_base + j] = f_avg;
  }
  if (a.label) {
    // each empty node takes the most frequent label of ALL eight siblings as they stand when
    // its turn comes (earlier empty siblings already carry theirs), smallest label on a tie
    int lab[8];
    for (int j = 0; j < 8; ++j) lab[j] = (int)a.label[i_base + j];
    for (int id = 0; id < 8; ++id) {
      if ((occ >> id) & 1) continue;
      int best = -1, best_cnt = 0;
      for (int u = 0; u < 8; ++u) {
        if (lab[u] < 0) continue;
        int c = 0;
        for (int w = 0; w < 8; ++w) c += lab[w] == lab[u] ? 1 : 0;
        if (c > best_cnt || (c == best_cnt && lab[u] < best)) { best = lab[u]; best_cnt = c; }
      }
      if (best_cnt > 0) { lab[id] = best; a.label[i_base + id] = (float)best; }
    }
  }
  if (a.has_dis && a.dis) {
    for (int id = 0; id < 8; ++id) {
      if ((occ >> id) & 1) continue;
      float dis = 0.0f;
      for (int j = 0; j < 8; ++j) {
        if (!((occ >> j) & 1)) continue;
        dis = __fadd_rn(dis, a.dis[i_base + j]);
        if (a.normal)
          for (int c = 0; c < 3; ++c) {
            const float xj = (float)((j >> (2 - c)) & 1), xi = (float)((id >> (2 - c)) & 1);
            dis = __fadd_rn(dis, __fmul_rn(__fmul_rn(a.normal[c * n + i_base + j], __fsub_rn(xj, xi)), a.imul));
          }
      }
      dis = div_rn(dis, count);
      if (dis > 3.0f) dis = 3.0f;
      if (dis < -3.0f) dis = -3.0f;
      if (fabsf(dis) < 1.0f) {
        unsigned cube_cases = 0;
        for (int k = 0; k < 8; ++k) {
          float fval = dis;
          for (int j = 0; j < 3; ++j)
            fval = __fadd_rn(fval, __fmul_rn(__fmul_rn(__fsub_rn(0.5f, kCorner[k][j]), n_avg[j]), a.imul));
          if (fval < 0) cube_cases |= 1u << k;
        }
        if (cube_cases != 255 && cube_cases != 0) dis = dis < 0 ? -1.0f : 1.0f;
      }
      a.dis[i_base + id] = dis;
    }
  }
}

// ---- trim_octree (octree.cpp:1004-1135) ------------------------------------------------------
enum { kDrop = 0, kDropChildren = 1, kKeep = 2 };

// one thread per node of level d-1: flags of its children at level d.  The test "was any
// non-empty node of the level kept" is taken per octree (trim_octree runs on one octree at a
// time, and a batch is trimmed octree by octree before merge_octrees joins them): the octree
// of a node is the index in the top 16 bits of its key, and `any_kept` / `best` hold one entry
// per octree.
__global__ __launch_bounds__(kBlock) void trim_flag_kernel(int* __restrict__ drop_d, const int* __restrict__ drop_p,
    const int* __restrict__ child_p, const int* __restrict__ child_d, const uint64_t* __restrict__ key_p,
    const float* __restrict__ nerr, const float* __restrict__ derr, int n_p, int has_dis, float th_dist, float th_norm,
    int* __restrict__ any_kept, unsigned long long* __restrict__ best) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  const int c = i < n_p ? child_p[i] : -1;
  const bool active = c != -1;
  const int b = active ? (int)(key_p[i] >> 48) : -1;
  // In case no non-empty node of the octree's level is kept, the candidate that is kept all the
  // same: a non-empty child of a kept parent with the largest normal error, the first one on a
  // tie (octree.cpp:1057-1073), as (error bits, ~index) so that one atomic maximum finds it.
  unsigned long long cand = 0;
  if (active) {
    const bool parent_kept = drop_p == nullptr || drop_p[i] == kKeep;
    bool kept = false;
    for (int j = 0; j < 8; ++j) {
      const int idx = c * 8 + j;
      int f = kKeep;
      const float e = nerr[idx];
      if (parent_kept) {
        if ((!has_dis || derr[idx] < th_dist) && e < th_norm) f = kDropChildren;
      } else {
        f = kDrop;
      }
      drop_d[idx] = f;
      const bool inner = child_d[idx] != -1;
      kept = kept || (f == kKeep && inner);
      if (parent_kept && inner && e > -1.0f) {
        const unsigned long long v = ((unsigned long long)__float_as_uint(e) << 32) | (unsigned long long)(0xffffffffu - (unsigned)idx);
        cand = v > cand ? v : cand;
      }
    }
    if (kept) any_kept[b] = 1;
  }
  // one atomic per wavefront where its nodes are of one octree (nearly always)
  const unsigned long long act = __ballot(active);
  if (act == 0) return;
  const int b0 = __builtin_amdgcn_readlane(b, __builtin_ctzll(act));
  if (__all(!active || b == b0)) {
    unsigned long long m = cand;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const unsigned long long other = __shfl_xor(m, o, 64);
      m = other > m ? other : m;
    }
    // both words only grow: a candidate that an earlier value already beats, or an octree that
    // already has a kept node, needs no atomic (a stale read costs one atomic, never a result)
    if ((threadIdx.x & 63) == 0 && m != 0 && any_kept[b0] == 0 && m > best[b0]) atomicMax(best + b0, m);
  } else if (cand != 0) {
    atomicMax(best + b, cand);
  }
}
// An octree without a kept non-empty node on the level keeps its candidate; without a candidate
// it is the octree's first node of the level (max_idx starts at 0, octree.cpp:1059).  One thread
// per octree.
__global__ void trim_fix_kernel(int* __restrict__ drop_d, const unsigned long long* __restrict__ best,
    const int* __restrict__ any_kept, const uint64_t* __restrict__ key_d, int n_d, int n_octrees) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= n_octrees || any_kept[b]) return;
  const unsigned long long v = best[b];
  int idx;
  if (v != 0) {
    idx = (int)(0xffffffffu - (unsigned)(v & 0xffffffffull));
  } else {   // the level's keys ascend with the octree index on top: first node of octree b
    int lo = 0, hi = n_d;
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if ((int)(key_d[mid] >> 48) < b) lo = mid + 1; else hi = mid;
    }
    if (lo >= n_d || (int)(key_d[lo] >> 48) != b) return;   // the octree has no node here
    idx = lo;
  }
  drop_d[idx] = kKeep;
}

// New positions of the kept nodes and new child links of every trimmed level in three launches
// (tile counts, their prefix per level, ranks): a node stays unless its flag is kDrop, and keeps
// its children if it is kKeep and has any.
struct TrimScanLevel {
  int n, first_tile;
  const int* drop; const int* child;
  int* pos;        // new index, -1: dropped
  int* nchild;     // new child link, -1: none
  int* total_keep; int* total_link;
};
struct TrimScanLevels {
  int n_levels, n_tiles;
  int* tile_count;     // [2][n_tiles]: kept nodes, kept links
  TrimScanLevel level[kMaxD];
};
__device__ inline int trim_scan_level(const TrimScanLevels& t, int tile) {
  int l = 0;
  while (l + 1 < t.n_levels && tile >= t.level[l + 1].first_tile) ++l;
  return l;
}
__global__ __launch_bounds__(kBlock) void trim_count_kernel(const TrimScanLevels t) {
  const TrimScanLevel& a = t.level[trim_scan_level(t, blockIdx.x)];
  const int base = ((int)blockIdx.x - a.first_tile) * kScanTile + threadIdx.x * kScanItems;
  int ck = 0, cl = 0;
#pragma unroll
  for (int j = 0; j < kScanItems; ++j) {
    if (base + j >= a.n) continue;
    const int f = a.drop[base + j];
    ck += f != kDrop ? 1 : 0;
    cl += (f == kKeep && a.child[base + j] != -1) ? 1 : 0;
  }
  int tk, tl;
  block_exclusive_scan(ck, &tk);
  block_exclusive_scan(cl, &tl);
  if (threadIdx.x == 0) { t.tile_count[blockIdx.x] = tk; t.tile_count[t.n_tiles + blockIdx.x] = tl; }
}
// one workgroup per (level, count): tile counts -> exclusive offsets within the level, and the total
__global__ __launch_bounds__(kBlock) void trim_tiles_kernel(const TrimScanLevels t) {
  const int l = blockIdx.x >> 1, which = blockIdx.x & 1;
  const TrimScanLevel& a = t.level[l];
  const int n_tiles = (l + 1 < t.n_levels ? t.level[l + 1].first_tile : t.n_tiles) - a.first_tile;
  int* tc = t.tile_count + which * t.n_tiles + a.first_tile;
  __shared__ int carry;
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  for (int start = 0; start < n_tiles; start += kBlock) {
    const int i = start + threadIdx.x;
    const int v = i < n_tiles ? tc[i] : 0;
    int total;
    const int ex = block_exclusive_scan(v, &total);
    const int c = carry;
    if (i < n_tiles) tc[i] = c + ex;
    __syncthreads();
    if (threadIdx.x == 0) carry = c + total;
    __syncthreads();
  }
  if (threadIdx.x == 0) *(which ? a.total_link : a.total_keep) = carry;
}
__global__ __launch_bounds__(kBlock) void trim_apply_kernel(const TrimScanLevels t) {
  const TrimScanLevel& a = t.level[trim_scan_level(t, blockIdx.x)];
  const int base = ((int)blockIdx.x - a.first_tile) * kScanTile + threadIdx.x * kScanItems;
  bool fk[kScanItems], fl[kScanItems];
  int ck = 0, cl = 0;
#pragma unroll
  for (int j = 0; j < kScanItems; ++j) {
    fk[j] = fl[j] = false;
    if (base + j < a.n) {
      const int f = a.drop[base + j];
      fk[j] = f != kDrop;
      fl[j] = f == kKeep && a.child[base + j] != -1;
    }
    ck += fk[j] ? 1 : 0;
    cl += fl[j] ? 1 : 0;
  }
  int total;
  int rk = t.tile_count[blockIdx.x] + block_exclusive_scan(ck, &total);
  int rl = t.tile_count[t.n_tiles + blockIdx.x] + block_exclusive_scan(cl, &total);
#pragma unroll
  for (int j = 0; j < kScanItems; ++j) {
    if (base + j < a.n) {
      a.pos[base + j] = fk[j] ? rk : -1;
      a.nchild[base + j] = fl[j] ? rl : -1;
    }
    rk += fk[j] ? 1 : 0;
    rl += fl[j] ? 1 : 0;
  }
}

// ---- serialization (octree.cpp:907-956) -----------------------------------------------------
// every level in one launch: the table is a kernel argument (about 2 KB)
struct GatherLevel {
  int n_old, n_new;
  const int* pos;            // new index of an old node, -1: dropped; null: identity
  const int* nchild;         // new child link; null: the old one
  const uint64_t* key; const int* child;
  const float *normal, *dis, *feature, *label, *pt;   // per-level signals (null: not stored)
  uint64_t* key_out; int* child_out; float* feature_out; float* label_out; float* split_out;
};
struct GatherLevels {
  int first_block[kMaxD + 1];   // of level d; [depth + 1] = all blocks
  int depth, key2xyz, key_channel, adaptive_split;
  int cn, ch_dis, cf, cp;
  GatherLevel level[kMaxD];
};
__global__ __launch_bounds__(kBlock) void gather_kernel(const GatherLevels g) {
  int d = 0;
  while (d < g.depth && (int)blockIdx.x >= g.first_block[d + 1]) ++d;
  const GatherLevel& a = g.level[d];
  const int i = ((int)blockIdx.x - g.first_block[d]) * kBlock + threadIdx.x;
  if (i >= a.n_old) return;
  const int k = a.pos ? a.pos[i] : i;
  if (k < 0) return;
  const int64_t no = a.n_old, nn = a.n_new;
  uint64_t key = a.key[i];
  if (g.key2xyz) {  // Octree::key_to_xyz, octree.cpp:1137-1156
    uint32_t x, y, z;
    morton_decode(key, d, &x, &y, &z);
    // the octree index of a batch stays in the top 16 bits (merge_octrees.cpp:126-131)
    key = (uint64_t)(x & 0xffff) | ((uint64_t)(y & 0xffff) << 16) | ((uint64_t)(z & 0xffff) << 32) | (key & 0xffff000000000000ull);
  }
  a.key_out[k] = key;
  if (g.key_channel == 2) a.key_out[nn + k] = 0;
  const int ch = a.nchild ? a.nchild[i] : a.child[i];
  a.child_out[k] = ch;
  float* f = a.feature_out;
  float nsum = 0.0f;
  if (f) {
    for (int c = 0; c < g.cn; ++c) { const float v = a.normal[c * no + i]; f[c * nn + k] = v; if (c < 3) nsum = __fadd_rn(nsum, fabsf(v)); }
    f += g.cn * nn;
    for (int c = 0; c < g.ch_dis; ++c) f[c * nn + k] = a.dis[c * no + i];
    f += g.ch_dis * nn;
    for (int c = 0; c < g.cf; ++c) f[c * nn + k] = a.feature[c * no + i];
    f += g.cf * nn;
    for (int c = 0; c < g.cp; ++c) f[c * nn + k] = a.pt[c * no + i];
  }
  if (a.label_out) a.label_out[k] = a.label[i];
  if (a.split_out) {  // calc_split_label, octree.cpp:1158-1178
    float s = 1.0f;
    if (ch == -1) s = (g.adaptive_split && nsum != 0.0f) ? 2.0f : 0.0f;
    a.split_out[k] = s;
  }
}
struct HeaderWords { uint32_t w[OCNN_HEADER_BYTES / 4]; };
__global__ void header_kernel(uint32_t* __restrict__ dst, const HeaderWords h) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < OCNN_HEADER_BYTES / 4) dst[i] = h.w[i];
}

inline size_t al(size_t v) { return (v + 255) & ~(size_t)255; }

}  // namespace

int adaptive_finish(const AdaptiveInput& in, ocnn_alloc_fn alloc, void* alloc_ctx, void* info_out, void** blob_out,
    hipStream_t s) {
  const Info& o0 = in.info0;
  const ocnn_build_params& P = in.params;
  const int D = o0.depth, fl = o0.full_layer;
  const int cn = in.ch_normal, cf = in.ch_feature, ch_dis = in.ch_dis, cp = in.has_pt ? 3 : 0;
  const bool adaptive = P.adaptive != 0;
  const float imul = 2.0f / sqrtf(3.0f);
  OCNN_REQUIRE(D <= 16, OCNN_E_BADARG, "depth %d", D);

  // ---- scratch layout
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t v = off; off += al(bytes); return v; };
  size_t o_normal[kMaxD], o_dis[kMaxD], o_feature[kMaxD], o_label[kMaxD], o_pt[kMaxD], o_nerr[kMaxD], o_derr[kMaxD];
  size_t o_dnum[kMaxD], o_didx[kMaxD], o_drop[kMaxD], o_pos[kMaxD], o_nchild[kMaxD];
  int max_n = 1;
  for (int d = 0; d <= D; ++d) {
    const size_t n = (size_t)o0.nnum[d] + 1;
    if (o0.nnum[d] > max_n) max_n = o0.nnum[d];
    o_normal[d] = take(4 * 3 * n); o_dis[d] = take(4 * 4 * n); o_feature[d] = take(4 * (size_t)(cf > 0 ? cf : 1) * n);
    o_label[d] = take(4 * n); o_pt[d] = take(4 * 3 * n); o_nerr[d] = take(4 * n); o_derr[d] = take(4 * n);
    o_dnum[d] = take(4 * n); o_didx[d] = take(4 * n); o_drop[d] = take(4 * n); o_pos[d] = take(4 * n);
    o_nchild[d] = take(4 * n);
  }
  const size_t nDp = (size_t)o0.nnum[D] + 1;
  const size_t nP = ((size_t)o0.nnum[D] + 3) & ~(size_t)3;   // packed rows in whole 16-byte units
  const size_t o_rank = take(4 * nDp), o_nrmP = take(4 * 3 * nP + 16), o_ptP = take(4 * 3 * nP + 16);
  const size_t o_featP = take(4 * (size_t)(cf > 0 ? cf : 1) * nP + 16), o_labP = take(4 * nP + 16);
  size_t level_tiles = 0;
  for (int d = 0; d <= D; ++d) level_tiles += (size_t)scan_tiles(o0.nnum[d]);
  const size_t o_scan = take(std::max(scan_scratch_bytes(max_n), sizeof(int) * 2 * (level_tiles + 1)));
  const int B = o0.batch_size;
  OCNN_REQUIRE(B >= 1 && B <= 65535, OCNN_E_BADARG, "batch size %d", B);
  const size_t o_counts = take(sizeof(int) * 64);      // [0..16] kept nodes, [17..33] kept links
  const size_t o_any = take(sizeof(int) * kMaxD * (size_t)B);                    // [d * B + octree]
  const size_t o_best = take(sizeof(unsigned long long) * kMaxD * (size_t)B);    // [d * B + octree]
  const size_t o_hdr = take(256);   // end of the block that starts cleared
  char* ws = static_cast<char*>(alloc(off, alloc_ctx));
  OCNN_REQUIRE(ws, OCNN_E_BADARG, "the allocator returned no memory for %zu bytes of scratch", off);
  OCNN_REQUIRE((reinterpret_cast<uintptr_t>(ws) & 7) == 0, OCNN_E_BADARG, "scratch not 8-byte aligned");
  fill_kernel<<<blocks_for((int64_t)((o_hdr - o_counts) / 4)), kBlock, 0, s>>>(reinterpret_cast<float*>(ws + o_counts),
      (int64_t)((o_hdr - o_counts) / 4), 0.0f);

  // ---- per-level views; the finest level lives in the first-stage blob
  char* b0 = in.blob0;
  const uint64_t* key[kMaxD]; const int* child[kMaxD];
  float *normal[kMaxD], *dis[kMaxD], *feature[kMaxD], *label[kMaxD], *pt[kMaxD], *nerr[kMaxD], *derr[kMaxD];
  int *dnum[kMaxD], *didx[kMaxD], *drop[kMaxD], *pos[kMaxD], *nchild[kMaxD];
  const bool has_label = in.has_label != 0;
  for (int d = 0; d <= D; ++d) {
    key[d] = reinterpret_cast<const uint64_t*>(b0 + o0.ptr_dis(OCNN_KEY, d));
    child[d] = reinterpret_cast<const int*>(b0 + o0.ptr_dis(OCNN_CHILD, d));
    normal[d] = cn ? reinterpret_cast<float*>(ws + o_normal[d]) : nullptr;
    dis[d] = ch_dis ? reinterpret_cast<float*>(ws + o_dis[d]) : nullptr;
    feature[d] = cf ? reinterpret_cast<float*>(ws + o_feature[d]) : nullptr;
    label[d] = has_label ? reinterpret_cast<float*>(ws + o_label[d]) : nullptr;
    pt[d] = cp ? reinterpret_cast<float*>(ws + o_pt[d]) : nullptr;
    nerr[d] = reinterpret_cast<float*>(ws + o_nerr[d]);
    derr[d] = reinterpret_cast<float*>(ws + o_derr[d]);
    dnum[d] = reinterpret_cast<int*>(ws + o_dnum[d]); didx[d] = reinterpret_cast<int*>(ws + o_didx[d]);
    drop[d] = reinterpret_cast<int*>(ws + o_drop[d]); pos[d] = reinterpret_cast<int*>(ws + o_pos[d]);
    nchild[d] = reinterpret_cast<int*>(ws + o_nchild[d]);
  }
  {
    const int64_t nD = o0.nnum[D];
    float* f = reinterpret_cast<float*>(b0 + o0.ptr_dis(OCNN_FEATURE, D));
    if (cn) { normal[D] = f; f += cn * nD; }
    if (ch_dis) { dis[D] = f; f += ch_dis * nD; }
    if (cf) { feature[D] = f; f += cf * nD; }
    if (cp) { pt[D] = f; f += cp * nD; }
    if (has_label) label[D] = reinterpret_cast<float*>(b0 + o0.ptr_dis(OCNN_LABEL, D));
  }
  int* d_counts = reinterpret_cast<int*>(ws + o_counts);
  int* d_any = reinterpret_cast<int*>(ws + o_any);
  unsigned long long* d_best = reinterpret_cast<unsigned long long*>(ws + o_best);

  // ---- covered ranges and signals of every depth
  {
    const int nD1 = D >= 1 ? o0.nnum[D - 1] : 0;
    if (nD1 > 0)
      cover_first_kernel<<<blocks_for(nD1), kBlock, 0, s>>>(dnum[D - 1], didx[D - 1], child[D - 1], nerr[D], derr[D], nD1);
    int d = D - 2;
    for (; d >= 0 && o0.nnum[d] > 8192; --d)
      cover_kernel<<<blocks_for(o0.nnum[d]), kBlock, 0, s>>>(dnum[d], didx[d], child[d], dnum[d + 1], didx[d + 1], o0.nnum[d]);
    if (d >= 0) {
      CoverTop t;
      memset(&t, 0, sizeof(t));
      t.d_top = d;
      for (int q = 0; q <= d + 1; ++q) { t.n[q] = o0.nnum[q]; t.dnum[q] = dnum[q]; t.didx[q] = didx[q]; t.child[q] = child[q]; }
      cover_top_kernel<<<1, 1024, 0, s>>>(t);
    }
  }
  OCNN_LAUNCH_OK("cover");
  int* rank_D = reinterpret_cast<int*>(ws + o_rank);
  float* nrm_P = reinterpret_cast<float*>(ws + o_nrmP);
  float* pt_P = reinterpret_cast<float*>(ws + o_ptP);
  float* feat_P = reinterpret_cast<float*>(ws + o_featP);
  float* lab_P = reinterpret_cast<float*>(ws + o_labP);
  {
    LeafPred lp{child[D]};
    LeafPack lo{rank_D, (int64_t)o0.nnum[D], (int64_t)nP, cf, normal[D], pt[D], feature[D], label[D], nrm_P, pt_P,
        feat_P, lab_P};
    hipError_t e = flag_scan(lp, lo, (int64_t)o0.nnum[D], reinterpret_cast<int*>(ws + o_scan), rank_D + o0.nnum[D], s);
    OCNN_REQUIRE(e == hipSuccess, OCNN_E_HIP, "leaf scan: %s", hipGetErrorString(e));
  }
  {
    SignalLevels L;
    memset(&L, 0, sizeof(L));
    static_assert(sizeof(SignalLevels) <= 2048, "the level table is passed as a kernel argument");
    int waves = 0, threads = 0;
    const int d_small = D - 2 > 0 ? D - 2 : 0;   // levels from here on: one thread per node
    {
      SignalArgs& a = L.common;
      a.depth = D; a.nD = o0.nnum[D]; a.cf = cf; a.ch_dis = ch_dis;
      a.adp_layer = o0.adp_layer; a.calc_nerr = adaptive && cn; a.calc_derr = adaptive && P.node_dis && cn;
      a.imul = imul;
      a.child_D = child[D]; a.nrm_D = normal[D]; a.pt_D = pt[D]; a.feat_D = feature[D]; a.lab_D = label[D];
      a.rank_D = rank_D; a.nrm_P = nrm_P; a.pt_P = pt_P; a.feat_P = feat_P; a.lab_P = lab_P; a.nP = (int64_t)nP;
      a.any_P = nrm_P;   // allocated whether or not the cloud has normals
    }
    for (int d = 0; d < D; ++d) {
      SignalLevel& l = L.level[d];
      l.n = o0.nnum[d];
      l.key = key[d]; l.child = child[d]; l.dnum = dnum[d]; l.didx = didx[d];
      l.normal = normal[d]; l.pt = pt[d]; l.feature = feature[d]; l.label = label[d]; l.dis = dis[d];
      l.nerr = nerr[d]; l.derr = derr[d];
      L.first_wave[d] = waves;
      L.first_thread[d] = threads;
      if (d < d_small) waves += l.n; else threads += l.n;
    }
    for (int d = D; d <= kMaxD; ++d) { L.first_wave[d] = waves; L.first_thread[d] = threads; }
    if (waves > 0) signal_kernel<<<blocks_for((int64_t)waves * 64), kBlock, 0, s>>>(L, D);
    if (threads > 0) signal_small_kernel<<<blocks_for(threads), kBlock, 0, s>>>(L, D);
  }
  OCNN_LAUNCH_OK("signal");

  // ---- extrapolation into the empty nodes (before trimming, as Octree::build does)
  if (P.extrapolate) {
    for (int d = D; d >= fl; --d) {
      ExtrapolateArgs a;
      a.n = o0.nnum[d]; a.cf = cf; a.has_dis = ch_dis != 0; a.imul = imul; a.d = d; a.key2xyz = P.key2xyz ? 1 : 0;
      a.per_octree = (d <= fl && a.n >= B) ? a.n / B : (a.n > 0 ? a.n : 1);
      a.key = key[d]; a.child = child[d]; a.normal = normal[d]; a.feature = feature[d]; a.label = label[d]; a.dis = dis[d];
      extrapolate_kernel<<<blocks_for((a.n + 7) / 8), kBlock, 0, s>>>(a);
    }
    OCNN_LAUNCH_OK("extrapolate");
  }

  // ---- trimming
  Info o = o0;
  o.adp_layer = P.adp_depth;
  o.is_adaptive = adaptive ? 1 : 0;
  o.has_node_dis = P.node_dis ? 1 : 0;
  o.key2xyz = P.key2xyz ? 1 : 0;
  o.extrapolate = P.extrapolate ? 1 : 0;
  o.save_pts = P.save_pts ? 1 : 0;
  o.set_property(OCNN_KEY, (P.key2xyz && D > 8) ? 2 : 1, -1);
  if (P.split_label) o.set_property(OCNN_SPLIT, 1, -1); else o.set_channel(OCNN_SPLIT, 0);
  const int out_dis = P.node_dis ? ch_dis : 0, out_pt = P.save_pts ? cp : 0;
  o.set_channel(OCNN_FEATURE, cn + out_dis + cf + out_pt);
  o.set_location(OCNN_FEATURE, -1);
  if (has_label) o.set_property(OCNN_LABEL, 1, -1);
  if (in.merged) {   // the header of merge_octrees (merge_octrees.cpp:92-107): neighbour tables at every depth
    OCNN_REQUIRE(o.channel(OCNN_KEY) == 1, OCNN_E_UNSUPPORTED, "octree_batch of two-channel keys (key2xyz with depth > 8)");
    o.set_property(OCNN_NEIGH, 8, -1);
  }
  const int A = o.adp_layer;
  if (adaptive) {
    OCNN_REQUIRE(A >= 1 && A <= D, OCNN_E_BADARG, "adp_depth %d", A);
    for (int d = A; d <= D; ++d) {
      const int n_p = o0.nnum[d - 1];
      const int* drop_p = d - 1 >= A ? drop[d - 1] : nullptr;
      int* any_kept = d_any + (size_t)d * B;
      // nodes whose parent is empty do not exist; every node of level d has a flag after this
      trim_flag_kernel<<<blocks_for(n_p), kBlock, 0, s>>>(drop[d], drop_p, child[d - 1], child[d], key[d - 1], nerr[d],
          derr[d], n_p, P.node_dis ? 1 : 0, P.th_distance, P.th_normal, any_kept, d_best + (size_t)d * B);
      trim_fix_kernel<<<blocks_for(B), kBlock, 0, s>>>(drop[d], d_best + (size_t)d * B, any_kept, key[d], o0.nnum[d], B);
    }
    OCNN_LAUNCH_OK("trim flags");
    {
      TrimScanLevels t;
      memset(&t, 0, sizeof(t));
      static_assert(sizeof(TrimScanLevels) <= 2048, "the level table is passed as a kernel argument");
      int tiles = 0;
      for (int d = A; d <= D; ++d) {
        TrimScanLevel& l = t.level[t.n_levels++];
        l.n = o0.nnum[d]; l.first_tile = tiles;
        l.drop = drop[d]; l.child = child[d]; l.pos = pos[d]; l.nchild = nchild[d];
        l.total_keep = d_counts + d; l.total_link = d_counts + 17 + d;
        tiles += scan_tiles(l.n);
      }
      t.n_tiles = tiles;
      t.tile_count = reinterpret_cast<int*>(ws + o_scan);
      if (tiles > 0) {
        trim_count_kernel<<<tiles, kBlock, 0, s>>>(t);
        trim_tiles_kernel<<<2 * t.n_levels, kBlock, 0, s>>>(t);
        trim_apply_kernel<<<tiles, kBlock, 0, s>>>(t);
      }
    }
    int h[64];
    {
      const int e = fetch_words(h, d_counts, 64, s);
      if (e) return e;
    }
    for (int d = A; d <= D; ++d) { o.nnum[d] = h[d]; o.nnum_nempty[d] = h[17 + d]; }
  }
  o.set_nnum_cum();
  OCNN_REQUIRE(o.set_ptr_dis(), OCNN_E_SHAPE, "the octree would exceed 2 GiB");
  memcpy(info_out, &o, sizeof(Info));

  // ---- serialization
  char* out = static_cast<char*>(alloc((size_t)o.sizeof_octree(), alloc_ctx));
  OCNN_REQUIRE(out, OCNN_E_BADARG, "the allocator returned no memory for the octree");
  OCNN_REQUIRE((reinterpret_cast<uintptr_t>(out) & 7) == 0, OCNN_E_BADARG, "blob not 8-byte aligned");
  *blob_out = out;
  {
    HeaderWords hdr;   // 720 bytes as a kernel argument: no copy, no wait
    memset(&hdr, 0, sizeof(hdr));
    memcpy(&hdr, &o, sizeof(Info));
    header_kernel<<<1, kBlock, 0, s>>>(reinterpret_cast<uint32_t*>(out), hdr);
  }
  {
    GatherLevels g;
    memset(&g, 0, sizeof(g));
    static_assert(sizeof(GatherLevels) <= 3072, "the level table is passed as a kernel argument");
    g.depth = D; g.key2xyz = o.key2xyz; g.key_channel = o.channel(OCNN_KEY); g.adaptive_split = adaptive ? 1 : 0;
    g.cn = cn; g.ch_dis = out_dis; g.cf = cf; g.cp = out_pt;
    int blocks = 0;
    for (int d = 0; d <= D; ++d) {
      const bool trimmed = adaptive && d >= A;
      GatherLevel& l = g.level[d];
      l.n_old = o0.nnum[d]; l.n_new = o.nnum[d];
      l.pos = trimmed ? pos[d] : nullptr;
      l.nchild = trimmed ? nchild[d] : nullptr;
      l.key = key[d]; l.child = child[d];
      l.normal = normal[d]; l.dis = dis[d]; l.feature = feature[d]; l.label = label[d]; l.pt = pt[d];
      l.key_out = reinterpret_cast<uint64_t*>(out + o.ptr_dis(OCNN_KEY, d));
      l.child_out = reinterpret_cast<int*>(out + o.ptr_dis(OCNN_CHILD, d));
      l.feature_out = o.channel(OCNN_FEATURE) > 0 ? reinterpret_cast<float*>(out + o.ptr_dis(OCNN_FEATURE, d)) : nullptr;
      l.label_out = o.has(OCNN_LABEL) ? reinterpret_cast<float*>(out + o.ptr_dis(OCNN_LABEL, d)) : nullptr;
      l.split_out = o.has(OCNN_SPLIT) ? reinterpret_cast<float*>(out + o.ptr_dis(OCNN_SPLIT, d)) : nullptr;
      g.first_block[d] = blocks;
      blocks += (int)blocks_for(l.n_old);
    }
    for (int d = D + 1; d <= kMaxD; ++d) g.first_block[d] = blocks;
    if (blocks > 0) gather_kernel<<<blocks, kBlock, 0, s>>>(g);
  }
  OCNN_LAUNCH_OK("serialize");
  if (in.merged) {
    // neighbour tables of the final structure (merge_octrees.cpp:185-197); the root level has
    // none and stays zero as in the reference's zero-initialised buffer
    fill_kernel<<<blocks_for((int64_t)o.nnum[0] * 8), kBlock, 0, s>>>(
        reinterpret_cast<float*>(out + o.ptr_dis(OCNN_NEIGH, 0)), (int64_t)o.nnum[0] * 8, 0.0f);
    for (int d = 1; d <= D;) {
      int* neigh = reinterpret_cast<int*>(out + o.ptr_dis(OCNN_NEIGH, d));
      if (d <= fl) {
        const int e = ocnn_calc_neigh_full(neigh, d, B, s);
        if (e) return e;
        ++d;
        continue;
      }
      if (o.nnum[d - 1] <= 0) { ++d; continue; }
      // the last levels in one launch (small levels: the chain of launches is what they cost)
      int count = 1;
      if (D - d < kNeighLevels && o.nnum[D] <= (1 << 21)) while (d + count <= D && o.nnum[d + count - 1] > 0) ++count;
      int* tables[kNeighLevels] = {nullptr, nullptr, nullptr};
      const int* links[kNeighLevels] = {nullptr, nullptr, nullptr};
      for (int i = 0; i < count; ++i) {
        tables[i] = reinterpret_cast<int*>(out + o.ptr_dis(OCNN_NEIGH, d + i));
        links[i] = reinterpret_cast<const int*>(out + o.ptr_dis(OCNN_CHILD, d + i - 1));
      }
      launch_neigh_sparse_levels(count, tables, reinterpret_cast<const int*>(out + o.ptr_dis(OCNN_NEIGH, d - 1)), links,
          o.nnum[d - 1], s);
      d += count;
    }
    OCNN_LAUNCH_OK("neighbours");
  }
  return OCNN_OK;
}

}  // namespace ocnn
