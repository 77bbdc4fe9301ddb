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

// ---- covered_depth_nodes (octree.cpp:958-1002): range of finest-level nodes under a node
// mode 0: finest level, 1: the level above, 2: any other level
__global__ void cover_kernel(int* __restrict__ dnum, int* __restrict__ didx, const int* __restrict__ child,
    const int* __restrict__ dnum_c, const int* __restrict__ didx_c, int n, int mode) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int num = 0, idx = -1;
  if (mode == 0) { num = 1; idx = i; }
  else {
    const int c = child[i];
    if (c >= 0) {
      if (mode == 1) { num = 8; idx = c * 8; }
      else {
        for (int j = 0; j < 8; ++j) num += dnum_c[c * 8 + j];
        for (int j = 0; j < 8; ++j)
          if (didx_c[c * 8 + j] != -1) { idx = didx_c[c * 8 + j]; break; }
      }
    }
  }
  dnum[i] = num;
  didx[i] = idx;
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
// partial sum is never -0: the chain starts at +0).  The next 256 leaves are requested before
// the current ones are added (the chain of a node high up in the tree covers the whole finest
// level: memory latency must not be paid per block).  sum[c] / last[c] get the sum and the
// last value of channel c on every lane.
constexpr int kPassValues = 8, kPassLeaves = 256;
template <int NV>
__device__ inline void ordered_sums(int k0, int k1, int lane, float* __restrict__ lds, const float* const (&row)[NV],
    float* sum, float* last) {
  static_assert(NV <= kPassValues, "LDS block too small");
  float acc = 0.0f;
  float4 vals[NV];
  auto request = [&](int base) {
    const int k = base + 4 * lane;
#pragma unroll
    for (int c = 0; c < NV; ++c) {
      float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      if (row[c] && k < k1) v = *reinterpret_cast<const float4*>(row[c] + k);
      v.x = (k >= k0 && k < k1) ? v.x : 0.0f;
      v.y = (k + 1 >= k0 && k + 1 < k1) ? v.y : 0.0f;
      v.z = (k + 2 >= k0 && k + 2 < k1) ? v.z : 0.0f;
      v.w = (k + 3 >= k0 && k + 3 < k1) ? v.w : 0.0f;
      vals[c] = v;
    }
  };
  const int kb = k0 < k1 ? (k0 & ~3) : k1;   // an empty range runs no block
  if (k0 < k1) request(kb);
  for (int base = kb; base < k1; base += kPassLeaves) {
#pragma unroll
    for (int c = 0; c < NV; ++c) *reinterpret_cast<float4*>(lds + c * kPassLeaves + 4 * lane) = vals[c];
    if (base + kPassLeaves < k1) request(base + kPassLeaves);
    __builtin_amdgcn_wave_barrier();   // same wavefront: the LDS unit keeps its accesses in order
    const int total = min(kPassLeaves, k1 - base);
    if (lane < NV) {
      // the adds form one dependent chain; the LDS reads of the next 16 leaves are in flight
      // while the current 16 are added
      constexpr int kStep = 16;
      const float4* src = reinterpret_cast<const float4*>(lds + lane * kPassLeaves);
      float4 cur[kStep / 4];
#pragma unroll
      for (int i = 0; i < kStep / 4; ++i) cur[i] = src[i];
      for (int t = 0; t < total; t += kStep) {
        float4 nxt[kStep / 4];
        const int tn = min(t + kStep, kPassLeaves - kStep);          // stays inside the block
#pragma unroll
        for (int i = 0; i < kStep / 4; ++i) nxt[i] = src[tn / 4 + i];
#pragma unroll
        for (int i = 0; i < kStep / 4; ++i) {
          acc = __fadd_rn(acc, cur[i].x); acc = __fadd_rn(acc, cur[i].y);
          acc = __fadd_rn(acc, cur[i].z); acc = __fadd_rn(acc, cur[i].w);
        }
#pragma unroll
        for (int i = 0; i < kStep / 4; ++i) cur[i] = nxt[i];
      }
    }
    __builtin_amdgcn_wave_barrier();
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
  int64_t nP;
  float *normal, *pt, *feature, *label, *dis, *nerr, *derr;   // level d (null: absent)
};

// One wavefront per node; every level above the finest in one launch, the root first (its
// chain is the longest, the others run beside it).
struct SignalLevels {
  int first_wave[kMaxD + 1];     // of level d; [depth] = total
  SignalArgs level[kMaxD - 1];
};
__global__ __launch_bounds__(kBlock) void signal_kernel(const SignalLevels* __restrict__ levels, int depth) {
  const int lane = threadIdx.x & 63;
  const int w = (int)((blockIdx.x * (unsigned)kBlock + threadIdx.x) >> 6);
  if (w >= levels->first_wave[depth]) return;
  int d = 0;
  while (w >= levels->first_wave[d + 1]) ++d;
  const SignalArgs& a = levels->level[d];
  const int i = w - levels->first_wave[d];
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
    ordered_sums<6>(k0, k1, lane, lds, rows6, sum6, last6);
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
    ordered_sums<kPassValues>(k0, k1, lane, lds, rows8, fsum, flast);
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
        float distance_min = 1.0e30f;
        for (int k = k0 + lane; k < k1; k += 64) {
          float dis = 0.0f;
          for (int c = 0; c < 3; ++c) {
            const float ptc = __fsub_rn(a.pt_P[c * nP + k], vk[c]);
            dis = __fadd_rn(dis, __fmul_rn(ptc, ptc));
          }
          distance_min = fminf(distance_min, sqrt_rn(dis));
        }
        distance_min = wave_min(distance_min);
        if (distance_min > distance_max2) distance_max2 = distance_min;
      }
      err = distance_max2 > distance_max1 ? distance_max2 : distance_max1;
    }
    if (lane == 0) a.derr[i] = err;
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
    // (L1 distance, the first one on a tie), octree.cpp:776-803.
    if (!(a.has_dis && a.dis)) return;
    for (int id = 0; id < 8; ++id) {
      const int i = i_base + id;
      float pti[3], ptj[3], dis_min = 1.0e30f;
      node_xyz(pti, a.key[i], a.d, a.key2xyz);
      int j_min = -1;
      for (int j = 0; j < a.n; ++j) {
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

// one thread per node of level d-1: flags of its children at level d
__global__ void trim_flag_kernel(int* __restrict__ drop_d, const int* __restrict__ drop_p, const int* __restrict__ child_p,
    const int* __restrict__ child_d, const float* __restrict__ nerr, const float* __restrict__ derr, int n_p,
    int has_dis, float th_dist, float th_norm, int* __restrict__ any_kept) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_p) return;
  const int c = child_p[i];
  if (c == -1) return;
  const bool parent_kept = drop_p == nullptr || drop_p[i] == kKeep;
  bool kept = false;
  for (int j = 0; j < 8; ++j) {
    const int idx = c * 8 + j;
    int f = kKeep;
    if (parent_kept) {
      if ((!has_dis || derr[idx] < th_dist) && nerr[idx] < th_norm) f = kDropChildren;
    } else {
      f = kDrop;
    }
    drop_d[idx] = f;
    kept = kept || (f == kKeep && child_d[idx] != -1);
  }
  if (kept) *any_kept = 1;
}
// if no non-empty node of the level was kept: the candidate with the largest normal error
// (the first one on a tie) is found ...
__global__ void trim_argmax_kernel(unsigned long long* __restrict__ best, const int* __restrict__ drop_p,
    const int* __restrict__ child_p, const int* __restrict__ child_d, const float* __restrict__ nerr, int n_p,
    const int* __restrict__ any_kept) {
  if (*any_kept) return;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_p) return;
  const int c = child_p[i];
  if (c == -1 || (drop_p != nullptr && drop_p[i] != kKeep)) return;
  for (int j = 0; j < 8; ++j) {
    const int idx = c * 8 + j;
    if (child_d[idx] == -1) continue;
    const float e = nerr[idx];
    if (!(e > -1.0f)) continue;
    atomicMax(best, ((unsigned long long)__float_as_uint(e) << 32) | (unsigned long long)(0xffffffffu - (unsigned)idx));
  }
}
// ... and kept
__global__ void trim_fix_kernel(int* __restrict__ drop_d, const unsigned long long* __restrict__ best,
    const int* __restrict__ any_kept) {
  if (*any_kept) return;
  const unsigned long long b = *best;
  const int idx = b == 0 ? 0 : (int)(0xffffffffu - (unsigned)(b & 0xffffffffull));
  drop_d[idx] = kKeep;
}

struct KeepPred {
  const int* drop;
  __device__ bool operator()(int64_t i) const { return drop[i] != kDrop; }
};
struct KeepOut {
  int* pos;
  __device__ void operator()(int64_t i, bool f, int rank) const { pos[i] = f ? rank : -1; }
};
struct LinkPred {
  const int* drop; const int* child;
  __device__ bool operator()(int64_t i) const { return drop[i] == kKeep && child[i] != -1; }
};
struct LinkOut {
  const int* drop; int* nchild;
  __device__ void operator()(int64_t i, bool f, int rank) const { nchild[i] = f ? rank : -1; }
};

// ---- serialization (octree.cpp:907-956) -----------------------------------------------------
struct GatherArgs {
  int d, n_old, n_new, key2xyz, key_channel, adaptive_split;
  const int* pos;            // new index of an old node, -1: dropped; null: identity
  const int* nchild;         // new child link; null: the old one
  const uint64_t* key; const int* child;
  const float *normal, *dis, *feature, *label, *pt;   // per-level signals (null: not stored)
  int cn, ch_dis, cf, cp;
  uint64_t* key_out; int* child_out; float* feature_out; float* label_out; float* split_out;
};
__global__ void gather_kernel(GatherArgs a) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= a.n_old) return;
  const int k = a.pos ? a.pos[i] : i;
  if (k < 0) return;
  const int64_t no = a.n_old, nn = a.n_new;
  uint64_t key = a.key[i];
  if (a.key2xyz) {  // Octree::key_to_xyz, octree.cpp:1137-1156
    uint32_t x, y, z;
    morton_decode(key, a.d, &x, &y, &z);
    key = (uint64_t)(x & 0xffff) | ((uint64_t)(y & 0xffff) << 16) | ((uint64_t)(z & 0xffff) << 32);
  }
  a.key_out[k] = key;
  if (a.key_channel == 2) a.key_out[nn + k] = 0;
  const int ch = a.nchild ? a.nchild[i] : a.child[i];
  a.child_out[k] = ch;
  float* f = a.feature_out;
  float nsum = 0.0f;
  if (f) {
    for (int c = 0; c < a.cn; ++c) { const float v = a.normal[c * no + i]; f[c * nn + k] = v; if (c < 3) nsum = __fadd_rn(nsum, fabsf(v)); }
    f += a.cn * nn;
    for (int c = 0; c < a.ch_dis; ++c) f[c * nn + k] = a.dis[c * no + i];
    f += a.ch_dis * nn;
    for (int c = 0; c < a.cf; ++c) f[c * nn + k] = a.feature[c * no + i];
    f += a.cf * nn;
    for (int c = 0; c < a.cp; ++c) f[c * nn + k] = a.pt[c * no + i];
  }
  if (a.label_out) a.label_out[k] = a.label[i];
  if (a.split_out) {  // calc_split_label, octree.cpp:1158-1178
    float s = 1.0f;
    if (ch == -1) s = (a.adaptive_split && nsum != 0.0f) ? 2.0f : 0.0f;
    a.split_out[k] = s;
  }
}
__global__ void header_kernel(uint32_t* __restrict__ dst, const uint32_t* __restrict__ src_words, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = src_words[i];
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
  const size_t o_scan = take(scan_scratch_bytes(max_n));
  const size_t o_counts = take(sizeof(int) * 64);      // [0..16] kept nodes, [17..33] kept links, [34..50] any_kept
  const size_t o_best = take(sizeof(unsigned long long) * kMaxD);
  const size_t o_hdr = take(OCNN_HEADER_BYTES);
  const size_t o_levels = take(sizeof(SignalLevels));
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
  unsigned long long* d_best = reinterpret_cast<unsigned long long*>(ws + o_best);

  // ---- covered ranges and signals of every depth
  for (int d = D; d >= 0; --d) {
    const int n = o0.nnum[d];
    cover_kernel<<<blocks_for(n), kBlock, 0, s>>>(dnum[d], didx[d], child[d], d < D ? dnum[d + 1] : nullptr,
        d < D ? didx[d + 1] : nullptr, n, d == D ? 0 : (d == D - 1 ? 1 : 2));
  }
  OCNN_LAUNCH_OK("cover");
  fill_kernel<<<blocks_for(o0.nnum[D]), kBlock, 0, s>>>(nerr[D], o0.nnum[D], 1.0e20f);
  fill_kernel<<<blocks_for(o0.nnum[D]), kBlock, 0, s>>>(derr[D], o0.nnum[D], 1.0e20f);
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
    SignalLevels* L = new SignalLevels;
    memset(L, 0, sizeof(SignalLevels));
    int waves = 0;
    for (int d = 0; d < D; ++d) {
      SignalArgs& a = L->level[d];
      a.d = d; a.depth = D; a.n = o0.nnum[d]; a.nD = o0.nnum[D]; a.cf = cf; a.ch_dis = ch_dis;
      a.adp_layer = o0.adp_layer; a.calc_nerr = adaptive && cn; a.calc_derr = adaptive && P.node_dis && cn;
      a.imul = imul;
      a.key = key[d]; a.child = child[d]; a.dnum = dnum[d]; a.didx = didx[d];
      a.child_D = child[D]; a.nrm_D = normal[D]; a.pt_D = pt[D]; a.feat_D = feature[D]; a.lab_D = label[D];
      a.rank_D = rank_D; a.nrm_P = nrm_P; a.pt_P = pt_P; a.feat_P = feat_P; a.lab_P = lab_P; a.nP = (int64_t)nP;
      a.normal = normal[d]; a.pt = pt[d]; a.feature = feature[d]; a.label = label[d]; a.dis = dis[d];
      a.nerr = nerr[d]; a.derr = derr[d];
      L->first_wave[d] = waves;
      waves += a.n;
    }
    for (int d = D; d <= kMaxD; ++d) L->first_wave[d] = waves;
    hipError_t e = hipMemcpyAsync(ws + o_levels, L, sizeof(SignalLevels), hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);   // the table is host memory of this call
    delete L;
    OCNN_REQUIRE(e == hipSuccess, OCNN_E_HIP, "level table: %s", hipGetErrorString(e));
    if (waves > 0)
      signal_kernel<<<blocks_for((int64_t)waves * 64), kBlock, 0, s>>>(reinterpret_cast<const SignalLevels*>(ws + o_levels), D);
  }
  OCNN_LAUNCH_OK("signal");

  // ---- extrapolation into the empty nodes (before trimming, as Octree::build does)
  if (P.extrapolate) {
    for (int d = D; d >= fl; --d) {
      ExtrapolateArgs a;
      a.n = o0.nnum[d]; a.cf = cf; a.has_dis = ch_dis != 0; a.imul = imul; a.d = d; a.key2xyz = P.key2xyz ? 1 : 0;
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
  const int A = o.adp_layer;
  if (adaptive) {
    OCNN_REQUIRE(A >= 1 && A <= D, OCNN_E_BADARG, "adp_depth %d", A);
    for (int d = A; d <= D; ++d) {
      const int n_p = o0.nnum[d - 1];
      const int* drop_p = d - 1 >= A ? drop[d - 1] : nullptr;
      int* any_kept = d_counts + 34 + d;
      // nodes whose parent is empty do not exist; every node of level d has a flag after this
      trim_flag_kernel<<<blocks_for(n_p), kBlock, 0, s>>>(drop[d], drop_p, child[d - 1], child[d], nerr[d], derr[d], n_p,
          P.node_dis ? 1 : 0, P.th_distance, P.th_normal, any_kept);
      trim_argmax_kernel<<<blocks_for(n_p), kBlock, 0, s>>>(d_best + d, drop_p, child[d - 1], child[d], nerr[d], n_p, any_kept);
      trim_fix_kernel<<<1, 1, 0, s>>>(drop[d], d_best + d, any_kept);
    }
    OCNN_LAUNCH_OK("trim flags");
    for (int d = A; d <= D; ++d) {
      const int n = o0.nnum[d];
      KeepPred kp{drop[d]};
      KeepOut ko{pos[d]};
      hipError_t e = flag_scan(kp, ko, (int64_t)n, reinterpret_cast<int*>(ws + o_scan), d_counts + d, s);
      OCNN_REQUIRE(e == hipSuccess, OCNN_E_HIP, "keep scan: %s", hipGetErrorString(e));
      LinkPred lp{drop[d], child[d]};
      LinkOut lo{drop[d], nchild[d]};
      e = flag_scan(lp, lo, (int64_t)n, reinterpret_cast<int*>(ws + o_scan), d_counts + 17 + d, s);
      OCNN_REQUIRE(e == hipSuccess, OCNN_E_HIP, "link scan: %s", hipGetErrorString(e));
    }
    int h[64];
    OCNN_HIP_OK(hipMemcpyAsync(h, d_counts, sizeof(h), hipMemcpyDeviceToHost, s));
    OCNN_HIP_OK(hipStreamSynchronize(s));
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
    uint32_t hdr[OCNN_HEADER_BYTES / 4];
    memset(hdr, 0, sizeof(hdr));
    memcpy(hdr, &o, sizeof(Info));
    // the words travel through the scratch block: a kernel argument of 720 bytes per launch
    // would do as well, but this launch is not on any critical path
    OCNN_HIP_OK(hipMemcpyAsync(ws + o_hdr, hdr, sizeof(hdr), hipMemcpyHostToDevice, s));
    OCNN_HIP_OK(hipStreamSynchronize(s));   // `hdr` lives on this stack frame
    header_kernel<<<1, kBlock, 0, s>>>(reinterpret_cast<uint32_t*>(out), reinterpret_cast<const uint32_t*>(ws + o_hdr),
        OCNN_HEADER_BYTES / 4);
  }
  for (int d = 0; d <= D; ++d) {
    const bool trimmed = adaptive && d >= A;
    GatherArgs g;
    memset(&g, 0, sizeof(g));
    g.d = d; g.n_old = o0.nnum[d]; g.n_new = o.nnum[d]; g.key2xyz = o.key2xyz; g.key_channel = o.channel(OCNN_KEY);
    g.adaptive_split = adaptive ? 1 : 0;
    g.pos = trimmed ? pos[d] : nullptr;
    g.nchild = trimmed ? nchild[d] : nullptr;
    g.key = key[d]; g.child = child[d];
    g.normal = normal[d]; g.dis = dis[d]; g.feature = feature[d]; g.label = label[d]; g.pt = pt[d];
    g.cn = cn; g.ch_dis = out_dis; g.cf = cf; g.cp = out_pt;
    g.key_out = reinterpret_cast<uint64_t*>(out + o.ptr_dis(OCNN_KEY, d));
    g.child_out = reinterpret_cast<int*>(out + o.ptr_dis(OCNN_CHILD, d));
    g.feature_out = o.channel(OCNN_FEATURE) > 0 ? reinterpret_cast<float*>(out + o.ptr_dis(OCNN_FEATURE, d)) : nullptr;
    g.label_out = o.has(OCNN_LABEL) ? reinterpret_cast<float*>(out + o.ptr_dis(OCNN_LABEL, d)) : nullptr;
    g.split_out = o.has(OCNN_SPLIT) ? reinterpret_cast<float*>(out + o.ptr_dis(OCNN_SPLIT, d)) : nullptr;
    if (g.n_old > 0) gather_kernel<<<blocks_for(g.n_old), kBlock, 0, s>>>(g);
  }
  OCNN_LAUNCH_OK("serialize");
  return OCNN_OK;
}

}  // namespace ocnn
