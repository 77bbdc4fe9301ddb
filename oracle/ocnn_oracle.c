/* TEST INFRASTRUCTURE -- CPU restatement ("oracle") of the O-CNN octree hot
 * path in plain C99.  See ocnn_oracle.h for the pinning status of each entry
 * point.  This file is the checker: the shipped HIP library never links,
 * loads or calls it.
 *
 * Paths in comments are relative to the reference checkout root. */
#include "ocnn_oracle.h"

#include <math.h>
#include <float.h>
#define ORC_COS(x) ((float)cos((double)(x)))
#define ORC_SIN(x) ((float)sin((double)(x)))
#include <stddef.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------ */
/* Wire format: OctreeInfo (octree/octree/octree_info.h:96-118), 716 bytes,
 * payload starts at 720 (octree_info.cpp:254-268). */
typedef struct {
  char magic[16];
  int batch_size, depth, full_layer, adp_layer;
  unsigned char is_adaptive; /* +3 pad */
  float th_dist, th_norm;
  unsigned char key2xyz, has_node_dis; /* +2 pad */
  int nnum[16], nnum_cum[16], nnum_nempty[16];
  int content_flags;
  int channels[16], locations[16];
  float bbmin[3], bbmax[3];
  unsigned char extrapolate, save_pts;
  char reserved[254];
  int ptr_dis[16];
} OInfo;

#define SA(c, n) typedef char static_assert_##n[(c) ? 1 : -1]
SA(sizeof(OInfo) == 716, size);
SA(offsetof(OInfo, th_dist) == 36, thd);
SA(offsetof(OInfo, key2xyz) == 44, k2x);
SA(offsetof(OInfo, nnum) == 48, nnum);
SA(offsetof(OInfo, content_flags) == 240, cf);
SA(offsetof(OInfo, bbmin) == 372, bb);
SA(offsetof(OInfo, extrapolate) == 396, ex);
SA(offsetof(OInfo, ptr_dis) == 652, pd);

enum { kKey = 1, kChild = 2, kNeigh = 4, kFeature = 8, kLabel = 16, kSplit = 32 };
#define KPTYPE 6
static const char kMagic[] = "_OCTREE_2.0_"; /* 64-bit keys: octree_info.cpp:7-11 */

/* PointsInfo (octree/octree/points_info.h:35-39), 88 bytes. */
typedef struct {
  char magic[16];
  int pt_num, content_flags;
  int channels[8], ptr_dis[8];
} PInfo;
SA(sizeof(PInfo) == 88, psize);
enum { pPoint = 1, pNormal = 2, pFeature = 4, pLabel = 8 };

static int prop_index(int ptype) { /* octree_info.cpp:283-291 */
  for (int i = 0; i < KPTYPE; ++i) if (ptype & (1 << i)) return i;
  return 0;
}
static int has_prop(const OInfo* o, int p) { return (o->content_flags & p) != 0; }
static int channel_of(const OInfo* o, int p) {
  return has_prop(o, p) ? o->channels[prop_index(p)] : 0;
}
static int location_of(const OInfo* o, int p) {
  return has_prop(o, p) ? o->locations[prop_index(p)] : 0;
}
static int size_of(int p) { /* octree_info.cpp:143-155 */
  if (p == kChild || p == kNeigh) return 4;
  if (p == kFeature || p == kLabel || p == kSplit) return 4;
  if (p == kKey) return 8;
  return 0;
}
static void info_reset(OInfo* o) { /* octree_info.cpp:75-78 */
  memset(o, 0, sizeof(*o));
  strcpy(o->magic, kMagic);
}
static void set_channel(OInfo* o, int p, int ch) { /* octree_info.cpp:231-243 */
  int i = prop_index(p);
  if (ch > 0) { o->channels[i] = ch; o->content_flags |= p; }
  else { o->channels[i] = 0; o->content_flags &= ~p; }
}
static void set_location(OInfo* o, int p, int lc) { o->locations[prop_index(p)] = lc; }
static void set_property(OInfo* o, int p, int ch, int lc) { set_channel(o, p, ch); set_location(o, p, lc); }
static void set_batch_size(OInfo* o, int b) { o->batch_size = b < 1 ? 1 : b; }
static void set_depth(OInfo* o, int d) { o->depth = o->full_layer < d ? d : o->full_layer; }
static void set_full_layer(OInfo* o, int fd) { o->full_layer = fd < 1 ? 1 : fd; }
static void set_nnum_cum(OInfo* o, int capacity) { /* octree_info.cpp:215-222 */
  o->nnum_cum[0] = 0;
  for (int d = 1; d < o->depth + 2; ++d) o->nnum_cum[d] = o->nnum_cum[d - 1] + o->nnum[d - 1];
  o->nnum_cum[o->depth + 2] = capacity > o->nnum_cum[o->depth + 1] ? capacity : o->nnum_cum[o->depth + 1];
}
static int total_nnum(const OInfo* o) { return o->nnum_cum[o->depth + 1]; }
static int total_capacity(const OInfo* o) { return o->nnum_cum[o->depth + 2]; }
static void set_ptr_dis(OInfo* o) { /* octree_info.cpp:254-268 */
  o->ptr_dis[0] = (int)((sizeof(OInfo) + 7) / 8 * 8);
  for (int i = 1; i <= KPTYPE; ++i) {
    int p = 1 << (i - 1);
    int lc = location_of(o, p);
    int num = lc == -1 ? total_capacity(o) : o->nnum[lc];
    o->ptr_dis[i] = o->ptr_dis[i - 1] + size_of(p) * num * o->channels[i - 1];
  }
}
static int ptr_dis(const OInfo* o, int p, int depth) { /* octree_info.cpp:157-167 */
  if (!has_prop(o, p)) return -1;
  int dis = o->ptr_dis[prop_index(p)];
  if (location_of(o, p) == -1) dis += o->nnum_cum[depth] * channel_of(o, p) * size_of(p);
  return dis;
}
static int sizeof_octree(const OInfo* o) { return o->ptr_dis[KPTYPE]; }
static float bbox_max_width(const OInfo* o) { /* octree_info.cpp:169-178 */
  float w = o->bbmax[0] - o->bbmin[0];
  for (int i = 1; i < 3; ++i) { float d = o->bbmax[i] - o->bbmin[i]; if (d > w) w = d; }
  if (w == 0.0f) w = 1.0e-10f;
  return w;
}
static void* prop_ptr(const void* blob, int p, int depth) {
  int dis = ptr_dis((const OInfo*)blob, p, depth);
  return dis < 0 ? NULL : (char*)blob + dis;
}

/* result of the last blob-producing call */
static char* g_last = NULL;
static int64_t g_last_sz = 0;
static char* result_alloc(int64_t sz) {
  free(g_last);
  g_last = (char*)calloc(sz > 0 ? (size_t)sz : 1, 1);
  g_last_sz = g_last ? sz : 0;
  return g_last;
}
int64_t orc_fetch(void* out, int64_t cap) {
  if (!g_last || g_last_sz > cap) return ORC_E_BADARG;
  memcpy(out, g_last, (size_t)g_last_sz);
  return g_last_sz;
}

/* ------------------------------------------------------------------------ */
/* Key math: octree/octree/octree_nn.cpp:551-575 */
static uint64_t compute_key(const uint64_t* pt, int depth) {
  uint64_t key = 0;
  for (int i = 0; i < depth; i++) {
    uint64_t mask = 1u << i;
    for (int j = 0; j < 3; j++) key |= (pt[j] & mask) << (2 * i + 2 - j);
  }
  return key;
}
static void compute_pt(uint64_t* pt, uint64_t key, int depth) {
  pt[0] = pt[1] = pt[2] = 0;
  for (int i = 0; i < depth; i++)
    for (int j = 0; j < 3; j++) {
      uint64_t mask = (uint64_t)1 << (3 * i + 2 - j);
      pt[j] |= (key & mask) >> (2 * i + 2 - j);
    }
}
/* octree_nn.cpp:578-619: packed xyz = four uint16 sub-fields (x,y,z,id) */
void orc_xyz2key(uint64_t* key, const uint64_t* xyz, int num, int depth) {
  for (int i = 0; i < num; ++i) {
    uint16_t f[4]; memcpy(f, xyz + i, 8);
    uint64_t pt[3] = { f[0], f[1], f[2] };
    uint64_t k = compute_key(pt, depth);
    uint16_t g[4]; memcpy(g, &k, 8);
    g[3] = f[3];
    memcpy(key + i, g, 8);
  }
}
void orc_key2xyz(uint64_t* xyz, const uint64_t* key, int num, int depth) {
  for (int i = 0; i < num; ++i) {
    uint64_t pt[3]; compute_pt(pt, key[i], depth);
    uint16_t f[4]; memcpy(f, key + i, 8);
    for (int j = 0; j < 3; ++j) f[j] = (uint16_t)pt[j];
    memcpy(xyz + i, f, 8);
  }
}
void orc_key2idx(int* idx, const uint64_t* key, int num) {
  for (int i = 0; i < num; ++i) idx[i] = (int)(key[i] >> 48);
}
/* octree_nn.cpp:541-548 */
void orc_search_key(int* idx, const uint64_t* key, int n_key, const uint64_t* query, int n_query) {
  for (int i = 0; i < n_query; ++i) {
    int lo = 0, hi = n_key; /* lower_bound */
    while (lo < hi) { int mid = lo + (hi - lo) / 2; if (key[mid] < query[i]) lo = mid + 1; else hi = mid; }
    idx[i] = (lo >= n_key || key[lo] != query[i]) ? -1 : lo;
  }
}

/* ------------------------------------------------------------------------ */
/* NeighHelper tables: octree/octree/octree_nn.cpp:6-81 */
static int g_ni3[216], g_parent[512], g_dis[64], g_tables_ready = 0;
static const int kSub111[] = { 13 };
static const int kSub222[] = { 13, 14, 16, 17, 22, 23, 25, 26 };
static const int kSub311[] = { 4, 13, 22 };
static const int kSub131[] = { 10, 13, 16 };
static const int kSub113[] = { 12, 13, 14 };
static const int kSub331[] = { 1, 4, 7, 10, 13, 16, 19, 22, 25 };
static const int kSub313[] = { 3, 4, 5, 12, 13, 14, 21, 22, 23 };
static const int kSub133[] = { 9, 10, 11, 12, 13, 14, 15, 16, 17 };
static void init_tables(void) {
  if (g_tables_ready) return;
  int id = 0;
  for (int ijk = 0; ijk < 8; ++ijk)
    for (int xyz = 0; xyz < 27; ++xyz) {
      int k = ijk % 2, p = ijk / 2, j = p % 2, i = p / 2;
      int z = xyz % 3, q = xyz / 3, y = q % 3, x = q / 3;
      g_ni3[id++] = ((x + i) << 4) | ((y + j) << 2) | (z + k);
    }
  int tmp[64]; id = 0;
  for (int x = 1; x < 5; ++x)
    for (int y = 1; y < 5; ++y)
      for (int z = 1; z < 5; ++z) {
        tmp[id] = (x / 2) * 9 + (y / 2) * 3 + (z / 2);
        g_dis[id] = ((x % 2) << 2) | ((y % 2) << 1) | (z % 2);
        id++;
      }
  for (int i = 0; i < 8; ++i)
    for (int j = 0; j < 64; ++j) g_parent[i * 64 + j] = g_ni3[i * 27 + tmp[j]];
  g_tables_ready = 1;
}
int orc_get_ni(const int* ks, int* out) { /* octree_nn.cpp:111-119 */
  init_tables();
  int code = ks[0] * 100 + ks[1] * 10 + ks[2];
  const int* sub = NULL; int sz = 0;
  switch (code) {
    case 333: memcpy(out, g_ni3, sizeof(g_ni3)); return 216;
    case 111: sub = kSub111; sz = 1; break;
    case 222: sub = kSub222; sz = 8; break;
    case 311: sub = kSub311; sz = 3; break;
    case 131: sub = kSub131; sz = 3; break;
    case 113: sub = kSub113; sz = 3; break;
    case 331: sub = kSub331; sz = 9; break;
    case 313: sub = kSub313; sz = 9; break;
    case 133: sub = kSub133; sz = 9; break;
    default: return ORC_E_UNSUPPORTED;
  }
  for (int i = 0; i < 8; ++i)
    for (int j = 0; j < sz; ++j) out[i * sz + j] = g_ni3[i * 27 + sub[j]];
  return 8 * sz;
}
void orc_get_parent(int* out) { init_tables(); memcpy(out, g_parent, sizeof(g_parent)); }
void orc_get_dis(int* out) { init_tables(); memcpy(out, g_dis, sizeof(g_dis)); }

/* octree_nn.cpp:357-380 */
void orc_calc_neigh_sparse(int* neigh_child, const int* neigh, const int* children, int node_num) {
  init_tables();
  for (int i = 0; i < node_num; ++i) {
    int l0 = children[i];
    if (l0 == -1) continue;
    const int* ngh0 = neigh + (i >> 3 << 6);
    const int* pi0 = g_parent + (i % 8) * 64;
    int* ngh1 = neigh_child + ((int64_t)l0 << 6);
    for (int j = 0; j < 64; ++j) {
      ngh1[j] = -1;
      int k = ngh0[pi0[j]];
      if (k != -1) { int l1 = children[k]; if (l1 != -1) ngh1[j] = (l1 << 3) + g_dis[j]; }
    }
  }
}
/* octree_nn.cpp:382-424 */
void orc_calc_neigh_full(int* neigh, int depth, int batch) {
  const uint64_t node_num = (uint64_t)1 << (3 * depth), bound = (uint64_t)1 << depth;
  for (uint64_t n = 0; n < (uint64_t)batch; ++n)
    for (uint64_t i = 0; i < node_num; i += 8) {
      uint64_t p0[3]; compute_pt(p0, i, depth);
      for (uint64_t x = 0; x < 4; ++x)
        for (uint64_t y = 0; y < 4; ++y)
          for (uint64_t z = 0; z < 4; ++z) {
            uint64_t p1[3] = { p0[0] + x - 1, p0[1] + y - 1, p0[2] + z - 1 };
            int v = -1;
            if ((p1[0] & bound) == 0 && (p1[1] & bound) == 0 && (p1[2] & bound) == 0)
              v = (int)(compute_key(p1, depth) + n * node_num);
            neigh[((x << 4) | (y << 2) | z) + i * 8 + n * node_num * 8] = v;
          }
    }
}

/* ------------------------------------------------------------------------ */
/* octree_nn.cpp:427-473 */
void orc_generate_key_child(uint64_t* key_child, const uint64_t* key, const int* child, int node_num) {
  for (int i = 0; i < node_num; ++i) {
    int label = child[i];
    if (label < 0) continue;
    uint16_t k0[4]; memcpy(k0, key + i, 8);
    for (int j = 0; j < 8; ++j) {
      uint16_t k1[4];
      k1[0] = (uint16_t)((k0[0] << 1) | ((j & 4) >> 2));
      k1[1] = (uint16_t)((k0[1] << 1) | ((j & 2) >> 1));
      k1[2] = (uint16_t)((k0[2] << 1) | (j & 1));
      k1[3] = k0[3];
      memcpy(key_child + 8 * (int64_t)label + j, k1, 8);
    }
  }
}
void orc_generate_key_full(uint64_t* key, int depth, int batch) {
  int node_num = 1 << (3 * depth);
  for (int n = 0; n < batch; ++n)
    for (int k = 0; k < node_num; ++k) {
      uint64_t pt[3]; compute_pt(pt, (uint64_t)k, depth);
      uint16_t f[4] = { (uint16_t)pt[0], (uint16_t)pt[1], (uint16_t)pt[2], (uint16_t)n };
      memcpy(key + (int64_t)n * node_num + k, f, 8);
    }
}
int orc_generate_label(int* label, const int* btm, int btm_h, int mask) {
  int top_h = 0;
  for (int i = 0; i < btm_h; ++i) label[i] = (mask == btm[i]) ? top_h++ : -1;
  return top_h;
}

/* ------------------------------------------------------------------------ */
/* octree_nn.cpp:163-185 */
void orc_pad_forward(float* Y, int Hy, int C, const float* X, int Hx, const int* label, float dval) {
  for (int c = 0; c < C; ++c)
    for (int h = 0; h < Hy; ++h)
      Y[(int64_t)c * Hy + h] = label[h] == -1 ? dval : X[(int64_t)c * Hx + label[h]];
}
void orc_pad_backward(float* X, int Hx, int C, const float* Y, int Hy, const int* label) {
  for (int c = 0; c < C; ++c)
    for (int h = 0; h < Hy; ++h)
      if (label[h] != -1) X[(int64_t)c * Hx + label[h]] = Y[(int64_t)c * Hy + h];
}
/* octree_gather / octree_gatherbk / octree_mask: GPU-only in the reference
 * (octree_nn.cu:756-830, declarations octree_nn.h:204-218).  gather is pad_forward with value 0
 * (octree_nn.cu:770-773); gatherbk zero-fills and scatter-adds, its index may repeat
 * (:782-801); mask zeroes the rows whose label equals `mask` (:805-818). */
void orc_octree_gather(float* top, int top_h, int channel, const float* btm, int btm_h, const int* idx) {
  orc_pad_forward(top, top_h, channel, btm, btm_h, idx, 0.0f);
}
void orc_octree_gatherbk(const float* top, int top_h, int channel, float* btm, int btm_h, const int* idx) {
  for (int64_t i = 0; i < (int64_t)channel * btm_h; ++i) btm[i] = 0.0f;
  for (int c = 0; c < channel; ++c)
    for (int h = 0; h < top_h; ++h)
      if (idx[h] != -1) btm[(int64_t)c * btm_h + idx[h]] += top[(int64_t)c * top_h + h];
}
void orc_octree_mask(float* out, const float* in, const int* label, int height, int mask, int num) {
  for (int i = 0; i < num; ++i) out[i] = label[i % height] == mask ? 0.0f : in[i];
}

/* Trilinear stencils between two levels.  Table: NeighHelper (octree_nn.cpp:83-108): for a node
 * with sibling index i, its child j and corner k, the slot (x << 4 | y << 2 | z) of the
 * parent-level node that corner k of the interpolation cell of that child falls into;
 * corner order 000, 001, 010, 100, 011, 101, 110, 111 of (x, y, z) = weights 27, 9, 9, 9, 3, 3, 3, 1. */
static const int kBilinearCorner[8][3] = {
  {0, 0, 0}, {0, 0, 1}, {0, 1, 0}, {1, 0, 0}, {0, 1, 1}, {1, 0, 1}, {1, 1, 0}, {1, 1, 1}};
void orc_get_bilinear(int* table) {
  for (int i = 0; i < 8; ++i) {
    int z0 = i % 2, y0 = (i / 2) % 2, x0 = i / 4;
    for (int j = 0; j < 8; ++j) {
      int z1 = j % 2, y1 = (j / 2) % 2, x1 = j / 4;
      for (int k = 0; k < 8; ++k) {
        int x2 = x0 + 1 + kBilinearCorner[k][0] * (2 * x1 - 1);
        int y2 = y0 + 1 + kBilinearCorner[k][1] * (2 * y1 - 1);
        int z2 = z0 + 1 + kBilinearCorner[k][2] * (2 * z1 - 1);
        table[(i << 6) | (j << 3) | k] = (x2 << 4) | (y2 << 2) | z2;
      }
    }
  }
}
/* bilinear_neigh_cpu, octree_nn.cpp:476-492: bidx[(8 child[i] + j) * 8 + k] for the children of
 * every non-empty node i of the level; entries of other rows are left as they are. */
void orc_bilinear_neigh(int* bidx, const int* neigh, const int* child, int node_num) {
  int table[512];
  orc_get_bilinear(table);
  for (int i = 0; i < node_num; ++i) {
    if (child[i] < 0) continue;
    const int* block = neigh + ((int64_t)(i >> 3) << 6);
    for (int j = 0; j < 8; ++j)
      for (int k = 0; k < 8; ++k)
        bidx[((int64_t)child[i] * 8 + j) * 8 + k] = block[table[((i % 8) << 6) | (j << 3) | k]];
  }
}
/* bilinear_xyz_cpu, octree_nn.cpp:494-530 (64-bit keys: four 16-bit fields x, y, z, id): the 8
 * cells of level d0 around the centre of a cell of level d1, nearest first, and the weights of
 * the nearest one per axis. */
void orc_bilinear_xyz(uint64_t* xyz0, float* fracs, int d0, const uint64_t* xyz1, int d1, int num) {
  const float scale = (float)(1 << (d1 - d0));
  for (int i = 0; i < num; ++i) {
    const uint16_t* in = (const uint16_t*)(xyz1 + i);
    int bnd[2][3];
    for (int c = 0; c < 3; ++c) {
      float pt = ((float)in[c] + 0.5f) / scale - 0.5f;
      int b = (int)pt;
      float frac = pt - (float)b;
      if (frac > 0.5f) { bnd[0][c] = b + 1; bnd[1][c] = b; }
      else { frac = 1 - frac; bnd[0][c] = b; bnd[1][c] = b + 1; }
      fracs[3 * (int64_t)i + c] = frac;
    }
    for (int j = 0; j < 8; ++j) {
      uint16_t* out = (uint16_t*)(xyz0 + (int64_t)i * 8 + j);
      for (int c = 0; c < 3; ++c) out[c] = (uint16_t)bnd[kBilinearCorner[j][c]][c];
      out[3] = in[3];
    }
  }
}

static void pad_backward_int(int* X, const int* Y, int Hy, const int* label) {
  for (int h = 0; h < Hy; ++h) if (label[h] != -1) X[label[h]] = Y[h];
}

/* octree_nn.cpp:188-241 */
void orc_octree2col(float* col, const float* data, int channel, int height,
    int kernel_sdim, int stride, const int* neigh, const int* ni, int height_col, int n) {
  const int64_t octree_h = (int64_t)height << (3 * (stride - 1));
  for (int c = 0; c < channel; ++c)
    for (int k = 0; k < kernel_sdim; ++k) {
      int64_t h_start = (int64_t)n * height_col;
      int64_t i_start = ((int64_t)c * kernel_sdim + k) * height_col - h_start;
      for (int64_t h = h_start; h < h_start + height_col; ++h) {
        if (h >= height) { col[i_start + h] = 0.0f; continue; }
        int64_t index = stride == 2 ? (h << 6) + ni[k] : (h >> 3 << 6) + ni[(h % 8) * kernel_sdim + k];
        int p = neigh[index];
        col[i_start + h] = p == -1 ? 0.0f : data[c * octree_h + p];
      }
    }
}
void orc_col2octree(const float* col, float* data, int channel, int height,
    int kernel_sdim, int stride, const int* neigh, const int* ni, int height_col, int n) {
  const int64_t octree_h = (int64_t)height << (3 * (stride - 1));
  if (n == 0) memset(data, 0, sizeof(float) * (size_t)(channel * octree_h));
  for (int c = 0; c < channel; ++c)
    for (int k = 0; k < kernel_sdim; ++k) {
      int64_t h_start = (int64_t)n * height_col;
      int64_t i_start = ((int64_t)c * kernel_sdim + k) * height_col - h_start;
      for (int64_t h = h_start; h < h_start + height_col; ++h) {
        if (h >= height) continue;
        int64_t index = stride == 2 ? (h << 6) + ni[k] : (h >> 3 << 6) + ni[(h % 8) * kernel_sdim + k];
        int p = neigh[index];
        if (p != -1) data[c * octree_h + p] += col[i_start + h];
      }
    }
}
/* octree_nn.cpp:244-298 */
void orc_octree2colP(float* col, const float* data, int channel, int height,
    int octree_h, int kernel_sdim, int stride, const int* neigh, const int* ni,
    const int* child, const int* ichild, int height_col, int n) {
  for (int c = 0; c < channel; ++c)
    for (int k = 0; k < kernel_sdim; ++k) {
      int64_t h_start = (int64_t)n * height_col;
      int64_t i_start = ((int64_t)c * kernel_sdim + k) * height_col - h_start;
      for (int64_t h = h_start; h < h_start + height_col; ++h) {
        if (h >= height) { col[i_start + h] = 0.0f; continue; }
        int64_t index;
        if (stride == 2) index = (h << 6) + ni[k];
        else { int hp = ichild[h]; index = ((int64_t)hp >> 3 << 6) + ni[(hp % 8) * kernel_sdim + k]; }
        int p = neigh[index];
        if (p >= 0) p = child[p];
        col[i_start + h] = p < 0 ? 0.0f : data[(int64_t)c * octree_h + p];
      }
    }
}
void orc_col2octreeP(const float* col, float* data, int channel, int height,
    int octree_h, int kernel_sdim, int stride, const int* neigh, const int* ni,
    const int* child, const int* ichild, int height_col, int n) {
  if (n == 0) memset(data, 0, sizeof(float) * (size_t)channel * (size_t)octree_h);
  for (int c = 0; c < channel; ++c)
    for (int k = 0; k < kernel_sdim; ++k) {
      int64_t h_start = (int64_t)n * height_col;
      int64_t i_start = ((int64_t)c * kernel_sdim + k) * height_col - h_start;
      for (int64_t h = h_start; h < h_start + height_col; ++h) {
        if (h >= height) continue;
        int64_t index;
        if (stride == 2) index = (h << 6) + ni[k];
        else { int hp = ichild[h]; index = ((int64_t)hp >> 3 << 6) + ni[(hp % 8) * kernel_sdim + k]; }
        int p = neigh[index];
        if (p >= 0) p = child[p];
        if (p >= 0) data[(int64_t)c * octree_h + p] += col[i_start + h];
      }
    }
}

/* octree_nn.cpp:301-354 */
void orc_max_pool(float* top, int top_h, int* mask, const float* btm, int btm_h, int channel) {
  for (int c = 0; c < channel; ++c) {
    for (int h = 0; h < top_h; ++h) {
      int hb = 8 * h;
      top[h] = btm[hb]; mask[h] = hb;
      for (int idx = hb + 1; idx < hb + 8; ++idx)
        if (btm[idx] > top[h]) { top[h] = btm[idx]; mask[h] = idx; }
    }
    mask += top_h; top += top_h; btm += btm_h;
  }
}
void orc_max_unpool(const float* top, int top_h, const int* mask, float* btm, int btm_h, int channel) {
  memset(btm, 0, sizeof(float) * (size_t)btm_h * (size_t)channel);
  for (int c = 0; c < channel; ++c) {
    for (int h = 0; h < top_h; ++h) btm[mask[h]] = top[h];
    mask += top_h; top += top_h; btm += btm_h;
  }
}
void orc_mask_pool(float* top, int top_h, const int* mask, const float* btm, int btm_h, int channel) {
  for (int c = 0; c < channel; ++c) {
    for (int h = 0; h < top_h; ++h) top[h] = btm[mask[h]];
    mask += top_h; top += top_h; btm += btm_h;
  }
}

/* ------------------------------------------------------------------------ */
/* Textbook SGEMM, row-major, k ascending per output element.  The reference
 * ships no CPU GEMMEngine (octree/octree/octree_conv.h:86 is only a pointer);
 * its data flow is octree/octree/octree_conv.cpp:157-207. */
void orc_sgemm(int transA, int transB, int M, int N, int K, const float* A,
    const float* B, float beta, float* C) {
  for (int m = 0; m < M; ++m) {
    float* c = C + (int64_t)m * N;
    if (beta == 0.0f) memset(c, 0, sizeof(float) * (size_t)N);
    else if (beta != 1.0f) for (int n = 0; n < N; ++n) c[n] *= beta;
    for (int k = 0; k < K; ++k) {
      float a = transA ? A[(int64_t)k * M + m] : A[(int64_t)m * K + k];
      if (!transB) {
        const float* b = B + (int64_t)k * N;
        for (int n = 0; n < N; ++n) c[n] += a * b[n];
      } else {
        for (int n = 0; n < N; ++n) c[n] += a * B[(int64_t)n * K + k];
      }
    }
  }
}

/* Shape rules of OctreeBaseConv::reshape (octree/octree/octree_conv.cpp:48-104). */
typedef struct {
  int top_depth, workspace_depth, top_h, workspace_h, child_h, ichild_h, octree_h;
} ConvShape;
static int conv_shape(const OInfo* o, int depth, int stride, int nempty, int deconv, ConvShape* s) {
  s->top_depth = s->workspace_depth = depth;
  if (stride == 2) {
    if (deconv) s->top_depth = s->workspace_depth = depth + 1;
    else s->top_depth = depth - 1;
    if (!(0 <= s->top_depth && s->top_depth <= o->depth)) return ORC_E_BADARG;
  }
  int top_h;
  if (!nempty) {
    top_h = o->nnum[s->top_depth];
    if (stride == 2 && !deconv) top_h = o->nnum_nempty[s->top_depth];
  } else top_h = o->nnum_nempty[s->top_depth];
  if (top_h == 0) top_h = 1;
  s->top_h = top_h;
  s->workspace_h = top_h;
  if (stride == 2) s->workspace_h = deconv ? o->nnum[s->top_depth] / 8 : o->nnum[depth] / 8;
  s->child_h = s->ichild_h = s->octree_h = 0;
  if (nempty) {
    s->child_h = o->nnum[s->workspace_depth];
    s->ichild_h = o->nnum_nempty[s->workspace_depth];
    s->octree_h = o->nnum_nempty[depth];
    if (stride == 2 && deconv) s->octree_h = o->nnum_nempty[s->top_depth];
  }
  return 0;
}
int orc_conv_top_h(const void* blob, int depth, int stride, int nempty, int is_deconv) {
  ConvShape s;
  int e = conv_shape((const OInfo*)blob, depth, stride, nempty, is_deconv, &s);
  return e < 0 ? e : s.top_h;
}
static int check_btm_h(const OInfo* o, int depth, int stride, int nempty, int deconv, int btm_h) {
  /* pytorch/cpp/octree_conv.cpp:72-78 */
  if ((stride == 2 && deconv) || nempty) return btm_h == o->nnum_nempty[depth];
  return btm_h == o->nnum[depth];
}
static int* make_ichild(const OInfo* o, const int* child, const ConvShape* s) {
  /* pytorch/cpp/octree_conv.cpp:108-117 */
  (void)o;
  int* seq = (int*)malloc(sizeof(int) * (size_t)(s->child_h + 1));
  int* ichild = (int*)calloc((size_t)(s->ichild_h + 1), sizeof(int));
  for (int i = 0; i < s->child_h; ++i) seq[i] = i;
  pad_backward_int(ichild, seq, s->child_h, child);
  free(seq);
  return ichild;
}
int orc_octree_conv(float* top, const float* btm, int channel_in, int btm_h,
    const float* weights, const void* blob, int depth, int num_output,
    const int* ks, int stride, int nempty) {
  const OInfo* o = (const OInfo*)blob;
  ConvShape s; int ni[216];
  if (depth <= 0 || num_output <= 0 || (stride != 1 && stride != 2)) return ORC_E_BADARG;
  int e = conv_shape(o, depth, stride, nempty, 0, &s); if (e < 0) return e;
  int nni = orc_get_ni(ks, ni); if (nni < 0) return nni;
  if (!check_btm_h(o, depth, stride, nempty, 0, btm_h)) return ORC_E_BADARG;
  int ksdim = ks[0] * ks[1] * ks[2], kdim = ksdim * channel_in;
  const int* neigh = (const int*)prop_ptr(blob, kNeigh, s.workspace_depth);
  float* col = (float*)malloc(sizeof(float) * (size_t)kdim * (size_t)s.workspace_h + 4);
  if (!col) return ORC_E_NOMEM;
  if (!nempty) {
    orc_octree2col(col, btm, channel_in, s.workspace_h, ksdim, stride, neigh, ni, s.workspace_h, 0);
  } else {
    const int* child = (const int*)prop_ptr(blob, kChild, s.workspace_depth);
    int* ichild = make_ichild(o, child, &s);
    orc_octree2colP(col, btm, channel_in, s.workspace_h, s.octree_h, ksdim, stride, neigh, ni,
        child, ichild, s.workspace_h, 0);
    free(ichild);
  }
  orc_sgemm(0, 0, num_output, s.workspace_h, kdim, weights, col, 0.0f, top);
  free(col);
  return s.top_h;
}
int orc_octree_deconv(float* top, const float* btm, int channel_in, int btm_h,
    const float* weights, const void* blob, int depth, int num_output,
    const int* ks, int stride, int nempty) {
  const OInfo* o = (const OInfo*)blob;
  ConvShape s; int ni[216];
  if (depth <= 0 || num_output <= 0 || (stride != 1 && stride != 2)) return ORC_E_BADARG;
  int e = conv_shape(o, depth, stride, nempty, 1, &s); if (e < 0) return e;
  int nni = orc_get_ni(ks, ni); if (nni < 0) return nni;
  if (!check_btm_h(o, depth, stride, nempty, 1, btm_h)) return ORC_E_BADARG;
  /* deconv: conv_out_channels = channel_in, conv_in_channels = num_output
   * (octree_conv.cpp:31-35); forward is backward_cpu_gemm
   * (pytorch/cpp/octree_conv.cpp:212). */
  int ksdim = ks[0] * ks[1] * ks[2], kdim = ksdim * num_output;
  const int* neigh = (const int*)prop_ptr(blob, kNeigh, s.workspace_depth);
  float* col = (float*)malloc(sizeof(float) * (size_t)kdim * (size_t)s.workspace_h + 4);
  if (!col) return ORC_E_NOMEM;
  orc_sgemm(1, 0, kdim, s.workspace_h, channel_in, weights, btm, 0.0f, col);
  if (!nempty) {
    orc_col2octree(col, top, num_output, s.workspace_h, ksdim, stride, neigh, ni, s.workspace_h, 0);
  } else {
    const int* child = (const int*)prop_ptr(blob, kChild, s.workspace_depth);
    int* ichild = make_ichild(o, child, &s);
    orc_col2octreeP(col, top, num_output, s.workspace_h, s.octree_h, ksdim, stride, neigh, ni,
        child, ichild, s.workspace_h, 0);
    free(ichild);
  }
  free(col);
  return s.top_h;
}


/* Gradients: OctreeConvGradOp / OctreeDeconvGradOp (pytorch/cpp/octree_conv.cpp:159-250) over
 * weight_cpu_gemm / backward_cpu_gemm / forward_cpu_gemm (octree_conv.cpp:190-268).
 *   conv:   grad_w[Co, Ci*K]  = grad_out[Co, H'] * octree2col(data_in)^T
 *           grad_data         = col2octree(W^T * grad_out)          (== deconv of grad_out)
 *   deconv: grad_w[Ci, Co*K]  = data_in[Ci, H'] * octree2col(grad_out)^T
 *           grad_data         = W * octree2col(grad_out)             (== conv of grad_out) */
static int conv_col(float* col, const float* x, int channel, const void* blob, const ConvShape* s,
    int ksdim, int stride, int nempty, const int* ni) {
  const OInfo* o = (const OInfo*)blob;
  const int* neigh = (const int*)prop_ptr(blob, kNeigh, s->workspace_depth);
  if (!nempty) {
    orc_octree2col(col, x, channel, s->workspace_h, ksdim, stride, neigh, ni, s->workspace_h, 0);
  } else {
    const int* child = (const int*)prop_ptr(blob, kChild, s->workspace_depth);
    int* ichild = make_ichild(o, child, s);
    orc_octree2colP(col, x, channel, s->workspace_h, s->octree_h, ksdim, stride, neigh, ni,
        child, ichild, s->workspace_h, 0);
    free(ichild);
  }
  return 0;
}
int orc_octree_conv_grad(float* grad_data, float* grad_w, const float* data_in, int channel_in, int btm_h,
    const float* weights, const float* grad_out, const void* blob, int depth, int num_output,
    const int* ks, int stride, int nempty) {
  const OInfo* o = (const OInfo*)blob;
  ConvShape s; int ni[216];
  if (depth <= 0 || num_output <= 0 || (stride != 1 && stride != 2)) return ORC_E_BADARG;
  int e = conv_shape(o, depth, stride, nempty, 0, &s); if (e < 0) return e;
  int nni = orc_get_ni(ks, ni); if (nni < 0) return nni;
  if (!check_btm_h(o, depth, stride, nempty, 0, btm_h)) return ORC_E_BADARG;
  int ksdim = ks[0] * ks[1] * ks[2], kdim = ksdim * channel_in;
  float* col = (float*)malloc(sizeof(float) * (size_t)kdim * (size_t)s.workspace_h + 4);
  if (!col) return ORC_E_NOMEM;
  conv_col(col, data_in, channel_in, blob, &s, ksdim, stride, nempty, ni);
  /* weight_cpu_gemm: weights_diff (zeroed) += top_diff * col^T */
  orc_sgemm(0, 1, num_output, kdim, s.workspace_h, grad_out, col, 0.0f, grad_w);
  /* backward_cpu_gemm: col_diff = W^T * top_diff, then col2octree */
  orc_sgemm(1, 0, kdim, s.workspace_h, num_output, weights, grad_out, 0.0f, col);
  const int* neigh = (const int*)prop_ptr(blob, kNeigh, s.workspace_depth);
  if (!nempty) {
    orc_col2octree(col, grad_data, channel_in, s.workspace_h, ksdim, stride, neigh, ni, s.workspace_h, 0);
  } else {
    const int* child = (const int*)prop_ptr(blob, kChild, s.workspace_depth);
    int* ichild = make_ichild(o, child, &s);
    orc_col2octreeP(col, grad_data, channel_in, s.workspace_h, s.octree_h, ksdim, stride, neigh, ni,
        child, ichild, s.workspace_h, 0);
    free(ichild);
  }
  free(col);
  return btm_h;
}
int orc_octree_deconv_grad(float* grad_data, float* grad_w, const float* data_in, int channel_in, int btm_h,
    const float* weights, const float* grad_out, const void* blob, int depth, int num_output,
    const int* ks, int stride, int nempty) {
  const OInfo* o = (const OInfo*)blob;
  ConvShape s; int ni[216];
  if (depth <= 0 || num_output <= 0 || (stride != 1 && stride != 2)) return ORC_E_BADARG;
  int e = conv_shape(o, depth, stride, nempty, 1, &s); if (e < 0) return e;
  int nni = orc_get_ni(ks, ni); if (nni < 0) return nni;
  if (!check_btm_h(o, depth, stride, nempty, 1, btm_h)) return ORC_E_BADARG;
  int ksdim = ks[0] * ks[1] * ks[2], kdim = ksdim * num_output;
  float* col = (float*)malloc(sizeof(float) * (size_t)kdim * (size_t)s.workspace_h + 4);
  if (!col) return ORC_E_NOMEM;
  conv_col(col, grad_out, num_output, blob, &s, ksdim, stride, nempty, ni);
  orc_sgemm(0, 1, channel_in, kdim, s.workspace_h, data_in, col, 0.0f, grad_w);
  orc_sgemm(0, 0, channel_in, s.workspace_h, kdim, weights, col, 0.0f, grad_data);
  free(col);
  return btm_h;
}

/* ------------------------------------------------------------------------ */
/* points2octree: pytorch/cpp/point2octree.cpp:5-34,
 * OctreeInfo::initialize octree/octree/octree_info.cpp:13-73,
 * Octree::build octree/octree/octree.cpp:74-121. */
typedef struct { uint64_t key, idx; } Code;
static int code_cmp(const void* a, const void* b) { /* std::sort of pair<key,idx>: octree.cpp:193 */
  const Code* x = (const Code*)a; const Code* y = (const Code*)b;
  if (x->key != y->key) return x->key < y->key ? -1 : 1;
  if (x->idx != y->idx) return x->idx < y->idx ? -1 : 1;
  return 0;
}
/* octree.cpp:890-904: in-place unique, returns new size, idx gets n_unique+1 entries */
static int unique_key(uint64_t* keys, int n, uint64_t* idx) {
  int ni = 0, j = 1;
  idx[ni++] = 0;
  for (int i = 1; i < n; i++)
    if (keys[i] != keys[i - 1]) { idx[ni++] = (uint64_t)i; keys[j++] = keys[i]; }
  idx[ni] = (uint64_t)n;
  return n > 0 ? j : 0;
}


/* ---- all-depth signals, extrapolation and trimming of Octree::build -------- */
/* MarchingCube::corner_ / edge_vert_ conventions, marching_cube_table.cpp:312-321.
 * The edge mask of a cube case (edge_table_) is the set of edges whose two end
 * corners lie on different sides, so it is derived instead of tabulated. */
static const float kCorner[8][3] = {
  { 0, 0, 0 }, { 0, 0, 1 }, { 0, 1, 1 }, { 0, 1, 0 }, { 1, 0, 0 }, { 1, 0, 1 }, { 1, 1, 1 }, { 1, 1, 0 } };
static const int kEdgeVert[12][2] = {
  { 0, 1 }, { 1, 2 }, { 2, 3 }, { 3, 0 }, { 4, 5 }, { 5, 6 }, { 6, 7 }, { 7, 4 }, { 0, 4 }, { 1, 5 }, { 2, 6 }, { 3, 7 } };
/* intersect_cube, marching_cube.cpp:83-98 with MarchingCube::contouring :40-65 (vertices only) */
static int intersect_cube(float* V, const float* pt, const float* pt_base, const float* normal) {
  float fval[8];
  for (int k = 0; k < 8; ++k) {
    fval[k] = 0.0f;
    for (int j = 0; j < 3; ++j) fval[k] += (kCorner[k][j] + pt_base[j] - pt[j]) * normal[j];
  }
  unsigned cube_case = 0;
  for (int i = 0; i < 8; ++i) if (fval[i] < 0.0f) cube_case |= 1u << i;
  int nv = 0;
  for (int e = 0; e < 12; ++e) {
    int v1 = kEdgeVert[e][0], v2 = kEdgeVert[e][1];
    if ((((cube_case >> v1) ^ (cube_case >> v2)) & 1u) == 0) continue;
    float df = fval[v2] - fval[v1];
    if (df == 0) df += 1.0e-10f;
    float t = -fval[v1] / df;
    for (int j = 0; j < 3; ++j) {
      float pj = kCorner[v1][j] + t * (kCorner[v2][j] - kCorner[v1][j]);
      V[3 * nv + j] = pj + pt_base[j];
    }
    nv++;
  }
  return nv;
}
static float norm2f(const float* v, int n) { /* math_functions.cpp:257-263 */
  float len = 0.0f;
  for (int i = 0; i < n; ++i) len += v[i] * v[i];
  return sqrtf(len);
}
/* OctreeParser::key2xyz<float>, octree_parser.cpp:151-165: with the key2xyz flag the
 * (still Morton) key is read as packed 16-bit fields, exactly as the reference does. */
static void key2xyz_f(float* xyz, uint64_t key, int depth, int flag) {
  if (flag) {
    uint16_t f[4]; memcpy(f, &key, 8);
    for (int c = 0; c < 3; ++c) xyz[c] = (float)f[c];
  } else {
    uint64_t pt[3]; compute_pt(pt, key, depth);
    for (int c = 0; c < 3; ++c) xyz[c] = (float)pt[c];
  }
}
typedef struct {
  int depth, full_layer, adp_layer, key2xyz;
  int ch_normal, ch_pt, ch_feature, ch_label, ch_dis, max_label;
  int has_dis;
  int nnum[17];
  uint64_t* keys[17]; int* children[17];
  float* normals[17]; float* pts[17]; float* features[17]; float* labels[17]; float* dis[17];
  float* nerr[17]; float* derr[17]; float* split[17];
  int* dnum[17]; int* didx[17];
} Tree;

/* covered_depth_nodes, octree.cpp:958-1002 */
static void covered_depth_nodes(Tree* t) {
  const int D = t->depth;
  for (int d = 0; d <= D; ++d) {
    t->dnum[d] = (int*)calloc((size_t)t->nnum[d] + 1, sizeof(int));
    t->didx[d] = (int*)malloc(sizeof(int) * ((size_t)t->nnum[d] + 1));
    for (int i = 0; i < t->nnum[d]; ++i) t->didx[d][i] = -1;
  }
  for (int i = 0; i < t->nnum[D]; ++i) { t->dnum[D][i] = 1; t->didx[D][i] = i; }
  for (int i = 0; i < t->nnum[D - 1]; ++i) {
    int c = t->children[D - 1][i];
    if (c == -1) continue;
    t->dnum[D - 1][i] = 8; t->didx[D - 1][i] = c * 8;
  }
  for (int d = D - 2; d >= 0; --d)
    for (int i = 0; i < t->nnum[d]; ++i) {
      int c = t->children[d][i];
      if (c == -1) continue;
      c *= 8;
      for (int j = 0; j < 8; ++j) t->dnum[d][i] += t->dnum[d + 1][c + j];
      for (int j = 0; j < 8; ++j)
        if (t->didx[d + 1][c + j] != -1) { t->didx[d][i] = t->didx[d + 1][c + j]; break; }
    }
}

/* calc_signal(calc_normal_err, calc_dist_err), octree.cpp:454-664 */
static void calc_signal_all(Tree* t, int calc_normal_err, int calc_dist_err) {
  const int D = t->depth, nD = t->nnum[D];
  const float imul = 2.0f / sqrtf(3.0f);
  const int* child_D = t->children[D];
  const float* nrm_D = t->normals[D]; const float* pt_D = t->pts[D];
  const float* feat_D = t->features[D]; const float* lab_D = t->labels[D];
  const int cn = t->ch_normal, cp = t->ch_pt, cf = t->ch_feature;
  const int has_normal = nrm_D != NULL, has_pt = pt_D != NULL, has_feature = feat_D != NULL,
      has_label = lab_D != NULL, has_dis = t->dis[D] != NULL;
  if (calc_normal_err) { t->nerr[D] = (float*)malloc(sizeof(float) * ((size_t)nD + 1)); for (int i = 0; i < nD; ++i) t->nerr[D][i] = 1.0e20f; }
  if (calc_dist_err) { t->derr[D] = (float*)malloc(sizeof(float) * ((size_t)nD + 1)); for (int i = 0; i < nD; ++i) t->derr[D][i] = 1.0e20f; }
  float* n_avg = (float*)calloc((size_t)(cn > 3 ? cn : 3) + 1, sizeof(float));
  float* f_avg = (float*)calloc((size_t)cf + 1, sizeof(float));
  int* l_avg = (int*)calloc((size_t)(t->max_label > 0 ? t->max_label : 1), sizeof(int));
  for (int d = D - 1; d >= 0; --d) {
    const int n = t->nnum[d];
    const int* dnum = t->dnum[d]; const int* didx = t->didx[d]; const int* child = t->children[d];
    const float scale = (float)(1 << (D - d));
    const int ch_dis = has_normal ? 1 : 4;
    if (has_normal) t->normals[d] = (float*)calloc((size_t)n * cn + 1, sizeof(float));
    if (has_pt) t->pts[d] = (float*)calloc((size_t)n * cp + 1, sizeof(float));
    if (has_feature) t->features[d] = (float*)calloc((size_t)n * cf + 1, sizeof(float));
    if (has_label) { t->labels[d] = (float*)malloc(sizeof(float) * ((size_t)n + 1)); for (int i = 0; i < n; ++i) t->labels[d][i] = -1.0f; }
    if (has_dis) t->dis[d] = (float*)calloc((size_t)n * ch_dis + 1, sizeof(float));
    if (calc_normal_err) { t->nerr[d] = (float*)malloc(sizeof(float) * ((size_t)n + 1)); for (int i = 0; i < n; ++i) t->nerr[d][i] = 1.0e20f; }
    if (calc_dist_err) { t->derr[d] = (float*)malloc(sizeof(float) * ((size_t)n + 1)); for (int i = 0; i < n; ++i) t->derr[d][i] = 1.0e20f; }
    for (int i = 0; i < n; ++i) {
      if (child[i] == -1) continue;
      const int j0 = didx[i], j1 = didx[i] + dnum[i];
      for (int c = 0; c < cn; ++c) n_avg[c] = 0.0f;
      if (has_normal) {
        for (int j = j0; j < j1; ++j) {
          if (child_D[j] == -1) continue;
          for (int c = 0; c < cn; ++c) n_avg[c] += nrm_D[(int64_t)c * nD + j];
        }
        float len = norm2f(n_avg, cn);
        if (len < 1.0e-6f) {
          for (int j = j0; j < j1; ++j) {
            if (child_D[j] == -1) continue;
            for (int c = 0; c < cn; ++c) n_avg[c] = nrm_D[(int64_t)c * nD + j];
          }
          len = norm2f(n_avg, cn) + 1.0e-30f;
        }
        for (int c = 0; c < cn; ++c) { n_avg[c] /= len; t->normals[d][(int64_t)c * n + i] = n_avg[c]; }
      }
      float count = 1.0e-30f;
      for (int j = j0; j < j1; ++j) if (child_D[j] != -1) count += 1.0f;
      float pt_avg[3] = { 0.0f, 0.0f, 0.0f };
      if (has_pt) {
        for (int j = j0; j < j1; ++j) {
          if (child_D[j] == -1) continue;
          for (int c = 0; c < cp; ++c) pt_avg[c] += pt_D[(int64_t)c * nD + j];
        }
        for (int c = 0; c < cp; ++c) { pt_avg[c] /= count * scale; t->pts[d][(int64_t)c * n + i] = pt_avg[c]; }
      }
      if (has_feature) {
        for (int c = 0; c < cf; ++c) f_avg[c] = 0.0f;
        for (int j = j0; j < j1; ++j) {
          if (child_D[j] == -1) continue;
          for (int c = 0; c < cf; ++c) f_avg[c] += feat_D[(int64_t)c * nD + j];
        }
        for (int c = 0; c < cf; ++c) { f_avg[c] /= count; t->features[d][(int64_t)c * n + i] = f_avg[c]; }
      }
      if (has_label) {
        int valid = 0;
        for (int l = 0; l < t->max_label; ++l) l_avg[l] = 0;
        for (int j = j0; j < j1; ++j) {
          int l = (int)lab_D[j];
          if (l < 0) continue;
          l_avg[l] += 1; valid += 1;
        }
        if (valid > 0) {
          int best = 0;
          for (int l = 1; l < t->max_label; ++l) if (l_avg[l] > l_avg[best]) best = l;
          t->labels[d][i] = (float)best;
        }
      }
      uint64_t ptu[3]; compute_pt(ptu, t->keys[d][i], d);
      float pt_base[3] = { (float)ptu[0], (float)ptu[1], (float)ptu[2] };
      if (has_dis) {
        float dis_avg[4] = { 0.0f, 0.0f, 0.0f, 0.0f };
        for (int c = 0; c < 3; ++c) {
          float fract = pt_avg[c] - pt_base[c];
          dis_avg[c] = fract - 0.5f;
          if (has_normal) dis_avg[3] += dis_avg[c] * n_avg[c]; else dis_avg[3] = 1.0f;
        }
        if (!has_normal) {
          for (int c = 0; c < 3; ++c) t->dis[d][(int64_t)c * n + i] = dis_avg[c];
          t->dis[d][3 * (int64_t)n + i] = dis_avg[3] * imul;
        } else t->dis[d][i] = dis_avg[3] * imul;
      }
      if (calc_normal_err && has_normal && d >= t->adp_layer) {
        float nm_err = 0.0f;
        for (int j = j0; j < j1; ++j) {
          if (child_D[j] == -1) continue;
          for (int c = 0; c < 3; ++c) { float tmp = nrm_D[(int64_t)c * nD + j] - n_avg[c]; nm_err += tmp * tmp; }
        }
        nm_err /= count;
        t->nerr[d][i] = nm_err;
      }
      if (calc_dist_err && has_pt && d >= t->adp_layer) {
        float distance_max1 = -1.0f;
        float pt_avg1[3] = { pt_avg[0] * scale, pt_avg[1] * scale, pt_avg[2] * scale };
        for (int j = j0; j < j1; ++j) {
          if (child_D[j] == -1) continue;
          float dis = 0.0f;
          for (int c = 0; c < 3; ++c) dis += (pt_D[(int64_t)c * nD + j] - pt_avg1[c]) * n_avg[c];
          dis = fabsf(dis);
          if (dis > distance_max1) distance_max1 = dis;
        }
        float distance_max2 = -1.0f;
        float vtx[36];
        int nv = intersect_cube(vtx, pt_avg, pt_base, n_avg);
        if (nv == 0) distance_max2 = 5.0e10f;
        for (int k = 0; k < 3 * nv; ++k) vtx[k] *= scale;
        for (int k = 0; k < nv; ++k) {
          float distance_min = 1.0e30f;
          for (int j = j0; j < j1; ++j) {
            if (child_D[j] == -1) continue;
            float dis = 0.0f;
            for (int c = 0; c < 3; ++c) { float ptc = pt_D[(int64_t)c * nD + j] - vtx[3 * k + c]; dis += ptc * ptc; }
            dis = sqrtf(dis);
            if (dis < distance_min) distance_min = dis;
          }
          if (distance_min > distance_max2) distance_max2 = distance_min;
        }
        t->derr[d][i] = distance_max2 > distance_max1 ? distance_max2 : distance_max1;
      }
    }
  }
  free(n_avg); free(f_avg); free(l_avg);
}

/* calc_split_label, octree.cpp:1158-1178 */
static void calc_split_label(Tree* t, int adaptive) {
  for (int d = 0; d <= t->depth; ++d) {
    const int n = t->nnum[d];
    free(t->split[d]);
    t->split[d] = (float*)malloc(sizeof(float) * ((size_t)n + 1));
    for (int i = 0; i < n; ++i) {
      t->split[d][i] = 1.0f;
      if (t->children[d][i] == -1) {
        t->split[d][i] = 0.0f;
        if (adaptive) {
          float a = fabsf(t->normals[d][i]) + fabsf(t->normals[d][n + i]) + fabsf(t->normals[d][2 * (int64_t)n + i]);
          if (a != 0) t->split[d][i] = 2.0f;
        }
      }
    }
  }
}

/* extrapolate_signal, octree.cpp:666-806 */
static void extrapolate_signal(Tree* t) {
  const int D = t->depth;
  const float imul = 2.0f / sqrtf(3.0f);
  const int cn = t->ch_normal, cf = t->ch_feature;
  const int has_dis = t->dis[D] != NULL, has_normal = t->normals[D] != NULL,
      has_feature = t->features[D] != NULL, has_label = t->labels[D] != NULL;
  static const float xyzs[8][3] = { { 0, 0, 0 }, { 0, 0, 1 }, { 0, 1, 0 }, { 0, 1, 1 }, { 1, 0, 0 }, { 1, 0, 1 }, { 1, 1, 0 }, { 1, 1, 1 } };
  float* n_avg = (float*)calloc((size_t)(cn > 3 ? cn : 3) + 1, sizeof(float));
  float* f_avg = (float*)calloc((size_t)cf + 1, sizeof(float));
  int* l_avg = (int*)calloc((size_t)(t->max_label > 0 ? t->max_label : 1), sizeof(int));
  for (int d = D; d >= t->full_layer; --d) {
    const int n = t->nnum[d];
    const int* child = t->children[d];
    float* normal_d = t->normals[d]; float* label_d = t->labels[d];
    float* feature_d = t->features[d]; float* dis_d = t->dis[d];
    for (int i = 0; i < n; ++i) {
      if (child[i] != -1) continue;
      const int id = i % 8, i_base = i - id;
      float count = 1.0e-30f;
      for (int j = i_base; j < i_base + 8; ++j) if (child[j] != -1) count += 1.0f;
      for (int c = 0; c < (cn > 3 ? cn : 3); ++c) n_avg[c] = 0.0f;
      if (has_normal) {
        for (int j = i_base; j < i_base + 8; ++j) {
          if (child[j] == -1) continue;
          for (int c = 0; c < cn; ++c) n_avg[c] += normal_d[(int64_t)c * n + j];
        }
        float ilen = 1.0f / (norm2f(n_avg, cn) + 1.0e-30f);
        for (int c = 0; c < cn; ++c) { n_avg[c] *= ilen; normal_d[(int64_t)c * n + i] = n_avg[c]; }
      }
      if (has_feature) {
        for (int c = 0; c < cf; ++c) f_avg[c] = 0.0f;
        for (int j = i_base; j < i_base + 8; ++j) {
          if (child[j] == -1) continue;
          for (int c = 0; c < cf; ++c) f_avg[c] += feature_d[(int64_t)c * n + j];
        }
        for (int c = 0; c < cf; ++c) { f_avg[c] /= count; feature_d[(int64_t)c * n + i] = f_avg[c]; }
      }
      if (has_label) {
        int valid = 0;
        for (int l = 0; l < t->max_label; ++l) l_avg[l] = 0;
        for (int j = i_base; j < i_base + 8; ++j) {
          int l = (int)label_d[j];
          if (l < 0) continue;
          l_avg[l] += 1; valid += 1;
        }
        if (valid > 0) {
          int best = 0;
          for (int l = 1; l < t->max_label; ++l) if (l_avg[l] > l_avg[best]) best = l;
          label_d[i] = (float)best;
        }
      }
      if (has_dis && count > 0.5f) {
        float dis = 0;
        for (int j = i_base; j < i_base + 8; ++j) {
          if (child[j] == -1) continue;
          dis += dis_d[j];
          for (int c = 0; c < cn; ++c) dis += normal_d[(int64_t)c * n + j] * (xyzs[j % 8][c] - xyzs[id][c]) * imul;
        }
        dis /= count;
        if (dis > 3.0f) dis = 3.0f;
        if (dis < -3.0f) dis = -3.0f;
        if (fabsf(dis) < 1.0f) {
          unsigned cube_cases = 0;
          for (int k = 0; k < 8; ++k) {
            float fval = dis;
            for (int j = 0; j < 3; ++j) fval += (0.5f - kCorner[k][j]) * n_avg[j] * imul;
            if (fval < 0) cube_cases |= 1u << k;
          }
          if (cube_cases != 255 && cube_cases != 0) dis = dis < 0 ? -1.0f : 1.0f;
        }
        dis_d[i] = dis;
      }
      if (has_dis && count < 0.5f) {
        int j_min = -1;
        float pti[3], ptj[3], dis_min = 1.0e30f;
        key2xyz_f(pti, t->keys[d][i], d, t->key2xyz);
        for (int j = 0; j < n; ++j) {
          if (child[j] == -1) continue;
          key2xyz_f(ptj, t->keys[d][j], d, t->key2xyz);
          float dd = fabsf(pti[0] - ptj[0]) + fabsf(pti[1] - ptj[1]) + fabsf(pti[2] - ptj[2]);
          if (dd < dis_min) { dis_min = dd; j_min = j; }
        }
        if (j_min < 0) continue; /* the reference indexes with -1 here (undefined); no such layer is ever built */
        float dis = dis_d[j_min];
        key2xyz_f(ptj, t->keys[d][j_min], d, t->key2xyz);
        for (int c = 0; c < cn; ++c) dis += normal_d[(int64_t)c * n + j_min] * (ptj[c] - pti[c]) * imul;
        if (dis > 0.0f) dis = 2.0f;
        if (dis < 0.0f) dis = -2.0f;
        dis_d[i] = dis;
      }
    }
  }
  free(n_avg); free(f_avg); free(l_avg);
}

/* trim_octree (structure and signals), octree.cpp:1004-1135 */
static void trim_signal(float** sig, int channel, int n_old, const unsigned char* drop, int n_new) {
  if (!*sig || channel == 0) return;
  float* out = (float*)malloc(sizeof(float) * ((size_t)n_new * channel + 1));
  int k = 0;
  for (int i = 0; i < n_old; ++i) {
    if (drop[i] == 0) continue;
    for (int c = 0; c < channel; ++c) out[(int64_t)c * n_new + k] = (*sig)[(int64_t)c * n_old + i];
    k++;
  }
  free(*sig); *sig = out;
}
static void trim_octree(Tree* t, float th_dist, float th_norm) {
  enum { kDrop = 0, kDropChildren = 1, kKeep = 2 };
  const int D = t->depth, A = t->adp_layer;
  unsigned char* drop[17];
  for (int d = 0; d <= D; ++d) { drop[d] = (unsigned char*)malloc((size_t)t->nnum[d] + 1); memset(drop[d], kKeep, (size_t)t->nnum[d] + 1); }
  for (int d = A; d <= D; ++d) {
    const int n_dp = t->nnum[d - 1];
    const int* child_d = t->children[d]; const int* child_dp = t->children[d - 1];
    int all_drop = 1;
    for (int i = 0; i < n_dp; ++i) {
      int c = child_dp[i];
      if (c == -1) continue;
      for (int j = 0; j < 8; ++j) {
        int idx = c * 8 + j;
        if (drop[d - 1][i] == kKeep) {
          if ((!t->has_dis || t->derr[d][idx] < th_dist) && t->nerr[d][idx] < th_norm) drop[d][idx] = kDropChildren;
        } else drop[d][idx] = kDrop;
        if (all_drop) all_drop = !(drop[d][idx] == kKeep && child_d[idx] != -1);
      }
    }
    if (all_drop) {
      int max_idx = 0; float max_err = -1.0f;
      for (int i = 0; i < n_dp; ++i) {
        int c = child_dp[i];
        if (c == -1 || drop[d - 1][i] != kKeep) continue;
        for (int j = 0; j < 8; ++j) {
          int idx = c * 8 + j;
          if (child_d[idx] != -1 && t->nerr[d][idx] > max_err) { max_err = t->nerr[d][idx]; max_idx = idx; }
        }
      }
      drop[d][max_idx] = kKeep;
    }
  }
  for (int d = A; d <= D; ++d) {
    const int n = t->nnum[d];
    int n_new = 0;
    for (int i = 0; i < n; ++i) if (drop[d][i] != kDrop) n_new++;
    uint64_t* key = (uint64_t*)malloc(sizeof(uint64_t) * ((size_t)n_new + 1));
    int* ch = (int*)malloc(sizeof(int) * ((size_t)n_new + 1));
    int k = 0, id = 0;
    for (int i = 0; i < n; ++i) {
      if (drop[d][i] == kDrop) continue;
      key[k] = t->keys[d][i];
      ch[k] = (drop[d][i] == kKeep && t->children[d][i] != -1) ? id++ : -1;
      k++;
    }
    free(t->keys[d]); t->keys[d] = key;
    free(t->children[d]); t->children[d] = ch;
    trim_signal(&t->dis[d], t->ch_dis, n, drop[d], n_new);
    trim_signal(&t->normals[d], t->ch_normal, n, drop[d], n_new);
    trim_signal(&t->features[d], t->ch_feature, n, drop[d], n_new);
    trim_signal(&t->labels[d], 1, n, drop[d], n_new);
    t->nnum[d] = n_new;
  }
  for (int d = 0; d <= D; ++d) free(drop[d]);
}

int64_t orc_points2octree(const void* points_blob, int depth, int full_depth,
    int node_dis, int node_feature, int split_label, int adaptive,
    int adp_depth, float th_normal, float th_distance, int extrapolate,
    int save_pts, int key2xyz, const float* bbmin_in, const float* bbmax_in) {
  const PInfo* pi = (const PInfo*)points_blob;
  if (strcmp(pi->magic, "_POINTS_1.0_") != 0 || pi->pt_num <= 0) return ORC_E_BADARG;
  const int npt = pi->pt_num;
  const char* base = (const char*)points_blob;
  const float* pts = (pi->content_flags & pPoint) ? (const float*)(base + pi->ptr_dis[0]) : NULL;
  const float* normals = (pi->content_flags & pNormal) ? (const float*)(base + pi->ptr_dis[1]) : NULL;
  const float* features = (pi->content_flags & pFeature) ? (const float*)(base + pi->ptr_dis[2]) : NULL;
  const float* labels = (pi->content_flags & pLabel) ? (const float*)(base + pi->ptr_dis[3]) : NULL;
  const int ch_normal = normals ? pi->channels[1] : 0;
  const int ch_feature = features ? pi->channels[2] : 0;
  const int ch_label = labels ? pi->channels[3] : 0;
  if (!pts) return ORC_E_BADARG;
  /* trim_octree reads normal_err_ (exists only with normals) and leaves avg_pts_ untrimmed */
  if (adaptive && (!normals || save_pts || adp_depth < 1)) return ORC_E_UNSUPPORTED;

  /* OctreeInfo::initialize, octree_info.cpp:13-73 */
  OInfo o; info_reset(&o);
  set_batch_size(&o, 1);
  set_depth(&o, depth);
  set_full_layer(&o, full_depth);
  o.adp_layer = adp_depth;
  o.is_adaptive = adaptive ? 1 : 0;
  o.has_node_dis = node_dis ? 1 : 0;
  o.key2xyz = key2xyz ? 1 : 0;
  o.extrapolate = extrapolate ? 1 : 0;
  o.save_pts = save_pts ? 1 : 0;
  o.th_norm = th_normal;
  o.th_dist = th_distance;
  set_property(&o, kKey, (key2xyz && depth > 8) ? 2 : 1, -1);
  set_property(&o, kChild, 1, -1);
  if (split_label) set_property(&o, kSplit, 1, -1);
  int channel = ch_normal + ch_feature;
  if (node_dis) { channel += 1; if (ch_normal == 0) channel += 3; }
  if (save_pts) channel += 3;
  set_channel(&o, kFeature, channel);
  set_location(&o, kFeature, (node_feature || adaptive) ? -1 : depth);
  if (ch_label == 1) {
    set_channel(&o, kLabel, 1);
    set_location(&o, kLabel, (node_feature || adaptive) ? -1 : depth);
  }
  for (int i = 0; i < 3; ++i) { o.bbmin[i] = -1.0f; o.bbmax[i] = 1.0f; }
  if (bbmin_in && bbmax_in)
    for (int i = 0; i < 3; ++i) { o.bbmin[i] = bbmin_in[i]; o.bbmax[i] = bbmax_in[i]; }
  depth = o.depth;
  const int full_layer = o.full_layer;
  if (depth < 1 || depth > 16 || full_layer > depth) return ORC_E_BADARG;

  /* normalize_pts, octree.cpp:155-170 */
  const float mul = (float)(1 << depth) / bbox_max_width(&o);
  float* pts_scaled = (float*)malloc(sizeof(float) * 3 * (size_t)npt);
  for (int i = 0; i < npt; i++)
    for (int j = 0; j < 3; j++) pts_scaled[3 * i + j] = (pts[3 * i + j] - o.bbmin[j]) * mul;

  /* sort_keys, octree.cpp:172-203 */
  Code* code = (Code*)malloc(sizeof(Code) * (size_t)npt);
  for (int i = 0; i < npt; i++) {
    uint64_t pt[3];
    for (int j = 0; j < 3; ++j) pt[j] = (uint64_t)pts_scaled[3 * i + j];
    code[i].key = compute_key(pt, depth);
    code[i].idx = (uint64_t)i;
  }
  qsort(code, (size_t)npt, sizeof(Code), code_cmp);
  uint64_t* node_keys = (uint64_t*)malloc(sizeof(uint64_t) * (size_t)npt);
  uint64_t* sorted_idx = (uint64_t*)malloc(sizeof(uint64_t) * (size_t)npt);
  for (int i = 0; i < npt; i++) { node_keys[i] = code[i].key; sorted_idx[i] = code[i].idx; }
  free(code);
  uint64_t* unique_idx = (uint64_t*)malloc(sizeof(uint64_t) * ((size_t)npt + 1));
  int n_keys = unique_key(node_keys, npt, unique_idx);

  /* build_structure, octree.cpp:205-283 */
  uint64_t* keys[17]; int* children[17]; int nnum[17] = { 0 };
  for (int d = 0; d <= 16; ++d) { keys[d] = NULL; children[d] = NULL; }
  for (int d = 0; d <= full_layer; d++) {
    int n = 1 << (3 * d);
    nnum[d] = n;
    keys[d] = (uint64_t*)malloc(sizeof(uint64_t) * (size_t)n);
    children[d] = (int*)malloc(sizeof(int) * (size_t)n);
    for (int i = 0; i < n; i++) { keys[d][i] = (uint64_t)i; children[d][i] = d != full_layer ? i : -1; }
  }
  uint64_t* parent_keys = (uint64_t*)malloc(sizeof(uint64_t) * ((size_t)n_keys + 1));
  uint64_t* parent_pidx = (uint64_t*)malloc(sizeof(uint64_t) * ((size_t)n_keys + 2));
  for (int d = depth; d > full_layer; --d) {
    int n = n_keys;
    for (int i = 0; i < n; i++) parent_keys[i] = node_keys[i] >> 3;
    int np = unique_key(parent_keys, n, parent_pidx);
    int nch = np << 3;
    nnum[d] = nch;
    keys[d] = (uint64_t*)malloc(sizeof(uint64_t) * ((size_t)nch + 1));
    children[d] = (int*)malloc(sizeof(int) * ((size_t)nch + 1));
    for (int i = 0; i < nch; i++) { keys[d][i] = (parent_keys[i >> 3] << 3) | (uint64_t)(i % 8); children[d][i] = -1; }
    for (int i = 0; i < np; i++)
      for (uint64_t j = parent_pidx[i]; j < parent_pidx[i + 1]; j++)
        children[d][(node_keys[j] & 7u) | ((uint64_t)i << 3)] = (int)j;
    memcpy(node_keys, parent_keys, sizeof(uint64_t) * (size_t)np);
    n_keys = np;
  }
  if (depth > full_layer)
    for (int i = 0; i < n_keys; i++) children[full_layer][node_keys[i]] = i;
  free(parent_keys); free(parent_pidx);

  /* calc_node_num, octree.cpp:285-309 */
  for (int d = 0; d <= depth; ++d) {
    o.nnum[d] = nnum[d];
    o.nnum_nempty[d] = 0;
    for (int i = nnum[d] - 1; i >= 0; i--)
      if (children[d][i] != -1) { o.nnum_nempty[d] = children[d][i] + 1; break; }
  }
  set_nnum_cum(&o, 0);
  set_ptr_dis(&o);

  /* calc_signal (finest level), octree.cpp:312-452 */
  const int nn = nnum[depth];
  const int* child_d = children[depth];
  float* avg_normals = NULL; float* avg_features = NULL; float* avg_labels = NULL;
  float* avg_pts = NULL; float* displacement = NULL;
  int ch_dis = 0, max_label_all = 0;
  if (normals) {
    avg_normals = (float*)calloc((size_t)ch_normal * (size_t)nn + 1, sizeof(float));
    float* acc = (float*)malloc(sizeof(float) * (size_t)(ch_normal + 1));
    for (int i = 0; i < nn; i++) {
      int t = child_d[i];
      if (t == -1) continue;
      for (int c = 0; c < ch_normal; ++c) acc[c] = 0.0f;
      for (uint64_t j = unique_idx[t]; j < unique_idx[t + 1]; j++) {
        uint64_t h = sorted_idx[j];
        for (int c = 0; c < ch_normal; ++c) acc[c] += normals[ch_normal * h + c];
      }
      float len = 0.0f;
      for (int c = 0; c < ch_normal; ++c) len += acc[c] * acc[c];
      float factor = sqrtf(len);
      if (factor < 1.0e-6f) {
        uint64_t h = sorted_idx[unique_idx[t]];
        for (int c = 0; c < ch_normal; ++c) acc[c] = normals[ch_normal * h + c];
        len = 0.0f;
        for (int c = 0; c < ch_normal; ++c) len += acc[c] * acc[c];
        factor = sqrtf(len) + 1.0e-30f;
      }
      for (int c = 0; c < ch_normal; ++c) avg_normals[(int64_t)c * nn + i] = acc[c] / factor;
    }
    free(acc);
  }
  if (features) {
    avg_features = (float*)calloc((size_t)ch_feature * (size_t)nn + 1, sizeof(float));
    float* acc = (float*)malloc(sizeof(float) * (size_t)(ch_feature + 1));
    for (int i = 0; i < nn; i++) {
      int t = child_d[i];
      if (t == -1) continue;
      for (int c = 0; c < ch_feature; ++c) acc[c] = 0.0f;
      for (uint64_t j = unique_idx[t]; j < unique_idx[t + 1]; j++) {
        uint64_t h = sorted_idx[j];
        for (int c = 0; c < ch_feature; ++c) acc[c] += features[ch_feature * h + c];
      }
      float factor = (float)(unique_idx[t + 1] - unique_idx[t]) + 1.0e-30f;
      for (int c = 0; c < ch_feature; ++c) avg_features[(int64_t)c * nn + i] = acc[c] / factor;
    }
    free(acc);
  }
  if (labels) {
    avg_labels = (float*)malloc(sizeof(float) * ((size_t)nn + 1));
    for (int i = 0; i < nn; ++i) avg_labels[i] = -1.0f;
    float mx = labels[0];
    for (int i = 1; i < npt; ++i) if (labels[i] > mx) mx = labels[i];
    int max_label = (int)mx + 1;
    max_label_all = max_label;
    int* cnt = (int*)malloc(sizeof(int) * (size_t)(max_label > 0 ? max_label : 1));
    for (int i = 0; i < nn; i++) {
      int t = child_d[i];
      if (t == -1) continue;
      int valid = 0;
      for (int l = 0; l < max_label; ++l) cnt[l] = 0;
      for (uint64_t j = unique_idx[t]; j < unique_idx[t + 1]; j++) {
        int l = (int)labels[sorted_idx[j]];
        if (l < 0) continue;
        cnt[l] += 1; valid += 1;
      }
      if (valid > 0) {
        int best = 0;
        for (int l = 1; l < max_label; ++l) if (cnt[l] > cnt[best]) best = l;
        avg_labels[i] = (float)best;
      }
    }
    free(cnt);
  }
  if (o.has_node_dis || o.save_pts) {
    const float mulD = 1.1547f;
    avg_pts = (float*)calloc(3 * (size_t)nn + 1, sizeof(float));
    ch_dis = normals ? 1 : 4;
    displacement = (float*)calloc((size_t)ch_dis * (size_t)nn + 1, sizeof(float));
    for (int i = 0; i < nn; i++) {
      int t = child_d[i];
      if (t == -1) continue;
      float avg_pt[3] = { 0.0f, 0.0f, 0.0f };
      for (uint64_t j = unique_idx[t]; j < unique_idx[t + 1]; j++) {
        uint64_t h = sorted_idx[j];
        for (int c = 0; c < 3; ++c) avg_pt[c] += pts_scaled[3 * h + c];
      }
      float dis[4] = { 0.0f, 0.0f, 0.0f, 0.0f };
      float factor = (float)(unique_idx[t + 1] - unique_idx[t]) + 1.0e-30f;
      for (int c = 0; c < 3; ++c) {
        avg_pt[c] /= factor;
        float ip = 0.0f;
        float fp = modff(avg_pt[c], &ip);
        dis[c] = fp - 0.5f;
        if (normals) dis[3] += dis[c] * avg_normals[(int64_t)c * nn + i];
        else dis[3] = 1.0f;
        avg_pts[(int64_t)c * nn + i] = avg_pt[c];
      }
      if (normals) displacement[i] = dis[3] * mulD;
      else {
        for (int c = 0; c < 3; ++c) displacement[(int64_t)c * nn + i] = dis[c];
        displacement[3 * (int64_t)nn + i] = dis[3] * mulD;
      }
    }
  }

  /* all-depth signals, split labels, extrapolation, trimming: Octree::build, octree.cpp:96-120 */
  Tree t; memset(&t, 0, sizeof(t));
  t.depth = depth; t.full_layer = full_layer; t.adp_layer = o.adp_layer; t.key2xyz = o.key2xyz;
  t.ch_normal = ch_normal; t.ch_pt = avg_pts ? 3 : 0; t.ch_feature = ch_feature; t.ch_label = avg_labels ? 1 : 0;
  t.ch_dis = ch_dis; t.has_dis = o.has_node_dis; t.max_label = max_label_all;
  for (int d = 0; d <= depth; ++d) { t.nnum[d] = nnum[d]; t.keys[d] = keys[d]; t.children[d] = children[d]; }
  t.normals[depth] = avg_normals; t.features[depth] = avg_features; t.labels[depth] = avg_labels;
  t.pts[depth] = avg_pts; t.dis[depth] = displacement;
  const int all_depths = location_of(&o, kFeature) == -1;
  if (all_depths) {
    covered_depth_nodes(&t);
    calc_signal_all(&t, o.is_adaptive && normals, o.is_adaptive && o.has_node_dis && normals);
  }
  if (split_label) calc_split_label(&t, o.is_adaptive);
  if (o.extrapolate && all_depths) extrapolate_signal(&t);
  if (o.is_adaptive) {
    trim_octree(&t, o.th_dist, o.th_norm);
    for (int d = 0; d <= depth; ++d) { /* calc_node_num, octree.cpp:285-309 */
      o.nnum[d] = t.nnum[d];
      o.nnum_nempty[d] = 0;
      for (int i = t.nnum[d] - 1; i >= 0; i--)
        if (t.children[d][i] != -1) { o.nnum_nempty[d] = t.children[d][i] + 1; break; }
    }
    set_nnum_cum(&o, 0);
    set_ptr_dis(&o);
    if (split_label) calc_split_label(&t, 1);
  }

  /* serialize, octree.cpp:907-956 */
  const int sz = sizeof_octree(&o);
  char* buf = result_alloc(sz);
  if (!buf) return ORC_E_NOMEM;
  memcpy(buf, &o, sizeof(o));
  {
    const int kch = channel_of(&o, kKey);
    uint64_t* kdst = (uint64_t*)prop_ptr(buf, kKey, 0);
    for (int d = 0; d <= depth; ++d) {
      const int n = t.nnum[d];
      if (o.key2xyz) { /* key_to_xyz, octree.cpp:1137-1156: nnum*channel entries, first nnum written */
        memset(kdst, 0, sizeof(uint64_t) * (size_t)n * kch);
        for (int i = 0; i < n; ++i) {
          uint64_t pt[3]; compute_pt(pt, t.keys[d][i], d);
          uint16_t f[4] = { (uint16_t)pt[0], (uint16_t)pt[1], (uint16_t)pt[2], 0 };
          memcpy(kdst + i, f, 8);
        }
      } else memcpy(kdst, t.keys[d], sizeof(uint64_t) * (size_t)n);
      kdst += (o.key2xyz ? (int64_t)n * kch : n);
    }
    int* cdst = (int*)prop_ptr(buf, kChild, 0);
    for (int d = 0; d <= depth; ++d) { memcpy(cdst, t.children[d], sizeof(int) * (size_t)t.nnum[d]); cdst += t.nnum[d]; }
    /* features = normals | displacement | point features | average points, per stored depth */
    float* fdst = (float*)prop_ptr(buf, kFeature, all_depths ? 0 : depth);
    if (fdst)
      for (int d = all_depths ? 0 : depth; d <= depth; ++d) {
        const int64_t n = t.nnum[d];
        if (t.normals[d]) { memcpy(fdst, t.normals[d], sizeof(float) * (size_t)(ch_normal * n)); fdst += ch_normal * n; }
        if (o.has_node_dis && t.dis[d]) { memcpy(fdst, t.dis[d], sizeof(float) * (size_t)(ch_dis * n)); fdst += ch_dis * n; }
        if (t.features[d]) { memcpy(fdst, t.features[d], sizeof(float) * (size_t)(ch_feature * n)); fdst += ch_feature * n; }
        if (o.save_pts && t.pts[d]) { memcpy(fdst, t.pts[d], sizeof(float) * (size_t)(3 * n)); fdst += 3 * n; }
      }
    float* ldst = (float*)prop_ptr(buf, kLabel, all_depths ? 0 : depth);
    if (ldst && avg_labels)
      for (int d = all_depths ? 0 : depth; d <= depth; ++d) { memcpy(ldst, t.labels[d], sizeof(float) * (size_t)t.nnum[d]); ldst += t.nnum[d]; }
    float* sdst = (float*)prop_ptr(buf, kSplit, 0);
    if (sdst)
      for (int d = 0; d <= depth; ++d) { memcpy(sdst, t.split[d], sizeof(float) * (size_t)t.nnum[d]); sdst += t.nnum[d]; }
  }
  for (int d = 0; d <= 16; ++d) {
    free(t.keys[d]); free(t.children[d]); free(t.normals[d]); free(t.features[d]); free(t.labels[d]);
    free(t.pts[d]); free(t.dis[d]); free(t.nerr[d]); free(t.derr[d]); free(t.split[d]); free(t.dnum[d]); free(t.didx[d]);
  }
  free(pts_scaled); free(node_keys); free(sorted_idx); free(unique_idx);
  return sz;
}


/* ------------------------------------------------------------------------ */
/* Point-cloud transforms: pytorch/cpp/transform_points.cpp:7-125 over
 * PointsParser (octree/octree/points_parser.cpp:42-260) and
 * math_functions.cpp:49-251.  Each works on a copy of the blob. */
static float* pprop(char* blob, int bit) { /* points_parser.cpp:22-36 */
  PInfo* pi = (PInfo*)blob;
  int idx = 0; while ((1 << idx) != bit) ++idx;
  if (!(pi->content_flags & bit)) return NULL;
  return (float*)(blob + pi->ptr_dis[idx]);
}
static void bounding_box(float* bbmin, float* bbmax, const float* pt, int npt) { /* math_functions.cpp:113-128 */
  if (npt < 1) return;
  for (int i = 0; i < 3; ++i) bbmin[i] = bbmax[i] = pt[i];
  for (int i = 1; i < npt; ++i)
    for (int j = 0; j < 3; ++j) {
      float tmp = pt[3 * i + j];
      if (tmp < bbmin[j]) bbmin[j] = tmp;
      if (tmp > bbmax[j]) bbmax[j] = tmp;
    }
}
/* the build without Miniball, math_functions.cpp:49-108 */
static void bounding_sphere(float* radius_out, float* center, const float* pt, int npt) {
  float bb[3][2] = { { FLT_MAX, -FLT_MAX }, { FLT_MAX, -FLT_MAX }, { FLT_MAX, -FLT_MAX } };
  int id[6] = { 0, 0, 0, 0, 0, 0 };
  for (int i = 0; i < 3 * npt; i += 3)
    for (int a = 0; a < 3; ++a) {
      if (pt[i + a] < bb[a][0]) { id[2 * a] = i; bb[a][0] = pt[i + a]; }
      if (pt[i + a] > bb[a][1]) { id[2 * a + 1] = i; bb[a][1] = pt[i + a]; }
    }
  float radius = 0; int choose = -1;
  for (int i = 0; i < 3; i++) {
    float dx = pt[id[2 * i]] - pt[id[2 * i + 1]];
    float dy = pt[id[2 * i] + 1] - pt[id[2 * i + 1] + 1];
    float dz = pt[id[2 * i] + 2] - pt[id[2 * i + 1] + 2];
    float r2 = dx * dx + dy * dy + dz * dz;
    if (r2 > radius) { radius = r2; choose = 2 * i; }
  }
  if (choose < 0) choose = 0; /* all points coincide: the reference reads id[-1] (undefined) */
  for (int c = 0; c < 3; ++c) center[c] = 0.5f * (pt[id[choose] + c] + pt[id[choose + 1] + c]);
  float radius2 = radius * 0.25f;
  radius = sqrtf(radius2);
  for (int i = 0; i < 3 * npt; i += 3) {
    float dx = pt[i] - center[0], dy = pt[i + 1] - center[1], dz = pt[i + 2] - center[2];
    float dis2 = dx * dx + dy * dy + dz * dz;
    if (dis2 > radius2) {
      float old_to_p = (float)sqrt((double)dis2);
      radius = (radius + old_to_p) * 0.5f;
      radius2 = radius * radius;
      float old_to_new = old_to_p - radius;
      for (int c = 0; c < 3; ++c) center[c] = (radius * center[c] + old_to_new * pt[i + c]) / old_to_p;
    }
  }
  *radius_out = radius;
}
int orc_bounding_sphere(const void* blob, int method_box, float* out4) {
  const PInfo* pi = (const PInfo*)blob;
  if (strcmp(pi->magic, "_POINTS_1.0_") != 0 || pi->pt_num <= 0) return ORC_E_BADARG;
  const float* pt = (const float*)((const char*)blob + pi->ptr_dis[0]);
  float radius = 0.0f, center[3] = { 0.0f, 0.0f, 0.0f };
  if (!method_box) bounding_sphere(&radius, center, pt, pi->pt_num);
  else {
    float bbmin[3] = { 0, 0, 0 }, bbmax[3] = { 0, 0, 0 };
    bounding_box(bbmin, bbmax, pt, pi->pt_num);
    for (int j = 0; j < 3; ++j) {
      center[j] = (bbmax[j] + bbmin[j]) / 2.0f;
      float width = (bbmax[j] - bbmin[j]) / 2.0f;
      radius += width * width;
    }
    radius = sqrtf(radius + 1.0e-20f);
  }
  out4[0] = radius; out4[1] = center[0]; out4[2] = center[1]; out4[3] = center[2];
  return 0;
}
static char* points_copy(const void* blob, int64_t bytes) {
  const PInfo* pi = (const PInfo*)blob;
  if (strcmp(pi->magic, "_POINTS_1.0_") != 0 || pi->pt_num <= 0) return NULL;
  char* out = result_alloc(bytes);
  if (out) memcpy(out, blob, (size_t)bytes);
  return out;
}
static void pts_translate(char* b, const float* t) { /* points_parser.cpp:42-51 */
  float* pt = pprop(b, pPoint); int npt = ((PInfo*)b)->pt_num;
  for (int i = 0; i < npt; ++i) for (int m = 0; m < 3; ++m) pt[3 * i + m] += t[m];
}
static void normalize_nx3(float* p, int npt) { /* math_functions.cpp:242-251 */
  for (int i = 0; i < npt; ++i) {
    float inv = 1.0f / (norm2f(p + 3 * i, 3) + 1.0e-15f);
    for (int m = 0; m < 3; ++m) p[3 * i + m] = p[3 * i + m] * inv;
  }
}
static void pts_scale(char* b, const float* s) { /* points_parser.cpp:75-101 */
  if ((s[0] == 1.0f && s[1] == 1.0f && s[2] == 1.0f) || s[0] == 0.0f || s[1] == 0.0f || s[2] == 0.0f) return;
  float* pt = pprop(b, pPoint); int npt = ((PInfo*)b)->pt_num;
  for (int i = 0; i < npt; ++i) for (int j = 0; j < 3; ++j) pt[3 * i + j] *= s[j];
  if (s[0] == s[1] && s[0] == s[2]) return;
  const float t[3] = { 1.0f / s[0], 1.0f / s[1], 1.0f / s[2] };
  float* nm = pprop(b, pNormal);
  if (nm) {
    for (int i = 0; i < npt; ++i) for (int j = 0; j < 3; ++j) nm[3 * i + j] *= t[j];
    normalize_nx3(nm, npt);
  }
}
static void matrix_prod(float* Cm, const float* A, const float* B, int M, int N, int K) { /* math_functions.cpp:185-196 */
  for (int n = 0; n < N; ++n)
    for (int m = 0; m < M; ++m) {
      Cm[n * M + m] = 0;
      for (int k = 0; k < K; ++k) Cm[n * M + m] += A[k * M + m] * B[n * K + k];
    }
}
void orc_rotation_matrix(float* rot, const float* angle) { /* math_functions.cpp:148-158 */
  float cosx = ORC_COS(angle[0]), sinx = ORC_SIN(angle[0]);
  float cosy = ORC_COS(angle[1]), siny = ORC_SIN(angle[1]);
  float cosz = ORC_COS(angle[2]), sinz = ORC_SIN(angle[2]);
  const float rotx[9] = { 1.0f, 0, 0, 0, cosx, sinx, 0, -sinx, cosx };
  const float roty[9] = { cosy, 0, -siny, 0, 1.0f, 0, siny, 0, cosy };
  const float rotz[9] = { cosz, sinz, 0, -sinz, cosz, 0, 0, 0, 1.0f };
  float tmp[9];
  matrix_prod(tmp, rotx, roty, 3, 3, 3);
  matrix_prod(rot, tmp, rotz, 3, 3, 3);
}
static void pts_rotate(char* b, const float* angles) { /* points_parser.cpp:118-131 */
  float rot[9];
  orc_rotation_matrix(rot, angles);
  int npt = ((PInfo*)b)->pt_num;
  float* tmp = (float*)malloc(sizeof(float) * 3 * (size_t)npt);
  float* pt = pprop(b, pPoint);
  matrix_prod(tmp, rot, pt, 3, npt, 3);
  memcpy(pt, tmp, sizeof(float) * 3 * (size_t)npt);
  float* nm = pprop(b, pNormal);
  if (nm) { matrix_prod(tmp, rot, nm, 3, npt, 3); memcpy(nm, tmp, sizeof(float) * 3 * (size_t)npt); }
  free(tmp);
}
int64_t orc_normalize_points(const void* blob, int64_t bytes, float radius, const float* center) {
  char* b = points_copy(blob, bytes); if (!b) return ORC_E_BADARG;
  const float dis[3] = { -center[0], -center[1], -center[2] };
  if (dis[0] != 0.0f || dis[1] != 0.0f || dis[2] != 0.0f) pts_translate(b, dis);
  const float inv = 1.0f / radius;
  const float scale[3] = { inv, inv, inv };
  if (scale[0] != 1.0f || scale[1] != 1.0f || scale[2] != 1.0f) pts_scale(b, scale);
  return bytes;
}
int64_t orc_transform_points(const void* blob, int64_t bytes, const float* angle, const float* scale,
    const float* jitter, float offset, const char* normal_axis) {
  char* b = points_copy(blob, bytes); if (!b) return ORC_E_BADARG;
  const float kEPS = 1.0e-10f;
  const int npt = ((PInfo*)b)->pt_num;
  float* pt = pprop(b, pPoint); float* nm = pprop(b, pNormal);
  if (offset > kEPS && nm) /* displace, points_parser.cpp:53-65 */
    for (int i = 0; i < npt; ++i) for (int m = 0; m < 3; ++m) pt[3 * i + m] += nm[3 * i + m] * offset;
  if (fabs(angle[0]) > kEPS || fabs(angle[1]) > kEPS || fabs(angle[2]) > kEPS) pts_rotate(b, angle);
  if (fabs(jitter[0]) > kEPS || fabs(jitter[1]) > kEPS || fabs(jitter[2]) > kEPS) pts_translate(b, jitter);
  if (scale[0] != 1.0f || scale[1] != 1.0f || scale[2] != 1.0f) pts_scale(b, scale);
  if (normal_axis && normal_axis[0] && nm) { /* orient_normal, points_parser.cpp:228-260 */
    if (!strcmp(normal_axis, "x") || !strcmp(normal_axis, "y") || !strcmp(normal_axis, "z")) {
      int j = normal_axis[0] - 'x';
      for (int i = 0; i < npt; ++i)
        if (nm[3 * i + j] < 0) for (int c = 0; c < 3; ++c) nm[3 * i + c] = -nm[3 * i + c];
    } else if (!strcmp(normal_axis, "xyz")) {
      for (int i = 0; i < 3 * npt; ++i) if (nm[i] < 0) nm[i] = -nm[i];
    }
  }
  return bytes;
}
int64_t orc_clip_points(const void* blob, int64_t bytes, const float* bbmin, const float* bbmax, int* in_bbox) {
  char* b = points_copy(blob, bytes); if (!b) return ORC_E_BADARG; /* points_parser.cpp:153-194 */
  PInfo* pi = (PInfo*)b;
  int npt = pi->pt_num, inside = 0;
  float* pts = pprop(b, pPoint);
  for (int i = 0; i < npt; ++i) {
    in_bbox[i] = bbmin[0] < pts[3 * i] && pts[3 * i] < bbmax[0] && bbmin[1] < pts[3 * i + 1] && pts[3 * i + 1] < bbmax[1] &&
        bbmin[2] < pts[3 * i + 2] && pts[3 * i + 2] < bbmax[2];
    inside += in_bbox[i];
  }
  if (inside == npt) return bytes;
  if (inside == 0) { inside = 1; in_bbox[0] = 1; for (int i = 0; i < 3; ++i) pts[i] = bbmin[i]; }
  for (int t = 0; t < 4; ++t) {
    if (!(pi->content_flags & (1 << t)) || pi->channels[t] == 0) continue;
    int ch = pi->channels[t];
    float* p = (float*)(b + pi->ptr_dis[t]);
    for (int i = 0, j = 0; i < npt; ++i) {
      if (!in_bbox[i]) continue;
      for (int c = 0; c < ch; ++c) p[j * ch + c] = p[i * ch + c];
      j++;
    }
  }
  pi->pt_num = inside;
  return bytes;
}


/* ------------------------------------------------------------------------ */
/* upgrade_key64, octree/octree/transform_octree.cpp:433-497: a blob written by a
 * 32-bit-key build ("_OCTREE_1.0_", 4-byte keys) -> the 64-bit-key layout. */
int64_t orc_upgrade_key64(const void* blob32, int64_t bytes) {
  const OInfo* in = (const OInfo*)blob32;
  if (bytes < (int64_t)sizeof(OInfo) || strcmp(in->magic, "_OCTREE_1.0_") != 0) return ORC_E_BADARG;
  OInfo o = *in;
  strcpy(o.magic, kMagic);
  set_ptr_dis(&o);
  const int sz = sizeof_octree(&o);
  char* out = result_alloc(sz);
  if (!out) return ORC_E_NOMEM;
  memcpy(out, &o, sizeof(o));
  const char* src = (const char*)blob32;
  const int num = total_nnum(&o), depth = o.depth;
  /* keys: widened one by one; packed xyz keys widen each of their four fields */
  const uint32_t* key_in = (const uint32_t*)(src + in->ptr_dis[0]);
  uint64_t* key_out = (uint64_t*)prop_ptr(out, kKey, 0);
  for (int i = 0; i < num; ++i) {
    if (o.key2xyz) {
      uint8_t f8[4]; uint16_t f16[4];
      memcpy(f8, key_in + i, 4);
      for (int j = 0; j < 4; ++j) f16[j] = (uint16_t)f8[j];
      memcpy(key_out + i, f16, 8);
    } else key_out[i] = (uint64_t)key_in[i];
  }
  memcpy(prop_ptr(out, kChild, 0), src + in->ptr_dis[1], sizeof(int) * (size_t)num);
  const int props[3] = { kFeature, kLabel, kSplit };
  for (int q = 0; q < 3; ++q) {
    const int p = props[q];
    if (!has_prop(&o, p)) continue;
    const int idx = prop_index(p);
    const int ch = p == kFeature ? channel_of(&o, p) : 1;
    const int d0 = location_of(&o, p) == depth ? depth : 0;
    for (int d = d0; d <= depth; ++d) {
      /* the input's per-depth offset follows octree_info.cpp:157-167 with ITS ptr_dis */
      int dis_in = in->ptr_dis[idx];
      if (location_of(&o, p) == -1) dis_in += in->nnum_cum[d] * channel_of(&o, p) * 4;
      memcpy(prop_ptr(out, p, d), src + dis_in, sizeof(float) * (size_t)o.nnum[d] * ch);
    }
  }
  return sz;
}

/* ------------------------------------------------------------------------ */
/* merge_octrees: octree/octree/merge_octrees.cpp:7-198,
 * consistency rule octree_info.cpp:118-130. */
static int is_consistent(const OInfo* a, const OInfo* b) {
  return strcmp(a->magic, b->magic) == 0 &&
      memcmp(a->channels, b->channels, sizeof(a->channels)) == 0 &&
      memcmp(a->locations, b->locations, sizeof(a->locations)) == 0 &&
      a->batch_size == b->batch_size && a->depth == b->depth &&
      a->full_layer == b->full_layer && a->adp_layer == b->adp_layer &&
      a->is_adaptive == b->is_adaptive && a->key2xyz == b->key2xyz &&
      a->has_node_dis == b->has_node_dis && a->content_flags == b->content_flags;
}
int64_t orc_octree_batch(const void* const* blobs, int B) {
  if (B < 1) return ORC_E_BADARG;
  const OInfo* first = (const OInfo*)blobs[0];
  const int depth = first->depth, full_layer = first->full_layer;
  if (depth < 1 || depth > 16) return ORC_E_BADARG;
  for (int i = 0; i < B; ++i) {
    const OInfo* oi = (const OInfo*)blobs[i];
    if (strcmp(oi->magic, kMagic) != 0 || !is_consistent(first, oi)) return ORC_E_BADARG;
  }
  const int D1 = depth + 1;
  int* cum = (int*)calloc((size_t)D1 * (size_t)(B + 1), sizeof(int));     /* nnum_cum_layer_ */
  int* cum_ne = (int*)calloc((size_t)D1 * (size_t)(B + 1), sizeof(int));  /* nnum_cum_nempty_layer_ */
  for (int d = 0; d < D1; ++d)
    for (int i = 0; i < B; ++i) {
      const OInfo* oi = (const OInfo*)blobs[i];
      cum[(i + 1) * D1 + d] = cum[i * D1 + d] + oi->nnum[d];
      cum_ne[(i + 1) * D1 + d] = cum_ne[i * D1 + d] + oi->nnum_nempty[d];
    }
  OInfo ob = *first; /* set_batch_info, merge_octrees.cpp:92-107 */
  set_batch_size(&ob, B);
  set_property(&ob, kNeigh, 8, -1);
  for (int d = 0; d < D1; ++d) { ob.nnum[d] = cum[B * D1 + d]; ob.nnum_nempty[d] = cum_ne[B * D1 + d]; }
  set_nnum_cum(&ob, 0);
  set_ptr_dis(&ob);
  const int sz = sizeof_octree(&ob);
  char* out = result_alloc(sz);
  if (!out) { free(cum); free(cum_ne); return ORC_E_NOMEM; }
  memcpy(out, &ob, sizeof(ob));

  for (int i = 0; i < B; ++i) {
    const void* in = blobs[i];
    const OInfo* oi = (const OInfo*)in;
    for (int d = 0; d < D1 && has_prop(&ob, kKey); ++d) { /* keys: batch id into sub-field 3 */
      uint64_t* des = (uint64_t*)prop_ptr(out, kKey, d) + cum[i * D1 + d];
      const uint64_t* src = (const uint64_t*)prop_ptr(in, kKey, d);
      for (int j = 0; j < oi->nnum[d]; ++j)
        des[j] = (src[j] & 0x0000FFFFFFFFFFFFull) | ((uint64_t)(uint16_t)i << 48);
    }
    for (int d = 0; d < D1 && has_prop(&ob, kChild); ++d) { /* children: offset by non-empty count */
      int* des = (int*)prop_ptr(out, kChild, d) + cum[i * D1 + d];
      const int* src = (const int*)prop_ptr(in, kChild, d);
      for (int j = 0; j < oi->nnum[d]; ++j) des[j] = src[j] == -1 ? -1 : src[j] + cum_ne[i * D1 + d];
    }
    if (has_prop(&ob, kFeature)) { /* features: interleave per channel */
      int fc = channel_of(&ob, kFeature);
      int d0 = location_of(&ob, kFeature) == depth ? depth : 0;
      for (int d = d0; d < D1; ++d)
        for (int c = 0; c < fc; ++c) {
          float* des = (float*)prop_ptr(out, kFeature, d) + (int64_t)c * ob.nnum[d] + cum[i * D1 + d];
          const float* src = (const float*)prop_ptr(in, kFeature, d) + (int64_t)c * oi->nnum[d];
          memcpy(des, src, sizeof(float) * (size_t)oi->nnum[d]);
        }
    }
    if (has_prop(&ob, kLabel)) {
      int d0 = location_of(&ob, kLabel) == depth ? depth : 0;
      for (int d = d0; d < D1; ++d)
        memcpy((float*)prop_ptr(out, kLabel, d) + cum[i * D1 + d], prop_ptr(in, kLabel, d),
            sizeof(float) * (size_t)oi->nnum[d]);
    }
    if (has_prop(&ob, kSplit)) {
      int d0 = location_of(&ob, kSplit) == depth ? depth : 0;
      for (int d = d0; d < D1; ++d)
        memcpy((float*)prop_ptr(out, kSplit, d) + cum[i * D1 + d], prop_ptr(in, kSplit, d),
            sizeof(float) * (size_t)oi->nnum[d]);
    }
  }
  for (int d = 1; d < D1; ++d) { /* merge_octrees.cpp:185-197 */
    if (d <= full_layer) orc_calc_neigh_full((int*)prop_ptr(out, kNeigh, d), d, B);
    else orc_calc_neigh_sparse((int*)prop_ptr(out, kNeigh, d), (const int*)prop_ptr(out, kNeigh, d - 1),
        (const int*)prop_ptr(out, kChild, d - 1), ob.nnum[d - 1]);
  }
  free(cum); free(cum_ne);
  return sz;
}

/* ------------------------------------------------------------------------ */
/* octree_new / octree_grow / octree_update / octree_set_property:
 * pytorch/cpp/octree_grow.cpp:13-190, pytorch/cpp/octree_property.cpp:308-325 */
int64_t orc_octree_new(int batch_size, int channel, int node_dis, int adaptive_layer) {
  if (batch_size < 1) return ORC_E_BADARG;
  OInfo o; info_reset(&o);
  set_batch_size(&o, batch_size);
  set_depth(&o, 0);
  set_full_layer(&o, 0);
  o.has_node_dis = node_dis ? 1 : 0;
  if (adaptive_layer > 1) { o.is_adaptive = 1; o.adp_layer = adaptive_layer; }
  o.key2xyz = 1;
  set_property(&o, kKey, 1, -1);
  set_property(&o, kChild, 1, -1);
  set_property(&o, kNeigh, 8, -1);
  set_property(&o, kFeature, channel, -1);
  for (int i = 0; i < 3; ++i) { o.bbmin[i] = 0.0f; o.bbmax[i] = 2.0f; }
  o.nnum[0] = batch_size;
  set_nnum_cum(&o, 0);
  o.nnum_nempty[0] = batch_size;
  set_ptr_dis(&o);
  int sz = sizeof_octree(&o);
  char* out = result_alloc(sz);
  if (!out) return ORC_E_NOMEM;
  memcpy(out, &o, sizeof(o));
  uint64_t* key = (uint64_t*)prop_ptr(out, kKey, 0);
  int* child = (int*)prop_ptr(out, kChild, 0);
  for (int i = 0; i < batch_size; ++i) { key[i] = (uint64_t)i; child[i] = i; }
  return sz;
}
int64_t orc_octree_grow(const void* in, int target_depth, int full_octree) {
  const OInfo* oi = (const OInfo*)in;
  if (target_depth < 1 || target_depth > 15) return ORC_E_BADARG;
  const int batch = oi->batch_size;
  const int node_num = oi->nnum_nempty[target_depth - 1] << 3;
  OInfo o = *oi; /* update_octreeinfo, octree_grow.cpp:57-73 */
  set_depth(&o, target_depth);
  if (full_octree) set_full_layer(&o, target_depth);
  float width = (float)(1 << target_depth);
  for (int i = 0; i < 3; ++i) { o.bbmin[i] = 0.0f; o.bbmax[i] = width; }
  o.nnum[target_depth] = node_num;
  o.nnum_nempty[target_depth] = node_num;
  set_nnum_cum(&o, 0);
  set_ptr_dis(&o);
  int sz = sizeof_octree(&o);
  char* out = result_alloc(sz);
  if (!out) return ORC_E_NOMEM;
  memcpy(out, &o, sizeof(o));
  /* copy_octree_gpu, octree_grow.cpp:75-87 */
  int64_t ncum = oi->nnum_cum[target_depth];
  memcpy(prop_ptr(out, kKey, 0), prop_ptr(in, kKey, 0), 8 * (size_t)(ncum * channel_of(oi, kKey)));
  memcpy(prop_ptr(out, kChild, 0), prop_ptr(in, kChild, 0), 4 * (size_t)(ncum * channel_of(oi, kChild)));
  memcpy(prop_ptr(out, kNeigh, 0), prop_ptr(in, kNeigh, 0), 4 * (size_t)(ncum * channel_of(oi, kNeigh)));
  if (has_prop(oi, kFeature))
    memcpy(prop_ptr(out, kFeature, 0), prop_ptr(in, kFeature, 0), 4 * (size_t)(ncum * channel_of(oi, kFeature)));
  int* neigh = (int*)prop_ptr(out, kNeigh, target_depth);
  uint64_t* key = (uint64_t*)prop_ptr(out, kKey, target_depth);
  int* child = (int*)prop_ptr(out, kChild, target_depth);
  if (full_octree) {
    orc_calc_neigh_full(neigh, target_depth, batch);
    orc_generate_key_full(key, target_depth, batch);
  } else {
    const int* label = (const int*)prop_ptr(out, kChild, target_depth - 1);
    orc_calc_neigh_sparse(neigh, (const int*)prop_ptr(out, kNeigh, target_depth - 1), label,
        o.nnum[target_depth - 1]);
    orc_generate_key_child(key, (const uint64_t*)prop_ptr(out, kKey, target_depth - 1), label,
        o.nnum[target_depth - 1]);
  }
  for (int i = 0; i < node_num; ++i) child[i] = i;
  return sz;
}
int64_t orc_octree_update(const void* in, const int* label, int n_label, int depth, int split) {
  const OInfo* oi = (const OInfo*)in;
  if (n_label != oi->nnum[depth]) return ORC_E_BADARG;
  int sz = sizeof_octree(oi);
  char* out = result_alloc(sz);
  if (!out) return ORC_E_NOMEM;
  memcpy(out, in, (size_t)sz);
  int* children = (int*)prop_ptr(out, kChild, depth);
  int split_num = orc_generate_label(children, label, n_label, split);
  if (split_num == 0) { split_num = 1; children[0] = 0; }
  ((OInfo*)out)->nnum_nempty[depth] = split_num;
  return sz;
}
int64_t orc_octree_set_property(const void* in, const float* data, int64_t count, int depth) {
  const OInfo* oi = (const OInfo*)in;
  if (count != (int64_t)oi->nnum[depth] * channel_of(oi, kFeature)) return ORC_E_BADARG;
  int sz = sizeof_octree(oi);
  char* out = result_alloc(sz);
  if (!out) return ORC_E_NOMEM;
  memcpy(out, in, (size_t)sz);
  memcpy(prop_ptr(out, kFeature, depth), data, sizeof(float) * (size_t)count);
  return sz;
}


/* ------------------------------------------------------------------------ */
/* octree_scan: ScanOctree, octree/octree/transform_octree.cpp:11-297, driven as
 * pytorch/cpp/transform_octree.cpp:5-22 does.  `axis` holds n_axis view directions
 * (3 floats each); a finest-level node is kept iff it is non-empty, faces one of the
 * views and is the nearest node of its pixel in that view's z-buffer.  Pinned against
 * the compiled reference (tests/test_oracle_scan.py). */
static float dot3(const float* a, const float* b) { return a[0] * b[0] + a[1] * b[1] + a[2] * b[2]; }
static void rotation_from_axes(float* rot, const float* axis0, const float* axis1) { /* math_functions.cpp:130-173 */
  float angle = dot3(axis0, axis1);
  if (angle < -1) angle = -1;
  if (angle > 1) angle = 1;
  angle = (float)acos((double)angle);
  float axis[3];
  axis[0] = axis0[1] * axis1[2] - axis0[2] * axis1[1];
  axis[1] = axis0[2] * axis1[0] - axis0[0] * axis1[2];
  axis[2] = axis0[0] * axis1[1] - axis0[1] * axis1[0];
  float ilen = (float)(1.0 / ((double)norm2f(axis, 3) + 1.0e-10));
  for (int i = 0; i < 3; ++i) axis[i] *= ilen;
  float cosa = ORC_COS(angle), cosa1 = 1 - cosa, sina = ORC_SIN(angle);
  rot[0] = cosa + axis[0] * axis[0] * cosa1;
  rot[1] = axis[0] * axis[1] * cosa1 + axis[2] * sina;
  rot[2] = axis[0] * axis[2] * cosa1 - axis[1] * sina;
  rot[3] = axis[0] * axis[1] * cosa1 - axis[2] * sina;
  rot[4] = cosa + axis[1] * axis[1] * cosa1;
  rot[5] = axis[1] * axis[2] * cosa1 + axis[0] * sina;
  rot[6] = axis[0] * axis[2] * cosa1 + axis[1] * sina;
  rot[7] = axis[1] * axis[2] * cosa1 - axis[0] * sina;
  rot[8] = cosa + axis[2] * axis[2] * cosa1;
}
/* the view frame and the pixel grid of one direction: set_axis + bbox_xy, transform_octree.cpp:13-92 */
void orc_scan_frame(float* frame /* x[3] y[3] z[3] bbmin[3] */, int* width, const float* z, int depth, float scale_) {
  float rot[9], z0[3] = { 0, 0, 1 };
  rotation_from_axes(rot, z0, z);
  float* x_ = frame; float* y_ = frame + 3; float* z_ = frame + 6; float* bbmin = frame + 9;
  for (int i = 0; i < 3; ++i) { x_[i] = rot[i]; y_[i] = rot[3 + i]; z_[i] = z[i]; }
  float bbmax[3];
  for (int i = 0; i < 3; ++i) { bbmin[i] = FLT_MAX; bbmax[i] = -FLT_MAX; }
  for (int i = 0; i < 8; ++i) {
    float pt[3] = { (float)(i / 4), (float)((i / 2) % 2), (float)(i % 2) };
    float x = dot3(pt, x_), y = dot3(pt, y_), zz = dot3(pt, z_);
    if (x < bbmin[0]) bbmin[0] = x;
    if (x > bbmax[0]) bbmax[0] = x;
    if (y < bbmin[1]) bbmin[1] = y;
    if (y > bbmax[1]) bbmax[1] = y;
    if (zz < bbmin[2]) bbmin[2] = zz;
    if (zz > bbmax[2]) bbmax[2] = zz;
  }
  float wmax = -1, scale = (float)(1 << depth);
  for (int i = 0; i < 3; ++i) {
    bbmax[i] *= scale; bbmin[i] *= scale;
    float dis = bbmax[i] - bbmin[i];
    if (dis > wmax) wmax = dis;
  }
  *width = (int)(wmax * scale_) + 2;
}
int64_t orc_octree_scan(const void* blob, const float* axis, int n_axis, float scale_) {
  const OInfo* oi = (const OInfo*)blob;
  const int depth = oi->depth, full = oi->full_layer;
  if (oi->batch_size != 1 || channel_of(oi, kKey) != 1) return ORC_E_UNSUPPORTED;
  const int num = oi->nnum[depth];
  unsigned char* drop[17];
  for (int d = 0; d <= depth; ++d) { drop[d] = (unsigned char*)malloc((size_t)oi->nnum[d] + 1); memset(drop[d], 1, (size_t)oi->nnum[d] + 1); }
  const uint64_t* key_D = (const uint64_t*)prop_ptr(blob, kKey, depth);
  const int* child_D = (const int*)prop_ptr(blob, kChild, depth);
  const int fch = channel_of(oi, kFeature), floc = location_of(oi, kFeature);
  const float* feat_D = has_prop(oi, kFeature) ? (const float*)prop_ptr(blob, kFeature, depth) : NULL;
  const int normal_ok = feat_D && (floc == -1 || floc == depth) && fch >= 3;
  for (int a = 0; a < n_axis; ++a) {
    float frame[12]; int width;
    orc_scan_frame(frame, &width, axis + 3 * a, depth, scale_);
    const float* x_ = frame; const float* y_ = frame + 3; const float* z_ = frame + 6; const float* bbmin = frame + 9;
    int* id_buffer = (int*)malloc(sizeof(int) * (size_t)width * width);
    float* z_buffer = (float*)malloc(sizeof(float) * (size_t)width * width);
    unsigned char* flags = (unsigned char*)malloc((size_t)num + 1);
    memset(flags, 1, (size_t)num + 1);
    for (int i = 0; i < width * width; ++i) { id_buffer[i] = -1; z_buffer[i] = FLT_MAX; }
    for (int i = 0; i < num; ++i) { /* z_buffer, transform_octree.cpp:99-138 */
      if (child_D[i] < 0) continue;
      float normal[3] = { 0, 0, 0 };
      if (normal_ok) for (int c = 0; c < 3; ++c) normal[c] = feat_D[(int64_t)c * num + i];
      if (dot3(normal, z_) >= 0) continue;
      float pt[3];
      key2xyz_f(pt, key_D[i], depth, oi->key2xyz);
      float x = (dot3(x_, pt) - bbmin[0]) * scale_;
      float y = (dot3(y_, pt) - bbmin[1]) * scale_;
      float z = dot3(z_, pt);
      int k = (int)(x + 0.5f) * width + (int)(y + 0.5f);
      if (z_buffer[k] > z) {
        z_buffer[k] = z;
        if (id_buffer[k] >= 0) flags[id_buffer[k]] = 1;
        id_buffer[k] = i;
        flags[i] = 0;
      }
    }
    for (int j = 0; j < num; ++j) if (flags[j] == 0) drop[depth][j] = 0;
    free(id_buffer); free(z_buffer); free(flags);
  }
  /* generate_flags, transform_octree.cpp:140-170 */
  for (int d = 0; d < full; ++d) memset(drop[d], 0, (size_t)oi->nnum[d]);
  for (int d = depth - 1; d >= full; --d) {
    const int* child_d = (const int*)prop_ptr(blob, kChild, d);
    for (int i = 0; i < oi->nnum[d]; ++i) {
      int j = child_d[i], dr = 1;
      if (j < 0) continue;
      for (int k = j * 8; k < j * 8 + 8; ++k) if (drop[d + 1][k] == 0) { dr = 0; break; }
      drop[d][i] = (unsigned char)dr;
    }
  }
  /* trim_octree, transform_octree.cpp:172-297 */
  OInfo o = *oi;
  int nne[17] = { 0 }, nn[17] = { 0 };
  for (int d = 0; d < full; ++d) nne[d] = 1 << (3 * d);
  for (int d = full; d <= depth; ++d) { int c = 0; for (int i = 0; i < oi->nnum[d]; ++i) if (drop[d][i] == 0) c++; nne[d] = c; }
  nn[0] = 1;
  for (int d = 1; d <= depth; ++d) nn[d] = 8 * nne[d - 1];
  for (int d = 0; d <= depth; ++d) { o.nnum[d] = nn[d]; o.nnum_nempty[d] = nne[d]; }
  set_nnum_cum(&o, 0);
  set_ptr_dis(&o);
  const int sz = sizeof_octree(&o);
  char* out = result_alloc(sz);
  if (!out) return ORC_E_NOMEM;
  memset(out, 0, (size_t)sz);
  memcpy(out, &o, sizeof(o));
  const int lloc = location_of(oi, kLabel), lch = channel_of(oi, kLabel);
  const int sloc = location_of(oi, kSplit), sch = channel_of(oi, kSplit);
  for (int d = 1; d <= depth; ++d) {
    const int num_p = oi->nnum[d - 1];
    const unsigned char* drop_p = drop[d - 1]; const unsigned char* drop_d = drop[d];
    const int* child_in = (const int*)prop_ptr(blob, kChild, d - 1);
    const uint64_t* key_in = (const uint64_t*)prop_ptr(blob, kKey, d);
    int* child_out = (int*)prop_ptr(out, kChild, d);
    uint64_t* key_out = (uint64_t*)prop_ptr(out, kKey, d);
    const int nnum_in = oi->nnum[d], nnum_out = o.nnum[d];
    const float* f_in = (fch && (floc == -1 || d == depth)) ? (const float*)prop_ptr(blob, kFeature, d) : NULL;
    float* f_out = f_in ? (float*)prop_ptr(out, kFeature, d) : NULL;
    const float* l_in = (lch && (lloc == -1 || d == depth)) ? (const float*)prop_ptr(blob, kLabel, d) : NULL;
    float* l_out = l_in ? (float*)prop_ptr(out, kLabel, d) : NULL;
    const float* s_in = (sch && (sloc == -1 || d == depth)) ? (const float*)prop_ptr(blob, kSplit, d) : NULL;
    float* s_out = s_in ? (float*)prop_ptr(out, kSplit, d) : NULL;
    int j = 0, id = 0;
    for (int i = 0; i < num_p; ++i) {
      if (drop_p[i] == 1) continue;
      const int t = child_in[i];
      for (int k = 8 * t; k < 8 * t + 8; ++k) {
        key_out[j] = key_in[k];
        child_out[j] = drop_d[k] == 0 ? id++ : -1;
        if (f_out) for (int c = 0; c < fch; ++c) f_out[(int64_t)c * nnum_out + j] = drop_d[k] == 0 ? f_in[(int64_t)c * nnum_in + k] : 0;
        if (l_out) l_out[j] = drop_d[k] == 0 ? l_in[k] : -1;
        if (s_out) s_out[j] = drop_d[k] == 0 ? s_in[k] : 0;
        j++;
      }
    }
  }
  for (int d = 0; d <= depth; ++d) free(drop[d]);
  return sz;
}

/* octree_dropout, octree/octree/transform_octree.cpp:286-431, with the Bernoulli flags of level
 * `depth_dropout` handed in (the reference draws them from an engine seeded with the clock).
 * A dropped node takes its whole subtree along; the levels below are compacted, the children
 * of the kept nodes renumbered.  At `depth_dropout` itself a dropped node KEEPS its old child
 * index (transform_octree.cpp:422-425) while the non-empty count only counts the kept ones. */
int64_t orc_octree_dropout(const void* blob, const unsigned char* flags, int depth_dropout) {
  const OInfo* oi = (const OInfo*)blob;
  const int depth = oi->depth, dd = depth_dropout;
  if (dd < 0 || dd > depth || channel_of(oi, kKey) != 1) return ORC_E_UNSUPPORTED;
  unsigned char* drop[17] = { 0 };
  drop[dd] = (unsigned char*)calloc((size_t)oi->nnum[dd] + 1, 1);
  for (int i = 0; i < oi->nnum[dd]; ++i) drop[dd][i] = flags[i] ? 1 : 0;
  for (int d = dd + 1; d <= depth; ++d) { /* :301-314 */
    drop[d] = (unsigned char*)calloc((size_t)oi->nnum[d] + 1, 1);
    const int* child_p = (const int*)prop_ptr(blob, kChild, d - 1);
    for (int i = 0; i < oi->nnum[d - 1]; ++i) {
      const int t = child_p[i];
      if (t < 0) continue;
      for (int j = 0; j < 8; ++j) drop[d][t * 8 + j] = drop[d - 1][i];
    }
  }
  OInfo o = *oi;
  for (int d = dd + 1; d <= depth; ++d) { /* :318-329 */
    int c = 0;
    for (int i = 0; i < oi->nnum[d]; ++i) if (drop[d][i] == 0) c++;
    o.nnum[d] = c;
  }
  set_nnum_cum(&o, 0);
  set_ptr_dis(&o);
  const int sz = sizeof_octree(&o);
  char* out = result_alloc(sz);
  if (!out) return ORC_E_NOMEM;
  memset(out, 0, (size_t)sz);
  /* levels 0..depth_dropout as they are (:339-361) */
  const int num = oi->nnum_cum[dd + 1];
  const int fch = channel_of(oi, kFeature), floc = location_of(oi, kFeature);
  const int lch = channel_of(oi, kLabel), lloc = location_of(oi, kLabel);
  const int sch = channel_of(oi, kSplit), sloc = location_of(oi, kSplit);
  memcpy(out, &o, sizeof(o));
  memcpy(prop_ptr(out, kKey, 0), prop_ptr(blob, kKey, 0), sizeof(uint64_t) * (size_t)num);
  memcpy(prop_ptr(out, kChild, 0), prop_ptr(blob, kChild, 0), sizeof(int) * (size_t)num);
  if (has_prop(oi, kFeature) && floc == -1)
    memcpy(prop_ptr(out, kFeature, 0), prop_ptr(blob, kFeature, 0), sizeof(float) * (size_t)num * fch);
  if (has_prop(oi, kLabel) && lloc == -1)
    memcpy(prop_ptr(out, kLabel, 0), prop_ptr(blob, kLabel, 0), sizeof(float) * (size_t)num * lch);
  if (has_prop(oi, kSplit) && sloc == -1)
    memcpy(prop_ptr(out, kSplit, 0), prop_ptr(blob, kSplit, 0), sizeof(float) * (size_t)num * sch);
  int nne[17] = { 0 };
  for (int d = dd + 1; d <= depth; ++d) { /* :365-416 */
    const int nnum_d = oi->nnum[d], nnum_o = o.nnum[d];
    const int* child_src = (const int*)prop_ptr(blob, kChild, d);
    const uint64_t* key_src = (const uint64_t*)prop_ptr(blob, kKey, d);
    int* child_des = (int*)prop_ptr(out, kChild, d);
    uint64_t* key_des = (uint64_t*)prop_ptr(out, kKey, d);
    const float* f_in = (has_prop(oi, kFeature) && (floc == -1 || d == depth)) ? (const float*)prop_ptr(blob, kFeature, d) : NULL;
    float* f_out = f_in ? (float*)prop_ptr(out, kFeature, d) : NULL;
    const float* l_in = (lch != 0 && (lloc == -1 || d == depth)) ? (const float*)prop_ptr(blob, kLabel, d) : NULL;
    float* l_out = l_in ? (float*)prop_ptr(out, kLabel, d) : NULL;
    const float* s_in = (sch != 0 && (sloc == -1 || d == depth)) ? (const float*)prop_ptr(blob, kSplit, d) : NULL;
    float* s_out = s_in ? (float*)prop_ptr(out, kSplit, d) : NULL;
    int id = 0;
    for (int i = 0, j = 0; i < nnum_d; ++i) {
      if (drop[d][i] != 0) continue;
      key_des[j] = key_src[i];
      child_des[j] = child_src[i] < 0 ? child_src[i] : id++;
      if (f_out) for (int c = 0; c < fch; ++c) f_out[(int64_t)c * nnum_o + j] = f_in[(int64_t)c * nnum_d + i];
      if (l_out) l_out[j] = l_in[i];
      if (s_out) s_out[j] = s_in[i];
      ++j;
    }
    nne[d] = id;
  }
  { /* :419-430 */
    int id = 0;
    const int* child_src = (const int*)prop_ptr(blob, kChild, dd);
    int* child_des = (int*)prop_ptr(out, kChild, dd);
    for (int i = 0; i < o.nnum[dd]; ++i)
      child_des[i] = (drop[dd][i] == 1 || child_src[i] < 0) ? child_src[i] : id++;
    for (int d = 0; d < dd; ++d) nne[d] = oi->nnum_nempty[d];
    nne[dd] = id;
  }
  for (int d = 0; d <= depth; ++d) ((OInfo*)out)->nnum_nempty[d] = nne[d];
  for (int d = dd; d <= depth; ++d) free(drop[d]);
  return sz;
}
