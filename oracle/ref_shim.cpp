// TEST INFRASTRUCTURE -- not part of the shipped library.
//
// extern "C" shim over the *real* reference CPU sources (compiled where they
// lie under /root/reference/octree/octree by oracle/Makefile into
// oracle/_ref/libocnn_ref.so).  The entry points mirror the ones exported by
// the C restatement (oracle/ocnn_oracle.c, prefix orc_) one-for-one so the
// same Python checker can drive either library.  Only tests, the smoke check
// and the bench's cpu_baseline leg may load this library.
//
// Nothing from the reference is copied here: this file only *calls* the
// reference's public functions (octree.h, merge_octrees.h, octree_nn.h,
// octree_samples.h).
#include <octree.h>
#include <merge_octrees.h>
#include <octree_nn.h>
#include <octree_samples.h>
#include <points.h>
#include <math_functions.h>
#include <transform_octree.h>

#include <cmath>
#include <ctime>
#include <random>
#include <string>

#include <cstdint>
#include <cstring>
#include <vector>

namespace {
std::vector<char> g_last;  // result of the last blob-producing call
int64_t keep(const std::vector<char>& v) {
  g_last = v;
  return (int64_t)g_last.size();
}
}  // namespace

extern "C" {

int64_t ref_fetch(void* out, int64_t cap) {
  if ((int64_t)g_last.size() > cap) return -1;
  memcpy(out, g_last.data(), g_last.size());
  return (int64_t)g_last.size();
}

// pytorch/cpp/point2octree.cpp:5-34 (+ optional bbox override, which is what
// octree/test/test_octree.cpp:34-84 does by hand).
int64_t ref_points2octree(const void* points_blob, int depth, int full_depth,
    int node_dis, int node_feature, int split_label, int adaptive,
    int adp_depth, float th_normal, float th_distance, int extrapolate,
    int save_pts, int key2xyz, const float* bbmin, const float* bbmax) {
  Points pts;
  pts.set(points_blob);
  std::string msg;
  if (!pts.info().check_format(msg)) return -1;
  OctreeInfo info;
  info.initialize(depth, full_depth, node_dis, node_feature, split_label,
      adaptive, adp_depth, th_distance, th_normal, key2xyz, extrapolate,
      save_pts, pts);
  if (bbmin && bbmax) info.set_bbox(bbmin, bbmax);
  Octree oct;
  oct.build(info, pts);
  return keep(oct.buffer());
}

int64_t ref_octree_batch(const void* const* blobs, int n) {
  std::vector<const char*> in;
  for (int i = 0; i < n; ++i) in.push_back((const char*)blobs[i]);
  std::vector<char> out;
  merge_octrees(out, in);
  return keep(out);
}

int64_t ref_octree_sample(const char* name) {
  size_t sz = 0;
  const unsigned char* p = octree::get_one_octree(name, &sz);
  if (!p || sz == 0) return -1;
  g_last.assign((const char*)p, (const char*)p + sz);
  return (int64_t)sz;
}

// octree/octree/transform_octree.cpp:433-497: 32-bit-key blob ("_OCTREE_1.0_") -> 64-bit keys
// pytorch/cpp/transform_octree.cpp:5-22
int64_t ref_octree_scan(const void* blob, const float* axis, int n_axis, float scale) {
  OctreeParser parser;
  parser.set_cpu(blob);
  ScanOctree scan_octree(scale);
  std::vector<float> ax(axis, axis + 3 * n_axis);
  std::vector<char> out;
  scan_octree.scan(out, parser, ax);
  return keep(out);
}

// octree/octree/transform_octree.cpp:286-431.  The reference seeds its engine with the wall
// clock's second.  The clock is read on both sides of the call; when the second did not
// change, the same engine and distribution are replayed here to hand the flags back, so a
// restatement can be compared on the very flags the reference drew.
int64_t ref_octree_dropout(const void* blob, int64_t bytes, int depth_dropout, float threshold, unsigned char* flags,
    int n_flags) {
  for (int attempt = 0; attempt < 8; ++attempt) {
    const time_t t0 = time(nullptr);
    std::string in((const char*)blob, (size_t)bytes);
    std::vector<char> out;
    octree_dropout(out, in, depth_dropout, threshold);
    if (time(nullptr) != t0) continue;
    std::default_random_engine generator(static_cast<unsigned>(t0));
    std::bernoulli_distribution distribution(threshold);
    for (int i = 0; i < n_flags; ++i) flags[i] = (unsigned char)static_cast<unsigned>(distribution(generator));
    return keep(out);
  }
  return -1;
}

int64_t ref_upgrade_key64(const void* blob32, int64_t bytes) {
  std::vector<char> in((const char*)blob32, (const char*)blob32 + bytes), out;
  upgrade_key64(out, in);
  return keep(out);
}

int ref_get_ni(const int* ks, int* out) {
  std::vector<int> k(ks, ks + 3);
  std::vector<int>& ni = NeighHelper::get_ni(k);
  memcpy(out, ni.data(), ni.size() * sizeof(int));
  return (int)ni.size();
}
void ref_get_parent(int* out) {
  memcpy(out, NeighHelper::get_parent_array().data(), 512 * sizeof(int));
}
void ref_get_dis(int* out) {
  memcpy(out, NeighHelper::get_dis_array().data(), 64 * sizeof(int));
}

void ref_calc_neigh_full(int* neigh, int depth, int batch) {
  calc_neigh_cpu(neigh, depth, batch);
}
void ref_calc_neigh_sparse(int* neigh_child, const int* neigh,
    const int* children, int node_num) {
  calc_neigh_cpu(neigh_child, neigh, children, node_num);
}

void ref_octree2col(float* col, const float* data, int channel, int height,
    int kernel_sdim, int stride, const int* neigh, const int* ni,
    int height_col, int n) {
  octree2col_cpu<float>(col, data, channel, height, kernel_sdim, stride, neigh,
      ni, height_col, n);
}
void ref_col2octree(const float* col, float* data, int channel, int height,
    int kernel_sdim, int stride, const int* neigh, const int* ni,
    int height_col, int n) {
  col2octree_cpu<float>(col, data, channel, height, kernel_sdim, stride, neigh,
      ni, height_col, n);
}
void ref_octree2colP(float* col, const float* data, int channel, int height,
    int octree_h, int kernel_sdim, int stride, const int* neigh, const int* ni,
    const int* child, const int* ichild, int height_col, int n) {
  octree2colP_cpu<float>(col, data, channel, height, octree_h, kernel_sdim,
      stride, neigh, ni, child, ichild, height_col, n);
}
void ref_col2octreeP(const float* col, float* data, int channel, int height,
    int octree_h, int kernel_sdim, int stride, const int* neigh, const int* ni,
    const int* child, const int* ichild, int height_col, int n) {
  col2octreeP_cpu<float>(col, data, channel, height, octree_h, kernel_sdim,
      stride, neigh, ni, child, ichild, height_col, n);
}

void ref_max_pool(float* top, int top_h, int* mask, const float* btm,
    int btm_h, int channel) {
  octree_max_pool_cpu<float>(top, top_h, mask, btm, btm_h, channel);
}
void ref_max_unpool(const float* top, int top_h, const int* mask, float* btm,
    int btm_h, int channel) {
  octree_max_unpool_cpu<float>(top, top_h, mask, btm, btm_h, channel);
}
void ref_mask_pool(float* top, int top_h, const int* mask, const float* btm,
    int btm_h, int channel) {
  octree_mask_pool_cpu<float>(top, top_h, mask, btm, btm_h, channel);
}
void ref_pad_forward(float* Y, int Hy, int C, const float* X, int Hx,
    const int* label, float dval) {
  pad_forward_cpu<float>(Y, Hy, C, X, Hx, label, dval);
}
void ref_pad_backward(float* X, int Hx, int C, const float* Y, int Hy,
    const int* label) {
  pad_backward_cpu<float>(X, Hx, C, Y, Hy, label);
}

void ref_generate_key_child(uint64_t* key_child, const uint64_t* key,
    const int* child, int node_num) {
  generate_key_cpu<uintk>((uintk*)key_child, (const uintk*)key, child, node_num);
}
void ref_generate_key_full(uint64_t* key, int depth, int batch) {
  generate_key_cpu<uintk>((uintk*)key, depth, batch);
}
int ref_generate_label(int* label, const int* btm, int btm_h, int mask) {
  int top_h = 0;
  generate_label_cpu<int>(label, top_h, btm, btm_h, mask);
  return top_h;
}
void ref_search_key(int* idx, const uint64_t* key, int n_key,
    const uint64_t* query, int n_query) {
  search_key_cpu<uintk>(idx, (const uintk*)key, n_key, (const uintk*)query,
      n_query);
}
void ref_get_bilinear(int* table512) {
  const vector<int>& t = NeighHelper::get_bilinear_array();
  for (int i = 0; i < 512; ++i) table512[i] = t[i];
}
void ref_bilinear_neigh(int* bidx, const int* neigh, const int* child, int node_num) {
  bilinear_neigh_cpu(bidx, neigh, child, node_num, NeighHelper::get_bilinear_array().data());
}
void ref_bilinear_xyz(uint64_t* xyz0, float* fracs, int d0, const uint64_t* xyz1, int d1, int num) {
  bilinear_xyz_cpu((uintk*)xyz0, fracs, d0, (const uintk*)xyz1, d1, num);
}
void ref_xyz2key(uint64_t* key, const uint64_t* xyz, int num, int depth) {
  xyz2key_cpu<uintk>((uintk*)key, (const uintk*)xyz, num, depth);
}
void ref_key2xyz(uint64_t* xyz, const uint64_t* key, int num, int depth) {
  key2xyz_cpu<uintk>((uintk*)xyz, (const uintk*)key, num, depth);
}
void ref_key2idx(int* idx, const uint64_t* key, int num) {
  key2idx_cpu<uintk>(idx, (const uintk*)key, num);
}


// pytorch/cpp/transform_points.cpp:7-125, on a copy of the blob (setup_transform).
int ref_bounding_sphere(const void* points_blob, int method_box, float* out4) {
  Points pts;
  pts.set(points_blob);
  std::string msg;
  if (!pts.info().check_format(msg)) return -1;
  float radius = 0.0f, center[3] = {0.0f};
  if (!method_box) {
    bounding_sphere(radius, center, pts.points(), pts.info().pt_num());
  } else {
    float bbmin[3] = {0.0f}, bbmax[3] = {0.0f};
    bounding_box(bbmin, bbmax, pts.points(), pts.info().pt_num());
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
static bool open_copy(const void* blob, int64_t bytes, Points& pts) {
  g_last.assign((const char*)blob, (const char*)blob + bytes);
  pts.set(g_last.data());
  std::string msg;
  return pts.info().check_format(msg);
}
int64_t ref_normalize_points(const void* blob, int64_t bytes, float radius, const float* center) {
  Points pts;
  if (!open_copy(blob, bytes, pts)) return -1;
  const float dis[3] = {-center[0], -center[1], -center[2]};
  if (dis[0] != 0.0f || dis[1] != 0.0f || dis[2] != 0.0f) pts.translate(dis);
  const float inv_radius = 1.0f / radius;
  const float scale[3] = {inv_radius, inv_radius, inv_radius};
  if (scale[0] != 1.0f || scale[1] != 1.0f || scale[2] != 1.0f) pts.scale(scale);
  return (int64_t)g_last.size();
}
int64_t ref_transform_points(const void* blob, int64_t bytes, const float* angle, const float* scale,
    const float* jitter, float offset, const char* normal_axis) {
  Points pts;
  if (!open_copy(blob, bytes, pts)) return -1;
  const float kEPS = 1.0e-10f;
  if (offset > kEPS) pts.displace(offset);
  if (fabs(angle[0]) > kEPS || fabs(angle[1]) > kEPS || fabs(angle[2]) > kEPS) pts.rotate(angle);
  if (fabs(jitter[0]) > kEPS || fabs(jitter[1]) > kEPS || fabs(jitter[2]) > kEPS) pts.translate(jitter);
  if (scale[0] != 1.0f || scale[1] != 1.0f || scale[2] != 1.0f) pts.scale(scale);
  std::string axis(normal_axis ? normal_axis : "");
  if (!axis.empty()) pts.orient_normal(axis);
  return (int64_t)g_last.size();
}
int64_t ref_clip_points(const void* blob, int64_t bytes, const float* bbmin, const float* bbmax, int* inbox_mask) {
  Points pts;
  if (!open_copy(blob, bytes, pts)) return -1;
  std::vector<int> mask = pts.clip(bbmin, bbmax);
  memcpy(inbox_mask, mask.data(), mask.size() * sizeof(int));
  return (int64_t)g_last.size();
}

}  // extern "C"
