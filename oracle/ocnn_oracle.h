/* TEST INFRASTRUCTURE -- CPU restatement ("oracle") of the O-CNN octree hot
 * path.  It is the checker the HIP library is compared against; it is never
 * linked into, loaded by, or called from the shipped library.  Only tests,
 * the smoke check and the bench's cpu_baseline leg may use it.
 *
 * Every function cites the reference file:line whose behaviour it restates
 * (paths relative to the reference checkout root).
 *
 * Pinning status (what independent evidence each function is checked against
 * in tests/):
 *   key math ............ closed form + literal vectors of the reference tests
 *   points2octree ....... literal known-answer test of octree/test/test_octree.cpp,
 *                         brute-force voxel dictionary, compiled reference
 *   octree_batch ........ literal vectors of pytorch/test/test_octree_property.py,
 *                         compiled reference
 *   neighbour tables .... brute-force (batch,x,y,z) dictionary, compiled reference
 *   octree2col/col2octree closed form on the full depth-1 layer, adjointness,
 *                         P == pad o col o depad identity, compiled reference
 *   conv / deconv ....... dense zero-padded conv3d on a full layer, adjointness
 *   conv / deconv grads . <grad_w, W'> == <grad_out, conv(x; W')> for random W' (the op is linear
 *                         in W), <grad_data, x'> == <grad_out, conv(x'; W)>, dense conv3d autograd
 *   upgrade_key64 ....... the reference's six embedded 32-bit sample blobs -> their 64-bit
 *                         forms (golden fixture), compiled reference on downgraded blobs
 *   point transforms .... compiled reference byte for byte; rotation = product of the three axis
 *                         rotations (closed form), clip = boolean mask + compaction (numpy)
 *   pool / unpool / pad . literal vectors of pytorch/test/test_octree_pool.py
 *   new/grow/update ..... MD5 of the rebuilt octree_2 quoted in
 *                         pytorch/test/test_octree_grow.py
 *   search_key .......... literal vectors of pytorch/test/test_octree_key.py
 *   bilinear neigh / xyz  compiled reference; the reference's own consistency test
 *                         (octree/test/test_octree_nn.cpp:23-84: corner weights 27,9,9,9,3,3,3,1
 *                         from the key geometry, and neigh stencil == xyz stencil looked up by key)
 *   gather / gatherbk / mask  (GPU-only in the reference) gather == pad_forward with 0 (pinned
 *                         above); gatherbk by brute force with repeated indices and the adjoint
 *                         identity <gather x, y> == <x, gatherbk y>; mask by its closed form
 *   adaptive build ...... (all-depth signals, error metrics, extrapolation, trimming:
 *                         octree/octree/octree.cpp:454-806, 958-1178) every literal of
 *                         octree/test/test_octree.cpp:196-331 (TestOctreeTrim), compiled
 *                         reference byte for byte on seeded smooth surfaces
 * Returns ORC_E_UNSUPPORTED only where the reference itself reads out of bounds: an adaptive
 * build without normals or with save_pts.
 */
#ifndef OCNN_ORACLE_H_
#define OCNN_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_E_BADARG      (-1)
#define ORC_E_UNSUPPORTED (-2)
#define ORC_E_NOMEM       (-3)

/* copy the blob produced by the last blob-producing call */
int64_t orc_fetch(void* out, int64_t cap);

int64_t orc_points2octree(const void* points_blob, int depth, int full_depth,
    int node_dis, int node_feature, int split_label, int adaptive,
    int adp_depth, float th_normal, float th_distance, int extrapolate,
    int save_pts, int key2xyz, const float* bbmin, const float* bbmax);
int64_t orc_octree_batch(const void* const* blobs, int n);

int64_t orc_octree_new(int batch_size, int channel, int node_dis, int adaptive_layer);
int64_t orc_octree_grow(const void* blob, int target_depth, int full_octree);
int64_t orc_octree_update(const void* blob, const int* label, int n_label, int depth, int split);
int64_t orc_octree_set_property(const void* blob, const float* data, int64_t count, int depth);

int  orc_get_ni(const int* ks, int* out);
void orc_get_parent(int* out);
void orc_get_dis(int* out);

void orc_calc_neigh_full(int* neigh, int depth, int batch);
void orc_calc_neigh_sparse(int* neigh_child, const int* neigh, const int* children, int node_num);

void orc_octree2col(float* col, const float* data, int channel, int height,
    int kernel_sdim, int stride, const int* neigh, const int* ni, int height_col, int n);
void orc_col2octree(const float* col, float* data, int channel, int height,
    int kernel_sdim, int stride, const int* neigh, const int* ni, int height_col, int n);
void orc_octree2colP(float* col, const float* data, int channel, int height,
    int octree_h, int kernel_sdim, int stride, const int* neigh, const int* ni,
    const int* child, const int* ichild, int height_col, int n);
void orc_col2octreeP(const float* col, float* data, int channel, int height,
    int octree_h, int kernel_sdim, int stride, const int* neigh, const int* ni,
    const int* child, const int* ichild, int height_col, int n);

void orc_max_pool(float* top, int top_h, int* mask, const float* btm, int btm_h, int channel);
void orc_max_unpool(const float* top, int top_h, const int* mask, float* btm, int btm_h, int channel);
void orc_mask_pool(float* top, int top_h, const int* mask, const float* btm, int btm_h, int channel);
void orc_pad_forward(float* Y, int Hy, int C, const float* X, int Hx, const int* label, float dval);
void orc_pad_backward(float* X, int Hx, int C, const float* Y, int Hy, const int* label);

void orc_generate_key_child(uint64_t* key_child, const uint64_t* key, const int* child, int node_num);
void orc_generate_key_full(uint64_t* key, int depth, int batch);
int  orc_generate_label(int* label, const int* btm, int btm_h, int mask);
void orc_octree_gather(float* top, int top_h, int channel, const float* btm, int btm_h, const int* idx);
void orc_octree_gatherbk(const float* top, int top_h, int channel, float* btm, int btm_h, const int* idx);
void orc_octree_mask(float* out, const float* in, const int* label, int height, int mask, int num);
void orc_get_bilinear(int* table512);
void orc_bilinear_neigh(int* bidx, const int* neigh, const int* child, int node_num);
void orc_bilinear_xyz(uint64_t* xyz0, float* fracs, int d0, const uint64_t* xyz1, int d1, int num);
void orc_search_key(int* idx, const uint64_t* key, int n_key, const uint64_t* query, int n_query);
void orc_xyz2key(uint64_t* key, const uint64_t* xyz, int num, int depth);
void orc_key2xyz(uint64_t* xyz, const uint64_t* key, int num, int depth);
void orc_key2idx(int* idx, const uint64_t* key, int num);

/* C[M,N] = op(A) * op(B), row-major, fp32 accumulate with k ascending */
void orc_sgemm(int transA, int transB, int M, int N, int K, const float* A,
    const float* B, float beta, float* C);

/* Output height of conv / deconv (octree/octree/octree_conv.cpp:48-81). */
int orc_conv_top_h(const void* blob, int depth, int stride, int nempty, int is_deconv);
/* conv: octree2col + GEMM; deconv: GEMM(W^T) + col2octree
 * (octree/octree/octree_conv.cpp:157-207, pytorch/cpp/octree_conv.cpp:131-213).
 * Returns top_h or a negative error. */
int orc_octree_conv(float* top, const float* btm, int channel_in, int btm_h,
    const float* weights, const void* blob, int depth, int num_output,
    const int* kernel_size, int stride, int nempty);
int orc_octree_deconv(float* top, const float* btm, int channel_in, int btm_h,
    const float* weights, const void* blob, int depth, int num_output,
    const int* kernel_size, int stride, int nempty);

/* upgrade_key64, octree/octree/transform_octree.cpp:433-497 (result through orc_fetch) */
int64_t orc_upgrade_key64(const void* blob32, int64_t bytes);

/* Point-cloud transforms, pytorch/cpp/transform_points.cpp:7-125.  The blob-producing calls
 * return the size of the transformed copy (orc_fetch). */
int orc_bounding_sphere(const void* points_blob, int method_box, float* out4);
int64_t orc_normalize_points(const void* points_blob, int64_t bytes, float radius, const float* center);
int64_t orc_transform_points(const void* points_blob, int64_t bytes, const float* angle, const float* scale,
    const float* jitter, float offset, const char* normal_axis);
int64_t orc_clip_points(const void* points_blob, int64_t bytes, const float* bbmin, const float* bbmax,
    int* inbox_mask);
void orc_rotation_matrix(float* rot, const float* angle);

/* OctreeConvGradOp / OctreeDeconvGradOp, pytorch/cpp/octree_conv.cpp:159-250:
 * grad_data has the shape of data_in, grad_w the shape of weights. */
int orc_octree_conv_grad(float* grad_data, float* grad_w, const float* data_in, int channel_in, int btm_h,
    const float* weights, const float* grad_out, const void* blob, int depth, int num_output,
    const int* kernel_size, int stride, int nempty);
int orc_octree_deconv_grad(float* grad_data, float* grad_w, const float* data_in, int channel_in, int btm_h,
    const float* weights, const float* grad_out, const void* blob, int depth, int num_output,
    const int* kernel_size, int stride, int nempty);

/* octree_dropout, octree/octree/transform_octree.cpp:286-431, with the random flags of level
 * `depth_dropout` (one byte per node, non-zero = dropped) as an argument. */
int64_t orc_octree_dropout(const void* blob, const unsigned char* flags, int depth_dropout);
/* octree_scan, pytorch/cpp/transform_octree.cpp:5-22 over ScanOctree
 * (octree/octree/transform_octree.cpp:11-297): the octree seen from n_axis directions
 * (orc_fetch).  orc_scan_frame: x, y, z axes and lower corner of one view, and its pixel width. */
int64_t orc_octree_scan(const void* blob, const float* axis, int n_axis, float scale);
void orc_scan_frame(float* frame12, int* width, const float* z, int depth, float scale);

#ifdef __cplusplus
}
#endif
#endif  /* OCNN_ORACLE_H_ */
