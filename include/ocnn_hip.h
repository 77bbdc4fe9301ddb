/* C-ABI of libocnn_hip.so: the O-CNN octree hot path as hand-written HIP
 * kernels for gfx950 (MI355X).
 *
 * Conventions
 *  - Every entry point returns 0 on success or a negative OCNN_E_* code; the
 *    message of the last failure on the calling thread is ocnn_last_error().
 *    Nothing aborts the process (the reference CHECK()s abort:
 *    octree/octree/logs.h:23-29).
 *  - Pointers named *_dev / data / top / btm / col / neigh / key ... are DEVICE
 *    pointers; `info` is always a HOST pointer to the 716-byte OctreeInfo
 *    header of the blob (octree/octree/octree_info.h:96-118).  The reference
 *    re-reads that header from the device with a blocking copy on every call
 *    (octree/octree/octree_parser.cu:4-27); here the caller keeps a host copy.
 *  - The caller owns every buffer; the library allocates nothing and never
 *    synchronises unless the function says so.  `stream` is a hipStream_t
 *    (NULL = default stream); all work of a call is enqueued on it.
 *  - Feature tensors are channel-major [C, H] as in the reference
 *    (pytorch/cpp/octree2col.cpp:59-62).  `dtype` selects the element type of
 *    feature/weight buffers: OCNN_F32 (reference precision) or OCNN_BF16
 *    (bf16 storage, fp32 accumulate; no counterpart in the reference, whose
 *    ops are float/double only: octree/octree/octree_conv.cpp:360-361).
 *  - Keys are 64-bit (the reference's KEY64 build, mandatory for its PyTorch
 *    frontend: pytorch/setup.py:29,58); child/neigh/mask/label are int32.
 *  - Neighbour index tables (`ni`, `parent`, `dis` of NeighHelper,
 *    octree/octree/octree_nn.cpp:6-81) live inside the library; where the
 *    reference takes a device `ni` pointer these functions take the host
 *    `kernel_size[3]` instead.
 */
#ifndef OCNN_HIP_H_
#define OCNN_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* ocnn_stream_t; /* hipStream_t */

enum { OCNN_F32 = 0, OCNN_BF16 = 1 };

enum {
  OCNN_OK = 0,
  OCNN_E_BADARG = -1,      /* null pointer, negative size, bad enum */
  OCNN_E_UNSUPPORTED = -2, /* valid request this build does not implement */
  OCNN_E_SHAPE = -3,       /* tensor height/channel disagrees with the octree */
  OCNN_E_WORKSPACE = -4,   /* workspace missing or too small */
  OCNN_E_HIP = -5,         /* a HIP runtime call failed */
  OCNN_E_FORMAT = -6       /* malformed OctreeInfo / PointsInfo header */
};

/* property selectors = OctreeInfo::PropType (octree/octree/octree_info.h:12-14) */
enum { OCNN_KEY = 1, OCNN_CHILD = 2, OCNN_NEIGH = 4, OCNN_FEATURE = 8, OCNN_LABEL = 16, OCNN_SPLIT = 32 };

#define OCNN_INFO_BYTES 716   /* sizeof(OctreeInfo) */
#define OCNN_HEADER_BYTES 720 /* payload offset, octree_info.cpp:258 */
#define OCNN_POINTS_INFO_BYTES 88 /* sizeof(PointsInfo), points_info.h:35-39 */

const char* ocnn_last_error(void);
int ocnn_version(void);
/* 0 when device `dev` exists and is a gfx950 part. */
int ocnn_device_check(int dev);

/* ---- OctreeInfo accessors (host only).  Replace OctreeInfo::node_num() etc.,
 * octree/octree/octree_info.h:34-61 and check_format octree_info.cpp:80-116. */
int ocnn_info_check(const void* info);
int ocnn_info_batch_size(const void* info);
int ocnn_info_depth(const void* info);
int ocnn_info_full_depth(const void* info);
int ocnn_info_is_key2xyz(const void* info);
int ocnn_info_node_num(const void* info, int depth);
int ocnn_info_node_num_nempty(const void* info, int depth);
int ocnn_info_node_num_cum(const void* info, int depth);
int ocnn_info_total_nnum(const void* info);
int ocnn_info_channel(const void* info, int ptype);
int ocnn_info_location(const void* info, int ptype);
/* byte offset of a property at a depth inside the blob, -1 if absent
 * (OctreeInfo::ptr_dis, octree_info.cpp:157-167) */
int64_t ocnn_info_ptr_dis(const void* info, int ptype, int depth);
int64_t ocnn_info_sizeof_octree(const void* info);

/* ---- padding: pad_forward_gpu / pad_backward_gpu, octree/octree/octree_nn.h:69-77,
 * octree_nn.cu:65-106.  pad_backward writes only the rows label[] names. */
int ocnn_pad_forward(void* Y, int Hy, int C, const void* X, int Hx, const int* label,
    float dval, int dtype, ocnn_stream_t stream);
int ocnn_pad_backward(void* X, int Hx, int C, const void* Y, int Hy, const int* label,
    int dtype, ocnn_stream_t stream);
/* pad_forward with one value per channel for the rows without a source (`fill`: device, fp32 [C],
 * rounded to `dtype`), no counterpart in the reference: what conv -> pad -> BatchNorm -> ReLU
 * (pytorch/ocnn/octree_conv.py:102-113 inside pytorch/ocnn/modules.py:23-36) leaves in an empty node
 * once the BatchNorm is folded into the convolution, relu(shift), in the same pass as the pad. */
int ocnn_pad_forward_fill(void* Y, int Hy, int C, const void* X, int Hx, const int* label,
    const float* fill, int dtype, ocnn_stream_t stream);
/* int32 variant used to invert `children` into `ichild`
 * (pytorch/cpp/octree2col.cpp:10-20): ichild[child[h]] = h. */
int ocnn_make_ichild(int* ichild, int n_nempty, const int* child, int n_node, ocnn_stream_t stream);

/* ---- octree2col / col2octree: octree/octree/octree_nn.h:80-120, octree_nn.cu:110-253.
 * Same argument meaning as the reference; `kernel_size` (host) replaces `ni`.
 * col2octree sets the rows of `data` on chunk n == 0 and adds to them on later chunks.
 * For the neighbour table of an octree it sums each row's taps in ascending tap order
 * (no atomics, same result on every run); the call first checks on the device that the
 * table maps back and forth consistently and otherwise scatter-adds as the reference
 * does, so any table gives the reference's result.  col2octreeP with stride 2 and a null
 * `ichild` always scatter-adds.
 * With these plain signatures the verdict of the check travels from the check kernel to the
 * summing kernels of the same call through one of 1024 words that the library holds per device,
 * chosen by a per-call counter: calls on ONE stream never share a live word; calls that overlap on
 * different streams share one only when 1024 or more col2octree calls were issued between them
 * (then a call may sum by the other's verdict: still the reference's result for octree tables,
 * wrong only if exactly one of the two tables is inconsistent).  ocnn_col2octree_cached below has
 * no such bound: the word is the caller's. */
int ocnn_octree2col(void* col, const void* data, int channel, int height, const int* kernel_size,
    int stride, const int* neigh, int height_col, int n, int dtype, ocnn_stream_t stream);
int ocnn_col2octree(const void* col, void* data, int channel, int height, const int* kernel_size,
    int stride, const int* neigh, int height_col, int n, int dtype, ocnn_stream_t stream);
int ocnn_octree2colP(void* col, const void* data, int channel, int height, int octree_h,
    const int* kernel_size, int stride, const int* neigh, const int* child, const int* ichild,
    int height_col, int n, int dtype, ocnn_stream_t stream);
int ocnn_col2octreeP(const void* col, void* data, int channel, int height, int octree_h,
    const int* kernel_size, int stride, const int* neigh, const int* child, const int* ichild,
    int height_col, int n, int dtype, ocnn_stream_t stream);

/* col2octree / col2octreeP (child == NULL / non-NULL) with the verdict on the table kept in a
 * word the caller owns, no counterpart in the reference.  The gather form of col2octree is
 * exact only for a table that maps back and forth consistently, which a check kernel verifies
 * on the device; with the plain signatures above that check runs in every call.  Here
 * `table_mark_dev` is an 8-byte device word that the caller zeroes once per (table, kernel
 * size, stride, chunking): a call with check_now != 0 runs the check and leaves its verdict in
 * the word, later calls with the same table and shape pass check_now = 0 and skip it (the
 * kernels read the verdict from the word).  One octree level, its own NEIGH table and a fixed
 * kernel shape -- what a Col2Octree module or a convolution's backward pass sees -- qualify. */
int ocnn_col2octree_cached(const void* col, void* data, int channel, int height, int octree_h,
    const int* kernel_size, int stride, const int* neigh, const int* child, const int* ichild,
    int height_col, int n, int dtype, unsigned long long* table_mark_dev, int check_now,
    ocnn_stream_t stream);

/* ---- pooling: octree/octree/octree_nn.h:122-139, octree_nn.cu:258-327.
 * mask holds absolute row indices; the first maximum wins. */
int ocnn_octree_max_pool(void* top, int top_h, int* mask, const void* btm, int btm_h,
    int channel, int dtype, ocnn_stream_t stream);
int ocnn_octree_max_unpool(const void* top, int top_h, const int* mask, void* btm, int btm_h,
    int channel, int dtype, ocnn_stream_t stream);
int ocnn_octree_mask_pool(void* top, int top_h, const int* mask, const void* btm, int btm_h,
    int channel, int dtype, ocnn_stream_t stream);

/* ---- neighbour tables: calc_neigh_gpu (both overloads),
 * octree/octree/octree_nn.h:142-147, octree_nn.cu:331-413. */
int ocnn_calc_neigh_sparse(int* neigh_child, const int* neigh, const int* children,
    int node_num, ocnn_stream_t stream);
int ocnn_calc_neigh_full(int* neigh, int depth, int batch_size, ocnn_stream_t stream);

/* ---- keys / labels: octree/octree/octree_nn.h:150-192, 229-240,
 * octree_nn.cu:417-488, 575-665. */
int ocnn_generate_key_child(uint64_t* key_child, const uint64_t* key, const int* child,
    int node_num, ocnn_stream_t stream);
int ocnn_generate_key_full(uint64_t* key, int depth, int batch_size, ocnn_stream_t stream);
/* label[i] = (btm[i]==mask) ? running count : -1; the count goes to *count_dev
 * (device int).  scratch_dev: at least ocnn_generate_label_scratch_bytes(btm_h). */
size_t ocnn_generate_label_scratch_bytes(int btm_h);
int ocnn_generate_label(int* label, int* count_dev, const int* btm, int btm_h, int mask,
    void* scratch_dev, size_t scratch_bytes, ocnn_stream_t stream);
int ocnn_sequence(int* ptr, int num, ocnn_stream_t stream);
int ocnn_search_key(int* idx, const uint64_t* key, int n_key, const uint64_t* query,
    int n_query, ocnn_stream_t stream);
/* search_key_gpu (octree/octree/octree_nn.h:180-181) for many queries in a large array: the same
 * result (position of the first equal key, -1 on a miss), through two tables of samples of `key`
 * that the call writes into workspace_dev (every 256th and every 16th key;
 * ocnn_search_key_workspace_bytes(n_key) bytes, 128-byte aligned).  With fewer than 16384 queries or
 * keys, or more than 3.1 M keys, the call is ocnn_search_key and the workspace may be null. */
size_t ocnn_search_key_workspace_bytes(int n_key);
int ocnn_search_key_indexed(int* idx, const uint64_t* key, int n_key, const uint64_t* query,
    int n_query, void* workspace_dev, size_t workspace_bytes, ocnn_stream_t stream);
int ocnn_xyz2key(uint64_t* key, const uint64_t* xyz, int num, int depth, ocnn_stream_t stream);
int ocnn_key2xyz(uint64_t* xyz, const uint64_t* key, int num, int depth, ocnn_stream_t stream);
int ocnn_key2idx(int* idx, const uint64_t* key, int num, ocnn_stream_t stream);

/* ---- octree convolution / deconvolution: OctreeConvOp / OctreeDeconvOp,
 * pytorch/cpp/octree_conv.cpp:131-213, shape rules octree/octree/octree_conv.cpp:10-122.
 * Implemented as an implicit GEMM on the matrix cores: the neighbour gather
 * feeds MFMA directly, no [Cin*K, H] column buffer is materialised.
 *   weights: [conv_out, conv_in*K] row-major with column index c*K + k
 *            (conv: [num_output, channel_in*K]; deconv: [channel_in, num_output*K])
 *   btm:     [channel_in, btm_h]     top: [num_output, top_h]
 * ocnn_conv_shape fills the output height, the input height the octree
 * demands (pytorch/cpp/octree_conv.cpp:72-78) and the workspace the call needs. */
int ocnn_conv_shape(const void* info, int depth, int channel_in, int num_output,
    const int* kernel_size, int stride, int nempty, int is_deconv, int dtype,
    int* top_h, int* btm_h, size_t* workspace_bytes);
int ocnn_octree_conv(void* top, const void* btm, int channel_in, int btm_h, const void* weights,
    const void* octree_dev, const void* info, int depth, int num_output, const int* kernel_size,
    int stride, int nempty, int dtype, void* workspace_dev, size_t workspace_bytes,
    ocnn_stream_t stream);
int ocnn_octree_deconv(void* top, const void* btm, int channel_in, int btm_h, const void* weights,
    const void* octree_dev, const void* info, int depth, int num_output, const int* kernel_size,
    int stride, int nempty, int dtype, void* workspace_dev, size_t workspace_bytes,
    ocnn_stream_t stream);

/* Convolution or deconvolution with the epilogue of the reference's conv -> BatchNorm -> ReLU
 * modules (pytorch/ocnn/modules.py:23-36) folded in: `weights` already carry the BatchNorm
 * scale, `bias` (device, fp32 [num_output], may be NULL) its shift; relu != 0 clamps at zero.
 * Bias and ReLU act on the fp32 accumulator before the store. */
int ocnn_octree_conv_fused(void* top, const void* btm, int channel_in, int btm_h, const void* weights,
    const float* bias, int relu, int is_deconv, const void* octree_dev, const void* info, int depth,
    int num_output, const int* kernel_size, int stride, int nempty, int dtype, void* workspace_dev,
    size_t workspace_bytes, ocnn_stream_t stream);

/* ocnn_octree_conv_fused with the caller's table of source rows for an operator over the non-empty
 * nodes (`sources_dev` / `sources_bytes` as ocnn_conv_rows_sources_bytes / ocnn_conv_rows_sources
 * make them for this octree, depth, kernel shape, stride and direction; NULL: the call is
 * ocnn_octree_conv_fused).  The table depends on the octree level and the operator's geometry alone,
 * so the layers of a depth share one; a call that brings it looks nothing up and makes no inverted
 * child links.  The results are the same bits.  Ignored by the operators that look nothing up
 * (nempty 0, 1x1x1, the fp32 2x2x2 stride-2 deconvolution).  No counterpart in the reference, which
 * makes its gather indices inside every call (octree_nn.cu:179-253). */
int ocnn_octree_conv_fused_sources(void* top, const void* btm, int channel_in, int btm_h, const void* weights,
    const float* bias, int relu, int is_deconv, const int* sources_dev, size_t sources_bytes, const void* octree_dev,
    const void* info, int depth, int num_output, const int* kernel_size, int stride, int nempty, int dtype,
    void* workspace_dev, size_t workspace_bytes, ocnn_stream_t stream);

/* Two 1x1x1 convolutions in one pass: hidden = W1 data + b1 (ReLU when relu1 != 0), out = W2 hidden
 * + b2, label (may be NULL) = argmax over the channels of out (the first of equal maxima).  It is
 * the prediction head of the reference's decoders, OctreeConv1x1BnRelu(C, 32) -> OctreeConv1x1(32, n)
 * (pytorch/ocnn/ounet.py:46-49, modules.py:71-107; with `logit.argmax(1)`, ounet.py:82-88 and
 * 114-119), with the BatchNorm folded into w1 / b1; the reference runs it as two torch Conv1d.
 * fp32, channel-major: data [channel_in, height], w1 [hidden, channel_in], w2 [num_output, hidden],
 * out [num_output, height], label int32 [height]; b1 / b2 may be NULL; hidden <= 32 and
 * num_output <= 8, else OCNN_E_UNSUPPORTED (run two ocnn_octree_conv_fused then).  The hidden
 * channels are not written anywhere. */
int ocnn_conv1x1_pair(float* out, int* label, const float* data, int channel_in, int height, const float* w1,
    const float* b1, int hidden, int relu1, const float* w2, const float* b2, int num_output, ocnn_stream_t stream);

/* Row-major activations, no counterpart in the reference (whose tensors are channel-major
 * [1, C, H, 1]): rows [H + 1][pitch] bf16, row h = the channels of node h, pitch = channels
 * rounded up to a multiple of 16, padding channels zero, row H all zero (what a missing
 * neighbour reads).  It is the layout the bf16 3x3x3 kernels gather from; the channel-major entry
 * points copy their input into it on every call.  A chain of convolutions converts once
 * (ocnn_rows_from_channels), runs ocnn_octree_conv_rows for every member, and converts back once
 * (ocnn_channels_from_rows).
 *   ocnn_octree_conv_rows: bf16; with nempty 0
 *     kernel 3x3x3 stride 1 (conv or deconv): rows of `depth` in and out; arithmetic and rounding
 *       as ocnn_octree_conv_fused, the results are bit-identical;
 *     kernel 2x2x2 stride 2, conv: rows of `depth` in, rows of ALL nodes of depth-1 out: the
 *       octree_pad that the reference's modules put behind the operator
 *       (pytorch/ocnn/octree_conv.py:102-127) is folded in, an empty node receives the bias alone;
 *     kernel 2x2x2 stride 2, deconv: rows of ALL nodes of `depth` in (the octree_depad of those
 *       modules is folded in), rows of depth+1 out; at most 256 input channels;
 *   with nempty 1 (rows = ranks of the non-empty nodes on both sides, the operator of the
 *   channel-major entry points, pytorch/cpp/octree_conv.cpp:131-216): kernel 3x3x3 stride 1 and
 *   kernel 2x2x2 stride 2, conv and deconv;
 *   anything else: OCNN_E_UNSUPPORTED.
 *   btm_pitch = 16 * ceil(channel_in / 16) (the stride-2 convolution also takes a larger multiple
 *   of 8: its input may be a channel slice of a wider tensor; so do the nempty operators).  top_pitch: channels per row of the tensor `top_rows`
 *   points into, a multiple of 8, at least 16 * ceil(num_output / 16); the call writes channels
 *   0 .. 16 * ceil(num_output / 16) - 1 of every row and of the zero row and nothing else, so
 *   `top_rows` may be a channel slice of a wider tensor.  ocnn_conv_rows_shape: row counts and
 *   workspace bytes of such a call. */
int ocnn_conv_rows_shape(const void* info, int depth, int channel_in, int num_output, const int* kernel_size,
    int stride, int nempty, int is_deconv, int dtype, int* top_h, int* btm_h, size_t* workspace_bytes);
int ocnn_octree_conv_rows(void* top_rows, int top_pitch, const void* btm_rows, int btm_pitch, int channel_in,
    int btm_h, const void* weights, const float* bias, int relu, int is_deconv, const void* octree_dev,
    const void* info, int depth, int num_output, const int* kernel_size, int stride, int nempty, int dtype,
    void* workspace_dev, size_t workspace_bytes, ocnn_stream_t stream);
/* The same operator for weights that do not change from call to call (inference): pack them once
 * (ocnn_conv_rows_packed_bytes bytes, 16-byte aligned; the order depends on the channel counts, the
 * kernel, the stride, nempty, is_deconv and, for nempty operators, on whether at least one node in
 * five of the level of the columns is non-empty: pack with the header of the octree the call will run on,
 * or of one like it) and pass the packed form; `ichild_dev`: the
 * inverted child links from ocnn_make_ichild for the operators that use them -- every nempty
 * operator (links of `depth`; of depth+1 for the stride-2 deconvolution) and the all-nodes stride-2
 * deconvolution (links of `depth`) -- or NULL, then the call computes them into the workspace
 * (ocnn_conv_rows_shape bytes are enough).  With both, no workspace is needed and the call launches
 * the convolution kernel alone.  `packed_bytes` must be what ocnn_conv_rows_packed_bytes returns for
 * the very operator of the call (OCNN_E_WORKSPACE otherwise: a buffer packed for another shape). */
int ocnn_conv_rows_packed_bytes(const void* info, int depth, int channel_in, int num_output, const int* kernel_size,
    int stride, int nempty, int is_deconv, int dtype, size_t* packed_bytes);
int ocnn_conv_rows_pack(void* packed_dev, size_t packed_bytes, const void* weights, const void* octree_dev,
    const void* info, int depth, int channel_in, int num_output, const int* kernel_size, int stride, int nempty,
    int is_deconv, int dtype, ocnn_stream_t stream);
int ocnn_octree_conv_rows_packed(void* top_rows, int top_pitch, const void* btm_rows, int btm_pitch, int channel_in,
    int btm_h, const void* packed_weights, size_t packed_bytes, const int* ichild_dev, const int* sources_dev,
    const float* bias, int relu, int is_deconv, const void* octree_dev, const void* info, int depth, int num_output,
    const int* kernel_size, int stride, int nempty, int dtype, void* workspace_dev, size_t workspace_bytes,
    ocnn_stream_t stream);
/* The nempty operators first look up, for every output column, the source row of each tap (through
 * the neighbour table and the child links).  The result depends on the octree, the depth, the
 * kernel shape, the stride and is_deconv only -- not on channels or weights -- so the layers of a
 * network that work on one level share it: ocnn_conv_rows_sources writes that table
 * (ocnn_conv_rows_sources_bytes bytes, int32; `ichild_dev` as above or NULL with a workspace of
 * ocnn_conv_rows_shape bytes), and ocnn_octree_conv_rows_packed takes it as `sources_dev` (NULL:
 * the rows are looked up tile by tile inside the convolution kernel).  With a table the call needs
 * no `ichild_dev`.  Same results in either case.  Depth-9 scene, 64 -> 64 over the non-empty
 * nodes: 0.061 ms with the table against 0.076 ms without. */
int ocnn_conv_rows_sources_bytes(const void* info, int depth, const int* kernel_size, int stride, int nempty,
    int is_deconv, size_t* sources_bytes);
int ocnn_conv_rows_sources(int* sources_dev, size_t sources_bytes, const int* ichild_dev, const void* octree_dev,
    const void* info, int depth, const int* kernel_size, int stride, int nempty, int is_deconv, void* workspace_dev,
    size_t workspace_bytes, ocnn_stream_t stream);
int ocnn_rows_from_channels(void* rows, int pitch, const void* data, int channel, int height, int dtype,
    ocnn_stream_t stream);
int ocnn_channels_from_rows(void* data, const void* rows, int pitch, int channel, int height, int dtype,
    ocnn_stream_t stream);

/* OctreeMaxPool on row-major activations (pytorch/ocnn/octree_pool.py:79-86: octree_max_pool at
 * `depth` followed by octree_pad at depth-1; no row-major counterpart in the reference): rows of
 * `depth` in, rows of ALL nodes of depth-1 out; a node with children takes the channel-wise
 * maximum of their eight rows (the first maximum wins), a node without gets zeros; the zero row
 * behind the last one and the padding channels are written.  mask_rows (may be NULL): int32
 * [nnum(depth-1) + 1][top_pitch], the absolute row of each maximum, -1 for an empty node.
 * Values and mask equal the channel-major pair bit for bit.  bf16; pitches as in
 * ocnn_octree_conv_rows, so that a conv -> pool -> conv chain (pytorch/ocnn/lenet.py:24-32) stays
 * in this layout. */
int ocnn_octree_max_pool_rows(void* top_rows, int top_pitch, int* mask_rows, const void* btm_rows, int btm_pitch,
    int channel, const void* octree_dev, const void* info, int depth, int dtype, ocnn_stream_t stream);

/* Test hook and tuning knob, no counterpart in the reference (process-wide: a thread that flips it
 * changes the kernel other threads' bf16 convolutions run from then on; their results do not
 * change, only their timing): 3x3x3 stride-1 bf16 convolutions over all nodes
 * run one of two kernels, chosen by the number of 1024-column tiles of the level; the
 * register-fed kernel takes levels of at least `tiles` tiles (default 192, about 200 000
 * octants).  0 restores the default, a negative value sends every level to it (the tests use
 * that to run it on small octrees).  Returns the previous threshold.  Both kernels add the same
 * products in the same order: the results do not depend on the choice. */
int ocnn_conv_bf16_tile_threshold(int tiles);

/* Test hook, no counterpart in the reference (process-wide, like the knob above): the bf16 row
 * kernels for tap sets of three taps or more exist in two forms that add the same products in the
 * same order -- weights staged in LDS for all taps of a tile, or read per live tap straight from
 * the packed weights (the default where it is faster: everywhere but the channel-major operators
 * with whole blocks of 128 output channels).  The fp32 kernel for the non-empty nodes has the same
 * two forms (the second one on levels where fewer than one node in five is non-empty) and follows
 * the same switch.  0 sends every call to the staged form, 1 restores the default, 2 is 1 with the
 * fp32 kernel's second form on every level (the tests run it on small octrees).  Returns the
 * previous setting of the bf16 kernels (0 or 1). */
int ocnn_conv_rows_direct(int on);

/* Test hook, no counterpart in the reference (process-wide): the weight gradient of the shapes
 * other than 3x3x3 stride 1 over all nodes (non-empty nodes, stride 2, smaller tap sets) with whole
 * 32-channel blocks and 32 or whole 64 output channels stages its source rows in LDS from a table
 * of row numbers; 0 sends these shapes to the register-fed kernel that serves every other channel
 * count, 1 restores the default.  Both add the same products, in different orders (fp32, 1e-4).
 * Returns the previous setting. */
int ocnn_conv_wgrad_staged(int on);

/* ocnn_octree_conv_fused for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments and results minus the workspace: the packed weights, the inverted
 * child links of the non-empty mode and, for the kernels that read one, the row-major copy of
 * the input go into an array of OCNN_STATIC_SCRATCH_BYTES bytes that the library holds on every
 * GPU it runs on until the process ends.  A call that needs more fails with OCNN_E_WORKSPACE and
 * a message that says how much (fp32 convolutions over all nodes and every 2x2x2 stride-2 fp32
 * or bf16 convolution need the packed weights only, so any octree size fits; bf16 3x3x3 and the
 * non-empty mode also need 2 or 4 bytes x padded channels x input rows).  The call allocates
 * nothing and waits for nothing.  All calls on one GPU share the array: calls that overlap on
 * one GPU (two streams, two threads) race; calls on one stream are ordered and safe.
 * ocnn_device_check(dev) resolves the array's address for `dev` ahead of time; otherwise the
 * first call on a device does. */
#define OCNN_STATIC_SCRATCH_BYTES (16u << 20)
int ocnn_octree_conv_static(void* top, const void* btm, int channel_in, int btm_h, const void* weights,
    const float* bias, int relu, int is_deconv, const void* octree_dev, const void* info, int depth,
    int num_output, const int* kernel_size, int stride, int nempty, int dtype, ocnn_stream_t stream);

/* ---- gradients: OctreeConvGradOp / OctreeDeconvGradOp, pytorch/cpp/octree_conv.cpp:159-250
 * (weight_gpu_gemm / backward_gpu_gemm / forward_gpu_gemm, octree/octree/octree_conv.cpp:276-356).
 * Arguments are those of the forward call plus `grad_out` [num_output, top_h]; the results have
 * the shapes of `data_in` and `weights`.  Either result pointer may be NULL to skip it.
 * The weight gradient contracts over the octree nodes on the matrix cores without a column
 * buffer and adds its partial sums in a fixed order (reproducible); the data gradient is the
 * transposed operator with the same weight buffer.  fp32 only (OCNN_E_UNSUPPORTED otherwise). */
int ocnn_conv_grad_workspace_bytes(const void* info, int depth, int channel_in, int num_output,
    const int* kernel_size, int stride, int nempty, int is_deconv, int dtype, size_t* workspace_bytes);
int ocnn_octree_conv_grad(void* grad_data, void* grad_weights, const void* data_in, int channel_in,
    int btm_h, const void* weights, const void* grad_out, const void* octree_dev, const void* info,
    int depth, int num_output, const int* kernel_size, int stride, int nempty, int dtype,
    void* workspace_dev, size_t workspace_bytes, ocnn_stream_t stream);
int ocnn_octree_deconv_grad(void* grad_data, void* grad_weights, const void* data_in, int channel_in,
    int btm_h, const void* weights, const void* grad_out, const void* octree_dev, const void* info,
    int depth, int num_output, const int* kernel_size, int stride, int nempty, int dtype,
    void* workspace_dev, size_t workspace_bytes, ocnn_stream_t stream);

/* ---- feature transfer between octrees and to free points.
 * ocnn_align_forward / backward: align_forward_gpu / align_backward_gpu
 * (octree/octree/octree_nn.h:196-201, octree_nn.cu:710-752): top[c, idx[h]] = btm[c, h] for
 * idx[h] != -1 (top is zero-filled first); backward gathers.  `octree_align`
 * (pytorch/cpp/octree_align.cpp:9-83) = key arrays of both octrees -> ocnn_search_key -> this.
 * ocnn_align_forward_ws: the same result with `inverse_ws` (top_h ints of device memory, contents
 * ignored and overwritten): idx is inverted there and every row of top is written once, its
 * source row or zero, instead of twice.  Where two rows of btm name one row of top (keys of an
 * octree never do) one of them wins, as in the scatter.
 * ocnn_align_forward_add: top[c, idx[h]] += btm[c, h] for idx[h] != -1, the rows of top that
 * nothing is moved to keep their values: `deconv + octree_align(skip, ...)` of the decoder loop
 * (pytorch/ocnn/ounet.py:109-111) in one pass over the two tensors.  Two rows of btm must not
 * name one row of top (keys of an octree never do).
 * ocnn_octree_interp: octree_nearest_pts (method 0) / octree_trilinear_pts (method 1) of
 * pytorch/ocnn/modules.py:209-275 in two kernels.  key[n_key]: the sorted Morton keys of the
 * searched depth (de-padded by the caller for nempty, as octree_search_key does,
 * pytorch/cpp/octree_key.cpp:83-132); pts [n_pts, 4] = (x, y, z in [0, 2^depth], batch id);
 * out [channel, n_pts].  idx / weight [n_pts * K] (K = 1 nearest, 8 linear) are filled for the
 * backward call, which zero-fills grad_data [channel, H] and scatters with fp32 atomics. */
int ocnn_align_forward(float* top, int top_h, int channel, const float* btm, int btm_h, const int* idx,
    ocnn_stream_t stream);
int ocnn_align_forward_add(float* top, int top_h, int channel, const float* btm, int btm_h, const int* idx,
    ocnn_stream_t stream);
int ocnn_align_forward_ws(float* top, int top_h, int channel, const float* btm, int btm_h, const int* idx,
    int* inverse_ws, ocnn_stream_t stream);
int ocnn_align_backward(const float* top, int top_h, int channel, float* btm, int btm_h, const int* idx,
    ocnn_stream_t stream);
int ocnn_octree_interp(float* out, const float* data, int channel, int H, const uint64_t* key, int n_key,
    const float* pts, int n_pts, int depth, int method, int* idx, float* weight, ocnn_stream_t stream);
/* The same with a workspace of ocnn_octree_interp_workspace_bytes(channel, H) bytes (16-byte
 * aligned; may be NULL): when the points ask for at least half as many rows as the level has,
 * the features are first copied row-major into it and every corner is read as one contiguous
 * row (several times faster for 64 channels).  Same results. */
size_t ocnn_octree_interp_workspace_bytes(int channel, int H);
int ocnn_octree_interp_ws(float* out, const float* data, int channel, int H, const uint64_t* key, int n_key,
    const float* pts, int n_pts, int depth, int method, int* idx, float* weight, void* workspace_dev,
    size_t workspace_bytes, ocnn_stream_t stream);
int ocnn_octree_interp_backward(float* grad_data, const float* grad_out, int channel, int H, int n_pts,
    int method, const int* idx, const float* weight, ocnn_stream_t stream);
/* The backward call with an optional workspace of
 * ocnn_octree_interp_backward_workspace_bytes(channel, H, n_pts, method) bytes (16-byte aligned):
 * the (point, corner) pairs are binned by node and every node sums its pairs (a gather, no
 * floating-point atomics); used when the points name at least half as many corners as the
 * level has nodes, the atomic scatter otherwise or without a workspace. */
size_t ocnn_octree_interp_backward_workspace_bytes(int channel, int H, int n_pts, int method);
int ocnn_octree_interp_backward_ws(float* grad_data, const float* grad_out, int channel, int H, int n_pts,
    int method, const int* idx, const float* weight, void* workspace_dev, size_t workspace_bytes,
    ocnn_stream_t stream);

/* ---- octree_gather_gpu / octree_gatherbk_gpu / octree_mask_gpu, octree/octree/octree_nn.h:204-218
 * (kernels octree_nn.cu:756-818).
 *   gather    top[c, h] = idx[h] != -1 ? btm[c, idx[h]] : 0   (the reference's pad_forward with 0)
 *   gatherbk  btm zero-filled, then btm[c, idx[h]] += top[c, h]; idx may name a row many times.
 *             With a workspace of ocnn_octree_gatherbk_workspace_bytes(channel, btm_h, top_h) bytes
 *             (16-byte aligned) the rows are binned by target and every target sums its sources,
 *             without floating-point atomics; without one (NULL) an atomic scatter-add as in the
 *             reference.  fp32.
 *   mask      out[i] = label[i % height] == mask ? 0 : in[i] for i < num */
int ocnn_octree_gather(void* top, int top_h, int channel, const void* btm, int btm_h, const int* idx, int dtype,
    ocnn_stream_t stream);
size_t ocnn_octree_gatherbk_workspace_bytes(int channel, int btm_h, int top_h);
int ocnn_octree_gatherbk(const float* top, int top_h, int channel, float* btm, int btm_h, const int* idx,
    void* workspace_dev, size_t workspace_bytes, ocnn_stream_t stream);
int ocnn_octree_mask(float* out, const float* in, const int* label, int height, int mask, int64_t num,
    ocnn_stream_t stream);

/* ---- trilinear stencils between two levels: bilinear_neigh_gpu / bilinear_xyz_gpu,
 * octree/octree/octree_nn.h:170-177 (kernels octree_nn.cu:491-565; the 512-entry table of
 * NeighHelper::get_bilinear_array, octree_nn.cpp:83-108, is internal).
 *   bilinear_neigh  bidx[(8 child[i] + j) * 8 + k] = node of the level of `neigh` in corner k of
 *                   the interpolation cell of child j of node i, for every non-empty node i
 *                   (node_num = nodes of that level); -1 where there is none.  Corner order
 *                   000, 001, 010, 100, 011, 101, 110, 111 of (x, y, z): weights 27, 9, 9, 9, 3, 3, 3, 1.
 *   bilinear_xyz    xyz0[8 i + k] = packed coordinates (x, y, z, id in 16-bit fields) of those
 *                   cells at level d0 for cell xyz1[i] of level d1 >= d0; fracs[3 i + c] = the
 *                   weight of the nearer cell along axis c. */
int ocnn_bilinear_neigh(int* bidx, const int* neigh, const int* child, int node_num, ocnn_stream_t stream);
int ocnn_bilinear_xyz(uint64_t* xyz0, float* fracs, int d0, const uint64_t* xyz1, int d1, int num,
    ocnn_stream_t stream);

/* ---- file formats.  A `.octree` / `.points` file is the serialized blob itself
 * (Octree::read_octree / write_octree, octree/octree/octree.cpp:41-68; Points::read_points /
 * write_points, points.cpp:9-37).  Files written by a 32-bit-key build carry "_OCTREE_1.0_" and
 * 4-byte keys: ocnn_upgrade_key64 (upgrade_key64, octree/octree/transform_octree.cpp:433-497)
 * converts one to the 64-bit layout on the HOST (both buffers are host memory).  With out == NULL
 * only *out_bytes is filled. */
int ocnn_upgrade_key64(const void* octree32, size_t bytes, void* out, size_t out_capacity, size_t* out_bytes);

/* ---- point-cloud transforms on the device: pytorch/cpp/transform_points.cpp:7-125 over
 * PointsParser (octree/octree/points_parser.cpp:42-260).  `points_info` is a HOST copy of the
 * cloud's 88-byte header.  Results are bit-identical to the host loops.
 *   ocnn_bounding_sphere   method_box = 0: the sphere of math_functions.cpp:49-108 (the build
 *                          without Miniball); 1: the bounding-box sphere (:22-30).  out4 (host) =
 *                          radius, centre; blocks until it has arrived.
 *   ocnn_normalize_points  translate by -center, scale by 1/radius (:51-71)
 *   ocnn_transform_points  displace along normals, rotate (angle[3], radians), jitter, scale,
 *                          orient normals ("", "x", "y", "z", "xyz") (:73-109); out may equal in
 *   ocnn_clip_points       keeps the points strictly inside the box (:111-125): the kept points
 *                          are compacted to the front of every array of `out_dev` (a copy of the
 *                          input otherwise, as the host's in-place compaction leaves it),
 *                          inbox_mask_dev[pt_num] gets 0/1, out_info (host, 88 bytes) the new
 *                          header; blocks once for the count. */
size_t ocnn_points_workspace_bytes(int pt_num);
int ocnn_bounding_sphere(const void* points_dev, const void* points_info, int method_box, float* out4,
    void* workspace_dev, size_t workspace_bytes, ocnn_stream_t stream);
int ocnn_normalize_points(void* out_dev, const void* in_dev, const void* points_info, float radius,
    const float* center, ocnn_stream_t stream);
int ocnn_transform_points(void* out_dev, const void* in_dev, const void* points_info, const float* angle,
    const float* scale, const float* jitter, float offset, const char* normal_axis, ocnn_stream_t stream);
int ocnn_clip_points(void* out_dev, void* out_info, int* inbox_mask_dev, const void* in_dev,
    const void* points_info, const float* bbmin, const float* bbmax, void* workspace_dev,
    size_t workspace_bytes, ocnn_stream_t stream);

/* ---- octree construction on the device: points2octree + octree_batch fused.
 * Replaces Octree::build (octree/octree/octree.cpp:74-121) driven as in
 * pytorch/cpp/point2octree.cpp:5-34, and merge_octrees
 * (octree/octree/merge_octrees.cpp:7-198) driven as in pytorch/cpp/octree_batch.cpp:5-22.
 *
 * One call builds n_clouds point clouds; the result is bit-identical to what
 * the reference produces for points2octree on each cloud (n_clouds == 1 and
 * merged == 0) or for octree_batch over those octrees (merged == 1, which
 * also fills the neighbour tables).
 *
 *   points_dev[i]   device pointer to the i-th serialized point cloud
 *   points_info[i]  host pointer to its 88-byte PointsInfo header
 * Step 1 (ocnn_points2octree_plan) sorts the points and counts the nodes; it
 * ends with ONE device-to-host copy of the node counts, waits for it, and
 * writes the finished OctreeInfo header to `info_out` (host).  The caller then
 * allocates ocnn_info_sizeof_octree(info_out) bytes and step 2
 * (ocnn_points2octree_emit) writes the blob.  The workspace must stay
 * untouched between the two steps.
 * The adaptive / node_feature / extrapolate options of the reference
 * (octree.cpp:454-806, 958-1135) take two rounds of allocation and go through
 * ocnn_points2octree only (the two-step form answers OCNN_E_UNSUPPORTED).  A
 * batch (n_clouds > 1, merged == 1) goes through both stages as one octree in
 * merged layout; the result equals octree_batch over the octrees built cloud by
 * cloud (the rule of trim_octree that keeps one node per level, octree.cpp:1055-1073,
 * and the nearest-node search of extrapolate_signal, octree.cpp:776-803, are
 * applied per octree).  Two-channel keys (key2xyz with depth > 8) cannot be
 * batched, as in merge_octrees. */
typedef struct {
  int depth, full_depth;
  int node_dis, node_feature, split_label, adaptive, adp_depth;
  float th_normal, th_distance;
  int extrapolate, save_pts, key2xyz;
  int merged;          /* 0: single-octree blob (n_clouds must be 1); 1: octree_batch blob;
                          2 (plan/emit only): batch layout without neighbour tables */
  int has_bbox;        /* 0: [-1,1]^3 as pytorch/cpp does (octree_info.cpp:68-69) */
  float bbmin[3], bbmax[3];
} ocnn_build_params;
size_t ocnn_points2octree_workspace_bytes(int64_t total_points, int n_clouds, int depth);
int ocnn_points2octree_plan(const void* const* points_dev, const void* const* points_info,
    int n_clouds, const ocnn_build_params* params, void* workspace_dev, size_t workspace_bytes,
    void* info_out, ocnn_stream_t stream);
int ocnn_points2octree_emit(void* octree_out_dev, const void* info, void* workspace_dev,
    size_t workspace_bytes, ocnn_stream_t stream);
/* Both steps in one call: after step 1 the blob is obtained from `alloc(bytes, alloc_ctx)`
 * (device memory, 8-byte aligned, owned by the caller; a null return fails the call) and
 * returned in *octree_out_dev.  Same result as the two steps; it spares the host work
 * between them, which is a sizeable part of a small build
 * (pytorch/cpp/point2octree.cpp:5-34 allocates its output tensor the same way, after
 * the build knows its size). */
/* The sort and the level scan chain their tiles through bounded waits.  The first attempt
 * of a plan orders tiles by workgroup index; if a wait of `polls` polls runs out, the plan is
 * repeated once with ticket order (slower, cannot starve).  ocnn_points2octree_wait_limit sets
 * `polls` (0 restores the default, a negative value fails every first attempt: used by the
 * tests to exercise the repeat) and returns the previous value;
 * ocnn_points2octree_ticket_reruns counts the repeats so far.  No counterpart in the
 * reference, whose build is sequential. */
int ocnn_points2octree_wait_limit(int polls);
int ocnn_points2octree_ticket_reruns(void);
typedef void* (*ocnn_alloc_fn)(size_t bytes, void* alloc_ctx);
int ocnn_points2octree(const void* const* points_dev, const void* const* points_info,
    int n_clouds, const ocnn_build_params* params, void* workspace_dev, size_t workspace_bytes,
    ocnn_alloc_fn alloc, void* alloc_ctx, void* info_out, void** octree_out_dev,
    ocnn_stream_t stream);

/* Both steps in one call for a caller that obtains the blob's memory BEFORE its size is known (a
 * guess from earlier builds of similar clouds): between the level scan and the emit launch the
 * device then waits for the host's look at the node counts only, not for an allocation.  Plain
 * octrees only (as ocnn_points2octree_plan).  OCNN_OK: the blob is the first
 * ocnn_info_sizeof_octree(info_out) bytes of `octree_buf_dev`.  OCNN_E_WORKSPACE: `capacity` is too
 * small; info_out is filled and the plan is kept, the caller allocates and calls
 * ocnn_points2octree_emit.  No counterpart in the reference. */
int ocnn_points2octree_into(const void* const* points_dev, const void* const* points_info, int n_clouds,
    const ocnn_build_params* params, void* workspace_dev, size_t workspace_bytes, void* octree_buf_dev,
    size_t capacity, void* info_out, ocnn_stream_t stream);

/* ---- octree_scan, pytorch/cpp/transform_octree.cpp:5-22 over ScanOctree
 * (octree/octree/transform_octree.cpp:11-297): the part of a single octree that is visible
 * from `n_axis` directions (`axis`: 3 floats each, host), z-buffered at `scale` pixels per
 * finest-level cell.  Scratch memory and the result come from `alloc` (see
 * ocnn_points2octree); one device-to-host copy (the surviving node counts) is waited for.
 * Bit-identical to the reference's result. */
int ocnn_octree_scan(const void* octree_dev, const void* info, const float* axis, int n_axis,
    float scale, ocnn_alloc_fn alloc, void* alloc_ctx, void* info_out, void** octree_out_dev,
    ocnn_stream_t stream);

/* ---- octree_dropout, octree/octree/transform_octree.cpp:286-431 (the `OctreeDrop` op,
 * tensorflow/libs/transform_octree_op.cc:40-56): the nodes of level `depth_dropout` whose
 * flag is set (`flags_dev`: one byte per node of that level, device memory) leave with their
 * whole subtrees; the levels below are compacted and the children renumbered.  The reference
 * draws the flags on the host from an engine seeded with the clock; here the caller draws
 * them (a Bernoulli sample of the drop ratio).  With `clear_dropped` 0 the result is
 * bit-identical to the reference's for the same flags: at `depth_dropout` itself a dropped
 * node then keeps its old child entry (transform_octree.cpp:422-425), which points past the
 * compacted level below, so such a blob must not be given to anything that follows the child
 * entries of that level (the neighbour tables of octree_batch).  With `clear_dropped` 1 those
 * entries are -1 and the result is an ordinary octree.  Scratch and result come from `alloc`;
 * one device-to-host copy (the node counts) is waited for. */
int ocnn_octree_dropout(const void* octree_dev, const void* info, const unsigned char* flags_dev,
    int depth_dropout, int clear_dropped, ocnn_alloc_fn alloc, void* alloc_ctx, void* info_out, void** octree_out_dev,
    ocnn_stream_t stream);

/* ---- octree_batch of already serialized octrees that live on the device
 * (merge_octrees, octree/octree/merge_octrees.cpp:7-198).  `out_info` (host)
 * is filled by ocnn_octree_batch_info from the n host headers; the caller
 * allocates ocnn_info_sizeof_octree(out_info) bytes for `out_dev`. */
int ocnn_octree_batch_info(const void* const* infos, int n, void* out_info);
size_t ocnn_octree_batch_workspace_bytes(int n, int depth);
/* waits once for its (small) host-to-device table upload before returning */
int ocnn_octree_batch(void* out_dev, const void* out_info, const void* const* octrees_dev,
    const void* const* infos, int n, void* workspace_dev, size_t workspace_bytes,
    ocnn_stream_t stream);

/* ---- decoder-side growth: octree_new / octree_grow / octree_update,
 * pytorch/cpp/octree_grow.cpp:13-190.  The *_info functions compute the
 * header of the result on the host; the caller allocates and the second
 * function fills the blob on the device (the header is written too). */
int ocnn_octree_new_info(int batch_size, int channel, int node_dis, int adaptive_layer, void* out_info);
int ocnn_octree_new(void* out_dev, const void* out_info, ocnn_stream_t stream);
int ocnn_octree_grow_info(const void* in_info, int target_depth, int full_octree, void* out_info);
int ocnn_octree_grow(void* out_dev, const void* out_info, const void* in_dev, const void* in_info,
    int target_depth, int full_octree, ocnn_stream_t stream);
/* octree_update rewrites children[depth] of `octree_dev` IN PLACE from
 * `label` (the caller clones first, as pytorch/cpp/octree_grow.cpp:165 does),
 * waits for the split count (written by the device into pinned host memory that
 * the call polls), patches nnum_nempty[depth] in `info` (host) and in the device
 * header.
 * ocnn_octree_update_copy is octree_update with the clone inside
 * (pytorch/cpp/octree_grow.cpp:164-190 as a whole): `out_dev` (as large as the blob
 * at `in_dev`, another buffer, both 16-byte aligned) gets the blob with the new
 * children[depth] and count; the copy runs in the launch that writes the
 * children, behind the one that counts, so the call returns with the count
 * while the copy is still on its way and the caller can size the next level. */
size_t ocnn_octree_update_scratch_bytes(int n_label);
int ocnn_octree_update(void* octree_dev, void* info, const int* label, int n_label, int depth,
    int split, void* scratch_dev, size_t scratch_bytes, ocnn_stream_t stream);
int ocnn_octree_update_copy(void* out_dev, const void* in_dev, void* info, const int* label, int n_label,
    int depth, int split, void* scratch_dev, size_t scratch_bytes, ocnn_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* OCNN_HIP_H_ */
