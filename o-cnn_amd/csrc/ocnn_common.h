// Shared host/device definitions of libocnn_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>

#include <stddef.h>
#include <stdint.h>
#include <string.h>

#include "../../include/ocnn_hip.h"

namespace ocnn {

// ---------------------------------------------------------------------------
// Serialized octree header.  Field order and sizes follow the reference's
// OctreeInfo (octree/octree/octree_info.h:96-118); offsets are asserted below.
struct Info {
  char magic[16];
  int batch_size, depth, full_layer, adp_layer;
  unsigned char is_adaptive;
  float th_dist, th_norm;
  unsigned char key2xyz, has_node_dis;
  int nnum[16], nnum_cum[16], nnum_nempty[16];
  int content_flags;
  int channels[16], locations[16];
  float bbmin[3], bbmax[3];
  unsigned char extrapolate, save_pts;
  char reserved[254];
  int ptr_dis_[16];

  static int index_of(int ptype) {
    for (int i = 0; i < 6; ++i) if (ptype & (1 << i)) return i;
    return 0;
  }
  bool has(int ptype) const { return (content_flags & ptype) != 0; }
  int channel(int ptype) const { return has(ptype) ? channels[index_of(ptype)] : 0; }
  int location(int ptype) const { return has(ptype) ? locations[index_of(ptype)] : 0; }
  static int size_of(int ptype) { return ptype == OCNN_KEY ? 8 : 4; }
  int total_nnum() const { return nnum_cum[depth + 1]; }
  int total_capacity() const { return nnum_cum[depth + 2]; }
  int64_t sizeof_octree() const { return ptr_dis_[6]; }
  // byte offset of (property, depth), -1 when the property is absent
  int64_t ptr_dis(int ptype, int d) const {
    if (!has(ptype)) return -1;
    int64_t dis = ptr_dis_[index_of(ptype)];
    if (location(ptype) == -1) dis += (int64_t)nnum_cum[d] * channel(ptype) * size_of(ptype);
    return dis;
  }
  void reset();
  void set_channel(int ptype, int ch);
  void set_location(int ptype, int lc) { locations[index_of(ptype)] = lc; }
  void set_property(int ptype, int ch, int lc) { set_channel(ptype, ch); set_location(ptype, lc); }
  void set_batch_size(int b) { batch_size = b < 1 ? 1 : b; }
  void set_depth(int d) { depth = full_layer < d ? d : full_layer; }
  void set_full_layer(int fd) { full_layer = fd < 1 ? 1 : fd; }
  void set_nnum_cum(int capacity = 0);
  // false: the blob would exceed what the 32-bit offsets of the serialized format can address
  bool set_ptr_dis();
  float bbox_max_width() const;
  bool consistent_with(const Info& o) const;
};
static_assert(sizeof(Info) == OCNN_INFO_BYTES, "OctreeInfo wire size");
static_assert(offsetof(Info, th_dist) == 36 && offsetof(Info, key2xyz) == 44, "layout");
static_assert(offsetof(Info, nnum) == 48 && offsetof(Info, nnum_cum) == 112, "layout");
static_assert(offsetof(Info, nnum_nempty) == 176 && offsetof(Info, content_flags) == 240, "layout");
static_assert(offsetof(Info, channels) == 244 && offsetof(Info, locations) == 308, "layout");
static_assert(offsetof(Info, bbmin) == 372 && offsetof(Info, extrapolate) == 396, "layout");
static_assert(offsetof(Info, ptr_dis_) == 652, "layout");

// Serialized point cloud header (octree/octree/points_info.h:35-39).
struct PointsInfo {
  char magic[16];
  int pt_num, content_flags;
  int channels[8], ptr_dis[8];
};
static_assert(sizeof(PointsInfo) == OCNN_POINTS_INFO_BYTES, "PointsInfo wire size");

inline const Info* as_info(const void* p) { return reinterpret_cast<const Info*>(p); }

// ---------------------------------------------------------------------------
// Errors: message kept per thread, codes returned to the caller.
int fail(int code, const char* fmt, ...);

#define OCNN_REQUIRE(cond, code, ...) \
  do { if (!(cond)) return ::ocnn::fail((code), __VA_ARGS__); } while (0)

#define OCNN_HIP_OK(expr)                                                        \
  do {                                                                           \
    hipError_t e__ = (expr);                                                     \
    if (e__ != hipSuccess)                                                       \
      return ::ocnn::fail(OCNN_E_HIP, "%s: %s", #expr, hipGetErrorString(e__)); \
  } while (0)

#define OCNN_LAUNCH_OK(name)                                                      \
  do {                                                                            \
    hipError_t e__ = hipGetLastError();                                           \
    if (e__ != hipSuccess)                                                        \
      return ::ocnn::fail(OCNN_E_HIP, "launch %s: %s", name, hipGetErrorString(e__)); \
  } while (0)

// resolves, for the current device, the address of the scratch array behind
// ocnn_octree_conv_static (conv.hip); cheap after the first call on a device
int prepare_builtin_scratch();

inline hipStream_t as_stream(ocnn_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// `n` (at most kFetchWords) 32-bit words of device memory that work queued on `s` produces, to
// host memory: a one-wavefront launch writes them into pinned memory and a sequence number
// behind them, and the call polls that number (the answer is a few microseconds behind the
// producing kernel; a copy into pageable memory plus a wait for the stream takes three to four
// times as long).  After 20 ms of polling the stream is asked, which also reports a failed launch.
constexpr int kFetchWords = 64;
int fetch_words(void* host_out, const void* dev_words, int n, hipStream_t s);

constexpr int kBlock = 256;
inline unsigned blocks_for(int64_t n, int per_block = kBlock) {
  int64_t b = (n + per_block - 1) / per_block;
  return (unsigned)(b < 1 ? 1 : b);
}

// ---------------------------------------------------------------------------
// Neighbour index tables (same content as the reference's NeighHelper,
// octree/octree/octree_nn.cpp:6-81), derived here from their closed forms.
//
// A sibling group (8 children of one parent) owns a 4x4x4 block of neighbour
// slots, slot = x<<4 | y<<2 | z, holding the node at offset (x-1, y-1, z-1) from
// sibling 0.  Tap (dx,dy,dz) in 0..2 of sibling (i,j,k) in 0..1 reads slot
// (dx+i, dy+j, dz+k): the two contributions add without carries.
struct KernelTaps {
  int count;        // K
  int tap[27];      // index into the 3x3x3 stencil, dx*9 + dy*3 + dz
};
// fills taps for a kernel_size triple; false if the shape is not one of the
// nine the reference supports (octree_nn.cpp:7-19)
bool kernel_taps(const int* kernel_size, KernelTaps* out);

__host__ __device__ inline int tap_slot(int tap) {       // slot of a tap for sibling 0
  return ((tap / 9) << 4) | (((tap / 3) % 3) << 2) | (tap % 3);
}
__host__ __device__ inline int sibling_slot(int sib) {   // slot offset of sibling (i,j,k)
  return ((sib >> 2) << 4) | (((sib >> 1) & 1) << 2) | (sib & 1);
}

// element types of feature buffers
template <int DT> struct Elem;
template <> struct Elem<OCNN_F32> { using type = float; };
template <> struct Elem<OCNN_BF16> { using type = uint16_t; };  // raw bf16 bits

__device__ inline float bf16_to_f32(uint16_t v) { return __uint_as_float(((uint32_t)v) << 16); }
__device__ inline uint16_t f32_to_bf16(float f) {  // round to nearest even
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);  // quiet NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

}  // namespace ocnn
