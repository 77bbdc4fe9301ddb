// Host-side pieces: error reporting, the OctreeInfo header arithmetic and the
// kernel-shape tables.  Layout rules follow octree/octree/octree_info.cpp:143-268.
#include "ocnn_common.h"

#include <atomic>
#include <chrono>
#include <cstdint>
#include <mutex>
#include <vector>

#include <stdarg.h>
#include <stdio.h>

namespace ocnn {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// ---- small results back to the host -------------------------------------------------------------
namespace {
struct FetchSlot { uint32_t w[kFetchWords]; int seq; int pad[63]; };
std::mutex g_fetch_mutex;
std::vector<FetchSlot*> g_fetch_free;
std::atomic<int> g_fetch_seq{1};

__global__ void fetch_words_kernel(FetchSlot* __restrict__ host, const uint32_t* __restrict__ dev, int n, int seq) {
  const int i = threadIdx.x;
  if (i < n) __hip_atomic_store(&host->w[i], dev[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  __threadfence_system();
  __syncthreads();
  if (i == 0) __hip_atomic_store(&host->seq, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}
}  // namespace

int fetch_words(void* host_out, const void* dev_words, int n, hipStream_t s) {
  OCNN_REQUIRE(host_out && dev_words && n >= 0 && n <= kFetchWords, OCNN_E_BADARG, "fetch of %d words", n);
  FetchSlot* slot = nullptr;
  {
    std::lock_guard<std::mutex> lock(g_fetch_mutex);
    if (!g_fetch_free.empty()) { slot = g_fetch_free.back(); g_fetch_free.pop_back(); }
  }
  if (!slot) {
    void* p = nullptr;
    OCNN_REQUIRE(hipHostMalloc(&p, sizeof(FetchSlot), hipHostMallocCoherent) == hipSuccess, OCNN_E_HIP,
        "no pinned host memory for a result of the device");
    memset(p, 0, sizeof(FetchSlot));
    slot = static_cast<FetchSlot*>(p);
  }
  const int seq = g_fetch_seq.fetch_add(1) & 0x3fffffff;
  fetch_words_kernel<<<1, kFetchWords, 0, s>>>(slot, static_cast<const uint32_t*>(dev_words), n, seq);
  hipError_t err = hipGetLastError();
  bool seen = false;
  if (err == hipSuccess) {
    const auto t0 = std::chrono::steady_clock::now();
    for (int spins = 0;; ++spins) {
      if (__atomic_load_n(&slot->seq, __ATOMIC_ACQUIRE) == seq) { seen = true; break; }
      if ((spins & 1023) == 1023 && std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(20)) break;
    }
    if (!seen) {
      err = hipStreamSynchronize(s);
      seen = err == hipSuccess && __atomic_load_n(&slot->seq, __ATOMIC_ACQUIRE) == seq;
    }
  }
  if (seen) memcpy(host_out, slot->w, sizeof(uint32_t) * (size_t)n);
  {
    std::lock_guard<std::mutex> lock(g_fetch_mutex);
    g_fetch_free.push_back(slot);
  }
  OCNN_REQUIRE(seen, OCNN_E_HIP, "a result of the device did not arrive: %s", hipGetErrorString(err));
  return OCNN_OK;
}

void Info::reset() {
  memset(this, 0, sizeof(Info));
  strcpy(magic, "_OCTREE_2.0_");
}

void Info::set_channel(int ptype, int ch) {
  int i = index_of(ptype);
  if (ch > 0) {
    channels[i] = ch;
    content_flags |= ptype;
  } else {
    channels[i] = 0;
    content_flags &= ~ptype;
  }
}

void Info::set_nnum_cum(int capacity) {
  nnum_cum[0] = 0;
  for (int d = 1; d < depth + 2; ++d) nnum_cum[d] = nnum_cum[d - 1] + nnum[d - 1];
  nnum_cum[depth + 2] = capacity > nnum_cum[depth + 1] ? capacity : nnum_cum[depth + 1];
}

bool Info::set_ptr_dis() {
  int64_t dis = OCNN_HEADER_BYTES;
  ptr_dis_[0] = (int)dis;
  bool fits = true;
  for (int i = 1; i <= 6; ++i) {
    int ptype = 1 << (i - 1);
    int lc = location(ptype);
    int num = lc == -1 ? total_capacity() : nnum[lc];
    dis += (int64_t)size_of(ptype) * num * channels[i - 1];
    if (dis > INT32_MAX || num < 0) fits = false;
    ptr_dis_[i] = fits ? (int)dis : INT32_MAX;
  }
  return fits;
}

float Info::bbox_max_width() const {
  float w = bbmax[0] - bbmin[0];
  for (int i = 1; i < 3; ++i) {
    float d = bbmax[i] - bbmin[i];
    if (d > w) w = d;
  }
  if (w == 0.0f) w = 1.0e-10f;
  return w;
}

bool Info::consistent_with(const Info& o) const {  // octree_info.cpp:118-130
  return strcmp(magic, o.magic) == 0 && memcmp(channels, o.channels, sizeof(channels)) == 0 &&
      memcmp(locations, o.locations, sizeof(locations)) == 0 && batch_size == o.batch_size &&
      depth == o.depth && full_layer == o.full_layer && adp_layer == o.adp_layer &&
      is_adaptive == o.is_adaptive && key2xyz == o.key2xyz && has_node_dis == o.has_node_dis &&
      content_flags == o.content_flags;
}

bool kernel_taps(const int* ks, KernelTaps* out) {
  if (!ks) return false;
  for (int a = 0; a < 3; ++a) if (ks[a] < 1 || ks[a] > 3) return false;
  // Per axis: size 3 -> offsets {0,1,2}; size 1 -> {1}; size 2 -> {1,2}
  // (the "222" kernel is the 8 octants on the positive side, octree_nn.cpp:13).
  // Mixed shapes containing a 2 (other than 222) are not in the reference's table.
  int code = ks[0] * 100 + ks[1] * 10 + ks[2];
  bool has2 = ks[0] == 2 || ks[1] == 2 || ks[2] == 2;
  if (has2 && code != 222) return false;
  int lo[3], hi[3];
  for (int a = 0; a < 3; ++a) {
    lo[a] = ks[a] == 3 ? 0 : 1;
    hi[a] = ks[a] == 1 ? 1 : 2;
  }
  int n = 0;
  for (int x = lo[0]; x <= hi[0]; ++x)
    for (int y = lo[1]; y <= hi[1]; ++y)
      for (int z = lo[2]; z <= hi[2]; ++z) out->tap[n++] = x * 9 + y * 3 + z;
  out->count = n;
  return true;
}

}  // namespace ocnn

using ocnn::Info;
using ocnn::as_info;

extern "C" {

const char* ocnn_last_error(void) { return ocnn::g_err; }
int ocnn_version(void) { return 100; }

int ocnn_device_check(int dev) {
  int n = 0;
  OCNN_HIP_OK(hipGetDeviceCount(&n));
  OCNN_REQUIRE(dev >= 0 && dev < n, OCNN_E_BADARG, "device %d of %d", dev, n);
  hipDeviceProp_t p;
  OCNN_HIP_OK(hipGetDeviceProperties(&p, dev));
  OCNN_REQUIRE(strncmp(p.gcnArchName, "gfx950", 6) == 0, OCNN_E_UNSUPPORTED,
      "device %d is %s, this library holds gfx950 code only", dev, p.gcnArchName);
  // set-up work that must not fall into a caller's first (possibly captured) operator call:
  // the address of the library's own scratch array on this device
  int cur = -1;
  OCNN_HIP_OK(hipGetDevice(&cur));
  if (cur != dev) OCNN_HIP_OK(hipSetDevice(dev));
  int e = ocnn::prepare_builtin_scratch();
  if (cur != dev) OCNN_HIP_OK(hipSetDevice(cur));
  return e;
}

int ocnn_info_check(const void* info) {  // octree_info.cpp:80-116
  OCNN_REQUIRE(info, OCNN_E_BADARG, "null info");
  const Info* o = as_info(info);
  OCNN_REQUIRE(memcmp(o->magic, "_OCTREE_2.0_", 13) == 0, OCNN_E_FORMAT,
      "octree magic is not _OCTREE_2.0_ (64-bit keys)");
  OCNN_REQUIRE(o->batch_size >= 0, OCNN_E_FORMAT, "batch_size %d", o->batch_size);
  OCNN_REQUIRE(o->depth >= 0 && o->depth <= 16, OCNN_E_FORMAT, "depth %d not in [0,16]", o->depth);
  OCNN_REQUIRE(o->full_layer >= 0 && o->full_layer <= (o->depth < 1 ? 1 : o->depth), OCNN_E_FORMAT,
      "full_layer %d not in [0,depth]", o->full_layer);
  for (int i = 0; i < 6; ++i) {
    OCNN_REQUIRE((o->channels[i] == 0) == ((o->content_flags & (1 << i)) == 0), OCNN_E_FORMAT,
        "content_flags inconsistent with channels[%d]", i);
    OCNN_REQUIRE(o->channels[i] == 0 || o->locations[i] == -1 || o->locations[i] == o->depth,
        OCNN_E_FORMAT, "locations[%d] = %d", i, o->locations[i]);
  }
  return OCNN_OK;
}
int ocnn_info_batch_size(const void* info) { return as_info(info)->batch_size; }
int ocnn_info_depth(const void* info) { return as_info(info)->depth; }
int ocnn_info_full_depth(const void* info) { return as_info(info)->full_layer; }
int ocnn_info_is_key2xyz(const void* info) { return as_info(info)->key2xyz; }
int ocnn_info_node_num(const void* info, int d) { return (d < 0 || d > 15) ? -1 : as_info(info)->nnum[d]; }
int ocnn_info_node_num_nempty(const void* info, int d) { return (d < 0 || d > 15) ? -1 : as_info(info)->nnum_nempty[d]; }
int ocnn_info_node_num_cum(const void* info, int d) { return (d < 0 || d > 15) ? -1 : as_info(info)->nnum_cum[d]; }
int ocnn_info_total_nnum(const void* info) { return as_info(info)->total_nnum(); }
int ocnn_info_channel(const void* info, int ptype) { return as_info(info)->channel(ptype); }
int ocnn_info_location(const void* info, int ptype) { return as_info(info)->location(ptype); }
int64_t ocnn_info_ptr_dis(const void* info, int ptype, int d) { return as_info(info)->ptr_dis(ptype, d); }
int64_t ocnn_info_sizeof_octree(const void* info) { return as_info(info)->sizeof_octree(); }

// upgrade_key64, octree/octree/transform_octree.cpp:433-497: a file written by a 32-bit-key build
// ("_OCTREE_1.0_": 4-byte keys) converted to the 64-bit-key layout every operator expects.
// A host-side format conversion done once when a file is loaded; both buffers are host memory.
int ocnn_upgrade_key64(const void* octree32, size_t bytes, void* out, size_t out_capacity, size_t* out_bytes) {
  OCNN_REQUIRE(octree32 && out_bytes, OCNN_E_BADARG, "null pointer");
  OCNN_REQUIRE(bytes >= sizeof(Info), OCNN_E_FORMAT, "blob shorter than its header");
  const Info* in = as_info(octree32);
  OCNN_REQUIRE(memcmp(in->magic, "_OCTREE_1.0_", 13) == 0, OCNN_E_FORMAT, "octree magic is not _OCTREE_1.0_");
  OCNN_REQUIRE(in->depth >= 0 && in->depth <= 16, OCNN_E_FORMAT, "depth %d not in [0,16]", in->depth);
  OCNN_REQUIRE((size_t)in->ptr_dis_[6] <= bytes, OCNN_E_FORMAT, "blob shorter than its header says");
  Info o = *in;
  memcpy(o.magic, "_OCTREE_2.0_", 13);
  OCNN_REQUIRE(o.set_ptr_dis(), OCNN_E_SHAPE, "the upgraded octree exceeds the 2 GiB the format can address");
  *out_bytes = (size_t)o.sizeof_octree();
  if (!out) return OCNN_OK;  // size query
  OCNN_REQUIRE(out_capacity >= *out_bytes, OCNN_E_WORKSPACE, "output %zu < %zu bytes", out_capacity, *out_bytes);
  memset(out, 0, *out_bytes);
  memcpy(out, &o, sizeof(o));
  const char* src = static_cast<const char*>(octree32);
  char* dst = static_cast<char*>(out);
  const int num = o.total_nnum(), depth = o.depth;
  const uint32_t* key_in = reinterpret_cast<const uint32_t*>(src + in->ptr_dis_[0]);
  uint64_t* key_out = reinterpret_cast<uint64_t*>(dst + o.ptr_dis(OCNN_KEY, 0));
  for (int i = 0; i < num; ++i) {
    if (o.key2xyz) {  // four 8-bit fields widen to four 16-bit fields
      uint8_t f8[4];
      uint16_t f16[4];
      memcpy(f8, key_in + i, 4);
      for (int j = 0; j < 4; ++j) f16[j] = f8[j];
      memcpy(key_out + i, f16, 8);
    } else {
      key_out[i] = key_in[i];
    }
  }
  memcpy(dst + o.ptr_dis(OCNN_CHILD, 0), src + in->ptr_dis_[1], sizeof(int) * (size_t)num);
  const int props[3] = {OCNN_FEATURE, OCNN_LABEL, OCNN_SPLIT};
  for (int q = 0; q < 3; ++q) {
    const int p = props[q];
    if (!o.has(p)) continue;
    const int ch = p == OCNN_FEATURE ? o.channel(p) : 1;
    const int d0 = o.location(p) == depth ? depth : 0;
    for (int d = d0; d <= depth; ++d) {
      int64_t dis_in = in->ptr_dis_[Info::index_of(p)];
      if (o.location(p) == -1) dis_in += (int64_t)in->nnum_cum[d] * o.channel(p) * 4;
      memcpy(dst + o.ptr_dis(p, d), src + dis_in, sizeof(float) * (size_t)o.nnum[d] * ch);
    }
  }
  return OCNN_OK;
}

}  // extern "C"
