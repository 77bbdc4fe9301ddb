// ATen side of the octree operators over libocnn_hip.so: the bodies a maintainer of the
// reference's PyTorch extension puts in place of pytorch/cpp/*.cpp and registers under the same
// names (pytorch/cpp/pybind.cpp:3-49).  The signatures are the reference's
// (pytorch/cpp/ocnn.h:11-72); the library sees plain pointers, sizes and the current HIP stream.
//
// binding/Makefile builds this file into the Python module `ocnn_aten` (g++, PyTorch's headers,
// -locnn_hip), and the GPU test suite calls every function of it and compares with the ctypes
// mirror (nn.py), which goes through the same C interface.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <c10/util/intrusive_ptr.h>

#include <dlfcn.h>

#include <cstring>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "ocnn_hip.h"

namespace {

using std::string;
using std::vector;
using torch::Tensor;

// ---- the host copy of an octree's header ----------------------------------------------------------
// The reference reads the 716-byte header back from the device in every operator call
// (octree/octree/octree_parser.cu:4-27), a blocking copy.  Here one copy is kept per blob tensor.
// What identifies a blob: its StorageImpl object (not the device address: the caching allocator
// hands addresses out again), the view's offset and length, and the tensor's version counter (an
// in-place write through torch bumps it).  An entry holds a weak reference to the StorageImpl, so
// that object's own address cannot be reused while the entry exists, and an entry whose storage
// has died is dropped.  Operators of this file that rewrite a header in place call forget().
struct HeaderCopy {
  c10::weak_intrusive_ptr<c10::StorageImpl> storage;
  const void* data;
  int64_t offset, numel;
  uint32_t version;
  unsigned char bytes[OCNN_HEADER_BYTES];
};

struct HeaderCache {
  std::mutex m;
  std::unordered_map<const c10::StorageImpl*, HeaderCopy> map;
  size_t sweep_at = 64;

  static uint32_t version_of(const Tensor& t) { return t.is_inference() ? 0u : (uint32_t)t._version(); }

  void sweep() {   // drop the entries whose storage is gone
    for (auto it = map.begin(); it != map.end();)
      it = it->second.storage.expired() ? map.erase(it) : std::next(it);
    sweep_at = map.size() * 2 + 64;
  }

  // copies the header into `out` (OCNN_HEADER_BYTES)
  void get(const Tensor& octree, unsigned char* out) {
    TORCH_CHECK(octree.scalar_type() == torch::kUInt8 && octree.dim() == 1 && octree.is_contiguous() &&
        octree.numel() >= OCNN_HEADER_BYTES, "an octree is a contiguous 1-D uint8 tensor of at least ",
        OCNN_HEADER_BYTES, " bytes");
    c10::StorageImpl* impl = octree.storage().unsafeGetStorageImpl();
    const uint32_t version = version_of(octree);
    {
      std::lock_guard<std::mutex> lock(m);
      auto it = map.find(impl);
      if (it != map.end()) {
        HeaderCopy& h = it->second;
        if (!h.storage.expired() && h.data == octree.data_ptr() && h.offset == octree.storage_offset() &&
            h.numel == octree.numel() && h.version == version) {
          std::memcpy(out, h.bytes, OCNN_HEADER_BYTES);
          return;
        }
        map.erase(it);
      }
    }
    HeaderCopy h{octree.storage().getWeakStorageImpl(),
                 octree.data_ptr(), octree.storage_offset(), octree.numel(), version, {0}};
    Tensor head = octree.slice(0, 0, OCNN_INFO_BYTES).cpu();   // blocking, once per blob
    std::memcpy(h.bytes, head.data_ptr(), OCNN_INFO_BYTES);
    TORCH_CHECK(ocnn_info_check(h.bytes) == OCNN_OK, ocnn_last_error());
    TORCH_CHECK(ocnn_info_sizeof_octree(h.bytes) <= octree.numel(), "octree tensor shorter than its header says");
    std::memcpy(out, h.bytes, OCNN_HEADER_BYTES);
    std::lock_guard<std::mutex> lock(m);
    if (map.size() >= sweep_at) sweep();
    map.erase(impl);
    map.emplace(impl, std::move(h));
  }

  // a header that this file has just written or computed on the host: no device read
  void put(const Tensor& octree, const unsigned char* bytes) {
    c10::StorageImpl* impl = octree.storage().unsafeGetStorageImpl();
    HeaderCopy h{octree.storage().getWeakStorageImpl(),
                 octree.data_ptr(), octree.storage_offset(), octree.numel(), version_of(octree), {0}};
    std::memcpy(h.bytes, bytes, OCNN_INFO_BYTES);
    std::lock_guard<std::mutex> lock(m);
    if (map.size() >= sweep_at) sweep();
    map.erase(impl);
    map.emplace(impl, std::move(h));
  }

  void forget(const Tensor& octree) {
    std::lock_guard<std::mutex> lock(m);
    map.erase(octree.storage().unsafeGetStorageImpl());
  }

  int64_t live() {
    std::lock_guard<std::mutex> lock(m);
    sweep();
    return (int64_t)map.size();
  }
};

HeaderCache& headers() {
  static HeaderCache c;
  return c;
}

struct Info {   // the header of one call, on the stack of the operator
  unsigned char bytes[OCNN_HEADER_BYTES];
  explicit Info(const Tensor& octree) { headers().get(octree, bytes); }
  const void* p() const { return bytes; }
  int nnum(int d) const { return ocnn_info_node_num(bytes, d); }
  int nnum_nempty(int d) const { return ocnn_info_node_num_nempty(bytes, d); }
  int depth() const { return ocnn_info_depth(bytes); }
  // device pointer of a property at a depth
  template <typename T>
  const T* prop(const Tensor& octree, int ptype, int d) const {
    int64_t off = ocnn_info_ptr_dis(bytes, ptype, d);
    TORCH_CHECK(off >= 0, "the octree has no property ", ptype, " at depth ", d);
    return reinterpret_cast<const T*>(static_cast<const unsigned char*>(octree.data_ptr()) + off);
  }
};

int dtype_of(const Tensor& t) {
  TORCH_CHECK(t.scalar_type() == torch::kFloat32 || t.scalar_type() == torch::kBFloat16,
      "octree operators: fp32 or bf16 features");
  return t.scalar_type() == torch::kBFloat16 ? OCNN_BF16 : OCNN_F32;
}

ocnn_stream_t current_stream() {
  return reinterpret_cast<ocnn_stream_t>(c10::hip::getCurrentHIPStream().stream());
}

void check(int rc) { TORCH_CHECK(rc == OCNN_OK, ocnn_last_error()); }

vector<int> three(vector<int> ks) {   // resize_with_last_val, pytorch/cpp/octree2col.cpp:26
  TORCH_CHECK(!ks.empty() && ks.size() <= 3, "kernel_size holds one to three numbers");
  while (ks.size() < 3) ks.push_back(ks.back());
  return ks;
}

Tensor bytes_on(const Tensor& like, size_t n) {
  return torch::empty({(int64_t)n + 16}, like.options().dtype(torch::kUInt8));
}

Tensor conv_forward(Tensor data_in, Tensor weights, Tensor octree, int depth, int num_output,
    vector<int> kernel_size, int stride, bool nempty, bool deconv, const Tensor* bias, bool relu) {
  kernel_size = three(kernel_size);
  data_in = data_in.contiguous();
  weights = weights.contiguous();
  TORCH_CHECK(weights.scalar_type() == data_in.scalar_type(), "weights and data must have the same dtype");
  Info info(octree);
  const int dt = dtype_of(data_in);
  int top_h = 0, btm_h = 0;
  size_t ws_bytes = 0;
  check(ocnn_conv_shape(info.p(), depth, (int)data_in.size(1), num_output, kernel_size.data(), stride,
      nempty ? 1 : 0, deconv ? 1 : 0, dt, &top_h, &btm_h, &ws_bytes));
  TORCH_CHECK(data_in.size(2) == btm_h, "input height ", data_in.size(2), ", the octree has ", btm_h);
  Tensor ws = bytes_on(octree, ws_bytes);
  Tensor out = torch::empty({1, num_output, top_h, 1}, data_in.options());
  Tensor b;
  if (bias) b = bias->to(torch::kFloat32).contiguous();
  check(ocnn_octree_conv_fused(out.data_ptr(), data_in.data_ptr(), (int)data_in.size(1), (int)data_in.size(2),
      weights.data_ptr(), bias ? b.data_ptr<float>() : nullptr, relu ? 1 : 0, deconv ? 1 : 0,
      octree.data_ptr(), info.p(), depth, num_output, kernel_size.data(), stride, nempty ? 1 : 0, dt,
      ws.data_ptr(), ws_bytes, current_stream()));
  return out;
}

vector<Tensor> conv_backward(Tensor data_in, Tensor weights, Tensor octree, Tensor grad_in, int depth,
    int num_output, vector<int> kernel_size, int stride, bool nempty, bool deconv) {
  kernel_size = three(kernel_size);
  data_in = data_in.contiguous();
  weights = weights.contiguous();
  grad_in = grad_in.contiguous();
  Info info(octree);
  size_t ws_bytes = 0;
  check(ocnn_conv_grad_workspace_bytes(info.p(), depth, (int)data_in.size(1), num_output, kernel_size.data(),
      stride, nempty ? 1 : 0, deconv ? 1 : 0, OCNN_F32, &ws_bytes));
  Tensor ws = bytes_on(octree, ws_bytes);
  // both results are written completely: no torch::zeros
  Tensor btm_out = torch::empty_like(data_in), weights_out = torch::empty_like(weights);
  auto fn = deconv ? ocnn_octree_deconv_grad : ocnn_octree_conv_grad;
  check(fn(btm_out.data_ptr(), weights_out.data_ptr(), data_in.data_ptr(), (int)data_in.size(1),
      (int)data_in.size(2), weights.data_ptr(), grad_in.data_ptr(), octree.data_ptr(), info.p(), depth,
      num_output, kernel_size.data(), stride, nempty ? 1 : 0, OCNN_F32, ws.data_ptr(), ws_bytes,
      current_stream()));
  return {btm_out, weights_out};
}

// inverted child links of a depth: ichild[child[h]] = h (pytorch/cpp/octree2col.cpp:10-20)
Tensor make_ichild(const Tensor& octree, const Info& info, int depth) {
  const int n = info.nnum(depth), ne = info.nnum_nempty(depth);
  Tensor ichild = torch::zeros({std::max(ne, 1)}, octree.options().dtype(torch::kInt32));
  check(ocnn_make_ichild(ichild.data_ptr<int>(), ne, info.prop<int>(octree, OCNN_CHILD, depth), n, current_stream()));
  return ichild;
}

}  // namespace

// ---- pytorch/cpp/octree_conv.cpp:131-283 (signatures pytorch/cpp/ocnn.h:31-46) -----------------------
Tensor octree_conv(Tensor data_in, Tensor weights, Tensor octree, int depth, int num_output,
    vector<int> kernel_size, int stride, bool nempty) {
  return conv_forward(data_in, weights, octree, depth, num_output, kernel_size, stride, nempty, false, nullptr, false);
}
Tensor octree_deconv(Tensor data_in, Tensor weights, Tensor octree, int depth, int num_output,
    vector<int> kernel_size, int stride, bool nempty) {
  return conv_forward(data_in, weights, octree, depth, num_output, kernel_size, stride, nempty, true, nullptr, false);
}
vector<Tensor> octree_conv_grad(Tensor data_in, Tensor weights, Tensor octree, Tensor grad_in, int depth,
    int num_output, vector<int> kernel_size, int stride, bool nempty) {
  return conv_backward(data_in, weights, octree, grad_in, depth, num_output, kernel_size, stride, nempty, false);
}
vector<Tensor> octree_deconv_grad(Tensor data_in, Tensor weights, Tensor octree, Tensor grad_in, int depth,
    int num_output, vector<int> kernel_size, int stride, bool nempty) {
  return conv_backward(data_in, weights, octree, grad_in, depth, num_output, kernel_size, stride, nempty, true);
}
// conv -> BatchNorm -> ReLU of pytorch/ocnn/modules.py:23-36 with the BatchNorm folded into
// `weights` and `bias` (no counterpart in the reference's extension)
Tensor octree_conv_bn_relu(Tensor data_in, Tensor weights, Tensor bias, Tensor octree, int depth, int num_output,
    vector<int> kernel_size, int stride, bool nempty, bool deconv, bool relu) {
  return conv_forward(data_in, weights, octree, depth, num_output, kernel_size, stride, nempty, deconv, &bias, relu);
}

// ---- pytorch/cpp/octree2col.cpp:47-237 -------------------------------------------------------------------
Tensor octree2col(Tensor data_in, Tensor octree, int depth, vector<int> kernel_size, int stride, bool nempty) {
  kernel_size = three(kernel_size);
  TORCH_CHECK(depth > 0, "Depth should be larger than 0");
  TORCH_CHECK(stride == 1 || stride == 2, "Unsupport stride");
  data_in = data_in.contiguous();
  Info info(octree);
  const int dt = dtype_of(data_in);
  const int channel = (int)data_in.size(1), btm_h = (int)data_in.size(2);
  const int K = kernel_size[0] * kernel_size[1] * kernel_size[2];
  const int* neigh = info.prop<int>(octree, OCNN_NEIGH, depth);
  if (!nempty) {
    TORCH_CHECK(btm_h == info.nnum(depth), "octree2col: height ", btm_h, " != node_num = ", info.nnum(depth));
    int top_h = btm_h;
    if (stride == 2) {
      top_h = btm_h / 8;
      TORCH_CHECK(top_h == info.nnum_nempty(depth - 1), "octree2col: stride-2 height mismatch");
    }
    Tensor out = torch::empty({channel, K, top_h}, data_in.options());   // every element is written
    check(ocnn_octree2col(out.data_ptr(), data_in.data_ptr(), channel, top_h, kernel_size.data(), stride, neigh,
        std::max(top_h, 1), 0, dt, current_stream()));
    return out;
  }
  TORCH_CHECK(btm_h == info.nnum_nempty(depth), "octree2col: height ", btm_h, " != node_num_nempty");
  Tensor ichild = make_ichild(octree, info, depth);
  const int top_h = stride == 1 ? btm_h : info.nnum_nempty(depth - 1);
  Tensor out = torch::empty({channel, K, top_h}, data_in.options());
  check(ocnn_octree2colP(out.data_ptr(), data_in.data_ptr(), channel, top_h, btm_h, kernel_size.data(), stride, neigh,
      info.prop<int>(octree, OCNN_CHILD, depth), ichild.data_ptr<int>(), std::max(top_h, 1), 0, dt, current_stream()));
  return out;
}

Tensor col2octree(Tensor grad_in, Tensor octree, int depth, vector<int> kernel_size, int stride, bool nempty) {
  kernel_size = three(kernel_size);
  TORCH_CHECK(depth > 0, "Depth should be larger than 0");
  TORCH_CHECK(stride == 1 || stride == 2, "Unsupport stride");
  grad_in = grad_in.contiguous();
  Info info(octree);
  const int dt = dtype_of(grad_in);
  const int channel = (int)grad_in.size(0), top_h = (int)grad_in.size(2);
  const int* neigh = info.prop<int>(octree, OCNN_NEIGH, depth);
  if (stride == 2) TORCH_CHECK(top_h == info.nnum_nempty(depth - 1), "col2octree: stride-2 height mismatch");
  if (!nempty) {
    const int btm_h = info.nnum(depth);
    Tensor out = torch::empty({1, channel, btm_h, 1}, grad_in.options());   // chunk 0 sets every row
    check(ocnn_col2octree(grad_in.data_ptr(), out.data_ptr(), channel, top_h, kernel_size.data(), stride, neigh,
        std::max(top_h, 1), 0, dt, current_stream()));
    return out;
  }
  const int btm_h = info.nnum_nempty(depth);
  if (stride == 1) TORCH_CHECK(top_h == btm_h, "col2octree: height mismatch");
  Tensor ichild = make_ichild(octree, info, depth);
  Tensor out = torch::empty({1, channel, btm_h, 1}, grad_in.options());
  check(ocnn_col2octreeP(grad_in.data_ptr(), out.data_ptr(), channel, top_h, btm_h, kernel_size.data(), stride, neigh,
      info.prop<int>(octree, OCNN_CHILD, depth), ichild.data_ptr<int>(), std::max(top_h, 1), 0, dt, current_stream()));
  return out;
}

// ---- pytorch/cpp/octree_pad.cpp:6-60 ----------------------------------------------------------------------
Tensor octree_pad(Tensor data_in, Tensor octree, int depth, float val) {
  TORCH_CHECK(depth >= 1, "Depth should be larger than 1");
  data_in = data_in.contiguous();
  Info info(octree);
  const int channel = (int)data_in.size(1), btm_h = (int)data_in.size(2), top_h = info.nnum(depth);
  TORCH_CHECK(btm_h == info.nnum_nempty(depth), "pad, d = ", depth, ", channel = ", channel, ": height ", btm_h,
      " != ", info.nnum_nempty(depth));
  Tensor out = torch::empty({1, channel, top_h, 1}, data_in.options());
  check(ocnn_pad_forward(out.data_ptr(), top_h, channel, data_in.data_ptr(), btm_h,
      info.prop<int>(octree, OCNN_CHILD, depth), val, dtype_of(data_in), current_stream()));
  return out;
}

Tensor octree_depad(Tensor data_in, Tensor octree, int depth) {
  TORCH_CHECK(depth >= 1, "Depth should be larger than 1");
  data_in = data_in.contiguous();
  Info info(octree);
  const int channel = (int)data_in.size(1), top_h = (int)data_in.size(2), btm_h = info.nnum_nempty(depth);
  TORCH_CHECK(top_h == info.nnum(depth), "depad, d = ", depth, ", channel = ", channel, ": height ", top_h,
      " != ", info.nnum(depth));
  Tensor out = torch::zeros({1, channel, btm_h, 1}, data_in.options());
  check(ocnn_pad_backward(out.data_ptr(), btm_h, channel, data_in.data_ptr(), top_h,
      info.prop<int>(octree, OCNN_CHILD, depth), dtype_of(data_in), current_stream()));
  return out;
}

// ---- pytorch/cpp/octree_pool.cpp:6-90 ---------------------------------------------------------------------
vector<Tensor> octree_max_pool(Tensor data_in, Tensor octree, int depth) {
  data_in = data_in.contiguous();
  Info info(octree);
  const int channel = (int)data_in.size(1), btm_h = (int)data_in.size(2);
  TORCH_CHECK(info.nnum(depth) == btm_h, "max_pool: height ", btm_h, " != node_num = ", info.nnum(depth));
  TORCH_CHECK(depth > 1, "Depth should be larger than 1");
  const int top_h = btm_h >> 3;
  Tensor top = torch::empty({1, channel, top_h, 1}, data_in.options());
  Tensor mask = torch::empty({1, channel, top_h, 1}, data_in.options().dtype(torch::kInt32));
  check(ocnn_octree_max_pool(top.data_ptr(), top_h, mask.data_ptr<int>(), data_in.data_ptr(), btm_h, channel,
      dtype_of(data_in), current_stream()));
  return {top, mask};
}

Tensor octree_max_unpool(Tensor data_in, Tensor mask, Tensor octree, int depth) {
  data_in = data_in.contiguous();
  mask = mask.contiguous();
  Info info(octree);
  const int channel = (int)data_in.size(1), top_h = (int)data_in.size(2);
  TORCH_CHECK(top_h == info.nnum_nempty(depth - 1), "max_unpool: height ", top_h, " != node_num_nempty");
  TORCH_CHECK(mask.scalar_type() == torch::kInt32 && mask.size(1) == channel && mask.size(2) == top_h,
      "max_unpool: mask shape");
  const int btm_h = top_h << 3;
  Tensor btm = torch::empty({1, channel, btm_h, 1}, data_in.options());   // the kernel writes the zeros
  check(ocnn_octree_max_unpool(data_in.data_ptr(), top_h, mask.data_ptr<int>(), btm.data_ptr(), btm_h, channel,
      dtype_of(data_in), current_stream()));
  return btm;
}

Tensor octree_mask_pool(Tensor data_in, Tensor mask, Tensor octree, int depth) {
  data_in = data_in.contiguous();
  mask = mask.contiguous();
  Info info(octree);
  const int channel = (int)data_in.size(1), btm_h = (int)data_in.size(2), top_h = (int)mask.size(2);
  TORCH_CHECK(info.nnum(depth) == btm_h && top_h == btm_h >> 3, "mask_pool: height mismatch");
  TORCH_CHECK(mask.scalar_type() == torch::kInt32 && mask.size(1) == channel, "mask_pool: mask shape");
  Tensor top = torch::empty({1, channel, top_h, 1}, data_in.options());
  check(ocnn_octree_mask_pool(top.data_ptr(), top_h, mask.data_ptr<int>(), data_in.data_ptr(), btm_h, channel,
      dtype_of(data_in), current_stream()));
  return top;
}

// ---- pytorch/cpp/octree_key.cpp:49-132 ----------------------------------------------------------------------
namespace {
Tensor key_op(Tensor t, int depth, bool to_key) {
  t = t.contiguous();
  TORCH_CHECK(t.numel() >= 1 && t.scalar_type() == torch::kInt64, "int64 keys, at least one");
  Tensor out = torch::empty_like(t);
  auto fn = to_key ? ocnn_xyz2key : ocnn_key2xyz;
  check(fn(reinterpret_cast<uint64_t*>(out.data_ptr<int64_t>()), reinterpret_cast<const uint64_t*>(t.data_ptr<int64_t>()),
      (int)t.numel(), depth, current_stream()));
  return out;
}
}  // namespace
Tensor octree_xyz2key(Tensor xyz, int depth) { return key_op(xyz, depth, true); }
Tensor octree_key2xyz(Tensor key, int depth) { return key_op(key, depth, false); }

Tensor octree_search_key(Tensor key, Tensor octree, int depth, bool key_is_xyz, bool nempty) {
  key = key.contiguous();
  TORCH_CHECK(key.numel() >= 1 && key.scalar_type() == torch::kInt64, "int64 keys, at least one");
  Info info(octree);
  if (key_is_xyz) key = key_op(key, depth, true);
  int des_h = info.nnum(depth);
  Tensor des = torch::from_blob(const_cast<int64_t*>(info.prop<int64_t>(octree, OCNN_KEY, depth)), {des_h},
      octree.options().dtype(torch::kInt64));
  if (nempty) {   // keys of the non-empty nodes, in node order (the reference depads the key array)
    Tensor child = torch::from_blob(const_cast<int*>(info.prop<int>(octree, OCNN_CHILD, depth)), {des_h},
        octree.options().dtype(torch::kInt32));
    des = des.masked_select(child.ge(0));
    des_h = info.nnum_nempty(depth);
  }
  if (ocnn_info_is_key2xyz(info.p()) && des_h > 0) des = key_op(des, depth, true);
  Tensor out = torch::empty({key.numel()}, octree.options().dtype(torch::kInt32));
  // many queries in a large array go through sample tables in a scratch tensor of this call
  Tensor ws = torch::empty({(int64_t)ocnn_search_key_workspace_bytes(des_h) + 128}, octree.options().dtype(torch::kUInt8));
  void* base = reinterpret_cast<void*>((reinterpret_cast<uintptr_t>(ws.data_ptr()) + 127) & ~(uintptr_t)127);
  check(ocnn_search_key_indexed(out.data_ptr<int>(), reinterpret_cast<const uint64_t*>(des.data_ptr<int64_t>()), des_h,
      reinterpret_cast<const uint64_t*>(key.data_ptr<int64_t>()), (int)key.numel(), base,
      ocnn_search_key_workspace_bytes(des_h), current_stream()));
  return out;
}

// ---- pytorch/cpp/octree_grow.cpp:13-190 -----------------------------------------------------------------------
Tensor octree_new(int batch_size, int channel, bool node_dis, int adaptive_layer) {
  unsigned char hdr[OCNN_HEADER_BYTES] = {0};
  check(ocnn_octree_new_info(batch_size, channel, node_dis ? 1 : 0, adaptive_layer, hdr));
  Tensor out = torch::empty({ocnn_info_sizeof_octree(hdr)},
      torch::TensorOptions().dtype(torch::kUInt8).device(torch::kCUDA, c10::hip::current_device()));
  check(ocnn_octree_new(out.data_ptr(), hdr, current_stream()));
  headers().put(out, hdr);
  return out;
}

Tensor octree_grow(Tensor octree_in, int target_depth, bool full_octree) {
  Info in(octree_in);
  unsigned char hdr[OCNN_HEADER_BYTES] = {0};
  check(ocnn_octree_grow_info(in.p(), target_depth, full_octree ? 1 : 0, hdr));
  Tensor out = torch::empty({ocnn_info_sizeof_octree(hdr)}, octree_in.options());
  check(ocnn_octree_grow(out.data_ptr(), hdr, octree_in.data_ptr(), in.p(), target_depth, full_octree ? 1 : 0,
      current_stream()));
  headers().put(out, hdr);
  return out;
}

// children[depth] from the split labels, on a copy of the blob (octree_grow.cpp:164-190)
Tensor octree_update(Tensor octree_in, Tensor label_in, int depth, int split) {
  Info in(octree_in);
  Tensor out = torch::empty_like(octree_in);   // the library copies the blob while it waits for the count
  unsigned char hdr[OCNN_HEADER_BYTES];
  std::memcpy(hdr, in.bytes, OCNN_HEADER_BYTES);
  Tensor label = label_in.contiguous().to(torch::kInt32);
  const int n = (int)label.numel();
  const size_t sb = ocnn_octree_update_scratch_bytes(n);
  Tensor ws = bytes_on(octree_in, sb);
  check(ocnn_octree_update_copy(out.data_ptr(), octree_in.data_ptr(), hdr, label.data_ptr<int>(), n, depth, split,
      ws.data_ptr(), sb, current_stream()));
  headers().put(out, hdr);
  return out;
}

// The same on the blob itself (no counterpart in the reference, which always clones): the header
// changes under the tensor's feet, so the cached copy is replaced by the patched one.
void octree_update_(Tensor octree, Tensor label_in, int depth, int split) {
  Info in(octree);
  unsigned char hdr[OCNN_HEADER_BYTES];
  std::memcpy(hdr, in.bytes, OCNN_HEADER_BYTES);
  Tensor label = label_in.contiguous().to(torch::kInt32);
  const int n = (int)label.numel();
  const size_t sb = ocnn_octree_update_scratch_bytes(n);
  Tensor ws = bytes_on(octree, sb);
  headers().forget(octree);
  check(ocnn_octree_update(octree.data_ptr(), hdr, label.data_ptr<int>(), n, depth, split, ws.data_ptr(), sb,
      current_stream()));
  headers().put(octree, hdr);
}

// ---- pytorch/cpp/octree_property.cpp:11-344, the entries the modules of pytorch/ocnn use ----------------------
Tensor octree_property(Tensor octree, string name, int depth) {
  Info info(octree);
  const int nnum = depth > 0 ? info.nnum(depth) : ocnn_info_total_nnum(info.p());
  auto ints = [&](vector<int> v) {
    return torch::tensor(v, torch::TensorOptions().dtype(torch::kInt32)).to(octree.device());
  };
  auto view = [&](int ptype, torch::ScalarType st, int64_t count) {
    int64_t off = ocnn_info_ptr_dis(info.p(), ptype, depth);
    TORCH_CHECK(off >= 0, "The octree has no ", name, ": d = ", depth);
    return torch::from_blob(static_cast<unsigned char*>(octree.data_ptr()) + off, {count}, octree.options().dtype(st)).clone();
  };
  if (name == "key" || name == "xyz") {
    const int ch = ocnn_info_channel(info.p(), OCNN_KEY);
    Tensor src = view(OCNN_KEY, torch::kInt64, (int64_t)ch * nnum);
    const bool is_xyz = ocnn_info_is_key2xyz(info.p()) != 0;
    if ((name == "key") != is_xyz) return src;
    TORCH_CHECK(depth > 0, "key conversion needs a depth");
    return key_op(src, depth, name == "key");
  }
  if (name == "child") return view(OCNN_CHILD, torch::kInt32, (int64_t)nnum * ocnn_info_channel(info.p(), OCNN_CHILD));
  if (name == "neigh") {
    const int ch = ocnn_info_channel(info.p(), OCNN_NEIGH);
    return view(OCNN_NEIGH, torch::kInt32, (int64_t)nnum * ch).view({nnum, ch});
  }
  if (name == "feature") {
    const int ch = ocnn_info_channel(info.p(), OCNN_FEATURE);
    return view(OCNN_FEATURE, torch::kFloat32, (int64_t)nnum * ch).view({1, ch, nnum, 1});
  }
  if (name == "label") return view(OCNN_LABEL, torch::kFloat32, (int64_t)nnum * ocnn_info_channel(info.p(), OCNN_LABEL));
  if (name == "split") return view(OCNN_SPLIT, torch::kFloat32, (int64_t)nnum * ocnn_info_channel(info.p(), OCNN_SPLIT));
  vector<int> v;
  const int D = info.depth();
  if (name == "node_num") {
    if (depth > 0) v = {info.nnum(depth)}; else for (int d = 0; d <= D; ++d) v.push_back(info.nnum(d));
  } else if (name == "node_num_ne" || name == "node_num_nempty") {
    if (depth > 0) v = {info.nnum_nempty(depth)}; else for (int d = 0; d <= D; ++d) v.push_back(info.nnum_nempty(d));
  } else if (name == "node_num_cum") {
    if (depth > 0) v = {ocnn_info_node_num_cum(info.p(), depth)};
    else for (int d = 0; d <= D + 1; ++d) v.push_back(ocnn_info_node_num_cum(info.p(), d));
  } else if (name == "batch_size") v = {ocnn_info_batch_size(info.p())};
  else if (name == "depth") v = {D};
  else if (name == "full_depth") v = {ocnn_info_full_depth(info.p())};
  else TORCH_CHECK(false, "Unsupport octree property: ", name);
  return ints(v);
}

// ---- row-major bf16 activations (no counterpart in the reference): rows [H + 1, pitch] ----------------
Tensor rows_from_channels(Tensor data) {
  data = data.contiguous();
  const int c = (int)data.size(1), h = (int)data.size(2), pitch = (c + 15) / 16 * 16;
  Tensor rows = torch::empty({h + 1, pitch}, data.options());
  check(ocnn_rows_from_channels(rows.data_ptr(), pitch, data.data_ptr(), c, h, dtype_of(data), current_stream()));
  return rows;
}

Tensor channels_from_rows(Tensor rows, int channels) {
  rows = rows.contiguous();
  const int h = (int)rows.size(0) - 1;
  Tensor data = torch::empty({1, channels, h, 1}, rows.options());
  check(ocnn_channels_from_rows(data.data_ptr(), rows.data_ptr(), (int)rows.size(1), channels, h, dtype_of(rows),
      current_stream()));
  return data;
}

// conv / deconv + bias + ReLU on row-major tensors; rows_in [H + 1, pitch(channel_in)] -> [top_h + 1, pitch(num_output)]
Tensor octree_conv_rows(Tensor rows_in, int channel_in, Tensor weights, Tensor bias, bool relu, Tensor octree,
    int depth, int num_output, vector<int> kernel_size, int stride, bool nempty, bool deconv) {
  kernel_size = three(kernel_size);
  TORCH_CHECK(rows_in.dim() == 2 && rows_in.stride(1) == 1, "rows_in is [H + 1, pitch] with unit channel stride");
  weights = weights.contiguous();
  Info info(octree);
  const int dt = dtype_of(rows_in);
  int top_h = 0, btm_h = 0;
  size_t ws_bytes = 0;
  check(ocnn_conv_rows_shape(info.p(), depth, channel_in, num_output, kernel_size.data(), stride, nempty ? 1 : 0,
      deconv ? 1 : 0, dt, &top_h, &btm_h, &ws_bytes));
  Tensor ws = bytes_on(octree, ws_bytes);
  Tensor out = torch::empty({top_h + 1, (num_output + 15) / 16 * 16}, rows_in.options());
  Tensor b;
  if (bias.defined() && bias.numel() > 0) b = bias.to(torch::kFloat32).contiguous();
  check(ocnn_octree_conv_rows(out.data_ptr(), (int)out.stride(0), rows_in.data_ptr(), (int)rows_in.stride(0), channel_in,
      (int)rows_in.size(0) - 1, weights.data_ptr(), b.defined() ? b.data_ptr<float>() : nullptr, relu ? 1 : 0,
      deconv ? 1 : 0, octree.data_ptr(), info.p(), depth, num_output, kernel_size.data(), stride, nempty ? 1 : 0, dt,
      ws.data_ptr(), ws_bytes, current_stream()));
  return out;
}

// ---- serialized point clouds (octree/octree/points_info.h:35-39: 88-byte header, then the xyz, normal,
// feature and label arrays, point-major) -------------------------------------------------------------------------
namespace {
struct PointsHeader {   // host copy of a cloud's header: a blocking read when the cloud lives on the device
  unsigned char bytes[OCNN_POINTS_INFO_BYTES];
  explicit PointsHeader(const Tensor& points) {
    TORCH_CHECK(points.scalar_type() == torch::kUInt8 && points.dim() == 1 && points.is_contiguous() &&
        points.numel() >= OCNN_POINTS_INFO_BYTES, "a point cloud is a contiguous 1-D uint8 tensor of at least ",
        OCNN_POINTS_INFO_BYTES, " bytes");
    Tensor head = points.slice(0, 0, OCNN_POINTS_INFO_BYTES).cpu();
    std::memcpy(bytes, head.data_ptr(), OCNN_POINTS_INFO_BYTES);
    TORCH_CHECK(std::memcmp(bytes, "_POINTS_1.0_", 12) == 0, "The version of points format is not _POINTS_1.0_");
    TORCH_CHECK(pt_num() > 0 && offset(4) <= points.numel(), "point cloud tensor shorter than its header says");
  }
  int word(int i) const { int v; std::memcpy(&v, bytes + 16 + 4 * i, 4); return v; }
  int pt_num() const { return word(0); }
  bool has(int t) const { return (word(1) >> t & 1) && word(2 + t) > 0; }
  int channel(int t) const { return word(2 + t); }
  int64_t offset(int t) const { return word(10 + t); }   // t = 4: the size of the cloud
};

Tensor on_device(const Tensor& t) {
  return t.is_cuda() ? t.contiguous() : t.contiguous().to(torch::Device(torch::kCUDA, c10::hip::current_device()));
}

int points_ptype(const string& property) {   // get_ptype, pytorch/cpp/points_property.cpp:9-24
  if (property == "xyz" || property == "xyzi") return 0;
  if (property == "normal") return 1;
  if (property == "feature") return 2;
  if (property == "label") return 3;
  TORCH_CHECK(false, "Unsupported Property: ", property);
}

// [pt_num, channel] float view of a property inside the cloud, undefined when the cloud has none
Tensor points_array(const Tensor& points, const PointsHeader& h, int t) {
  if (!h.has(t)) return Tensor();
  return torch::from_blob(static_cast<unsigned char*>(points.data_ptr()) + h.offset(t), {h.pt_num(), h.channel(t)},
      points.options().dtype(torch::kFloat32));
}

const float* three_floats(vector<float>& v, const char* what) {   // resize_with_last_val on floats
  TORCH_CHECK(!v.empty() && v.size() <= 3, what, " holds one to three numbers");
  while (v.size() < 3) v.push_back(v.back());
  return v.data();
}

struct Aligned {   // scratch bytes of one call, 256-byte aligned
  Tensor t;
  void* p;
  Aligned(const Tensor& like, size_t n) : t(torch::empty({(int64_t)n + 256}, like.options().dtype(torch::kUInt8))) {
    p = reinterpret_cast<void*>((reinterpret_cast<uintptr_t>(t.data_ptr()) + 255) & ~(uintptr_t)255);
  }
};

// the allocator the library calls back for scratch blocks and the result of a build or a scan
struct TensorPool {
  torch::TensorOptions options;
  vector<Tensor> blocks;
  static void* alloc(size_t bytes, void* ctx) {
    TensorPool* self = static_cast<TensorPool*>(ctx);
    self->blocks.push_back(torch::empty({(int64_t)std::max<size_t>(bytes, 1)}, self->options));
    return self->blocks.back().data_ptr();
  }
  Tensor take(void* p) const {   // (scratch blocks come first: the last match is the result)
    for (auto it = blocks.rbegin(); it != blocks.rend(); ++it)
      if (it->data_ptr() == p) return *it;
    TORCH_CHECK(false, "the library returned memory that its allocator did not hand out");
  }
};
}  // namespace

// ---- pytorch/cpp/points_property.cpp:38-165 ------------------------------------------------------------------
Tensor points_new(Tensor pts, Tensor normals, Tensor features, Tensor labels) {
  TORCH_CHECK(pts.defined() && pts.numel() > 0 && pts.numel() % 3 == 0, "Error occurs when setting points");
  pts = pts.reshape({-1, 3}).to(torch::kFloat32).contiguous();
  const int64_t n = pts.size(0);
  vector<Tensor> parts;
  int chans[4] = {3, 0, 0, 0}, flags = 1;
  const Tensor* rest[3] = {&normals, &features, &labels};
  parts.push_back(Tensor());   // the header's place
  parts.push_back(pts.reshape({-1}).view(torch::kUInt8));
  for (int i = 1; i < 4; ++i) {
    const Tensor& a = *rest[i - 1];
    if (!a.defined() || a.numel() == 0) continue;
    TORCH_CHECK(a.numel() % n == 0, "Error occurs when setting points");
    Tensor b = a.reshape({n, -1}).to(torch::kFloat32).to(pts.device()).contiguous();
    TORCH_CHECK((i != 1 || b.size(1) == 3) && (i != 3 || b.size(1) == 1), "normals need 3 channels and labels 1");
    chans[i] = (int)b.size(1);
    flags |= 1 << i;
    parts.push_back(b.reshape({-1}).view(torch::kUInt8));
  }
  Tensor hdr = torch::zeros({OCNN_POINTS_INFO_BYTES}, torch::TensorOptions().dtype(torch::kUInt8));
  unsigned char* h = hdr.data_ptr<uint8_t>();
  std::memcpy(h, "_POINTS_1.0_", 12);
  int words[18] = {0};
  words[0] = (int)n;
  words[1] = flags;
  int64_t dis = OCNN_POINTS_INFO_BYTES;
  for (int t = 0; t < 4; ++t) {
    words[2 + t] = chans[t];
    words[10 + t] = (int)dis;
    dis += 4 * n * chans[t];
  }
  words[14] = (int)dis;
  std::memcpy(h + 16, words, sizeof(words));
  parts[0] = hdr.to(pts.device());
  return torch::cat(parts);
}

Tensor points_property(Tensor points, string property) {
  points = points.contiguous();
  PointsHeader h(points);
  Tensor a = points_array(points, h, points_ptype(property));
  return a.defined() ? a.clone() : a;
}

Tensor points_batch_property(vector<Tensor> tensors_in, string property) {
  const int t = points_ptype(property);
  vector<Tensor> parts;
  int channel = -1;
  for (size_t i = 0; i < tensors_in.size(); ++i) {
    Tensor p = tensors_in[i].contiguous();
    PointsHeader h(p);
    Tensor a = points_array(p, h, t);
    TORCH_CHECK(a.defined(), "The specified property does not exist.");
    if (channel < 0) channel = h.channel(t);
    TORCH_CHECK(h.channel(t) == channel, "The specified channel_out is wrong.");
    if (property == "xyzi") a = torch::cat({a, torch::full({h.pt_num(), 1}, (float)i, a.options())}, 1);
    parts.push_back(a);
  }
  return torch::cat(parts, 0);
}

Tensor points_set_property(Tensor points, Tensor data, string property) {
  TORCH_CHECK(data.dim() == 2, "data is [pt_num, channel]");
  points = points.contiguous();
  PointsHeader h(points);
  const int t = points_ptype(property);
  TORCH_CHECK(h.has(t), "The property does not exist.");
  TORCH_CHECK(data.size(1) == h.channel(t), "The channel is wrong.");
  TORCH_CHECK(data.size(0) == h.pt_num(), "The point number is wrong.");
  Tensor out = points.clone();
  points_array(out, h, t).copy_(data.to(torch::kFloat32));
  return out;
}

// ---- pytorch/cpp/transform_points.cpp:7-125, on the device ------------------------------------------------------
vector<float> bounding_sphere(Tensor data_in, string method) {
  Tensor points = on_device(data_in);
  PointsHeader h(data_in.is_cuda() ? points : data_in.contiguous());
  const size_t wb = ocnn_points_workspace_bytes(h.pt_num());
  Aligned ws(points, wb);
  vector<float> out(4);
  check(ocnn_bounding_sphere(points.data_ptr(), h.bytes, method == "sphere" ? 0 : 1, out.data(), ws.p, wb,
      current_stream()));
  return out;
}

Tensor normalize_points(Tensor data_in, float radius, vector<float> center) {
  Tensor points = on_device(data_in);
  PointsHeader h(data_in.is_cuda() ? points : data_in.contiguous());
  Tensor out = torch::empty_like(points);
  check(ocnn_normalize_points(out.data_ptr(), points.data_ptr(), h.bytes, radius, three_floats(center, "center"),
      current_stream()));
  return out;
}

Tensor transform_points(Tensor data_in, vector<float> angle, vector<float> scale, vector<float> jitter, float offset,
    string normal_axis) {
  Tensor points = on_device(data_in);
  PointsHeader h(data_in.is_cuda() ? points : data_in.contiguous());
  Tensor out = torch::empty_like(points);
  check(ocnn_transform_points(out.data_ptr(), points.data_ptr(), h.bytes, three_floats(angle, "angle"),
      three_floats(scale, "scale"), three_floats(jitter, "jitter"), offset, normal_axis.c_str(), current_stream()));
  return out;
}

vector<Tensor> clip_points(Tensor data_in, vector<float> bbmin, vector<float> bbmax) {
  Tensor points = on_device(data_in);
  PointsHeader h(data_in.is_cuda() ? points : data_in.contiguous());
  Tensor out = torch::empty_like(points);
  Tensor mask = torch::empty({h.pt_num()}, points.options().dtype(torch::kInt32));
  unsigned char new_hdr[OCNN_POINTS_INFO_BYTES];
  const size_t wb = ocnn_points_workspace_bytes(h.pt_num());
  Aligned ws(points, wb);
  check(ocnn_clip_points(out.data_ptr(), new_hdr, mask.data_ptr<int>(), points.data_ptr(), h.bytes,
      three_floats(bbmin, "bbmin"), three_floats(bbmax, "bbmax"), ws.p, wb, current_stream()));
  return {out, mask};
}

// ---- pytorch/cpp/point2octree.cpp:5-34 ----------------------------------------------------------------------------
Tensor points2octree(Tensor points_in, int depth, int full_depth, bool node_dis, bool node_feature, bool split_label,
    bool adaptive, int adp_depth, float th_normal, float th_distance, bool extrapolate, bool save_pts, bool key2xyz) {
  Tensor points = on_device(points_in);
  PointsHeader h(points_in.is_cuda() ? points : points_in.contiguous());
  ocnn_build_params bp;
  std::memset(&bp, 0, sizeof(bp));
  bp.depth = depth;
  bp.full_depth = full_depth;
  bp.node_dis = node_dis;
  bp.node_feature = node_feature;
  bp.split_label = split_label;
  bp.adaptive = adaptive;
  bp.adp_depth = adp_depth;
  bp.th_normal = th_normal;
  bp.th_distance = th_distance;
  bp.extrapolate = extrapolate;
  bp.save_pts = save_pts;
  bp.key2xyz = key2xyz;
  const size_t wb = ocnn_points2octree_workspace_bytes(h.pt_num(), 1, std::max(depth, std::max(full_depth, 1)));
  TORCH_CHECK(wb > 0, "bad build arguments (points ", h.pt_num(), ", depth ", depth, ")");
  Aligned ws(points, wb);
  TensorPool pool{points.options(), {}};
  const void* dev[1] = {points.data_ptr()};
  const void* hdr[1] = {h.bytes};
  unsigned char info[OCNN_HEADER_BYTES] = {0};
  void* out_ptr = nullptr;
  check(ocnn_points2octree(dev, hdr, 1, &bp, ws.p, wb, &TensorPool::alloc, &pool, info, &out_ptr, current_stream()));
  Tensor out = pool.take(out_ptr);
  headers().put(out, info);
  return out;
}

// ---- pytorch/cpp/octree_batch.cpp:5-22 ------------------------------------------------------------------------------
Tensor octree_batch(vector<Tensor> tensors_in) {
  const int n = (int)tensors_in.size();
  TORCH_CHECK(n > 0, "octree_batch of nothing");
  vector<Tensor> octs;
  vector<Info> infos;
  vector<const void*> info_ptrs, dev_ptrs;
  octs.reserve(n);
  infos.reserve(n);
  for (const Tensor& t : tensors_in) {
    octs.push_back(on_device(t));
    infos.emplace_back(octs.back());
  }
  for (int i = 0; i < n; ++i) {
    info_ptrs.push_back(infos[i].p());
    dev_ptrs.push_back(octs[i].data_ptr());
  }
  unsigned char hdr[OCNN_HEADER_BYTES] = {0};
  check(ocnn_octree_batch_info(info_ptrs.data(), n, hdr));
  Tensor out = torch::empty({ocnn_info_sizeof_octree(hdr)}, octs[0].options());
  const size_t wb = ocnn_octree_batch_workspace_bytes(n, ocnn_info_depth(hdr));
  Tensor ws = bytes_on(out, wb);
  check(ocnn_octree_batch(out.data_ptr(), hdr, dev_ptrs.data(), info_ptrs.data(), n, ws.data_ptr(), wb,
      current_stream()));
  headers().put(out, hdr);
  return out;
}

// ---- pytorch/cpp/octree_samples.cpp:5-18: `octree_1` .. `octree_6` as CPU uint8 tensors, from the package's data
// file (data/octree_samples.npz beside this module's folder; numpy reads it) ---------------------------------------
int64_t octree_header_copies();
vector<Tensor> octree_samples(vector<string> names) {
  namespace py = pybind11;
  Dl_info self;   // where this shared object was loaded from
  TORCH_CHECK(dladdr(reinterpret_cast<const void*>(&octree_header_copies), &self) != 0 && self.dli_fname,
      "cannot locate the module's file");
  string path(self.dli_fname);
  const size_t slash = path.rfind('/');
  path = (slash == string::npos ? string(".") : path.substr(0, slash)) + "/../data/octree_samples.npz";
  py::object z = py::module_::import("numpy").attr("load")(path);
  py::object from_numpy = py::module_::import("torch").attr("from_numpy");
  vector<Tensor> out;
  for (const string& name : names) {
    TORCH_CHECK(z.attr("files").attr("__contains__")(name).cast<bool>(), "The specified octree does not exist : ", name);
    out.push_back(from_numpy(z.attr("__getitem__")(name).attr("copy")()).cast<Tensor>());
  }
  return out;
}

// ---- pytorch/cpp/octree_property.cpp:308-325: a copy with the features of one depth replaced -------------------------
Tensor octree_set_property(Tensor octree_in, Tensor data_in, int depth) {
  Info info(octree_in);
  const int64_t count = (int64_t)info.nnum(depth) * ocnn_info_channel(info.p(), OCNN_FEATURE);
  TORCH_CHECK(data_in.numel() == count, "Wrong Property Size");
  const int64_t off = ocnn_info_ptr_dis(info.p(), OCNN_FEATURE, depth);
  TORCH_CHECK(off >= 0, "The octree has no feature: d = ", depth);
  Tensor out = octree_in.clone();
  torch::from_blob(static_cast<unsigned char*>(out.data_ptr()) + off, {count}, out.options().dtype(torch::kFloat32))
      .copy_(data_in.to(torch::kFloat32).reshape({-1}));
  headers().put(out, info.bytes);
  return out;
}

// ---- pytorch/cpp/octree_key.cpp:11-47: int16 [N, 4] (x, y, z, id) <-> int64 [N], a copy of the bits -------------------
Tensor octree_encode_key(Tensor xyz) {
  TORCH_CHECK(xyz.dim() == 2 && xyz.size(1) == 4, "The input must be [N, 4]");
  return xyz.to(torch::kInt16).contiguous().view(torch::kInt64).reshape({-1}).clone();
}

Tensor octree_decode_key(Tensor key) {
  TORCH_CHECK(key.dim() == 1 && key.scalar_type() == torch::kInt64, "The dim of input tensor must be 1.");
  return key.contiguous().view(torch::kInt16).reshape({-1, 4}).clone();
}

// ---- pytorch/cpp/transform_octree.cpp:5-22 ------------------------------------------------------------------------------
Tensor octree_scan(Tensor octree_in, vector<float> axis, float scale) {
  Tensor octree = on_device(octree_in);
  Info info(octree);
  TORCH_CHECK(!axis.empty() && axis.size() % 3 == 0, "axis needs 3 floats per direction");
  TensorPool pool{octree.options(), {}};
  unsigned char hdr[OCNN_HEADER_BYTES] = {0};
  void* out_ptr = nullptr;
  check(ocnn_octree_scan(octree.data_ptr(), info.p(), axis.data(), (int)axis.size() / 3, scale, &TensorPool::alloc, &pool,
      hdr, &out_ptr, current_stream()));
  Tensor out = pool.take(out_ptr);
  headers().put(out, hdr);
  return out;
}

// ---- pytorch/cpp/octree_align.cpp:9-83 -------------------------------------------------------------------------------------
namespace {
// sorted Morton keys of a depth (converted from packed xyz where the octree stores those)
Tensor morton_keys(const Tensor& octree, const Info& info, int depth) {
  const int h = info.nnum(depth);
  Tensor key = torch::from_blob(const_cast<int64_t*>(info.prop<int64_t>(octree, OCNN_KEY, depth)), {h},
      octree.options().dtype(torch::kInt64));
  if (ocnn_info_is_key2xyz(info.p()) && h > 0) key = key_op(key, depth, true);
  return key;
}
}  // namespace

vector<Tensor> octree_align(Tensor src_data, Tensor src_octree, Tensor des_octree, int depth) {
  src_data = src_data.contiguous();
  TORCH_CHECK(src_data.scalar_type() == torch::kFloat32, "octree_align is fp32");
  Info sinfo(src_octree), dinfo(des_octree);
  const int channel = (int)src_data.size(1), src_h = (int)src_data.size(2), des_h = dinfo.nnum(depth);
  TORCH_CHECK(sinfo.nnum(depth) == src_h, "octree_align: ", src_h, " rows, the source octree has ", sinfo.nnum(depth),
      " nodes at depth ", depth);
  Tensor src_key = morton_keys(src_octree, sinfo, depth), des_key = morton_keys(des_octree, dinfo, depth);
  Tensor idx = torch::empty({src_h}, src_data.options().dtype(torch::kInt32));
  // the queries are sorted themselves: the plain search walks the same cache lines lane by lane
  check(ocnn_search_key(idx.data_ptr<int>(), reinterpret_cast<const uint64_t*>(des_key.data_ptr<int64_t>()), des_h,
      reinterpret_cast<const uint64_t*>(src_key.data_ptr<int64_t>()), src_h, current_stream()));
  Tensor out = torch::empty({1, channel, des_h, 1}, src_data.options());
  Tensor inverse = torch::empty({std::max(des_h, 1)}, idx.options());
  check(ocnn_align_forward_ws(out.data_ptr<float>(), des_h, channel, src_data.data_ptr<float>(), src_h,
      idx.data_ptr<int>(), inverse.data_ptr<int>(), current_stream()));
  return {out, idx};
}

Tensor octree_align_grad(Tensor des_grad, Tensor idx_tensor) {
  des_grad = des_grad.contiguous();
  idx_tensor = idx_tensor.contiguous();
  TORCH_CHECK(des_grad.scalar_type() == torch::kFloat32 && idx_tensor.scalar_type() == torch::kInt32,
      "octree_align_grad: fp32 gradients, int32 indices");
  const int channel = (int)des_grad.size(1), des_h = (int)des_grad.size(2), src_h = (int)idx_tensor.numel();
  Tensor out = torch::empty({1, channel, src_h, 1}, des_grad.options());
  check(ocnn_align_backward(des_grad.data_ptr<float>(), des_h, channel, out.data_ptr<float>(), src_h,
      idx_tensor.data_ptr<int>(), current_stream()));
  return out;
}

// Test hooks for the header copies: the bytes this file would use for `octree`, and how many
// copies are alive (entries of dead tensors are dropped first).
Tensor octree_header(Tensor octree) {
  Info info(octree);
  Tensor out = torch::empty({OCNN_INFO_BYTES}, torch::TensorOptions().dtype(torch::kUInt8));
  std::memcpy(out.data_ptr(), info.bytes, OCNN_INFO_BYTES);
  return out;
}
int64_t octree_header_copies() { return headers().live(); }

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  namespace py = pybind11;
  m.def("octree_conv", &octree_conv, "octree based convolution");
  m.def("octree_deconv", &octree_deconv, "octree based deconvolution");
  m.def("octree_conv_grad", &octree_conv_grad, "octree based convolution, gradients");
  m.def("octree_deconv_grad", &octree_deconv_grad, "octree based deconvolution, gradients");
  m.def("octree2col", &octree2col, "octree based convolution: gather the taps");
  m.def("col2octree", &col2octree, "octree based convolution: scatter the taps");
  m.def("octree_pad", &octree_pad, "pad", py::arg("data_in"), py::arg("octree"), py::arg("depth"), py::arg("val") = 0.0f);
  m.def("octree_depad", &octree_depad, "depad");
  m.def("octree_max_pool", &octree_max_pool, "max pooling");
  m.def("octree_max_unpool", &octree_max_unpool, "max unpooling");
  m.def("octree_mask_pool", &octree_mask_pool, "pooling through a given mask");
  m.def("octree_xyz2key", &octree_xyz2key, "packed xyz -> Morton key");
  m.def("octree_key2xyz", &octree_key2xyz, "Morton key -> packed xyz");
  m.def("octree_search_key", &octree_search_key, "index of keys in an octree level", py::arg("key"), py::arg("octree"),
      py::arg("depth"), py::arg("key_is_xyz") = true, py::arg("nempty") = false);
  m.def("octree_new", &octree_new, "an octree with the root level only", py::arg("batch_size") = 1, py::arg("channel") = 4,
      py::arg("node_dis") = true, py::arg("adaptive_layer") = 0);
  m.def("octree_grow", &octree_grow, "add one level", py::arg("octree"), py::arg("target_depth"),
      py::arg("full_octree") = false);
  m.def("octree_update", &octree_update, "children of a level from split labels", py::arg("octree"), py::arg("label"),
      py::arg("depth"), py::arg("split") = 1);
  m.def("octree_update_", &octree_update_, "octree_update on the blob itself");
  m.def("octree_property", &octree_property, "a property of an octree", py::arg("octree"), py::arg("property"),
      py::arg("depth") = 0);
  m.def("octree_conv_bn_relu", &octree_conv_bn_relu, "convolution with folded BatchNorm and ReLU");
  m.def("rows_from_channels", &rows_from_channels, "[1, C, H, 1] bf16 -> rows [H + 1, pitch]");
  m.def("channels_from_rows", &channels_from_rows, "rows [H + 1, pitch] -> [1, C, H, 1]");
  m.def("octree_conv_rows", &octree_conv_rows, "convolution on row-major bf16 activations");
  m.def("octree_batch", &octree_batch, "merge a batch of octrees");
  m.def("octree_samples", &octree_samples, "the sample octrees of the package");
  m.def("points2octree", &points2octree, "one octree from one point cloud");
  m.def("octree_set_property", &octree_set_property, "a copy with the features of one depth replaced", py::arg("octree"),
      py::arg("data"), py::arg("depth"));
  m.def("transform_points", &transform_points, "rotate, scale, jitter a point cloud");
  m.def("clip_points", &clip_points, "keep the points inside a box");
  m.def("normalize_points", &normalize_points, "move to a centre and scale by 1 / radius");
  m.def("bounding_sphere", &bounding_sphere, "radius and centre of a bounding sphere");
  m.def("octree_encode_key", &octree_encode_key, "int16 (x, y, z, id) -> int64 key");
  m.def("octree_decode_key", &octree_decode_key, "int64 key -> int16 (x, y, z, id)");
  m.def("octree_scan", &octree_scan, "the part of an octree seen from given directions", py::arg("octree"),
      py::arg("axis"), py::arg("scale") = 1.0f);
  m.def("octree_align", &octree_align, "features moved to the nodes of another octree", py::arg("src_data"),
      py::arg("src_octree"), py::arg("des_octree"), py::arg("depth"));
  m.def("octree_align_grad", &octree_align_grad, "backward of octree_align");
  m.def("points_batch_property", &points_batch_property, "a property of several point clouds, stacked");
  m.def("points_property", &points_property, "a property of a point cloud");
  m.def("points_set_property", &points_set_property, "a copy of a point cloud with one property replaced");
  m.def("points_new", &points_new, "a serialized point cloud from its arrays");
  m.def("octree_header", &octree_header, "the host copy of an octree's header (test hook)");
  m.def("octree_header_copies", &octree_header_copies, "live header copies (test hook)");
}
