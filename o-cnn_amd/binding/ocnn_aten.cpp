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
  Tensor out = octree_in.clone();
  unsigned char hdr[OCNN_HEADER_BYTES];
  std::memcpy(hdr, in.bytes, OCNN_HEADER_BYTES);
  Tensor label = label_in.contiguous().to(torch::kInt32);
  const int n = (int)label.numel();
  const size_t sb = ocnn_octree_update_scratch_bytes(n);
  Tensor ws = bytes_on(octree_in, sb);
  check(ocnn_octree_update(out.data_ptr(), hdr, label.data_ptr<int>(), n, depth, split, ws.data_ptr(), sb,
      current_stream()));
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
  m.def("octree_search_key", &octree_search_key, "index of keys in an octree level");
  m.def("octree_new", &octree_new, "an octree with the root level only");
  m.def("octree_grow", &octree_grow, "add one level");
  m.def("octree_update", &octree_update, "children of a level from split labels");
  m.def("octree_update_", &octree_update_, "octree_update on the blob itself");
  m.def("octree_property", &octree_property, "a property of an octree", py::arg("octree"), py::arg("property"),
      py::arg("depth") = 0);
  m.def("octree_conv_bn_relu", &octree_conv_bn_relu, "convolution with folded BatchNorm and ReLU");
  m.def("rows_from_channels", &rows_from_channels, "[1, C, H, 1] bf16 -> rows [H + 1, pitch]");
  m.def("channels_from_rows", &channels_from_rows, "rows [H + 1, pitch] -> [1, C, H, 1]");
  m.def("octree_conv_rows", &octree_conv_rows, "convolution on row-major bf16 activations");
  m.def("octree_header", &octree_header, "the host copy of an octree's header (test hook)");
  m.def("octree_header_copies", &octree_header_copies, "live header copies (test hook)");
}
