// ATen side of the convolution operators over libocnn_hip.so: the bodies a maintainer of the
// reference's PyTorch extension puts in place of OctreeConvOp / OctreeDeconvOp /
// OctreeConvGradOp (pytorch/cpp/octree_conv.cpp:131-283) and registers under the same names
// (pytorch/cpp/pybind.cpp:17-24).  The signatures are the reference's (pytorch/cpp/ocnn.h:20-33);
// the library sees plain pointers, sizes and the current HIP stream.
//
// This file is compiled against include/ocnn_hip.h and PyTorch's headers by the test suite
// (syntax and types; the test does not link it), so that the documented drop-in cannot drift
// away from the C interface.  The package itself ships the same mapping in Python (nn.py).
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>

#include <cstring>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "ocnn_hip.h"

namespace {

using torch::Tensor;
using std::vector;

// One host copy of the 716-byte header per blob tensor, keyed by the tensor's storage: the
// reference reads the header back from the device in every operator call
// (octree/octree/octree_parser.cu:4-27).
struct HeaderCopy { unsigned char bytes[OCNN_HEADER_BYTES]; };
const void* host_info(const Tensor& octree) {
  static std::mutex m;
  static std::unordered_map<const void*, HeaderCopy> cache;
  std::lock_guard<std::mutex> lock(m);
  const void* key = octree.data_ptr();
  auto it = cache.find(key);
  if (it == cache.end()) {
    HeaderCopy h;
    std::memset(&h, 0, sizeof(h));
    Tensor head = octree.flatten().slice(0, 0, OCNN_INFO_BYTES).cpu();
    std::memcpy(h.bytes, head.data_ptr(), OCNN_INFO_BYTES);
    it = cache.emplace(key, h).first;
  }
  return it->second.bytes;
}

int dtype_of(const Tensor& t) {
  TORCH_CHECK(t.scalar_type() == torch::kFloat32 || t.scalar_type() == torch::kBFloat16,
      "octree convolution: fp32 or bf16 features");
  return t.scalar_type() == torch::kBFloat16 ? OCNN_BF16 : OCNN_F32;
}

ocnn_stream_t current_stream() {
  return reinterpret_cast<ocnn_stream_t>(c10::hip::getCurrentHIPStream().stream());
}

Tensor conv_forward(Tensor data_in, Tensor weights, Tensor octree, int depth, int num_output,
    vector<int> kernel_size, int stride, bool nempty, bool deconv, const Tensor* bias, bool relu) {
  TORCH_CHECK(kernel_size.size() == 3, "kernel_size holds three numbers");
  data_in = data_in.contiguous();
  weights = weights.contiguous();
  const void* info = host_info(octree);
  const int dt = dtype_of(data_in);
  int top_h = 0, btm_h = 0;
  size_t ws_bytes = 0;
  int rc = ocnn_conv_shape(info, depth, (int)data_in.size(1), num_output, kernel_size.data(), stride,
      nempty ? 1 : 0, deconv ? 1 : 0, dt, &top_h, &btm_h, &ws_bytes);
  TORCH_CHECK(rc == OCNN_OK, ocnn_last_error());
  TORCH_CHECK(data_in.size(2) == btm_h, "input height ", data_in.size(2), ", the octree has ", btm_h);
  Tensor ws = torch::empty({(int64_t)ws_bytes}, octree.options().dtype(torch::kUInt8));
  Tensor out = torch::empty({1, num_output, top_h, 1}, data_in.options());
  Tensor b;
  if (bias) b = bias->to(torch::kFloat32).contiguous();
  rc = ocnn_octree_conv_fused(out.data_ptr(), data_in.data_ptr(), (int)data_in.size(1), (int)data_in.size(2),
      weights.data_ptr(), bias ? b.data_ptr<float>() : nullptr, relu ? 1 : 0, deconv ? 1 : 0,
      octree.data_ptr(), info, depth, num_output, kernel_size.data(), stride, nempty ? 1 : 0, dt,
      ws.data_ptr(), ws_bytes, current_stream());
  TORCH_CHECK(rc == OCNN_OK, ocnn_last_error());
  return out;
}

vector<Tensor> conv_backward(Tensor data_in, Tensor weights, Tensor octree, Tensor grad_in, int depth,
    int num_output, vector<int> kernel_size, int stride, bool nempty, bool deconv) {
  TORCH_CHECK(kernel_size.size() == 3, "kernel_size holds three numbers");
  data_in = data_in.contiguous();
  weights = weights.contiguous();
  grad_in = grad_in.contiguous();
  const void* info = host_info(octree);
  size_t ws_bytes = 0;
  int rc = ocnn_conv_grad_workspace_bytes(info, depth, (int)data_in.size(1), num_output, kernel_size.data(),
      stride, nempty ? 1 : 0, deconv ? 1 : 0, OCNN_F32, &ws_bytes);
  TORCH_CHECK(rc == OCNN_OK, ocnn_last_error());
  Tensor ws = torch::empty({(int64_t)ws_bytes}, octree.options().dtype(torch::kUInt8));
  // both results are written completely: no torch::zeros
  Tensor btm_out = torch::empty_like(data_in), weights_out = torch::empty_like(weights);
  auto fn = deconv ? ocnn_octree_deconv_grad : ocnn_octree_conv_grad;
  rc = fn(btm_out.data_ptr(), weights_out.data_ptr(), data_in.data_ptr(), (int)data_in.size(1),
      (int)data_in.size(2), weights.data_ptr(), grad_in.data_ptr(), octree.data_ptr(), info, depth,
      num_output, kernel_size.data(), stride, nempty ? 1 : 0, OCNN_F32, ws.data_ptr(), ws_bytes,
      current_stream());
  TORCH_CHECK(rc == OCNN_OK, ocnn_last_error());
  return {btm_out, weights_out};
}

}  // namespace

// pytorch/cpp/ocnn.h:20-33
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

// ---- row-major bf16 activations (no counterpart in the reference): rows [H + 1, pitch] ----------------
Tensor rows_from_channels(Tensor data) {
  data = data.contiguous();
  const int c = (int)data.size(1), h = (int)data.size(2), pitch = (c + 15) / 16 * 16;
  Tensor rows = torch::empty({h + 1, pitch}, data.options());
  int rc = ocnn_rows_from_channels(rows.data_ptr(), pitch, data.data_ptr(), c, h, dtype_of(data), current_stream());
  TORCH_CHECK(rc == OCNN_OK, ocnn_last_error());
  return rows;
}

Tensor channels_from_rows(Tensor rows, int channels) {
  rows = rows.contiguous();
  const int h = (int)rows.size(0) - 1;
  Tensor data = torch::empty({1, channels, h, 1}, rows.options());
  int rc = ocnn_channels_from_rows(data.data_ptr(), rows.data_ptr(), (int)rows.size(1), channels, h, dtype_of(rows),
      current_stream());
  TORCH_CHECK(rc == OCNN_OK, ocnn_last_error());
  return data;
}

// conv / deconv + bias + ReLU on row-major tensors; rows_in [H + 1, pitch(channel_in)] -> [top_h + 1, pitch(num_output)]
Tensor octree_conv_rows(Tensor rows_in, int channel_in, Tensor weights, Tensor bias, bool relu, Tensor octree,
    int depth, int num_output, vector<int> kernel_size, int stride, bool nempty, bool deconv) {
  TORCH_CHECK(kernel_size.size() == 3, "kernel_size holds three numbers");
  TORCH_CHECK(rows_in.dim() == 2 && rows_in.stride(1) == 1, "rows_in is [H + 1, pitch] with unit channel stride");
  weights = weights.contiguous();
  const void* info = host_info(octree);
  const int dt = dtype_of(rows_in);
  int top_h = 0, btm_h = 0;
  size_t ws_bytes = 0;
  int rc = ocnn_conv_rows_shape(info, depth, channel_in, num_output, kernel_size.data(), stride, nempty ? 1 : 0,
      deconv ? 1 : 0, dt, &top_h, &btm_h, &ws_bytes);
  TORCH_CHECK(rc == OCNN_OK, ocnn_last_error());
  Tensor ws = torch::empty({(int64_t)ws_bytes + 16}, octree.options().dtype(torch::kUInt8));
  Tensor out = torch::empty({top_h + 1, (num_output + 15) / 16 * 16}, rows_in.options());
  Tensor b;
  if (bias.defined() && bias.numel() > 0) b = bias.to(torch::kFloat32).contiguous();
  rc = ocnn_octree_conv_rows(out.data_ptr(), (int)out.stride(0), rows_in.data_ptr(), (int)rows_in.stride(0), channel_in,
      (int)rows_in.size(0) - 1, weights.data_ptr(), b.defined() ? b.data_ptr<float>() : nullptr, relu ? 1 : 0,
      deconv ? 1 : 0, octree.data_ptr(), info, depth, num_output, kernel_size.data(), stride, nempty ? 1 : 0, dt,
      ws.data_ptr(), ws_bytes, current_stream());
  TORCH_CHECK(rc == OCNN_OK, ocnn_last_error());
  return out;
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("octree_conv", &octree_conv, "octree based convolution");
  m.def("octree_deconv", &octree_deconv, "octree based deconvolution");
  m.def("octree_conv_grad", &octree_conv_grad, "octree based convolution, gradients");
  m.def("octree_deconv_grad", &octree_deconv_grad, "octree based deconvolution, gradients");
  m.def("octree_conv_bn_relu", &octree_conv_bn_relu, "convolution with folded BatchNorm and ReLU");
  m.def("rows_from_channels", &rows_from_channels, "[1, C, H, 1] bf16 -> rows [H + 1, pitch]");
  m.def("channels_from_rows", &channels_from_rows, "rows [H + 1, pitch] -> [1, C, H, 1]");
  m.def("octree_conv_rows", &octree_conv_rows, "convolution on row-major bf16 activations");
}
