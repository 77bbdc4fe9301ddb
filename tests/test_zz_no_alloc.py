"""ocnn_octree_conv_static: the convolution entry point whose workspace is the library's own
device array (for callers that cannot allocate).  Called through the C-ABI and compared with
ocnn_octree_conv_fused, the entry point it is a variant of: same kernels, so the results must be
bit-identical.  Every case makes two calls in a row on the shared array, the second on a
smaller input (a shallower level of the same octree)."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle.checker import OctreeBlob, make_points_blob

pytestmark = pytest.mark.gpu

STATIC_BYTES = 16 << 20


def T(a):
  return torch.from_numpy(np.ascontiguousarray(a))


@pytest.fixture(scope="module")
def tree(oc, orc, synthetic):
  pbs = [make_points_blob(*synthetic.shape_cloud(4000, 71 + i)[:2]) for i in range(3)]
  host = orc.octree_batch([orc.points2octree(p, 6, 2) for p in pbs])
  return {"host": host, "dev": T(host).cuda(), "blob": OctreeBlob(host)}


def conv_static(oc, x, w, bias, relu, deconv, octree, depth, num_output, ks, stride, nempty):
  """One call of ocnn_octree_conv_static; the output tensor is the only allocation, made by
  the caller as the entry point demands."""
  nn = oc.nn
  info = nn.octree_info(octree)
  ksc = (C.c_int * 3)(*ks)
  dt = oc.lib.F32 if x.dtype == torch.float32 else oc.lib.BF16
  top_h, need_h = C.c_int(), C.c_int()
  oc.lib.call("ocnn_conv_shape", info.p, depth, x.size(1), num_output, ksc, stride, int(nempty), int(deconv), dt,
              C.byref(top_h), C.byref(need_h), None)
  assert need_h.value == x.size(2)
  out = torch.full((1, num_output, top_h.value, 1), float("nan"), dtype=x.dtype, device="cuda")
  code = oc.lib.get().ocnn_octree_conv_static(
      C.c_void_p(out.data_ptr()), C.c_void_p(x.data_ptr()), x.size(1), x.size(2), C.c_void_p(w.data_ptr()),
      C.c_void_p(bias.data_ptr() if bias is not None else 0), int(relu), int(deconv),
      C.c_void_p(octree.data_ptr()), info.p, depth, num_output, ksc, stride, int(nempty), dt,
      C.c_void_p(torch.cuda.current_stream().cuda_stream))
  return code, out


CASES = [
    # dtype, ks, stride, nempty, deconv, Cin, Cout, relu
    (torch.float32, [3, 3, 3], 1, False, False, 64, 64, True),    # packed weights only
    (torch.float32, [3, 3, 3], 1, False, True, 32, 48, False),
    (torch.float32, [2, 2, 2], 2, False, False, 64, 64, False),
    (torch.float32, [2, 2, 2], 2, False, True, 32, 32, True),     # touches no scratch at all
    (torch.float32, [3, 3, 3], 1, True, False, 24, 40, True),     # + inverted child links + input copy
    (torch.float32, [3, 1, 1], 1, False, False, 16, 16, False),   # general kernel: input copy
    (torch.bfloat16, [3, 3, 3], 1, False, False, 64, 64, True),   # + row-major bf16 copy
    (torch.bfloat16, [2, 2, 2], 2, False, False, 64, 32, False),
    (torch.bfloat16, [2, 2, 2], 2, False, True, 32, 64, False),
    (torch.bfloat16, [3, 3, 3], 1, True, False, 32, 32, False),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "%s-%s-s%d-ne%d-de%d-%d-%d" % (
    str(c[0]).split(".")[-1], "".join(map(str, c[1])), c[2], c[3], c[4], c[5], c[6]))
def test_static_equals_workspace_form(oc, tree, case):
  dtype, ks, stride, nempty, deconv, cin, cout, relu = case
  b, dev = tree["blob"], tree["dev"]
  K = ks[0] * ks[1] * ks[2]
  g = torch.Generator().manual_seed(5)
  w = (torch.randn((cin, cout * K) if deconv else (cout, cin * K), generator=g) * 0.05).to(dtype).cuda()
  bias = (torch.randn(cout, generator=g) * 0.1).cuda()
  # two calls in a row on the shared array: depth 6 first, then the smaller depth 5 (a
  # stride-2 deconvolution writes one level below its input, so it starts at depth 5)
  for depth in ((5, 4) if (stride == 2 and deconv) else (6, 5)):
    rows = int(b.nnum_nempty[depth]) if (nempty or (stride == 2 and deconv)) else int(b.nnum[depth])
    x = torch.randn((1, cin, rows, 1), generator=g).to(dtype).cuda()
    exp = oc.nn.octree_conv_fused(x, w, bias, relu, dev, depth, cout, ks, stride, nempty, deconv=deconv)
    code, got = conv_static(oc, x, w, bias, relu, deconv, dev, depth, cout, ks, stride, nempty)
    assert code == 0, oc.lib.get().ocnn_last_error().decode()
    torch.cuda.synchronize()
    assert got.shape == exp.shape
    assert torch.equal(got.view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                       exp.view(torch.int16 if dtype == torch.bfloat16 else torch.int32)), (depth, case)


def test_static_matches_the_oracle(oc, orc, tree):
  """Not only equal to the other entry point: right.  fp32 within 1e-4 of the CPU oracle."""
  b, dev, host = tree["blob"], tree["dev"], tree["host"]
  rng = np.random.default_rng(9)
  w = (rng.standard_normal((32, 16 * 27)) * 0.05).astype(np.float32)
  for depth in (6, 4):
    H = int(b.nnum[depth])
    x = rng.standard_normal((16, H)).astype(np.float32)
    code, got = conv_static(oc, T(x).cuda().view(1, 16, H, 1), T(w).cuda(), None, False, False, dev, depth, 32,
                            [3, 3, 3], 1, False)
    assert code == 0
    exp = orc.octree_conv(x, w, host, depth, 32, [3, 3, 3], 1, False)
    err = np.abs(got.cpu().numpy().reshape(exp.shape) - exp).max() / np.abs(exp).max()
    assert err < 1e-4, (depth, err)


def test_static_refuses_what_does_not_fit(oc, tree):
  """bf16 3x3x3 needs a row-major copy of the input: 512 channels x 2 bytes x rows is beyond
  the array; the call must say so and leave the output untouched."""
  b, dev = tree["blob"], tree["dev"]
  H = int(b.nnum[6])
  assert (H + 1) * 512 * 2 > STATIC_BYTES
  x = torch.zeros((1, 512, H, 1), dtype=torch.bfloat16, device="cuda")
  w = torch.zeros((32, 512 * 27), dtype=torch.bfloat16, device="cuda")
  code, out = conv_static(oc, x, w, None, False, False, dev, 6, 32, [3, 3, 3], 1, False)
  assert code == -4
  msg = oc.lib.get().ocnn_last_error().decode()
  assert "scratch" in msg and str(STATIC_BYTES) in msg, msg
  torch.cuda.synchronize()
  assert bool(torch.isnan(out.float()).all())
  # a call that fits still works afterwards
  x2 = torch.randn((1, 8, H, 1), device="cuda")
  w2 = torch.randn((8, 8 * 27), device="cuda") * 0.05
  code, got = conv_static(oc, x2, w2, None, False, False, dev, 6, 8, [3, 3, 3], 1, False)
  assert code == 0
  assert torch.equal(got, oc.nn.octree_conv_fused(x2, w2, None, False, dev, 6, 8, [3, 3, 3], 1, False))
