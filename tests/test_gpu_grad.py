"""GPU parity of the gradient operators (OctreeConvGradOp / OctreeDeconvGradOp,
pytorch/cpp/octree_conv.cpp:159-250) against the oracle, whose gradients are pinned by the
adjoint identities and by torch's dense conv3d autograd; plus the autograd wiring of the
modules.  fp32, tolerance 1e-4 relative to the largest magnitude."""
import numpy as np
import pytest
import torch

from oracle.checker import OctreeBlob, make_points_blob

pytestmark = pytest.mark.gpu
TOL = 1e-4


def T(a):
  return torch.from_numpy(np.ascontiguousarray(a))


def relerr(got, exp):
  return float(np.abs(got.astype(np.float64) - exp).max() / (np.abs(exp).max() + 1e-30))


@pytest.fixture(scope="module")
def tree(oc, orc, synthetic):
  pbs = [make_points_blob(*synthetic.shape_cloud(3000, 71 + i)[:2]) for i in range(2)]
  host = orc.octree_batch([orc.points2octree(p, 5, 2) for p in pbs])
  return host, T(host).cuda(), OctreeBlob(host)


CASES = [([3, 3, 3], 1, False), ([3, 3, 3], 1, True), ([2, 2, 2], 2, False), ([2, 2, 2], 2, True),
         ([3, 1, 1], 1, False), ([1, 1, 1], 1, False), ([3, 3, 1], 1, True),
         ([3, 3, 3], 2, False), ([3, 3, 3], 2, True), ([3, 1, 3], 2, False), ([1, 1, 1], 2, True)]


@pytest.mark.parametrize("ks,stride,nempty", CASES)
@pytest.mark.parametrize("ci,co", [(3, 5), (40, 70), (64, 64)])
def test_conv_grad_vs_oracle(oc, orc, tree, ks, stride, nempty, ci, co):
  host, dev, b = tree
  d, K = 5, ks[0] * ks[1] * ks[2]
  rng = np.random.default_rng(ci * 100 + co + K)
  hin = int(b.nnum_nempty[d] if nempty else b.nnum[d])
  x = rng.standard_normal((ci, hin)).astype(np.float32)
  w = (rng.standard_normal((co, ci * K)) * 0.1).astype(np.float32)
  top_h = orc.octree_conv(x, w, host, d, co, ks, stride, nempty).shape[1]
  g = rng.standard_normal((co, top_h)).astype(np.float32)
  egd, egw = orc.octree_conv_grad(x, w, g, host, d, co, ks, stride, nempty)
  gd, gw = oc.nn.octree_conv_grad(T(x).cuda().view(1, ci, hin, 1), T(w).cuda(), dev,
                                  T(g).cuda().view(1, co, top_h, 1), d, co, ks, stride, nempty)
  assert gd.shape == (1, ci, hin, 1) and gw.shape == w.shape
  assert relerr(gw.cpu().numpy(), egw) < TOL
  assert relerr(gd.cpu().numpy().reshape(egd.shape), egd) < TOL


@pytest.mark.parametrize("ks,stride,nempty", CASES)
@pytest.mark.parametrize("ci,co", [(5, 3), (70, 40)])
def test_deconv_grad_vs_oracle(oc, orc, tree, ks, stride, nempty, ci, co):
  host, dev, b = tree
  d, K = 4, ks[0] * ks[1] * ks[2]
  rng = np.random.default_rng(ci * 100 + co + K + 1)
  hin = int(b.nnum_nempty[d] if (nempty or stride == 2) else b.nnum[d])
  x = rng.standard_normal((ci, hin)).astype(np.float32)
  w = (rng.standard_normal((ci, co * K)) * 0.1).astype(np.float32)
  top_h = orc.octree_deconv(x, w, host, d, co, ks, stride, nempty).shape[1]
  g = rng.standard_normal((co, top_h)).astype(np.float32)
  egd, egw = orc.octree_deconv_grad(x, w, g, host, d, co, ks, stride, nempty)
  gd, gw = oc.nn.octree_deconv_grad(T(x).cuda().view(1, ci, hin, 1), T(w).cuda(), dev,
                                    T(g).cuda().view(1, co, top_h, 1), d, co, ks, stride, nempty)
  assert relerr(gw.cpu().numpy(), egw) < TOL
  assert relerr(gd.cpu().numpy().reshape(egd.shape), egd) < TOL


@pytest.mark.parametrize("ci,co", [(32, 128), (128, 64), (32, 32), (64, 32)])
def test_conv_grad_wide_channels(oc, orc, tree, ci, co):
  """3x3x3 stride 1 over all nodes with channel counts in whole 32 / 64 blocks: the weight
  gradient runs its LDS-staged form with several channel and row tiles per slice."""
  host, dev, b = tree
  d = 5
  rng = np.random.default_rng(ci + co)
  hin = int(b.nnum[d])
  x = rng.standard_normal((ci, hin)).astype(np.float32)
  w = (rng.standard_normal((co, ci * 27)) * 0.1).astype(np.float32)
  g = rng.standard_normal((co, hin)).astype(np.float32)
  egd, egw = orc.octree_conv_grad(x, w, g, host, d, co, [3, 3, 3], 1, False)
  gd, gw = oc.nn.octree_conv_grad(T(x).cuda().view(1, ci, hin, 1), T(w).cuda(), dev,
                                  T(g).cuda().view(1, co, hin, 1), d, co, [3, 3, 3], 1, False)
  assert relerr(gw.cpu().numpy(), egw) < TOL
  assert relerr(gd.cpu().numpy().reshape(egd.shape), egd) < TOL
  # deconvolution: the roles of the two tensors swap in the weight gradient
  wd = (rng.standard_normal((ci, co * 27)) * 0.1).astype(np.float32)
  egd, egw = orc.octree_deconv_grad(x, wd, g, host, d, co, [3, 3, 3], 1, False)
  gd, gw = oc.nn.octree_deconv_grad(T(x).cuda().view(1, ci, hin, 1), T(wd).cuda(), dev,
                                    T(g).cuda().view(1, co, hin, 1), d, co, [3, 3, 3], 1, False)
  assert relerr(gw.cpu().numpy(), egw) < TOL
  assert relerr(gd.cpu().numpy().reshape(egd.shape), egd) < TOL


@pytest.mark.parametrize("ks,stride,nempty", [([3, 3, 3], 1, True), ([2, 2, 2], 2, False), ([2, 2, 2], 2, True),
                                              ([3, 1, 1], 1, False), ([3, 3, 1], 1, True), ([3, 3, 3], 2, False)])
@pytest.mark.parametrize("ci,co", [(32, 64), (64, 32), (96, 128)])
def test_weight_gradient_staged_forms(oc, orc, tree, ks, stride, nempty, ci, co):
  """The shapes other than 3x3x3 stride 1 over all nodes with whole 32-channel blocks: the weight
  gradient stages its source rows in LDS from a table of row offsets (2x2x2 stride 2 over all nodes
  reads the finer level in place).  Against the oracle, and against the register-fed kernel that
  serves every other channel count (same products, another order of addition); both for the
  convolution and for the deconvolution, whose weight gradient swaps the two tensors."""
  host, dev, b = tree
  L = oc.lib.get()
  d, K = 5, ks[0] * ks[1] * ks[2]
  rng = np.random.default_rng(ci * 7 + co + K)
  hin = int(b.nnum_nempty[d] if nempty else b.nnum[d])
  x = rng.standard_normal((ci, hin)).astype(np.float32)
  w = (rng.standard_normal((co, ci * K)) * 0.1).astype(np.float32)
  top_h = orc.octree_conv(x, w, host, d, co, ks, stride, nempty).shape[1]
  g = rng.standard_normal((co, top_h)).astype(np.float32)
  _, egw = orc.octree_conv_grad(x, w, g, host, d, co, ks, stride, nempty)
  args = (T(x).cuda().view(1, ci, hin, 1), T(w).cuda(), dev, T(g).cuda().view(1, co, top_h, 1), d, co, ks, stride, nempty)
  _, gw = oc.nn.octree_conv_grad(*args, need_data=False)
  assert relerr(gw.cpu().numpy(), egw) < TOL
  before = L.ocnn_conv_wgrad_staged(0)
  try:
    _, gw_reg = oc.nn.octree_conv_grad(*args, need_data=False)
  finally:
    L.ocnn_conv_wgrad_staged(before)
  assert relerr(gw_reg.cpu().numpy(), egw) < TOL
  assert relerr(gw.cpu().numpy(), gw_reg.cpu().numpy().astype(np.float64)) < TOL
  _, again = oc.nn.octree_conv_grad(*args, need_data=False)
  assert torch.equal(gw, again)   # fixed order of addition: the same bits run to run
  # deconvolution at stride 2 lives one level up
  dd = d - 1 if stride == 2 else d
  hd = int(b.nnum_nempty[dd] if (nempty or stride == 2) else b.nnum[dd])
  xd = rng.standard_normal((ci, hd)).astype(np.float32)
  wd = (rng.standard_normal((ci, co * K)) * 0.1).astype(np.float32)
  top_d = orc.octree_deconv(xd, wd, host, dd, co, ks, stride, nempty).shape[1]
  gd_ = rng.standard_normal((co, top_d)).astype(np.float32)
  _, egw = orc.octree_deconv_grad(xd, wd, gd_, host, dd, co, ks, stride, nempty)
  _, gw = oc.nn.octree_deconv_grad(T(xd).cuda().view(1, ci, hd, 1), T(wd).cuda(), dev, T(gd_).cuda().view(1, co, top_d, 1),
                                   dd, co, ks, stride, nempty, need_data=False)
  assert relerr(gw.cpu().numpy(), egw) < TOL


def test_grad_errors(oc, tree):
  host, dev, b = tree
  x = torch.zeros(1, 4, int(b.nnum[5]), 1, device="cuda")
  w = torch.zeros(8, 4 * 27, device="cuda")
  with pytest.raises(oc.lib.OcnnError) as e:
    oc.nn.octree_conv_grad(x, w, dev, torch.zeros(1, 8, 7, 1, device="cuda"), 5, 8, [3, 3, 3], 1, False)
  assert e.value.code == -3
  with pytest.raises(oc.lib.OcnnError) as e:   # gradients are fp32 only
    oc.nn.octree_conv_grad(x.bfloat16(), w.bfloat16(), dev, torch.zeros(1, 8, int(b.nnum[5]), 1, device="cuda",
                           dtype=torch.bfloat16), 5, 8, [3, 3, 3], 1, False)
  assert e.value.code == -2


def test_modules_backpropagate(oc, orc, tree):
  """OctreeConv(stride 2) -> OctreeMaxPool -> OctreeMaxUnpool -> OctreeDeconv(stride 2): the
  gradients autograd assembles equal the chain of oracle adjoints."""
  host, dev, b = tree
  torch.manual_seed(0)
  L = oc.layers
  conv = L.OctreeConv(5, 6, 8, [2], 2).cuda()
  deconv = L.OctreeDeconv(4, 8, 6, [2], 2).cuda()
  pool, unpool = L.OctreeMaxPool(4, return_indices=True), L.OctreeMaxUnpool(3)
  x = torch.randn(1, 6, int(b.nnum[5]), 1, device="cuda", requires_grad=True)
  y4 = conv(x, dev)                       # depth 4, padded
  p3, mask = pool(y4, dev)                # depth 3
  u4 = unpool(p3, mask, dev)              # depth 4
  out = deconv(u4 + y4, dev)              # depth 5
  gout = torch.randn_like(out)
  out.backward(gout)

  # the same chain through the oracle
  wc, wd = conv.weights.detach().cpu().numpy(), deconv.weights.detach().cpu().numpy()
  xh = x.detach().cpu().numpy().reshape(6, -1)
  child4, child3 = b.prop("child", 4), b.prop("child", 3)
  y4ne = orc.octree_conv(xh, wc, host, 5, 8, [2, 2, 2], 2)
  y4h = orc.pad(y4ne, child4)
  p3ne, maskh = orc.max_pool(y4h)
  u4h = orc.max_unpool(p3ne, maskh)
  s4 = (u4h + y4h)[:, child4 >= 0]
  g = gout.cpu().numpy().reshape(6, -1)
  g_s4, g_wd = orc.octree_deconv_grad(s4, wd, g, host, 4, 6, [2, 2, 2], 2)
  g_sum4 = orc.pad(g_s4, child4)                                   # depad backward
  g_p3ne = orc.mask_pool(g_sum4, maskh)                            # unpool backward
  g_y4 = g_sum4 + orc.max_unpool(g_p3ne, maskh)       # pool backward (pad <-> depad cancel)
  g_x, g_wc = orc.octree_conv_grad(xh, wc, g_y4[:, child4 >= 0], host, 5, 8, [2, 2, 2], 2)
  assert np.array_equal(mask.cpu().numpy().reshape(maskh.shape), maskh)
  assert relerr(deconv.weights.grad.cpu().numpy(), g_wd) < TOL
  assert relerr(conv.weights.grad.cpu().numpy(), g_wc) < TOL
  assert relerr(x.grad.cpu().numpy().reshape(g_x.shape), g_x) < TOL
  _ = child3


def test_weight_gradient_identity_at_full_size(oc, synthetic):
  """Depth-7 batch: <grad_w, W'> == <grad_out, conv(x; W')> with both sides computed on the GPU,
  and the result is reproducible run to run (fixed summation order)."""
  F = oc.nn
  clouds = []
  for i in range(4):
    p, n, _ = synthetic.shape_cloud(50000, 200 + i)
    blob = make_points_blob(p, n)
    t = T(blob).cuda()
    t._ocnn_points_info = blob[:88].copy()
    clouds.append(t)
  octree = F.points2octree_batch(clouds, 7, 2)
  H = F.octree_info(octree).nnum(7)
  g = torch.Generator().manual_seed(3)
  x = torch.randn(1, 64, H, 1, generator=g).cuda()
  w = (torch.randn(64, 64 * 27, generator=g) * 0.02).cuda()
  w2 = torch.randn(64, 64 * 27, generator=g).cuda()
  gy = torch.randn(1, 64, H, 1, generator=g).cuda()
  gd, gw = F.octree_conv_grad(x, w, octree, gy, 7, 64, [3, 3, 3], 1, False)
  lhs = (gw.double() * w2.double()).sum().item()
  rhs = (gy.double() * F.octree_conv(x, w2, octree, 7, 64, [3, 3, 3], 1, False).double()).sum().item()
  assert abs(lhs - rhs) < 1e-4 * max(abs(lhs), abs(rhs), (gw.double().norm() * w2.double().norm()).item() * 1e-2)
  x2 = torch.randn(1, 64, H, 1, generator=g).cuda()
  lhs = (gd.double() * x2.double()).sum().item()
  rhs = (gy.double() * F.octree_conv(x2, w, octree, 7, 64, [3, 3, 3], 1, False).double()).sum().item()
  assert abs(lhs - rhs) < 1e-4 * max(abs(lhs), abs(rhs), (gd.double().norm() * x2.double().norm()).item() * 1e-2)
  _, gw_again = F.octree_conv_grad(x, w, octree, gy, 7, 64, [3, 3, 3], 1, False)
  assert torch.equal(gw, gw_again)


@pytest.mark.parametrize("ks,stride,nempty", [([3, 3, 3], 1, True), ([2, 2, 2], 2, False), ([2, 2, 2], 2, True)])
def test_staged_weight_gradient_identity_at_full_size(oc, synthetic, ks, stride, nempty):
  """Depth-7 batch of four 50 k clouds, 64 -> 64: <grad_w, W'> == <grad_out, conv(x; W')> for the
  shapes whose weight gradient stages its rows from a table (or reads the finer level in place),
  both sides on the GPU, and the same bits run to run."""
  F = oc.nn
  clouds = []
  for i in range(4):
    p, n, _ = synthetic.shape_cloud(50000, 200 + i)
    blob = make_points_blob(p, n)
    t = T(blob).cuda()
    t._ocnn_points_info = blob[:88].copy()
    clouds.append(t)
  octree = F.points2octree_batch(clouds, 7, 2)
  info = F.octree_info(octree)
  K = ks[0] * ks[1] * ks[2]
  hin = info.nnum_nempty(7) if nempty else info.nnum(7)
  g = torch.Generator().manual_seed(4)
  x = torch.randn(1, 64, hin, 1, generator=g).cuda()
  w = (torch.randn(64, 64 * K, generator=g) * 0.02).cuda()
  w2 = torch.randn(64, 64 * K, generator=g).cuda()
  y = F.octree_conv(x, w2, octree, 7, 64, ks, stride, nempty)
  gy = torch.randn(y.shape, generator=g).cuda()
  _, gw = F.octree_conv_grad(x, w, octree, gy, 7, 64, ks, stride, nempty, need_data=False)
  lhs = (gw.double() * w2.double()).sum().item()
  rhs = (gy.double() * y.double()).sum().item()
  assert abs(lhs - rhs) < 1e-4 * max(abs(lhs), abs(rhs), (gw.double().norm() * w2.double().norm()).item() * 1e-2)
  _, again = F.octree_conv_grad(x, w, octree, gy, 7, 64, ks, stride, nempty, need_data=False)
  assert torch.equal(gw, again)
  # the deconvolution's weight gradient: the same geometry with the tensors swapped
  d = 6 if stride == 2 else 7
  hd = info.nnum_nempty(d) if (nempty or stride == 2) else info.nnum(d)
  xd = torch.randn(1, 64, hd, 1, generator=g).cuda()
  wd2 = torch.randn(64, 64 * K, generator=g).cuda()
  yd = F.octree_deconv(xd, wd2, octree, d, 64, ks, stride, nempty)
  gyd = torch.randn(yd.shape, generator=g).cuda()
  _, gwd = F.octree_deconv_grad(xd, w, octree, gyd, d, 64, ks, stride, nempty, need_data=False)
  lhs = (gwd.double() * wd2.double()).sum().item()
  rhs = (gyd.double() * yd.double()).sum().item()
  assert abs(lhs - rhs) < 1e-4 * max(abs(lhs), abs(rhs), (gwd.double().norm() * wd2.double().norm()).item() * 1e-2)
