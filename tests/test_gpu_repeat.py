"""Every operator of the hot path, run three times on the depth-9 scene of BASELINE config 4: the
results must be equal bit for bit.  None of the kernels uses float atomics on this path, so a
difference from run to run is a race or a hazard (one was found this way: a 16-byte store whose
data registers were overwritten before the store had read them showed up as a few wrong words per
million outputs, and only at this size)."""
import numpy as np
import pytest
import torch

from oracle.checker import make_points_blob

pytestmark = pytest.mark.gpu


def T(a):
  return torch.from_numpy(np.ascontiguousarray(a))


@pytest.fixture(scope="module")
def scene(oc, synthetic):
  p, n, f = synthetic.room_cloud(250000, 3)
  return oc.nn.points2octree_batch([T(make_points_blob(p, n, f)).cuda()], 9, 2)


def same(fn, what):
  first = fn()
  first = first if isinstance(first, (tuple, list)) else (first,)
  for _ in range(2):
    again = fn()
    again = again if isinstance(again, (tuple, list)) else (again,)
    for a, b in zip(first, again):
      assert torch.equal(a, b), what
  return first[0]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_convolutions_repeat(oc, scene, dtype):
  F = oc.nn
  info = F.octree_info(scene)
  g = torch.Generator().manual_seed(12)
  C = 32
  H9, Hne9, Hne8 = info.nnum(9), info.nnum_nempty(9), info.nnum_nempty(8)
  x = torch.randn(1, C, H9, 1, generator=g).to(dtype).cuda()
  xne = torch.randn(1, C, Hne9, 1, generator=g).to(dtype).cuda()
  x8 = torch.randn(1, C, Hne8, 1, generator=g).to(dtype).cuda()
  w3 = (torch.randn(48, C * 27, generator=g) * 0.05).to(dtype).cuda()
  w2 = (torch.randn(48, C * 8, generator=g) * 0.05).to(dtype).cuda()
  wd = (torch.randn(C, 48 * 8, generator=g) * 0.05).to(dtype).cuda()
  bias = torch.randn(48, generator=g).cuda()
  same(lambda: F.octree_conv(x, w3, scene, 9, 48, [3, 3, 3], 1, False), "conv333")
  same(lambda: F.octree_conv_fused(x, w3, bias, True, scene, 9, 48, [3, 3, 3], 1, False), "conv333 fused")
  same(lambda: F.octree_conv(x, w2, scene, 9, 48, [2, 2, 2], 2, False), "conv222 s2")
  same(lambda: F.octree_conv(xne, w3, scene, 9, 48, [3, 3, 3], 1, True), "conv333 nempty")
  same(lambda: F.octree_conv(xne, w2, scene, 9, 48, [2, 2, 2], 2, True), "conv222 s2 nempty")
  same(lambda: F.octree_deconv(x8, wd, scene, 8, 48, [2, 2, 2], 2, False), "deconv222 s2")
  same(lambda: F.octree_deconv(x8, wd, scene, 8, 48, [2, 2, 2], 2, True), "deconv222 s2 nempty")


def test_gradients_repeat(oc, scene):
  F = oc.nn
  info = F.octree_info(scene)
  g = torch.Generator().manual_seed(13)
  H9 = info.nnum(9)
  x = torch.randn(1, 32, H9, 1, generator=g).cuda()
  w = (torch.randn(32, 32 * 27, generator=g) * 0.05).cuda()
  gy = torch.randn(1, 32, H9, 1, generator=g).cuda()
  same(lambda: F.octree_conv_grad(x, w, scene, gy, 9, 32, [3, 3, 3], 1, False), "conv333 gradients")


def test_streaming_operators_repeat(oc, scene):
  F = oc.nn
  info = F.octree_info(scene)
  g = torch.Generator().manual_seed(14)
  H9, H8, Hne8 = info.nnum(9), info.nnum(8), info.nnum_nempty(8)
  x = torch.randn(1, 16, H9, 1, generator=g).cuda()
  top = same(lambda: F.octree_max_pool(x, scene, 9), "max_pool")
  _, mask = F.octree_max_pool(x, scene, 9)
  same(lambda: F.octree_max_unpool(top, mask, scene, 9), "max_unpool")
  padded = same(lambda: F.octree_pad(top, scene, 8), "pad")
  same(lambda: F.octree_depad(padded, scene, 8), "depad")
  col = same(lambda: F.octree2col(x[:, :4].contiguous(), scene, 9, [3, 3, 3], 1, False), "octree2col")
  same(lambda: F.col2octree(col, scene, 9, [3, 3, 3], 1, False), "col2octree")


def test_build_repeat(oc, synthetic):
  p, n, f = synthetic.room_cloud(250000, 3)
  blob = T(make_points_blob(p, n, f)).cuda()
  same(lambda: oc.nn.points2octree_batch([blob], 9, 2), "points2octree")
