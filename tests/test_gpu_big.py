"""Tensors of more than 2^31 elements on the depth-9 scene of BASELINE config 4: every operator
indexes them with 64-bit offsets.  Checked through size-independent properties: an operator
works channel by channel (or is linear in the channels), so a slice of the big result equals
the small result of that slice, which the parity tests pin against the oracle."""
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
  octree = oc.nn.points2octree_batch([T(make_points_blob(p, n, f)).cuda()], 9, 2)
  return octree, oc.nn.octree_info(octree)


def test_octree2col_and_back_beyond_2g_elements(oc, scene):
  octree, info = scene
  H, C, K = info.nnum(9), 64, 27
  assert C * K * H > 2 ** 31
  g = torch.Generator(device="cuda").manual_seed(1)
  x = torch.randn(1, C, H, 1, device="cuda", generator=g)
  col = oc.nn.octree2col(x, octree, 9, [3, 3, 3], 1, False)
  assert col.shape == (C, K, H)
  for c in (0, 1, 19, 20, 41, 63):      # 20 * K * H is the first channel past 2^31 elements
    one = oc.nn.octree2col(x[:, c:c + 1].contiguous(), octree, 9, [3, 3, 3], 1, False)
    assert torch.equal(col[c], one[0]), c
  back = oc.nn.col2octree(col, octree, 9, [3, 3, 3], 1, False)
  assert back.shape == (1, C, H, 1)
  for c in (0, 19, 20, 63):
    one = oc.nn.col2octree(col[c:c + 1].contiguous(), octree, 9, [3, 3, 3], 1, False)
    assert torch.equal(back[0, c], one[0, 0]), c
  del col, back
  torch.cuda.empty_cache()


def test_streaming_operators_beyond_2g_elements(oc, scene):
  """Pooling, unpooling, padding over 1536 channels of the depth-9 level (2.3 G elements)."""
  octree, info = scene
  H, C = info.nnum(9), 1536
  assert C * H > 2 ** 31
  g = torch.Generator(device="cuda").manual_seed(2)
  x = torch.randn(1, C, H, 1, device="cuda", generator=g)
  probes = (0, 700, 1437, 1438, 1535)   # 1437 * H < 2^31 <= 1438 * H
  assert 1437 * H < 2 ** 31 <= 1438 * H
  top, mask = oc.nn.octree_max_pool(x, octree, 9)
  un = oc.nn.octree_max_unpool(top, mask, octree, 9)
  for c in probes:
    xc = x[:, c:c + 1].contiguous()
    t1, m1 = oc.nn.octree_max_pool(xc, octree, 9)
    assert torch.equal(top[0, c], t1[0, 0]) and torch.equal(mask[0, c], m1[0, 0]), c
    assert torch.equal(un[0, c], oc.nn.octree_max_unpool(t1, m1, octree, 9)[0, 0]), c
  del top, mask, un
  # depad at depth 9 (H -> non-empty rows), pad back: the non-empty rows return, the others are 0
  dp = oc.nn.octree_depad(x, octree, 9)
  assert dp.shape[2] == info.nnum_nempty(9)
  pd = oc.nn.octree_pad(dp, octree, 9)
  child = oc.nn.octree_property(octree, "child", 9)
  for c in probes:
    assert torch.equal(dp[0, c, :, 0], x[0, c, :, 0][child >= 0]), c
    assert torch.equal(pd[0, c, :, 0], torch.where(child >= 0, x[0, c, :, 0], torch.zeros((), device="cuda"))), c
  del dp, pd, x
  torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_conv_output_beyond_2g_elements(oc, scene, dtype):
  """3x3x3 convolution 8 -> 1536 channels over the depth-9 level (2.3 G output elements): a
  block of output channels equals the convolution with that block of the weights; the weight
  gradient works row by row likewise and the data gradient is the sum over the two halves."""
  octree, info = scene
  H, Ci, Co = info.nnum(9), 8, 1536
  g = torch.Generator(device="cuda").manual_seed(3)
  x = torch.randn(1, Ci, H, 1, device="cuda", generator=g).to(dtype)
  w = (torch.randn(Co, Ci * 27, device="cuda", generator=g) * 0.05).to(dtype)
  conv = lambda ww: oc.nn.octree_conv(x, ww, octree, 9, ww.shape[0], [3, 3, 3], 1, False)
  y = conv(w)
  assert y.shape == (1, Co, H, 1) and y.numel() > 2 ** 31
  for lo in (0, 1408, 1472):              # 1437 * H < 2^31 <= 1438 * H: the last two blocks lie past it
    part = conv(w[lo:lo + 64].contiguous())
    assert torch.equal(y[0, lo:lo + 64], part[0]), lo
  if dtype == torch.float32:
    gy = y
    gx, gw = oc.nn.octree_conv_grad(x, w, octree, gy, 9, Co, [3, 3, 3], 1, False)
    half = Co // 2
    parts = [oc.nn.octree_conv_grad(x, w[a:a + half].contiguous(), octree, gy[:, a:a + half].contiguous(), 9, half,
                                    [3, 3, 3], 1, False) for a in (0, half)]
    ref = parts[0][0] + parts[1][0]
    assert float((gx - ref).abs().max() / ref.abs().max()) < 1e-4
    for i, a in enumerate((0, half)):
      assert float((gw[a:a + half] - parts[i][1]).abs().max() / parts[i][1].abs().max()) < 1e-4
  del y
  torch.cuda.empty_cache()
