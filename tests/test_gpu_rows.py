"""Row-major bf16 activations: ocnn_rows_from_channels / ocnn_channels_from_rows and
ocnn_octree_conv_rows against the channel-major operators (pytorch/cpp/octree_conv.cpp:131-157
semantics).  The row-major convolution runs the same kernel on the same operands in the same
order as the channel-major one, so the bar is bit equality, and the channel-major operator is
itself checked against the oracle in test_gpu_ops.py / test_gpu_windows.py."""
import numpy as np
import pytest
import torch

from oracle.checker import make_points_blob

pytestmark = pytest.mark.gpu


def T(a):
  return torch.from_numpy(np.ascontiguousarray(a))


@pytest.fixture(scope="module")
def octree(oc, synthetic):
  clouds = []
  for i in range(3):
    p, n, _ = synthetic.shape_cloud(6000, 70 + i)
    clouds.append(T(make_points_blob(p, n)).cuda())
  return oc.nn.points2octree_batch(clouds, 6, 2)


def test_rows_round_trip(oc):
  F = oc.nn
  g = torch.Generator().manual_seed(5)
  for c, h in ((1, 8), (3, 1000), (16, 64), (20, 4104), (64, 33000), (70, 8)):
    x = torch.randn(1, c, h, 1, generator=g).bfloat16().cuda()
    rows = F.to_rows(x)
    assert rows.shape == (h + 1, F.rows_pitch(c))
    assert torch.equal(rows[:h, :c], x.view(c, h).t())
    assert not rows[h].any() and not rows[:, c:].any()
    assert torch.equal(F.from_rows(rows, c), x)


@pytest.mark.parametrize("cin,cout", [(3, 32), (64, 64), (32, 48), (20, 70), (16, 130)])
def test_conv_rows_equals_channel_major(oc, octree, cin, cout):
  F = oc.nn
  info = F.octree_info(octree)
  g = torch.Generator().manual_seed(cin * 1000 + cout)
  for depth in (6, 4):
    H = info.nnum(depth)
    x = torch.randn(1, cin, H, 1, generator=g).bfloat16().cuda()
    bias = torch.randn(cout, generator=g).cuda()
    for deconv in (False, True):
      shape = (cin, cout * 27) if deconv else (cout, cin * 27)
      w = (torch.randn(*shape, generator=g) * 0.05).bfloat16().cuda()
      for b, relu in ((None, False), (bias, True), (bias, False), (None, True)):
        exp = F.octree_conv_fused(x, w, b, relu, octree, depth, cout, [3, 3, 3], 1, False, deconv=deconv)
        rows = F.octree_conv_rows(F.to_rows(x), cin, w, octree, depth, cout, bias=b, relu=relu, deconv=deconv)
        assert rows.shape == (H + 1, F.rows_pitch(cout))
        assert not rows[H].any(), "the row behind the last one must be zero"
        assert not rows[:, cout:].any(), "padding channels must be zero"
        assert torch.equal(F.from_rows(rows, cout), exp), (depth, deconv, relu, b is not None)


def test_conv_rows_chain(oc, octree):
  """two members: the second reads what the first wrote, zero row and padding included"""
  F = oc.nn
  info = F.octree_info(octree)
  g = torch.Generator().manual_seed(9)
  H = info.nnum(6)
  x = torch.randn(1, 24, H, 1, generator=g).bfloat16().cuda()
  w1 = (torch.randn(40, 24 * 27, generator=g) * 0.05).bfloat16().cuda()
  w2 = (torch.randn(64, 40 * 27, generator=g) * 0.05).bfloat16().cuda()
  b1, b2 = torch.randn(40, generator=g).cuda(), torch.randn(64, generator=g).cuda()
  mid = torch.full((H + 1, F.rows_pitch(40)), float("nan"), dtype=torch.bfloat16, device="cuda")   # must be overwritten whole
  F.octree_conv_rows(F.to_rows(x), 24, w1, octree, 6, 40, bias=b1, relu=True, out=mid)
  got = F.from_rows(F.octree_conv_rows(mid, 40, w2, octree, 6, 64, bias=b2, relu=True), 64)
  y = F.octree_conv_fused(x, w1, b1, True, octree, 6, 40, [3, 3, 3], 1, False)
  exp = F.octree_conv_fused(y, w2, b2, True, octree, 6, 64, [3, 3, 3], 1, False)
  assert torch.equal(got, exp)


def test_conv_rows_rejects(oc, octree):
  F = oc.nn
  x = torch.zeros(F.octree_info(octree).nnum(6) + 1, 16, dtype=torch.bfloat16, device="cuda")
  w = torch.zeros(32, 16 * 27, dtype=torch.bfloat16, device="cuda")
  with pytest.raises(oc.nn.OcnnError):
    F.octree_conv_rows(x[:-1].contiguous(), 16, w, octree, 6, 32)       # one row short
  with pytest.raises(oc.nn.OcnnError):
    F.octree_conv_rows(x, 20, w, octree, 6, 32)                         # pitch does not match the channels
