"""Operator calls on different streams must not share scratch memory: the Python mirror keeps one
workspace per (device, stream, tag).  Two different convolutions are queued alternately on two
streams, so that their kernels overlap on the device, and every result is compared with the one
computed alone on the default stream."""
import numpy as np
import pytest
import torch

from oracle.checker import make_points_blob

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_convs_on_two_streams(oc, orc, synthetic, dtype):
  pbs = [make_points_blob(*synthetic.shape_cloud(20000, 301 + i)[:2]) for i in range(4)]
  octree = oc.nn.points2octree_batch([torch.from_numpy(p) for p in pbs], 7, 2)
  info = oc.nn.octree_info(octree)
  H, Hne = info.nnum(7), info.nnum_nempty(7)
  g = torch.Generator().manual_seed(3)
  xa = torch.randn((1, 32, H, 1), generator=g).to(dtype).cuda()
  xb = torch.randn((1, 48, Hne, 1), generator=g).to(dtype).cuda()
  wa = (torch.randn((64, 32 * 27), generator=g) * 0.05).to(dtype).cuda()
  wb = (torch.randn((32, 48 * 27), generator=g) * 0.05).to(dtype).cuda()

  def conv_a():
    return oc.nn.octree_conv(xa, wa, octree, 7, 64, [3, 3, 3], 1, False)

  def conv_b():   # non-empty mode: inverted child links and a row-major copy live in the workspace
    return oc.nn.octree_conv(xb, wb, octree, 7, 32, [3, 3, 3], 1, True)

  exp_a, exp_b = conv_a(), conv_b()
  torch.cuda.synchronize()
  sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
  got_a, got_b = [], []
  for _ in range(6):
    with torch.cuda.stream(sa):
      got_a.append(conv_a())
    with torch.cuda.stream(sb):
      got_b.append(conv_b())
  torch.cuda.synchronize()
  for y in got_a:
    assert torch.equal(y, exp_a)
  for y in got_b:
    assert torch.equal(y, exp_b)
  keys = [k for k in oc.nn._workspaces if k[2] == "conv"]
  assert len({k[1] for k in keys}) >= 3   # default stream and the two side streams
