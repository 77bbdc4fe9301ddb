"""GPU parity of octree_scan (pytorch/cpp/transform_octree.cpp:5-22): the scanned octree equals
the oracle's byte for byte (the oracle equals the compiled reference, tests/test_oracle_scan.py)."""
import numpy as np
import pytest
import torch

from oracle.checker import OctreeBlob, make_points_blob
from test_oracle_scan import CASES, sphere_octree

pytestmark = pytest.mark.gpu


def T(a):
  return torch.from_numpy(np.ascontiguousarray(a))


@pytest.mark.parametrize("case", range(len(CASES)))
def test_scan_vs_oracle(oc, orc, case):
  rng = np.random.default_rng(900 + case)
  for trial in range(6):
    blob = sphere_octree(orc, int(rng.integers(500, 6000)), 10 * case + trial, int(rng.integers(4, 7)), **CASES[case])
    n_axis = 1 + trial % 3
    axis = rng.standard_normal((n_axis, 3)).astype(np.float32)
    axis /= np.linalg.norm(axis, axis=1, keepdims=True)
    if trial == 4:
      axis[0] = [0, 0, 1]
    if trial == 5:
      axis[0] = [0, 0, -1]
    scale = float(rng.choice([1.0, 0.5, 2.0]))
    got = oc.nn.octree_scan(T(blob), axis, scale).cpu().numpy()
    exp = orc.octree_scan(blob, axis, scale)
    assert got.size == exp.size and np.array_equal(got, exp), (case, trial)


def test_scan_scene_and_errors(oc, orc, synthetic):
  """The depth-8 room built on the device, scanned from two sides; a batched octree is refused."""
  p, n, f = synthetic.room_cloud(60000, 4)
  pb = make_points_blob(p, n, f)
  octree = oc.nn.points2octree(T(pb), 8, 2)
  axis = np.float32([[0.3, -0.5, -0.8], [-0.6, 0.6, 0.5]])
  axis /= np.linalg.norm(axis, axis=1, keepdims=True)
  got = oc.nn.octree_scan(octree, axis).cpu().numpy()
  assert np.array_equal(got, orc.octree_scan(octree.cpu().numpy(), axis, 1.0))
  b = OctreeBlob(got)
  assert 0 < b.nnum_nempty[8] < OctreeBlob(octree.cpu().numpy()).nnum_nempty[8]
  # the scanned octree is a valid input of octree_batch and of the operators
  merged = oc.nn.octree_batch([oc.nn.octree_scan(octree, axis)])
  assert np.array_equal(merged.cpu().numpy(), orc.octree_batch([got]))
  with pytest.raises(oc.lib.OcnnError):
    oc.nn.octree_scan(merged, axis)


@pytest.mark.parametrize("case", range(len(CASES)))
def test_dropout_vs_oracle(oc, orc, case):
  """octree_dropout (octree/octree/transform_octree.cpp:286-431) for given flags: byte for byte
  the oracle's blob (the oracle equals the compiled reference on the flags the reference drew,
  tests/test_oracle_dropout.py)."""
  rng = np.random.default_rng(1200 + case)
  for trial in range(6):
    depth = int(rng.integers(4, 7))
    blob = sphere_octree(orc, int(rng.integers(500, 6000)), 10 * case + trial, depth, **CASES[case])
    if trial == 3:
      blob = orc.octree_batch([blob, sphere_octree(orc, 900, 77 + case, depth, **CASES[case])])
    dd = int(rng.integers(0, depth + 1))
    ratio = float(rng.choice([0.0, 0.2, 0.5, 0.9, 1.0]))
    flags = (rng.uniform(size=OctreeBlob(blob).nnum[dd]) < ratio).astype(np.uint8)
    got = oc.nn.octree_dropout(T(blob), dd, ratio, flags=T(flags)).cpu().numpy()
    exp = orc.octree_dropout(blob, flags, dd)
    assert got.size == exp.size and np.array_equal(got, exp), (case, trial, dd, ratio)


def test_dropout_scene_draws_and_errors(oc, orc, synthetic):
  """The depth-8 room: flags drawn on the device at the given ratio, the result a valid input
  of octree_batch; the same generator state gives the same octree; bad arguments raise."""
  p, n, f = synthetic.room_cloud(60000, 4)
  octree = oc.nn.points2octree(T(make_points_blob(p, n, f)), 8, 2)
  src = OctreeBlob(octree.cpu().numpy())
  g = torch.Generator(device="cuda")
  g.manual_seed(5)
  a = oc.nn.octree_dropout(octree, 5, 0.3, generator=g)
  g.manual_seed(5)
  b = oc.nn.octree_drop(octree, 5, 0.3, generator=g)
  assert torch.equal(a, b)
  out = OctreeBlob(a.cpu().numpy())
  kept = out.nnum[6] / src.nnum[6]
  assert 0.6 < kept < 0.8 and list(out.nnum[:6]) == list(src.nnum[:6])
  for d in range(6, 9):
    assert out.nnum[d] == 8 * out.nnum_nempty[d - 1]
  # with the child entries of the dropped nodes cleared the result is an ordinary octree
  g.manual_seed(5)
  c = oc.nn.octree_dropout(octree, 5, 0.3, generator=g, clear_dropped=True)
  fixed = a.cpu().numpy().copy()
  ch = OctreeBlob(fixed).prop("child", 5)
  stale = (ch >= out.nnum_nempty[5]) | ((ch >= 0) & (ch != np.cumsum(ch >= 0) - 1))
  cc = OctreeBlob(c.cpu().numpy()).prop("child", 5)
  assert (cc[cc >= 0] == np.arange(out.nnum_nempty[5])).all() and (cc >= 0).sum() == out.nnum_nempty[5]
  assert stale.sum() > 0
  merged = oc.nn.octree_batch([c])
  assert np.array_equal(merged.cpu().numpy(), orc.octree_batch([c.cpu().numpy()]))
  with pytest.raises(ValueError):
    oc.nn.octree_dropout(octree, 9, 0.3)
  with pytest.raises(ValueError):
    oc.nn.octree_dropout(octree, 5, 0.3, flags=torch.zeros(3, dtype=torch.uint8))
