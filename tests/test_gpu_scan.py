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
