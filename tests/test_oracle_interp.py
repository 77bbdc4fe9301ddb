"""Pins the numpy restatement of octree_align and of the point interpolation compositions."""
import numpy as np

from oracle import interp
from oracle.checker import OctreeBlob


def test_align_literals(orc, samples):
  """pytorch/test/test_octree_align.py:13-75, the three cases."""
  one = orc.octree_batch([samples["octree_1"]])
  two = orc.octree_batch([samples["octree_1"], samples["octree_1"]])
  rng = np.random.default_rng(0)
  x16, x8 = rng.random((3, 16), np.float32), rng.random((3, 8), np.float32)
  out, idx = interp.octree_align(orc, x16, two, two, 5)
  assert np.array_equal(out, x16) and np.array_equal(idx, np.arange(16))
  assert np.array_equal(interp.octree_align_grad(np.ones_like(out), idx), np.ones((3, 16)))
  out, idx = interp.octree_align(orc, x8, one, two, 5)
  assert np.array_equal(out, np.concatenate([x8, np.zeros((3, 8), np.float32)], axis=1))
  assert np.array_equal(idx, np.arange(8))
  out, idx = interp.octree_align(orc, x16, two, one, 5)
  assert np.array_equal(out, x16[:, :8]) and np.array_equal(idx, list(range(8)) + [-1] * 8)
  g = interp.octree_align_grad(np.ones_like(out), idx)
  assert np.array_equal(g, np.concatenate([np.ones((3, 8)), np.zeros((3, 8))], axis=1))


def test_trilinear_literal(orc, samples):
  """pytorch/test/test_octree_trilinear.py:9-15."""
  blob = orc.octree_batch([samples["octree_1"], samples["octree_1"]])
  out = interp.octree_trilinear(orc, np.ones((3, 16), np.float32), blob, 4, 5)
  assert out.shape == (3, 16) and np.all(out == 1.0)


def full_layer(orc, samples, depth):
  blob = orc.octree_batch([samples["octree_1"]])   # full_layer 2: depths 1, 2 are full grids
  b = OctreeBlob(blob)
  key = b.prop("key", depth).copy()
  xyz = np.ascontiguousarray(key if b.key2xyz else orc.key2xyz(key, depth)).view(np.int16).reshape(-1, 4)
  return blob, xyz[:, :3].astype(np.float32)


def test_interpolation_closed_forms(orc, samples):
  depth = 2
  blob, centre = full_layer(orc, samples, depth)
  coef = np.float32([[1.0, -2.0, 0.5], [0.25, 0.0, 3.0]])
  data = (coef @ (centre.T + 0.5) + np.float32([[0.1], [-1.0]])).astype(np.float32)   # affine in the voxel centre
  rng = np.random.default_rng(1)
  # interior points (all eight surrounding centres exist): trilinear reproduces an affine function
  p = rng.uniform(0.5, 2 ** depth - 0.5, (200, 3)).astype(np.float32)
  pts = np.concatenate([p, np.zeros((200, 1), np.float32)], axis=1)
  out = interp.octree_trilinear_pts(orc, data, blob, depth, pts)
  assert np.allclose(out, coef @ p.T + np.float32([[0.1], [-1.0]]), atol=1e-5)
  # a point at a voxel centre takes that voxel's value, with either method
  at = np.concatenate([centre + 0.5, np.zeros((centre.shape[0], 1), np.float32)], axis=1)
  assert np.allclose(interp.octree_trilinear_pts(orc, data, blob, depth, at), data, atol=1e-6)
  assert np.array_equal(interp.octree_nearest_pts(orc, data, blob, depth, at), data)
  # nearest: every point of a voxel maps to it; a point of another batch index misses
  q = np.concatenate([centre + rng.uniform(0.01, 0.99, centre.shape).astype(np.float32),
                      np.zeros((centre.shape[0], 1), np.float32)], axis=1)
  assert np.array_equal(interp.octree_nearest_pts(orc, data, blob, depth, q), data)
  q[:, 3] = 1
  assert np.all(interp.octree_nearest_pts(orc, data, blob, depth, q) == 0)
  # near a face only the existing corners count and the weights are renormalised: constants stay
  edge = np.float32([[0.1, 1.3, 2.2, 0], [3.9, 3.95, 0.2, 0]])
  ones = np.ones((1, data.shape[1]), np.float32)
  assert np.allclose(interp.octree_trilinear_pts(orc, ones, blob, depth, edge), 1.0, atol=1e-6)
