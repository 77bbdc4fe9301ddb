"""Pins octree_new / octree_grow / octree_update / octree_set_property."""
import hashlib

import numpy as np

from oracle.checker import OctreeBlob


def rebuild_octree_2(impl, samples):
  """The script pytorch/test/test_octree_grow.py:6-19."""
  gt = OctreeBlob(samples["octree_2"])
  depth, channel = 5, 3
  o = impl.octree_new(1, channel, False, 0)
  o = impl.octree_grow(o, 1, True)
  o = impl.octree_grow(o, 2, True)
  for d in range(2, depth + 1):
    label = (gt.prop("child", d) > -1).astype(np.int32)
    o = impl.octree_update(o, label, d, 1)
    if d < depth:
      o = impl.octree_grow(o, d + 1, False)
  return impl.octree_set_property(o, gt.prop("feature", depth), depth)


def test_grow_md5(orc, samples):
  """The MD5 quoted at pytorch/test/test_octree_grow.py:22-24 for the rebuilt octree."""
  o = rebuild_octree_2(orc, samples)
  assert hashlib.md5(o.tobytes()).hexdigest().upper() == "D569D5BB23D34795C5FD81397F56275B"


def test_grown_structure_equals_sample(orc, samples):
  o, gt = OctreeBlob(rebuild_octree_2(orc, samples)), OctreeBlob(samples["octree_2"])
  low48 = np.uint64(0xFFFFFFFFFFFF)  # the samples carry their own id field; compare x, y, z
  for d in range(1, 6):
    assert np.array_equal(o.prop("key", d) & low48, gt.prop("key", d) & low48)
  for d in range(6):
    assert np.array_equal(o.prop("child", d), gt.prop("child", d))
  assert np.array_equal(o.prop("feature", 5), gt.prop("feature", 5))


def test_update_degenerate(orc, samples):
  o = orc.octree_new(2, 1, False, 0)
  o = orc.octree_grow(o, 1, True)
  o = orc.octree_update(o, np.zeros(16, np.int32), 1, 1)  # nothing splits: one node is kept
  b = OctreeBlob(o)
  assert b.nnum_nempty[1] == 1 and b.prop("child", 1)[0] == 0 and np.all(b.prop("child", 1)[1:] == -1)
