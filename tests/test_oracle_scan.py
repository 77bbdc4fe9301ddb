"""octree_scan (ScanOctree, octree/octree/transform_octree.cpp:11-297): the C restatement
against the compiled reference on seeded octrees and view directions, plus what the
definition fixes without either."""
import numpy as np
import pytest

from oracle.checker import OctreeBlob, make_points_blob


def sphere_octree(orc, n, seed, depth, **kw):
  rng = np.random.default_rng(seed)
  u = rng.standard_normal((n, 3))
  u /= np.linalg.norm(u, axis=1, keepdims=True)
  feat = rng.uniform(0, 1, (n, 2)).astype(np.float32)
  lab = rng.integers(0, 5, n).astype(np.float32)
  pb = make_points_blob((u * 0.8).astype(np.float32), u.astype(np.float32), feat, lab)
  return orc.points2octree(pb, depth, 2, **kw)


CASES = [dict(), dict(node_dis=True, split_label=True), dict(node_feature=True, split_label=True),
         dict(key2xyz=True), dict(adaptive=True, node_dis=True, split_label=True, adp_depth=3)]


@pytest.mark.parametrize("case", range(len(CASES)))
def test_scan_vs_compiled_reference(orc, ref, case):
  rng = np.random.default_rng(900 + case)
  for trial in range(6):
    blob = sphere_octree(orc, int(rng.integers(500, 6000)), 10 * case + trial, int(rng.integers(4, 7)), **CASES[case])
    n_axis = 1 + trial % 3
    axis = rng.standard_normal((n_axis, 3)).astype(np.float32)
    axis /= np.linalg.norm(axis, axis=1, keepdims=True)
    if trial == 4:
      axis[0] = [0, 0, 1]      # the rotation to the view frame degenerates to the identity
    if trial == 5:
      axis[0] = [0, 0, -1]
    scale = float(rng.choice([1.0, 0.5, 2.0]))
    a = orc.octree_scan(blob, axis, scale)
    b = ref.octree_scan(blob, axis, scale)
    assert np.array_equal(a, b), (case, trial)


def test_scan_keeps_only_what_faces_the_view(orc):
  """Closed form: seen along -z (view axis (0,0,-1)... the kept leaves have normals with a
  negative component along the axis, at most one per pixel column, and every kept node of a
  level has a kept parent; the structure stays a valid octree."""
  blob = sphere_octree(orc, 5000, 3, 5)
  axis = np.float32([[0, 0, 1]])
  out = OctreeBlob(orc.octree_scan(blob, axis, 1.0))
  src = OctreeBlob(blob)
  assert list(out.nnum[:3]) == list(src.nnum[:3])
  for d in range(1, 6):
    assert out.nnum[d] == 8 * out.nnum_nempty[d - 1]
    c = out.prop("child", d)
    assert np.array_equal(c[c >= 0], np.arange(out.nnum_nempty[d]))
  c5 = out.prop("child", 5)
  nz = out.prop("feature", 5)[2]
  assert (nz[c5 >= 0] < 0).all() and 0 < out.nnum_nempty[5] < src.nnum_nempty[5]
  # one kept leaf per (x, y) column at most: along +z the pixel of a node is its (x, y)
  k = out.prop("key", 5)[c5 >= 0]
  from oracle.checker import Checker
  xyz = Checker("orc").key2xyz(k, 5)
  cols = (xyz & 0xffff).astype(np.int64) * 65536 + ((xyz >> 16) & 0xffff).astype(np.int64)
  assert len(np.unique(cols)) == len(cols)
  # dropped nodes carry zero features and label -1
  f5 = out.prop("feature", 5)
  assert (f5[:, c5 < 0] == 0).all() and (out.prop("label", 5)[c5 < 0] == -1).all()
