"""Pins of the oracle's trilinear-stencil functions (bilinear_neigh / bilinear_xyz,
octree/octree/octree_nn.cpp:83-108, 476-530) and of octree_gather / gatherbk / mask
(octree_nn.cu:756-818), CPU only.  The stencils are checked against the compiled reference and
through the reference's own consistency test (octree/test/test_octree_nn.cpp:23-84)."""
import numpy as np
import pytest

from oracle.checker import OctreeBlob, make_points_blob


@pytest.fixture(scope="module")
def batches(orc, samples, synthetic):
  out = [orc.octree_batch([samples["octree_1"]]), orc.octree_batch([samples[n] for n in ("octree_2", "octree_1")])]
  pb = make_points_blob(*synthetic.shape_cloud(3000, 17)[:2])
  out.append(orc.octree_batch([orc.points2octree(pb, 6, 2, key2xyz=True), orc.points2octree(pb, 6, 2, key2xyz=True)]))
  return [OctreeBlob(b) for b in out]


def stencil(orc_or_ref, b, d):
  return orc_or_ref.bilinear_neigh(b.prop("neigh", d).reshape(-1), b.prop("child", d), int(b.nnum[d + 1]))


def test_table_and_stencils_equal_the_compiled_reference(orc, ref, batches):
  assert np.array_equal(orc.get_bilinear(), ref.get_bilinear())
  for b in batches:
    for d in range(1, b.depth):
      if b.nnum[d + 1] == 0:
        continue
      got, exp = stencil(orc, b, d), stencil(ref, b, d)
      assert np.array_equal(got, exp), d
      assert (got != -7).all()          # every child row was written
      keys = b.prop("key", d + 1)
      xo, fo = orc.bilinear_xyz(keys, d, d + 1)
      xr, fr = ref.bilinear_xyz(keys, d, d + 1)
      assert np.array_equal(xo, xr) and np.array_equal(fo, fr)
      # two levels apart, as the decoder's skip connections ask for
      if d >= 2:
        xo, fo = orc.bilinear_xyz(keys, d - 1, d + 1)
        xr, fr = ref.bilinear_xyz(keys, d - 1, d + 1)
        assert np.array_equal(xo, xr) and np.array_equal(fo, fr)


def test_reference_consistency_check(orc, batches):
  """octree/test/test_octree_nn.cpp:23-84 on octree_1, depth 4 (and on every other level and
  batch): the corner weights follow from the key geometry, and the stencil from the neighbour
  table equals the stencil from coordinates looked up by key."""
  weights = np.array([27, 9, 9, 9, 3, 3, 3, 1])
  for b in batches:
    assert b.key2xyz
    for d in range(1, b.depth):
      n1 = int(b.nnum[d + 1])
      if n1 == 0:
        continue
      bidx = stencil(orc, b, d)
      key0, key1 = b.prop("key", d), b.prop("key", d + 1)
      c0 = key0.view(np.uint16).reshape(-1, 4)[:, :3].astype(np.float32) + 0.5
      c1 = (key1.view(np.uint16).reshape(-1, 4)[:, :3].astype(np.float32) + 0.5) / 2.0
      for k in range(8):
        j = bidx[:, k]
        ok = j >= 0
        dis = np.abs(c0[j[ok]] - c1[ok])
        assert (dis < 1.0).all()
        assert (np.prod(((1 - dis) * 4).astype(np.int32), axis=1) == weights[k]).all()
      xyz10, _ = orc.bilinear_xyz(key1, d, d + 1)
      key10 = orc.xyz2key(xyz10.reshape(-1), d)
      key_octree = orc.xyz2key(key0, d)
      sidx = orc.search_key(key_octree, key10).reshape(-1, 8)
      # Where the two agree: a corner beyond the upper face (coordinate 2^d) has no node in the
      # neighbour table, and its key wraps around; at the lower face the coordinate form
      # truncates -0.25 to cell 0 and so names cells 0 and 1 where the table names -1 and 0
      # (the reference's test octree does not touch that face).  Everywhere else: equal.
      coords = xyz10.reshape(-1).view(np.uint16).reshape(-1, 8, 4)[:, :, :3]
      inside = (coords < (1 << d)).all(axis=2)
      off_low_face = (key1.view(np.uint16).reshape(-1, 4)[:, :3] >= 1).all(axis=1)
      assert (bidx[~inside & off_low_face[:, None]] == -1).all()
      sel = inside & off_low_face[:, None]
      assert sel.any() and np.array_equal(sidx[sel], bidx[sel])


def test_gather_mask_closed_forms(orc):
  rng = np.random.default_rng(5)
  btm = rng.standard_normal((5, 40)).astype(np.float32)
  idx = rng.integers(-1, 40, 300).astype(np.int32)          # repeated targets, some -1
  top = orc.octree_gather(btm, idx)
  exp = np.where(idx[None, :] >= 0, btm[:, np.maximum(idx, 0)], 0.0)
  assert np.array_equal(top, exp)
  assert np.array_equal(top, orc.pad(btm, idx, 0.0))
  y = rng.standard_normal((5, 300)).astype(np.float32)
  back = orc.octree_gatherbk(y, idx, 40)
  brute = np.zeros((5, 40), np.float64)
  for h in range(300):
    if idx[h] >= 0:
      brute[:, idx[h]] += y[:, h]
  assert np.allclose(back, brute, atol=1e-5)
  # adjoint identity: <gather(x), y> == <x, gatherbk(y)>
  assert abs(float((top.astype(np.float64) * y).sum()) - float((btm.astype(np.float64) * back).sum())) < 1e-3
  label = rng.integers(0, 3, 40).astype(np.int32)
  assert np.array_equal(orc.octree_mask(btm, label, 1), np.where(label[None, :] == 1, 0.0, btm).astype(np.float32))
