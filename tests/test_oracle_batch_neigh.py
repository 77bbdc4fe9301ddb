"""Pins the oracle's octree_batch (merge_octrees) and neighbour tables."""
import numpy as np
import pytest

from oracle.checker import OctreeBlob, make_points_blob


def test_property_literals(orc, samples):
  """pytorch/test/test_octree_property.py:9-54 on a batch of two octree_1."""
  b = OctreeBlob(orc.octree_batch([samples["octree_1"]] * 2))
  assert np.array_equal(orc.key2idx(b.prop("key", 5)), [0] * 8 + [1] * 8)
  f = np.zeros((3, 16), np.float32)
  f[:, 0] = f[:, 8] = 3.0 ** 0.5 / 3.0
  assert np.allclose(b.prop("feature", 5), f)
  c = -np.ones(16, np.int32)
  c[0], c[8] = 0, 1
  assert np.array_equal(b.prop("child", 5), c)
  assert list(b.nnum[:6]) == [2, 16, 128, 16, 16, 16]
  assert list(b.nnum_cum[:7]) == [0, 2, 18, 146, 162, 178, 194]
  assert (b.batch_size, b.depth, b.full_layer) == (2, 5, 2)
  assert b.channel("neigh") == 8 and b.location("neigh") == -1


def test_merge_relations(orc, samples):
  """caffe/src/caffe/test/test_octree_util.cpp:15-118: keys get the octree index, child
  links are offset by the non-empty counts of the octrees before, features interleave."""
  for names in (["octree_1", "octree_2"], ["octree_2", "octree_2", "octree_1"], ["octree_3", "octree_4"],
                ["octree_6", "octree_5"][::-1] if False else ["octree_5", "octree_5"]):
    srcs = [OctreeBlob(samples[n]) for n in names]
    m = OctreeBlob(orc.octree_batch([samples[n] for n in names]))
    D = m.depth
    for d in range(D + 1):
      assert m.nnum[d] == sum(s.nnum[d] for s in srcs)
      assert m.nnum_nempty[d] == sum(s.nnum_nempty[d] for s in srcs)
      off = ne = 0
      mk, mc = m.prop("key", d), m.prop("child", d)
      for i, s in enumerate(srcs):
        n = int(s.nnum[d])
        sk, sc = s.prop("key", d), s.prop("child", d)
        assert np.array_equal(mk[off:off + n] & np.uint64(0xFFFFFFFFFFFF), sk & np.uint64(0xFFFFFFFFFFFF))
        assert np.all((mk[off:off + n] >> np.uint64(48)) == i)
        assert np.array_equal(mc[off:off + n], np.where(sc < 0, -1, sc + ne))
        for name in ("feature", "label", "split"):
          if m.has(name) and (m.location(name) == -1 or d == D):
            mp = np.atleast_2d(m.prop(name, d))
            sp = np.atleast_2d(s.prop(name, d))
            assert np.array_equal(mp[:, off:off + n], sp), (name, d)
        off += n
        ne += int(s.nnum_nempty[d])


def brute_force_neigh(b, d):
  """Definition of the table: slot (x,y,z) of a sibling group holds the node at offset
  (x-1, y-1, z-1) from sibling 0, found through a dictionary (octree, x, y, z) -> index
  (the hash formulation of caffe/src/caffe/util/octree.cpp:330-370)."""
  keys = b.prop("key", d)
  n = keys.size
  if b.key2xyz:
    xs = (keys & np.uint64(0xFFFF)).astype(np.int64)
    ys = ((keys >> np.uint64(16)) & np.uint64(0xFFFF)).astype(np.int64)
    zs = ((keys >> np.uint64(32)) & np.uint64(0xFFFF)).astype(np.int64)
  else:
    m = (keys & np.uint64(0xFFFFFFFFFFFF)).astype(np.int64)
    xs = np.zeros(n, np.int64); ys = np.zeros(n, np.int64); zs = np.zeros(n, np.int64)
    for i in range(d):
      xs |= ((m >> (3 * i + 2)) & 1) << i
      ys |= ((m >> (3 * i + 1)) & 1) << i
      zs |= ((m >> (3 * i)) & 1) << i
  ids = (keys >> np.uint64(48)).astype(np.int64)
  table = {(int(i), int(x), int(y), int(z)): j for j, (i, x, y, z) in enumerate(zip(ids, xs, ys, zs))}
  out = -np.ones((n // 8, 64), np.int32)
  for g in range(n // 8):
    j = 8 * g
    for x in range(4):
      for y in range(4):
        for z in range(4):
          out[g, x * 16 + y * 4 + z] = table.get(
              (int(ids[j]), int(xs[j]) + x - 1, int(ys[j]) + y - 1, int(zs[j]) + z - 1), -1)
  return out


def test_neigh_vs_brute_force(orc, samples, synthetic):
  blobs = [orc.octree_batch([samples["octree_1"], samples["octree_2"], samples["octree_2"]]),
           orc.octree_batch([samples["octree_6"], samples["octree_5"], samples["octree_6"]])]
  pbs = [make_points_blob(*synthetic.shape_cloud(1500, 7 + i)[:2]) for i in range(3)]
  blobs.append(orc.octree_batch([orc.points2octree(p, 6, 2) for p in pbs]))
  blobs.append(orc.octree_batch([orc.points2octree(p, 5, 3, key2xyz=True) for p in pbs]))
  for blob in blobs:
    b = OctreeBlob(blob)
    for d in range(1, b.depth + 1):
      assert np.array_equal(b.prop("neigh", d), brute_force_neigh(b, d)), d


def test_neigh_full_closed_form(orc):
  for depth, batch in ((1, 1), (2, 3), (3, 2)):
    got = orc.calc_neigh_full(depth, batch).reshape(batch, -1, 64)
    n = 8 ** depth
    for bi in range(batch):
      for g in range(n // 8):
        i = 8 * g
        x0 = y0 = z0 = 0
        for t in range(depth):
          x0 |= ((i >> (3 * t + 2)) & 1) << t
          y0 |= ((i >> (3 * t + 1)) & 1) << t
          z0 |= ((i >> (3 * t)) & 1) << t
        for s in range(64):
          x, y, z = x0 + (s >> 4) - 1, y0 + ((s >> 2) & 3) - 1, z0 + (s & 3) - 1
          if min(x, y, z) < 0 or max(x, y, z) >= (1 << depth):
            exp = -1
          else:
            k = 0
            for t in range(depth):
              k |= ((x >> t) & 1) << (3 * t + 2) | ((y >> t) & 1) << (3 * t + 1) | ((z >> t) & 1) << (3 * t)
            exp = k + bi * n
          assert got[bi, g, s] == exp


def test_batch_vs_compiled_reference(orc, ref, samples, synthetic):
  for names in (["octree_1"] * 2, ["octree_1", "octree_2"], ["octree_2", "octree_2", "octree_1"],
                ["octree_1", "octree_2", "octree_2", "octree_1"], ["octree_3", "octree_4"],
                ["octree_5", "octree_5"], ["octree_6"] * 3):
    blobs = [samples[n] for n in names]
    assert np.array_equal(orc.octree_batch(blobs), ref.octree_batch(blobs)), names
  pbs = [make_points_blob(*synthetic.shape_cloud(2000, 50 + i)[:2]) for i in range(5)]
  singles = [ref.points2octree(p, 6, 2) for p in pbs]
  assert np.array_equal(orc.octree_batch(singles), ref.octree_batch(singles))


def test_inconsistent_batch_is_rejected(orc, samples):
  with pytest.raises(RuntimeError):
    orc.octree_batch([samples["octree_1"], samples["octree_3"]])
