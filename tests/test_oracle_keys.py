"""Pins the oracle's key math against closed forms and the literal vectors of the
reference's own tests."""
import numpy as np

from oracle.checker import OctreeBlob


def pack(x, y, z, i):
  return (np.uint64(x) | (np.uint64(y) << np.uint64(16)) | (np.uint64(z) << np.uint64(32))
          | (np.uint64(i) << np.uint64(48)))


def interleave(x, y, z, depth):
  """Bit i of x, y, z lands at bits 3i+2, 3i+1, 3i (octree/octree/octree_nn.cpp:551-560)."""
  k = 0
  for i in range(depth):
    k |= ((x >> i) & 1) << (3 * i + 2) | ((y >> i) & 1) << (3 * i + 1) | ((z >> i) & 1) << (3 * i)
  return k


def test_xyz2key_literals(orc):
  # caffe/src/caffe/test/test_octree_util.cpp:255-271 (depth 5):
  # (0,0,0,id 1) -> 0, (1,1,1,id 2) -> 7, (1,2,3,id 0) -> 29; the id travels unchanged
  xyz = np.array([pack(0, 0, 0, 1), pack(1, 1, 1, 2), pack(1, 2, 3, 0)], np.uint64)
  key = orc.xyz2key(xyz, 5)
  assert [int(k) & 0xFFFFFFFFFFFF for k in key] == [0, 7, 29]
  assert [int(k) >> 48 for k in key] == [1, 2, 0]


def test_xyz2key_closed_form_and_round_trip(orc):
  rng = np.random.default_rng(0)
  for depth in (1, 5, 8, 13, 16):
    n = 500
    x, y, z = (rng.integers(0, 1 << depth, n) for _ in range(3))
    ids = rng.integers(0, 1 << 15, n)
    xyz = np.array([pack(a, b, c, d) for a, b, c, d in zip(x, y, z, ids)], np.uint64)
    key = orc.xyz2key(xyz, depth)
    exp = np.array([interleave(int(a), int(b), int(c), depth) | (int(d) << 48)
                    for a, b, c, d in zip(x, y, z, ids)], np.uint64)
    assert np.array_equal(key, exp)
    assert np.array_equal(orc.key2xyz(key, depth), xyz)
    assert np.array_equal(orc.key2idx(key), ids.astype(np.int32))


def test_xyz_key_64_literal(orc):
  # pytorch/test/test_octree_key.py:45-52: keys longer than 32 bits (depth 13)
  xyz = np.array([pack(2049, 4095, 8011, 1), pack(511, 4095, 8011, 0)], np.uint64)
  key = orc.xyz2key(xyz, 13)
  assert (int(key[0]) & 0xFFFFFFFFFFFF) >= (1 << 32)
  assert np.array_equal(orc.key2xyz(key, 13), xyz)


def test_decode_literal(orc, samples):
  # pytorch/test/test_octree_key.py:9-24: depth-5 xyz of two octree_1 in a batch
  octree = orc.octree_batch([samples["octree_1"], samples["octree_1"]])
  b = OctreeBlob(octree)
  assert b.key2xyz
  xyz = b.prop("key", 5)
  gt = [(16, 16, 16), (16, 16, 17), (16, 17, 16), (16, 17, 17), (17, 16, 16), (17, 16, 17),
        (17, 17, 16), (17, 17, 17)]
  exp = np.array([pack(x, y, z, i) for i in (0, 1) for (x, y, z) in gt], np.uint64)
  assert np.array_equal(xyz, exp)
  key = orc.xyz2key(xyz, 5)
  assert np.array_equal(orc.key2xyz(key, 5), xyz)


def test_search_key_literal(orc, samples):
  # pytorch/test/test_octree_key.py:31-43
  octree = orc.octree_batch([samples["octree_1"], samples["octree_1"]])
  b = OctreeBlob(octree)
  keys = orc.xyz2key(b.prop("key", 5), 5)
  assert np.array_equal(np.sort(keys), keys)
  q = np.array([28673, 281474976739335, 10], np.uint64)
  assert np.array_equal(orc.search_key(keys, q), [1, 15, -1])
  child = b.prop("child", 5)
  keys_ne = keys[child >= 0]
  q = np.array([28672, 28673, 281474976739328, 10], np.uint64)
  assert np.array_equal(orc.search_key(keys_ne, q), [0, -1, 1, -1])


def test_search_key_vs_searchsorted(orc):
  rng = np.random.default_rng(3)
  keys = np.unique(rng.integers(0, 1 << 40, 3000).astype(np.uint64))
  q = np.concatenate([keys[::7], rng.integers(0, 1 << 40, 500).astype(np.uint64)])
  pos = np.searchsorted(keys, q)
  exp = np.where((pos < keys.size) & (keys[np.minimum(pos, keys.size - 1)] == q), pos, -1)
  assert np.array_equal(orc.search_key(keys, q), exp.astype(np.int32))


def test_generate_key_and_label(orc):
  # generate_key_full = packed xyz of the Morton index; children keys append one bit per axis
  for depth in (1, 2, 3):
    full = orc.generate_key_full(depth, 2)
    n = 8 ** depth
    exp = []
    for b in range(2):
      for k in range(n):
        x = y = z = 0
        for i in range(depth):
          x |= ((k >> (3 * i + 2)) & 1) << i
          y |= ((k >> (3 * i + 1)) & 1) << i
          z |= ((k >> (3 * i)) & 1) << i
        exp.append(pack(x, y, z, b))
    assert np.array_equal(full, np.array(exp, np.uint64))
  key = orc.generate_key_full(2, 2)
  child = np.full(key.size, -1, np.int32)
  child[[3, 70, 100]] = [0, 1, 2]
  kc = orc.generate_key_child(key, child, 24)
  assert np.array_equal(orc.xyz2key(kc, 3)[:8] & np.uint64(0xFFFFFFFFFFFF),
                        (np.uint64(3) << np.uint64(3)) + np.arange(8, dtype=np.uint64))
  assert np.all(orc.key2idx(kc)[8:] == 1)
  lab, n = orc.generate_label(np.array([1, 0, 1, 2, 1], np.int32), 1)
  assert n == 3 and np.array_equal(lab, [0, -1, 1, -1, 2])


def test_tables_closed_form(orc):
  # ni of a kernel shape = the 3x3x3 table restricted to the shape's taps
  ni3 = orc.get_ni([3, 3, 3]).reshape(8, 27)
  for s in range(8):
    i, j, k = s >> 2, (s >> 1) & 1, s & 1
    for t in range(27):
      x, y, z = t // 9, (t // 3) % 3, t % 3
      assert ni3[s, t] == ((x + i) << 4 | (y + j) << 2 | (z + k))
  taps = {(1, 1, 1): [13], (2, 2, 2): [13, 14, 16, 17, 22, 23, 25, 26], (3, 1, 1): [4, 13, 22],
          (1, 3, 1): [10, 13, 16], (1, 1, 3): [12, 13, 14], (3, 3, 1): [1, 4, 7, 10, 13, 16, 19, 22, 25],
          (3, 1, 3): [3, 4, 5, 12, 13, 14, 21, 22, 23], (1, 3, 3): list(range(9, 18))}
  for ks, t in taps.items():
    assert np.array_equal(orc.get_ni(list(ks)).reshape(8, -1), ni3[:, t])
