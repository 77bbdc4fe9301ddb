"""Pins the oracle's points2octree (Octree::build) restatement."""
import numpy as np
import pytest

from conftest import sha
from oracle.checker import OctreeBlob, make_points_blob


def three_point_cloud():
  # octree/test/test_octree.cpp:17-23
  pts = [0, 0, 0, 1, 1, 0, 1.0625, 1.0625, 0]
  normals = [1, 0, 0, -1, 0, 0, 0, 1, 0]
  features = [1, -1, 2, -2, 3, -3]
  labels = [0, 2, 2]
  return make_points_blob(pts, normals, features, labels)


def test_build_known_answer(orc):
  """octree/test/test_octree.cpp:92-190 (TestOctreeBuild), every literal of it."""
  blob = orc.points2octree(three_point_cloud(), 5, 1, node_dis=True, split_label=True,
                           bbmin=[0, 0, 0], bbmax=[2, 2, 2])
  b = OctreeBlob(blob)
  assert (b.depth, b.full_layer) == (5, 1)
  assert list(b.nnum[:6]) == [1, 8, 16, 16, 16, 16]
  assert list(b.nnum_cum[:7]) == [0, 1, 9, 25, 41, 57, 73]
  assert list(b.nnum_nempty[:6]) == [1, 2, 2, 2, 2, 3]
  keys = [0, 0, 1, 2, 3, 4, 5, 6, 7,
          0, 1, 2, 3, 4, 5, 6, 7, 48, 49, 50, 51, 52, 53, 54, 55,
          0, 1, 2, 3, 4, 5, 6, 7, 384, 385, 386, 387, 388, 389, 390, 391,
          0, 1, 2, 3, 4, 5, 6, 7, 3072, 3073, 3074, 3075, 3076, 3077, 3078, 3079,
          0, 1, 2, 3, 4, 5, 6, 7, 24576, 24577, 24578, 24579, 24580, 24581, 24582, 24583]
  assert np.array_equal(np.concatenate([b.prop("key", d) for d in range(6)]), np.array(keys, np.uint64))
  children = [0, 0, -1, -1, -1, -1, -1, 1, -1,
              0, -1, -1, -1, -1, -1, -1, -1, 1, -1, -1, -1, -1, -1, -1, -1,
              0, -1, -1, -1, -1, -1, -1, -1, 1, -1, -1, -1, -1, -1, -1, -1,
              0, -1, -1, -1, -1, -1, -1, -1, 1, -1, -1, -1, -1, -1, -1, -1,
              0, -1, -1, -1, -1, -1, -1, -1, 1, -1, -1, -1, -1, -1, 2, -1]
  assert np.array_equal(np.concatenate([b.prop("child", d) for d in range(6)]), children)
  f = np.zeros((6, 16), np.float32)
  f[0, 0], f[0, 8], f[1, 14] = 1, -1, 1                    # normals
  f[3, 0], f[3, 8], f[3, 14] = -0.57735, 0.57735, -0.57735  # displacement
  f[4, 0], f[4, 8], f[4, 14] = 1, 2, 3
  f[5, 0], f[5, 8], f[5, 14] = -1, -2, -3
  assert b.channel("feature") == 6
  # the reference test compares against the 6-digit literal 0.57735f with EXPECT_EQ only
  # because 1.1547f * 0.5 rounds there; here: exact for the integers, 1e-6 for the rest
  got = b.prop("feature", 5)
  assert np.array_equal(got[[0, 1, 2, 4, 5]], f[[0, 1, 2, 4, 5]])
  assert np.allclose(got[3], f[3], atol=1e-6) and np.array_equal(got[3] == 0, f[3] == 0)
  assert got[3, 0] == np.float32(-0.5) * np.float32(1.1547)
  labels = [0, -1, -1, -1, -1, -1, -1, -1, 2, -1, -1, -1, -1, -1, 2, -1]
  assert np.array_equal(b.prop("label", 5), np.array(labels, np.float32))
  split = [1, 1, 0, 0, 0, 0, 0, 1, 0,
           1, 0, 0, 0, 0, 0, 0, 0, 1, 0, 0, 0, 0, 0, 0, 0,
           1, 0, 0, 0, 0, 0, 0, 0, 1, 0, 0, 0, 0, 0, 0, 0,
           1, 0, 0, 0, 0, 0, 0, 0, 1, 0, 0, 0, 0, 0, 0, 0,
           1, 0, 0, 0, 0, 0, 0, 0, 1, 0, 0, 0, 0, 0, 1, 0]
  assert np.array_equal(np.concatenate([b.prop("split", d) for d in range(6)]), np.array(split, np.float32))


def test_sample_fixtures_match_reference_md5(samples):
  """pytorch/test/test_octree_grow.py:22-24 quotes the MD5 of sample octree_2."""
  import hashlib
  assert hashlib.md5(samples["octree_2"].tobytes()).hexdigest().upper() == "FEB7C4AF43669EB0FC62632C71D1C938"


def test_sample_headers(samples):
  # octree/octree/octree_samples.cpp: octree_1 holds one point, depth 5, full layer 2
  b = OctreeBlob(samples["octree_1"])
  assert (b.depth, b.full_layer, b.channel("feature")) == (5, 2, 3)
  assert list(b.nnum[:6]) == [1, 8, 64, 8, 8, 8]
  b2 = OctreeBlob(samples["octree_2"])
  assert int(b2.nnum[4]) == 144  # pytorch/test/test_octree_conv.py:13 (152 = 8 + 144)
  for k, s in samples.items():
    assert OctreeBlob(s).size == s.size, k


def brute_force_structure(pts, depth, full_layer):
  """Independent construction: dictionary of occupied voxels per depth."""
  cells = np.floor((pts.astype(np.float32) - np.float32(-1)) * np.float32((1 << depth) / 2.0)).astype(np.int64)
  occ = [None] * (depth + 1)
  occ[depth] = {tuple(c) for c in cells}
  for d in range(depth - 1, -1, -1):
    occ[d] = {(x >> 1, y >> 1, z >> 1) for (x, y, z) in occ[d + 1]}

  def morton(c, d):
    k = 0
    for i in range(d):
      k |= ((c[0] >> i) & 1) << (3 * i + 2) | ((c[1] >> i) & 1) << (3 * i + 1) | ((c[2] >> i) & 1) << (3 * i)
    return k
  keys, children = [], []
  for d in range(depth + 1):
    if d <= full_layer:
      k = list(range(8 ** d))
    else:
      parents = sorted(morton(c, d - 1) for c in occ[d - 1])
      k = [(p << 3) | o for p in parents for o in range(8)]
    occ_keys = sorted(morton(c, d) for c in occ[d])
    rank = {key: i for i, key in enumerate(occ_keys)}
    if d < full_layer:
      ch = list(range(8 ** d))
    elif d == depth and depth == full_layer:
      ch = [-1] * len(k)
    else:
      ch = [rank.get(key, -1) for key in k]
    keys.append(np.array(k, np.uint64))
    children.append(np.array(ch, np.int32))
  return keys, children


@pytest.mark.parametrize("seed,n,depth,fd", [(0, 200, 4, 2), (1, 1500, 6, 2), (2, 50, 5, 1), (3, 1, 5, 2),
                                             (4, 3000, 3, 3), (5, 700, 7, 3)])
def test_build_vs_brute_force(orc, seed, n, depth, fd):
  rng = np.random.default_rng(seed)
  pts = rng.uniform(-0.999, 0.999, (n, 3)).astype(np.float32)
  nrm = rng.standard_normal((n, 3)).astype(np.float32)
  b = OctreeBlob(orc.points2octree(make_points_blob(pts, nrm), depth, fd))
  keys, children = brute_force_structure(pts, depth, fd)
  for d in range(depth + 1):
    assert np.array_equal(b.prop("key", d), keys[d]), d
    assert np.array_equal(b.prop("child", d), children[d]), d
  # finest-level signal: normalised sum of the normals of the points of each voxel
  if depth > fd:
    cells = np.floor((pts - np.float32(-1)) * np.float32((1 << depth) / 2.0)).astype(np.int64)
    feat = b.prop("feature", depth)
    key_d = b.prop("key", depth)
    child_d = b.prop("child", depth)
    lookup = {int(k): i for i, k in enumerate(key_d)}
    acc = {}
    for c, v in zip(cells, nrm):
      k = 0
      for i in range(depth):
        k |= ((int(c[0]) >> i) & 1) << (3 * i + 2) | ((int(c[1]) >> i) & 1) << (3 * i + 1) | ((int(c[2]) >> i) & 1) << (3 * i)
      acc[k] = acc.get(k, np.zeros(3)) + v.astype(np.float64)
    for k, v in acc.items():
      node = lookup[k]
      assert child_d[node] >= 0
      nv = v / max(np.linalg.norm(v), 1e-30)
      if np.linalg.norm(v) > 1e-4:
        assert np.allclose(feat[:, node], nv, atol=2e-5)
    assert np.all(feat[:, child_d < 0] == 0)


def test_invariants(orc, synthetic):
  pts, nrm, _ = synthetic.shape_cloud(4000, 123)
  b = OctreeBlob(orc.points2octree(make_points_blob(pts, nrm), 7, 2))
  for d in range(3, 8):
    k, kp = b.prop("key", d), b.prop("key", d - 1)
    cp = b.prop("child", d - 1)
    assert b.nnum[d] == 8 * b.nnum_nempty[d - 1]
    assert np.all(np.diff(k.astype(np.int64)) > 0)
    parents = kp[cp >= 0]
    assert np.array_equal(k >> np.uint64(3), np.repeat(parents, 8))
    c = b.prop("child", d)
    assert np.array_equal(c[c >= 0], np.arange(b.nnum_nempty[d]))


FLAG_CASES = [dict(), dict(node_dis=True), dict(split_label=True), dict(save_pts=True),
              dict(key2xyz=True), dict(node_dis=True, split_label=True, save_pts=True, key2xyz=True)]


@pytest.mark.parametrize("case", range(len(FLAG_CASES)))
def test_build_vs_compiled_reference(orc, ref, case):
  kw = FLAG_CASES[case]
  rng = np.random.default_rng(10 + case)
  for trial in range(4):
    n = int(rng.integers(1, 3000))
    pts = rng.uniform(-0.999, 0.999, (n, 3)).astype(np.float32)
    nrm = rng.standard_normal((n, 3)).astype(np.float32) if trial != 1 else None
    feat = rng.uniform(0, 1, (n, 2)).astype(np.float32) if trial >= 1 else None
    lab = rng.integers(-1, 4, n).astype(np.float32) if trial == 2 else None
    pb = make_points_blob(pts, nrm, feat, lab)
    depth = int(rng.integers(2, 10))
    fd = int(rng.integers(1, min(depth, 3) + 1))
    assert np.array_equal(orc.points2octree(pb, depth, fd, **kw), ref.points2octree(pb, depth, fd, **kw))


def test_golden_config1(orc, synthetic, hashes):
  pts, nrm, _ = synthetic.sphere_cloud(3000, 0)
  pb = make_points_blob(pts, nrm)
  assert sha(pb) == hashes["cfg1"]["input"], "the seeded generator drifted"
  z = np.load(__import__("os").path.join(__import__("conftest").GOLDEN, "cfg1_octree.npz"))
  single = orc.points2octree(pb, 5, 2)
  assert np.array_equal(single, z["octree"])
  assert sha(orc.octree_batch([single])) == hashes["cfg1"]["batch"]


def test_unsupported_is_reported(orc):
  # trimming reads the per-node normal error, which exists only for clouds with normals
  pb = make_points_blob([[0, 0, 0]])
  with pytest.raises(RuntimeError):
    orc.points2octree(pb, 5, 2, adaptive=True)


def test_adaptive_known_answer(orc):
  """octree/test/test_octree.cpp:196-331 (TestOctreeTrim), every literal of it."""
  blob = orc.points2octree(three_point_cloud(), 5, 1, node_dis=True, split_label=True, adaptive=True,
                           adp_depth=3, th_normal=5.0, th_distance=3.0, bbmin=[0, 0, 0], bbmax=[2, 2, 2])
  b = OctreeBlob(blob)
  assert (b.depth, b.full_layer, b.adp_layer) == (5, 1, 3)
  assert list(b.nnum[:6]) == [1, 8, 16, 16, 16, 8]
  assert list(b.nnum_cum[:7]) == [0, 1, 9, 25, 41, 57, 65]
  assert list(b.nnum_nempty[:6]) == [1, 2, 2, 2, 1, 1]
  g8 = list(range(8))
  keys = [0] + g8 + g8 + list(range(48, 56)) + g8 + list(range(384, 392)) + g8 + list(range(3072, 3080)) + g8
  assert np.concatenate([b.prop("key", d) for d in range(6)]).tolist() == keys
  m7 = [-1] * 7
  children = ([0, 0, -1, -1, -1, -1, -1, 1, -1] + [0] + m7 + [1] + m7 + [0] + m7 + [1] + m7 +
              [0] + m7 + [-1] + m7 + [0] + m7)
  assert np.concatenate([b.prop("child", d) for d in range(6)]).tolist() == children
  assert b.channel("feature") == 6
  z7, z15 = [0.0] * 7, [0.0] * 15
  s = 0.707107
  f0 = [0, 1.0, 0, -0.180422, 2.0, -2.0]
  f1 = ([1.0, 0, 0, 0, 0, 0, -s, 0] + [0, 0, 0, 0, 0, 0, s, 0] + [0.0] * 8 + [-0.57735] + z7 +
        [1.0, 0, 0, 0, 0, 0, 2.5, 0] + [-1.0, 0, 0, 0, 0, 0, -2.5, 0])
  f2 = ([1.0] + z7 + [-s] + z7 + [0.0] * 8 + [s] + z7 + [0.0] * 16 + [-0.57735] + z15 +
        [1.0] + z7 + [2.5] + z7 + [-1.0] + z7 + [-2.5] + z7)
  f5 = [1.0] + z7 + [0.0] * 16 + [-0.57735] + z7 + [1.0] + z7 + [-1.0] + z7
  for d, want in enumerate([f0, f1, f2, f2, f2, f5]):
    np.testing.assert_allclose(b.prop("feature", d).reshape(-1), np.float32(want), rtol=1e-5, atol=1e-6)
  l7 = [-1.0] * 7
  labels = ([2.0, 0, -1, -1, -1, -1, -1, 2.0, -1] + ([0.0] + l7 + [2.0] + l7) * 3 + [0.0] + l7)
  assert np.concatenate([b.prop("label", d) for d in range(6)]).tolist() == labels
  s7 = [0.0] * 7
  split = ([1.0, 1.0, 0, 0, 0, 0, 0, 1.0, 0] + ([1.0] + s7 + [1.0] + s7) * 2 + [1.0] + s7 + [2.0] + s7 +
           [1.0] + s7)
  assert np.concatenate([b.prop("split", d) for d in range(6)]).tolist() == split


ADAPTIVE_CASES = [
    dict(adaptive=True, node_dis=True, split_label=True),
    dict(adaptive=True, node_dis=True, split_label=True, extrapolate=True),
    dict(adaptive=True),
    dict(node_feature=True),
    dict(node_feature=True, node_dis=True, extrapolate=True, split_label=True),
    dict(node_feature=True, save_pts=True, node_dis=True),
    dict(adaptive=True, node_dis=True, key2xyz=True, extrapolate=True, split_label=True),
]


def smooth_cloud(rng, n, kind):
  """Points on an ellipsoid or on a tilted plane: smooth enough for the trimming to act."""
  if kind == 0:
    u = rng.standard_normal((n, 3))
    u /= np.linalg.norm(u, axis=1, keepdims=True)
    ax = np.array([1, 0.6, 0.4])
    pts, nrm = u * 0.8 * ax, u / ax
  else:
    pts = rng.uniform(-0.9, 0.9, (n, 3))
    pts[:, 2] = 0.3 * pts[:, 0] + 0.1
    nrm = np.tile(np.array([[-0.3, 0, 1.0]]), (n, 1))
  nrm = nrm / np.linalg.norm(nrm, axis=1, keepdims=True)
  return pts.astype(np.float32), nrm.astype(np.float32)


@pytest.mark.parametrize("case", range(len(ADAPTIVE_CASES)))
def test_adaptive_build_vs_compiled_reference(orc, ref, case):
  """All-depth signals, error metrics, extrapolation and trimming (octree.cpp:454-806, 958-1178)
  byte for byte against the compiled reference."""
  kw = ADAPTIVE_CASES[case]
  rng = np.random.default_rng(50 + case)
  for trial in range(5):
    n = int(rng.integers(200, 5000))
    pts, nrm = smooth_cloud(rng, n, trial % 2)
    feat = rng.uniform(0, 1, (n, 2)).astype(np.float32) if trial >= 2 else None
    lab = rng.integers(-1, 4, n).astype(np.float32) if trial >= 3 else None
    if trial == 4:
      lab = np.where(lab > 0, lab * 700 + 5, lab).astype(np.float32)   # label values beyond any small table
    pb = make_points_blob(pts, nrm, feat, lab)
    depth = int(rng.integers(4, 8))
    fd = int(rng.integers(1, 3))
    extra = dict(adp_depth=int(rng.integers(fd + 1, depth + 1)), th_normal=float(rng.choice([0.1, 0.3, 5.0])),
                 th_distance=float(rng.choice([0.5, 2.0, 3.0])))
    a = orc.points2octree(pb, depth, fd, **extra, **kw)
    b = ref.points2octree(pb, depth, fd, **extra, **kw)
    assert np.array_equal(a, b)


def test_adaptive_golden(orc, hashes):
  """The committed hash was written from the compiled reference (tests/golden/make_golden.py)."""
  rng = np.random.default_rng(77)
  pts, nrm = smooth_cloud(rng, 4000, 0)
  pb = make_points_blob(pts, nrm)
  assert sha(pb) == hashes["adaptive"]["input"], "the seeded generator drifted"
  blob = orc.points2octree(pb, 6, 2, node_dis=True, split_label=True, adaptive=True, adp_depth=4,
                           th_normal=0.1, th_distance=2.0)
  assert sha(blob) == hashes["adaptive"]["octree"]


def test_golden_config5(orc, synthetic, hashes):
  """BASELINE config 5 inputs at full size: 16 adaptive octrees at depth 7, merged."""
  blobs = [make_points_blob(*synthetic.shape_cloud(50000, 300 + i)[:2]) for i in range(16)]
  assert sha(np.concatenate(blobs)) == hashes["cfg5"]["input"], "the seeded generator drifted"
  singles = [orc.points2octree(b, 7, 2, node_dis=True, split_label=True, adaptive=True, adp_depth=4,
                               th_normal=0.1, th_distance=2.0) for b in blobs]
  assert sha(singles[0]) == hashes["cfg5"]["first_single"]
  assert sha(orc.octree_batch(singles)) == hashes["cfg5"]["batch"]
