"""GPU parity: octree construction, batching, neighbour tables, keys, growth.
Everything integer/byte valued is compared bit for bit with the CPU oracle."""
import hashlib

import numpy as np
import pytest
import torch

from conftest import GOLDEN, sha
from oracle.checker import OctreeBlob, make_points_blob

pytestmark = pytest.mark.gpu


def T(a):
  return torch.from_numpy(np.ascontiguousarray(a))


def three_point_cloud():
  return make_points_blob([0, 0, 0, 1, 1, 0, 1.0625, 1.0625, 0], [1, 0, 0, -1, 0, 0, 0, 1, 0],
                          [1, -1, 2, -2, 3, -3], [0, 2, 2])


def test_build_known_answer_on_gpu(oc, orc):
  """The known-answer cloud of octree/test/test_octree.cpp:92-190 (custom bounding box,
  normals + features + labels, displacement, split labels)."""
  pb = three_point_cloud()
  got = oc.nn._build([T(pb)], False, 5, 1, True, False, True, False, 4, 0.1, 2.0, False, False, False,
                     bbox=([0, 0, 0], [2, 2, 2]))
  exp = orc.points2octree(pb, 5, 1, node_dis=True, split_label=True, bbmin=[0, 0, 0], bbmax=[2, 2, 2])
  assert np.array_equal(got.cpu().numpy(), exp)
  b = OctreeBlob(got.cpu().numpy())
  assert list(b.nnum_nempty[:6]) == [1, 2, 2, 2, 2, 3]
  assert np.array_equal(b.prop("label", 5)[[0, 8, 14]], [0, 2, 2])


def test_build_golden_config1(oc, synthetic, hashes):
  pts, nrm, _ = synthetic.sphere_cloud(3000, 0)
  pb = make_points_blob(pts, nrm)
  assert sha(pb) == hashes["cfg1"]["input"]
  z = np.load(GOLDEN + "/cfg1_octree.npz")
  single = oc.nn.points2octree(T(pb), 5, 2)
  assert np.array_equal(single.cpu().numpy(), z["octree"])
  assert sha(oc.nn.points2octree_batch([T(pb)], 5, 2).cpu().numpy()) == hashes["cfg1"]["batch"]
  assert sha(oc.nn.octree_batch([single]).cpu().numpy()) == hashes["cfg1"]["batch"]


FLAG_CASES = [dict(), dict(node_dis=True), dict(split_label=True), dict(save_pts=True), dict(key2xyz=True),
              dict(node_dis=True, split_label=True, save_pts=True, key2xyz=True)]


@pytest.mark.parametrize("case", range(len(FLAG_CASES)))
def test_build_random_vs_oracle(oc, orc, case):
  kw = FLAG_CASES[case]
  rng = np.random.default_rng(100 + case)
  for trial in range(5):
    n = int(rng.integers(1, 5000))
    pts = rng.uniform(-0.999, 0.999, (n, 3)).astype(np.float32)
    nrm = rng.standard_normal((n, 3)).astype(np.float32) if trial != 1 else None
    feat = rng.uniform(0, 1, (n, 1 + trial % 3)).astype(np.float32) if trial >= 1 else None
    lab = rng.integers(-1, 6, n).astype(np.float32) if trial in (2, 4) else None
    pb = make_points_blob(pts, nrm, feat, lab)
    depth = int(rng.integers(2, 10))
    fd = int(rng.integers(1, min(depth, 3) + 1))
    got = oc.nn.points2octree(T(pb), depth, fd, **kw).cpu().numpy()
    assert np.array_equal(got, orc.points2octree(pb, depth, fd, **kw)), (trial, n, depth, fd, kw)


def test_build_edge_cases(oc, orc):
  rng = np.random.default_rng(7)
  one = make_points_blob([[0.3, -0.2, 0.7]], [[0, 0, 1]])
  same_voxel = make_points_blob(np.full((500, 3), 0.123, np.float32) + rng.uniform(0, 1e-4, (500, 3)).astype(np.float32),
                                rng.standard_normal((500, 3)).astype(np.float32))
  cancelling = make_points_blob([[0.5, 0.5, 0.5], [0.5, 0.5, 0.5]], [[1, 0, 0], [-1, 0, 0]])  # |sum of normals| < 1e-6
  corner = make_points_blob([[-1, -1, -1], [0.9999, 0.9999, 0.9999], [0, 0, 0]], [[1, 0, 0]] * 3)
  for pb in (one, same_voxel, cancelling, corner):
    for depth, fd in ((5, 2), (3, 3), (9, 1), (1, 1), (2, 1)):
      got = oc.nn.points2octree(T(pb), depth, fd, node_dis=True).cpu().numpy()
      assert np.array_equal(got, orc.points2octree(pb, depth, fd, node_dis=True)), (depth, fd)


def test_build_wide_features_and_many_clouds(oc, orc):
  """More feature channels than the leaf kernel stages in LDS, more clouds than one launch
  of the cloud table carries, labels and displacement together."""
  rng = np.random.default_rng(21)
  n = 3000
  pts = rng.uniform(-0.999, 0.999, (n, 3)).astype(np.float32)
  nrm = rng.standard_normal((n, 3)).astype(np.float32)
  feat = rng.uniform(0, 1, (n, 11)).astype(np.float32)
  lab = rng.integers(0, 4, n).astype(np.float32)
  pb = make_points_blob(pts, nrm, feat, lab)
  for kw in (dict(), dict(node_dis=True, save_pts=True)):
    got = oc.nn.points2octree(T(pb), 6, 2, **kw).cpu().numpy()
    assert np.array_equal(got, orc.points2octree(pb, 6, 2, **kw)), kw
  blobs = []
  for i in range(70):
    m = int(rng.integers(1, 400))
    blobs.append(make_points_blob(rng.uniform(-0.999, 0.999, (m, 3)).astype(np.float32),
                                  rng.standard_normal((m, 3)).astype(np.float32)))
  got = oc.nn.points2octree_batch([T(b) for b in blobs], 5, 2).cpu().numpy()
  assert np.array_equal(got, orc.octree_batch([orc.points2octree(b, 5, 2) for b in blobs]))


def test_build_dense_tiles_and_feature_overflow(oc, orc):
  """A signal tile (1024 nodes) stages 256 leaves a round: dense levels take several rounds, with
  labels and a batch's cloud table in LDS beside them; five feature channels are one more than
  the leaf loop keeps in registers while the tile still stages them (at most 8 channels)."""
  rng = np.random.default_rng(33)
  n = 6000
  pts = rng.uniform(-0.999, 0.999, (n, 3)).astype(np.float32)
  nrm = rng.standard_normal((n, 3)).astype(np.float32)
  lab = rng.integers(0, 5, n).astype(np.float32)
  dense = make_points_blob(pts, nrm, rng.uniform(0, 1, (n, 3)).astype(np.float32), lab)
  five = make_points_blob(pts, None, rng.uniform(0, 1, (n, 5)).astype(np.float32), lab)
  for pb in (dense, five):
    for depth, fd in ((4, 2), (5, 3), (4, 1)):   # 4096 / 32768 nodes at the finest level, most of them leaves at depth 4
      got = oc.nn.points2octree(T(pb), depth, fd, node_dis=True).cpu().numpy()
      assert np.array_equal(got, orc.points2octree(pb, depth, fd, node_dis=True)), (depth, fd)
  blobs = []
  for i in range(5):
    m = int(rng.integers(2000, 5000))
    blobs.append(make_points_blob(rng.uniform(-0.999, 0.999, (m, 3)).astype(np.float32),
                                  rng.standard_normal((m, 3)).astype(np.float32),
                                  rng.uniform(0, 1, (m, 2)).astype(np.float32), rng.integers(0, 3, m).astype(np.float32)))
  got = oc.nn.points2octree_batch([T(b) for b in blobs], 4, 2).cpu().numpy()
  assert np.array_equal(got, orc.octree_batch([orc.points2octree(b, 4, 2) for b in blobs]))


def test_build_two_steps_and_ticket_repeat(oc, orc, synthetic):
  """The plan / emit pair gives the blob of the one-call entry point; a first attempt that is
  made to fail from the host is repeated with ticket order and gives the same blob."""
  import ctypes as C
  p, nrm, f = synthetic.room_cloud(60000, 5)
  pb = make_points_blob(p, nrm, f)
  exp = orc.octree_batch([orc.points2octree(pb, 8, 2)])
  cloud = T(pb).cuda()
  L = oc.lib.get()
  hdr = pb[:88].copy()
  bp = oc.lib.BuildParams(depth=8, full_depth=2, adp_depth=4, th_normal=0.1, th_distance=2.0, merged=1)
  ws_bytes = L.ocnn_points2octree_workspace_bytes(60000, 1, 8)
  ws = torch.empty(ws_bytes + 256, dtype=torch.uint8, device="cuda")
  base = (ws.data_ptr() + 255) & ~255
  dev = (C.c_void_p * 1)(cloud.data_ptr())
  hp = (C.c_void_p * 1)(hdr.ctypes.data)
  info = np.zeros(716, np.uint8)
  stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
  oc.lib.call("ocnn_points2octree_plan", dev, hp, 1, C.byref(bp), C.c_void_p(base), C.c_size_t(ws_bytes),
              C.c_void_p(info.ctypes.data), stream)
  size = L.ocnn_info_sizeof_octree(C.c_void_p(info.ctypes.data))
  assert size == exp.size
  out = torch.empty(size, dtype=torch.uint8, device="cuda")
  oc.lib.call("ocnn_points2octree_emit", C.c_void_p(out.data_ptr()), C.c_void_p(info.ctypes.data),
              C.c_void_p(base), C.c_size_t(ws_bytes), stream)
  assert np.array_equal(out.cpu().numpy(), exp)
  # emit without a plan on this workspace is an error, not a crash
  assert L.ocnn_points2octree_emit(C.c_void_p(out.data_ptr()), C.c_void_p(info.ctypes.data), C.c_void_p(base),
                                   C.c_size_t(ws_bytes), stream) != 0

  before = L.ocnn_points2octree_ticket_reruns()
  old = L.ocnn_points2octree_wait_limit(-1)
  try:
    got = oc.nn.points2octree_batch([cloud], 8, 2)
  finally:
    L.ocnn_points2octree_wait_limit(old)
  assert L.ocnn_points2octree_ticket_reruns() == before + 1
  assert np.array_equal(got.cpu().numpy(), exp)
  assert np.array_equal(oc.nn.points2octree_batch([cloud], 8, 2).cpu().numpy(), exp)
  assert L.ocnn_points2octree_ticket_reruns() == before + 1


def test_build_large_tiles(oc, synthetic):
  """More than 2^19 points (the larger sort tile): the structure invariants hold and the blob
  equals the blob of batching the separately built octrees."""
  clouds = []
  for i in range(3):
    p, nrm, f = synthetic.room_cloud(200000, 11 + i)
    clouds.append(T(make_points_blob(p, nrm, f)).cuda())
  fused = oc.nn.points2octree_batch(clouds, 8, 2)
  singles = [oc.nn.points2octree(c, 8, 2) for c in clouds]
  assert torch.equal(fused, oc.nn.octree_batch(singles))
  b = OctreeBlob(fused.cpu().numpy())
  for d in range(3, 9):
    assert b.nnum[d] == 8 * b.nnum_nempty[d - 1]
    c = b.prop("child", d)
    assert np.array_equal(c[c >= 0], np.arange(b.nnum_nempty[d]))


def test_build_rejects_what_it_cannot_do(oc):
  pb = make_points_blob([[0, 0, 0]])          # no normals: trimming has no normal error to read
  with pytest.raises(oc.lib.OcnnError) as e:
    oc.nn.points2octree(T(pb), 5, 2, adaptive=True)
  assert e.value.code == -2
  pb = make_points_blob([[0, 0, 0]], [[1, 0, 0]])
  with pytest.raises(oc.lib.OcnnError) as e:
    oc.nn.points2octree(T(pb), 5, 2, adaptive=True, save_pts=True)
  assert e.value.code == -2
  bad = pb.copy()
  bad[0] = 0
  with pytest.raises(oc.lib.OcnnError) as e:
    oc.nn.points2octree(T(bad), 5, 2)
  assert e.value.code == -6


def test_adaptive_known_answer_on_gpu(oc, orc):
  """octree/test/test_octree.cpp:196-331 (TestOctreeTrim) built on the device."""
  pb = three_point_cloud()
  kw = dict(node_dis=True, split_label=True, adaptive=True, adp_depth=3, th_normal=5.0, th_distance=3.0)
  got = oc.nn._build([T(pb)], False, 5, 1, True, False, True, True, 3, 5.0, 3.0, False, False, False,
                     bbox=([0, 0, 0], [2, 2, 2])).cpu().numpy()
  assert np.array_equal(got, orc.points2octree(pb, 5, 1, bbmin=[0, 0, 0], bbmax=[2, 2, 2], **kw))
  b = OctreeBlob(got)
  assert list(b.nnum[:6]) == [1, 8, 16, 16, 16, 8] and list(b.nnum_nempty[:6]) == [1, 2, 2, 2, 1, 1]
  assert b.prop("split", 4).tolist() == [1.0] + [0.0] * 7 + [2.0] + [0.0] * 7


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
def test_adaptive_build_vs_oracle(oc, orc, case):
  """All-depth signals, error metrics, extrapolation and trimming (octree.cpp:454-806,
  958-1178) on the device: the blob equals the oracle's byte for byte (the oracle equals the
  compiled reference on these very cases)."""
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
    got = oc.nn.points2octree(T(pb), depth, fd, **extra, **kw).cpu().numpy()
    exp = orc.points2octree(pb, depth, fd, **extra, **kw)
    assert got.size == exp.size and np.array_equal(got, exp), (trial, n, depth, fd, extra, kw)


@pytest.mark.parametrize("case", range(len(ADAPTIVE_CASES)))
def test_adaptive_batch_in_one_pass_vs_oracle(oc, orc, case):
  """A batch of clouds through both stages of the builder as ONE octree in merged layout: the
  blob equals merge_octrees over the octrees the oracle builds cloud by cloud.  The clouds
  differ in size and smoothness, so with the loose thresholds some octrees of a batch fall
  under the "keep one node per level" rule of trim_octree (octree.cpp:1055-1073) and others do
  not: that rule is the one step that is taken per octree."""
  kw = ADAPTIVE_CASES[case]   # depth <= 7 below: one key channel also with key2xyz, which merge_octrees needs
  rng = np.random.default_rng(900 + case)
  for trial in range(4):
    n_clouds = int(rng.integers(2, 6))
    depth = int(rng.integers(4, 8))
    fd = int(rng.integers(1, 3))
    extra = dict(adp_depth=int(rng.integers(fd + 1, depth + 1)), th_normal=float(rng.choice([0.1, 0.3, 5.0])),
                 th_distance=float(rng.choice([0.5, 2.0, 3.0])))
    pbs = []
    for c in range(n_clouds):
      n = int(rng.integers(1, 40)) if (trial == 3 and c == 1) else int(rng.integers(200, 5000))
      pts, nrm = smooth_cloud(rng, n, int(rng.integers(0, 2)))
      if c % 2 == 1:   # a rough cloud next to the smooth ones
        nrm = rng.standard_normal((n, 3)).astype(np.float32)
        nrm /= np.linalg.norm(nrm, axis=1, keepdims=True)
      feat = rng.uniform(0, 1, (n, 2)).astype(np.float32) if trial >= 2 else None
      lab = rng.integers(-1, 4, n).astype(np.float32) if trial >= 3 else None
      pbs.append(make_points_blob(pts, nrm, feat, lab))
    got = oc.nn.points2octree_batch([T(pb) for pb in pbs], depth, fd, **extra, **kw).cpu().numpy()
    exp = orc.octree_batch([orc.points2octree(pb, depth, fd, **extra, **kw) for pb in pbs])
    assert got.size == exp.size and np.array_equal(got, exp), (trial, n_clouds, depth, fd, extra, kw)
    if trial == 0:   # a batch of one is still a batch blob (neighbour tables, batch header)
      one = oc.nn.points2octree_batch([T(pbs[0])], depth, fd, **extra, **kw).cpu().numpy()
      assert np.array_equal(one, orc.octree_batch([orc.points2octree(pbs[0], depth, fd, **extra, **kw)]))


def test_adaptive_golden_and_config5_on_gpu(oc, synthetic, hashes):
  """The committed hashes were written from the compiled reference: one small adaptive octree
  and BASELINE config 5's input (16 adaptive octrees at depth 7, merged), built on the device."""
  rng = np.random.default_rng(77)
  pts, nrm = smooth_cloud(rng, 4000, 0)
  pb = make_points_blob(pts, nrm)
  assert sha(pb) == hashes["adaptive"]["input"]
  kw = dict(node_dis=True, split_label=True, adaptive=True, adp_depth=4, th_normal=0.1, th_distance=2.0)
  assert sha(oc.nn.points2octree(T(pb), 6, 2, **kw).cpu().numpy()) == hashes["adaptive"]["octree"]
  blobs = [make_points_blob(*synthetic.shape_cloud(50000, 300 + i)[:2]) for i in range(16)]
  assert sha(np.concatenate(blobs)) == hashes["cfg5"]["input"]
  clouds = [T(b).cuda() for b in blobs]
  assert sha(oc.nn.points2octree(clouds[0], 7, 2, **kw).cpu().numpy()) == hashes["cfg5"]["first_single"]
  assert sha(oc.nn.points2octree_batch(clouds, 7, 2, **kw).cpu().numpy()) == hashes["cfg5"]["batch"]


@pytest.mark.parametrize("cfg,n_clouds,n_pts,depth,seed0", [("cfg2", 32, 10000, 6, 100), ("cfg3", 16, 50000, 7, 200)])
def test_full_size_batches_hash(oc, synthetic, hashes, cfg, n_clouds, n_pts, depth, seed0):
  """BASELINE configs 2 and 3 at full size: the fused build+batch blob and the blob of
  batching separately built octrees both hash to what the compiled reference produced."""
  blobs = [make_points_blob(*synthetic.shape_cloud(n_pts, seed0 + i)[:2]) for i in range(n_clouds)]
  assert sha(np.concatenate(blobs)) == hashes[cfg]["input"]
  clouds = [T(b).cuda() for b in blobs]
  fused = oc.nn.points2octree_batch(clouds, depth, 2)
  assert sha(fused.cpu().numpy()) == hashes[cfg]["batch"]
  singles = [oc.nn.points2octree(c, depth, 2) for c in clouds]
  assert sha(singles[0].cpu().numpy()) == hashes[cfg]["first_single"]
  assert sha(oc.nn.octree_batch(singles).cpu().numpy()) == hashes[cfg]["batch"]


def test_full_size_scene_hash(oc, synthetic, hashes):
  p, n, f = synthetic.room_cloud(250000, 3)
  pb = make_points_blob(p, n, f)
  assert sha(pb) == hashes["cfg4"]["input"]
  cloud = T(pb).cuda()
  assert sha(oc.nn.points2octree(cloud, 9, 2).cpu().numpy()) == hashes["cfg4"]["single"]
  merged = oc.nn.points2octree_batch([cloud], 9, 2)
  assert sha(merged.cpu().numpy()) == hashes["cfg4"]["batch"]
  # size-independent invariants of the structure at full size
  b = OctreeBlob(merged.cpu().numpy())
  for d in range(3, 10):
    assert b.nnum[d] == 8 * b.nnum_nempty[d - 1]
    k = b.prop("key", d).astype(np.int64)
    assert np.all(np.diff(k) > 0)
    c = b.prop("child", d)
    assert np.array_equal(c[c >= 0], np.arange(b.nnum_nempty[d]))


def test_octree_batch_samples(oc, orc, samples):
  for names in (["octree_1"] * 2, ["octree_1", "octree_2"], ["octree_2", "octree_2", "octree_1"],
                ["octree_1", "octree_2", "octree_2", "octree_1"], ["octree_3", "octree_4"],
                ["octree_5", "octree_5"], ["octree_6"] * 3):
    got = oc.nn.octree_batch([T(samples[n]) for n in names]).cpu().numpy()
    assert np.array_equal(got, orc.octree_batch([samples[n] for n in names])), names
  with pytest.raises(oc.lib.OcnnError) as e:
    oc.nn.octree_batch([T(samples["octree_1"]), T(samples["octree_3"])])
  assert e.value.code == -6 and "not consistent" in str(e.value)


def test_property_literals(oc, samples):
  """pytorch/test/test_octree_property.py:9-54."""
  octree = oc.nn.octree_batch([T(samples["octree_1"])] * 2)
  P = oc.nn.octree_property
  assert np.array_equal(P(octree, "index", 5).cpu().numpy(), [0] * 8 + [1] * 8)
  f = np.zeros((3, 16), np.float32)
  f[:, 0] = f[:, 8] = 3.0 ** 0.5 / 3.0
  assert np.allclose(P(octree, "feature", 5).cpu().numpy(), f[None, :, :, None])
  c = -np.ones(16)
  c[0], c[8] = 0, 1
  assert np.array_equal(P(octree, "child", 5).cpu().numpy(), c)
  parts = torch.cat([P(octree, "child", d) for d in range(1, 6)])
  assert np.array_equal(P(octree, "child").cpu().numpy()[2:], parts.cpu().numpy())
  assert P(octree, "node_num", 5).item() == 16 and P(octree, "node_num_cum", 5).item() == 178
  assert np.array_equal(P(octree, "node_num").cpu().numpy(), [2, 16, 128, 16, 16, 16])
  assert np.array_equal(P(octree, "node_num_cum").cpu().numpy(), [0, 2, 18, 146, 162, 178, 194])
  assert (P(octree, "batch_size").item(), P(octree, "depth").item(), P(octree, "full_depth").item()) == (2, 5, 2)
  assert tuple(P(octree, "neigh", 5).shape) == (16, 8)
  with pytest.raises(oc.lib.OcnnError):
    P(octree, "nonsense")


def test_neighbour_kernels(oc, orc, samples, synthetic):
  import ctypes as C
  st = lambda: C.c_void_p(torch.cuda.current_stream().cuda_stream)
  for depth, batch in ((1, 1), (2, 3), (3, 2), (5, 2)):
    out = torch.empty(batch * 8 ** depth * 8, dtype=torch.int32, device="cuda")
    oc.lib.call("ocnn_calc_neigh_full", C.c_void_p(out.data_ptr()), depth, batch, st())
    assert np.array_equal(out.cpu().numpy(), orc.calc_neigh_full(depth, batch))
  pbs = [make_points_blob(*synthetic.shape_cloud(3000, 11 + i)[:2]) for i in range(3)]
  b = OctreeBlob(orc.octree_batch([orc.points2octree(p, 7, 2) for p in pbs]))
  for d in range(3, 8):
    neigh, child = b.prop("neigh", d - 1).reshape(-1), b.prop("child", d - 1)
    out = torch.full((int(b.nnum[d]) * 8,), -7, dtype=torch.int32, device="cuda")
    neigh_d, child_d = T(neigh).cuda(), T(child).cuda()
    oc.lib.call("ocnn_calc_neigh_sparse", C.c_void_p(out.data_ptr()), C.c_void_p(neigh_d.data_ptr()),
                C.c_void_p(child_d.data_ptr()), child.size, st())
    assert np.array_equal(out.cpu().numpy(), b.prop("neigh", d).reshape(-1)), d


def pack(x, y, z, i):
  return (x | (y << 16) | (z << 32) | (i << 48))


def test_key_ops(oc, orc, samples):
  """pytorch/test/test_octree_key.py."""
  F = oc.nn
  octree = F.octree_batch([T(samples["octree_1"])] * 2)
  xyz = F.octree_property(octree, "xyz", 5)
  pts = F.octree_decode_key(xyz)
  gt = [[16, 16, 16], [16, 16, 17], [16, 17, 16], [16, 17, 17], [17, 16, 16], [17, 16, 17], [17, 17, 16], [17, 17, 17]]
  exp = np.array([g + [i] for i in (0, 1) for g in gt], np.int16)
  assert np.array_equal(pts.cpu().numpy(), exp)
  assert torch.equal(F.octree_encode_key(pts), xyz)
  key = F.octree_xyz2key(xyz, 5)
  assert torch.equal(F.octree_key2xyz(key, 5), xyz)
  assert torch.equal(F.octree_property(octree, "key", 5), key)
  q = torch.tensor([28673, 281474976739335, 10], dtype=torch.int64, device="cuda")
  assert F.octree_search_key(q, octree, 5, False, False).cpu().tolist() == [1, 15, -1]
  q = torch.tensor([28672, 28673, 281474976739328, 10], dtype=torch.int64, device="cuda")
  assert F.octree_search_key(q, octree, 5, False, True).cpu().tolist() == [0, -1, 1, -1]
  assert F.octree_search_key(xyz[[3, 12]], octree, 5, True, False).cpu().tolist() == [3, 12]
  x64 = torch.tensor([[2049, 4095, 8011, 1], [511, 4095, 8011, 0]], dtype=torch.int16, device="cuda")
  enc = F.octree_encode_key(x64)
  assert torch.equal(F.octree_decode_key(F.octree_key2xyz(F.octree_xyz2key(enc, 13), 13)), x64)
  rng = np.random.default_rng(5)
  for depth in (1, 4, 9, 16):
    v = rng.integers(0, 1 << 62, 4000).astype(np.uint64)
    vt = T(v.view(np.int64)).cuda()
    assert np.array_equal(F.octree_xyz2key(vt, depth).cpu().numpy().view(np.uint64), orc.xyz2key(v, depth))
    assert np.array_equal(F.octree_key2xyz(vt, depth).cpu().numpy().view(np.uint64), orc.key2xyz(v, depth))


def test_generate_key_label_search(oc, orc):
  import ctypes as C
  st = lambda: C.c_void_p(torch.cuda.current_stream().cuda_stream)
  P = lambda t: C.c_void_p(t.data_ptr())
  for depth, batch in ((1, 2), (3, 3)):
    out = torch.empty(batch * 8 ** depth, dtype=torch.int64, device="cuda")
    oc.lib.call("ocnn_generate_key_full", P(out), depth, batch, st())
    assert np.array_equal(out.cpu().numpy().view(np.uint64), orc.generate_key_full(depth, batch))
  rng = np.random.default_rng(6)
  key = orc.generate_key_full(3, 2)
  child = np.full(key.size, -1, np.int32)
  sel = np.sort(rng.choice(key.size, 300, replace=False))
  child[sel] = np.arange(300)
  out = torch.zeros(2400, dtype=torch.int64, device="cuda")
  key_d, child_d = T(key.view(np.int64)).cuda(), T(child).cuda()
  oc.lib.call("ocnn_generate_key_child", P(out), P(key_d), P(child_d), key.size, st())
  assert np.array_equal(out.cpu().numpy().view(np.uint64), orc.generate_key_child(key, child, 2400))
  for n in (1, 5, 1023, 1024, 1025, 300000):
    btm = rng.integers(0, 3, n).astype(np.int32)
    lab = torch.empty(n, dtype=torch.int32, device="cuda")
    cnt = torch.zeros(1, dtype=torch.int32, device="cuda")
    sb = oc.lib.get().ocnn_generate_label_scratch_bytes(n)
    scratch = torch.empty(sb, dtype=torch.uint8, device="cuda")
    btm_d = T(btm).cuda()
    oc.lib.call("ocnn_generate_label", P(lab), P(cnt), P(btm_d), n, 1, P(scratch), C.c_size_t(sb), st())
    exp, total = orc.generate_label(btm, 1)
    assert np.array_equal(lab.cpu().numpy(), exp) and cnt.item() == total
  keys = np.unique(rng.integers(0, 1 << 50, 100000).astype(np.uint64))
  q = np.concatenate([keys[::13], rng.integers(0, 1 << 50, 5000).astype(np.uint64)])
  idx = torch.empty(q.size, dtype=torch.int32, device="cuda")
  keys_d, q_d = T(keys.view(np.int64)).cuda(), T(q.view(np.int64)).cuda()
  oc.lib.call("ocnn_search_key", P(idx), P(keys_d), keys.size, P(q_d), q.size, st())
  assert np.array_equal(idx.cpu().numpy(), orc.search_key(keys, q))


@pytest.mark.parametrize("n_key", [16384, 16385, 40000, 65536 + 17, 1 << 20])
def test_search_key_through_sample_tables(oc, orc, n_key):
  """search_key_gpu (octree_nn.h:180-181) for many queries in a large array: two tables of samples
  (every 256th and every 16th key) written per call, the same positions as the plain search.
  Sizes around the table strides, queries below the first and above the last key, every sampled
  key and its neighbours, runs of equal keys (the first one is the answer, as lower_bound gives)."""
  import ctypes as C
  st = lambda: C.c_void_p(torch.cuda.current_stream().cuda_stream)
  P = lambda t: C.c_void_p(t.data_ptr())
  rng = np.random.default_rng(n_key)
  keys = np.sort(rng.integers(1000, 1 << 50, n_key).astype(np.uint64))
  if n_key == 40000:   # runs of equal keys across the sample boundaries
    keys[240:300] = keys[240]
    keys[4090:4100] = keys[4090]
    keys = np.sort(keys)
  hits = np.concatenate([keys[::16], keys[15::16], keys[1::256], keys[-3:], keys[:3]])
  q = np.concatenate([hits, hits + np.uint64(1), rng.integers(0, 1 << 50, 30000).astype(np.uint64),
                      np.array([0, 999, keys[-1] + np.uint64(5), (1 << 63)], dtype=np.uint64)])
  q = q[rng.permutation(q.size)]
  assert q.size >= 16384
  q_d = T(q.view(np.int64)).cuda()
  nb = oc.lib.get().ocnn_search_key_workspace_bytes(n_key)
  ws = torch.empty(nb, dtype=torch.uint8, device="cuda")
  exp = orc.search_key(keys, q)
  # the windows are cut at the 128-byte lines of the array as it lies in memory: every offset of
  # its first key inside a line (a key array inside an octree blob starts anywhere)
  padded = torch.zeros(n_key + 16, dtype=torch.int64, device="cuda")
  for off in (0, 1, 7, 15):
    keys_d = padded[off:off + n_key]
    keys_d.copy_(T(keys.view(np.int64)))
    assert (keys_d.data_ptr() & 127) == 8 * off
    idx = torch.full((q.size,), -7, dtype=torch.int32, device="cuda")
    oc.lib.call("ocnn_search_key_indexed", P(idx), P(keys_d), n_key, P(q_d), q.size, P(ws), C.c_size_t(nb), st())
    assert np.array_equal(idx.cpu().numpy(), exp), off
  plain = torch.empty_like(idx)
  oc.lib.call("ocnn_search_key", P(plain), P(keys_d), n_key, P(q_d), q.size, st())
  assert torch.equal(idx, plain)
  # few queries: the call is the plain search and needs no workspace
  few = torch.empty(100, dtype=torch.int32, device="cuda")
  oc.lib.call("ocnn_search_key_indexed", P(few), P(keys_d), n_key, P(q_d), 100, None, C.c_size_t(0), st())
  assert np.array_equal(few.cpu().numpy(), exp[:100])
  with pytest.raises(oc.lib.OcnnError) as e:
    oc.lib.call("ocnn_search_key_indexed", P(idx), P(keys_d), n_key, P(q_d), q.size, P(ws), C.c_size_t(64), st())
  assert e.value.code == -4


def test_grow_md5_on_gpu(oc, samples):
  """pytorch/test/test_octree_grow.py: rebuild octree_2 with new/grow/update/set_property."""
  F = oc.nn
  gt = T(samples["octree_2"]).cuda()
  depth, channel = 5, 3
  o = F.octree_new(1, channel, False)
  o = F.octree_grow(o, 1, True)
  o = F.octree_grow(o, 2, True)
  for d in range(2, depth + 1):
    label = (F.octree_property(gt, "child", d) > -1).to(torch.int32)
    o = F.octree_update(o, label, d, 1)
    if d < depth:
      o = F.octree_grow(o, d + 1, False)
  o = F.octree_set_property(o, F.octree_property(gt, "feature", depth), depth)
  assert hashlib.md5(o.cpu().numpy().tobytes()).hexdigest().upper() == "D569D5BB23D34795C5FD81397F56275B"


def test_update_degenerate_and_errors(oc, orc):
  F = oc.nn
  o = F.octree_grow(F.octree_new(2, 1, False), 1, True)
  u = F.octree_update(o, torch.zeros(16, dtype=torch.int32), 1, 1)
  exp = orc.octree_update(orc.octree_grow(orc.octree_new(2, 1, False, 0), 1, True), np.zeros(16, np.int32), 1, 1)
  assert np.array_equal(u.cpu().numpy(), exp)
  assert F.octree_info(u).nnum_nempty(1) == 1
  with pytest.raises(oc.lib.OcnnError) as e:
    F.octree_update(o, torch.zeros(15, dtype=torch.int32), 1, 1)
  assert e.value.code == -3
  with pytest.raises(oc.lib.OcnnError):
    F.octree_grow(o, 3, False)


def test_update_in_place_and_with_the_clone_inside(oc, orc, samples):
  """ocnn_octree_update (in place, on the caller's clone) and ocnn_octree_update_copy (the clone of
  pytorch/cpp/octree_grow.cpp:165 inside the call, beside the scan) give the same blob, the oracle's,
  for blobs whose child array starts at an odd word and for the case where nothing splits; the source
  blob stays untouched; writing onto the source is refused."""
  import ctypes as C
  F = oc.nn
  L = oc.lib.get()
  P = lambda t: C.c_void_p(t.data_ptr())
  rng = np.random.default_rng(7)
  for name in ("octree_1", "octree_2", "octree_3"):
    host = orc.octree_batch([samples[name]])
    src = T(host).cuda()
    info = F.octree_info(src)
    for depth in (info.depth, info.depth - 1):
      n = info.nnum(depth)
      for labels in (rng.integers(0, 2, n).astype(np.int32), np.zeros(n, np.int32)):
        exp = orc.octree_update(host, labels, depth, 1)
        lab = T(labels).cuda()
        got = F.octree_update(src, lab, depth, 1)                       # the copy form
        assert np.array_equal(got.cpu().numpy(), exp), (name, depth)
        assert np.array_equal(src.cpu().numpy(), host)
        assert F.octree_info(got).nnum_nempty(depth) == max(int(labels.sum()), 1)
        mine = src.clone()                                              # in place
        raw = np.array(info.raw, copy=True)
        sb = L.ocnn_octree_update_scratch_bytes(n)
        ws = torch.empty(sb + 256, dtype=torch.uint8, device="cuda")
        oc.lib.call("ocnn_octree_update", P(mine), C.c_void_p(raw.ctypes.data), P(lab), n, depth, 1, P(ws), C.c_size_t(sb), None)
        torch.cuda.synchronize()
        assert torch.equal(mine, got) and np.array_equal(raw[:716], exp[:716])
        own = src.clone()                                               # the same through the Python mirror
        F.octree_info(own)
        back = F.octree_update(own, lab, depth, 1, inplace=True)
        assert back is own and torch.equal(own, got)
        assert F.octree_info(own).nnum_nempty(depth) == max(int(labels.sum()), 1)
  raw = np.array(info.raw, copy=True)
  with pytest.raises(oc.lib.OcnnError) as e:
    oc.lib.call("ocnn_octree_update_copy", P(src), P(src), C.c_void_p(raw.ctypes.data), P(lab), n, depth, 1, P(ws), C.c_size_t(sb), None)
  assert e.value.code == -1


def test_octree_beyond_the_format_limit_is_refused(oc, synthetic):
  """The serialized format addresses its payload with 32-bit offsets (octree_info.h: ptr_dis_),
  so an octree above 2 GiB cannot be represented: an error code, never a wrapped size."""
  F = oc.nn
  p, n, f = synthetic.room_cloud(250000, 3)
  clouds = []
  for i in range(24):
    blob = make_points_blob(p + np.float32(1e-4 * i), n, f)
    t = T(blob).cuda()
    t._ocnn_points_info = blob[:88].copy()
    clouds.append(t)
  with pytest.raises(oc.lib.OcnnError) as e:
    F.points2octree_batch(clouds, 9, 2)
  assert e.value.code == -3 and "2 GiB" in str(e.value)
  # the workspace is reusable after the refusal
  o = F.points2octree_batch(clouds[:2], 9, 2)
  assert F.octree_info(o).batch_size == 2


@pytest.mark.parametrize("n_scenes,depth", [(1, 9), (3, 9), (2, 7)], ids=["three_levels", "two_levels", "small"])
def test_neighbour_tables_of_fused_levels_at_full_size(oc, synthetic, n_scenes, depth):
  """The build writes the neighbour tables of its last sparse levels in one launch (three levels up
  to 2 M nodes on the finest, two up to 8 M, one above).  Whatever it fused, every sparse level's
  table must be what calc_neigh makes of the level above (ocnn_calc_neigh_sparse, one level a
  launch, checked against the oracle in test_gpu_ops.py): the identity that defines the table
  (octree/octree/octree_nn.cpp:357-380), at the sizes that pick each form."""
  import ctypes as C
  F = oc.nn
  p, n, f = synthetic.room_cloud(250000, 3)
  clouds = [T(make_points_blob(p + np.float32(1e-4 * i), n, f)).cuda() for i in range(n_scenes)]
  octree = F.points2octree_batch(clouds, depth, 2)
  info = F.octree_info(octree)
  finest = info.nnum(depth)
  if n_scenes == 3:
    assert 1 << 21 < finest <= 1 << 23      # the size class that fuses two levels
  else:
    assert finest <= 1 << 21                # ... three
  P = lambda t: C.c_void_p(t.data_ptr())
  checked = 0
  for d in range(info.full_depth + 1, depth + 1):
    above = F.octree_property(octree, "neigh", d - 1).contiguous()
    child = F.octree_property(octree, "child", d - 1).contiguous()
    got = F.octree_property(octree, "neigh", d)
    exp = torch.empty_like(got)
    oc.lib.call("ocnn_calc_neigh_sparse", P(exp), P(above), P(child), info.nnum(d - 1), None)
    torch.cuda.synchronize()
    assert torch.equal(got, exp), d
    checked += 1
  assert checked >= 3
