"""GPU parity of the point-cloud transforms (pytorch/cpp/transform_points.cpp:7-125) against the
oracle, byte for byte, and of the whole normalise -> transform -> clip -> points2octree chain of
pytorch/ocnn/transforms.py:105-125 run on the device."""
import numpy as np
import pytest
import torch

from oracle.checker import make_points_blob
from test_oracle_points import cloud

pytestmark = pytest.mark.gpu


def T(a):
  return torch.from_numpy(np.ascontiguousarray(a))


def test_transforms_bit_exact(oc, orc):
  F = oc.nn
  rng = np.random.default_rng(3)
  for trial in range(24):
    n = int(rng.integers(1, 6000)) if trial else 1
    pb = make_points_blob(*cloud(rng, n, trial))
    dev = T(pb).cuda()
    for m in ("sphere", "box"):
      assert np.array_equal(np.float32(F.bounding_sphere(dev, m)), orc.bounding_sphere(pb, m)), (trial, m)
    bs = orc.bounding_sphere(pb, "sphere")
    x = F.normalize_points(dev, float(bs[0]), bs[1:].tolist())
    xh = orc.normalize_points(pb, bs[0], bs[1:])
    assert np.array_equal(x.cpu().numpy(), xh)
    ang = (rng.integers(-180, 180, 3) * 3.14159265 / 180).astype(np.float32) if trial % 5 else np.zeros(3, np.float32)
    sc = rng.uniform(0.75, 1.25, 3).astype(np.float32) if trial % 2 else np.full(3, 1.2, np.float32)
    jit = rng.uniform(-0.25, 0.25, 3).astype(np.float32)
    off, ax = float(rng.choice([0.0, 0.01])), str(rng.choice(["", "x", "y", "z", "xyz"]))
    t = F.transform_points(x, ang.tolist(), sc.tolist(), jit.tolist(), off, ax)
    th = orc.transform_points(xh, ang, sc, jit, off, ax)
    assert np.array_equal(t.cpu().numpy(), th), (trial, ax)
    c, mask = F.clip_points(t, [-1.0] * 3, [1.0] * 3)
    ch, mh = orc.clip_points(th, [-1] * 3, [1] * 3)
    assert np.array_equal(mask.cpu().numpy(), mh)
    assert np.array_equal(c.cpu().numpy(), ch)
    assert np.array_equal(c._ocnn_points_info, ch[:88])


def test_clip_degenerate_and_errors(oc, orc):
  F = oc.nn
  pb = make_points_blob(np.full((5, 3), 9.0, np.float32), np.tile(np.float32([[0, 0, 1]]), (5, 1)))
  c, mask = F.clip_points(T(pb).cuda(), [-1.0] * 3, [1.0] * 3)
  ch, mh = orc.clip_points(pb, [-1] * 3, [1] * 3)
  assert np.array_equal(c.cpu().numpy(), ch) and mask.cpu().tolist() == mh.tolist() == [1, 0, 0, 0, 0]
  bad = T(pb.copy())
  bad[0] = 0
  with pytest.raises(oc.lib.OcnnError) as e:
    F.bounding_sphere(bad.cuda())
  assert e.value.code == -6


def test_transform_compose_on_device(oc, orc, synthetic):
  """NormalizePoints -> TransformPoints (+ clip) -> Points2Octree, then octree_batch."""
  F = oc.nn
  rng = np.random.default_rng(4)
  singles, dev_octrees = [], []
  for i in range(3):
    p, n, _ = synthetic.shape_cloud(8000, 400 + i)
    pb = make_points_blob(p * np.float32(3.0) + np.float32(0.5), n)
    ang = (rng.integers(-10, 10, 3) * 3.14159265 / 180).astype(np.float32)
    sc = rng.uniform(0.8, 1.25, 3).astype(np.float32)
    jit = rng.uniform(-0.2, 0.2, 3).astype(np.float32)
    # host chain through the oracle
    bs = orc.bounding_sphere(pb, "sphere")
    h = orc.normalize_points(pb, bs[0], bs[1:])
    h = orc.transform_points(h, ang, sc, jit, 0.0, "")
    h, hm = orc.clip_points(h, [-1] * 3, [1] * 3)
    singles.append(orc.points2octree(h, 6, 2))
    # device chain
    d = T(pb).cuda()
    r = F.bounding_sphere(d, "sphere")
    d = F.normalize_points(d, r[0], r[1:])
    d = F.transform_points(d, ang.tolist(), sc.tolist(), jit.tolist(), 0.0, "")
    d, dm = F.clip_points(d, [-1.0] * 3, [1.0] * 3)
    assert np.array_equal(dm.cpu().numpy(), hm) and 0 < hm.sum() < hm.size
    o = F.points2octree(d, 6, 2)
    assert np.array_equal(o.cpu().numpy(), singles[-1])
    dev_octrees.append(o)
  assert np.array_equal(F.octree_batch(dev_octrees).cpu().numpy(), orc.octree_batch(singles))


def test_transform_classes_follow_the_reference_pipeline(oc, orc, synthetic):
  """transforms.TransformCompose / collate_octrees (pytorch/ocnn/transforms.py:6-148) with numpy's
  generator seeded: the same draws through the oracle chain give the same octrees, points and
  masks; building the batch inside collate gives the same merged octree."""
  tr = oc.transforms
  flags = dict(depth=6, full_depth=2, distort=True, angle=[10, 180, 5], scale=0.2, jitter=0.125,
               angle_interval=[1, 5, 1], uniform_scale=False, bsphere="sphere")
  clouds = []
  for i in range(3):
    p, n, _ = synthetic.shape_cloud(6000, 500 + i)
    clouds.append(make_points_blob(p * np.float32(2.0) - np.float32(0.3), n))
  compose = tr.TransformCompose(flags)
  np.random.seed(11)
  samples = [compose(T(pb).cuda(), i) for i, pb in enumerate(clouds)]
  for s, lab in zip(samples, (3, 1, 4)):
    s["label"] = lab
  np.random.seed(11)
  host = []
  for pb, s in zip(clouds, samples):
    drawn = tr.draw_distortion(flags["angle"], flags["scale"], flags["jitter"], flags["angle_interval"], False)
    bs = orc.bounding_sphere(pb, "sphere")
    h = orc.normalize_points(pb, bs[0], bs[1:])
    h = orc.transform_points(h, np.float32(drawn[0]), np.float32(drawn[1]), np.float32(drawn[2]), 0.0, "")
    h, hm = orc.clip_points(h, [-1] * 3, [1] * 3)
    assert np.array_equal(s["inbox_mask"].cpu().numpy(), hm)
    assert np.array_equal(s["points"].cpu().numpy(), h)
    host.append(orc.points2octree(h, 6, 2))
    assert np.array_equal(s["octree"].cpu().numpy(), host[-1])
  merged = orc.octree_batch(host)
  out = tr.collate_octrees(samples)
  assert np.array_equal(out["octree"].cpu().numpy(), merged) and out["label"].tolist() == [3, 1, 4]
  assert len(out["points"]) == 3
  # samples without octrees: the batch is built in one pass at collate time
  late = tr.TransformCompose(flags, octree=False)
  np.random.seed(11)
  bare = [late(T(pb).cuda(), i) for i, pb in enumerate(clouds)]
  assert "octree" not in bare[0]
  out2 = tr.collate_octrees(bare, points2octree=late.points2octree)
  assert np.array_equal(out2["octree"].cpu().numpy(), merged)
  # no distortion: identity transform, only normalisation and clipping
  plain = tr.TransformCompose(dict(depth=5, distort=False, radius=2.0, center=(0.1, 0.0, -0.1)))
  s = plain(T(clouds[0]).cuda())
  h = orc.normalize_points(clouds[0], 2.0, (0.1, 0.0, -0.1))
  h = orc.transform_points(h, np.zeros(3, np.float32), np.ones(3, np.float32), np.zeros(3, np.float32), 0.0, "")
  h, hm = orc.clip_points(h, [-1] * 3, [1] * 3)
  assert np.array_equal(s["octree"].cpu().numpy(), orc.points2octree(h, 5, 2))


def test_scene_size(oc, orc, synthetic):
  """250 000 points: the sphere's sequential growth and the compaction at full size."""
  F = oc.nn
  p, n, f = synthetic.room_cloud(250000, 3)
  pb = make_points_blob(p * np.float32(1.3), n, f)
  dev = T(pb).cuda()
  assert np.array_equal(np.float32(F.bounding_sphere(dev, "sphere")), orc.bounding_sphere(pb, "sphere"))
  c, mask = F.clip_points(dev, [-1.0] * 3, [1.0] * 3)
  ch, mh = orc.clip_points(pb, [-1] * 3, [1] * 3)
  assert 0 < mh.sum() < mh.size
  assert np.array_equal(mask.cpu().numpy(), mh) and np.array_equal(c.cpu().numpy(), ch)
