"""Pins the oracle's point-cloud transforms (pytorch/cpp/transform_points.cpp:7-125)."""
import numpy as np
import pytest

from oracle.checker import make_points_blob


def cloud(rng, n, trial):
  pts = (rng.standard_normal((n, 3)) * rng.uniform(0.1, 3)).astype(np.float32) + rng.uniform(-1, 1, 3).astype(np.float32)
  nrm = rng.standard_normal((n, 3)).astype(np.float32) if trial % 3 else None
  feat = rng.uniform(0, 1, (n, 2)).astype(np.float32) if trial % 2 else None
  lab = rng.integers(0, 4, n).astype(np.float32) if trial % 4 == 0 else None
  return pts, nrm, feat, lab


def arrays(blob):
  """xyz / normal / feature / label arrays of a points blob (octree/octree/points_info.h:35-39)."""
  i = blob[16:88].view(np.int32)
  n, flags, ch, dis = int(i[0]), int(i[1]), i[2:6], i[10:15]
  out = []
  for t in range(4):
    if flags & (1 << t):
      out.append(blob[dis[t]:dis[t] + 4 * n * ch[t]].view(np.float32).reshape(n, ch[t]))
    else:
      out.append(None)
  return out


def test_transforms_vs_compiled_reference(orc, ref):
  rng = np.random.default_rng(0)
  for trial in range(30):
    n = int(rng.integers(1, 5000))
    pb = make_points_blob(*cloud(rng, n, trial))
    for m in ("sphere", "box"):
      assert np.array_equal(orc.bounding_sphere(pb, m), ref.bounding_sphere(pb, m))
    bs = orc.bounding_sphere(pb, "sphere")
    x = orc.normalize_points(pb, bs[0], bs[1:])
    assert np.array_equal(x, ref.normalize_points(pb, bs[0], bs[1:]))
    ang = (rng.integers(-180, 180, 3) * 3.14159265 / 180).astype(np.float32) if trial % 5 else np.zeros(3, np.float32)
    sc = rng.uniform(0.75, 1.25, 3).astype(np.float32) if trial % 2 else np.full(3, 1.2, np.float32)
    jit = rng.uniform(-0.25, 0.25, 3).astype(np.float32)
    off, ax = float(rng.choice([0.0, 0.01])), str(rng.choice(["", "x", "y", "z", "xyz"]))
    t = orc.transform_points(x, ang, sc, jit, off, ax)
    assert np.array_equal(t, ref.transform_points(x, ang, sc, jit, off, ax))
    (c1, m1), (c2, m2) = orc.clip_points(t, [-1] * 3, [1] * 3), ref.clip_points(t, [-1] * 3, [1] * 3)
    assert np.array_equal(c1, c2) and np.array_equal(m1, m2)
  # nothing inside the box: point 0 is kept and moved to the box corner
  pb = make_points_blob(np.full((5, 3), 9.0, np.float32))
  (c1, m1), (c2, m2) = orc.clip_points(pb, [-1] * 3, [1] * 3), ref.clip_points(pb, [-1] * 3, [1] * 3)
  assert np.array_equal(c1, c2) and m1.tolist() == [1, 0, 0, 0, 0] == m2.tolist()


def test_transforms_closed_forms(orc):
  """What the mathematics fixes, independent of the reference build."""
  rng = np.random.default_rng(1)
  pts = (rng.standard_normal((2000, 3)) * 0.7).astype(np.float32)
  nrm = rng.standard_normal((2000, 3)).astype(np.float32)
  nrm /= np.linalg.norm(nrm, axis=1, keepdims=True)
  feat = rng.uniform(0, 1, (2000, 2)).astype(np.float32)
  lab = rng.integers(0, 4, 2000).astype(np.float32)
  pb = make_points_blob(pts, nrm, feat, lab)
  # every point lies inside the bounding sphere; the box sphere is centred on the box
  r, cx, cy, cz = orc.bounding_sphere(pb, "sphere")
  assert np.all(np.linalg.norm(pts - [cx, cy, cz], axis=1) <= r * (1 + 1e-5))
  rb = orc.bounding_sphere(pb, "box")
  assert np.allclose(rb[1:], (pts.max(0) + pts.min(0)) / 2, atol=1e-6)
  assert np.isclose(rb[0], np.linalg.norm((pts.max(0) - pts.min(0)) / 2), rtol=1e-6)
  # normalise = (p - c) / r
  p2 = arrays(orc.normalize_points(pb, r, [cx, cy, cz]))[0]
  assert np.allclose(p2, (pts - [cx, cy, cz]) / r, atol=1e-6)
  # a rotation about z by 90 degrees maps (x, y, z) -> (-y, x, z) in the reference's convention
  # R = Rx Ry Rz with column-major 3x3 blocks; normals rotate with the points, lengths are kept
  ang = np.array([0.3, -1.1, 2.0], np.float32)
  cx_, sx = np.cos(ang[0]), np.sin(ang[0]); cy_, sy = np.cos(ang[1]), np.sin(ang[1]); cz_, sz = np.cos(ang[2]), np.sin(ang[2])
  Rx = np.array([[1, 0, 0], [0, cx_, -sx], [0, sx, cx_]])
  Ry = np.array([[cy_, 0, sy], [0, 1, 0], [-sy, 0, cy_]])
  Rz = np.array([[cz_, -sz, 0], [sz, cz_, 0], [0, 0, 1]])
  R = Rx @ Ry @ Rz
  out = arrays(orc.transform_points(pb, ang, [1, 1, 1], [0, 0, 0]))
  assert np.allclose(out[0], pts @ R.T, atol=1e-5)
  assert np.allclose(out[1], nrm @ R.T, atol=1e-5)
  assert np.array_equal(out[2], feat)
  # non-uniform scale: points scale, normals scale inversely and are renormalised; jitter adds
  out = arrays(orc.transform_points(pb, [0, 0, 0], [2, 1, 0.5], [0.1, 0.2, 0.3], 0.0, "z"))
  assert np.allclose(out[0], (pts + [0.1, 0.2, 0.3]) * [2, 1, 0.5], atol=1e-5)
  n2 = nrm / [2, 1, 0.5]
  n2 /= np.linalg.norm(n2, axis=1, keepdims=True)
  n2[n2[:, 2] < 0] *= -1
  assert np.allclose(out[1], n2, atol=1e-5)
  # clip == boolean mask + compaction of every array
  clipped, mask = orc.clip_points(pb, [-1] * 3, [1] * 3)
  inside = np.all((pts > -1) & (pts < 1), axis=1)
  assert np.array_equal(mask.astype(bool), inside) and 0 < inside.sum() < len(pts)
  got = arrays(clipped)
  for a, b in zip(got, (pts, nrm, feat, lab.reshape(-1, 1))):
    assert np.array_equal(a, b[inside])
