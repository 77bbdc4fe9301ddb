"""Seeded synthetic point clouds of the benchmark configurations (numpy, CPU).

Every generator returns float32 arrays (points [N,3], normals [N,3], features or None)
with the points strictly inside (-1, 1)^3: a coordinate of exactly +1 maps to cell
2^depth, which the Morton interleave wraps to cell 0 (only `depth` bits of each
coordinate are kept, octree/octree/octree_nn.cpp:551-560), and the reference pipeline
clips to the open box before building (octree/octree/points_parser.cpp:159-161).
"""
import numpy as np

SHRINK = np.float32(1.0 - 2.0 ** -12)


def sphere_cloud(n=3000, seed=0):
  """Uniform samples on the unit sphere; the normal equals the position."""
  rng = np.random.default_rng(seed)
  v = rng.standard_normal((n, 3))
  p = v / np.linalg.norm(v, axis=1, keepdims=True)
  nrm = p.astype(np.float32)
  pts = (p * float(SHRINK)).astype(np.float32)
  return pts, nrm, None


def _random_rotation(rng):
  q = rng.standard_normal(4)
  q /= np.linalg.norm(q)
  w, x, y, z = q
  return np.array([[1 - 2 * (y * y + z * z), 2 * (x * y - z * w), 2 * (x * z + y * w)],
                   [2 * (x * y + z * w), 1 - 2 * (x * x + z * z), 2 * (y * z - x * w)],
                   [2 * (x * z - y * w), 2 * (y * z + x * w), 1 - 2 * (x * x + y * y)]])


def _sample_ellipsoid(rng, n, axes):
  u = rng.standard_normal((n, 3))
  u /= np.linalg.norm(u, axis=1, keepdims=True)
  p = u * axes
  nrm = u / axes
  nrm /= np.linalg.norm(nrm, axis=1, keepdims=True)
  return p, nrm


def _sample_box(rng, n, half, faces=(0, 1, 2, 3, 4, 5)):
  """Area-weighted samples on the chosen faces (axis*2 + side) of an axis-aligned box."""
  areas = np.array([4 * half[(f // 2 + 1) % 3] * half[(f // 2 + 2) % 3] for f in faces])
  face = rng.choice(len(faces), size=n, p=areas / areas.sum())
  p = rng.uniform(-1.0, 1.0, (n, 3)) * half
  nrm = np.zeros((n, 3))
  for i, f in enumerate(faces):
    sel = face == i
    ax, side = f // 2, 1.0 if f % 2 else -1.0
    p[sel, ax] = side * half[ax]
    nrm[sel, ax] = side
  return p, nrm


def shape_cloud(n=10000, seed=100):
  """Union of 1-4 random ellipsoids / boxes (semi-axes U[0.2, 0.8], random rotation and
  offset), surface-sampled with analytic normals and normalised by its bounding box."""
  rng = np.random.default_rng(seed)
  k = int(rng.integers(1, 5))
  counts = np.full(k, n // k)
  counts[: n - counts.sum()] += 1
  P, Nrm = [], []
  for i in range(k):
    axes = rng.uniform(0.2, 0.8, 3)
    R = _random_rotation(rng)
    c = rng.uniform(-0.3, 0.3, 3)
    if rng.random() < 0.5:
      p, nr = _sample_ellipsoid(rng, int(counts[i]), axes)
    else:
      p, nr = _sample_box(rng, int(counts[i]), axes)
    P.append(p @ R.T + c)
    Nrm.append(nr @ R.T)
  p = np.concatenate(P)
  nrm = np.concatenate(Nrm)
  lo, hi = p.min(0), p.max(0)
  center, radius = (lo + hi) / 2, (hi - lo).max() / 2
  p = (p - center) / radius * float(SHRINK)
  return p.astype(np.float32), nrm.astype(np.float32), None


def room_cloud(n=250000, seed=3, n_boxes=20):
  """Indoor room 5 m x 5 m x 3 m: floor, four walls and `n_boxes` axis-aligned boxes
  standing on the floor (edge lengths U[0.3, 1.5] m), sampled by area; RGB features
  U[0, 1].  Normalised by the 5 m width, so a depth-9 cell is about 0.98 cm."""
  rng = np.random.default_rng(seed)
  W, Hh = 5.0, 3.0
  surfaces = []  # (centre, half extents, faces)
  room_half = np.array([W / 2, W / 2, Hh / 2])
  # inward-facing room shell without ceiling: floor = face z-, walls = x-, x+, y-, y+
  surfaces.append((np.array([0.0, 0.0, Hh / 2]), room_half, (0, 1, 2, 3, 4), -1.0))
  for _ in range(n_boxes):
    size = rng.uniform(0.3, 1.5, 3)
    half = size / 2
    cx = rng.uniform(-W / 2 + half[0], W / 2 - half[0])
    cy = rng.uniform(-W / 2 + half[1], W / 2 - half[1])
    surfaces.append((np.array([cx, cy, half[2]]), half, (0, 1, 2, 3, 5), 1.0))
  areas = []
  for _, half, faces, _ in surfaces:
    areas.append(sum(4 * half[(f // 2 + 1) % 3] * half[(f // 2 + 2) % 3] for f in faces))
  areas = np.array(areas)
  counts = np.floor(n * areas / areas.sum()).astype(int)
  counts[0] += n - counts.sum()
  P, Nrm = [], []
  for (c, half, faces, sign), m in zip(surfaces, counts):
    p, nr = _sample_box(rng, int(m), half, faces)
    P.append(p + c)
    Nrm.append(nr * sign)
  p = np.concatenate(P)
  nrm = np.concatenate(Nrm)
  rgb = rng.uniform(0.0, 1.0, (n, 3))
  p = (p - np.array([0.0, 0.0, Hh / 2])) / (W / 2) * float(SHRINK)
  return p.astype(np.float32), nrm.astype(np.float32), rgb.astype(np.float32)
