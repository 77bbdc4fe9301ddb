"""Full-size levels against the oracle, on windows of 4096 output columns.

The oracle (octree2col chunk + textbook SGEMM, one host core) finishes a 4096-column window of a
64 -> 64 convolution in about a second, a whole level of a million octants would take minutes.
So the depth-9 scene of BASELINE config 4 and the depth-7 batch of config 3 (all 16 clouds) are
convolved whole on the GPU and compared with the oracle on the first window, a middle one, the
last (partial) one and the one that straddles the boundary between the column ranges of two
XCDs.  3x3x3 stride 1 and 2x2x2 stride 2, fp32 (1e-4) and bf16 (2e-2), conv and deconv, all
nodes and non-empty nodes; max_pool and pad on the same windows bit for bit.

Two measures per window: the largest error relative to the largest magnitude of the window, and
an element-wise bound |got - exp| <= tol * (|exp| + rms of the output channel in the window):
a wrong value in a channel of small magnitude passes the first and fails the second."""
import numpy as np
import pytest
import torch

from oracle.checker import OctreeBlob, make_points_blob

pytestmark = pytest.mark.gpu

WINDOW = 4096
TOL_F32, TOL_BF16 = 1e-4, 2e-2


def T(a):
  return torch.from_numpy(np.ascontiguousarray(a))


def bf16_round(a):
  return T(a).bfloat16().float().numpy()


def check(got, exp, tol, what):
  assert got.shape == exp.shape, what
  scale = float(np.abs(exp).max())
  assert scale > 0, what
  assert float(np.abs(got - exp).max()) / scale < tol, what
  rms = np.sqrt((exp.astype(np.float64) ** 2).mean(axis=1, keepdims=True)).astype(np.float32)
  bad = np.abs(got - exp) > tol * (np.abs(exp) + rms)
  assert not bad.any(), (what, int(bad.sum()), np.argwhere(bad)[:4].tolist())


def window_ids(n_cols, tile_cols):
  """first, middle, last (partial unless n_cols is a multiple), and the window holding the first
  column of the second XCD's range (the kernels give each of 8 XCDs a contiguous range of tiles)"""
  n_win = (n_cols + WINDOW - 1) // WINDOW
  tiles = (n_cols + tile_cols - 1) // tile_cols
  xcd_col = ((tiles + 7) // 8) * tile_cols
  ids = {0, n_win // 2, n_win - 1, min(n_win - 1, max(0, (xcd_col - 1) // WINDOW))}
  return sorted(ids)


class Level:
  """Host copies of what the oracle needs from one depth of a built octree."""

  def __init__(self, blob_dev, depth):
    self.blob = OctreeBlob(blob_dev.cpu().numpy())
    self.depth = depth
    self.neigh = self.blob.prop("neigh", depth).reshape(-1)
    self.child = self.blob.prop("child", depth)
    self.H = int(self.blob.nnum[depth])
    self.Hne = int((self.child >= 0).sum())


def conv_window(orc, x, w, neigh, ks, stride, n_cols, win):
  """columns [win * WINDOW, ...) of W x octree2col(x), by the oracle"""
  C = x.shape[0]
  K = int(np.prod(ks))
  ni = orc.get_ni(ks)
  col = np.zeros((C * K, WINDOW), np.float32)
  import ctypes as Ct
  P = lambda a: a.ctypes.data_as(Ct.c_void_p)
  orc.fn("octree2col")(P(col), P(x), C, n_cols, K, stride, P(neigh), P(ni), WINDOW, win)
  cols = min(WINDOW, n_cols - win * WINDOW)
  return orc.sgemm(w, col)[:, :cols]


@pytest.fixture(scope="module")
def scene(oc, synthetic):
  p, n, f = synthetic.room_cloud(250000, 3)
  octree = oc.nn.points2octree_batch([T(make_points_blob(p, n, f)).cuda()], 9, 2)
  return octree, Level(octree, 9)


@pytest.fixture(scope="module")
def batch16(oc, synthetic):
  clouds = []
  for i in range(16):
    p, n, _ = synthetic.shape_cloud(50000, 200 + i)
    clouds.append(T(make_points_blob(p, n)).cuda())
  octree = oc.nn.points2octree_batch(clouds, 7, 2)
  return octree, Level(octree, 7)


def run_level(oc, orc, octree, lv, seed):
  F = oc.nn
  d, H, C = lv.depth, lv.H, 64
  rng = np.random.default_rng(seed)
  x = rng.standard_normal((C, H)).astype(np.float32)
  w3 = (rng.standard_normal((C, C * 27)) * 0.02).astype(np.float32)
  w2 = (rng.standard_normal((C, C * 8)) * 0.02).astype(np.float32)
  xd = T(x).cuda().view(1, C, H, 1)
  x16, w3_16, w2_16 = bf16_round(x), bf16_round(w3), bf16_round(w2)

  # 3x3x3 stride 1 over all nodes: fp32, bf16, and the deconvolution (mirrored taps)
  y = F.octree_conv(xd, T(w3).cuda(), octree, d, C, [3, 3, 3], 1, False).cpu().numpy().reshape(C, H)
  y16 = F.octree_conv(xd.bfloat16(), T(w3).cuda().bfloat16(), octree, d, C, [3, 3, 3], 1, False)
  y16 = y16.float().cpu().numpy().reshape(C, H)
  for win in window_ids(H, 256):
    a, b = win * WINDOW, min(H, (win + 1) * WINDOW)
    check(y[:, a:b], conv_window(orc, x, w3, lv.neigh, [3, 3, 3], 1, H, win), TOL_F32, ("conv333 f32", d, win))
  for win in window_ids(H, 1024):       # the register-fed bf16 kernel works on tiles of 1024 columns
    a, b = win * WINDOW, min(H, (win + 1) * WINDOW)
    check(y16[:, a:b], conv_window(orc, x16, w3_16, lv.neigh, [3, 3, 3], 1, H, win), TOL_BF16,
          ("conv333 bf16", d, win))
  del y, y16

  # 2x2x2 stride 2 over all nodes: the columns are the parents
  Hp = H // 8
  z = F.octree_conv(xd, T(w2).cuda(), octree, d, C, [2, 2, 2], 2, False).cpu().numpy().reshape(C, Hp)
  z16 = F.octree_conv(xd.bfloat16(), T(w2).cuda().bfloat16(), octree, d, C, [2, 2, 2], 2, False)
  z16 = z16.float().cpu().numpy().reshape(C, Hp)
  for win in window_ids(Hp, 256):
    a, b = win * WINDOW, min(Hp, (win + 1) * WINDOW)
    check(z[:, a:b], conv_window(orc, x, w2, lv.neigh, [2, 2, 2], 2, Hp, win), TOL_F32, ("conv222 f32", d, win))
    check(z16[:, a:b], conv_window(orc, x16, w2_16, lv.neigh, [2, 2, 2], 2, Hp, win), TOL_BF16,
          ("conv222 bf16", d, win))
  del z, z16

  # non-empty nodes only (the reference's ScanNet setting): columns and rows are ranks of the
  # non-empty nodes, the oracle's octree2colP does the chunk
  import ctypes as Ct
  P = lambda a: a.ctypes.data_as(Ct.c_void_p)
  Hne = lv.Hne
  ichild = np.flatnonzero(lv.child >= 0).astype(np.int32)
  xne = np.ascontiguousarray(x[:, :Hne])
  xne16 = bf16_round(xne)
  yn = F.octree_conv(T(xne).cuda().view(1, C, Hne, 1), T(w3).cuda(), octree, d, C, [3, 3, 3], 1, True)
  yn = yn.cpu().numpy().reshape(C, Hne)
  yn16 = F.octree_conv(T(xne).cuda().view(1, C, Hne, 1).bfloat16(), T(w3).cuda().bfloat16(), octree, d, C,
                       [3, 3, 3], 1, True).float().cpu().numpy().reshape(C, Hne)
  ni = orc.get_ni([3, 3, 3])
  for win in window_ids(Hne, 256):
    a, b = win * WINDOW, min(Hne, (win + 1) * WINDOW)
    for data, wts, got, tol, tag in ((xne, w3, yn, TOL_F32, "f32"), (xne16, w3_16, yn16, TOL_BF16, "bf16")):
      col = np.zeros((C * 27, WINDOW), np.float32)
      orc.fn("octree2colP")(P(col), P(data), C, Hne, Hne, 27, 1, P(lv.neigh), P(ni), P(lv.child), P(ichild),
                            WINDOW, win)
      check(got[:, a:b], orc.sgemm(wts, col)[:, :b - a], tol, ("conv333 nempty " + tag, d, win))
  del yn, yn16

  # max_pool (values and argmax indices) and pad on the same windows, bit for bit
  C8 = 8
  top, mask = F.octree_max_pool(xd[:, :C8].contiguous(), octree, d)
  top, mask = top.cpu().numpy().reshape(C8, Hp), mask.cpu().numpy().reshape(C8, Hp)
  for win in window_ids(Hp, 1024):
    a, b = win * WINDOW, min(Hp, (win + 1) * WINDOW)
    et, em = orc.max_pool(x[:C8, 8 * a:8 * b])
    assert np.array_equal(top[:, a:b], et), ("max_pool", d, win)
    assert np.array_equal(mask[:, a:b], em + 8 * a), ("max_pool mask", d, win)
  padded = F.octree_pad(T(xne[:C8]).cuda().view(1, C8, Hne, 1), octree, d).cpu().numpy().reshape(C8, H)
  for win in window_ids(H, 1024):
    a, b = win * WINDOW, min(H, (win + 1) * WINDOW)
    assert np.array_equal(padded[:, a:b], orc.pad(xne[:C8], lv.child[a:b])), ("pad", d, win)


def test_scene_depth9_windows(oc, orc, scene):
  octree, lv = scene
  run_level(oc, orc, octree, lv, 41)


def test_batch16_depth7_windows(oc, orc, batch16):
  octree, lv = batch16
  assert lv.blob.batch_size == 16
  run_level(oc, orc, octree, lv, 43)
