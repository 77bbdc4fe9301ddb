"""Full-size levels against the oracle, on windows of 4096 output columns.

The oracle (octree2col chunk + textbook SGEMM, one host core) finishes a 4096-column window of a
64 -> 64 convolution in about a second, a whole level of a million octants would take minutes.
So the depth-9 scene of BASELINE config 4 and the depth-7 batch of config 3 (all 16 clouds) are
convolved whole on the GPU and compared with the oracle on the first window, a middle one, the
last (partial) one and the one that straddles the boundary between the column ranges of two
XCDs.  3x3x3 stride 1 and 2x2x2 stride 2, fp32 (1e-4) and bf16 (2e-2), convolution and
deconvolution, all nodes and non-empty nodes; max_pool and pad on the same windows bit for bit.
The wide operators of the configurations (128 -> 128, 128 -> 256, 3 -> 32; the row-major stride-2
deconvolution with 128 and 256 input channels) run on the depth-8 level of the scene.

A window of a deconvolution: at stride 1 the operator is the convolution with mirrored taps and
transposed weights (node p receives from its neighbour at the opposite offset), an identity that
test_mirrored_taps_identity_on_a_small_octree first checks against the oracle's own
deconvolution (W^T X scattered by col2octree, octree_conv.cpp:300-325); at stride 2 the window is
a range of parents, whose columns W^T X the oracle's col2octree scatters onto their children.

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


# ---- deconvolution windows and wide channels --------------------------------------------------------------
def mirrored(wd, cout, K):
  """deconvolution weights [Cin, Cout * K] -> the convolution weights [Cout, Cin * K] that give the
  same operator at stride 1: tap k of the scatter is tap K - 1 - k of the gather"""
  cin = wd.shape[0]
  return np.ascontiguousarray(wd.reshape(cin, cout, K)[:, :, ::-1].transpose(1, 0, 2).reshape(cout, cin * K))


def test_mirrored_taps_identity_on_a_small_octree(orc, synthetic):
  """pins the expectation used for the stride-1 deconvolution windows below"""
  pbs = [make_points_blob(*synthetic.shape_cloud(3000, 71 + i)[:2]) for i in range(2)]
  host = orc.octree_batch([orc.points2octree(p, 5, 2) for p in pbs])
  b = OctreeBlob(host)
  rng = np.random.default_rng(5)
  for d in (4, 5):
    H = int(b.nnum[d])
    x = rng.standard_normal((6, H)).astype(np.float32)
    wd = (rng.standard_normal((6, 10 * 27)) * 0.1).astype(np.float32)
    exp = orc.octree_deconv(x, wd, host, d, 10, [3, 3, 3], 1)
    got = orc.octree_conv(x, mirrored(wd, 10, 27), host, d, 10, [3, 3, 3], 1)
    assert np.abs(got - exp).max() < 1e-5 * np.abs(exp).max()
    # and over the non-empty nodes
    ne = b.prop("child", d) >= 0
    xn = np.ascontiguousarray(x[:, :int(ne.sum())])
    exp = orc.octree_deconv(xn, wd, host, d, 10, [3, 3, 3], 1, True)
    got = orc.octree_conv(xn, mirrored(wd, 10, 27), host, d, 10, [3, 3, 3], 1, True)
    assert np.abs(got - exp).max() < 1e-5 * np.abs(exp).max()


def deconv_s2_window(orc, xp, wd, cout, neigh_child_level, a, b):
  """rows 8a .. 8b of the 2x2x2 stride-2 deconvolution: columns W^T X of the parents a .. b, scattered
  onto their children by the oracle's col2octree through the child level's neighbour table"""
  col = orc.sgemm(wd, np.ascontiguousarray(xp[:, a:b]), transA=True)            # [Cout * 8, b - a]
  sub = neigh_child_level[a * 64:b * 64]
  sub = np.where(sub >= 0, sub - 8 * a, -1).astype(np.int32)
  return orc.col2octree(col.reshape(cout, 8, b - a), [2, 2, 2], 2, sub, b - a)


def run_deconv_level(oc, orc, octree, lv, lv_parent, seed, C=64):
  """3x3x3 stride-1 deconvolution at lv.depth and 2x2x2 stride-2 deconvolution from the level above
  onto lv.depth, fp32 and bf16, all nodes and non-empty nodes"""
  import ctypes as Ct
  P = lambda a: a.ctypes.data_as(Ct.c_void_p)
  F = oc.nn
  d, H, Hne = lv.depth, lv.H, lv.Hne
  rng = np.random.default_rng(seed)
  x = rng.standard_normal((C, H)).astype(np.float32)
  wd3 = (rng.standard_normal((C, C * 27)) * 0.02).astype(np.float32)
  wm3 = mirrored(wd3, C, 27)
  x16, wd3_16 = bf16_round(x), bf16_round(wd3)
  wm3_16 = mirrored(wd3_16, C, 27)
  xd = T(x).cuda().view(1, C, H, 1)
  y = F.octree_deconv(xd, T(wd3).cuda(), octree, d, C, [3, 3, 3], 1, False).cpu().numpy().reshape(C, H)
  y16 = F.octree_deconv(xd.bfloat16(), T(wd3).cuda().bfloat16(), octree, d, C, [3, 3, 3], 1, False)
  y16 = y16.float().cpu().numpy().reshape(C, H)
  for win in window_ids(H, 1024):
    a, b = win * WINDOW, min(H, (win + 1) * WINDOW)
    check(y[:, a:b], conv_window(orc, x, wm3, lv.neigh, [3, 3, 3], 1, H, win), TOL_F32, ("deconv333 f32", d, win))
    check(y16[:, a:b], conv_window(orc, x16, wm3_16, lv.neigh, [3, 3, 3], 1, H, win), TOL_BF16,
          ("deconv333 bf16", d, win))
  del y, y16
  ichild = np.flatnonzero(lv.child >= 0).astype(np.int32)
  xne = np.ascontiguousarray(x[:, :Hne])
  xne16 = bf16_round(xne)
  xn = T(xne).cuda().view(1, C, Hne, 1)
  yn = F.octree_deconv(xn, T(wd3).cuda(), octree, d, C, [3, 3, 3], 1, True).cpu().numpy().reshape(C, Hne)
  yn16 = F.octree_deconv(xn.bfloat16(), T(wd3).cuda().bfloat16(), octree, d, C, [3, 3, 3], 1, True)
  yn16 = yn16.float().cpu().numpy().reshape(C, Hne)
  ni = orc.get_ni([3, 3, 3])
  for win in window_ids(Hne, 256):
    a, b = win * WINDOW, min(Hne, (win + 1) * WINDOW)
    for data, wts, got, tol, tag in ((xne, wm3, yn, TOL_F32, "f32"), (xne16, wm3_16, yn16, TOL_BF16, "bf16")):
      col = np.zeros((C * 27, WINDOW), np.float32)
      orc.fn("octree2colP")(P(col), P(data), C, Hne, Hne, 27, 1, P(lv.neigh), P(ni), P(lv.child), P(ichild),
                            WINDOW, win)
      check(got[:, a:b], orc.sgemm(wts, col)[:, :b - a], tol, ("deconv333 nempty " + tag, d, win))
  del yn, yn16

  # 2x2x2 stride 2 from the level above: its non-empty nodes are the columns, the rows are lv's nodes
  Hp = lv_parent.Hne
  assert 8 * Hp == H
  xp = rng.standard_normal((C, Hp)).astype(np.float32)
  wd2 = (rng.standard_normal((C, C * 8)) * 0.05).astype(np.float32)
  xp16, wd2_16 = bf16_round(xp), bf16_round(wd2)
  xpd = T(xp).cuda().view(1, C, Hp, 1)
  z = F.octree_deconv(xpd, T(wd2).cuda(), octree, d - 1, C, [2, 2, 2], 2, False).cpu().numpy().reshape(C, H)
  z16 = F.octree_deconv(xpd.bfloat16(), T(wd2).cuda().bfloat16(), octree, d - 1, C, [2, 2, 2], 2, False)
  z16 = z16.float().cpu().numpy().reshape(C, H)
  zn = F.octree_deconv(xpd, T(wd2).cuda(), octree, d - 1, C, [2, 2, 2], 2, True).cpu().numpy().reshape(C, Hne)
  zn16 = F.octree_deconv(xpd.bfloat16(), T(wd2).cuda().bfloat16(), octree, d - 1, C, [2, 2, 2], 2, True)
  zn16 = zn16.float().cpu().numpy().reshape(C, Hne)
  for win in window_ids(Hp, 256):
    a, b = win * WINDOW, min(Hp, (win + 1) * WINDOW)
    exp = deconv_s2_window(orc, xp, wd2, C, lv.neigh, a, b)
    exp16 = deconv_s2_window(orc, xp16, wd2_16, C, lv.neigh, a, b)
    check(z[:, 8 * a:8 * b], exp, TOL_F32, ("deconv222 f32", d, win))
    check(z16[:, 8 * a:8 * b], exp16, TOL_BF16, ("deconv222 bf16", d, win))
    # over the non-empty nodes the rows are the ranks of the non-empty children (col2octreeP ==
    # depad of col2octree, pytorch/test/test_octree2col.py:99-132): a contiguous range of ranks
    keep = lv.child[8 * a:8 * b] >= 0
    ranks = lv.child[8 * a:8 * b][keep]
    if ranks.size:
      assert ranks[-1] - ranks[0] + 1 == ranks.size
      check(zn[:, ranks[0]:ranks[-1] + 1], exp[:, keep], TOL_F32, ("deconv222 nempty f32", d, win))
      check(zn16[:, ranks[0]:ranks[-1] + 1], exp16[:, keep], TOL_BF16, ("deconv222 nempty bf16", d, win))


def test_scene_depth9_deconv_windows(oc, orc, scene):
  octree, lv = scene
  run_deconv_level(oc, orc, octree, lv, Level(octree, 8), 45)


def test_batch16_depth7_deconv_windows(oc, orc, batch16):
  octree, lv = batch16
  run_deconv_level(oc, orc, octree, lv, Level(octree, 6), 47)


WIDE_WINDOW = 1024


def wide_ids(n_cols):
  n = (n_cols + WIDE_WINDOW - 1) // WIDE_WINDOW
  return sorted({0, n // 2, n - 1})


def conv_window_wide(orc, x, w, neigh, n_cols, win):
  import ctypes as Ct
  P = lambda a: a.ctypes.data_as(Ct.c_void_p)
  C = x.shape[0]
  ni = orc.get_ni([3, 3, 3])
  col = np.zeros((C * 27, WIDE_WINDOW), np.float32)
  orc.fn("octree2col")(P(col), P(x), C, n_cols, 27, 1, P(neigh), P(ni), WIDE_WINDOW, win)
  return orc.sgemm(w, col)[:, :min(WIDE_WINDOW, n_cols - win * WIDE_WINDOW)]


@pytest.mark.parametrize("cin,cout", [(128, 128), (128, 256), (3, 32)])
def test_scene_depth8_wide_channel_windows(oc, orc, scene, cin, cout):
  """The channel widths of BASELINE config 4 (128 -> 128, 128 -> 256) and config 2 (3 -> 32, and
  128 -> 256 again) on a level large enough for the big-level kernels (741 784 octants): 3x3x3
  stride 1, fp32 and bf16, channel-major and row-major, all nodes and non-empty nodes."""
  import ctypes as Ct
  P = lambda a: a.ctypes.data_as(Ct.c_void_p)
  F = oc.nn
  octree, _ = scene
  lv = Level(octree, 8)
  d, H, Hne = 8, lv.H, lv.Hne
  rng = np.random.default_rng(1000 + cin + cout)
  x = rng.standard_normal((cin, H)).astype(np.float32)
  w = (rng.standard_normal((cout, cin * 27)) * 0.02).astype(np.float32)
  x16, w16 = bf16_round(x), bf16_round(w)
  xd, wdv = T(x).cuda().view(1, cin, H, 1), T(w).cuda()
  y = F.octree_conv(xd, wdv, octree, d, cout, [3, 3, 3], 1, False).cpu().numpy().reshape(cout, H)
  y16 = F.octree_conv(xd.bfloat16(), wdv.bfloat16(), octree, d, cout, [3, 3, 3], 1, False)
  rows = F.octree_conv_rows(F.to_rows(xd.bfloat16()), cin, wdv.bfloat16(), octree, d, cout)
  assert torch.equal(F.from_rows(rows, cout), y16)          # same products in the same order
  y16 = y16.float().cpu().numpy().reshape(cout, H)
  for win in wide_ids(H):
    a, b = win * WIDE_WINDOW, min(H, (win + 1) * WIDE_WINDOW)
    check(y[:, a:b], conv_window_wide(orc, x, w, lv.neigh, H, win), TOL_F32, ("wide f32", cin, cout, win))
    check(y16[:, a:b], conv_window_wide(orc, x16, w16, lv.neigh, H, win), TOL_BF16, ("wide bf16", cin, cout, win))
  del y, y16, rows
  # non-empty nodes
  ichild = np.flatnonzero(lv.child >= 0).astype(np.int32)
  xne = np.ascontiguousarray(x[:, :Hne])
  xne16 = bf16_round(xne)
  xn = T(xne).cuda().view(1, cin, Hne, 1)
  yn = F.octree_conv(xn, wdv, octree, d, cout, [3, 3, 3], 1, True).cpu().numpy().reshape(cout, Hne)
  yn16 = F.octree_conv(xn.bfloat16(), wdv.bfloat16(), octree, d, cout, [3, 3, 3], 1, True)
  rows = F.octree_conv_rows(F.to_rows(xn.bfloat16()), cin, wdv.bfloat16(), octree, d, cout, nempty=True)
  assert torch.equal(F.from_rows(rows, cout), yn16)
  yn16 = yn16.float().cpu().numpy().reshape(cout, Hne)
  ni = orc.get_ni([3, 3, 3])
  for win in wide_ids(Hne):
    a, b = win * WIDE_WINDOW, min(Hne, (win + 1) * WIDE_WINDOW)
    for data, wts, got, tol, tag in ((xne, w, yn, TOL_F32, "f32"), (xne16, w16, yn16, TOL_BF16, "bf16")):
      col = np.zeros((cin * 27, WIDE_WINDOW), np.float32)
      orc.fn("octree2colP")(P(col), P(data), cin, Hne, Hne, 27, 1, P(lv.neigh), P(ni), P(lv.child), P(ichild),
                            WIDE_WINDOW, win)
      check(got[:, a:b], orc.sgemm(wts, col)[:, :b - a], tol, ("wide nempty " + tag, cin, cout, win))


@pytest.mark.parametrize("cin,cout", [(128, 64), (256, 128)])
def test_scene_wide_stride2_rows_windows(oc, orc, scene, cin, cout):
  """The row-major 2x2x2 stride-2 pair with the decoder's widths (8 and 16 k-steps of input
  channels): deconvolution depth 7 -> 8 (depad folded in) and convolution depth 8 -> 7 (pad folded
  in), bf16, against the oracle on windows of parents."""
  F = oc.nn
  octree, _ = scene
  lv8, lv7 = Level(octree, 8), Level(octree, 7)
  rng = np.random.default_rng(2000 + cin)
  H7, Hne7, H8 = lv7.H, lv7.Hne, lv8.H
  # deconvolution: input on ALL nodes of depth 7 (the operator depads), output on depth 8
  x = bf16_round(rng.standard_normal((cin, H7)).astype(np.float32))
  wd = bf16_round((rng.standard_normal((cin, cout * 8)) * 0.05).astype(np.float32))
  rows = F.octree_conv_rows(F.to_rows(T(x).cuda().view(1, cin, H7, 1).bfloat16()), cin, T(wd).cuda().bfloat16(), octree,
                            7, cout, deconv=True, kernel_size=(2, 2, 2), stride=2)
  z = F.from_rows(rows, cout).float().cpu().numpy().reshape(cout, H8)
  xp = np.ascontiguousarray(x[:, lv7.child >= 0])           # depad
  for win in wide_ids(Hne7):
    a, b = win * WIDE_WINDOW, min(Hne7, (win + 1) * WIDE_WINDOW)
    check(z[:, 8 * a:8 * b], deconv_s2_window(orc, xp, wd, cout, lv8.neigh, a, b), TOL_BF16, ("deconv rows", cin, win))
  # convolution: input on depth 8, output on ALL nodes of depth 7 (empty nodes: zero without a bias)
  x8 = bf16_round(rng.standard_normal((cin, H8)).astype(np.float32))
  w = bf16_round((rng.standard_normal((cout, cin * 8)) * 0.05).astype(np.float32))
  rows = F.octree_conv_rows(F.to_rows(T(x8).cuda().view(1, cin, H8, 1).bfloat16()), cin, T(w).cuda().bfloat16(), octree,
                            8, cout, kernel_size=(2, 2, 2), stride=2)
  y = F.from_rows(rows, cout).float().cpu().numpy().reshape(cout, H7)
  ne7 = np.flatnonzero(lv7.child >= 0)
  assert not y[:, lv7.child < 0].any()
  import ctypes as Ct
  P = lambda a: a.ctypes.data_as(Ct.c_void_p)
  ni = orc.get_ni([2, 2, 2])
  for win in wide_ids(Hne7):
    a, b = win * WIDE_WINDOW, min(Hne7, (win + 1) * WIDE_WINDOW)
    col = np.zeros((cin * 8, WIDE_WINDOW), np.float32)
    orc.fn("octree2col")(P(col), P(x8), cin, Hne7, 8, 2, P(lv8.neigh), P(ni), WIDE_WINDOW, win)
    check(y[:, ne7[a:b]], orc.sgemm(w, col)[:, :b - a], TOL_BF16, ("conv rows", cin, win))
