"""Pins the oracle's octree2col / col2octree / conv / deconv / pool / pad."""
import numpy as np
import pytest
import torch

from oracle.checker import OctreeBlob, make_points_blob

IDX_MAPS = {(3, 3, 3): list(range(27)), (1, 1, 1): [13], (2, 2, 2): [13, 14, 16, 17, 22, 23, 25, 26],
            (3, 1, 1): [4, 13, 22], (3, 3, 1): [1, 4, 7, 10, 13, 16, 19, 22, 25]}


def closed_form_col(data, ks, stride):
  """pytorch/test/test_octree2col.py:23-50: octree2col on the full depth-1 layer."""
  idx_map = IDX_MAPS[tuple(ks)]
  K = len(idx_map)
  C = data.shape[0]
  top_h = 8 if stride == 1 else 1
  out = np.zeros((C, K, top_h), np.float32)
  for c in range(C):
    for k in range(K):
      for h in range(top_h):
        z, y, x = h & 1, (h & 2) >> 1, h >> 2
        t = idx_map[k]
        dz, dy, dx = t % 3, (t // 3) % 3, t // 9
        z, y, x = z + dz - 1, y + dy - 1, x + dx - 1
        if -1 < x < 2 and -1 < y < 2 and -1 < z < 2:
          out[c, k, h] = data[c, x * 4 + y * 2 + z]
  return out


@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("ks", [[3, 3, 3], [2, 2, 2], [3, 1, 1], [3, 3, 1], [1, 1, 1]])
def test_octree2col_closed_form(orc, samples, ks, stride):
  b = OctreeBlob(orc.octree_batch([samples["octree_1"]]))
  data = np.random.default_rng(0).uniform(-1, 1, (3, 8)).astype(np.float32)
  height = 8 if stride == 1 else 1
  col = orc.octree2col(data, ks, stride, b.prop("neigh", 1).reshape(-1), height)
  assert np.array_equal(col, closed_form_col(data, ks, stride))


@pytest.fixture(scope="module")
def batch4(orc, samples):
  blob = orc.octree_batch([samples[n] for n in ("octree_1", "octree_2", "octree_2", "octree_1")])
  return blob, OctreeBlob(blob)


@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("ks", [[3, 3, 3], [2, 2, 2], [3, 1, 1], [3, 3, 1], [1, 1, 1]])
def test_col2octree_is_adjoint(orc, batch4, ks, stride):
  _, b = batch4
  d = 4
  H = int(b.nnum[d])
  height = H if stride == 1 else H // 8
  rng = np.random.default_rng(1)
  x = rng.standard_normal((3, H)).astype(np.float32)
  neigh = b.prop("neigh", d).reshape(-1)
  col = orc.octree2col(x, ks, stride, neigh, height)
  y = rng.standard_normal(col.shape).astype(np.float32)
  back = orc.col2octree(y, ks, stride, neigh, height)
  assert np.isclose(np.vdot(col.astype(np.float64), y), np.vdot(x.astype(np.float64), back), rtol=1e-5)


@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("ks", [[3, 3, 3], [2, 2, 2], [3, 1, 1], [3, 3, 1], [1, 1, 1]])
def test_octree2colP_identity(orc, batch4, ks, stride):
  """pytorch/test/test_octree2col.py:99-132: octree2colP == pad -> octree2col -> depad."""
  _, b = batch4
  d = 4
  H, Hne = int(b.nnum[d]), int(b.nnum_nempty[d])
  child = b.prop("child", d)
  neigh = b.prop("neigh", d).reshape(-1)
  ichild = np.zeros(Hne, np.int32)
  ichild[child[child >= 0]] = np.nonzero(child >= 0)[0]
  rng = np.random.default_rng(2)
  x = rng.uniform(0, 1, (5, Hne)).astype(np.float32)
  padded = orc.pad(x, child)
  if stride == 1:
    out1 = orc.octree2col(padded, ks, 1, neigh, H)
    K = out1.shape[1]
    out1 = orc.depad(out1.reshape(5 * K, H), child, Hne).reshape(5, K, Hne)
    out2 = orc.octree2colP(x, ks, 1, neigh, child, ichild, Hne)
  else:
    hc = int(b.nnum_nempty[d - 1])
    out1 = orc.octree2col(padded, ks, 2, neigh, hc)
    out2 = orc.octree2colP(x, ks, 2, neigh, child, ichild, hc)
  assert np.array_equal(out1, out2)
  g = rng.uniform(0, 1, out2.shape).astype(np.float32)
  hcol = out2.shape[2]
  back2 = orc.col2octreeP(g, ks, stride, neigh, child, ichild, hcol, Hne)
  if stride == 1:
    gp = orc.pad(g.reshape(-1, Hne), child).reshape(5, -1, H)
    back1 = orc.depad(orc.col2octree(gp, ks, 1, neigh, H), child, Hne)
  else:
    back1 = orc.depad(orc.col2octree(g, ks, 2, neigh, hcol), child, Hne)
  assert np.allclose(back1, back2, atol=1e-6)


def test_pad_depad(orc, batch4):
  _, b = batch4
  child = b.prop("child", 4)
  x = np.random.default_rng(3).standard_normal((4, int(b.nnum_nempty[4]))).astype(np.float32)
  y = orc.pad(x, child, 7.5)
  assert np.all(y[:, child < 0] == 7.5)
  assert np.array_equal(y[:, child >= 0], x[:, child[child >= 0]])
  assert np.array_equal(orc.depad(y, child, x.shape[1]), x)


def test_sgemm(orc):
  rng = np.random.default_rng(4)
  A, B = rng.standard_normal((7, 13)).astype(np.float32), rng.standard_normal((13, 9)).astype(np.float32)
  assert np.allclose(orc.sgemm(A, B), A.astype(np.float64) @ B, atol=1e-5)
  assert np.allclose(orc.sgemm(A.T.copy(), B, transA=True), A.astype(np.float64) @ B, atol=1e-5)
  assert np.allclose(orc.sgemm(A, B.T.copy(), transB=True), A.astype(np.float64) @ B, atol=1e-5)


def morton_to_grid(x, depth):
  """[C, 8^depth] in Morton order -> [C, 2^d, 2^d, 2^d] indexed (x, y, z)."""
  n = 8 ** depth
  idx = np.arange(n)
  xs = np.zeros(n, np.int64); ys = np.zeros(n, np.int64); zs = np.zeros(n, np.int64)
  for i in range(depth):
    xs |= ((idx >> (3 * i + 2)) & 1) << i
    ys |= ((idx >> (3 * i + 1)) & 1) << i
    zs |= ((idx >> (3 * i)) & 1) << i
  return xs, ys, zs


@pytest.mark.parametrize("depth", [1, 2])
def test_conv_full_layer_is_dense_conv3d(orc, samples, depth):
  """On a full layer the octree conv is a zero-padded dense 3-D cross-correlation
  (library routine: torch.nn.functional.conv3d), after Morton -> xyz reordering."""
  blob = orc.octree_batch([samples["octree_1"]])
  n, S = 8 ** depth, 2 ** depth
  rng = np.random.default_rng(5)
  Ci, Co = 3, 4
  x = rng.standard_normal((Ci, n)).astype(np.float32)
  w = rng.standard_normal((Co, Ci * 27)).astype(np.float32)
  y = orc.octree_conv(x, w, blob, depth, Co, [3, 3, 3], 1)
  xs, ys, zs = morton_to_grid(x, depth)
  grid = np.zeros((1, Ci, S, S, S), np.float32)
  grid[0][:, xs, ys, zs] = x
  # weight column c*27 + (dx*9 + dy*3 + dz) -> kernel [Co, Ci, dx, dy, dz]
  wk = torch.from_numpy(w.reshape(Co, Ci, 3, 3, 3))
  dense = torch.nn.functional.conv3d(torch.from_numpy(grid), wk, padding=1)[0].numpy()
  assert np.allclose(y, dense[:, xs, ys, zs], atol=1e-5)
  # deconv with the same (transposed-role) weights is the adjoint of conv
  wd = rng.standard_normal((Co, Ci * 27)).astype(np.float32)   # deconv: [channel_in=Co, num_output*K]
  g = rng.standard_normal((Co, n)).astype(np.float32)
  yd = orc.octree_deconv(g, wd, blob, depth, Ci, [3, 3, 3], 1)
  yc = orc.octree_conv(x, wd, blob, depth, Co, [3, 3, 3], 1)
  assert np.isclose(np.vdot(yc.astype(np.float64), g), np.vdot(x.astype(np.float64), yd), rtol=1e-5)


@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("ks", [[3, 3, 3], [2, 2, 2], [3, 1, 1], [3, 3, 1], [1, 1, 1]])
def test_conv_equals_col_times_weights_and_nempty_identity(orc, samples, ks, stride):
  """pytorch/test/test_octree_conv.py:10-90: OctreeConv == W x octree2col (OctreeConvFast), and
  nempty conv == mask -> conv -> select."""
  blob = orc.octree_batch([samples["octree_1"], samples["octree_2"]])
  b = OctreeBlob(blob)
  d, Ci, Co = 4, 3, 5
  H = int(b.nnum[d])
  assert H == 152
  K = ks[0] * ks[1] * ks[2]
  rng = np.random.default_rng(6)
  x = rng.uniform(-1, 1, (Ci, H)).astype(np.float32)
  w = rng.uniform(-0.3, 0.3, (Co, Ci * K)).astype(np.float32)
  neigh = b.prop("neigh", d).reshape(-1)
  height = H if stride == 1 else H // 8
  col = orc.octree2col(x, ks, stride, neigh, height).reshape(Ci * K, height)
  y = orc.octree_conv(x, w, blob, d, Co, ks, stride)
  assert np.allclose(y, w.astype(np.float64) @ col, atol=1e-5)
  mask3 = b.prop("child", d) >= 0
  d_out = d if stride == 1 else d - 1
  mask4 = b.prop("child", d_out) >= 0
  y3 = orc.octree_conv(x[:, mask3], w, blob, d, Co, ks, stride, nempty=True)
  y4 = orc.octree_conv(x * mask3, w, blob, d, Co, ks, stride)
  if stride == 2:
    y4 = orc.pad(y4, b.prop("child", d_out))
  assert np.allclose(y3, y4[:, mask4], atol=1e-6)


@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("ks", [[3, 3, 3], [2, 2, 2], [3, 1, 1]])
def test_deconv_is_adjoint_of_conv(orc, samples, ks, stride):
  blob = orc.octree_batch([samples["octree_2"], samples["octree_1"]])
  b = OctreeBlob(blob)
  Ci, Co, K = 3, 4, ks[0] * ks[1] * ks[2]
  rng = np.random.default_rng(7)
  for nempty in (False, True):
    # conv maps depth dc -> (dc or dc-1); deconv with the same W maps back
    dc = 4
    dd = dc if stride == 1 else dc - 1
    hx = int(b.nnum_nempty[dc] if nempty else b.nnum[dc])
    w = rng.standard_normal((Co, Ci * K)).astype(np.float32)
    x = rng.standard_normal((Ci, hx)).astype(np.float32)
    y = orc.octree_conv(x, w, blob, dc, Co, ks, stride, nempty)
    g = rng.standard_normal(y.shape).astype(np.float32)
    back = orc.octree_deconv(g, w, blob, dd, Ci, ks, stride, nempty)
    assert back.shape == x.shape
    assert np.isclose(np.vdot(y.astype(np.float64), g), np.vdot(x.astype(np.float64), back), rtol=1e-4)


def test_pool_literals(orc):
  """pytorch/test/test_octree_pool.py:10-60."""
  data = np.array([[1.1, 2.2, 3.3, 4.4, 5.5, 6.6, 7.7, 8.8], [8.1, 7.2, 6.3, 5.4, 4.5, 3.6, 2.7, 1.8]], np.float32)
  data = np.concatenate([data, data], axis=1)
  top, mask = orc.max_pool(data)
  assert np.array_equal(mask, [[7, 15], [0, 8]])
  assert np.array_equal(top, np.array([[8.8, 8.8], [8.1, 8.1]], np.float32))
  un = orc.max_unpool(data[:, [0, 8]] * 0 + np.array([[1.1, 1.1], [8.1, 8.1]], np.float32), mask)
  exp = np.zeros((2, 16), np.float32)
  exp[0, 7] = exp[0, 15] = 1.1
  exp[1, 0] = exp[1, 8] = 8.1
  assert np.array_equal(un, exp)
  m2 = np.array([[1, 9], [2, 10]], np.int32)
  un2 = orc.max_unpool(np.array([[1.1, 1.1], [8.1, 8.1]], np.float32), m2)
  exp2 = np.zeros((2, 16), np.float32)
  exp2[0, 1] = exp2[0, 9] = 1.1
  exp2[1, 2] = exp2[1, 10] = 8.1
  assert np.array_equal(un2, exp2)
  assert np.array_equal(orc.mask_pool(data, m2), np.array([[2.2, 2.2], [6.3, 6.3]], np.float32))


def test_pool_vs_numpy(orc):
  x = np.random.default_rng(8).integers(-3, 3, (6, 8 * 40)).astype(np.float32)  # many ties
  top, mask = orc.max_pool(x)
  r = x.reshape(6, -1, 8)
  assert np.array_equal(top, r.max(2))
  assert np.array_equal(mask, r.argmax(2) + 8 * np.arange(40))  # first maximum wins


def test_kernels_vs_compiled_reference(orc, ref, batch4):
  _, b = batch4
  rng = np.random.default_rng(9)
  d = 4
  H, Hne = int(b.nnum[d]), int(b.nnum_nempty[d])
  neigh, child = b.prop("neigh", d).reshape(-1), b.prop("child", d)
  ichild = np.zeros(Hne, np.int32)
  ichild[child[child >= 0]] = np.nonzero(child >= 0)[0]
  x = rng.standard_normal((4, H)).astype(np.float32)
  xn = rng.standard_normal((4, Hne)).astype(np.float32)
  for ks in ([3, 3, 3], [2, 2, 2], [3, 1, 1], [1, 3, 1], [1, 1, 3], [3, 3, 1], [3, 1, 3], [1, 3, 3], [1, 1, 1]):
    assert np.array_equal(orc.get_ni(ks), ref.get_ni(ks))
    for stride in (1, 2):
      h = H if stride == 1 else H // 8
      c1, c2 = orc.octree2col(x, ks, stride, neigh, h), ref.octree2col(x, ks, stride, neigh, h)
      assert np.array_equal(c1, c2)
      assert np.array_equal(orc.col2octree(c1, ks, stride, neigh, h), ref.col2octree(c1, ks, stride, neigh, h))
      hp = Hne if stride == 1 else H // 8
      p1 = orc.octree2colP(xn, ks, stride, neigh, child, ichild, hp)
      assert np.array_equal(p1, ref.octree2colP(xn, ks, stride, neigh, child, ichild, hp))
      assert np.array_equal(orc.col2octreeP(p1, ks, stride, neigh, child, ichild, hp, Hne),
                            ref.col2octreeP(p1, ks, stride, neigh, child, ichild, hp, Hne))
  assert np.array_equal(orc.get_parent(), ref.get_parent())
  assert np.array_equal(orc.get_dis(), ref.get_dis())
  t1, m1 = orc.max_pool(x)
  t2, m2 = ref.max_pool(x)
  assert np.array_equal(t1, t2) and np.array_equal(m1, m2)
  assert np.array_equal(orc.max_unpool(t1, m1), ref.max_unpool(t1, m1))
  assert np.array_equal(orc.mask_pool(x, m1), ref.mask_pool(x, m1))
  assert np.array_equal(orc.pad(xn, child, 2.0), ref.pad(xn, child, 2.0))
  assert np.array_equal(orc.depad(x, child, Hne), ref.depad(x, child, Hne))
  for dd in (1, 2, 3):
    assert np.array_equal(orc.calc_neigh_full(dd, 2), ref.calc_neigh_full(dd, 2))
    assert np.array_equal(orc.generate_key_full(dd, 2), ref.generate_key_full(dd, 2))
  n5 = int(b.nnum[5])
  assert np.array_equal(orc.calc_neigh_sparse(neigh, child, n5), ref.calc_neigh_sparse(neigh, child, n5))
  k4 = b.prop("key", 4)
  assert np.array_equal(orc.generate_key_child(k4, child, n5), ref.generate_key_child(k4, child, n5))
  lab = rng.integers(0, 3, 100).astype(np.int32)
  assert np.array_equal(orc.generate_label(lab, 1)[0], ref.generate_label(lab, 1)[0])
  keys = np.unique(rng.integers(0, 1 << 50, 500).astype(np.uint64))
  q = rng.integers(0, 1 << 50, 100).astype(np.uint64)
  assert np.array_equal(orc.search_key(keys, q), ref.search_key(keys, q))
  assert np.array_equal(orc.xyz2key(keys, 9), ref.xyz2key(keys, 9))
  assert np.array_equal(orc.key2xyz(keys, 9), ref.key2xyz(keys, 9))
  assert np.array_equal(orc.key2idx(keys), ref.key2idx(keys))


@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("ks", [[3, 3, 3], [2, 2, 2], [3, 1, 1], [1, 1, 1]])
def test_conv_grads_are_the_adjoints(orc, samples, ks, stride):
  """The op is bilinear: <grad_w, W'> == <grad_out, conv(x; W')> for every W' and
  <grad_data, x'> == <grad_out, conv(x'; W)> for every x' (OctreeConvGradOp,
  pytorch/cpp/octree_conv.cpp:159-189); the same for the deconvolution."""
  blob = orc.octree_batch([samples["octree_2"], samples["octree_1"]])
  b = OctreeBlob(blob)
  Ci, Co, K = 3, 4, ks[0] * ks[1] * ks[2]
  rng = np.random.default_rng(8)
  dot = lambda a, c: float(np.vdot(a.astype(np.float64), c.astype(np.float64)))
  for nempty in (False, True):
    dc = 4
    hx = int(b.nnum_nempty[dc] if nempty else b.nnum[dc])
    x = rng.standard_normal((Ci, hx)).astype(np.float32)
    w = rng.standard_normal((Co, Ci * K)).astype(np.float32)
    y = orc.octree_conv(x, w, blob, dc, Co, ks, stride, nempty)
    g = rng.standard_normal(y.shape).astype(np.float32)
    gd, gw = orc.octree_conv_grad(x, w, g, blob, dc, Co, ks, stride, nempty)
    assert gd.shape == x.shape and gw.shape == w.shape
    for _ in range(3):
      w2 = rng.standard_normal(w.shape).astype(np.float32)
      x2 = rng.standard_normal(x.shape).astype(np.float32)
      assert np.isclose(dot(gw, w2), dot(g, orc.octree_conv(x, w2, blob, dc, Co, ks, stride, nempty)), rtol=1e-4)
      assert np.isclose(dot(gd, x2), dot(g, orc.octree_conv(x2, w, blob, dc, Co, ks, stride, nempty)), rtol=1e-4)
    # a single weight entry: grad_w[m, j] == <grad_out, conv(x; e_mj)>
    m, j = 2, (Ci * K) // 2
    e = np.zeros_like(w); e[m, j] = 1.0
    assert np.isclose(gw[m, j], dot(g, orc.octree_conv(x, e, blob, dc, Co, ks, stride, nempty)), rtol=1e-4, atol=1e-5)
    # deconvolution: input at dd, weights [Cin_d, Cout_d * K]
    dd = dc if stride == 1 else dc - 1
    hd = int(b.nnum_nempty[dd] if (nempty or stride == 2) else b.nnum[dd])
    xd = rng.standard_normal((Co, hd)).astype(np.float32)
    wd = rng.standard_normal((Co, Ci * K)).astype(np.float32)
    yd = orc.octree_deconv(xd, wd, blob, dd, Ci, ks, stride, nempty)
    gy = rng.standard_normal(yd.shape).astype(np.float32)
    gd, gw = orc.octree_deconv_grad(xd, wd, gy, blob, dd, Ci, ks, stride, nempty)
    assert gd.shape == xd.shape and gw.shape == wd.shape
    for _ in range(3):
      w2 = rng.standard_normal(wd.shape).astype(np.float32)
      x2 = rng.standard_normal(xd.shape).astype(np.float32)
      assert np.isclose(dot(gw, w2), dot(gy, orc.octree_deconv(xd, w2, blob, dd, Ci, ks, stride, nempty)), rtol=1e-4)
      assert np.isclose(dot(gd, x2), dot(gy, orc.octree_deconv(x2, wd, blob, dd, Ci, ks, stride, nempty)), rtol=1e-4)


def test_conv_grads_full_layer_match_dense_autograd(orc, samples):
  """On a full layer the gradients are those of torch's dense conv3d."""
  depth = 2
  blob = orc.octree_batch([samples["octree_1"]])
  n, S = 8 ** depth, 2 ** depth
  rng = np.random.default_rng(9)
  Ci, Co = 3, 4
  x = rng.standard_normal((Ci, n)).astype(np.float32)
  w = rng.standard_normal((Co, Ci * 27)).astype(np.float32)
  g = rng.standard_normal((Co, n)).astype(np.float32)
  gd, gw = orc.octree_conv_grad(x, w, g, blob, depth, Co, [3, 3, 3], 1)
  xs, ys, zs = morton_to_grid(x, depth)
  grid = np.zeros((1, Ci, S, S, S), np.float32)
  grid[0][:, xs, ys, zs] = x
  gg = np.zeros((1, Co, S, S, S), np.float32)
  gg[0][:, xs, ys, zs] = g
  xt = torch.from_numpy(grid).requires_grad_(True)
  wt = torch.from_numpy(w.reshape(Co, Ci, 3, 3, 3).copy()).requires_grad_(True)
  torch.nn.functional.conv3d(xt, wt, padding=1).backward(torch.from_numpy(gg))
  assert np.allclose(gw, wt.grad.numpy().reshape(Co, Ci * 27), atol=1e-4)
  assert np.allclose(gd, xt.grad.numpy()[0][:, xs, ys, zs], atol=1e-4)
