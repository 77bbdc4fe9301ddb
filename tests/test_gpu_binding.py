"""The compiled ATen binding (o-cnn_amd/binding/ocnn_aten.cpp: the bodies that replace
pytorch/cpp/*.cpp, registered under the reference's names) against the ctypes mirror nn.py.
Both go through the same C interface, so every result must be equal bit for bit; nn.py in turn
is what the parity tests compare with the oracle.  One case is the binding's own: the host copy
of the octree header must follow the blob tensor, not its device address."""
import gc

import numpy as np
import pytest
import torch

from oracle.checker import OctreeBlob, make_points_blob

pytestmark = pytest.mark.gpu


def T(a):
  return torch.from_numpy(np.ascontiguousarray(a))


@pytest.fixture(scope="module")
def aten(oc):
  return oc.lib.aten()


@pytest.fixture(scope="module")
def tree(oc, orc, synthetic):
  pbs = [make_points_blob(*synthetic.shape_cloud(4000, 51 + i)[:2]) for i in range(3)]
  host = orc.octree_batch([orc.points2octree(p, 6, 2) for p in pbs])
  return {"host": host, "dev": T(host).cuda(), "blob": OctreeBlob(host)}


def same(a, b):
  return a.dtype == b.dtype and a.shape == b.shape and torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nempty", [False, True])
def test_conv_family_equals_the_mirror(oc, aten, tree, dtype, nempty):
  b, dev = tree["blob"], tree["dev"]
  g = torch.Generator(device="cuda").manual_seed(3)
  for d, ks, stride, cin, cout in ((5, [3, 3, 3], 1, 16, 32), (5, [2, 2, 2], 2, 16, 24), (4, [3, 1, 1], 1, 5, 7),
                                   (5, [3], 1, 8, 8)):
    K = int(np.prod(ks)) if len(ks) == 3 else ks[0] ** 3
    h = int(b.nnum_nempty[d] if nempty else b.nnum[d])
    x = torch.randn(1, cin, h, 1, device="cuda", generator=g).to(dtype)
    w = (torch.randn(cout, cin * K, device="cuda", generator=g) * 0.05).to(dtype)
    y = aten.octree_conv(x, w, dev, d, cout, ks, stride, nempty)
    assert same(y, oc.nn.octree_conv(x, w, dev, d, cout, ks, stride, nempty)), (d, ks, stride)
    # deconvolution: at stride 2 the input lives one level up
    dd = d - 1 if stride == 2 else d
    hd = int(b.nnum_nempty[dd] if (nempty or stride == 2) else b.nnum[dd])
    xd = torch.randn(1, cin, hd, 1, device="cuda", generator=g).to(dtype)
    wd = (torch.randn(cin, cout * K, device="cuda", generator=g) * 0.05).to(dtype)
    yd = aten.octree_deconv(xd, wd, dev, dd, cout, ks, stride, nempty)
    assert same(yd, oc.nn.octree_deconv(xd, wd, dev, dd, cout, ks, stride, nempty)), (d, ks, stride)
    if dtype == torch.float32:
      gy = torch.randn_like(y)
      ga, gw = aten.octree_conv_grad(x, w, dev, gy, d, cout, ks, stride, nempty)
      ra, rw = oc.nn.octree_conv_grad(x, w, dev, gy, d, cout, ks, stride, nempty)
      assert same(ga, ra) and same(gw, rw)
      gyd = torch.randn_like(yd)
      ga, gw = aten.octree_deconv_grad(xd, wd, dev, gyd, dd, cout, ks, stride, nempty)
      ra, rw = oc.nn.octree_deconv_grad(xd, wd, dev, gyd, dd, cout, ks, stride, nempty)
      assert same(ga, ra) and same(gw, rw)
      bias = torch.randn(cout, device="cuda", generator=g)
      yf = aten.octree_conv_bn_relu(x, w, bias, dev, d, cout, ks, stride, nempty, False, True)
      assert same(yf, oc.nn.octree_conv_fused(x, w, bias, True, dev, d, cout, ks, stride, nempty))


def test_col_pad_pool_equal_the_mirror(oc, aten, tree):
  b, dev = tree["blob"], tree["dev"]
  d = 5
  H, Hne = int(b.nnum[d]), int(b.nnum_nempty[d])
  g = torch.Generator(device="cuda").manual_seed(4)
  for dtype in (torch.float32, torch.bfloat16):
    x = torch.randn(1, 6, H, 1, device="cuda", generator=g).to(dtype)
    xn = torch.randn(1, 6, Hne, 1, device="cuda", generator=g).to(dtype)
    for ks, stride in (([3, 3, 3], 1), ([2, 2, 2], 2), ([3, 1, 3], 1), ([3, 3, 3], 2)):
      for nempty, src in ((False, x), (True, xn)):
        col = aten.octree2col(src, dev, d, ks, stride, nempty)
        assert same(col, oc.nn.octree2col(src, dev, d, ks, stride, nempty)), (ks, stride, nempty)
        if dtype == torch.float32:
          back = aten.col2octree(col, dev, d, ks, stride, nempty)
          assert same(back, oc.nn.col2octree(col, dev, d, ks, stride, nempty)), (ks, stride, nempty)
    assert same(aten.octree_pad(xn, dev, d), oc.nn.octree_pad(xn, dev, d))
    assert same(aten.octree_pad(xn, dev, d, 2.5), oc.nn.octree_pad(xn, dev, d, 2.5))
    assert same(aten.octree_depad(x, dev, d), oc.nn.octree_depad(x, dev, d))
    top, mask = aten.octree_max_pool(x, dev, d)
    rt, rm = oc.nn.octree_max_pool(x, dev, d)
    assert same(top, rt) and same(mask, rm)
    assert same(aten.octree_max_unpool(top, mask, dev, d), oc.nn.octree_max_unpool(rt, rm, dev, d))
    assert same(aten.octree_mask_pool(x, mask, dev, d), oc.nn.octree_mask_pool(x, rm, dev, d))
  with pytest.raises(RuntimeError):
    aten.octree_pad(x, dev, d)          # wrong height
  with pytest.raises(RuntimeError):
    aten.octree_max_pool(xn, dev, d)


def test_keys_and_properties_equal_the_mirror(oc, aten, tree):
  b, dev = tree["blob"], tree["dev"]
  d = 5
  for name in ("key", "xyz", "child", "neigh", "feature", "node_num", "node_num_ne", "node_num_cum", "batch_size",
               "depth", "full_depth"):
    for dep in ((d, 6, 0) if name.startswith("node_num") else (d, 6) if name != "feature" else (6,)):
      assert same(aten.octree_property(dev, name, dep), oc.nn.octree_property(dev, name, dep)), (name, dep)
  key = oc.nn.octree_property(dev, "key", d)
  xyz = aten.octree_key2xyz(key, d)
  assert same(xyz, oc.nn.octree_key2xyz(key, d)) and same(aten.octree_xyz2key(xyz, d), key)
  query = torch.cat([key[::3], key[:50] + (1 << 40)])
  for nempty in (False, True):
    assert same(aten.octree_search_key(query, dev, d, False, nempty), oc.nn.octree_search_key(query, dev, d, False, nempty))
  assert same(aten.octree_search_key(xyz[::5], dev, d, True, False), oc.nn.octree_search_key(xyz[::5], dev, d, True, False))


def grow_chain(mod, labels):
  """octree_new -> grow (full levels) -> [update, grow] with the given split labels per depth."""
  o = mod.octree_new(2, 3, True, 0)
  o = mod.octree_grow(o, 1, True)
  o = mod.octree_grow(o, 2, True)
  for d, lab in labels:
    o = mod.octree_update(o, lab, d, 1)
    o = mod.octree_grow(o, d + 1, False)
  return o


def test_grow_chain_equals_the_mirror(oc, aten):
  g = torch.Generator(device="cuda").manual_seed(5)
  labels = []
  n = 2 * 64
  for d in (2, 3, 4):
    lab = (torch.rand(n, device="cuda", generator=g) < 0.5).to(torch.int32)
    labels.append((d, lab))
    n = 8 * int(lab.sum())
  a, r = grow_chain(aten, labels), grow_chain(oc.nn, labels)
  assert same(a, r)
  x = torch.randn(1, 4, n, 1, device="cuda", generator=g)
  w = torch.randn(8, 4 * 27, device="cuda", generator=g)
  assert same(aten.octree_conv(x, w, a, 5, 8, [3, 3, 3], 1, False), oc.nn.octree_conv(x, w, r, 5, 8, [3, 3, 3], 1, False))


def test_header_copy_follows_the_tensor_on_the_device(oc, orc, aten, tree, samples):
  """Two different octrees, one after the other at the SAME device address, with an in-place
  octree_update in between: every call must see the header of the blob it is given (a copy
  keyed by the address would hand the second octree the first one's node counts)."""
  host_a = tree["host"]
  host_b = orc.octree_batch([samples[n] for n in ("octree_1", "octree_2")])
  assert host_a.size > host_b.size
  ia, ib = OctreeBlob(host_a), OctreeBlob(host_b)
  g = torch.Generator(device="cuda").manual_seed(6)

  def conv_on(octree, blob, d):
    h = int(blob.nnum[d])
    x = torch.randn(1, 4, h, 1, device="cuda", generator=g)
    w = torch.randn(6, 4 * 27, device="cuda", generator=g)
    got = aten.octree_conv(x, w, octree, d, 6, [3, 3, 3], 1, False)
    assert same(got, oc.nn.octree_conv(x, w, octree.clone(), d, 6, [3, 3, 3], 1, False))
    return h

  a = torch.empty(host_a.size, dtype=torch.uint8, device="cuda")
  a.copy_(T(host_a))
  addr = a.data_ptr()
  conv_on(a, ia, 5)
  assert np.array_equal(aten.octree_header(a).numpy(), host_a[:716])
  # in-place update of the children of depth 5 on the blob itself: nnum_nempty[5] changes
  lab = (torch.rand(int(ia.nnum[5]), device="cuda", generator=g) < 0.3).to(torch.int32)
  aten.octree_update_(a, lab, 5, 1)
  hdr = aten.octree_header(a).numpy()
  assert np.array_equal(hdr, a[:716].cpu().numpy()) and not np.array_equal(hdr, host_a[:716])
  assert int(np.frombuffer(hdr.tobytes(), np.int32, 16, 176)[5]) == int(lab.sum())
  del a
  gc.collect()
  # the allocator serves the next request of that size class from the block just freed
  b_full = torch.empty(host_a.size, dtype=torch.uint8, device="cuda")
  if b_full.data_ptr() != addr:
    pytest.skip("the allocator did not hand the address out again")
  b = b_full[:host_b.size]
  b.copy_(T(host_b))
  assert b.data_ptr() == addr
  assert np.array_equal(aten.octree_header(b).numpy(), host_b[:716])
  conv_on(b, ib, 3)
  top, mask = aten.octree_max_pool(torch.randn(1, 2, int(ib.nnum[3]), 1, device="cuda", generator=g), b, 3)
  assert top.shape[2] == int(ib.nnum[3]) // 8
  # a write through torch into the same tensor (version counter) is seen too
  b_full.copy_(T(host_a))
  assert np.array_equal(aten.octree_header(b_full).numpy(), host_a[:716])
  conv_on(b_full, ia, 4)


def cloud(synthetic, n, seed, features=False, labels=False):
  pts, nrm = synthetic.shape_cloud(n, seed)[:2]
  rng = np.random.default_rng(seed)
  feat = rng.standard_normal((pts.shape[0], 2)).astype(np.float32) if features else None
  lab = rng.integers(0, 5, (pts.shape[0], 1)).astype(np.float32) if labels else None
  return pts, nrm, feat, lab


def test_points_ops_equal_the_mirror(oc, aten, synthetic):
  pts, nrm, feat, lab = cloud(synthetic, 3000, 61, features=True, labels=True)
  args = [T(a).cuda() for a in (pts, nrm, feat, lab)]
  p = aten.points_new(*args)
  assert same(p, oc.nn.points_new(*args))
  assert np.array_equal(p.cpu().numpy(), make_points_blob(pts, nrm, feat, lab))
  # without the optional arrays: empty tensors, as the reference's Python side passes them
  none = torch.zeros(0)
  p2 = aten.points_new(args[0], args[1], none, none)
  assert np.array_equal(p2.cpu().numpy(), make_points_blob(pts, nrm))
  for name in ("xyz", "normal", "feature", "label"):
    assert same(aten.points_property(p, name), oc.nn.points_property(p, name)), name
  assert aten.points_property(p2, "feature") is None and aten.points_property(p2, "label") is None
  for name in ("xyz", "xyzi", "normal"):
    assert same(aten.points_batch_property([p, p2, p], name), oc.nn.points_batch_property([p, p2, p], name)), name
  with pytest.raises(RuntimeError):
    aten.points_batch_property([p, p2], "feature")
  new_nrm = torch.randn(pts.shape[0], 3, device="cuda")
  assert same(aten.points_set_property(p, new_nrm, "normal"), oc.nn.points_set_property(p, new_nrm, "normal"))
  with pytest.raises(RuntimeError):
    aten.points_set_property(p2, torch.zeros(pts.shape[0], 2, device="cuda"), "feature")
  with pytest.raises(RuntimeError):
    aten.points_set_property(p, torch.zeros(pts.shape[0] - 1, 3, device="cuda"), "normal")
  # transforms: device clouds and host clouds (the reference keeps clouds on the host) give the same bytes
  for src in (p, p.cpu()):
    for method in ("sphere", "box"):
      assert aten.bounding_sphere(src, method) == oc.nn.bounding_sphere(p, method)
    r, c = 0.8, [0.1, -0.05, 0.02]
    assert same(aten.normalize_points(src, r, c), oc.nn.normalize_points(p, r, c))
    for axis in ("", "y", "xyz"):
      tr = ([0.3, -0.2, 1.1], [1.1, 0.9, 1.0], [0.05, 0.0, -0.02], 0.01, axis)
      assert same(aten.transform_points(src, *tr), oc.nn.transform_points(p, *tr)), axis
    assert same(aten.transform_points(src, [0.5], [0.9], [0.0], 0.0, ""), oc.nn.transform_points(p, [0.5], [0.9], [0.0], 0.0, ""))
    got, exp = aten.clip_points(src, [-0.5, -0.4, -0.6], [0.5, 0.6, 0.3]), oc.nn.clip_points(p, [-0.5, -0.4, -0.6], [0.5, 0.6, 0.3])
    assert same(got[0], exp[0]) and same(got[1], exp[1]) and 0 < int(got[1].sum()) < pts.shape[0]
  with pytest.raises(RuntimeError):
    aten.points_property(torch.zeros(200, dtype=torch.uint8), "xyz")   # no magic string


@pytest.mark.parametrize("opts", [
    dict(depth=6, full_depth=2),
    dict(depth=5, full_depth=3, node_dis=True, split_label=True, save_pts=True),
    dict(depth=6, full_depth=2, key2xyz=True),
    dict(depth=6, full_depth=2, node_dis=True, node_feature=True),
    dict(depth=6, full_depth=2, node_dis=True, adaptive=True, adp_depth=3, th_normal=0.2, th_distance=1.5),
    dict(depth=6, full_depth=2, node_dis=True, adaptive=True, adp_depth=3, extrapolate=True),
], ids=["plain", "dis_split_pts", "key2xyz", "node_feature", "adaptive", "adaptive_extrapolate"])
def test_build_and_batch_equal_the_mirror(oc, aten, synthetic, opts):
  order = ("depth", "full_depth", "node_dis", "node_feature", "split_label", "adaptive", "adp_depth", "th_normal",
           "th_distance", "extrapolate", "save_pts", "key2xyz")
  full = dict(full_depth=2, node_dis=False, node_feature=False, split_label=False, adaptive=False, adp_depth=4,
              th_normal=0.1, th_distance=2.0, extrapolate=False, save_pts=False, key2xyz=False)
  full.update(opts)
  clouds = [T(make_points_blob(*cloud(synthetic, 2500 + 300 * i, 70 + i)[:2])) for i in range(3)]
  got, exp = [], []
  for i, c in enumerate(clouds):
    src = c.cuda() if i != 1 else c                     # one cloud comes from the host
    got.append(aten.points2octree(src, *[full[k] for k in order]))
    exp.append(oc.nn.points2octree(c.cuda(), **full))
    assert same(got[-1], exp[-1]), i
    assert np.array_equal(aten.octree_header(got[-1]).numpy(), exp[-1][:716].cpu().numpy())
  merged, merged_exp = aten.octree_batch(got), oc.nn.octree_batch(exp)
  assert same(merged, merged_exp)
  assert np.array_equal(aten.octree_header(merged).numpy(), merged_exp[:716].cpu().numpy())
  assert same(aten.octree_batch([g.cpu() for g in got]), merged_exp)   # host blobs, as a data loader hands them over
  d = full["depth"]
  assert same(aten.octree_property(merged, "feature", d), oc.nn.octree_property(merged_exp, "feature", d))
  with pytest.raises(RuntimeError):
    aten.points2octree(clouds[0].cuda(), 0, 2, False, False, False, False, 4, 0.1, 2.0, False, False, False)


def test_samples_set_property_keys_scan_align_equal_the_mirror(oc, aten, samples, tree, synthetic):
  names = ["octree_%d" % i for i in range(1, 7)]
  for a, r, n in zip(aten.octree_samples(names), oc.nn.octree_samples(names), names):
    assert same(a, r) and np.array_equal(a.numpy(), samples[n]), n
  with pytest.raises(RuntimeError):
    aten.octree_samples(["octree_7"])
  dev, b = tree["dev"], tree["blob"]
  d = 6
  feat = oc.nn.octree_property(dev, "feature", d)
  new = torch.randn_like(feat)
  got = aten.octree_set_property(dev, new, d)
  assert same(got, oc.nn.octree_set_property(dev, new, d))
  assert same(aten.octree_property(got, "feature", d), new) and same(aten.octree_property(dev, "feature", d), feat)
  with pytest.raises(RuntimeError):
    aten.octree_set_property(dev, new[:, :, :-1], d)
  xyz = torch.randint(0, 64, (500, 4), dtype=torch.int16, device="cuda")
  key = aten.octree_encode_key(xyz)
  assert same(key, oc.nn.octree_encode_key(xyz)) and same(aten.octree_decode_key(key), xyz)
  with pytest.raises(RuntimeError):
    aten.octree_encode_key(xyz[:, :3])
  # scan: one octree, two view directions; then features of the scanned octree on the nodes of the whole one
  single = aten.points2octree(T(make_points_blob(*cloud(synthetic, 6000, 81)[:2])).cuda(), 6, 2, True, False, False, False,
                              4, 0.1, 2.0, False, False, False)
  axis = [0.0, 0.0, 1.0, 0.6, 0.0, 0.8]
  part = aten.octree_scan(single, axis, 1.0)
  assert same(part, oc.nn.octree_scan(single, axis, 1.0)) and same(aten.octree_scan(single, axis[:3]), oc.nn.octree_scan(single, axis[:3]))
  assert np.array_equal(aten.octree_header(part).numpy(), part[:716].cpu().numpy())
  whole, part_b = aten.octree_batch([single]), aten.octree_batch([part])
  for dep in (4, 6):
    h = int(aten.octree_property(part_b, "node_num", dep)[0])
    assert 0 < h < int(aten.octree_property(whole, "node_num", dep)[0]) or dep == 4
    x = torch.randn(1, 5, h, 1, device="cuda")
    (ga, gi), (ea, ei) = aten.octree_align(x, part_b, whole, dep), oc.nn.octree_align(x, part_b, whole, dep)
    assert same(ga, ea) and same(gi, ei) and int((gi >= 0).sum()) == h
    grad = torch.randn_like(ga)
    assert same(aten.octree_align_grad(grad, gi), oc.nn.octree_align_grad(grad, gi))
  with pytest.raises(RuntimeError):
    aten.octree_align(torch.randn(1, 5, 7, 1, device="cuda"), part_b, whole, 6)
