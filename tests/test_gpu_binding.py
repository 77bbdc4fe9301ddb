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
