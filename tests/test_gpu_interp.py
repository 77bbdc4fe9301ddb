"""GPU parity of octree_align, of the fused nearest / trilinear point interpolation and of the
point-cloud property accessors against the oracle restatements (oracle/interp.py), including the
reference's own literal cases (pytorch/test/test_octree_align.py, test_octree_trilinear.py,
test_points_property.py).  Indices bit-exact; fp32 values within 1e-5."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import interp
from oracle.checker import OctreeBlob, make_points_blob

pytestmark = pytest.mark.gpu


def T(a):
  return torch.from_numpy(np.ascontiguousarray(a))


def test_align_reference_cases_with_gradients(oc, orc, samples):
  one = oc.nn.octree_batch([T(samples["octree_1"])])
  two = oc.nn.octree_batch([T(samples["octree_1"]), T(samples["octree_1"])])
  A = oc.autograd.octree_align
  x = torch.rand(1, 3, 16, 1).cuda().requires_grad_()
  out, idx = A(x, two, two, 5)
  out.sum().backward()
  assert torch.equal(out, x) and idx.cpu().tolist() == list(range(16)) and torch.all(x.grad == 1)
  x = torch.rand(1, 3, 8, 1).cuda().requires_grad_()
  out, idx = A(x, one, two, 5)
  out.sum().backward()
  assert torch.equal(out, torch.cat([x, torch.zeros(1, 3, 8, 1).cuda()], dim=2))
  assert idx.cpu().tolist() == list(range(8)) and torch.all(x.grad == 1)
  x = torch.rand(1, 3, 16, 1).cuda().requires_grad_()
  out, idx = A(x, two, one, 5)
  out.sum().backward()
  assert torch.equal(out, x[:, :, :8]) and idx.cpu().tolist() == list(range(8)) + [-1] * 8
  assert torch.equal(x.grad, torch.cat([torch.ones(1, 3, 8, 1), torch.zeros(1, 3, 8, 1)], 2).cuda())


def test_align_between_different_octrees(oc, orc, synthetic):
  """Encoder octree -> decoder octree of another shape (the skip connections of
  pytorch/ocnn/ounet.py:82)."""
  pa = make_points_blob(*synthetic.shape_cloud(3000, 11)[:2])
  pb = make_points_blob(*synthetic.shape_cloud(3000, 12)[:2])
  ha = orc.octree_batch([orc.points2octree(pa, 5, 2), orc.points2octree(pb, 5, 2)])
  hb = orc.octree_batch([orc.points2octree(pb, 5, 2, key2xyz=True), orc.points2octree(pa, 5, 2, key2xyz=True)])
  rng = np.random.default_rng(0)
  for d in (3, 4, 5):
    x = rng.standard_normal((7, int(OctreeBlob(ha).nnum[d]))).astype(np.float32)
    exp, eidx = interp.octree_align(orc, x, ha, hb, d)
    out, idx = oc.nn.octree_align(T(x).cuda().view(1, 7, -1, 1), T(ha).cuda(), T(hb).cuda(), d)
    assert np.array_equal(idx.cpu().numpy(), eidx) and 0 < (eidx >= 0).sum() < eidx.size
    assert np.array_equal(out.cpu().numpy().reshape(exp.shape), exp)
    # the sum behind the transfer (`deconv + skip`, pytorch/ocnn/ounet.py:111) in the same pass
    base = rng.standard_normal(exp.shape).astype(np.float32)
    acc = T(base).cuda().view(1, 7, -1, 1)
    got, idx2 = oc.nn.octree_align(T(x).cuda().view(1, 7, -1, 1), T(ha).cuda(), T(hb).cuda(), d, add_to=acc)
    assert got.data_ptr() == acc.data_ptr() and torch.equal(idx2, idx)
    assert np.array_equal(got.cpu().numpy().reshape(exp.shape), base + exp)
    g = rng.standard_normal(exp.shape).astype(np.float32)
    back = oc.nn.octree_align_grad(T(g).cuda().view(1, 7, -1, 1), idx)
    assert np.array_equal(back.cpu().numpy().reshape(x.shape), interp.octree_align_grad(g, eidx))


def test_align_forward_forms_agree(oc):
  """ocnn_align_forward (zero fill + scatter, the reference's form, octree_nn.cu:710-730) and
  ocnn_align_forward_ws (inverted index, every row written once) through the C-ABI: equal bits on an
  index with holes on both sides, stale values in the output, and empty inputs."""
  import ctypes as C
  P = lambda t: C.c_void_p(t.data_ptr())
  st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
  g = torch.Generator().manual_seed(5)
  for btm_h, top_h in ((1000, 1500), (1500, 700), (64, 64), (0, 40), (40, 0)):
    keep = torch.rand(btm_h, generator=g) < 0.7
    target = torch.randperm(max(top_h, 1), generator=g)[:btm_h] if top_h else torch.zeros(0, dtype=torch.int64)
    idx = torch.full((btm_h,), -1, dtype=torch.int32)
    n = min(btm_h, target.numel())
    idx[:n] = torch.where(keep[:n], target[:n].to(torch.int32), torch.tensor(-1, dtype=torch.int32))
    x = torch.randn(5, btm_h, generator=g)
    # (an empty tensor has no address: every buffer holds one element more than it needs)
    x_d = torch.cat([x.reshape(-1), torch.zeros(1)]).cuda()
    idx_d = torch.cat([idx, torch.zeros(1, dtype=torch.int32)]).cuda()
    a = torch.full((5 * top_h + 1,), 7.0, device="cuda")
    b = torch.full((5 * top_h + 1,), 9.0, device="cuda")
    inv = torch.full((top_h + 1,), 123, dtype=torch.int32, device="cuda")
    oc.lib.call("ocnn_align_forward", P(a), top_h, 5, P(x_d), btm_h, P(idx_d), st)
    oc.lib.call("ocnn_align_forward_ws", P(b), top_h, 5, P(x_d), btm_h, P(idx_d), P(inv), st)
    assert torch.equal(a[:-1], b[:-1]), (btm_h, top_h)
    assert float(a[-1]) == 7.0 and float(b[-1]) == 9.0 and int(inv[-1]) == 123   # nothing written past the end
    exp = torch.zeros(5, top_h)
    ok = idx >= 0
    exp[:, idx[ok].long()] = x[:, ok]
    assert torch.equal(a[:-1].cpu().view(5, top_h), exp), (btm_h, top_h)


def test_trilinear_reference_case(oc, samples):
  octree = oc.nn.octree_batch([T(samples["octree_1"]), T(samples["octree_1"])])
  data = torch.ones(1, 3, 16, 1).cuda()
  out = oc.octree_trilinear(data, octree, 4, 5)
  assert out.shape == (1, 3, 16, 1) and torch.all(out == 1.0)


@pytest.mark.parametrize("nempty", [False, True])
@pytest.mark.parametrize("key2xyz", [False, True])
def test_interpolation_vs_oracle(oc, orc, synthetic, nempty, key2xyz):
  blobs = [orc.points2octree(make_points_blob(*synthetic.shape_cloud(4000, 21 + i)[:2]), 5, 2, key2xyz=key2xyz)
           for i in range(2)]
  host = orc.octree_batch(blobs)
  b = OctreeBlob(host)
  dev = T(host).cuda()
  rng = np.random.default_rng(2)
  for d in (3, 5):
    H = int(b.nnum_nempty[d] if nempty else b.nnum[d])
    data = rng.standard_normal((6, H)).astype(np.float32)
    # points near occupied voxels (some outside, some on faces) + uniformly random ones
    key = b.prop("key", d)[b.prop("child", d) >= 0]
    xyz = (key if key2xyz else orc.key2xyz(key.copy(), d)).view(np.int16).reshape(-1, 4).astype(np.float32)
    near = xyz[rng.integers(0, len(xyz), 1500)] + np.concatenate(
        [rng.uniform(-0.8, 1.8, (1500, 3)), np.zeros((1500, 1))], axis=1).astype(np.float32)
    rand = np.concatenate([rng.uniform(0, 2 ** d, (500, 3)), rng.integers(0, 2, (500, 1))], axis=1).astype(np.float32)
    pts = np.clip(np.concatenate([near, rand]), [0.51, 0.51, 0.51, 0], [2 ** d - 0.01] * 3 + [1]).astype(np.float32)
    dd = T(data).cuda().view(1, 6, H, 1)
    for method, fn in (("nearest", interp.octree_nearest_pts), ("linear", interp.octree_trilinear_pts)):
      exp = fn(orc, data, host, d, pts, nempty)
      out, idx, w = oc.nn.octree_interp_pts(dd, dev, d, T(pts).cuda(), method, nempty)
      got = out.cpu().numpy().reshape(exp.shape)
      assert np.abs(exp).max() > 0
      assert np.allclose(got, exp, atol=1e-5), (d, method, float(np.abs(got - exp).max()))
      # adjoint: <interp(x), g> == <x, interp^T(g)>
      g = rng.standard_normal(exp.shape).astype(np.float32)
      back = oc.nn.octree_interp_pts_grad(T(g).cuda().view(1, 6, -1, 1), idx, w, H, method)
      lhs = float(np.vdot(got.astype(np.float64), g))
      rhs = float(np.vdot(data.astype(np.float64), back.cpu().numpy().reshape(data.shape)))
      assert abs(lhs - rhs) < 1e-4 * max(1.0, abs(lhs))
      # element by element: the scatter written out with numpy from the returned corners
      ii, ww = idx.cpu().numpy().reshape(len(pts), -1), w.cpu().numpy().reshape(len(pts), -1).astype(np.float64)
      ww = np.where(ii >= 0, ww, 0.0)
      if method == "linear":
        ww = ww / (ww.sum(axis=1, keepdims=True) + 1e-10)
      dense = np.zeros((6, H))
      for m in range(ii.shape[1]):
        ok = ii[:, m] >= 0
        for c in range(6):
          np.add.at(dense[c], ii[ok, m], ww[ok, m] * g.reshape(6, -1)[c, ok])
      assert np.allclose(back.cpu().numpy().reshape(6, H), dense, atol=1e-4)
      # the entry point without a workspace scatters channel-major: same values
      plain = torch.empty(6, H, dtype=torch.float32, device="cuda")
      gg = T(g).cuda().contiguous()
      vp = lambda t: ctypes.c_void_p(t.data_ptr())
      oc.lib.call("ocnn_octree_interp_backward", vp(plain), vp(gg), 6, H, len(pts), int(method == "linear"),
                  vp(idx), vp(w), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
      assert np.allclose(plain.cpu().numpy(), dense, atol=1e-4)
  # the module form: points in [-1, 1], gradients through autograd
  H = int(b.nnum[5])
  x = torch.randn(1, 6, H, 1, device="cuda", requires_grad=True)
  p = T(np.concatenate([rng.uniform(-0.9, 0.9, (300, 3)), rng.integers(0, 2, (300, 1))], axis=1).astype(np.float32)).cuda()
  y = oc.OctreeInterp(5, "linear")(x, dev, p)
  y.sum().backward()
  assert y.shape == (1, 6, 300, 1) and x.grad.shape == x.shape


def test_points_property_reference_case(oc):
  """pytorch/test/test_points_property.py:11-63."""
  F = oc.nn
  points = torch.arange(15, dtype=torch.float32).reshape([-1, 3])
  index = torch.tensor([[0.0], [0.0], [0.0], [1.0], [1.0]])
  points4 = torch.cat([points, index], dim=1)
  normals = torch.arange(0, 1.5, 0.1, dtype=torch.float32).reshape([-1, 3])
  labels = torch.arange(5, dtype=torch.float32)
  feats = torch.arange(10, dtype=torch.float32).reshape([-1, 2])
  pts1 = F.points_new(points[:3], normals[:3], feats[:3], labels[:3])
  pts2 = F.points_new(points[3:], normals[3:], feats[3:], labels[3:])
  assert torch.equal(F.points_batch_property([pts1, pts2], 'label').view(-1), labels)
  assert torch.equal(F.points_batch_property([pts1, pts2], 'normal'), normals)
  assert torch.equal(F.points_batch_property([pts1, pts2], 'xyz'), points)
  assert torch.equal(F.points_batch_property([pts1, pts2], 'xyzi'), points4)
  assert torch.equal(F.points_batch_property([pts1, pts2], 'feature'), feats)
  assert torch.equal(F.points_property(pts1, 'xyz'), points[:3])
  assert torch.equal(F.points_property(pts1, 'normal'), normals[:3])
  assert torch.equal(F.points_property(pts1, 'feature'), feats[:3])
  assert torch.equal(F.points_property(pts1, 'label').view(-1), labels[:3])
  points_set = -torch.arange(9, dtype=torch.float32).reshape([-1, 3])
  pts3 = F.points_set_property(pts1, points_set, 'xyz')
  assert torch.equal(F.points_property(pts3, 'xyz'), points_set)
  feats_set = -torch.arange(6, dtype=torch.float32).reshape([-1, 2])
  pts4 = F.points_set_property(pts3, feats_set, 'feature')
  assert torch.equal(F.points_property(pts4, 'feature'), feats_set)
  assert torch.equal(F.points_property(pts4, 'xyz'), points_set)
  # the same on device-resident clouds
  d1 = pts1.cuda()
  assert torch.equal(F.points_property(d1, 'normal').cpu(), normals[:3])
