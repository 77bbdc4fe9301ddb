"""octree_gather / gatherbk / mask and the trilinear stencils (bilinear_neigh / bilinear_xyz,
octree/octree/octree_nn.h:170-177, 204-218) on the GPU against the oracle: indices and keys
bit-exact, the scatter-add within 1e-5."""
import numpy as np
import pytest
import torch

from oracle.checker import OctreeBlob, make_points_blob

pytestmark = pytest.mark.gpu


def T(a):
  return torch.from_numpy(np.ascontiguousarray(a))


@pytest.fixture(scope="module")
def tree(oc, orc, samples, synthetic):
  pbs = [make_points_blob(*synthetic.shape_cloud(4000, 51 + i)[:2]) for i in range(2)]
  host = orc.octree_batch([orc.points2octree(p, 6, 2, key2xyz=True) for p in pbs])
  shost = orc.octree_batch([samples["octree_1"]])
  return [(h, T(h).cuda(), OctreeBlob(h)) for h in (host, shost)]


def test_bilinear_stencils(oc, orc, tree):
  for host, dev, b in tree:
    for d in range(1, b.depth):
      if b.nnum[d + 1] == 0:
        continue
      exp = orc.bilinear_neigh(b.prop("neigh", d).reshape(-1), b.prop("child", d), int(b.nnum[d + 1]))
      got = oc.nn.octree_bilinear_neigh(dev, d)
      assert np.array_equal(got.cpu().numpy(), exp), d
      keys = b.prop("key", d + 1)
      for d0 in (d, max(d - 1, 0)):
        xe, fe = orc.bilinear_xyz(keys, d0, d + 1)
        xg, fg = oc.nn.octree_bilinear_xyz(T(keys.view(np.int64)).cuda(), d + 1, d0)
        assert np.array_equal(xg.cpu().numpy().view(np.uint64), xe)
        assert np.array_equal(fg.cpu().numpy(), fe)     # same float steps: bit-identical


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gather_vs_oracle(oc, orc, dtype):
  rng = np.random.default_rng(2)
  for C_, H, Ht in ((5, 1000, 3000), (64, 4096, 1024), (3, 17, 5)):
    btm = rng.standard_normal((C_, H)).astype(np.float32)
    idx = rng.integers(-1, H, Ht).astype(np.int32)
    x = T(btm).cuda().view(1, C_, H, 1).to(dtype)
    got = oc.nn.octree_gather(x, T(idx).cuda())
    exp = orc.octree_gather(x.float().cpu().numpy().reshape(C_, H), idx)
    assert np.array_equal(got.float().cpu().numpy().reshape(C_, Ht), exp)


def test_gatherbk_and_mask_vs_oracle(oc, orc):
  rng = np.random.default_rng(3)
  L = oc.lib.get()
  import ctypes as C
  for C_, H, Ht in ((5, 1000, 3000), (64, 2048, 20000), (3, 17, 5), (8, 5000, 100)):
    idx = rng.integers(-1, H, Ht).astype(np.int32)
    y = rng.standard_normal((C_, Ht)).astype(np.float32)
    exp = orc.octree_gatherbk(y, idx, H)
    got = oc.nn.octree_gatherbk(T(y).cuda().view(1, C_, Ht, 1), T(idx).cuda(), H)
    assert np.abs(got.cpu().numpy().reshape(C_, H) - exp).max() <= 1e-5 * max(1.0, np.abs(exp).max())
    # the form without a workspace (atomic scatter, as the reference does it): same values
    yd, out = T(y).cuda(), torch.empty((C_, H), device="cuda")
    code = L.ocnn_octree_gatherbk(C.c_void_p(yd.data_ptr()), Ht, C_, C.c_void_p(out.data_ptr()), H,
                                  C.c_void_p(T(idx).cuda().data_ptr()), None, C.c_size_t(0), None)
    assert code == 0
    torch.cuda.synchronize()
    assert np.abs(out.cpu().numpy() - exp).max() <= 1e-5 * max(1.0, np.abs(exp).max())
    # adjoint of gather
    x = rng.standard_normal((C_, H)).astype(np.float32)
    gx = oc.nn.octree_gather(T(x).cuda().view(1, C_, H, 1), T(idx).cuda()).cpu().numpy().reshape(C_, Ht)
    assert abs(float((gx.astype(np.float64) * y).sum()) - float((x.astype(np.float64) * exp).sum())) < 1e-2
    label = rng.integers(0, 3, H).astype(np.int32)
    m = oc.nn.octree_mask(T(x).cuda().view(1, C_, H, 1), T(label).cuda(), 2)
    assert np.array_equal(m.cpu().numpy().reshape(C_, H), orc.octree_mask(x, label, 2))
