"""Seeded sweep over small random configurations: every case builds a random batch of clouds on
the GPU and runs a random operator configuration on it; everything is compared with the CPU
oracle (structure and integer results bit-exactly, fp32 within 1e-4 of the largest magnitude).
The cases reach corners the hand-picked tests do not: single-point clouds, depth == full_depth,
one or many channels, every kernel shape with either stride, empty levels."""
import numpy as np
import pytest
import torch

from oracle.checker import OctreeBlob, make_points_blob

pytestmark = pytest.mark.gpu

KS = [[3, 3, 3], [2, 2, 2], [3, 1, 1], [1, 3, 1], [1, 1, 3], [3, 3, 1], [3, 1, 3], [1, 3, 3], [1, 1, 1]]
TOL = 1e-4


def T(a):
  return torch.from_numpy(np.ascontiguousarray(a))


def relerr(got, exp):
  return float(np.abs(got.astype(np.float64) - exp).max() / (np.abs(exp).max() + 1e-30))


def random_cloud(rng, kind, n):
  if kind == 0:
    p = rng.uniform(-1, 1, (n, 3))
  elif kind == 1:
    p = rng.normal(0, 0.2, (n, 3))
  elif kind == 2:
    v = rng.normal(size=(n, 3))
    p = v / np.linalg.norm(v, axis=1, keepdims=True) * 0.9
  else:  # many points per leaf
    p = np.repeat(rng.uniform(-1, 1, (n // 50 + 1, 3)), 50, axis=0)[:n]
    p = p + rng.normal(0, 1e-3, p.shape)
  p = p.astype(np.float32).clip(-0.999, 0.999)
  nr = rng.normal(size=(len(p), 3)).astype(np.float32)
  nr /= np.linalg.norm(nr, axis=1, keepdims=True) + 1e-9
  return p, nr


@pytest.mark.parametrize("block", range(4))
def test_random_builds_and_operators(oc, orc, block):
  F = oc.nn
  for seed in range(block * 12, block * 12 + 12):
    rng = np.random.default_rng(1000 + seed)
    depth = int(rng.integers(2, 8))
    fd = int(rng.integers(1, min(depth, 3) + 1))
    B = int(rng.integers(1, 5))
    nfeat = int(rng.integers(0, 4))
    pbs = []
    for _ in range(B):
      p, nr = random_cloud(rng, seed % 4, int(rng.integers(1, 3000)))
      ft = rng.uniform(0, 1, (len(p), nfeat)).astype(np.float32)
      pbs.append(make_points_blob(p, nr, ft if nfeat else None))
    tag = "seed %d depth %d full %d batch %d" % (seed, depth, fd, B)
    ref = orc.octree_batch([orc.points2octree(pb, depth, fd) for pb in pbs])
    dev = F.points2octree_batch([T(pb).cuda() for pb in pbs], depth, fd)
    assert np.array_equal(dev.cpu().numpy(), ref), tag
    merged = F.octree_batch([F.points2octree(T(pb).cuda(), depth, fd) for pb in pbs])
    assert np.array_equal(merged.cpu().numpy(), ref), tag
    blob = OctreeBlob(ref)
    d = max(int(rng.integers(fd, depth + 1)), 1)
    H, Hne = int(blob.nnum[d]), int(blob.nnum_nempty[d])
    C, Co = int(rng.integers(1, 20)), int(rng.integers(1, 40))
    ks = KS[int(rng.integers(0, len(KS)))]
    stride = int(rng.integers(1, 3))
    nempty = bool(rng.integers(0, 2))
    if stride == 2 and d < 2:
      stride = 1
    Hin = Hne if nempty else H
    if Hin == 0:
      continue
    tag += " d %d %s stride %d nempty %d channels %d -> %d" % (d, ks, stride, nempty, C, Co)
    K = int(np.prod(ks))
    x = rng.standard_normal((C, Hin)).astype(np.float32)
    w = (rng.standard_normal((Co, C * K)) * 0.1).astype(np.float32)
    xd = T(x).cuda().view(1, C, Hin, 1)
    ye = orc.octree_conv(x, w, ref, d, Co, ks, stride, nempty)
    y = F.octree_conv(xd, T(w).cuda(), dev, d, Co, ks, stride, nempty)
    assert ye.size == 0 or relerr(y.cpu().numpy().reshape(ye.shape), ye) < TOL, tag
    g = rng.standard_normal(ye.shape).astype(np.float32)
    if ye.size:
      egd, egw = orc.octree_conv_grad(x, w, g, ref, d, Co, ks, stride, nempty)
      gd, gw = F.octree_conv_grad(xd, T(w).cuda(), dev, T(g).cuda().view(1, Co, -1, 1), d, Co, ks, stride, nempty)
      assert relerr(gw.cpu().numpy(), egw) < TOL and relerr(gd.cpu().numpy().reshape(egd.shape), egd) < TOL, tag
    if stride == 1 or d < depth:
      hin_d = Hin if stride == 1 else Hne
      if hin_d > 0:
        xq = x if stride == 1 else rng.standard_normal((C, hin_d)).astype(np.float32)
        wd = (rng.standard_normal((C, Co * K)) * 0.1).astype(np.float32)
        ye = orc.octree_deconv(xq, wd, ref, d, Co, ks, stride, nempty)
        y = F.octree_deconv(T(xq).cuda().view(1, C, hin_d, 1), T(wd).cuda(), dev, d, Co, ks, stride, nempty)
        assert ye.size == 0 or relerr(y.cpu().numpy().reshape(ye.shape), ye) < TOL, tag
    neigh, child = blob.prop("neigh", d).reshape(-1), blob.prop("child", d)
    col = F.octree2col(xd, dev, d, ks, stride, nempty)
    if nempty:
      ichild = np.zeros(max(Hne, 1), np.int32)
      ichild[child[child >= 0]] = np.nonzero(child >= 0)[0]
      hp = Hne if stride == 1 else int(blob.nnum_nempty[d - 1])
      ce = orc.octree2colP(x, ks, stride, neigh, child, ichild, hp)
      be = orc.col2octreeP(ce, ks, stride, neigh, child, ichild, hp, Hne)
    else:
      h = H if stride == 1 else H // 8
      ce = orc.octree2col(x, ks, stride, neigh, h)
      be = orc.col2octree(ce, ks, stride, neigh, h)
    assert np.array_equal(col.cpu().numpy(), ce), tag
    back = F.col2octree(col, dev, d, ks, stride, nempty)
    assert be.size == 0 or relerr(back.cpu().numpy().reshape(be.shape), be) < TOL, tag
    if not nempty and d >= 2:
      top, mask = F.octree_max_pool(xd, dev, d)
      et, em = orc.max_pool(x)
      assert np.array_equal(top.cpu().numpy().reshape(et.shape), et), tag
      assert np.array_equal(mask.cpu().numpy().reshape(em.shape), em), tag
      pd = F.octree_pad(top, dev, d - 1, 0.25)
      assert np.array_equal(pd.cpu().numpy().reshape(C, -1), orc.pad(et, blob.prop("child", d - 1), 0.25)), tag
      assert np.array_equal(F.octree_depad(pd, dev, d - 1).cpu().numpy().reshape(et.shape), et), tag
      assert np.array_equal(F.octree_max_unpool(top, mask, dev, d).cpu().numpy().reshape(C, H), orc.max_unpool(et, em)), tag


@pytest.mark.parametrize("block", range(2))
def test_random_growth_and_adaptive_builds(oc, orc, block):
  F = oc.nn
  for seed in range(block * 12, block * 12 + 12):
    rng = np.random.default_rng(5000 + seed)
    depth, fd, B = int(rng.integers(3, 7)), int(rng.integers(1, 3)), int(rng.integers(1, 4))
    o_ref, o_dev = orc.octree_new(B, 3, False, 0), F.octree_new(B, 3, False, 0)
    for d in range(1, fd + 1):
      o_ref, o_dev = orc.octree_grow(o_ref, d, True), F.octree_grow(o_dev, d, True)
    for d in range(fd, depth + 1):
      n = int(OctreeBlob(o_ref).nnum[d])
      lab = (rng.uniform(size=n) < rng.uniform(0.0, 0.6)).astype(np.int32)
      if seed % 7 == 0 and d == fd + 1:
        lab[:] = 0   # nothing splits: one node is kept (octree_grow.cpp:180-185)
      o_ref, o_dev = orc.octree_update(o_ref, lab, d, 1), F.octree_update(o_dev, T(lab).cuda(), d, 1)
      assert np.array_equal(o_dev.cpu().numpy(), o_ref), ("update", seed, d)
      if d < depth:
        o_ref, o_dev = orc.octree_grow(o_ref, d + 1, False), F.octree_grow(o_dev, d + 1, False)
        assert np.array_equal(o_dev.cpu().numpy(), o_ref), ("grow", seed, d)
    n = int(rng.integers(50, 4000))
    v = rng.normal(size=(n, 3))
    v /= np.linalg.norm(v, axis=1, keepdims=True)
    p = (v * rng.uniform(0.3, 0.95)).astype(np.float32)
    if seed % 3 == 1:
      p[:, 2] *= 0.05
    pb = make_points_blob(p, v.astype(np.float32))
    dd = int(rng.integers(3, 7))
    opts = dict(node_dis=bool(rng.integers(0, 2)), node_feature=bool(rng.integers(0, 2)),
                split_label=bool(rng.integers(0, 2)), adaptive=bool(rng.integers(0, 2)),
                adp_depth=min(int(rng.integers(1, 4)), dd), th_normal=float(rng.uniform(0.05, 0.3)),
                th_distance=float(rng.uniform(0.5, 3.0)), extrapolate=bool(rng.integers(0, 2)),
                save_pts=bool(rng.integers(0, 2)), key2xyz=bool(rng.integers(0, 2)))
    try:
      exp = orc.points2octree(pb, dd, 2, **opts)
    except RuntimeError:
      continue   # a combination the reference's builder rejects
    got = F.points2octree(T(pb), dd, 2, **opts)
    assert np.array_equal(got.cpu().numpy(), exp), ("build", seed, dd, opts)


CH = [3, 8, 16, 24, 32, 48, 64, 96, 128, 160, 256]
SHAPES = [([3, 3, 3], 1), ([3, 3, 3], 1), ([2, 2, 2], 2), ([2, 2, 2], 2), ([1, 1, 1], 1), ([3, 1, 1], 1), ([3, 3, 1], 1)]


def bf16_round(a):
  return T(a).bfloat16().float().numpy()


@pytest.mark.parametrize("block", range(4))
def test_random_wide_channel_operators(oc, orc, synthetic, block):
  """Seeded cases at the channel widths the networks use (3 .. 256, also 48, 96, 160) on levels of
  hundreds to tens of thousands of nodes: convolution and deconvolution of a random shape, stride
  and node set in fp32 (1e-4) and bf16 (2e-2, operands rounded to bf16 first) with both fp32
  gradients, and for the shapes the row-major entry points serve (3x3x3 stride 1, 2x2x2 stride
  2) the same operator on row-major tensors with bias and ReLU, with and without kept weights."""
  F = oc.nn

  def close(got, exp, tol, what):
    if exp.size:
      err = float(np.abs(got.reshape(exp.shape) - exp).max()) / (float(np.abs(exp).max()) + 1e-30)
      assert err < tol, (what, err)

  for seed in range(block * 6, block * 6 + 6):
    rng = np.random.default_rng(7000 + seed)
    depth = int(rng.integers(5, 8))
    B = int(rng.integers(1, 4))
    npts = int(rng.integers(2000, 30000))
    pbs = []
    for b in range(B):
      p, n, _ = (synthetic.shape_cloud if rng.integers(0, 2) else synthetic.room_cloud)(npts, seed * 10 + b)
      pbs.append(make_points_blob(p, n))
    host = orc.octree_batch([orc.points2octree(pb, depth, 2) for pb in pbs])
    dev = F.points2octree_batch([T(pb).cuda() for pb in pbs], depth, 2)
    assert np.array_equal(dev.cpu().numpy(), host), seed
    blob = OctreeBlob(host)
    for rep in range(3):
      d = int(rng.integers(3, depth + 1))
      ks, stride = SHAPES[int(rng.integers(0, len(SHAPES)))]
      nempty = bool(rng.integers(0, 2))
      C, Co = CH[int(rng.integers(0, len(CH)))], CH[int(rng.integers(0, len(CH)))]
      H, Hne = int(blob.nnum[d]), int(blob.nnum_nempty[d])
      Hin = Hne if nempty else H
      K = int(np.prod(ks))
      if Hin == 0 or Hin * K * C * Co > 1e9:
        continue
      tag = "seed %d rep %d depth %d/%d H %d Hne %d %s stride %d nempty %d %d -> %d" % (seed, rep, d, depth, H, Hne, ks, stride, nempty, C, Co)
      x = bf16_round(rng.standard_normal((C, Hin)).astype(np.float32))
      w = bf16_round((rng.standard_normal((Co, C * K)) / np.sqrt(C * K)).astype(np.float32))
      ye = orc.octree_conv(x, w, host, d, Co, ks, stride, nempty)
      xd, wdv = T(x).cuda().view(1, C, Hin, 1), T(w).cuda()
      close(F.octree_conv(xd, wdv, dev, d, Co, ks, stride, nempty).cpu().numpy(), ye, TOL, tag + " conv fp32")
      close(F.octree_conv(xd.bfloat16(), wdv.bfloat16(), dev, d, Co, ks, stride, nempty).float().cpu().numpy(), ye, 2e-2, tag + " conv bf16")
      if ye.size:
        g = rng.standard_normal(ye.shape).astype(np.float32)
        egd, egw = orc.octree_conv_grad(x, w, g, host, d, Co, ks, stride, nempty)
        gd, gw = F.octree_conv_grad(xd, wdv, dev, T(g).cuda().view(1, Co, -1, 1), d, Co, ks, stride, nempty)
        close(gw.cpu().numpy(), egw, TOL, tag + " weight gradient")
        close(gd.cpu().numpy(), egd, TOL, tag + " data gradient")
      rows_kind = (ks == [3, 3, 3] and stride == 1) or (ks == [2, 2, 2] and stride == 2)
      if rows_kind and ye.size:
        bias = (rng.standard_normal(Co) * 0.2).astype(np.float32)
        exp = ye if (stride == 1 or nempty) else orc.pad(ye, blob.prop("child", d - 1))
        exp = np.maximum(exp + bias[:, None], 0)
        for const in (False, True):
          r = F.octree_conv_rows(F.to_rows(xd.bfloat16()), C, wdv.bfloat16(), dev, d, Co, bias=T(bias).cuda(), relu=True,
                                 kernel_size=tuple(ks), stride=stride, nempty=nempty, constant_weights=const)
          assert not r[-1].any() and not r[:, Co:].any(), tag
          close(F.from_rows(r, Co).float().cpu().numpy(), exp, 2e-2, tag + " conv on rows, kept weights %d" % const)
      if stride == 1 or d < depth:
        hin_d = Hin if stride == 1 else Hne
        if hin_d == 0:
          continue
        xq = x if stride == 1 else bf16_round(rng.standard_normal((C, hin_d)).astype(np.float32))
        wd = bf16_round((rng.standard_normal((C, Co * K)) / np.sqrt(C)).astype(np.float32))
        ye = orc.octree_deconv(xq, wd, host, d, Co, ks, stride, nempty)
        xqd = T(xq).cuda().view(1, C, hin_d, 1)
        close(F.octree_deconv(xqd, T(wd).cuda(), dev, d, Co, ks, stride, nempty).cpu().numpy(), ye, TOL, tag + " deconv fp32")
        close(F.octree_deconv(xqd.bfloat16(), T(wd).cuda().bfloat16(), dev, d, Co, ks, stride, nempty).float().cpu().numpy(), ye,
              2e-2, tag + " deconv bf16")
        if ye.size:
          g = rng.standard_normal(ye.shape).astype(np.float32)
          egd, egw = orc.octree_deconv_grad(xq, wd, g, host, d, Co, ks, stride, nempty)
          gd, gw = F.octree_deconv_grad(xqd, T(wd).cuda(), dev, T(g).cuda().view(1, Co, -1, 1), d, Co, ks, stride, nempty)
          close(gw.cpu().numpy(), egw, TOL, tag + " deconv weight gradient")
          close(gd.cpu().numpy(), egd, TOL, tag + " deconv data gradient")
        if rows_kind and ye.size:
          for const in (False, True):
            if stride == 1 or nempty:
              rin = F.to_rows(xqd.bfloat16())
            else:   # rows of ALL nodes of the depth in; what the empty ones hold must not be read
              full = np.full((C, H), 3.0, np.float32)
              child = blob.prop("child", d)
              full[:, child >= 0] = xq[:, child[child >= 0]]
              rin = F.to_rows(T(full).cuda().view(1, C, H, 1).bfloat16())
            r = F.octree_conv_rows(rin, C, T(wd).cuda().bfloat16(), dev, d, Co, deconv=True, kernel_size=tuple(ks),
                                   stride=stride, nempty=nempty, constant_weights=const)
            assert not r[-1].any() and not r[:, Co:].any(), tag
            close(F.from_rows(r, Co).float().cpu().numpy(), ye, 2e-2, tag + " deconv on rows, kept weights %d" % const)
