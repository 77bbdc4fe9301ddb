"""BASELINE config 5 at test size: a batch of ADAPTIVE octrees (built by the CPU oracle, whose
adaptive build is pinned against the compiled reference) is merged on the GPU, and the
shape-completion decoder loop (2x2x2 stride-2 deconv up, 3x3x3 conv, split labels from the
ground truth, octree_update, octree_grow) rebuilds the ground-truth structure level by level.
Structure is compared bit-exactly, features within 1e-4 (fp32)."""
import numpy as np
import pytest
import torch

from oracle.checker import OctreeBlob, make_points_blob

pytestmark = pytest.mark.gpu

ADAPTIVE = dict(node_dis=True, split_label=True, adaptive=True, adp_depth=3, th_normal=0.1, th_distance=2.0)


def T(a):
  return torch.from_numpy(np.ascontiguousarray(a))


def relerr(got, exp):
  return float(np.abs(got.astype(np.float64) - exp).max() / (np.abs(exp).max() + 1e-30))


@pytest.fixture(scope="module")
def adaptive_clouds(synthetic):
  return [make_points_blob(*synthetic.shape_cloud(4000, 300 + i)[:2]) for i in range(3)]


@pytest.fixture(scope="module")
def adaptive_batch(orc, adaptive_clouds):
  singles = [orc.points2octree(pb, 5, 2, **ADAPTIVE) for pb in adaptive_clouds]
  return singles, orc.octree_batch(singles)


def test_adaptive_octrees_built_on_gpu(oc, adaptive_clouds, adaptive_batch):
  """The decoder's input is built on the device too: adaptive points2octree per cloud, then
  octree_batch, byte for byte the oracle's batch."""
  singles, host = adaptive_batch
  built = [oc.nn.points2octree(T(pb), 5, 2, **ADAPTIVE) for pb in adaptive_clouds]
  for got, exp in zip(built, singles):
    assert np.array_equal(got.cpu().numpy(), exp)
  assert np.array_equal(oc.nn.points2octree_batch([T(pb) for pb in adaptive_clouds], 5, 2, **ADAPTIVE).cpu().numpy(), host)


def test_adaptive_octrees_merge_on_gpu(oc, orc, adaptive_batch):
  """octree_batch over octrees whose features / labels live at every depth (location -1) and
  that carry split labels (merge_octrees.cpp:144-177)."""
  singles, host = adaptive_batch
  b = OctreeBlob(host)
  assert b.is_adaptive and b.location("feature") == -1 and b.has("split") and b.channel("feature") == 4
  assert any((b.prop("split", d) == 2).any() for d in range(3, 6)), "nothing was trimmed"
  got = oc.nn.octree_batch([T(s) for s in singles]).cpu().numpy()
  assert np.array_equal(got, host)
  # the merged adaptive octree is a valid operand of the operators: neighbour-table conv at depth 4
  rng = np.random.default_rng(0)
  x = rng.standard_normal((4, int(b.nnum[4]))).astype(np.float32)
  w = (rng.standard_normal((8, 4 * 27)) * 0.1).astype(np.float32)
  exp = orc.octree_conv(x, w, host, 4, 8, [3, 3, 3], 1)
  out = oc.nn.octree_conv(T(x).cuda().view(1, 4, -1, 1), T(w).cuda(), T(host).cuda(), 4, 8, [3, 3, 3], 1, False)
  assert relerr(out.cpu().numpy().reshape(exp.shape), exp) < 1e-4


def oracle_decoder(orc, code, params, labels, depth, full_depth, batch, skips=None, blob_in=None):
  """pytorch/ocnn/ounet.py:72-131 through the oracle: deconv up, aligned skip added, conv, the
  prediction head (two 1x1x1 convolutions) and its argmax, update, grow."""
  from oracle import interp
  o = orc.octree_new(batch, 4, True, 0)
  for d in range(1, full_depth + 1):
    o = orc.octree_grow(o, d, True)
  feats = {full_depth: code}
  for d in range(full_depth, depth + 1):
    if d > full_depth:
      child = OctreeBlob(o).prop("child", d - 1)
      w, bias = params[("up", d)]
      x = orc.octree_deconv(feats[d - 1][:, child >= 0], w, o, d - 1, w.shape[1] // 8, [2, 2, 2], 2)
      x = np.maximum(x + bias[:, None], 0)
      if skips is not None:
        skip, _ = interp.octree_align(orc, skips[d], blob_in, o, d)
        x = x + skip
      w, bias = params[("conv", d)]
      feats[d] = np.maximum(orc.octree_conv(x, w, o, d, w.shape[0], [3, 3, 3], 1) + bias[:, None], 0)
    if ("predict", d) in params:
      (w1, b1), (w2, b2) = params[("predict", d)]
      hidden = np.maximum(orc.octree_conv(feats[d], w1, o, d, w1.shape[0], [1, 1, 1], 1) + b1[:, None], 0)
      feats[("logit", d)] = orc.octree_conv(hidden, w2, o, d, w2.shape[0], [1, 1, 1], 1) + b2[:, None]
    o = orc.octree_update(o, labels[d], d, 1)
    if d < depth:
      o = orc.octree_grow(o, d + 1, False)
  return o, feats


def test_completion_decoder_rebuilds_ground_truth(oc, orc, adaptive_batch):
  singles, host = adaptive_batch
  gt = OctreeBlob(host)
  depth, fd, batch = 5, 2, 3
  labels = {d: (gt.prop("split", d) == 1).astype(np.int32) for d in range(fd, depth + 1)}
  rng = np.random.default_rng(5)
  chans = {2: 32, 3: 24, 4: 16, 5: 8}
  params = {}
  for d in range(fd + 1, depth + 1):
    params[("up", d)] = ((rng.standard_normal((chans[d - 1], chans[d] * 8)) * 0.2).astype(np.float32),
                         (rng.standard_normal(chans[d]) * 0.1).astype(np.float32))
    params[("conv", d)] = ((rng.standard_normal((chans[d], chans[d] * 27)) * 0.1).astype(np.float32),
                           (rng.standard_normal(chans[d]) * 0.1).astype(np.float32))
  code = rng.standard_normal((chans[fd], batch * 8 ** fd)).astype(np.float32)

  exp_o, exp_f = oracle_decoder(orc, code, params, labels, depth, fd, batch)
  dev_params = {k: (T(w).cuda(), T(b).cuda()) for k, (w, b) in params.items()}
  got_o, got_f = oc.stacks.completion_decoder(
      T(code).cuda().view(1, chans[fd], -1, 1), dev_params, {d: T(l).cuda() for d, l in labels.items()},
      depth, fd, batch_size=batch, channel_out=4)
  assert np.array_equal(got_o.cpu().numpy(), exp_o)            # keys, children, neighbours, header
  for d in range(fd + 1, depth + 1):
    assert relerr(got_f[d].cpu().numpy().reshape(exp_f[d].shape), exp_f[d]) < 1e-4, d

  # the grown structure IS the ground truth's: same node counts, same voxels, same child links
  g = OctreeBlob(got_o.cpu().numpy())
  F = oc.nn
  gt_dev = T(host).cuda()
  for d in range(fd, depth + 1):
    assert g.nnum[d] == gt.nnum[d] and g.nnum_nempty[d] == gt.nnum_nempty[d]
    assert torch.equal(F.octree_property(got_o, "xyz", d), F.octree_property(gt_dev, "xyz", d))
    assert np.array_equal(g.prop("child", d), gt.prop("child", d))


def test_completion_decoder_with_skips_and_split_prediction(oc, orc, synthetic, adaptive_batch):
  """The loop as pytorch/ocnn/ounet.py:72-131 runs it: the encoder's features of every depth live
  on ANOTHER octree (the network's input), are moved onto the growing octree by octree_align and
  added behind the deconvolution; a 1x1x1 head predicts the split label of every node.  The
  ground-truth labels decide the structure (ounet.py:89-90), so the logits are compared with the
  oracle chain on that structure (fp32), and the argmax wherever the oracle's two logits are not
  within rounding of each other.  Then `decode_shape` (ounet.py:118-119): the predicted labels
  themselves drive update / grow, and the result must be the octree the oracle grows from them."""
  singles, host = adaptive_batch
  gt = OctreeBlob(host)
  depth, fd, batch = 5, 2, 3
  # the input octree: the same three shapes built plainly (another structure than the adaptive one)
  pbs = [make_points_blob(*synthetic.shape_cloud(2500, 300 + i)[:2]) for i in range(3)]
  host_in = orc.octree_batch([orc.points2octree(pb, depth, fd) for pb in pbs])
  bin_ = OctreeBlob(host_in)
  labels = {d: (gt.prop("split", d) == 1).astype(np.int32) for d in range(fd, depth + 1)}
  rng = np.random.default_rng(15)
  chans = {2: 32, 3: 24, 4: 16, 5: 8}
  params = {}
  for d in range(fd, depth + 1):
    if d > fd:
      params[("up", d)] = ((rng.standard_normal((chans[d - 1], chans[d] * 8)) * 0.2).astype(np.float32),
                           (rng.standard_normal(chans[d]) * 0.1).astype(np.float32))
      params[("conv", d)] = ((rng.standard_normal((chans[d], chans[d] * 27)) * 0.1).astype(np.float32),
                             (rng.standard_normal(chans[d]) * 0.1).astype(np.float32))
    params[("predict", d)] = (((rng.standard_normal((32, chans[d])) * 0.3).astype(np.float32),
                               (rng.standard_normal(32) * 0.1).astype(np.float32)),
                              ((rng.standard_normal((2, 32)) * 0.3).astype(np.float32),
                               (rng.standard_normal(2) * 0.1).astype(np.float32)))
  code = rng.standard_normal((chans[fd], batch * 8 ** fd)).astype(np.float32)
  skips = {d: rng.standard_normal((chans[d], int(bin_.nnum[d]))).astype(np.float32) for d in range(fd + 1, depth + 1)}

  def dev(v):
    return tuple(dev(x) for x in v) if isinstance(v, tuple) else T(v).cuda()

  dev_params = {k: dev(v) for k, v in params.items()}
  dev_skips = {d: T(v).cuda().view(1, v.shape[0], -1, 1) for d, v in skips.items()}
  code_dev = T(code).cuda().view(1, chans[fd], -1, 1)

  exp_o, exp_f = oracle_decoder(orc, code, params, labels, depth, fd, batch, skips, host_in)
  got_o, got_f = oc.stacks.completion_decoder(code_dev, dev_params, {d: T(l).cuda() for d, l in labels.items()},
                                              depth, fd, batch_size=batch, skips=dev_skips, octree_in=T(host_in).cuda())
  assert np.array_equal(got_o.cpu().numpy(), exp_o)
  used = 0
  for d in range(fd, depth + 1):
    if d > fd:
      assert relerr(got_f[d].cpu().numpy().reshape(exp_f[d].shape), exp_f[d]) < 1e-4, d
    logit = exp_f[("logit", d)]
    assert relerr(got_f[("logit", d)].cpu().numpy().reshape(logit.shape), logit) < 1e-4, d
    clear = np.abs(logit[0] - logit[1]) > 1e-3 * np.abs(logit).max()
    used += int(clear.sum())
    assert np.array_equal(got_f[("label", d)].cpu().numpy()[clear], logit.argmax(0).astype(np.int32)[clear]), d
  assert used > 100

  # decode_shape: the predictions grow the octree; the oracle grows one from the same labels
  free_o, free_f = oc.stacks.completion_decoder(code_dev, dev_params, None, depth, fd, batch_size=batch,
                                                skips=dev_skips, octree_in=T(host_in).cuda())
  pred = {d: free_f[("label", d)].cpu().numpy() for d in range(fd, depth + 1)}
  assert sum(int(p.sum()) for p in pred.values()) > 0
  exp_free, _ = oracle_decoder(orc, code, params, pred, depth, fd, batch, skips, host_in)
  assert np.array_equal(free_o.cpu().numpy(), exp_free)


def test_completion_decoder_full_size_regrows_config5(oc, synthetic, hashes):
  """BASELINE config 5 at FULL size: 16 adaptive octrees at depth 7 built on the device (the
  blob's SHA-256 is the compiled reference's), then the decoder loop with the benchmark's widths
  (256 -> 32), the aligned skips and the split heads, driven by the ground truth's split labels.
  The regrown octree must have the ground truth's structure bit for bit at every depth: node
  counts, coordinates, child links and neighbour tables."""
  from conftest import sha
  F = oc.nn
  kw = dict(node_dis=True, split_label=True, adaptive=True, adp_depth=4, th_normal=0.1, th_distance=2.0)
  clouds = [T(make_points_blob(*synthetic.shape_cloud(50000, 300 + i)[:2])).cuda() for i in range(16)]
  gt = F.points2octree_batch(clouds, 7, 2, **kw)
  assert sha(gt.cpu().numpy()) == hashes["cfg5"]["batch"]
  plain = F.points2octree_batch(clouds, 7, 2)              # the network's input octree (skips live here)
  ginfo, pinfo = F.octree_info(gt), F.octree_info(plain)
  depth, fd, batch = 7, 2, 16
  g = torch.Generator(device="cuda").manual_seed(9)
  ch = {2: 256, 3: 128, 4: 64, 5: 32, 6: 32, 7: 32}
  rnd = lambda *shape, s=0.05: torch.randn(*shape, device="cuda", generator=g) * s
  params = {}
  for d in range(fd, depth + 1):
    if d > fd:
      params[("up", d)] = (rnd(ch[d - 1], ch[d] * 8), rnd(ch[d]))
      params[("conv", d)] = (rnd(ch[d], ch[d] * 27), rnd(ch[d]))
    params[("predict", d)] = ((rnd(32, ch[d]), rnd(32)), (rnd(2, 32), rnd(2)))
  labels = {d: (F.octree_property(gt, "split", d) == 1).to(torch.int32) for d in range(fd, depth + 1)}
  skips = {d: rnd(1, ch[d], pinfo.nnum(d), 1, s=1.0) for d in range(fd + 1, depth + 1)}
  code = rnd(1, ch[fd], batch * 8 ** fd, 1, s=1.0)
  out, feats = oc.stacks.completion_decoder(code, params, labels, depth, fd, batch_size=batch, skips=skips,
                                            octree_in=plain)
  oinfo = F.octree_info(out)
  for d in range(fd, depth + 1):
    assert oinfo.nnum(d) == ginfo.nnum(d) and oinfo.nnum_nempty(d) == ginfo.nnum_nempty(d), d
    for name in ("xyz", "child", "neigh"):
      assert torch.equal(F.octree_property(out, name, d), F.octree_property(gt, name, d)), (name, d)
    assert feats[("label", d)].shape[0] == ginfo.nnum(d)
    assert torch.isfinite(feats[("logit", d)]).all()
