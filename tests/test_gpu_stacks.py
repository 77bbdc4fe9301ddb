"""GPU parity of the operator sequences of the benchmark configurations (conv -> BatchNorm ->
ReLU folded into one kernel, pooling, stride-2 down / up sampling) against the same sequence
run through the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle.checker import OctreeBlob, make_points_blob

pytestmark = pytest.mark.gpu


def T(a):
  return torch.from_numpy(np.ascontiguousarray(a))


def relerr(got, exp):
  return float(np.abs(got.astype(np.float64) - exp).max() / (np.abs(exp).max() + 1e-30))


@pytest.fixture(scope="module")
def tree(oc, orc, synthetic):
  pbs = [make_points_blob(*synthetic.shape_cloud(3000, 61 + i)[:2]) for i in range(2)]
  host = orc.octree_batch([orc.points2octree(p, 6, 2) for p in pbs])
  return host, T(host).cuda(), OctreeBlob(host)


def test_fold_bn_matches_batchnorm(oc):
  """BatchNorm2d(eps = 1e-3) in eval mode after a linear map == the folded weights and bias."""
  g = torch.Generator().manual_seed(0)
  cout, cin, K, H = 6, 4, 27, 50
  w = torch.randn(cout, cin * K, generator=g)
  col = torch.randn(cin * K, H, generator=g)
  bn = torch.nn.BatchNorm2d(cout, eps=1e-3)
  with torch.no_grad():
    bn.weight.copy_(torch.rand(cout, generator=g) + 0.5)
    bn.bias.copy_(torch.randn(cout, generator=g))
    bn.running_mean.copy_(torch.randn(cout, generator=g))
    bn.running_var.copy_(torch.rand(cout, generator=g) + 0.2)
  bn.eval()
  exp = bn((w @ col).view(1, cout, H, 1)).view(cout, H)
  wf, bf = oc.stacks.fold_bn(w, bn.weight.data, bn.bias.data, bn.running_mean, bn.running_var)
  assert torch.allclose(wf @ col + bf[:, None], exp, atol=1e-5)
  # deconv layout [Cin, Cout*K]
  wd = torch.randn(cin, cout * 8, generator=g)
  x = torch.randn(cin, H, generator=g)
  full = (wd.t() @ x).view(cout, 8, H)
  exp = bn(full.reshape(1, cout, 8 * H, 1)).view(cout, 8, H)
  wf, bf = oc.stacks.fold_bn(wd, bn.weight.data, bn.bias.data, bn.running_mean, bn.running_var,
                             deconv=True, kdim=8)
  assert torch.allclose((wf.t() @ x).view(cout, 8, H) + bf[:, None, None], exp, atol=1e-5)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 2e-2)])
def test_fused_bias_relu(oc, orc, tree, dtype, tol):
  host, dev, b = tree
  rng = np.random.default_rng(1)
  for (ks, stride, deconv, nempty, d) in (([3, 3, 3], 1, False, False, 5), ([2, 2, 2], 2, False, False, 5),
                                          ([2, 2, 2], 2, True, False, 4), ([3, 3, 3], 1, False, True, 5),
                                          ([3, 3, 3], 1, True, False, 5), ([3, 1, 1], 1, False, False, 5)):
    K = ks[0] * ks[1] * ks[2]
    ci, co = 16, 40
    hin = int(b.nnum_nempty[d] if (nempty or (stride == 2 and deconv)) else b.nnum[d])
    x = rng.standard_normal((ci, hin)).astype(np.float32)
    w = (rng.standard_normal((ci, co * K) if deconv else (co, ci * K)) * 0.1).astype(np.float32)
    bias = rng.standard_normal(co).astype(np.float32)
    fn = orc.octree_deconv if deconv else orc.octree_conv
    exp = np.maximum(fn(x, w, host, d, co, ks, stride, nempty) + bias[:, None], 0)
    got = oc.nn.octree_conv_fused(T(x).cuda().view(1, ci, hin, 1).to(dtype), T(w).cuda().to(dtype),
                                  T(bias).cuda(), True, dev, d, co, ks, stride, nempty, deconv=deconv)
    assert relerr(got.float().cpu().numpy().reshape(exp.shape), exp) < tol, (ks, stride, deconv, nempty)


def test_lenet_trunk(oc, orc, tree):
  """conv -> (folded BN) -> ReLU -> max_pool -> pad from depth 6 down to depth 2, channels
  3 -> 32 -> 64 -> 128 -> 256 (BASELINE config 2)."""
  host, dev, b = tree
  rng = np.random.default_rng(2)
  chans = {6: (3, 32), 5: (32, 64), 4: (64, 128), 3: (128, 256)}
  params, data = {}, b.prop("feature", 6).copy()
  x = data
  for d in range(6, 2, -1):
    ci, co = chans[d]
    w = (rng.standard_normal((co, ci * 27)) * (1.0 / np.sqrt(ci * 27))).astype(np.float32)
    bias = (rng.standard_normal(co) * 0.1).astype(np.float32)
    params[d] = (T(w).cuda(), T(bias).cuda())
    y = np.maximum(orc.octree_conv(x, w, host, d, co, [3, 3, 3], 1) + bias[:, None], 0)
    top, _ = orc.max_pool(y)
    x = orc.pad(top, b.prop("child", d - 1))
  got = oc.stacks.lenet_trunk(dev, 6, params)
  assert tuple(got.shape) == (1, 256, int(b.nnum[2]), 1)
  assert relerr(got.cpu().numpy().reshape(x.shape), x) < 1e-4
  p16 = {d: (w.bfloat16(), bb) for d, (w, bb) in params.items()}
  got16 = oc.stacks.lenet_trunk(dev, 6, p16, data=T(data).cuda().view(1, 3, -1, 1).bfloat16())
  # four bf16 layers against the fp32 chain: the same 2e-2 as a single operator (each layer rounds
  # its inputs and outputs to 8 significant bits, about 4e-3 of the largest value per layer, and
  # ReLU plus max pooling do not amplify it: the chain measures 4e-3 as well)
  assert relerr(got16.float().cpu().numpy().reshape(x.shape), x) < 2e-2


@pytest.mark.parametrize("nempty", [False, True])
def test_unet_trunk(oc, orc, tree, nempty):
  """Encoder / decoder op order of BASELINE config 4 at small scale: channels 32-64-128,
  2x2x2 stride-2 down convs, stride-2 deconvs up, skip concatenation."""
  host, dev, b = tree
  rng = np.random.default_rng(3)
  depth, stages = 6, 2
  ch = {6: 16, 5: 32, 4: 64}
  params, P = {}, {}

  def mk(key, shape, fan):
    w = (rng.standard_normal(shape) / np.sqrt(fan)).astype(np.float32)
    bias = (rng.standard_normal(shape[0] if key[0] != "up" else shape[1] // 8) * 0.1).astype(np.float32)
    params[key] = (T(w).cuda(), T(bias).cuda())
    P[key] = (w, bias)

  mk(("conv", 6), (ch[6], 3 * 27), 81)
  for d in (6, 5):
    mk(("down", d), (ch[d - 1], ch[d] * 8), ch[d] * 8)
    mk(("conv", d - 1), (ch[d - 1], ch[d - 1] * 27), ch[d - 1] * 27)
  for d in (4, 5):
    mk(("up", d), (ch[d], ch[d + 1] * 8), ch[d])
    mk(("dec", d + 1), (ch[d + 1], 2 * ch[d + 1] * 27), 2 * ch[d + 1] * 27)

  def chain(rnd):
    """the operator sequence through the oracle; `rnd` rounds weights and every stored activation
    (identity for fp32, round-to-bf16 for the bf16 trunks, which store bf16 between operators)"""
    def cbr(x, key, d, ks, stride, deconv=False):
      w, bias = P[key]
      w = rnd(w)
      cout = w.shape[1] // 8 if deconv else w.shape[0]
      if deconv and not nempty:
        x = orc.depad(x, b.prop("child", d), int(b.nnum_nempty[d]))
      fn = orc.octree_deconv if deconv else orc.octree_conv
      y = fn(x, w, host, d, cout, ks, stride, nempty)
      if (not deconv) and stride == 2 and not nempty:
        y = orc.pad(y, b.prop("child", d - 1))          # conv -> pad -> BN -> ReLU
      return rnd(np.maximum(y + bias[:, None], 0))

    x0 = rnd(b.prop("feature", 6).copy())
    if nempty:
      x0 = x0[:, b.prop("child", 6) >= 0]
    feats = {6: cbr(x0, ("conv", 6), 6, [3, 3, 3], 1)}
    d = 6
    for _ in range(stages):
      x = cbr(feats[d], ("down", d), d, [2, 2, 2], 2)
      d -= 1
      feats[d] = cbr(x, ("conv", d), d, [3, 3, 3], 1)
    x = feats[d]
    for _ in range(stages):
      x = cbr(x, ("up", d), d, [2, 2, 2], 2, deconv=True)
      d += 1
      x = cbr(np.concatenate([feats[d], x], 0), ("dec", d), d, [3, 3, 3], 1)
    return x

  x = chain(lambda a: a)
  got = oc.stacks.unet_trunk(dev, 6, params, stages=stages, nempty=nempty)
  assert relerr(got.cpu().numpy().reshape(x.shape), x) < 1e-4
  # bf16, channel-major and row-major between the operators, against the oracle chain that rounds
  # what those trunks round (weights, input, every stored activation); what is left is the order
  # of the fp32 sums and the occasional value that rounds the other way, far inside 2e-2
  x16 = chain(lambda a: T(a).bfloat16().float().numpy())
  p16 = {k: (w.bfloat16(), bias) for k, (w, bias) in params.items()}
  data16 = T(b.prop("feature", 6)).cuda().view(1, 3, -1, 1).bfloat16()
  if nempty:
    data16 = oc.nn.octree_depad(data16, dev, 6)
  got16 = oc.stacks.unet_trunk(dev, 6, p16, data=data16, stages=stages, nempty=nempty)
  assert relerr(got16.float().cpu().numpy().reshape(x16.shape), x16) < 2e-2
  rows16 = oc.stacks.unet_trunk_rows(dev, 6, p16, data=data16, stages=stages, nempty=nempty)
  assert relerr(rows16.float().cpu().numpy().reshape(x16.shape), x16) < 2e-2
  assert relerr(x16, x) < 2e-2          # and the rounded chain stays near the fp32 chain


def test_column_modules(oc, orc, tree):
  """Octree2Col / Col2Octree (pytorch/ocnn/octree2col.py:40-81) against the oracle, with gradients."""
  host, dev, b = tree
  rng = np.random.default_rng(8)
  d = 5
  H = int(b.nnum[d])
  x = rng.standard_normal((1, 3, H, 1)).astype(np.float32)
  xd = T(x).cuda().requires_grad_(True)
  col = oc.Octree2Col(d, [3, 3, 3], 1)(xd, dev)
  exp = orc.octree2col(x.reshape(3, H), [3, 3, 3], 1, b.prop("neigh", d), H)
  assert np.array_equal(col.detach().cpu().numpy(), exp.reshape(col.shape))
  back = oc.Col2Octree(d, [3, 3, 3], 1)(col, dev)
  expb = orc.col2octree(exp, [3, 3, 3], 1, b.prop("neigh", d), H)
  assert relerr(back.detach().cpu().numpy().reshape(3, H), expb.reshape(3, H)) < 1e-6
  back.sum().backward()
  assert xd.grad is not None and xd.grad.shape == xd.shape


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_operator_sequence_replays_from_a_graph(oc, tree, dtype):
  """The operators launch kernels only (no memset nodes, no waits, no allocation besides torch's
  own): a captured LeNet trunk, replayed several times with eager work and synchronisations in
  between, gives the eager result every time, also after its input has been rewritten."""
  host, dev, b = tree
  g = torch.Generator().manual_seed(3)
  chans = {6: (3, 32), 5: (32, 64), 4: (64, 128), 3: (128, 256)}
  params = {d: ((torch.randn(co, ci * 27, generator=g) / (ci * 27) ** 0.5).cuda().to(dtype),
                (torch.randn(co, generator=g) * 0.1).cuda()) for d, (ci, co) in chans.items()}
  H6 = int(b.nnum[6])
  x = torch.randn(1, 3, H6, 1, generator=g).cuda().to(dtype)
  run = lambda: oc.stacks.lenet_trunk(dev, 6, params, data=x)
  side = torch.cuda.Stream()
  side.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(side):
    for _ in range(2):
      run()
  torch.cuda.current_stream().wait_stream(side)
  graph = torch.cuda.CUDAGraph()
  with torch.cuda.graph(graph):
    out = run()
  for rep in range(4):
    if rep == 2:
      x.copy_(torch.randn(1, 3, H6, 1, generator=g).cuda().to(dtype))   # new input, same graph
    graph.replay()
    torch.cuda.synchronize()
    eager = run()
    torch.cuda.synchronize()
    assert torch.equal(out, eager), rep
