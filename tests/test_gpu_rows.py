"""Row-major bf16 activations: ocnn_rows_from_channels / ocnn_channels_from_rows and
ocnn_octree_conv_rows against the channel-major operators (pytorch/cpp/octree_conv.cpp:131-157
semantics).  The row-major convolution runs the same kernel on the same operands in the same
order as the channel-major one, so the bar is bit equality, and the channel-major operator is
itself checked against the oracle in test_gpu_ops.py / test_gpu_windows.py."""
import numpy as np
import pytest
import torch

from oracle.checker import make_points_blob

pytestmark = pytest.mark.gpu


def T(a):
  return torch.from_numpy(np.ascontiguousarray(a))


@pytest.fixture(scope="module")
def octree(oc, synthetic):
  clouds = []
  for i in range(3):
    p, n, _ = synthetic.shape_cloud(6000, 70 + i)
    clouds.append(T(make_points_blob(p, n)).cuda())
  return oc.nn.points2octree_batch(clouds, 6, 2)


def test_rows_round_trip(oc):
  F = oc.nn
  g = torch.Generator().manual_seed(5)
  for c, h in ((1, 8), (3, 1000), (16, 64), (20, 4104), (64, 33000), (70, 8)):
    x = torch.randn(1, c, h, 1, generator=g).bfloat16().cuda()
    rows = F.to_rows(x)
    assert rows.shape == (h + 1, F.rows_pitch(c))
    assert torch.equal(rows[:h, :c], x.view(c, h).t())
    assert not rows[h].any() and not rows[:, c:].any()
    assert torch.equal(F.from_rows(rows, c), x)


@pytest.mark.parametrize("cin,cout", [(3, 32), (64, 64), (32, 48), (20, 70), (16, 130)])
def test_conv_rows_equals_channel_major(oc, octree, cin, cout):
  F = oc.nn
  info = F.octree_info(octree)
  g = torch.Generator().manual_seed(cin * 1000 + cout)
  for depth in (6, 4):
    H = info.nnum(depth)
    x = torch.randn(1, cin, H, 1, generator=g).bfloat16().cuda()
    bias = torch.randn(cout, generator=g).cuda()
    for deconv in (False, True):
      shape = (cin, cout * 27) if deconv else (cout, cin * 27)
      w = (torch.randn(*shape, generator=g) * 0.05).bfloat16().cuda()
      for b, relu in ((None, False), (bias, True), (bias, False), (None, True)):
        exp = F.octree_conv_fused(x, w, b, relu, octree, depth, cout, [3, 3, 3], 1, False, deconv=deconv)
        rows = F.octree_conv_rows(F.to_rows(x), cin, w, octree, depth, cout, bias=b, relu=relu, deconv=deconv)
        assert rows.shape == (H + 1, F.rows_pitch(cout))
        assert not rows[H].any(), "the row behind the last one must be zero"
        assert not rows[:, cout:].any(), "padding channels must be zero"
        assert torch.equal(F.from_rows(rows, cout), exp), (depth, deconv, relu, b is not None)


def test_conv_rows_chain(oc, octree):
  """two members: the second reads what the first wrote, zero row and padding included"""
  F = oc.nn
  info = F.octree_info(octree)
  g = torch.Generator().manual_seed(9)
  H = info.nnum(6)
  x = torch.randn(1, 24, H, 1, generator=g).bfloat16().cuda()
  w1 = (torch.randn(40, 24 * 27, generator=g) * 0.05).bfloat16().cuda()
  w2 = (torch.randn(64, 40 * 27, generator=g) * 0.05).bfloat16().cuda()
  b1, b2 = torch.randn(40, generator=g).cuda(), torch.randn(64, generator=g).cuda()
  mid = torch.full((H + 1, F.rows_pitch(40)), float("nan"), dtype=torch.bfloat16, device="cuda")   # must be overwritten whole
  F.octree_conv_rows(F.to_rows(x), 24, w1, octree, 6, 40, bias=b1, relu=True, out=mid)
  got = F.from_rows(F.octree_conv_rows(mid, 40, w2, octree, 6, 64, bias=b2, relu=True), 64)
  y = F.octree_conv_fused(x, w1, b1, True, octree, 6, 40, [3, 3, 3], 1, False)
  exp = F.octree_conv_fused(y, w2, b2, True, octree, 6, 64, [3, 3, 3], 1, False)
  assert torch.equal(got, exp)


def test_conv_rows_rejects(oc, octree):
  F = oc.nn
  x = torch.zeros(F.octree_info(octree).nnum(6) + 1, 16, dtype=torch.bfloat16, device="cuda")
  w = torch.zeros(32, 16 * 27, dtype=torch.bfloat16, device="cuda")
  with pytest.raises(oc.nn.OcnnError):
    F.octree_conv_rows(x[:-1].contiguous(), 16, w, octree, 6, 32)       # one row short
  with pytest.raises(oc.nn.OcnnError):
    F.octree_conv_rows(x, 20, w, octree, 6, 32)                         # pitch does not match the channels


def bf16_round(a):
  return T(a).bfloat16().float().numpy()


def close(got, exp, tol, what):
  """largest error against the largest magnitude, and element-wise against |exp| + the channel's rms"""
  assert got.shape == exp.shape, what
  assert float(np.abs(got - exp).max()) / float(np.abs(exp).max()) < tol, what
  rms = np.sqrt((exp.astype(np.float64) ** 2).mean(axis=1, keepdims=True)).astype(np.float32)
  bad = np.abs(got - exp) > tol * (np.abs(exp) + rms)
  assert not bad.any(), (what, int(bad.sum()))


@pytest.fixture(scope="module")
def small(oc, orc, synthetic):
  from oracle.checker import OctreeBlob
  pbs = [make_points_blob(*synthetic.shape_cloud(3000, 61 + i)[:2]) for i in range(2)]
  host = orc.octree_batch([orc.points2octree(p, 6, 2) for p in pbs])
  return host, T(host).cuda(), OctreeBlob(host)


@pytest.mark.parametrize("cin,cout", [(16, 32), (32, 64), (24, 40), (128, 256), (64, 16), (48, 64), (80, 32), (160, 24)])
def test_stride2_rows_against_oracle(oc, orc, small, cin, cout):
  """2x2x2 stride 2 with the pad / depad of the reference's modules folded in
  (pytorch/ocnn/octree_conv.py:102-127), bias and ReLU fused: 2e-2 against the oracle in fp32 on
  bf16-rounded operands."""
  host, dev, b = small
  F = oc.nn
  rng = np.random.default_rng(cin * 7 + cout)
  d = 6
  H = int(b.nnum[d])
  x = bf16_round(rng.standard_normal((cin, H)).astype(np.float32))
  bias = (rng.standard_normal(cout) * 0.2).astype(np.float32)
  xr = F.to_rows(T(x).cuda().view(1, cin, H, 1).bfloat16())
  # convolution: nodes of depth 5 out, an empty node holds relu(bias)
  w = bf16_round((rng.standard_normal((cout, cin * 8)) / np.sqrt(cin * 8)).astype(np.float32))
  y = orc.pad(orc.octree_conv(x, w, host, d, cout, [2, 2, 2], 2, False), b.prop("child", d - 1))
  exp = np.maximum(y + bias[:, None], 0)
  rows = F.octree_conv_rows(xr, cin, T(w).cuda().bfloat16(), dev, d, cout, bias=T(bias).cuda(), relu=True,
                            kernel_size=(2, 2, 2), stride=2)
  assert rows.shape == (int(b.nnum[d - 1]) + 1, F.rows_pitch(cout))
  assert not rows[-1].any() and not rows[:, cout:].any()
  close(F.from_rows(rows, cout).float().cpu().numpy().reshape(exp.shape), exp, 2e-2, ("conv", cin, cout))
  # deconvolution from depth 5 to depth 6: rows of all nodes of depth 5 in, the non-empty ones are used
  d = 5
  H = int(b.nnum[d])
  x = bf16_round(rng.standard_normal((cin, H)).astype(np.float32))
  w = bf16_round((rng.standard_normal((cin, cout * 8)) / np.sqrt(cin)).astype(np.float32))
  xne = orc.depad(x, b.prop("child", d), int(b.nnum_nempty[d]))
  exp = orc.octree_deconv(xne, w, host, d, cout, [2, 2, 2], 2, False) + bias[:, None]
  xr = F.to_rows(T(x).cuda().view(1, cin, H, 1).bfloat16())
  wide = torch.full((int(b.nnum[d + 1]) + 1, F.rows_pitch(cout) + 32), 7.0, dtype=torch.bfloat16, device="cuda")
  rows = F.octree_conv_rows(xr, cin, T(w).cuda().bfloat16(), dev, d, cout, bias=T(bias).cuda(), relu=False,
                            deconv=True, kernel_size=(2, 2, 2), stride=2, out=wide[:, 16:16 + F.rows_pitch(cout)])
  assert (wide[:, :16] == 7).all() and (wide[:, 16 + F.rows_pitch(cout):] == 7).all(), "wrote outside its slice"
  assert not rows[-1].any() and not rows[:, cout:].any()
  close(F.from_rows(rows.contiguous(), cout).float().cpu().numpy().reshape(exp.shape), exp, 2e-2, ("deconv", cin, cout))


def test_unet_trunk_rows(oc, small):
  """the row-major trunk against the channel-major bf16 trunk (same operators, the 3x3x3 ones
  bit-identical, the stride-2 ones summed in another order): 2e-2 over the whole chain, as for a
  single bf16 operator (measured: below 1e-2)"""
  host, dev, b = small
  rng = np.random.default_rng(3)
  ch = {6: 16, 5: 32, 4: 64}
  params = {}

  def mk(key, shape, fan):
    w = (rng.standard_normal(shape) / np.sqrt(fan)).astype(np.float32)
    bias = (rng.standard_normal(shape[0] if key[0] != "up" else shape[1] // 8) * 0.1).astype(np.float32)
    params[key] = (T(w).cuda().bfloat16(), T(bias).cuda())

  mk(("conv", 6), (ch[6], 3 * 27), 81)
  for d in (6, 5):
    mk(("down", d), (ch[d - 1], ch[d] * 8), ch[d] * 8)
    mk(("conv", d - 1), (ch[d - 1], ch[d - 1] * 27), ch[d - 1] * 27)
  for d in (4, 5):
    mk(("up", d), (ch[d], ch[d + 1] * 8), ch[d])
    mk(("dec", d + 1), (ch[d + 1], 2 * ch[d + 1] * 27), 2 * ch[d + 1] * 27)
  data = oc.nn.octree_property(dev, "feature", 6).bfloat16()
  exp = oc.stacks.unet_trunk(dev, 6, params, data=data, stages=2).float().cpu().numpy()
  got = oc.stacks.unet_trunk_rows(dev, 6, params, data=data, stages=2).float().cpu().numpy()
  close(got.reshape(got.shape[1], -1), exp.reshape(exp.shape[1], -1), 2e-2, "unet trunk")


def test_rows_operators_full_size(oc, synthetic):
  """The depth-9 scene (1.5 M octants): 3x3x3 bit-identical to the channel-major operator, the
  stride-2 pair within 2e-2 of it, and every operator the same on a second run (a store whose data
  registers were overwritten too early showed up only at this size, as a few words that changed
  from run to run)."""
  F, S = oc.nn, oc.stacks
  p, n, f = synthetic.room_cloud(250000, 3)
  octree = F.points2octree_batch([T(make_points_blob(p, n, f)).cuda()], 9, 2)
  info = F.octree_info(octree)
  g = torch.Generator().manual_seed(4)
  H9 = info.nnum(9)
  x = torch.randn(1, 32, H9, 1, generator=g).bfloat16().cuda()
  w3 = (torch.randn(32, 32 * 27, generator=g) * 0.05).bfloat16().cuda()
  wd = (torch.randn(64, 32 * 8, generator=g) * 0.08).bfloat16().cuda()
  wu = (torch.randn(64, 32 * 8, generator=g) * 0.1).bfloat16().cuda()
  b32, b64 = torch.randn(32, generator=g).cuda() * 0.2, torch.randn(64, generator=g).cuda() * 0.2
  xr = F.to_rows(x)

  def same(fn):
    a = fn()
    for _ in range(2):
      assert torch.equal(a, fn()), "results change from run to run"
    return a

  y = same(lambda: F.octree_conv_rows(xr, 32, w3, octree, 9, 32, bias=b32, relu=True))
  y_ref = F.octree_conv_fused(x, w3, b32, True, octree, 9, 32, [3, 3, 3], 1, False)
  assert torch.equal(F.from_rows(y, 32), y_ref)
  dn = same(lambda: F.octree_conv_rows(y, 32, wd, octree, 9, 64, bias=b64, relu=True, kernel_size=(2, 2, 2), stride=2))
  dn_ref = S.conv_bn_relu(y_ref, wd, b64, octree, 9, 64, (2, 2, 2), 2)
  close(F.from_rows(dn, 64).float().cpu().numpy().reshape(64, -1), dn_ref.float().cpu().numpy().reshape(64, -1), 2e-2, "down")
  up = same(lambda: F.octree_conv_rows(dn, 64, wu, octree, 8, 32, bias=b32, relu=True, deconv=True,
                                       kernel_size=(2, 2, 2), stride=2))
  up_ref = S.conv_bn_relu(dn_ref, wu, b32, octree, 8, 32, (2, 2, 2), 2, deconv=True)
  close(F.from_rows(up, 32).float().cpu().numpy().reshape(32, -1), up_ref.float().cpu().numpy().reshape(32, -1), 2e-2, "up")


@pytest.mark.parametrize("cin,cout", [(3, 32), (64, 64), (24, 40), (48, 128), (128, 256), (80, 32), (176, 48)])
def test_nonempty_rows_equal_channel_major(oc, octree, cin, cout):
  """over the non-empty nodes the row-major operators run the kernel of the channel-major entry
  points on the same operands in the same order: equal bits, for 3x3x3 stride 1 and for 2x2x2
  stride 2, convolution and deconvolution"""
  F = oc.nn
  info = F.octree_info(octree)
  g = torch.Generator().manual_seed(cin * 31 + cout)
  bias = torch.randn(cout, generator=g).cuda()
  for depth in (6, 5):
    Hne = info.nnum_nempty(depth)
    x = torch.randn(1, cin, Hne, 1, generator=g).bfloat16().cuda()
    xr = F.to_rows(x)
    for ks, stride, deconv in (([3, 3, 3], 1, False), ([3, 3, 3], 1, True), ([2, 2, 2], 2, False), ([2, 2, 2], 2, True)):
      if deconv and stride == 2 and depth == 6:
        continue   # no level below the finest one
      K = ks[0] * ks[1] * ks[2]
      shape = (cin, cout * K) if deconv else (cout, cin * K)
      w = (torch.randn(*shape, generator=g) * 0.05).bfloat16().cuda()
      for b, relu in ((None, False), (bias, True)):
        exp = F.octree_conv_fused(x, w, b, relu, octree, depth, cout, ks, stride, True, deconv=deconv)
        rows = F.octree_conv_rows(xr, cin, w, octree, depth, cout, bias=b, relu=relu, deconv=deconv,
                                  kernel_size=tuple(ks), stride=stride, nempty=True)
        assert rows.shape == (exp.size(2) + 1, F.rows_pitch(cout))
        assert not rows[-1].any() and not rows[:, cout:].any()
        assert torch.equal(F.from_rows(rows, cout), exp), (depth, ks, stride, deconv, relu)


def test_unet_trunk_rows_nonempty(oc, small):
  host, dev, b = small
  rng = np.random.default_rng(5)
  ch = {6: 16, 5: 32, 4: 64}
  params = {}

  def mk(key, shape, fan):
    w = (rng.standard_normal(shape) / np.sqrt(fan)).astype(np.float32)
    bias = (rng.standard_normal(shape[0] if key[0] != "up" else shape[1] // 8) * 0.1).astype(np.float32)
    params[key] = (T(w).cuda().bfloat16(), T(bias).cuda())

  mk(("conv", 6), (ch[6], 3 * 27), 81)
  for d in (6, 5):
    mk(("down", d), (ch[d - 1], ch[d] * 8), ch[d] * 8)
    mk(("conv", d - 1), (ch[d - 1], ch[d - 1] * 27), ch[d - 1] * 27)
  for d in (4, 5):
    mk(("up", d), (ch[d], ch[d + 1] * 8), ch[d])
    mk(("dec", d + 1), (ch[d + 1], 2 * ch[d + 1] * 27), 2 * ch[d + 1] * 27)
  data = oc.nn.octree_depad(oc.nn.octree_property(dev, "feature", 6).bfloat16(), dev, 6)
  exp = oc.stacks.unet_trunk(dev, 6, params, data=data, stages=2, nempty=True)
  got = oc.stacks.unet_trunk_rows(dev, 6, params, data=data, stages=2, nempty=True)
  assert torch.equal(got, exp)   # every member is bit-identical to its channel-major counterpart


def test_packed_weights_and_cached_links(oc, octree):
  """constant_weights=True keeps the packed weights with the weight tensor and the inverted child
  links with the octree: the same bits as the plain call, also after the weights were written to"""
  F = oc.nn
  info = F.octree_info(octree)
  g = torch.Generator().manual_seed(77)
  bias = torch.randn(48, generator=g).cuda()
  for nempty in (False, True):
    for ks, stride, deconv, depth in (((3, 3, 3), 1, False, 6), ((2, 2, 2), 2, False, 6), ((2, 2, 2), 2, True, 5)):
      K = ks[0] * ks[1] * ks[2]
      H = info.nnum_nempty(depth) if nempty else info.nnum(depth)
      x = F.to_rows(torch.randn(1, 32, H, 1, generator=g).bfloat16().cuda())
      shape = (32, 48 * K) if deconv else (48, 32 * K)
      w = (torch.randn(*shape, generator=g) * 0.05).bfloat16().cuda()
      kw = dict(bias=bias, relu=True, deconv=deconv, kernel_size=ks, stride=stride, nempty=nempty)
      for _ in range(2):
        exp = F.octree_conv_rows(x, 32, w, octree, depth, 48, **kw)
        for _ in range(2):   # the second call finds everything in place
          got = F.octree_conv_rows(x, 32, w, octree, depth, 48, constant_weights=True, **kw)
          assert torch.equal(got, exp), (nempty, ks, stride, deconv)
        w.mul_(1.5)        # a write to the tensor: the next call packs again


def test_packed_weights_of_another_shape_are_refused(oc, octree):
  """The packed form carries no shape: the call checks its byte count against the operator it is
  asked to run, and a write that bypasses the version counter needs forget_cached."""
  import ctypes as C
  F = oc.nn
  info = F.octree_info(octree)
  H = info.nnum(6)
  g = torch.Generator().manual_seed(78)
  x = F.to_rows(torch.randn(1, 32, H, 1, generator=g).bfloat16().cuda())
  w = (torch.randn(48, 32 * 27, generator=g) * 0.05).bfloat16().cuda()
  F.octree_conv_rows(x, 32, w, octree, 6, 48, constant_weights=True)
  (stamp, packed), = w._ocnn_rows_packed.values()
  out = torch.empty(H + 1, 128, dtype=torch.bfloat16, device="cuda")
  ks = (C.c_int * 3)(3, 3, 3)
  P = lambda t: C.c_void_p(t.data_ptr())
  args = lambda cout, nbytes: (P(out), 128, P(x), x.stride(0), 32, H, P(packed), C.c_size_t(nbytes), None, None, None, 0, 0,
                               P(octree), info.p, 6, cout, ks, 1, 0, 1, None, C.c_size_t(0),
                               C.c_void_p(torch.cuda.current_stream().cuda_stream))
  L = oc.lib.get()
  assert L.ocnn_octree_conv_rows_packed(*args(48, packed.numel())) == 0
  assert L.ocnn_octree_conv_rows_packed(*args(128, packed.numel())) == -4       # packed for 48 output channels
  assert L.ocnn_octree_conv_rows_packed(*args(48, packed.numel() - 16)) == -4
  # a write through .data is invisible to the version counter: the stale pack is used until forgotten
  exp_old = F.octree_conv_rows(x, 32, w, octree, 6, 48, constant_weights=True)
  w.data.mul_(2.0)
  assert w._version == stamp[0]
  assert torch.equal(F.octree_conv_rows(x, 32, w, octree, 6, 48, constant_weights=True), exp_old)
  F.forget_cached(w)
  assert torch.equal(F.octree_conv_rows(x, 32, w, octree, 6, 48, constant_weights=True),
                     F.octree_conv_rows(x, 32, w, octree, 6, 48))


def test_max_pool_rows_equals_channel_major(oc, octree):
  """max_pool + pad on row-major activations: values and mask bit-equal to the channel-major pair
  (which the oracle checks in test_gpu_ops.py), zero row and padding channels written."""
  F = oc.nn
  info = F.octree_info(octree)
  g = torch.Generator().manual_seed(91)
  for depth in (6, 4, 3):
    for c in (3, 16, 40, 64):
      H, Hp = info.nnum(depth), info.nnum(depth - 1)
      x = torch.randn(1, c, H, 1, generator=g).bfloat16().cuda()
      x[0, :, 1::8] = x[0, :, 0::8]      # ties between siblings 0 and 1: the first maximum must win
      top, mask = F.octree_max_pool(x, octree, depth)
      exp = F.octree_pad(top, octree, depth - 1)
      rows, mrows = F.octree_max_pool_rows(F.to_rows(x), c, octree, depth, return_mask=True)
      assert rows.shape == (Hp + 1, F.rows_pitch(c))
      assert torch.equal(F.from_rows(rows, c), exp), (depth, c)
      assert not rows[Hp].any() and not rows[:, c:].any()
      child = F.octree_property(octree, "child", depth - 1)
      exp_mask = torch.full((c, Hp), -1, dtype=torch.int32, device="cuda")
      exp_mask[:, child >= 0] = mask.view(c, -1)
      assert torch.equal(mrows[:Hp, :c].t(), exp_mask), (depth, c)
      assert torch.equal(F.octree_max_pool_rows(F.to_rows(x), c, octree, depth), rows)


def test_lenet_trunk_rows(oc, octree):
  """conv -> ReLU -> max_pool (+pad) from depth 6 down to depth 2 on row-major activations == the
  channel-major bf16 trunk, bit for bit (same kernels, same operands, same order)."""
  g = torch.Generator().manual_seed(92)
  chans = {6: (3, 32), 5: (32, 64), 4: (64, 128), 3: (128, 256)}
  params = {d: ((torch.randn(co, ci * 27, generator=g) / (ci * 27) ** 0.5).bfloat16().cuda(),
                (torch.randn(co, generator=g) * 0.1).cuda()) for d, (ci, co) in chans.items()}
  info = oc.nn.octree_info(octree)
  x = torch.randn(1, 3, info.nnum(6), 1, generator=g).bfloat16().cuda()
  exp = oc.stacks.lenet_trunk(octree, 6, params, data=x)
  for cw in (False, True, True):
    got = oc.stacks.lenet_trunk_rows(octree, 6, params, data=x, constant_weights=cw)
    assert torch.equal(got, exp)


def test_row_kernel_forms_and_source_tables_agree(oc, octree):
  """Over the non-empty nodes the bf16 row kernels exist in two forms (weights staged in LDS /
  read per live tap), and the source rows of a tile come from a table made ahead (kept with the
  octree under constant_weights) or from the look-up inside the kernel: every combination gives
  the same bits."""
  F = oc.nn
  L = oc.lib.get()
  info = F.octree_info(octree)
  g = torch.Generator().manual_seed(93)
  try:
    for depth, cin, cout, ks, stride, deconv in ((6, 32, 48, (3, 3, 3), 1, False), (5, 64, 128, (3, 3, 3), 1, True),
                                                 (6, 16, 32, (2, 2, 2), 2, False), (5, 24, 16, (2, 2, 2), 2, True)):
      K = ks[0] * ks[1] * ks[2]
      H = info.nnum_nempty(depth)
      x = torch.randn(1, cin, H, 1, generator=g).bfloat16().cuda()
      xr = F.to_rows(x)
      shape = (cin, cout * K) if deconv else (cout, cin * K)
      w = (torch.randn(*shape, generator=g) * 0.05).bfloat16().cuda()
      kw = dict(deconv=deconv, kernel_size=ks, stride=stride, nempty=True)
      results = []
      for form in (0, 1):
        L.ocnn_conv_rows_direct(form)
        F.forget_cached(octree)
        results.append(F.octree_conv_rows(xr, cin, w, octree, depth, cout, **kw))                          # look-up in the kernel
        results.append(F.octree_conv_rows(xr, cin, w, octree, depth, cout, constant_weights=True, **kw))   # table kept
        results.append(F.octree_conv_rows(xr, cin, w, octree, depth, cout, constant_weights=True, **kw))
        fn = F.octree_deconv if deconv else F.octree_conv
        results.append(F.to_rows(fn(x, w, octree, depth, cout, list(ks), stride, True)))                     # channel-major
      for r in results[1:]:
        assert torch.equal(r, results[0]), (depth, cin, cout, ks, stride, deconv)
  finally:
    L.ocnn_conv_rows_direct(1)


def test_row_kernel_workgroup_sizes_at_scene_levels(oc, synthetic):
  """The barrier-free row kernel runs in workgroups of four, two or one wavefront, picked by how the
  level's tiles spread over the device (depth 6 of the scene: four; depth 7: two; depth 9: one).
  Whatever the size, it forms the same products in the same order as the staged kernel (always 256
  columns a workgroup), so at each of those levels the two forms, row-major and channel-major,
  give the same bits."""
  F = oc.nn
  L = oc.lib.get()
  p, n, f = synthetic.room_cloud(250000, 3)
  octree = F.points2octree_batch([T(make_points_blob(p, n, f)).cuda()], 9, 2)
  info = F.octree_info(octree)
  g = torch.Generator().manual_seed(17)
  try:
    for depth, cin, cout in ((6, 256, 256), (7, 128, 128), (7, 64, 64), (9, 64, 64), (9, 32, 32)):
      H = info.nnum_nempty(depth)
      x = torch.randn(1, cin, H, 1, generator=g).bfloat16().cuda()
      xr = F.to_rows(x)
      w = (torch.randn(cout, cin * 27, generator=g) * 0.05).bfloat16().cuda()
      b = (torch.randn(cout, generator=g) * 0.1).cuda()
      results = []
      for form in (1, 0):
        L.ocnn_conv_rows_direct(form)
        F.forget_cached(octree)
        results.append(F.octree_conv_rows(xr, cin, w, octree, depth, cout, bias=b, relu=True, nempty=True))
        results.append(F.to_rows(F.octree_conv_fused(x, w, b, True, octree, depth, cout, [3, 3, 3], 1, True)))
      for r in results[1:]:
        assert torch.equal(r, results[0]), (depth, cin, cout)
      assert float(results[0].float().abs().max()) > 0
  finally:
    L.ocnn_conv_rows_direct(1)


def test_rows_small_levels_take_either_kernel(oc, octree):
  """Row-major 3x3x3 over all nodes: a small level runs the LDS kernel with a row-major store, a
  large one the register-fed kernel; forced onto the register-fed kernel (the test hook of the tile
  threshold) the small level gives the same bits, with and without bias + ReLU, conv and deconv,
  also into a channel slice of a wider tensor, and they are the channel-major operator's."""
  F = oc.nn
  L = oc.lib.get()
  info = F.octree_info(octree)
  g = torch.Generator().manual_seed(23)
  try:
    for depth, cin, cout, deconv in ((6, 32, 64, False), (5, 48, 130, False), (6, 16, 32, True), (4, 128, 256, False)):
      H = info.nnum(depth)
      x = torch.randn(1, cin, H, 1, generator=g).bfloat16().cuda()
      xr = F.to_rows(x)
      shape = (cin, cout * 27) if deconv else (cout, cin * 27)
      w = (torch.randn(*shape, generator=g) * 0.05).bfloat16().cuda()
      b = (torch.randn(cout, generator=g) * 0.1).cuda()
      res = []
      for thr in (0, -1):
        L.ocnn_conv_bf16_tile_threshold(thr)
        res.append(F.octree_conv_rows(xr, cin, w, octree, depth, cout, bias=b, relu=True, deconv=deconv))
        res.append(F.octree_conv_rows(xr, cin, w, octree, depth, cout, deconv=deconv))
        wide = torch.full((H + 1, F.rows_pitch(cout) + 32), 7.0, dtype=torch.bfloat16, device="cuda")
        F.octree_conv_rows(xr, cin, w, octree, depth, cout, bias=b, relu=True, deconv=deconv, out=wide[:, 16:16 + F.rows_pitch(cout)])
        assert torch.equal(wide[:, 16:16 + F.rows_pitch(cout)], res[-2]) and bool((wide[:, :16] == 7).all()) and bool((wide[:, 16 + F.rows_pitch(cout):] == 7).all())
      assert torch.equal(res[0], res[2]) and torch.equal(res[1], res[3]), (depth, cin, cout, deconv)
      ref = F.octree_conv_fused(x, w, b, True, octree, depth, cout, [3, 3, 3], 1, False, deconv=deconv)
      assert torch.equal(F.from_rows(res[0], cout), ref), (depth, cin, cout, deconv)
      assert bool((res[0][H] == 0).all()) and bool((res[0][:, cout:] == 0).all())
  finally:
    L.ocnn_conv_bf16_tile_threshold(0)
