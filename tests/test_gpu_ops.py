"""GPU parity of the feature operators: octree2col / col2octree, conv / deconv (fp32 within
1e-4 relative, bf16 within 2e-2 relative of the CPU oracle), pooling and padding (bit exact)."""
import numpy as np
import pytest
import torch

from oracle.checker import OctreeBlob, make_points_blob

pytestmark = pytest.mark.gpu

TOL_F32 = 1e-4   # relative to the largest magnitude of the expected tensor
TOL_BF16 = 2e-2

KERNELS = [[3, 3, 3], [2, 2, 2], [3, 1, 1], [1, 3, 1], [1, 1, 3], [3, 3, 1], [3, 1, 3], [1, 3, 3], [1, 1, 1]]


def T(a):
  return torch.from_numpy(np.ascontiguousarray(a))


def relerr(got, exp):
  return float(np.abs(got.astype(np.float64) - exp).max() / (np.abs(exp).max() + 1e-30))


@pytest.fixture(scope="module")
def tree(oc, orc, samples, synthetic):
  """A batch of three built octrees (depth 6) plus the sample batch of the reference tests."""
  pbs = [make_points_blob(*synthetic.shape_cloud(4000, 31 + i)[:2]) for i in range(3)]
  host = orc.octree_batch([orc.points2octree(p, 6, 2) for p in pbs])
  shost = orc.octree_batch([samples[n] for n in ("octree_1", "octree_2", "octree_2", "octree_1")])
  return {"host": host, "dev": T(host).cuda(), "blob": OctreeBlob(host),
          "shost": shost, "sdev": T(shost).cuda(), "sblob": OctreeBlob(shost)}


def closed_form_col(data, idx_map, stride):
  K, C = len(idx_map), data.shape[0]
  top_h = 8 if stride == 1 else 1
  out = np.zeros((C, K, top_h), np.float32)
  for c in range(C):
    for k in range(K):
      for h in range(top_h):
        z, y, x = h & 1, (h & 2) >> 1, h >> 2
        t = idx_map[k]
        z, y, x = z + t % 3 - 1, y + (t // 3) % 3 - 1, x + t // 9 - 1
        if -1 < x < 2 and -1 < y < 2 and -1 < z < 2:
          out[c, k, h] = data[c, x * 4 + y * 2 + z]
  return out


def test_octree2col_closed_form(oc, samples):
  """pytorch/test/test_octree2col.py:23-67 incl. the nempty variant on the all-non-empty depth 1."""
  maps = {(3, 3, 3): list(range(27)), (2, 2, 2): [13, 14, 16, 17, 22, 23, 25, 26], (3, 1, 1): [4, 13, 22],
          (3, 3, 1): [1, 4, 7, 10, 13, 16, 19, 22, 25], (1, 1, 1): [13]}
  octree = oc.nn.octree_batch([T(samples["octree_1"])])
  data = np.random.default_rng(0).uniform(-1, 1, (1, 3, 8, 1)).astype(np.float32)
  for stride in (1, 2):
    for ks, m in maps.items():
      exp = closed_form_col(data.reshape(3, 8), m, stride)
      for nempty in (False, True):
        got = oc.nn.octree2col(T(data).cuda(), octree, 1, list(ks), stride, nempty)
        assert np.array_equal(got.cpu().numpy(), exp), (ks, stride, nempty)


@pytest.mark.parametrize("stride", [1, 2])
def test_col_ops_vs_oracle(oc, orc, tree, stride):
  b, dev = tree["blob"], tree["dev"]
  d = 5
  H, Hne = int(b.nnum[d]), int(b.nnum_nempty[d])
  neigh, child = b.prop("neigh", d).reshape(-1), b.prop("child", d)
  ichild = np.zeros(Hne, np.int32)
  ichild[child[child >= 0]] = np.nonzero(child >= 0)[0]
  rng = np.random.default_rng(1)
  x = rng.standard_normal((5, H)).astype(np.float32)
  xn = rng.standard_normal((5, Hne)).astype(np.float32)
  for ks in KERNELS:
    h = H if stride == 1 else H // 8
    col = oc.nn.octree2col(T(x).cuda().view(1, 5, H, 1), dev, d, ks, stride, False)
    exp = orc.octree2col(x, ks, stride, neigh, h)
    assert np.array_equal(col.cpu().numpy(), exp), ks
    colb = oc.nn.octree2col(T(x).cuda().view(1, 5, H, 1).bfloat16(), dev, d, ks, stride, False)
    assert torch.equal(colb, T(exp).cuda().bfloat16())
    back = oc.nn.col2octree(col, dev, d, ks, stride, False)
    assert relerr(back.cpu().numpy().reshape(5, H), orc.col2octree(exp, ks, stride, neigh, h)) < TOL_F32
    hp = Hne if stride == 1 else H // 8
    colp = oc.nn.octree2col(T(xn).cuda().view(1, 5, Hne, 1), dev, d, ks, stride, True)
    expp = orc.octree2colP(xn, ks, stride, neigh, child, ichild, hp)
    assert np.array_equal(colp.cpu().numpy(), expp), ks
    backp = oc.nn.col2octree(colp, dev, d, ks, stride, True)
    assert relerr(backp.cpu().numpy().reshape(5, Hne),
                  orc.col2octreeP(expp, ks, stride, neigh, child, ichild, hp, Hne)) < TOL_F32


def test_octree2col_chunks_and_unaligned_rows(oc, orc, tree):
  """octree2col through the C-ABI in column chunks (chunk n holds columns n*height_col ..., the
  columns past the last node are zero, octree_nn.cpp:188-214), written into a buffer that does
  not start on a 256-byte line, for all nodes and for the non-empty ones, fp32 and bf16."""
  import ctypes as C
  b = tree["blob"]
  d = 5
  H, Hne = int(b.nnum[d]), int(b.nnum_nempty[d])
  neigh, child = b.prop("neigh", d).reshape(-1), b.prop("child", d)
  ichild = np.zeros(Hne, np.int32)
  ichild[child[child >= 0]] = np.nonzero(child >= 0)[0]
  rng = np.random.default_rng(11)
  P = lambda t, off=0: C.c_void_p(t.data_ptr() + off)
  st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
  neigh_d, child_d, ichild_d = T(neigh).cuda(), T(child).cuda(), T(ichild).cuda()
  Cc = 11   # more than one channel chunk, the last one ragged
  x = rng.standard_normal((Cc, H)).astype(np.float32)
  xn = rng.standard_normal((Cc, Hne)).astype(np.float32)
  for dt, tt in ((0, torch.float32), (1, torch.bfloat16)):
    x_d, xn_d = T(x).cuda().to(tt), T(xn).cuda().to(tt)
    xr, xnr = x_d.float().cpu().numpy(), xn_d.float().cpu().numpy()
    for ks, stride in (([3, 3, 3], 1), ([2, 2, 2], 2), ([1, 3, 3], 1), ([3, 3, 3], 2)):
      K = int(np.prod(ks))
      ksc = (C.c_int * 3)(*ks)
      h = H if stride == 1 else H // 8
      full = orc.octree2col(xr, ks, stride, neigh, h)
      hc = (h + 2) // 3 + 5
      for n in range(3):
        exp = np.zeros((Cc, K, hc), np.float32)
        w = max(0, min(h, (n + 1) * hc) - n * hc)
        exp[:, :, :w] = full[:, :, n * hc:n * hc + w]
        buf = torch.full((Cc * K * hc + 64,), 9.0, device="cuda", dtype=tt)
        skew = 3 * buf.element_size()   # the output starts three elements into the buffer
        oc.lib.call("ocnn_octree2col", P(buf, skew), P(x_d), Cc, h, ksc, stride, P(neigh_d), hc, n, dt, st)
        got = buf.float().cpu().numpy()
        assert np.array_equal(got[3:3 + Cc * K * hc].reshape(Cc, K, hc), exp), (dt, ks, stride, n)
        assert np.all(got[:3] == 9.0) and np.all(got[3 + Cc * K * hc:] == 9.0), "wrote outside the chunk"
      hp = Hne if stride == 1 else H // 8
      fullp = orc.octree2colP(xnr, ks, stride, neigh, child, ichild, hp)
      hc = (hp + 1) // 2 + 3
      for n in range(2):
        exp = np.zeros((Cc, K, hc), np.float32)
        w = max(0, min(hp, (n + 1) * hc) - n * hc)
        exp[:, :, :w] = fullp[:, :, n * hc:n * hc + w]
        buf = torch.full((Cc * K * hc + 64,), 9.0, device="cuda", dtype=tt)
        skew = 5 * buf.element_size()
        oc.lib.call("ocnn_octree2colP", P(buf, skew), P(xn_d), Cc, hp, Hne, ksc, stride, P(neigh_d), P(child_d),
                    P(ichild_d), hc, n, dt, st)
        got = buf.float().cpu().numpy()
        assert np.array_equal(got[5:5 + Cc * K * hc].reshape(Cc, K, hc), exp), ("P", dt, ks, stride, n)
        assert np.all(got[:5] == 9.0) and np.all(got[5 + Cc * K * hc:] == 9.0), "wrote outside the chunk"


def test_octree2col_many_channels_large_level(oc, orc, synthetic):
  """From about 5 channels per workgroup on (levels of 100 000 nodes and more), stride 1 over all
  nodes runs the kernel that copies each sibling octet of a tile once per channel.  A room at
  depth 8 against the oracle, bit exact, fp32 and bf16: with the level's own table, with a table
  whose groups partly name random rows (those tiles name more octets than the copy holds and
  gather from memory) and in two column chunks through the C-ABI (octree_nn.cpp:188-214)."""
  import ctypes as C
  d = 8
  p, n, f = synthetic.room_cloud(60000, 5)
  host = orc.octree_batch([orc.points2octree(make_points_blob(p, n, f), d, 2)])
  b, dev = OctreeBlob(host), T(host).cuda()
  H = int(b.nnum[d])
  assert H >= 100000, H
  neigh = b.prop("neigh", d).reshape(-1, 64)
  rng = np.random.default_rng(21)
  tiles = (H + 63 + 255) // 256
  Cc = 5 * max(1, 2048 // tiles)
  x = rng.standard_normal((Cc, H)).astype(np.float32)
  for tt in (torch.float32, torch.bfloat16):
    x_d = T(x).cuda().to(tt)
    xr = x_d.float().cpu().numpy()
    for ks in ([3, 3, 3], [3, 1, 3]):
      col = oc.nn.octree2col(x_d.view(1, Cc, H, 1), dev, d, ks, 1, False)
      exp = orc.octree2col(xr, ks, 1, neigh.reshape(-1), H)
      assert np.array_equal(col.float().cpu().numpy(), exp), (tt, ks)
      del col, exp
  # any table: a third of the groups name random rows or nothing
  odd = neigh.copy()
  pick = np.nonzero(np.arange(len(odd)) % 96 < 32)[0]
  odd[pick] = rng.integers(-1, H, (len(pick), 64))
  Pp = lambda t, off=0: C.c_void_p(t.data_ptr() + off)
  st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
  ksc = (C.c_int * 3)(3, 3, 3)
  x_d, odd_d = T(x).cuda(), T(odd.reshape(-1)).cuda()
  exp = orc.octree2col(x, [3, 3, 3], 1, odd.reshape(-1), H)
  out = torch.empty(Cc * 27 * H, device="cuda")
  oc.lib.call("ocnn_octree2col", Pp(out), Pp(x_d), Cc, H, ksc, 1, Pp(odd_d), H, 0, 0, st)
  assert np.array_equal(out.cpu().numpy().reshape(Cc, 27, H), exp)
  Cc2 = 2 * Cc                      # half the tiles per chunk: twice the channels to stay on that kernel
  x2 = np.concatenate([x, x[::-1]])
  exp2 = np.concatenate([exp, exp[::-1]])
  x2_d = T(x2).cuda()
  hc = (H + 1) // 2 + 3
  for n in range(2):
    want = np.zeros((Cc2, 27, hc), np.float32)
    w = min(H, (n + 1) * hc) - n * hc
    want[:, :, :w] = exp2[:, :, n * hc:n * hc + w]
    buf = torch.full((Cc2 * 27 * hc + 64,), 9.0, device="cuda")
    oc.lib.call("ocnn_octree2col", Pp(buf, 12), Pp(x2_d), Cc2, H, ksc, 1, Pp(odd_d), hc, n, 0, st)
    got = buf.cpu().numpy()
    assert np.array_equal(got[3:3 + Cc2 * 27 * hc].reshape(Cc2, 27, hc), want), n
    assert np.all(got[:3] == 9.0) and np.all(got[3 + Cc2 * 27 * hc:] == 9.0), "wrote outside the chunk"


def test_col2octree_any_table_and_chunks(oc, orc, tree):
  """col2octree through the C-ABI in column chunks (octree_nn.cpp:216-241 adds chunk n to the
  rows the earlier chunks left), on the octree's own table and on tables that are not
  neighbour tables of any octree: entries shuffled inside each sibling block, and all
  entries naming one row, where the sum must still be the scatter-add of the reference."""
  import ctypes as C
  b = tree["blob"]
  d = 5
  H, Hne = int(b.nnum[d]), int(b.nnum_nempty[d])
  own, child = b.prop("neigh", d).reshape(-1).copy(), b.prop("child", d)
  ichild = np.zeros(Hne, np.int32)
  ichild[child[child >= 0]] = np.nonzero(child >= 0)[0]
  rng = np.random.default_rng(7)
  shuffled = own.reshape(-1, 64).copy()
  for row in shuffled[::3]:
    rng.shuffle(row)
  same = np.where(own >= 0, 5, -1).astype(np.int32)
  P = lambda t: C.c_void_p(t.data_ptr())
  st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
  child_d, ichild_d = T(child).cuda(), T(ichild).cuda()
  for name, table in (("own", own), ("shuffled", shuffled.reshape(-1)), ("same", same)):
    table_d = T(table.astype(np.int32)).cuda()
    for ks, stride in (([3, 3, 3], 1), ([2, 2, 2], 2), ([3, 1, 3], 1), ([3, 3, 3], 2)):
      K = int(np.prod(ks))
      ksc = (C.c_int * 3)(*ks)
      h = H if stride == 1 else H // 8
      col = rng.standard_normal((5, K, h)).astype(np.float32)
      exp = orc.col2octree(col, ks, stride, table, h)
      # three chunks, the last one ragged; the second height is a multiple of 4, which the tiled
      # gather kernel of the 27 taps asks of a chunk's first column
      for hc in ((h + 2) // 3, (h // 3 + 4) // 4 * 4):
        out = torch.full((5, H), 7.0, device="cuda")       # stale values the first chunk must replace
        for n in range(3):
          piece = np.zeros((5, K, hc), np.float32)
          w = max(0, min(h, (n + 1) * hc) - n * hc)
          piece[:, :, :w] = col[:, :, n * hc:n * hc + w]
          piece_d = T(piece).cuda()
          oc.lib.call("ocnn_col2octree", P(piece_d), P(out), 5, h, ksc, stride, P(table_d), hc, n, 0, st)
        assert relerr(out.cpu().numpy(), exp) < TOL_F32, (name, ks, stride, hc)
      hp = Hne if stride == 1 else H // 8
      colp = rng.standard_normal((5, K, hp)).astype(np.float32)
      expp = orc.col2octreeP(colp, ks, stride, table, child, ichild, hp, Hne)
      outp = torch.full((5, Hne), 7.0, device="cuda")
      colp_d = T(colp).cuda()
      oc.lib.call("ocnn_col2octreeP", P(colp_d), P(outp), 5, hp, Hne, ksc, stride, P(table_d), P(child_d),
                  P(ichild_d), hp, 0, 0, st)
      assert relerr(outp.cpu().numpy(), expp) < TOL_F32, (name, "P", ks, stride)
      # the same through the entry point that keeps the verdict on the table in a word of the
      # caller: the first call checks, the second reads the word (and must agree for a table that
      # failed the check as much as for one that passed)
      for mode, args, want in (("plain", (5, h, h << (3 * (stride - 1))), exp), ("P", (5, hp, Hne), expp)):
        mark = torch.zeros(1, dtype=torch.int64, device="cuda")
        src = T(col).cuda() if mode == "plain" else colp_d
        for check_now in (1, 0):
          got = torch.full((5, H if mode == "plain" else Hne), 7.0, device="cuda")
          oc.lib.call("ocnn_col2octree_cached", P(src), P(got), *args, ksc, stride, P(table_d),
                      P(child_d) if mode == "P" else C.c_void_p(0), P(ichild_d) if mode == "P" else C.c_void_p(0),
                      args[1], 0, 0, P(mark), check_now, st)
          assert relerr(got.cpu().numpy(), want) < TOL_F32, (name, mode, ks, stride, check_now)
        if name == "own":
          assert int(mark.item()) == 0, (mode, ks, stride)     # an octree's own table passes the check
      if stride == 2:   # without the inverse child table only the scatter form can run
        outq = torch.full((5, Hne), 7.0, device="cuda")
        oc.lib.call("ocnn_col2octreeP", P(colp_d), P(outq), 5, hp, Hne, ksc, stride, P(table_d),
                    P(child_d), C.c_void_p(0), hp, 0, 0, st)
        assert relerr(outq.cpu().numpy(), expp) < TOL_F32, (name, "P, no ichild", ks, stride)


def test_col2octree_sums_in_the_reference_order(oc, orc, tree):
  """The gather forms add the taps of a row in ascending order, which is the order in which the
  reference's loops (channel, tap, column: octree_nn.cpp:216-241) reach that row: the sums are
  equal bit for bit, on random col entries (not an octree2col image) so that every tap counts.
  Depth 6 of the tree spans several 1024-row tiles of the 27-tap kernel."""
  b, dev = tree["blob"], tree["dev"]
  rng = np.random.default_rng(21)
  for d in (4, 6):
    H = int(b.nnum[d])
    neigh = b.prop("neigh", d).reshape(-1)
    for ks in ([3, 3, 3], [3, 1, 3]):
      K = int(np.prod(ks))
      col = rng.standard_normal((11, K, H)).astype(np.float32)
      exp = orc.col2octree(col, ks, 1, neigh, H)
      got = oc.nn.col2octree(T(col).cuda(), dev, d, ks, 1, False)
      assert np.array_equal(got.cpu().numpy().reshape(11, H), exp), (d, ks)


CONV_CASES = [(ks, s, ne) for ks in KERNELS for s in (1, 2) for ne in (False, True)]


@pytest.mark.parametrize("ks,stride,nempty", CONV_CASES)
def test_conv_vs_oracle(oc, orc, tree, ks, stride, nempty):
  b, dev, host = tree["blob"], tree["dev"], tree["host"]
  d = 5
  K = ks[0] * ks[1] * ks[2]
  rng = np.random.default_rng(2)
  for ci, co in ((3, 32), (20, 70)):
    hin = int(b.nnum_nempty[d] if nempty else b.nnum[d])
    x = rng.standard_normal((ci, hin)).astype(np.float32)
    w = (rng.standard_normal((co, ci * K)) * 0.1).astype(np.float32)
    exp = orc.octree_conv(x, w, host, d, co, ks, stride, nempty)
    xt, wt = T(x).cuda().view(1, ci, hin, 1), T(w).cuda()
    got = oc.nn.octree_conv(xt, wt, dev, d, co, ks, stride, nempty)
    assert tuple(got.shape) == (1, co, exp.shape[1], 1)
    assert relerr(got.cpu().numpy().reshape(exp.shape), exp) < TOL_F32
    got16 = oc.nn.octree_conv(xt.bfloat16(), wt.bfloat16(), dev, d, co, ks, stride, nempty)
    assert got16.dtype == torch.bfloat16
    assert relerr(got16.float().cpu().numpy().reshape(exp.shape), exp) < TOL_BF16


DECONV_CASES = [(ks, s, ne) for ks in KERNELS for s in (1, 2) for ne in (False, True)]


@pytest.mark.parametrize("ks,stride,nempty", DECONV_CASES)
def test_deconv_vs_oracle(oc, orc, tree, ks, stride, nempty):
  b, dev, host = tree["blob"], tree["dev"], tree["host"]
  d = 5 if stride == 1 else 4
  K = ks[0] * ks[1] * ks[2]
  rng = np.random.default_rng(3)
  for ci, co in ((8, 5), (33, 40)):
    hin = int(b.nnum_nempty[d] if (nempty or stride == 2) else b.nnum[d])
    x = rng.standard_normal((ci, hin)).astype(np.float32)
    w = (rng.standard_normal((ci, co * K)) * 0.1).astype(np.float32)
    exp = orc.octree_deconv(x, w, host, d, co, ks, stride, nempty)
    xt, wt = T(x).cuda().view(1, ci, hin, 1), T(w).cuda()
    got = oc.nn.octree_deconv(xt, wt, dev, d, co, ks, stride, nempty)
    assert relerr(got.cpu().numpy().reshape(exp.shape), exp) < TOL_F32
    got16 = oc.nn.octree_deconv(xt.bfloat16(), wt.bfloat16(), dev, d, co, ks, stride, nempty)
    assert relerr(got16.float().cpu().numpy().reshape(exp.shape), exp) < TOL_BF16


@pytest.mark.parametrize("ci,co", [(16, 24), (32, 7), (64, 64), (128, 40), (120, 64), (48, 16), (256, 32)])
def test_deconv_stride2_bf16_channel_widths(oc, orc, tree, ci, co):
  """The 2x2x2 stride-2 bf16 deconvolution over all nodes picks its kernel by the number of
  16-channel k-steps of the input (1, 2, 4, 8: columns held in registers; anything else: the
  general form) and stores the eight children of a (parent, channel) pair as one 16-byte piece
  after a swap between the two lanes of the parent: every width against the oracle, odd output
  channel counts included, with and without bias + ReLU."""
  b, dev, host = tree["blob"], tree["dev"], tree["host"]
  rng = np.random.default_rng(100 + ci + co)
  d = 4
  hin = int(b.nnum_nempty[d])
  x = T(rng.standard_normal((ci, hin)).astype(np.float32)).bfloat16()
  w = T((rng.standard_normal((ci, co * 8)) * 0.1).astype(np.float32)).bfloat16()
  bias = rng.standard_normal(co).astype(np.float32)
  exp = orc.octree_deconv(x.float().numpy(), w.float().numpy(), host, d, co, [2, 2, 2], 2, False)
  got = oc.nn.octree_deconv(x.cuda().view(1, ci, hin, 1), w.cuda(), dev, d, co, [2, 2, 2], 2, False)
  assert relerr(got.float().cpu().numpy().reshape(exp.shape), exp) < TOL_BF16
  gotf = oc.nn.octree_conv_fused(x.cuda().view(1, ci, hin, 1), w.cuda(), T(bias).cuda(), True, dev, d, co, [2, 2, 2], 2,
                                 False, deconv=True)
  assert relerr(gotf.float().cpu().numpy().reshape(exp.shape), np.maximum(exp + bias[:, None], 0)) < TOL_BF16


def test_bf16_register_kernel_small_levels(oc, orc, tree):
  """The bf16 3x3x3 stride-1 kernel for large levels (operands straight into registers, 32
  sibling groups x 8 siblings per wavefront), forced onto small levels whose group counts are
  no multiple of its tile: against the oracle (2e-2), and bit for bit against the LDS kernel
  that serves these sizes by default (same products, same order).  Conv and deconv, ragged
  channel counts, more than one pass over the output channels, fused bias + ReLU."""
  b, dev, host = tree["blob"], tree["dev"], tree["host"]
  L = oc.lib.get()
  rng = np.random.default_rng(11)
  try:
    for d, ci, co in ((5, 3, 32), (5, 20, 70), (4, 64, 64), (6, 16, 130), (3, 40, 8), (6, 64, 64)):
      H = int(b.nnum[d])
      x = rng.standard_normal((ci, H)).astype(np.float32)
      w = (rng.standard_normal((co, ci * 27)) * 0.1).astype(np.float32)
      wd = (rng.standard_normal((ci, co * 27)) * 0.1).astype(np.float32)
      bias = rng.standard_normal(co).astype(np.float32)
      xt = T(x).cuda().view(1, ci, H, 1).bfloat16()
      res = {}
      for name, thr in (("lds", 1 << 30), ("reg", -1)):
        L.ocnn_conv_bf16_tile_threshold(thr)
        res[name] = (oc.nn.octree_conv(xt, T(w).cuda().bfloat16(), dev, d, co, [3, 3, 3], 1, False),
                     oc.nn.octree_deconv(xt, T(wd).cuda().bfloat16(), dev, d, co, [3, 3, 3], 1, False),
                     oc.nn.octree_conv_fused(xt, T(w).cuda().bfloat16(), T(bias).cuda(), True, dev, d, co,
                                             [3, 3, 3], 1, False))
      for got_l, got_r in zip(res["lds"], res["reg"]):
        assert torch.equal(got_l.view(torch.int16), got_r.view(torch.int16)), (d, ci, co)
      exp = orc.octree_conv(x, w, host, d, co, [3, 3, 3], 1, False)
      assert relerr(res["reg"][0].float().cpu().numpy().reshape(exp.shape), exp) < TOL_BF16
      expd = orc.octree_deconv(x, wd, host, d, co, [3, 3, 3], 1, False)
      assert relerr(res["reg"][1].float().cpu().numpy().reshape(expd.shape), expd) < TOL_BF16
      expf = np.maximum(exp + bias[:, None], 0)
      assert relerr(res["reg"][2].float().cpu().numpy().reshape(expf.shape), expf) < TOL_BF16
  finally:
    L.ocnn_conv_bf16_tile_threshold(0)


def test_conv_wide_channels(oc, orc, tree):
  """Channel counts of the benchmark stacks, incl. more than one pass over the output tiles."""
  b, dev, host = tree["blob"], tree["dev"], tree["host"]
  rng = np.random.default_rng(4)
  for d, ci, co in ((4, 64, 64), (4, 128, 256), (3, 256, 32), (4, 64, 100), (4, 1, 1)):
    H = int(b.nnum[d])
    x = rng.standard_normal((ci, H)).astype(np.float32)
    w = (rng.standard_normal((co, ci * 27)) * 0.02).astype(np.float32)
    exp = orc.octree_conv(x, w, host, d, co, [3, 3, 3], 1)
    got = oc.nn.octree_conv(T(x).cuda().view(1, ci, H, 1), T(w).cuda(), dev, d, co, [3, 3, 3], 1, False)
    assert relerr(got.cpu().numpy().reshape(exp.shape), exp) < TOL_F32, (d, ci, co)
    got16 = oc.nn.octree_conv(T(x).cuda().view(1, ci, H, 1).bfloat16(), T(w).cuda().bfloat16(), dev, d, co,
                              [3, 3, 3], 1, False)
    assert relerr(got16.float().cpu().numpy().reshape(exp.shape), exp) < TOL_BF16, (d, ci, co)


def test_conv_wide_channels_nonempty(oc, orc, tree):
  """The row kernels with whole blocks of 128 output channels (four row tiles a pass, 32-channel
  stages in bf16), input channel counts that leave a partial last stage, more than one pass, and
  the stride-2 shapes of the U-Net trunk, over the non-empty nodes."""
  b, dev, host = tree["blob"], tree["dev"], tree["host"]
  rng = np.random.default_rng(6)
  for d, ci, co, ks, stride in ((5, 64, 128, [3, 3, 3], 1), (4, 48, 256, [3, 3, 3], 1), (4, 80, 128, [3, 3, 3], 1),
                                (5, 128, 384, [3, 1, 1], 1), (5, 64, 128, [2, 2, 2], 2), (4, 256, 128, [3, 3, 3], 1)):
    K = ks[0] * ks[1] * ks[2]
    hin = int(b.nnum_nempty[d])
    x = rng.standard_normal((ci, hin)).astype(np.float32)
    w = (rng.standard_normal((co, ci * K)) * 0.02).astype(np.float32)
    exp = orc.octree_conv(x, w, host, d, co, ks, stride, True)
    xt, wt = T(x).cuda().view(1, ci, hin, 1), T(w).cuda()
    got = oc.nn.octree_conv(xt, wt, dev, d, co, ks, stride, True)
    assert relerr(got.cpu().numpy().reshape(exp.shape), exp) < TOL_F32, (d, ci, co, ks)
    got16 = oc.nn.octree_conv(xt.bfloat16(), wt.bfloat16(), dev, d, co, ks, stride, True)
    assert relerr(got16.float().cpu().numpy().reshape(exp.shape), exp) < TOL_BF16, (d, ci, co, ks)
  # deconvolution over the non-empty nodes with 128 output channels
  d, ci, co = 4, 64, 128
  hin = int(b.nnum_nempty[d])
  x = rng.standard_normal((ci, hin)).astype(np.float32)
  w = (rng.standard_normal((ci, co * 8)) * 0.05).astype(np.float32)
  exp = orc.octree_deconv(x, w, host, d, co, [2, 2, 2], 2, True)
  got16 = oc.nn.octree_deconv(T(x).cuda().view(1, ci, hin, 1).bfloat16(), T(w).cuda().bfloat16(), dev, d, co,
                              [2, 2, 2], 2, True)
  assert relerr(got16.float().cpu().numpy().reshape(exp.shape), exp) < TOL_BF16


def test_conv_on_reference_sample_batch(oc, orc, tree):
  """The shapes of pytorch/test/test_octree_conv.py: depth 4, 3 -> 5 channels."""
  sb, sdev, shost = tree["sblob"], tree["sdev"], tree["shost"]
  rng = np.random.default_rng(5)
  d = 4
  H = int(sb.nnum[d])
  x = rng.uniform(-1, 1, (3, H)).astype(np.float32)
  for ks in ([3, 3, 3], [2, 2, 2], [3, 1, 1], [3, 3, 1], [1, 1, 1]):
    for stride in (1, 2):
      K = ks[0] * ks[1] * ks[2]
      w = rng.uniform(-0.5, 0.5, (5, 3 * K)).astype(np.float32)
      conv = oc.OctreeConv(d, 3, 5, ks, stride).cuda()
      fast = oc.OctreeConvFast(d, 3, 5, ks, stride).cuda()
      with torch.no_grad():
        conv.weights.copy_(T(w))
        fast.weights.copy_(T(w))
      xt = T(x).cuda().view(1, 3, H, 1)
      y1, y2 = conv(xt, sdev), fast(xt, sdev)
      assert y1.shape == y2.shape
      assert torch.allclose(y1, y2, atol=1e-5)
      exp = orc.octree_conv(x, w, shost, d, 5, ks, stride)
      if stride == 2:
        exp = orc.pad(exp, sb.prop("child", d - 1))
      assert relerr(y1.detach().cpu().numpy().reshape(exp.shape), exp) < TOL_F32
      # gradients of the fused operator == gradients of octree2col + mm (the reference's own
      # comparison, pytorch/test/test_octree_conv.py:55-72)
      want_x = True
      xg1 = xt.clone().requires_grad_(want_x)
      xg2 = xt.clone().requires_grad_(want_x)
      gy = torch.randn_like(y1)
      conv(xg1, sdev).backward(gy)
      fast(xg2, sdev).backward(gy)
      if want_x:
        assert torch.allclose(xg1.grad, xg2.grad, atol=1e-5)
      assert torch.allclose(conv.weights.grad, fast.weights.grad, atol=1e-4)
      # nempty identity of the reference test: mask -> conv -> select
      mask3 = T(sb.prop("child", d) >= 0).cuda()
      d_out = d if stride == 1 else d - 1
      mask4 = T(sb.prop("child", d_out) >= 0).cuda()
      conv_ne = oc.OctreeConv(d, 3, 5, ks, stride, True).cuda()
      with torch.no_grad():
        conv_ne.weights.copy_(T(w))
      y3 = conv_ne(xt[:, :, mask3], sdev)
      y4 = conv(xt * mask3.view(1, 1, -1, 1).float(), sdev)[:, :, mask4]
      assert torch.allclose(y3, y4, atol=1e-5)


def test_deconv_layers(oc, orc, tree):
  sb, sdev, shost = tree["sblob"], tree["sdev"], tree["shost"]
  rng = np.random.default_rng(6)
  for ks, stride in (([3, 3, 3], 1), ([2, 2, 2], 2), ([3, 1, 1], 1)):
    d = 4 if stride == 1 else 3
    H = int(sb.nnum[d])
    K = ks[0] * ks[1] * ks[2]
    x = rng.uniform(-1, 1, (3, H)).astype(np.float32)
    w = rng.uniform(-0.5, 0.5, (3, 5 * K)).astype(np.float32)
    dec = oc.OctreeDeconv(d, 3, 5, ks, stride).cuda()
    fast = oc.OctreeDeconvFast(d, 3, 5, ks, stride).cuda()
    with torch.no_grad():
      dec.weights.copy_(T(w))
      fast.weights.copy_(T(w))
    xt = T(x).cuda().view(1, 3, H, 1)
    y1, y2 = dec(xt, sdev), fast(xt, sdev)
    assert y1.shape == y2.shape and torch.allclose(y1, y2, atol=1e-5)
    xg1 = xt.clone().requires_grad_(True)
    xg2 = xt.clone().requires_grad_(True)
    gy = torch.randn_like(y1)
    dec(xg1, sdev).backward(gy)
    fast(xg2, sdev).backward(gy)
    assert torch.allclose(xg1.grad, xg2.grad, atol=1e-5)
    assert torch.allclose(dec.weights.grad, fast.weights.grad, atol=1e-4)


def test_conv_shape_errors(oc, tree):
  dev, b = tree["dev"], tree["blob"]
  x = torch.zeros(1, 4, int(b.nnum[5]) + 1, 1, device="cuda")
  w = torch.zeros(8, 4 * 27, device="cuda")
  with pytest.raises(oc.lib.OcnnError) as e:
    oc.nn.octree_conv(x, w, dev, 5, 8, [3, 3, 3], 1, False)
  assert e.value.code == -3
  with pytest.raises(oc.lib.OcnnError) as e:
    oc.nn.octree_conv(x, w, dev, 5, 8, [2, 3, 3], 1, False)
  assert e.value.code == -2
  with pytest.raises(oc.lib.OcnnError) as e:
    oc.nn.octree_conv(x, w, dev, 9, 8, [3, 3, 3], 1, False)
  assert e.value.code == -1
  single = oc.nn.points2octree(T(make_points_blob([[0, 0, 0]], [[1, 0, 0]])), 5, 2)
  with pytest.raises(oc.lib.OcnnError) as e:   # no neighbour table without octree_batch
    oc.nn.octree_conv(torch.zeros(1, 4, 8, 1, device="cuda"), w, single, 5, 8, [3, 3, 3], 1, False)
  assert e.value.code == -6


def test_pool_literals(oc, samples):
  """pytorch/test/test_octree_pool.py:10-101 (forward values and masks)."""
  octree = oc.nn.octree_batch([T(samples["octree_1"])] * 2)
  data = np.array([[1.1, 2.2, 3.3, 4.4, 5.5, 6.6, 7.7, 8.8], [8.1, 7.2, 6.3, 5.4, 4.5, 3.6, 2.7, 1.8]], np.float32)
  data = np.concatenate([data, data], axis=1).reshape(1, 2, 16, 1)
  out_gt = np.zeros((2, 16), np.float32)
  out_gt[0, [0, 8]], out_gt[1, [0, 8]] = 8.8, 8.1
  out, mask = oc.OctreeMaxPool(5, return_indices=True)(T(data).cuda(), octree)
  assert np.array_equal(mask.cpu().numpy(), np.array([[[[7], [15]], [[0], [8]]]], np.int32))
  assert np.array_equal(out.cpu().numpy().reshape(2, 16), out_gt)
  # unpool: depth 4 -> 5 with a hand-written mask
  m = T(np.array([[[[1], [9]], [[2], [10]]]], np.int32)).cuda()
  un = oc.OctreeMaxUnpool(4)(T(data).cuda(), m, octree)
  un_gt = np.zeros((2, 16), np.float32)
  un_gt[0, [1, 9]], un_gt[1, [2, 10]] = 1.1, 8.1
  assert np.array_equal(un.cpu().numpy().reshape(2, 16), un_gt)
  avg_in = np.array([[8.0, 2.2, 3.3, 4.4, 5.5, 6.6, 7.6, 0.8], [12.0, 7.0, 6.0, 5.0, 4.0, 3.0, 3.0, 8.0]], np.float32)
  avg_in = np.concatenate([avg_in, avg_in], axis=1).reshape(1, 2, 16, 1)
  avg = oc.OctreeAvgPool(5)(T(avg_in).cuda(), octree).cpu().numpy().reshape(2, 16)
  avg_gt = np.zeros((2, 16), np.float32)
  avg_gt[0, [0, 8]], avg_gt[1, [0, 8]] = 4.8, 6.0
  assert np.allclose(avg, avg_gt)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_pool_pad_vs_oracle(oc, orc, tree, dtype):
  b, dev = tree["blob"], tree["dev"]
  d = 6
  H = int(b.nnum[d])
  rng = np.random.default_rng(7)
  x = rng.integers(-4, 4, (9, H)).astype(np.float32) / 2   # many ties, exactly representable in bf16
  xt = T(x).cuda().view(1, 9, H, 1).to(dtype)
  top, mask = oc.nn.octree_max_pool(xt, dev, d)
  et, em = orc.max_pool(x)
  assert np.array_equal(top.float().cpu().numpy().reshape(et.shape), et)
  assert np.array_equal(mask.cpu().numpy().reshape(em.shape), em)
  un = oc.nn.octree_max_unpool(top, mask, dev, d)
  assert np.array_equal(un.float().cpu().numpy().reshape(9, H), orc.max_unpool(et, em))
  mp = oc.nn.octree_mask_pool(xt, mask, dev, d)
  assert np.array_equal(mp.float().cpu().numpy().reshape(et.shape), orc.mask_pool(x, em))
  # a mask that points outside its own sibling group (never produced by max_pool)
  foreign = em.copy()
  foreign[:, ::5] = (foreign[:, ::5] + 8 * 3) % H
  un2 = oc.nn.octree_max_unpool(top, T(foreign).cuda().view(1, 9, -1, 1), dev, d)
  got, exp = un2.float().cpu().numpy().reshape(9, H), orc.max_unpool(et, foreign)
  clash = np.zeros((9, H), bool)   # positions hit twice have no defined winner in the reference either
  for c in range(9):
    idx, cnt = np.unique(foreign[c], return_counts=True)
    clash[c, idx[cnt > 1]] = True
  assert np.array_equal(got[~clash], exp[~clash])
  child = b.prop("child", d - 1)
  pd = oc.nn.octree_pad(top, dev, d - 1, 1.5)
  assert np.array_equal(pd.float().cpu().numpy().reshape(9, -1), orc.pad(et, child, 1.5))
  dp = oc.nn.octree_depad(pd, dev, d - 1)
  assert np.array_equal(dp.float().cpu().numpy().reshape(et.shape), et)
  with pytest.raises(oc.lib.OcnnError) as e:
    oc.nn.octree_pad(xt, dev, d - 1)
  assert e.value.code == -3


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_pad_any_labels(oc, orc, dtype):
  """pad_forward / pad_backward through the C-ABI (octree_nn.cpp:163-185) with label arrays that are
  not the ascending ranks an octree has: shuffled, with gaps, out of range, a wide spread inside one
  tile, several tiles, unaligned rows; rows of X that no label names keep their old content."""
  import ctypes as C
  rng = np.random.default_rng(5)
  P = lambda t, off=0: C.c_void_p(t.data_ptr() + off)
  st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
  dt = 0 if dtype == torch.float32 else 1
  Cc = 11
  cases = []
  Hy, Hx = 5000, 1300
  lab = np.full(Hy, -1, np.int32)
  pos = np.sort(rng.choice(Hy, Hx, replace=False))
  lab[pos] = np.arange(Hx)                                   # an octree's kind of labels
  cases.append(("ranks", lab.copy(), Hx))
  lab2 = lab.copy(); lab2[pos] = rng.permutation(Hx)          # distinct, any order
  cases.append(("shuffled", lab2, Hx))
  lab3 = lab.copy(); lab3[pos[::7]] = -1; lab3[pos[3::11]] = Hx + 5   # gaps and rows outside X
  cases.append(("gaps", lab3, Hx))
  lab4 = np.full(Hy, -1, np.int32); lab4[pos] = np.arange(Hx) * 3     # wide spread
  cases.append(("spread", lab4, 3 * Hx))
  for name, l, hx in cases:
    x = (rng.integers(-8, 8, (Cc, hx)) / 2).astype(np.float32)
    y = (rng.integers(-8, 8, (Cc, Hy)) / 2).astype(np.float32)
    l_d = T(l).cuda()
    # forward, into a buffer that starts 3 elements past a line boundary
    ybuf = torch.full((Cc * Hy + 8,), 9.0, device="cuda", dtype=dtype)
    x_d = T(x).cuda().to(dtype)
    es = ybuf.element_size()
    oc.lib.call("ocnn_pad_forward", P(ybuf, 3 * es), Hy, Cc, P(x_d), hx, P(l_d), C.c_float(1.5), dt, st)
    exp = np.where((l >= 0) & (l < hx), x[:, np.clip(l, 0, hx - 1)], np.float32(1.5))
    got = ybuf.float().cpu().numpy()
    assert np.array_equal(got[3:3 + Cc * Hy].reshape(Cc, Hy), exp), name
    assert np.all(got[:3] == 9.0) and np.all(got[3 + Cc * Hy:] == 9.0), name
    # backward: rows of X named by a label take the row of Y, the others stay
    xbuf = torch.full((Cc * hx + 8,), 7.0, device="cuda", dtype=dtype)
    y_d = T(y).cuda().to(dtype)
    oc.lib.call("ocnn_pad_backward", P(xbuf, 5 * es), hx, Cc, P(y_d), Hy, P(l_d), dt, st)
    expx = np.full((Cc, hx), 7.0, np.float32)
    ok = (l >= 0) & (l < hx)
    expx[:, l[ok]] = y[:, ok]
    gotx = xbuf.float().cpu().numpy()
    assert np.array_equal(gotx[5:5 + Cc * hx].reshape(Cc, hx), expx), name
    assert np.all(gotx[:5] == 7.0) and np.all(gotx[5 + Cc * hx:] == 7.0), name


def test_full_size_properties(oc, synthetic):
  """Size-independent properties on the depth-9 scene of BASELINE config 4: linearity of
  the convolution, unpool/mask-pool round trip, depad(pad(x)) == x."""
  p, n, f = synthetic.room_cloud(250000, 3)
  octree = oc.nn.points2octree_batch([T(make_points_blob(p, n, f)).cuda()], 9, 2)
  info = oc.nn.octree_info(octree)
  H = info.nnum(9)
  g = torch.Generator().manual_seed(0)
  C = 64
  x = torch.randn(1, C, H, 1, generator=g).cuda()
  y = torch.randn(1, C, H, 1, generator=g).cuda()
  w = (torch.randn(C, C * 27, generator=g) * 0.02).cuda()
  conv = lambda t: oc.nn.octree_conv(t, w, octree, 9, C, [3, 3, 3], 1, False)
  lhs = conv(2.0 * x - 3.0 * y)
  rhs = 2.0 * conv(x) - 3.0 * conv(y)
  assert float((lhs - rhs).abs().max() / rhs.abs().max()) < 1e-4
  top, mask = oc.nn.octree_max_pool(x, octree, 9)
  un = oc.nn.octree_max_unpool(top, mask, octree, 9)
  assert torch.equal(oc.nn.octree_mask_pool(un, mask, octree, 9), top)
  assert int((un != 0).sum()) <= top.numel()
  assert torch.equal(un.view(C, -1, 8).amax(2), torch.clamp(top.view(C, -1), min=0) * (top.view(C, -1) > 0)
                     + torch.clamp(top.view(C, -1), max=0) * 0)
  pd = oc.nn.octree_pad(top, octree, 8)
  assert torch.equal(oc.nn.octree_depad(pd, octree, 8), top)
  # stride-2 conv then deconv keep the documented heights
  w2 = (torch.randn(C, C * 8, generator=g) * 0.02).cuda()
  down = oc.nn.octree_conv(x, w2, octree, 9, C, [2, 2, 2], 2, False)
  assert down.shape[2] == info.nnum_nempty(8)
  up = oc.nn.octree_deconv(down, w2, octree, 8, C, [2, 2, 2], 2, False)
  assert up.shape[2] == H


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_pad_with_a_value_per_channel(oc, orc, tree, dtype):
  """ocnn_pad_forward_fill: the oracle's pad where a node has a source row, the channel's own value
  (rounded to the tensor's type) where it has none."""
  b, dev = tree["blob"], tree["dev"]
  rng = np.random.default_rng(17)
  for d, Cc in ((5, 7), (4, 64), (3, 130)):
    child = b.prop("child", d)
    Hne = int(b.nnum_nempty[d])
    x = T(rng.standard_normal((Cc, Hne)).astype(np.float32)).to(dtype)
    fill = T(rng.standard_normal(Cc).astype(np.float32))
    got = oc.nn.octree_pad_fill(x.cuda().view(1, Cc, Hne, 1), dev, d, fill.cuda())
    exp = T(orc.pad(x.float().numpy(), child)).to(dtype)
    exp[:, child < 0] = fill.to(dtype)[:, None]
    assert got.dtype == dtype and torch.equal(got.cpu().view(Cc, -1), exp), (d, Cc)


@pytest.mark.parametrize("cin,hidden,nout", [(3, 32, 2), (32, 32, 2), (64, 32, 4), (130, 20, 5), (256, 32, 8), (5, 1, 1)])
def test_two_1x1x1_convolutions_in_one_pass(oc, orc, tree, cin, hidden, nout):
  """The prediction head of pytorch/ocnn/ounet.py:46-49 (1x1x1 conv -> ReLU -> 1x1x1 conv with bias)
  as one kernel against the oracle's two convolutions, 1e-4 of the largest magnitude; the labels
  are the argmax of the kernel's own logits (ounet.py:117-118), and the operator-by-operator
  path gives the same within the tolerance.  Levels of 64 to 5 000+ nodes (partial tiles); heights
  of 1, 63 and 257 columns against the matrix product in float64, which is what a 1x1x1
  convolution is."""
  F = oc.nn
  rng = np.random.default_rng(cin * 100 + hidden * 10 + nout)
  host, dev, blob = tree["host"], tree["dev"], tree["blob"]
  for d in (2, 5, 6):
    H = int(blob.nnum[d])
    x = rng.standard_normal((cin, H)).astype(np.float32)
    w1 = (rng.standard_normal((hidden, cin)) / np.sqrt(cin)).astype(np.float32)
    w2 = (rng.standard_normal((nout, hidden)) / np.sqrt(hidden)).astype(np.float32)
    b1 = (rng.standard_normal(hidden) * 0.3).astype(np.float32)
    b2 = (rng.standard_normal(nout) * 0.3).astype(np.float32)
    hid = np.maximum(orc.octree_conv(x, w1, host, d, hidden, [1, 1, 1], 1, False) + b1[:, None], 0)
    exp = orc.octree_conv(hid, w2, host, d, nout, [1, 1, 1], 1, False) + b2[:, None]
    xd = T(x).cuda().view(1, cin, H, 1)
    out, label = F.conv1x1_pair(xd, T(w1).cuda(), T(b1).cuda(), T(w2).cuda(), T(b2).cuda(), return_label=True)
    got = out.cpu().numpy().reshape(nout, H)
    assert np.abs(got - exp).max() <= 1e-4 * max(np.abs(exp).max(), 1.0), (d, cin, hidden, nout)
    assert np.array_equal(label.cpu().numpy(), got.argmax(0).astype(np.int32)), (d, cin, hidden, nout)
    # no biases, no ReLU, no labels
    plain = F.conv1x1_pair(xd, T(w1).cuda(), None, T(w2).cuda(), None, relu=False)
    e2 = orc.octree_conv(orc.octree_conv(x, w1, host, d, hidden, [1, 1, 1], 1, False), w2, host, d, nout, [1, 1, 1], 1, False)
    assert np.abs(plain.cpu().numpy().reshape(nout, H) - e2).max() <= 1e-4 * max(np.abs(e2).max(), 1.0)
    # the head of the decoder stack takes this kernel; operator by operator it is two convolutions
    two = oc.stacks.conv_bn_relu(oc.stacks.conv_bn_relu(xd, T(w1).cuda(), T(b1).cuda(), dev, d, hidden, (1, 1, 1)),
                                 T(w2).cuda(), T(b2).cuda(), dev, d, nout, (1, 1, 1), relu=False)
    assert np.abs(two.cpu().numpy().reshape(nout, H) - exp).max() <= 1e-4 * max(np.abs(exp).max(), 1.0)
  for H in (1, 63, 257):
    x = rng.standard_normal((cin, H)).astype(np.float32)
    exp = w2.astype(np.float64) @ np.maximum(w1.astype(np.float64) @ x + b1[:, None], 0) + b2[:, None]
    out, label = F.conv1x1_pair(T(x).cuda().view(1, cin, H, 1), T(w1).cuda(), T(b1).cuda(), T(w2).cuda(), T(b2).cuda(),
                                return_label=True)
    got = out.cpu().numpy().reshape(nout, H)
    assert np.abs(got - exp).max() <= 1e-4 * max(np.abs(exp).max(), 1.0), (H, cin, hidden, nout)
    assert np.array_equal(label.cpu().numpy(), got.argmax(0).astype(np.int32))
  with pytest.raises(oc.nn.OcnnError):
    F.conv1x1_pair(xd, torch.zeros(33, cin).cuda(), None, torch.zeros(2, 33).cuda(), None)
  with pytest.raises(oc.nn.OcnnError):
    F.conv1x1_pair(xd, torch.zeros(8, cin).cuda(), None, torch.zeros(9, 8).cuda(), None)


def test_fp32_nonempty_kernel_forms(oc, orc, tree):
  """The fp32 kernel over the non-empty nodes in its two forms (weights of every tap staged through
  LDS; weights read per live tap by each wavefront, the choice on sparse levels): the same sums in
  the same order, so equal bits, and the oracle's result within 1e-4; convolution, deconvolution
  and both gradients; channel counts with partial stages and one or more passes; tap sets of 27, 9
  and 3; levels from a few hundred to thousands of rows (workgroups of one to four wavefronts)."""
  b, dev, host = tree["blob"], tree["dev"], tree["host"]
  L = oc.lib.get()
  rng = np.random.default_rng(16)
  try:
    for d, ci, co, ks in ((6, 3, 32, [3, 3, 3]), (6, 64, 64, [3, 3, 3]), (5, 20, 70, [3, 3, 3]), (5, 40, 32, [3, 3, 1]),
                          (4, 72, 130, [3, 1, 1]), (3, 128, 64, [3, 3, 3]), (6, 33, 40, [1, 3, 3])):
      K = ks[0] * ks[1] * ks[2]
      hin = int(b.nnum_nempty[d])
      x = rng.standard_normal((ci, hin)).astype(np.float32)
      w = (rng.standard_normal((co, ci * K)) / np.sqrt(ci * K)).astype(np.float32)
      wd = (rng.standard_normal((ci, co * K)) / np.sqrt(ci * K)).astype(np.float32)
      g = rng.standard_normal((co, hin)).astype(np.float32)
      xt, wt, wdt, gt = T(x).cuda().view(1, ci, hin, 1), T(w).cuda(), T(wd).cuda(), T(g).cuda().view(1, co, hin, 1)
      got = {}
      for form in (0, 2):
        L.ocnn_conv_rows_direct(form)
        got[form] = (oc.nn.octree_conv(xt, wt, dev, d, co, ks, 1, True), oc.nn.octree_deconv(xt, wdt, dev, d, co, ks, 1, True),
                     *oc.nn.octree_conv_grad(xt, wt, dev, gt, d, co, ks, 1, True))
      for i, name in enumerate(("conv", "deconv", "data gradient", "weight gradient")):
        assert torch.equal(got[0][i], got[2][i]), (name, d, ci, co, ks)
      exp = orc.octree_conv(x, w, host, d, co, ks, 1, True)
      assert relerr(got[2][0].cpu().numpy().reshape(exp.shape), exp) < TOL_F32, (d, ci, co, ks)
      exp = orc.octree_deconv(x, wd, host, d, co, ks, 1, True)
      assert relerr(got[2][1].cpu().numpy().reshape(exp.shape), exp) < TOL_F32, (d, ci, co, ks)
      egd, egw = orc.octree_conv_grad(x, w, g, host, d, co, ks, 1, True)
      assert relerr(got[2][2].cpu().numpy().reshape(egd.shape), egd) < TOL_F32, (d, ci, co, ks)
      assert relerr(got[2][3].cpu().numpy().reshape(egw.shape), egw) < TOL_F32, (d, ci, co, ks)
  finally:
    L.ocnn_conv_rows_direct(1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_nonempty_convolutions_with_a_kept_table_of_sources(oc, orc, tree, dtype):
  """Over the non-empty nodes the Python mirror keeps the table of source rows with the octree and
  hands it to ocnn_octree_conv_fused_sources; the plain entry points look the rows up in the kernel.
  Equal bits (conv and deconv, 3x3x3 / 3x1x1 stride 1 and 2x2x2 stride 2), the oracle's result within
  the tolerance, one table per (depth, shape, direction) shared by the layers of a depth, and a new
  one after the octree was written to."""
  import ctypes as C
  F = oc.nn
  b, host = tree["blob"], tree["host"]
  dev = T(host).cuda()
  info = F.octree_info(dev)
  P = lambda t: C.c_void_p(t.data_ptr())
  rng = np.random.default_rng(23)
  tol = TOL_F32 if dtype == torch.float32 else TOL_BF16
  code = 0 if dtype == torch.float32 else 1
  for d, ci, co, ks, stride in ((5, 24, 40, [3, 3, 3], 1), (6, 16, 16, [3, 1, 1], 1), (5, 32, 64, [2, 2, 2], 2)):
    K = ks[0] * ks[1] * ks[2]
    for deconv in (False, True):
      hin = int(b.nnum_nempty[d])
      x = T(rng.standard_normal((ci, hin)).astype(np.float32)).to(dtype).cuda().view(1, ci, hin, 1)
      shape = (ci, co * K) if deconv else (co, ci * K)
      w = T((rng.standard_normal(shape) / np.sqrt(ci * K)).astype(np.float32)).to(dtype).cuda()
      got = (F.octree_deconv if deconv else F.octree_conv)(x, w, dev, d, co, ks, stride, True)
      again = (F.octree_deconv if deconv else F.octree_conv)(x, w, dev, d, co, ks, stride, True)
      assert torch.equal(got, again)
      # the plain entry point, no table
      ksc = (C.c_int * 3)(*ks)
      top_h, need_h, wsb = C.c_int(), C.c_int(), C.c_size_t()
      oc.lib.call("ocnn_conv_shape", info.p, d, ci, co, ksc, stride, 1, int(deconv), code, C.byref(top_h), C.byref(need_h), C.byref(wsb))
      ws = torch.empty(wsb.value + 256, dtype=torch.uint8, device="cuda")
      base = (ws.data_ptr() + 255) & ~255
      plain = torch.empty_like(got)
      oc.lib.call("ocnn_octree_deconv" if deconv else "ocnn_octree_conv", P(plain), P(x), ci, hin, P(w), P(dev), info.p, d, co,
                  ksc, stride, 1, code, C.c_void_p(base), C.c_size_t(wsb.value), None)
      torch.cuda.synchronize()
      assert torch.equal(got, plain), (d, ks, stride, deconv)
      fn = orc.octree_deconv if deconv else orc.octree_conv
      exp = fn(x.float().cpu().numpy().reshape(ci, hin), w.float().cpu().numpy(), host, d, co, ks, stride, True)
      assert relerr(got.float().cpu().numpy().reshape(exp.shape), exp) < tol, (d, ks, stride, deconv)
  tables = dev.__dict__["_ocnn_sources"]
  kept = [k for k in tables if k != "version"]
  assert (5, (3, 3, 3), 1, False) in kept and (5, (3, 3, 3), 1, True) in kept
  if dtype == torch.bfloat16:
    assert tables[(5, (2, 2, 2), 2, False)] is not None
  # a write through torch bumps the version: the tables are made again
  first = tables[(5, (3, 3, 3), 1, False)]
  dev[-1] = dev[-1]
  x = T(rng.standard_normal((8, int(b.nnum_nempty[5]))).astype(np.float32)).to(dtype).cuda().view(1, 8, -1, 1)
  w = T((rng.standard_normal((8, 8 * 27)) * 0.1).astype(np.float32)).to(dtype).cuda()
  F.octree_conv(x, w, dev, 5, 8, [3, 3, 3], 1, True)
  assert dev.__dict__["_ocnn_sources"][(5, (3, 3, 3), 1, False)] is not first
