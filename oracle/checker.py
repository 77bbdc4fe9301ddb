"""TEST INFRASTRUCTURE -- ctypes front end of the two CPU checkers.

`Checker("orc")` drives the C restatement (oracle/libocnn_oracle.so);
`Checker("ref")` drives the real reference compiled from its own sources
(oracle/_ref/libocnn_ref.so, present only where oracle/Makefile could build it
or where the prebuilt file travelled).  Both export the same entry points, so
every test can be run against either.

Also holds `OctreeBlob`, an independent numpy reader of the serialized octree
wire format (octree/octree/octree_info.h:96-118, octree_info.cpp:157-167,
254-268) used by the tests to look inside blobs.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module; the shipped package never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORC_SO = os.path.join(HERE, "libocnn_oracle.so")
REF_SO = os.path.join(HERE, "_ref", "libocnn_ref.so")

PROP = {"key": 1, "child": 2, "neigh": 4, "feature": 8, "label": 16, "split": 32}
_PROP_DTYPE = {1: np.uint64, 2: np.int32, 4: np.int32, 8: np.float32,
               16: np.float32, 32: np.float32}


def build_oracle():
  subprocess.check_call(["make", "-s", "-C", HERE, "oracle"])


def have_ref():
  return os.path.exists(REF_SO)


def _p(a):
  return a.ctypes.data_as(C.c_void_p)


def _f32(a):
  return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
  return np.ascontiguousarray(a, dtype=np.int32)


def _u64(a):
  return np.ascontiguousarray(a, dtype=np.uint64)


class OctreeBlob:
  """numpy view over a serialized octree (host bytes)."""

  def __init__(self, blob):
    self.b = np.ascontiguousarray(np.asarray(blob, dtype=np.uint8))
    h = self.b[:716]
    i32 = lambda off, n=1: h[off:off + 4 * n].view(np.int32).copy()
    self.magic = bytes(h[:16]).split(b"\0")[0].decode()
    self.batch_size = int(i32(16)[0])
    self.depth = int(i32(20)[0])
    self.full_layer = int(i32(24)[0])
    self.adp_layer = int(i32(28)[0])
    self.is_adaptive = bool(h[32])
    self.th_dist = float(h[36:40].view(np.float32)[0])
    self.th_norm = float(h[40:44].view(np.float32)[0])
    self.key2xyz = bool(h[44])
    self.has_node_dis = bool(h[45])
    self.nnum = i32(48, 16)
    self.nnum_cum = i32(112, 16)
    self.nnum_nempty = i32(176, 16)
    self.content_flags = int(i32(240)[0])
    self.channels = i32(244, 16)
    self.locations = i32(308, 16)
    self.bbmin = h[372:384].view(np.float32).copy()
    self.bbmax = h[384:396].view(np.float32).copy()
    self.extrapolate = bool(h[396])
    self.save_pts = bool(h[397])
    self.ptr_dis = i32(652, 16)
    self.size = int(self.ptr_dis[6])

  def has(self, name):
    return (self.content_flags & PROP[name]) != 0

  def channel(self, name):
    p = PROP[name]
    return int(self.channels[p.bit_length() - 1]) if self.has(name) else 0

  def location(self, name):
    p = PROP[name]
    return int(self.locations[p.bit_length() - 1]) if self.has(name) else 0

  def prop(self, name, depth):
    """array of one property at one depth: [channel, nnum(depth)] (neigh: [nnum/8, 64])."""
    p = PROP[name]
    if not self.has(name):
      return None
    idx = p.bit_length() - 1
    ch = int(self.channels[idx])
    dt = np.dtype(_PROP_DTYPE[p])
    off = int(self.ptr_dis[idx])
    if self.location(name) == -1:
      off += int(self.nnum_cum[depth]) * ch * dt.itemsize
    n = int(self.nnum[depth])
    a = self.b[off:off + n * ch * dt.itemsize].view(dt)
    if name == "neigh":
      return a.reshape(-1, 64)
    if ch == 1:
      return a
    return a.reshape(ch, n)


class Checker:
  def __init__(self, prefix="orc"):
    self.prefix = prefix
    if prefix == "orc":
      if not os.path.exists(ORC_SO):
        build_oracle()
      self.lib = C.CDLL(ORC_SO)
    elif prefix == "ref":
      self.lib = C.CDLL(REF_SO)
    else:
      raise ValueError(prefix)
    for n in ("fetch", "points2octree", "octree_batch", "octree_sample",
              "octree_new", "octree_grow", "octree_update", "octree_set_property",
              "normalize_points", "transform_points", "clip_points", "upgrade_key64", "octree_scan", "octree_dropout"):
      f = getattr(self.lib, prefix + "_" + n, None)
      if f is not None:
        f.restype = C.c_int64

  def fn(self, name):
    return getattr(self.lib, self.prefix + "_" + name)

  def _fetch(self, sz):
    if sz < 0:
      raise RuntimeError("%s call failed with code %d" % (self.prefix, sz))
    out = np.zeros(sz, np.uint8)
    got = self.fn("fetch")(_p(out), C.c_int64(sz))
    assert got == sz
    return out

  # ---- blob producers ------------------------------------------------------
  def points2octree(self, points_blob, depth, full_depth=2, node_dis=False,
                    node_feature=False, split_label=False, adaptive=False,
                    adp_depth=4, th_normal=0.1, th_distance=2.0,
                    extrapolate=False, save_pts=False, key2xyz=False,
                    bbmin=None, bbmax=None):
    pb = np.ascontiguousarray(points_blob, dtype=np.uint8)
    bmin = _f32(bbmin) if bbmin is not None else None
    bmax = _f32(bbmax) if bbmax is not None else None
    sz = self.fn("points2octree")(
        _p(pb), int(depth), int(full_depth), int(node_dis), int(node_feature),
        int(split_label), int(adaptive), int(adp_depth), C.c_float(th_normal),
        C.c_float(th_distance), int(extrapolate), int(save_pts), int(key2xyz),
        _p(bmin) if bmin is not None else None,
        _p(bmax) if bmax is not None else None)
    return self._fetch(sz)

  # ---- point-cloud transforms (pytorch/cpp/transform_points.cpp) --------------------------
  def bounding_sphere(self, points_blob, method="sphere"):
    pb = np.ascontiguousarray(points_blob, dtype=np.uint8)
    out = np.zeros(4, np.float32)
    if self.fn("bounding_sphere")(_p(pb), int(method != "sphere"), _p(out)) < 0:
      raise RuntimeError("bounding_sphere failed")
    return out

  def normalize_points(self, points_blob, radius, center):
    pb = np.ascontiguousarray(points_blob, dtype=np.uint8)
    return self._fetch(self.fn("normalize_points")(_p(pb), C.c_int64(pb.size), C.c_float(radius),
                                                   _p(_f32(center))))

  def transform_points(self, points_blob, angle, scale, jitter, offset=0.0, normal_axis=""):
    pb = np.ascontiguousarray(points_blob, dtype=np.uint8)
    return self._fetch(self.fn("transform_points")(
        _p(pb), C.c_int64(pb.size), _p(_f32(angle)), _p(_f32(scale)), _p(_f32(jitter)),
        C.c_float(offset), normal_axis.encode()))

  def clip_points(self, points_blob, bbmin, bbmax):
    pb = np.ascontiguousarray(points_blob, dtype=np.uint8)
    npt = int(pb[16:20].view(np.int32)[0])
    mask = np.zeros(npt, np.int32)
    out = self._fetch(self.fn("clip_points")(_p(pb), C.c_int64(pb.size), _p(_f32(bbmin)), _p(_f32(bbmax)),
                                             _p(mask)))
    return out, mask

  def octree_batch(self, blobs):
    blobs = [np.ascontiguousarray(b, dtype=np.uint8) for b in blobs]
    arr = (C.c_void_p * len(blobs))(*[b.ctypes.data for b in blobs])
    return self._fetch(self.fn("octree_batch")(arr, len(blobs)))

  def octree_scan(self, blob, axis, scale=1.0):
    b = np.ascontiguousarray(blob, dtype=np.uint8)
    ax = np.ascontiguousarray(axis, dtype=np.float32).reshape(-1)
    assert ax.size % 3 == 0
    return self._fetch(self.fn("octree_scan")(_p(b), _p(ax), ax.size // 3, C.c_float(scale)))

  def octree_dropout(self, blob, flags, depth_dropout):
    """The restatement: the flags of level `depth_dropout` are an argument."""
    assert self.prefix == "orc"
    b = np.ascontiguousarray(blob, dtype=np.uint8)
    f = np.ascontiguousarray(flags, dtype=np.uint8)
    assert f.size == OctreeBlob(b).nnum[depth_dropout]
    return self._fetch(self.fn("octree_dropout")(_p(b), _p(f), int(depth_dropout)))

  def octree_dropout_drawn(self, blob, depth_dropout, threshold):
    """The compiled reference: returns its result and the flags it drew."""
    assert self.prefix == "ref"
    b = np.ascontiguousarray(blob, dtype=np.uint8)
    f = np.zeros(int(OctreeBlob(b).nnum[depth_dropout]), np.uint8)
    out = self._fetch(self.fn("octree_dropout")(_p(b), C.c_int64(b.size), int(depth_dropout), C.c_float(threshold),
                                                _p(f), int(f.size)))
    return out, f

  def upgrade_key64(self, blob32):
    b = np.ascontiguousarray(blob32, dtype=np.uint8)
    return self._fetch(self.fn("upgrade_key64")(_p(b), C.c_int64(b.size)))

  def octree_sample(self, name):
    return self._fetch(self.fn("octree_sample")(name.encode()))

  def octree_new(self, batch_size, channel, node_dis=False, adaptive_layer=0):
    return self._fetch(self.fn("octree_new")(batch_size, channel, int(node_dis), adaptive_layer))

  def octree_grow(self, blob, target_depth, full_octree):
    b = np.ascontiguousarray(blob, dtype=np.uint8)
    return self._fetch(self.fn("octree_grow")(_p(b), target_depth, int(full_octree)))

  def octree_update(self, blob, label, depth, split):
    b = np.ascontiguousarray(blob, dtype=np.uint8)
    lab = _i32(label)
    return self._fetch(self.fn("octree_update")(_p(b), _p(lab), lab.size, depth, split))

  def octree_set_property(self, blob, data, depth):
    b = np.ascontiguousarray(blob, dtype=np.uint8)
    d = _f32(data)
    return self._fetch(self.fn("octree_set_property")(_p(b), _p(d), C.c_int64(d.size), depth))

  # ---- tables ----------------------------------------------------------------
  def get_ni(self, kernel_size):
    ks = _i32(kernel_size)
    out = np.zeros(216, np.int32)
    n = self.fn("get_ni")(_p(ks), _p(out))
    assert n > 0
    return out[:n].copy()

  def get_parent(self):
    out = np.zeros(512, np.int32)
    self.fn("get_parent")(_p(out))
    return out

  def get_dis(self):
    out = np.zeros(64, np.int32)
    self.fn("get_dis")(_p(out))
    return out

  # ---- neighbour tables ------------------------------------------------------
  def calc_neigh_full(self, depth, batch):
    out = np.zeros(batch * (8 ** depth) * 8, np.int32)
    self.fn("calc_neigh_full")(_p(out), depth, batch)
    return out

  def calc_neigh_sparse(self, neigh, children, n_child_nodes):
    neigh, children = _i32(neigh), _i32(children)
    out = np.full(n_child_nodes * 8, -1, np.int32)
    self.fn("calc_neigh_sparse")(_p(out), _p(neigh), _p(children), children.size)
    return out

  # ---- octree2col / col2octree ------------------------------------------------
  def octree2col(self, data, kernel_size, stride, neigh, height):
    """data [C, H_in]; height = number of output columns."""
    data = _f32(data)
    ni = self.get_ni(kernel_size)
    K = int(np.prod(kernel_size))
    Cc = data.shape[0]
    col = np.empty((Cc, K, height), np.float32)
    self.fn("octree2col")(_p(col), _p(data), Cc, height, K, stride, _p(_i32(neigh)),
                          _p(ni), height, 0)
    return col

  def col2octree(self, col, kernel_size, stride, neigh, height):
    col = _f32(col)
    ni = self.get_ni(kernel_size)
    Cc, K, hc = col.shape
    assert hc == height
    out = np.empty((Cc, height << (3 * (stride - 1))), np.float32)
    self.fn("col2octree")(_p(col), _p(out), Cc, height, K, stride, _p(_i32(neigh)),
                          _p(ni), height, 0)
    return out

  def octree2colP(self, data, kernel_size, stride, neigh, child, ichild, height):
    data = _f32(data)
    ni = self.get_ni(kernel_size)
    K = int(np.prod(kernel_size))
    Cc, oh = data.shape
    col = np.empty((Cc, K, height), np.float32)
    self.fn("octree2colP")(_p(col), _p(data), Cc, height, oh, K, stride, _p(_i32(neigh)),
                           _p(ni), _p(_i32(child)), _p(_i32(ichild)), height, 0)
    return col

  def col2octreeP(self, col, kernel_size, stride, neigh, child, ichild, height, octree_h):
    col = _f32(col)
    ni = self.get_ni(kernel_size)
    Cc, K, _ = col.shape
    out = np.empty((Cc, octree_h), np.float32)
    self.fn("col2octreeP")(_p(col), _p(out), Cc, height, octree_h, K, stride,
                           _p(_i32(neigh)), _p(ni), _p(_i32(child)), _p(_i32(ichild)),
                           height, 0)
    return out

  # ---- pooling / padding -------------------------------------------------------
  def max_pool(self, btm):
    btm = _f32(btm)
    Cc, H = btm.shape
    top = np.empty((Cc, H // 8), np.float32)
    mask = np.empty((Cc, H // 8), np.int32)
    self.fn("max_pool")(_p(top), H // 8, _p(mask), _p(btm), H, Cc)
    return top, mask

  def max_unpool(self, top, mask):
    top, mask = _f32(top), _i32(mask)
    Cc, th = top.shape
    btm = np.empty((Cc, th * 8), np.float32)
    self.fn("max_unpool")(_p(top), th, _p(mask), _p(btm), th * 8, Cc)
    return btm

  def mask_pool(self, btm, mask):
    btm, mask = _f32(btm), _i32(mask)
    Cc, H = btm.shape
    th = mask.shape[1]
    top = np.empty((Cc, th), np.float32)
    self.fn("mask_pool")(_p(top), th, _p(mask), _p(btm), H, Cc)
    return top

  def pad(self, X, label, dval=0.0):
    X, label = _f32(X), _i32(label)
    Cc, Hx = X.shape
    Y = np.empty((Cc, label.size), np.float32)
    self.fn("pad_forward")(_p(Y), label.size, Cc, _p(X), Hx, _p(label), C.c_float(dval))
    return Y

  def depad(self, Y, label, Hx):
    Y, label = _f32(Y), _i32(label)
    Cc, Hy = Y.shape
    X = np.zeros((Cc, Hx), np.float32)
    self.fn("pad_backward")(_p(X), Hx, Cc, _p(Y), Hy, _p(label))
    return X

  def octree_gather(self, btm, idx):
    btm, idx = _f32(btm), _i32(idx)
    Cc, Hb = btm.shape
    top = np.empty((Cc, idx.size), np.float32)
    self.fn("octree_gather")(_p(top), idx.size, Cc, _p(btm), Hb, _p(idx))
    return top

  def octree_gatherbk(self, top, idx, btm_h):
    top, idx = _f32(top), _i32(idx)
    Cc, Ht = top.shape
    btm = np.empty((Cc, btm_h), np.float32)
    self.fn("octree_gatherbk")(_p(top), Ht, Cc, _p(btm), btm_h, _p(idx))
    return btm

  def octree_mask(self, data, label, mask):
    data, label = _f32(data), _i32(label)
    out = np.empty_like(data)
    self.fn("octree_mask")(_p(out), _p(data), _p(label), label.size, int(mask), data.size)
    return out

  # ---- trilinear stencils ------------------------------------------------------
  def get_bilinear(self):
    t = np.zeros(512, np.int32)
    self.fn("get_bilinear")(_p(t))
    return t

  def bilinear_neigh(self, neigh, child, n_child_nodes):
    neigh, child = _i32(neigh), _i32(child)
    bidx = np.full(n_child_nodes * 8, -7, np.int32)
    self.fn("bilinear_neigh")(_p(bidx), _p(neigh), _p(child), child.size)
    return bidx.reshape(-1, 8)

  def bilinear_xyz(self, xyz1, d0, d1):
    xyz1 = _u64(xyz1)
    xyz0 = np.zeros(xyz1.size * 8, np.uint64)
    fracs = np.zeros(xyz1.size * 3, np.float32)
    self.fn("bilinear_xyz")(_p(xyz0), _p(fracs), d0, _p(xyz1), d1, xyz1.size)
    return xyz0.reshape(-1, 8), fracs.reshape(-1, 3)

  # ---- keys ------------------------------------------------------------------
  def generate_key_child(self, key, child, n_out):
    key, child = _u64(key), _i32(child)
    out = np.zeros(n_out, np.uint64)
    self.fn("generate_key_child")(_p(out), _p(key), _p(child), child.size)
    return out

  def generate_key_full(self, depth, batch):
    out = np.zeros(batch * 8 ** depth, np.uint64)
    self.fn("generate_key_full")(_p(out), depth, batch)
    return out

  def generate_label(self, btm, mask):
    btm = _i32(btm)
    out = np.empty(btm.size, np.int32)
    n = self.fn("generate_label")(_p(out), _p(btm), btm.size, mask)
    return out, n

  def search_key(self, key, query):
    key, query = _u64(key), _u64(query)
    out = np.empty(query.size, np.int32)
    self.fn("search_key")(_p(out), _p(key), key.size, _p(query), query.size)
    return out

  def xyz2key(self, xyz, depth):
    xyz = _u64(xyz)
    out = np.empty_like(xyz)
    self.fn("xyz2key")(_p(out), _p(xyz), xyz.size, depth)
    return out

  def key2xyz(self, key, depth):
    key = _u64(key)
    out = np.empty_like(key)
    self.fn("key2xyz")(_p(out), _p(key), key.size, depth)
    return out

  def key2idx(self, key):
    key = _u64(key)
    out = np.empty(key.size, np.int32)
    self.fn("key2idx")(_p(out), _p(key), key.size)
    return out

  # ---- conv (C restatement only) ---------------------------------------------
  def sgemm(self, A, B, transA=False, transB=False):
    A, B = _f32(A), _f32(B)
    M = A.shape[1] if transA else A.shape[0]
    K = A.shape[0] if transA else A.shape[1]
    N = B.shape[0] if transB else B.shape[1]
    out = np.empty((M, N), np.float32)
    self.fn("sgemm")(int(transA), int(transB), M, N, K, _p(A), _p(B), C.c_float(0.0), _p(out))
    return out

  def _conv(self, name, deconv, data, weights, blob, depth, num_output, kernel_size,
            stride, nempty):
    data, weights = _f32(data), _f32(weights)
    blob = np.ascontiguousarray(blob, dtype=np.uint8)
    ks = _i32(kernel_size)
    top_h = self.fn("conv_top_h")(_p(blob), depth, stride, int(nempty), int(deconv))
    if top_h < 0:
      raise RuntimeError("bad conv shape")
    top = np.zeros((num_output, top_h), np.float32)
    r = self.fn(name)(_p(top), _p(data), data.shape[0], data.shape[1], _p(weights),
                      _p(blob), depth, num_output, _p(ks), stride, int(nempty))
    if r < 0:
      raise RuntimeError("%s failed: %d" % (name, r))
    return top

  def octree_conv(self, data, weights, blob, depth, num_output, kernel_size, stride, nempty=False):
    return self._conv("octree_conv", False, data, weights, blob, depth, num_output,
                      kernel_size, stride, nempty)

  def octree_deconv(self, data, weights, blob, depth, num_output, kernel_size, stride, nempty=False):
    return self._conv("octree_deconv", True, data, weights, blob, depth, num_output,
                      kernel_size, stride, nempty)

  def _grad(self, name, data, weights, grad_out, blob, depth, num_output, kernel_size, stride, nempty):
    data, weights, grad_out = _f32(data), _f32(weights), _f32(grad_out)
    blob = np.ascontiguousarray(blob, dtype=np.uint8)
    ks = _i32(kernel_size)
    gd, gw = np.zeros_like(data), np.zeros_like(weights)
    r = self.fn(name)(_p(gd), _p(gw), _p(data), data.shape[0], data.shape[1], _p(weights), _p(grad_out),
                      _p(blob), depth, num_output, _p(ks), stride, int(nempty))
    if r < 0:
      raise RuntimeError("%s failed: %d" % (name, r))
    return gd, gw

  def octree_conv_grad(self, data, weights, grad_out, blob, depth, num_output, kernel_size, stride,
                       nempty=False):
    """-> (grad_data, grad_weights), pytorch/cpp/octree_conv.cpp:159-189."""
    return self._grad("octree_conv_grad", data, weights, grad_out, blob, depth, num_output, kernel_size,
                      stride, nempty)

  def octree_deconv_grad(self, data, weights, grad_out, blob, depth, num_output, kernel_size, stride,
                         nempty=False):
    return self._grad("octree_deconv_grad", data, weights, grad_out, blob, depth, num_output, kernel_size,
                      stride, nempty)


def make_points_blob(pts, normals=None, features=None, labels=None):
  """Serialized point cloud (octree/octree/points_info.h:35-39, points.cpp:96-148):
  88-byte header then xyz, normal, feature, label arrays, point-major."""
  pts = _f32(pts).reshape(-1, 3)
  n = pts.shape[0]
  arrs = [pts]
  chans = [3, 0, 0, 0]
  flags = 1
  for i, a in enumerate((normals, features, labels), start=1):
    if a is None:
      continue
    a = _f32(a).reshape(n, -1)
    chans[i] = a.shape[1]
    flags |= 1 << i
    arrs.append(a)
  hdr = np.zeros(88, np.uint8)
  hdr[:12] = np.frombuffer(b"_POINTS_1.0_", np.uint8)
  ints = hdr[16:].view(np.int32)
  ints[0] = n
  ints[1] = flags
  ints[2:6] = chans
  dis = [88]
  for c in chans:
    dis.append(dis[-1] + 4 * n * c)
  ints[10:15] = dis
  return np.concatenate([hdr] + [a.reshape(-1).view(np.uint8) for a in arrs])
