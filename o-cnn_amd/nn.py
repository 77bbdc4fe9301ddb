"""Host-side mirror of the reference's `ocnn.nn` extension (pytorch/cpp/pybind.cpp:3-49,
signatures pytorch/cpp/ocnn.h:11-72) over the C-ABI of libocnn_hip.so.

Same function names, argument order, tensor shapes and depth conventions as the
reference.  PyTorch only provides device memory and the current stream; every
computation happens in the HIP library.  Differences a caller can see:
  * octrees and point clouds live on the GPU (a CPU tensor is moved there); the
    results of `points2octree` and `octree_batch` are CUDA tensors;
  * the 716-byte octree header is read back from the device once per blob tensor
    and cached on the tensor object, not once per operator call;
  * failures raise `OcnnError` instead of aborting the process;
  * `points2octree_batch` (build + octree_batch fused in one pass) and bfloat16
    feature tensors are additions.
"""
import ctypes as C

import numpy as np
import torch

from . import lib as _lib
from .lib import BF16, F32, OcnnError, BuildParams  # noqa: F401
from .lib import CHILD, FEATURE, KEY, LABEL, NEIGH, SPLIT, HEADER_BYTES, INFO_BYTES

__all__ = [
    "points2octree", "points2octree_batch", "octree_batch", "octree_property",
    "octree_set_property", "octree2col", "col2octree", "octree_conv", "octree_deconv",
    "octree_conv_fused",
    "octree_pad", "octree_depad", "octree_max_pool", "octree_max_unpool", "octree_mask_pool",
    "octree_encode_key", "octree_decode_key", "octree_xyz2key", "octree_key2xyz",
    "octree_search_key", "octree_new", "octree_grow", "octree_update", "points_new",
    "octree_gather", "octree_gatherbk", "octree_mask", "octree_bilinear_neigh", "octree_bilinear_xyz",
    "octree_info", "octree_pad_fill", "forget_cached", "octree_max_pool_rows", "octree_scan", "octree_dropout", "octree_drop", "octree_samples",
]


# ---- plumbing ---------------------------------------------------------------------
def _ptr(t):
  return C.c_void_p(t.data_ptr() if t is not None else 0)


def _stream():
  return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev():
  if not torch.cuda.is_available():
    raise RuntimeError("o-cnn_amd needs a GPU: there is no CPU path")
  return torch.device("cuda", torch.cuda.current_device())


def _dtype_code(t):
  if t.dtype == torch.float32:
    return F32
  if t.dtype == torch.bfloat16:
    return BF16
  raise TypeError("feature tensors must be float32 or bfloat16, got %s" % t.dtype)


def _ks(kernel_size):
  ks = list(kernel_size)
  while len(ks) < 3:           # resize_with_last_val, pytorch/ocnn/octree_conv.py:8-12
    ks.append(ks[-1])
  return (C.c_int * 3)(*ks[:3]), ks[:3]


_workspaces = {}


def _workspace(nbytes, tag="main"):
  """A cached, growing device scratch buffer per (device, stream, tag).  Calls that share a
  workspace must not overlap, and calls on one stream never do; calls on different streams get
  different buffers.  A buffer is allocated while its stream is current, so when it is
  outgrown and dropped the caching allocator hands the block out again only in that stream's
  order: kernels still queued on the stream keep their memory."""
  key = (torch.cuda.current_device(), torch.cuda.current_stream().cuda_stream, tag)
  buf = _workspaces.get(key)
  if buf is None or buf.numel() < nbytes:
    buf = torch.empty(max(int(nbytes), 1 << 20), dtype=torch.uint8, device=_dev())
    _workspaces[key] = buf
  return buf


class _Info:
  """Host copy of an octree header plus typed accessors (through the C-ABI)."""

  def __init__(self, raw):
    self.raw = np.ascontiguousarray(raw[:INFO_BYTES], dtype=np.uint8).copy()
    self.p = C.c_void_p(self.raw.ctypes.data)
    L = _lib.get()
    self._L = L
    self.depth = L.ocnn_info_depth(self.p)
    self.full_depth = L.ocnn_info_full_depth(self.p)
    self.batch_size = L.ocnn_info_batch_size(self.p)
    self.key2xyz = bool(L.ocnn_info_is_key2xyz(self.p))

  def nnum(self, d):
    return self._L.ocnn_info_node_num(self.p, d)

  def nnum_nempty(self, d):
    return self._L.ocnn_info_node_num_nempty(self.p, d)

  def nnum_cum(self, d):
    return self._L.ocnn_info_node_num_cum(self.p, d)

  def total_nnum(self):
    return self._L.ocnn_info_total_nnum(self.p)

  def channel(self, ptype):
    return self._L.ocnn_info_channel(self.p, ptype)

  def location(self, ptype):
    return self._L.ocnn_info_location(self.p, ptype)

  def ptr_dis(self, ptype, d):
    return self._L.ocnn_info_ptr_dis(self.p, ptype, d)

  def size(self):
    return self._L.ocnn_info_sizeof_octree(self.p)


def octree_info(octree):
  """Header of an octree blob tensor; read from the device at most once per tensor."""
  info = getattr(octree, "_ocnn_info", None)
  if info is None:
    if octree.dtype != torch.uint8 or octree.dim() != 1 or octree.numel() < HEADER_BYTES:
      raise ValueError("an octree is a 1-D uint8 tensor of at least %d bytes" % HEADER_BYTES)
    info = _Info(octree[:INFO_BYTES].cpu().numpy())
    _lib.call("ocnn_info_check", info.p)
    octree._ocnn_info = info
  return info


def _attach(octree, raw_info):
  octree._ocnn_info = _Info(raw_info)
  return octree


def _to_dev(t):
  if t.is_cuda:
    return t.contiguous()
  info = getattr(t, "_ocnn_info", None)
  out = t.contiguous().to(_dev())
  if info is not None:
    out._ocnn_info = info
  return out


def _prop_view(octree, info, ptype, depth, count, dtype):
  """1-D view of `count` elements of a property at a depth inside the blob."""
  off = info.ptr_dis(ptype, depth)
  if off < 0:
    return None
  itemsize = torch.empty((), dtype=dtype).element_size()
  return octree[off:off + count * itemsize].view(dtype)


# ---- octree construction -------------------------------------------------------------
def _points_header(points):
  hdr = points[:_lib.POINTS_INFO_BYTES].cpu().numpy().copy()
  return hdr


_ALLOC_FN = C.CFUNCTYPE(C.c_void_p, C.c_size_t, C.c_void_p)


_blob_bytes_per_point = {}   # build settings -> bytes of blob per input point, from earlier builds


def _build(points_list, merged, depth, full_depth, node_dis, node_feature, split_label, adaptive,
           adp_depth, th_normal, th_distance, extrapolate, save_pts, key2xyz, bbox=None, ws_tag="build"):
  pts = [_to_dev(p) for p in points_list]
  hdrs = [getattr(p, "_ocnn_points_info", None) for p in points_list]
  for i, h in enumerate(hdrs):
    if h is None:
      hdrs[i] = _points_header(pts[i])
  n = len(pts)
  total = int(sum(int(h[16:20].view(np.int32)[0]) for h in hdrs))
  L = _lib.get()
  bp = BuildParams(depth=depth, full_depth=full_depth, node_dis=int(node_dis),
                   node_feature=int(node_feature), split_label=int(split_label),
                   adaptive=int(adaptive), adp_depth=adp_depth, th_normal=th_normal,
                   th_distance=th_distance, extrapolate=int(extrapolate), save_pts=int(save_pts),
                   key2xyz=int(key2xyz), merged=int(merged), has_bbox=int(bbox is not None))
  if bbox is not None:
    bp.bbmin = (C.c_float * 3)(*bbox[0])
    bp.bbmax = (C.c_float * 3)(*bbox[1])
  eff_depth = max(depth, max(full_depth, 1))
  ws_bytes = L.ocnn_points2octree_workspace_bytes(total, n, eff_depth)
  if ws_bytes == 0:
    raise OcnnError(-1, "bad build arguments (points %d, clouds %d, depth %d)" % (total, n, depth))
  ws = _workspace(ws_bytes + 256, ws_tag)
  base = (ws.data_ptr() + 255) & ~255
  dev_ptrs = (C.c_void_p * n)(*[p.data_ptr() for p in pts])
  hdr_ptrs = (C.c_void_p * n)(*[h.ctypes.data for h in hdrs])
  info_raw = np.zeros(INFO_BYTES, np.uint8)
  if not (node_feature or adaptive):
    # A plain octree: the blob's memory is obtained before the build, sized from the bytes per point
    # that earlier builds with these settings took, so that the device does not sit idle while the
    # interpreter allocates between the level scan and the emit step.  A guess that turns out too
    # small costs one more allocation; the blob is a view of the (slightly larger) buffer.
    key = (n, depth, full_depth, bool(node_dis), bool(split_label), bool(save_pts), bool(key2xyz), bool(merged),
           hdrs[0][20:24].tobytes(), hdrs[0][24:56].tobytes())
    ratio = _blob_bytes_per_point.get(key)
    cap = int(ratio * total * 1.125) + (1 << 16) if ratio else 0
    if cap:
      buf = torch.empty(cap, dtype=torch.uint8, device=_dev())
      rc = L.ocnn_points2octree_into(dev_ptrs, hdr_ptrs, n, C.byref(bp), C.c_void_p(base), C.c_size_t(ws_bytes),
                                     _ptr(buf), C.c_size_t(cap), C.c_void_p(info_raw.ctypes.data), _stream())
      if rc not in (0, -4):
        _lib.check(rc)
    else:
      _lib.call("ocnn_points2octree_plan", dev_ptrs, hdr_ptrs, n, C.byref(bp), C.c_void_p(base),
                C.c_size_t(ws_bytes), C.c_void_p(info_raw.ctypes.data), _stream())
      rc = -4
    info = _Info(info_raw)
    size = info.size()
    if rc == -4:
      buf = torch.empty(size, dtype=torch.uint8, device=_dev())
      _lib.call("ocnn_points2octree_emit", _ptr(buf), info.p, C.c_void_p(base), C.c_size_t(ws_bytes), _stream())
    _blob_bytes_per_point[key] = max(size / max(total, 1), 0.9 * ratio if ratio else 0.0)
    out = buf[:size]
    out._ocnn_info = info
    return out
  holder = []

  def alloc(nbytes, _ctx):
    t = torch.empty(int(nbytes), dtype=torch.uint8, device=_dev())
    holder.append(t)
    return t.data_ptr()

  out_ptr = C.c_void_p()
  _lib.call("ocnn_points2octree", dev_ptrs, hdr_ptrs, n, C.byref(bp), C.c_void_p(base),
            C.c_size_t(ws_bytes), _ALLOC_FN(alloc), None, C.c_void_p(info_raw.ctypes.data),
            C.byref(out_ptr), _stream())
  out = [t for t in holder if t.data_ptr() == out_ptr.value][-1]   # (scratch blocks come first)
  out._ocnn_info = _Info(info_raw)
  return out


def points2octree(points, depth, full_depth=2, node_dis=False, node_feature=False,
                  split_label=False, adaptive=False, adp_depth=4, th_normal=0.1,
                  th_distance=2.0, extrapolate=False, save_pts=False, key2xyz=False):
  """pytorch/cpp/point2octree.cpp:5-34 -- one serialized octree from one point cloud."""
  return _build([points], False, depth, full_depth, node_dis, node_feature, split_label,
                adaptive, adp_depth, th_normal, th_distance, extrapolate, save_pts, key2xyz)


def points2octree_batch(points_list, depth, full_depth=2, node_dis=False, node_feature=False,
                        split_label=False, adaptive=False, adp_depth=4, th_normal=0.1,
                        th_distance=2.0, extrapolate=False, save_pts=False, key2xyz=False):
  """`octree_batch([points2octree(p, ...) for p in points_list])` in one device pass
  (the composition `collate_octrees` performs, pytorch/ocnn/transforms.py:127-148)."""
  return _build(list(points_list), True, depth, full_depth, node_dis, node_feature, split_label,
                adaptive, adp_depth, th_normal, th_distance, extrapolate, save_pts, key2xyz)


def octree_samples(names):
  """pytorch/cpp/octree_samples.cpp:5-18 -- the small sample octrees the reference embeds
  (`octree_1` .. `octree_6`, 64-bit keys) as CPU uint8 tensors; data file of this package."""
  import os
  z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "data", "octree_samples.npz"))
  out = []
  for name in names:
    if name not in z.files:
      raise OcnnError(-1, "The specified octree does not exist : %s" % name)
    out.append(torch.from_numpy(z[name].copy()))
  return out


def octree_dropout(octree, depth_dropout, threshold, flags=None, generator=None, clear_dropped=False):
  """octree/octree/transform_octree.cpp:286-431 (`octree_drop(octree, depth, ratio)`,
  tensorflow/libs/transform_octree_op.cc:40-56): every node of level `depth_dropout` leaves
  with probability `threshold`, together with its subtree.  The reference draws the flags from
  an engine seeded with the clock; here they come from torch's generator on the device, or from
  `flags` (one entry per node of the level, non-zero = dropped).  As in the reference, a dropped
  node of level `depth_dropout` keeps its old child entry (transform_octree.cpp:422-425);
  `clear_dropped=True` writes -1 there instead, which octree_batch needs for its neighbour
  tables."""
  octree = _to_dev(octree)
  info = octree_info(octree)
  if not 0 <= depth_dropout <= info.depth:
    raise ValueError("depth_dropout %d outside [0, %d]" % (depth_dropout, info.depth))
  n = int(info.nnum(depth_dropout))
  if flags is None:
    flags = torch.rand(n, device=_dev(), generator=generator) < float(threshold)
  flags = torch.as_tensor(flags).to(_dev()).ne(0).to(torch.uint8).contiguous()
  if flags.numel() != n:
    raise ValueError("%d flags for the %d nodes of level %d" % (flags.numel(), n, depth_dropout))
  holder = []

  def alloc(nbytes, _ctx):
    t = torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=_dev())
    holder.append(t)
    return t.data_ptr()

  info_raw = np.zeros(INFO_BYTES, np.uint8)
  out_ptr = C.c_void_p()
  _lib.call("ocnn_octree_dropout", _ptr(octree), info.p, _ptr(flags), int(depth_dropout), int(bool(clear_dropped)),
            _ALLOC_FN(alloc), None,
            C.c_void_p(info_raw.ctypes.data), C.byref(out_ptr), _stream())
  out = [t for t in holder if t.data_ptr() == out_ptr.value][-1]
  out._ocnn_info = _Info(info_raw)
  return out


octree_drop = octree_dropout


def octree_scan(octree, axis, scale=1.0):
  """pytorch/cpp/transform_octree.cpp:5-22 -- the part of a single octree seen from the view
  directions `axis` (3 floats per direction), as the completion data set makes its partial
  scans (pytorch/projects/datasets/completion.py:9-36)."""
  octree = _to_dev(octree)
  info = octree_info(octree)
  ax = np.ascontiguousarray(np.asarray(axis, dtype=np.float32).reshape(-1))
  if ax.size == 0 or ax.size % 3:
    raise ValueError("axis needs 3 floats per direction")
  holder = []

  def alloc(nbytes, _ctx):
    t = torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=_dev())
    holder.append(t)
    return t.data_ptr()

  info_raw = np.zeros(INFO_BYTES, np.uint8)
  out_ptr = C.c_void_p()
  _lib.call("ocnn_octree_scan", _ptr(octree), info.p, C.c_void_p(ax.ctypes.data), ax.size // 3,
            C.c_float(scale), _ALLOC_FN(alloc), None, C.c_void_p(info_raw.ctypes.data), C.byref(out_ptr),
            _stream())
  out = [t for t in holder if t.data_ptr() == out_ptr.value][-1]
  out._ocnn_info = _Info(info_raw)
  return out


def octree_batch(octrees):
  """pytorch/cpp/octree_batch.cpp:5-22 -- merge serialized octrees, add neighbour tables."""
  octs = [_to_dev(o) for o in octrees]
  infos = [octree_info(o) for o in octs]
  n = len(octs)
  L = _lib.get()
  info_ptrs = (C.c_void_p * n)(*[i.raw.ctypes.data for i in infos])
  out_raw = np.zeros(INFO_BYTES, np.uint8)
  _lib.call("ocnn_octree_batch_info", info_ptrs, n, C.c_void_p(out_raw.ctypes.data))
  out_info = _Info(out_raw)
  out = torch.empty(out_info.size(), dtype=torch.uint8, device=_dev())
  ws_bytes = L.ocnn_octree_batch_workspace_bytes(n, out_info.depth)
  ws = _workspace(ws_bytes, "batch")
  dev_ptrs = (C.c_void_p * n)(*[o.data_ptr() for o in octs])
  _lib.call("ocnn_octree_batch", _ptr(out), out_info.p, dev_ptrs, info_ptrs, n, _ptr(ws),
            C.c_size_t(ws_bytes), _stream())
  out._ocnn_info = out_info
  return out


def points_new(pts, normals=None, features=None, labels=None):
  """pytorch/cpp/points_property.cpp `points_new`: serialized point cloud (88-byte header,
  then xyz, normal, feature, label arrays point-major: octree/octree/points.cpp:96-148)."""
  dev = pts.device
  pts = pts.reshape(-1, 3).to(torch.float32).contiguous()
  n = pts.shape[0]
  if n == 0:
    raise ValueError("empty point cloud")
  arrs, chans, flags = [pts], [3, 0, 0, 0], 1
  for i, a in enumerate((normals, features, labels), start=1):
    if a is None or a.numel() == 0:
      continue
    a = a.reshape(n, -1).to(torch.float32).contiguous()
    if (i == 1 and a.shape[1] != 3) or (i == 3 and a.shape[1] != 1):
      raise ValueError("normals need 3 channels and labels 1")
    chans[i] = a.shape[1]
    flags |= 1 << i
    arrs.append(a)
  hdr = np.zeros(_lib.POINTS_INFO_BYTES, np.uint8)
  hdr[:12] = np.frombuffer(b"_POINTS_1.0_", np.uint8)
  ints = hdr[16:].view(np.int32)
  ints[0], ints[1] = n, flags
  ints[2:6] = chans
  dis = [_lib.POINTS_INFO_BYTES]
  for c in chans:
    dis.append(dis[-1] + 4 * n * c)
  ints[10:15] = dis
  parts = [torch.from_numpy(hdr).to(dev)] + [a.reshape(-1).view(torch.uint8) for a in arrs]
  out = torch.cat(parts)
  out._ocnn_points_info = hdr
  return out


# ---- point-cloud transforms (pytorch/cpp/transform_points.cpp) ---------------------------------
def _points_hdr(points):
  hdr = getattr(points, "_ocnn_points_info", None)
  if hdr is None:
    hdr = _points_header(points)
    points._ocnn_points_info = hdr
  return hdr


def _f3(v):
  v = [float(x) for x in v]
  while len(v) < 3:
    v.append(v[-1])
  return (C.c_float * 3)(*v[:3])


def _points_ws(hdr):
  nbytes = _lib.get().ocnn_points_workspace_bytes(int(hdr[16:20].view(np.int32)[0]))
  ws = _workspace(nbytes + 256, "points")
  return C.c_void_p((ws.data_ptr() + 255) & ~255), C.c_size_t(nbytes)


def bounding_sphere(points, method="sphere"):
  """-> [radius, cx, cy, cz] (pytorch/cpp/transform_points.cpp:7-35).  'sphere' is the reference
  build without Miniball (octree/octree/math_functions.cpp:49-108), anything else the sphere
  around the bounding box."""
  points = _to_dev(points)
  hdr = _points_hdr(points)
  out = (C.c_float * 4)()
  base, nbytes = _points_ws(hdr)
  _lib.call("ocnn_bounding_sphere", _ptr(points), C.c_void_p(hdr.ctypes.data), int(method != "sphere"), out,
            base, nbytes, _stream())
  return [float(x) for x in out]


def normalize_points(points, radius, center):
  """pytorch/cpp/transform_points.cpp:51-71."""
  points = _to_dev(points)
  hdr = _points_hdr(points)
  out = torch.empty_like(points)
  _lib.call("ocnn_normalize_points", _ptr(out), _ptr(points), C.c_void_p(hdr.ctypes.data), C.c_float(radius),
            _f3(center), _stream())
  out._ocnn_points_info = hdr
  return out


def transform_points(points, angle, scale, jitter, offset=0.0, normal_axis=""):
  """pytorch/cpp/transform_points.cpp:73-109 (angles in radians)."""
  points = _to_dev(points)
  hdr = _points_hdr(points)
  out = torch.empty_like(points)
  _lib.call("ocnn_transform_points", _ptr(out), _ptr(points), C.c_void_p(hdr.ctypes.data), _f3(angle), _f3(scale),
            _f3(jitter), C.c_float(offset), normal_axis.encode(), _stream())
  out._ocnn_points_info = hdr
  return out


def clip_points(points, bbmin, bbmax):
  """-> [points, inbox_mask int32] (pytorch/cpp/transform_points.cpp:111-125); the mask stays on
  the device."""
  points = _to_dev(points)
  hdr = _points_hdr(points)
  npt = int(hdr[16:20].view(np.int32)[0])
  out = torch.empty_like(points)
  mask = torch.empty(npt, dtype=torch.int32, device=points.device)
  new_hdr = np.zeros(_lib.POINTS_INFO_BYTES, np.uint8)
  base, nbytes = _points_ws(hdr)
  _lib.call("ocnn_clip_points", _ptr(out), C.c_void_p(new_hdr.ctypes.data), _ptr(mask), _ptr(points),
            C.c_void_p(hdr.ctypes.data), _f3(bbmin), _f3(bbmax), base, nbytes, _stream())
  out._ocnn_points_info = new_hdr
  return [out, mask]


# ---- files ------------------------------------------------------------------------------------
def upgrade_key64(octree32):
  """upgrade_key64 (octree/octree/transform_octree.cpp:433-497) on a host uint8 tensor / array."""
  raw = np.ascontiguousarray(octree32.cpu().numpy() if torch.is_tensor(octree32) else octree32, dtype=np.uint8)
  nbytes = C.c_size_t()
  _lib.call("ocnn_upgrade_key64", C.c_void_p(raw.ctypes.data), C.c_size_t(raw.size), None, C.c_size_t(0),
            C.byref(nbytes))
  out = np.empty(nbytes.value, np.uint8)
  _lib.call("ocnn_upgrade_key64", C.c_void_p(raw.ctypes.data), C.c_size_t(raw.size), C.c_void_p(out.ctypes.data),
            C.c_size_t(out.size), C.byref(nbytes))
  return torch.from_numpy(out)


def read_octree(path):
  """A `.octree` file is the serialized blob (Octree::read_octree, octree/octree/octree.cpp:41-55);
  a file from a 32-bit-key build is upgraded on the way in.  Returns a host uint8 tensor."""
  raw = np.fromfile(path, dtype=np.uint8)
  if raw.size < INFO_BYTES:
    raise OcnnError(-6, "%s: shorter than an octree header" % path)
  if bytes(raw[:12]) == b"_OCTREE_1.0_":
    return upgrade_key64(raw)
  _Info(raw)  # validates the header
  return torch.from_numpy(raw)


def write_octree(octree, path):
  """Octree::write_octree, octree/octree/octree.cpp:57-68."""
  octree.cpu().numpy().tofile(path)


def read_points(path):
  """Points::read_points, octree/octree/points.cpp:9-27 -> host uint8 tensor."""
  raw = np.fromfile(path, dtype=np.uint8)
  if raw.size < _lib.POINTS_INFO_BYTES or bytes(raw[:12]) != b"_POINTS_1.0_":
    raise OcnnError(-6, "%s: not a _POINTS_1.0_ file" % path)
  out = torch.from_numpy(raw)
  out._ocnn_points_info = raw[:_lib.POINTS_INFO_BYTES].copy()
  return out


def write_points(points, path):
  """Points::write_points, octree/octree/points.cpp:29-37."""
  points.cpu().numpy().tofile(path)


# ---- properties ------------------------------------------------------------------------
def octree_property(octree, property, depth=0):
  """pytorch/cpp/octree_property.cpp:11-344."""
  info = octree_info(octree)
  name = property
  nnum = info.nnum(depth) if depth > 0 else info.total_nnum()
  dev = octree.device
  if name in ("key", "xyz"):
    ch = info.channel(KEY)
    src = _prop_view(octree, info, KEY, depth, ch * nnum, torch.int64)
    convert = info.key2xyz if name == "key" else not info.key2xyz
    if not convert:
      return src.clone()
    fn = "ocnn_xyz2key" if name == "key" else "ocnn_key2xyz"
    src_d = _to_dev(src)
    out = torch.zeros_like(src_d)
    if depth > 0:
      _lib.call(fn, _ptr(out), _ptr(src_d), ch * nnum, depth, _stream())
    else:   # depth 0 is left as zero, as in the reference loop (d = 1 .. depth)
      for d in range(1, info.depth + 1):
        n_d, c_d = info.nnum(d), info.nnum_cum(d)
        if n_d:
          _lib.call(fn, _ptr(out[c_d:c_d + n_d]), _ptr(src_d[c_d:c_d + n_d]), n_d, d, _stream())
    return out.to(dev)
  if name == "index":
    ch = info.channel(KEY)
    src = _to_dev(_prop_view(octree, info, KEY, depth, ch * nnum, torch.int64))
    out = torch.zeros(ch * nnum, dtype=torch.int32, device=src.device)
    _lib.call("ocnn_key2idx", _ptr(out), _ptr(src), ch * nnum, _stream())
    return out.to(dev)
  if name == "child":
    return _prop_view(octree, info, CHILD, depth, nnum * info.channel(CHILD), torch.int32).clone()
  if name == "neigh":
    ch = info.channel(NEIGH)
    return _prop_view(octree, info, NEIGH, depth, nnum * ch, torch.int32).clone().view(nnum, ch)
  if name == "feature":
    ch = info.channel(FEATURE)
    v = _prop_view(octree, info, FEATURE, depth, nnum * ch, torch.float32)
    if v is None:
      raise OcnnError(-6, "The features do not exist: d = %d" % depth)
    return v.clone().view(1, ch, nnum, 1)
  if name == "label":
    return _prop_view(octree, info, LABEL, depth, nnum * info.channel(LABEL), torch.float32).clone()
  if name == "split":
    return _prop_view(octree, info, SPLIT, depth, nnum * info.channel(SPLIT), torch.float32).clone()
  ints = None
  if name == "node_num":
    ints = [info.nnum(depth)] if depth > 0 else [info.nnum(d) for d in range(info.depth + 1)]
  elif name in ("node_num_ne", "node_num_nempty"):
    ints = [info.nnum_nempty(depth)] if depth > 0 else \
        [info.nnum_nempty(d) for d in range(info.depth + 1)]
  elif name == "node_num_cum":
    ints = [info.nnum_cum(depth)] if depth > 0 else [info.nnum_cum(d) for d in range(info.depth + 2)]
  elif name == "batch_size":
    ints = [info.batch_size]
  elif name == "depth":
    ints = [info.depth]
  elif name == "full_depth":
    ints = [info.full_depth]
  if ints is None:
    raise OcnnError(-1, "Unsupport octree property: %s" % name)
  return torch.tensor(ints, dtype=torch.int32, device=dev)


def octree_set_property(octree, data, depth):
  """pytorch/cpp/octree_property.cpp:308-325 -- returns a copy with the features of one depth replaced."""
  info = octree_info(octree)
  count = info.nnum(depth) * info.channel(FEATURE)
  if data.numel() != count:
    raise OcnnError(-3, "Wrong Property Size")
  out = octree.clone()
  out._ocnn_info = info
  _prop_view(out, info, FEATURE, depth, count, torch.float32).copy_(
      data.to(torch.float32).reshape(-1))
  return out


# ---- octree2col / col2octree ---------------------------------------------------------------
def _ichild(octree, info, depth):
  n, ne = info.nnum(depth), info.nnum_nempty(depth)
  child = _prop_view(octree, info, CHILD, depth, n, torch.int32)
  ichild = torch.zeros(max(ne, 1), dtype=torch.int32, device=octree.device)
  _lib.call("ocnn_make_ichild", _ptr(ichild), ne, _ptr(child), n, _stream())
  return child, ichild


def octree2col(data_in, octree, depth, kernel_size, stride, nempty):
  """pytorch/cpp/octree2col.cpp:47-237: [1,C,H,1] -> [C, K, H_out]."""
  octree = _to_dev(octree)
  info = octree_info(octree)
  ksc, ks = _ks(kernel_size)
  data_in = data_in.contiguous()
  dt = _dtype_code(data_in)
  channel, btm_h = data_in.size(1), data_in.size(2)
  K = ks[0] * ks[1] * ks[2]
  neigh = _prop_view(octree, info, NEIGH, depth, info.nnum(depth) * 8, torch.int32)
  if not nempty:
    if btm_h != info.nnum(depth):
      raise OcnnError(-3, "octree2col: height %d != node_num(%d) = %d" % (btm_h, depth, info.nnum(depth)))
    top_h = btm_h
    if stride == 2:
      top_h = btm_h // 8
      if top_h != info.nnum_nempty(depth - 1):
        raise OcnnError(-3, "octree2col: stride-2 height mismatch")
    out = torch.empty(channel, K, top_h, dtype=data_in.dtype, device=data_in.device)
    _lib.call("ocnn_octree2col", _ptr(out), _ptr(data_in), channel, top_h, ksc, stride, _ptr(neigh),
              max(top_h, 1), 0, dt, _stream())
    return out
  if btm_h != info.nnum_nempty(depth):
    raise OcnnError(-3, "octree2col: height %d != node_num_nempty(%d)" % (btm_h, depth))
  child, ichild = _ichild(octree, info, depth)
  top_h = btm_h if stride == 1 else info.nnum_nempty(depth - 1)
  out = torch.empty(channel, K, top_h, dtype=data_in.dtype, device=data_in.device)
  _lib.call("ocnn_octree2colP", _ptr(out), _ptr(data_in), channel, top_h, btm_h, ksc, stride,
            _ptr(neigh), _ptr(child), _ptr(ichild), max(top_h, 1), 0, dt, _stream())
  return out


def col2octree(grad_in, octree, depth, kernel_size, stride, nempty):
  """pytorch/cpp/octree2col.cpp:95-237: [C, K, H_out] -> [1,C,H,1] (scatter-add)."""
  octree = _to_dev(octree)
  info = octree_info(octree)
  ksc, ks = _ks(kernel_size)
  grad_in = grad_in.contiguous()
  dt = _dtype_code(grad_in)
  channel, top_h = grad_in.size(0), grad_in.size(2)
  neigh = _prop_view(octree, info, NEIGH, depth, info.nnum(depth) * 8, torch.int32)
  if stride == 2 and top_h != info.nnum_nempty(depth - 1):
    raise OcnnError(-3, "col2octree: stride-2 height mismatch")
  # The verdict on the level's table (does it map back and forth consistently, so that the sum
  # may be gathered) is kept with the octree tensor, one device word per (depth, kernel, stride,
  # mode): the first call checks the table on the device, later calls read the word.
  marks = getattr(octree, "_ocnn_col_marks", None)
  if marks is None:
    marks = octree._ocnn_col_marks = {}
  # one word per (table, shape, version of the blob) AND stream: the first call on a stream checks
  # the table on that stream, so no call reads a word whose check is still queued on another stream
  key = (depth, tuple(ks), stride, bool(nempty), top_h, octree._version, torch.cuda.current_stream().cuda_stream)
  mark = marks.get(key)
  check_now = mark is None
  if check_now:
    mark = marks[key] = torch.zeros(1, dtype=torch.int64, device=grad_in.device)
  if not nempty:
    btm_h = info.nnum(depth)
    out = torch.empty(1, channel, btm_h, 1, dtype=grad_in.dtype, device=grad_in.device)
    _lib.call("ocnn_col2octree_cached", _ptr(grad_in), _ptr(out), channel, top_h, top_h << (3 * (stride - 1)), ksc,
              stride, _ptr(neigh), None, None, max(top_h, 1), 0, dt, _ptr(mark), int(check_now), _stream())
    return out
  btm_h = info.nnum_nempty(depth)
  if stride == 1 and top_h != btm_h:
    raise OcnnError(-3, "col2octree: height mismatch")
  child, ichild = _ichild(octree, info, depth)
  out = torch.empty(1, channel, btm_h, 1, dtype=grad_in.dtype, device=grad_in.device)
  _lib.call("ocnn_col2octree_cached", _ptr(grad_in), _ptr(out), channel, top_h, btm_h, ksc, stride,
            _ptr(neigh), _ptr(child), _ptr(ichild), max(top_h, 1), 0, dt, _ptr(mark), int(check_now), _stream())
  return out


# ---- convolution -------------------------------------------------------------------------------
def _conv_sources(octree, info, depth, kernel_size, ksc, stride, is_deconv, ws_base, ws_bytes):
  """The source row of every (tap, column) of an operator over the non-empty nodes, made once per
  octree version, depth, kernel shape and direction and kept with the octree tensor (every layer
  of that depth reads the same table; the row-major entry points share it).  None for an
  operator that looks nothing up."""
  tables = octree.__dict__.setdefault("_ocnn_sources", {})
  if tables.get("version") != octree._version:
    tables.clear()
    tables["version"] = octree._version
  skey = (depth, tuple(int(k) for k in kernel_size), stride, bool(is_deconv))
  sources = tables.get(skey, False)
  if sources is False:
    sources = None
    nb = C.c_size_t()
    try:
      _lib.call("ocnn_conv_rows_sources_bytes", info.p, depth, ksc, stride, 1, int(is_deconv), C.byref(nb))
    except OcnnError:       # a shape the row-major operators do not serve: the kernel looks its rows up itself
      nb = C.c_size_t(0)
    if nb.value:
      sources = torch.empty(nb.value // 4, dtype=torch.int32, device=octree.device)
      _lib.call("ocnn_conv_rows_sources", _ptr(sources), C.c_size_t(nb.value), None, _ptr(octree), info.p, depth, ksc,
                stride, 1, int(is_deconv), C.c_void_p(ws_base), C.c_size_t(ws_bytes), _stream())
    tables[skey] = sources
  return sources


def _conv(fn, is_deconv, data_in, weights, octree, depth, num_output, kernel_size, stride, nempty,
          bias=None, relu=False, out=None):
  octree = _to_dev(octree)
  info = octree_info(octree)
  ksc, ks3 = _ks(kernel_size)
  data_in = data_in.contiguous()
  weights = weights.contiguous()
  dt = _dtype_code(data_in)
  if weights.dtype != data_in.dtype:
    raise TypeError("weights and data must have the same dtype")
  channel_in, btm_h = data_in.size(1), data_in.size(2)
  top_h, need_h, ws_bytes = C.c_int(), C.c_int(), C.c_size_t()
  _lib.call("ocnn_conv_shape", info.p, depth, channel_in, num_output, ksc, stride, int(nempty),
            int(is_deconv), dt, C.byref(top_h), C.byref(need_h), C.byref(ws_bytes))
  ws = _workspace(ws_bytes.value + 256, "conv")
  base = (ws.data_ptr() + 255) & ~255
  shape = (1, num_output, top_h.value, 1)
  if out is None:
    out = torch.empty(shape, dtype=data_in.dtype, device=data_in.device)
  elif (tuple(out.shape) != shape or out.dtype != data_in.dtype or out.device != data_in.device
        or not out.is_contiguous()):
    # e.g. a channel slice of a larger [1, C, H, 1] tensor: the result lands there directly
    raise OcnnError(-3, "out must be a contiguous %s %s tensor on %s" % (shape, data_in.dtype, data_in.device))
  sources = None
  # (1x1x1 and the fp32 2x2x2 stride-2 deconvolution have kernels of their own that look nothing up)
  own_kernel = ks3 == [1, 1, 1] or (dt == F32 and is_deconv and stride == 2 and ks3 == [2, 2, 2])
  if nempty and top_h.value > 0 and btm_h > 0 and not own_kernel:
    sources = _conv_sources(octree, info, depth, ks3, ksc, stride, is_deconv, base, ws_bytes.value)
  if fn == "ocnn_octree_conv_fused" or sources is not None:
    if bias is not None:
      bias = bias.to(torch.float32).contiguous()
      if bias.numel() != num_output:
        raise OcnnError(-3, "bias needs num_output entries")
    _lib.call("ocnn_octree_conv_fused_sources", _ptr(out), _ptr(data_in), channel_in, btm_h, _ptr(weights), _ptr(bias),
              int(relu), int(is_deconv), _ptr(sources), C.c_size_t(sources.numel() * 4 if sources is not None else 0),
              _ptr(octree), info.p, depth, num_output, ksc, stride, int(nempty), dt,
              C.c_void_p(base), C.c_size_t(ws_bytes.value), _stream())
  else:
    _lib.call(fn, _ptr(out), _ptr(data_in), channel_in, btm_h, _ptr(weights), _ptr(octree), info.p,
              depth, num_output, ksc, stride, int(nempty), dt, C.c_void_p(base),
              C.c_size_t(ws_bytes.value), _stream())
  return out


def octree_conv(data_in, weights, octree, depth, num_output, kernel_size, stride, nempty):
  """pytorch/cpp/octree_conv.cpp:131-157: [1,Ci,H,1] x [Co, Ci*K] -> [1,Co,top_h,1]."""
  return _conv("ocnn_octree_conv", False, data_in, weights, octree, depth, num_output,
               kernel_size, stride, nempty)


def octree_deconv(data_in, weights, octree, depth, num_output, kernel_size, stride, nempty):
  """pytorch/cpp/octree_conv.cpp:189-216: weights are [Ci, Co*K]."""
  return _conv("ocnn_octree_deconv", True, data_in, weights, octree, depth, num_output,
               kernel_size, stride, nempty)


def octree_conv_fused(data_in, weights, bias, relu, octree, depth, num_output, kernel_size, stride,
                      nempty, deconv=False, out=None):
  """conv (or deconv) + per-channel bias + optional ReLU in one kernel: the inference form of
  the reference's conv -> BatchNorm -> ReLU modules (pytorch/ocnn/modules.py:23-36) once the
  BatchNorm statistics are folded into `weights` and `bias`.  `out`: where the result goes, e.g.
  a channel slice of the tensor a later layer reads as a concatenation."""
  return _conv("ocnn_octree_conv_fused", deconv, data_in, weights, octree, depth, num_output,
               kernel_size, stride, nempty, bias=bias, relu=relu, out=out)


def conv1x1_pair(data, w1, b1, w2, b2, relu=True, return_label=False):
  """Two 1x1x1 convolutions in one pass over `data` [1, C, H, 1] fp32: relu(w1 data + b1) -> w2 . + b2,
  the prediction head of pytorch/ocnn/ounet.py:46-49 with the BatchNorm folded into (w1, b1).
  w1 [hidden <= 32, C], w2 [n_out <= 8, hidden]; the biases may be None.  Returns the logits
  [1, n_out, H, 1], and with return_label their argmax over the channels (int32 [H], the labels of
  ounet.py:117-118) from the same kernel."""
  data = data.contiguous()
  if data.dtype != torch.float32:
    raise TypeError("conv1x1_pair is fp32")
  c, h = data.size(1), data.size(2)
  w1, w2 = w1.contiguous().float(), w2.contiguous().float()
  hidden, n_out = w1.size(0), w2.size(0)
  if w1.numel() != hidden * c or w2.numel() != n_out * hidden:
    raise OcnnError(-3, "conv1x1_pair: weights [%d, %d] and [%d, %d] expected" % (hidden, c, n_out, hidden))
  b1 = None if b1 is None else b1.contiguous().float()
  b2 = None if b2 is None else b2.contiguous().float()
  out = torch.empty(1, n_out, h, 1, dtype=torch.float32, device=data.device)
  label = torch.empty(h, dtype=torch.int32, device=data.device) if return_label else None
  _lib.call("ocnn_conv1x1_pair", _ptr(out), _ptr(label), _ptr(data), c, h, _ptr(w1), _ptr(b1), hidden, int(relu),
            _ptr(w2), _ptr(b2), n_out, _stream())
  return (out, label) if return_label else out


def forget_cached(tensor):
  """Drops what this module keeps with a tensor between calls: the packed weights of
  octree_conv_rows(constant_weights=True), and for an octree blob the inverted child links, the
  col2octree table verdicts and the host copy of the header.  For writes that the tensor's version
  counter does not see."""
  for name in ("_ocnn_rows_packed", "_ocnn_ichild", "_ocnn_sources", "_ocnn_col_marks", "_ocnn_info"):
    tensor.__dict__.pop(name, None)


def rows_pitch(channels):
  """channels per row of the row-major layout: padded to whole 16-channel steps"""
  return (int(channels) + 15) // 16 * 16


def to_rows(data):
  """[1, C, H, 1] bf16 (the reference's channel-major layout) -> rows [H + 1, pitch]: row h holds the
  channels of node h, padding channels and row H are zero (row H is what a missing neighbour reads)."""
  data = data.contiguous()
  if data.dtype != torch.bfloat16:
    raise TypeError("row-major tensors are bf16")
  c, h = data.size(1), data.size(2)
  rows = torch.empty(h + 1, rows_pitch(c), dtype=data.dtype, device=data.device)
  _lib.call("ocnn_rows_from_channels", _ptr(rows), rows.size(1), _ptr(data), c, h, _dtype_code(data), _stream())
  return rows


def from_rows(rows, channels):
  """rows [H + 1, pitch] -> [1, channels, H, 1]"""
  rows = rows.contiguous()
  h = rows.size(0) - 1
  data = torch.empty(1, channels, h, 1, dtype=rows.dtype, device=rows.device)
  _lib.call("ocnn_channels_from_rows", _ptr(data), _ptr(rows), rows.size(1), channels, h, _dtype_code(rows), _stream())
  return data


def octree_conv_rows(rows_in, channel_in, weights, octree, depth, num_output, bias=None, relu=False,
                     deconv=False, out=None, kernel_size=(3, 3, 3), stride=1, nempty=False, constant_weights=False):
  """Convolutions over all nodes in bf16, row-major on both sides: the arithmetic of octree_conv /
  octree_conv_fused (pytorch/cpp/octree_conv.cpp:131-216) on tensors that a chain of convolutions
  keeps in the layout the kernels gather from, so that no member of the chain copies its input.
    3x3x3 stride 1: rows of `depth` in and out (bit-identical to the channel-major operator);
    2x2x2 stride 2 conv: rows of `depth` in, rows of ALL nodes of depth-1 out -- the octree_pad of
      the reference's modules (pytorch/ocnn/octree_conv.py:102-127) is folded in, an empty node
      receives the bias alone;
    2x2x2 stride 2 deconv: rows of ALL nodes of `depth` in (the octree_depad of those modules is
      folded in), rows of depth+1 out.
  With nempty=True the rows on both sides are the ranks of the non-empty nodes, as in the
  channel-major operators (3x3x3 stride 1 and 2x2x2 stride 2, conv and deconv).
  constant_weights=True (inference): the packed form of `weights` is kept with the tensor (and
  packed again when the tensor's version counter or address changes), the inverted child links
  with the octree, so that a call launches the convolution kernel alone.  A write that bypasses
  the version counter (`weights.data.copy_(...)`, a raw-pointer write into the octree) is not
  seen: pass constant_weights=False then, or call forget_cached(weights) / forget_cached(octree)
  after such a write.
  rows_in: [H + 1, rows_pitch(channel_in)] as to_rows makes it.  `out`: [top_h + 1, P] with
  P >= rows_pitch(num_output), or columns c0 .. c0 + rows_pitch(num_output) of such a tensor (a
  slice of what a later layer reads as a concatenation); returns `out`."""
  octree = _to_dev(octree)
  info = octree_info(octree)
  ksc, _ = _ks(kernel_size)
  weights = weights.contiguous()
  if rows_in.dim() != 2 or rows_in.stride(1) != 1:
    raise OcnnError(-3, "rows_in must be [H + 1, pitch] with unit channel stride")
  dt = _dtype_code(rows_in)
  if weights.dtype != rows_in.dtype:
    raise TypeError("weights and data must have the same dtype")
  btm_h = rows_in.size(0) - 1
  top_h, need_h, ws_bytes = C.c_int(), C.c_int(), C.c_size_t()
  _lib.call("ocnn_conv_rows_shape", info.p, depth, channel_in, num_output, ksc, stride, int(nempty), int(deconv), dt,
            C.byref(top_h), C.byref(need_h), C.byref(ws_bytes))
  ws = _workspace(ws_bytes.value + 256, "conv")
  base = (ws.data_ptr() + 255) & ~255
  cpad = rows_pitch(num_output)
  if out is None:
    out = torch.empty(top_h.value + 1, cpad, dtype=rows_in.dtype, device=rows_in.device)
  elif (out.dim() != 2 or out.size(0) != top_h.value + 1 or out.size(1) < cpad or out.stride(1) != 1
        or out.dtype != rows_in.dtype or out.device != rows_in.device):
    raise OcnnError(-3, "out must be [%d, >= %d] %s with unit channel stride" % (top_h.value + 1, cpad, rows_in.dtype))
  if bias is not None:
    bias = bias.to(torch.float32).contiguous()
    if bias.numel() != num_output:
      raise OcnnError(-3, "bias needs num_output entries")
  if constant_weights:
    # (the byte count is part of the key: it also tells the two orders apart that a 64-channel
    # pass over the non-empty nodes can be packed in, which one depends on the level)
    nbytes = C.c_size_t()
    _lib.call("ocnn_conv_rows_packed_bytes", info.p, depth, channel_in, num_output, ksc, stride, int(nempty),
              int(deconv), dt, C.byref(nbytes))
    key = (channel_in, num_output, tuple(kernel_size), stride, bool(nempty), bool(deconv), nbytes.value)
    cache = weights.__dict__.setdefault("_ocnn_rows_packed", {})
    ent = cache.get(key)
    stamp = (weights._version, weights.data_ptr())
    if ent is None or ent[0] != stamp:
      packed = torch.empty(nbytes.value, dtype=torch.uint8, device=weights.device)
      _lib.call("ocnn_conv_rows_pack", _ptr(packed), C.c_size_t(nbytes.value), _ptr(weights), _ptr(octree), info.p, depth,
                channel_in, num_output, ksc, stride, int(nempty), int(deconv), dt, _stream())
      ent = cache[key] = (stamp, packed)
    links = None
    sources = None
    link_depth = depth + 1 if (deconv and stride == 2 and nempty) else depth
    if nempty:
      # the source row of every (tap, column): the same for every layer on this level with this
      # kernel shape, kept with the octree
      tables = octree.__dict__.setdefault("_ocnn_sources", {})
      if tables.get("version") != octree._version:
        tables.clear()
        tables["version"] = octree._version
      skey = (depth, tuple(kernel_size), stride, bool(deconv))
      sources = tables.get(skey, False)
      if sources is False:
        nb = C.c_size_t()
        _lib.call("ocnn_conv_rows_sources_bytes", info.p, depth, ksc, stride, 1, int(deconv), C.byref(nb))
        sources = None       # an operator that looks nothing up (the 2x2x2 stride-2 deconvolution)
        if nb.value:
          sources = torch.empty(nb.value // 4, dtype=torch.int32, device=octree.device)
          _lib.call("ocnn_conv_rows_sources", _ptr(sources), C.c_size_t(nb.value), None, _ptr(octree), info.p, depth, ksc,
                    stride, 1, int(deconv), C.c_void_p(base), C.c_size_t(ws_bytes.value), _stream())
        tables[skey] = sources
    elif deconv and stride == 2:
      links_of = octree.__dict__.setdefault("_ocnn_ichild", {})
      if links_of.get("version") != octree._version:      # the blob was written to through torch
        links_of.clear()
        links_of["version"] = octree._version
      links = links_of.get(link_depth)
      if links is None:
        child = octree_property(octree, "child", link_depth).view(-1)
        links = torch.empty(info.nnum_nempty(link_depth) + 1, dtype=torch.int32, device=octree.device)
        _lib.call("ocnn_make_ichild", _ptr(links), info.nnum_nempty(link_depth), _ptr(child), child.numel(), _stream())
        links_of[link_depth] = links
    _lib.call("ocnn_octree_conv_rows_packed", _ptr(out), out.stride(0), _ptr(rows_in), rows_in.stride(0), channel_in,
              btm_h, _ptr(ent[1]), C.c_size_t(ent[1].numel()), _ptr(links), _ptr(sources), _ptr(bias), int(relu), int(deconv), _ptr(octree), info.p, depth,
              num_output, ksc, stride, int(nempty), dt, C.c_void_p(base), C.c_size_t(ws_bytes.value), _stream())
    return out
  _lib.call("ocnn_octree_conv_rows", _ptr(out), out.stride(0), _ptr(rows_in), rows_in.stride(0), channel_in, btm_h,
            _ptr(weights), _ptr(bias), int(relu), int(deconv), _ptr(octree), info.p, depth, num_output, ksc, stride,
            int(nempty), dt, C.c_void_p(base), C.c_size_t(ws_bytes.value), _stream())
  return out


def octree_max_pool_rows(rows_in, channels, octree, depth, return_mask=False):
  """OctreeMaxPool (pytorch/ocnn/octree_pool.py:79-86: max_pool at `depth`, then pad at depth-1)
  on row-major bf16 activations: [H_depth + 1, pitch] -> [H_{depth-1} + 1, pitch], empty nodes
  zero; with return_mask also the int32 rows of the maxima ([H_{depth-1} + 1, pitch], -1 for an
  empty node).  Bit-equal to the channel-major pair."""
  octree = _to_dev(octree)
  info = octree_info(octree)
  if rows_in.dim() != 2 or rows_in.stride(1) != 1 or rows_in.size(0) != info.nnum(depth) + 1:
    raise OcnnError(-3, "rows_in must be [%d, pitch] with unit channel stride" % (info.nnum(depth) + 1))
  top_h = info.nnum(depth - 1)
  pitch = rows_pitch(channels)
  out = torch.empty(top_h + 1, pitch, dtype=rows_in.dtype, device=rows_in.device)
  mask = torch.empty(top_h + 1, pitch, dtype=torch.int32, device=rows_in.device) if return_mask else None
  _lib.call("ocnn_octree_max_pool_rows", _ptr(out), pitch, _ptr(mask), _ptr(rows_in), rows_in.stride(0), channels,
            _ptr(octree), info.p, depth, _dtype_code(rows_in), _stream())
  return (out, mask) if return_mask else out


def _conv_grad(fn, is_deconv, data_in, weights, octree, grad_in, depth, num_output, kernel_size, stride,
               nempty, need_data=True, need_weights=True):
  octree = _to_dev(octree)
  info = octree_info(octree)
  ksc, _ = _ks(kernel_size)
  data_in, weights, grad_in = data_in.contiguous(), weights.contiguous(), grad_in.contiguous()
  dt = _dtype_code(data_in)
  if weights.dtype != data_in.dtype or grad_in.dtype != data_in.dtype:
    raise TypeError("data, weights and gradient must have the same dtype")
  channel_in, btm_h = data_in.size(1), data_in.size(2)
  top_h, need_h, ws_bytes = C.c_int(), C.c_int(), C.c_size_t()
  _lib.call("ocnn_conv_shape", info.p, depth, channel_in, num_output, ksc, stride, int(nempty),
            int(is_deconv), dt, C.byref(top_h), C.byref(need_h), None)
  if grad_in.size(1) != num_output or grad_in.size(2) != top_h.value:
    raise OcnnError(-3, "gradient shape %s, the operator's output is [1, %d, %d, 1]" %
                    (tuple(grad_in.shape), num_output, top_h.value))
  _lib.call("ocnn_conv_grad_workspace_bytes", info.p, depth, channel_in, num_output, ksc, stride,
            int(nempty), int(is_deconv), dt, C.byref(ws_bytes))
  ws = _workspace(ws_bytes.value + 256, "conv")
  base = (ws.data_ptr() + 255) & ~255
  grad_data = torch.empty_like(data_in) if need_data else None
  grad_w = torch.empty_like(weights) if need_weights else None
  if grad_data is None and grad_w is None:
    return [None, None]
  _lib.call(fn, _ptr(grad_data), _ptr(grad_w), _ptr(data_in), channel_in, btm_h, _ptr(weights),
            _ptr(grad_in), _ptr(octree), info.p, depth, num_output, ksc, stride, int(nempty), dt,
            C.c_void_p(base), C.c_size_t(ws_bytes.value), _stream())
  return [grad_data, grad_w]


def octree_conv_grad(data_in, weights, octree, grad_in, depth, num_output, kernel_size, stride, nempty,
                     need_data=True, need_weights=True):
  """pytorch/cpp/octree_conv.cpp:159-189 -> [grad_data, grad_weights] (fp32); a gradient that is
  not needed is skipped and returned as None."""
  return _conv_grad("ocnn_octree_conv_grad", False, data_in, weights, octree, grad_in, depth, num_output,
                    kernel_size, stride, nempty, need_data, need_weights)


def octree_deconv_grad(data_in, weights, octree, grad_in, depth, num_output, kernel_size, stride, nempty,
                       need_data=True, need_weights=True):
  """pytorch/cpp/octree_conv.cpp:218-250 -> [grad_data, grad_weights] (fp32)."""
  return _conv_grad("ocnn_octree_deconv_grad", True, data_in, weights, octree, grad_in, depth, num_output,
                    kernel_size, stride, nempty, need_data, need_weights)


# ---- pad / pool ------------------------------------------------------------------------------------
def octree_pad(data_in, octree, depth, val=0.0):
  """pytorch/cpp/octree_pad.cpp:6-32."""
  octree = _to_dev(octree)
  info = octree_info(octree)
  if depth < 1:
    raise OcnnError(-1, "Depth should be larger than 1")
  data_in = data_in.contiguous()
  channel, btm_h = data_in.size(1), data_in.size(2)
  if btm_h != info.nnum_nempty(depth):
    raise OcnnError(-3, "pad, d = %d, channel = %d: height %d != %d" %
                    (depth, channel, btm_h, info.nnum_nempty(depth)))
  top_h = info.nnum(depth)
  child = _prop_view(octree, info, CHILD, depth, top_h, torch.int32)
  out = torch.empty(1, channel, top_h, 1, dtype=data_in.dtype, device=data_in.device)
  _lib.call("ocnn_pad_forward", _ptr(out), top_h, channel, _ptr(data_in), btm_h, _ptr(child),
            C.c_float(val), _dtype_code(data_in), _stream())
  return out


def octree_pad_fill(data_in, octree, depth, fill):
  """octree_pad with one value per channel (`fill`, fp32 [C]) in the empty nodes instead of a scalar."""
  octree = _to_dev(octree)
  info = octree_info(octree)
  data_in = data_in.contiguous()
  channel, btm_h = data_in.size(1), data_in.size(2)
  if btm_h != info.nnum_nempty(depth):
    raise OcnnError(-3, "pad, d = %d, channel = %d: height %d != %d" % (depth, channel, btm_h, info.nnum_nempty(depth)))
  fill = fill.to(torch.float32).contiguous()
  if fill.numel() != channel:
    raise OcnnError(-3, "fill needs one value per channel")
  top_h = info.nnum(depth)
  child = _prop_view(octree, info, CHILD, depth, top_h, torch.int32)
  out = torch.empty(1, channel, top_h, 1, dtype=data_in.dtype, device=data_in.device)
  _lib.call("ocnn_pad_forward_fill", _ptr(out), top_h, channel, _ptr(data_in), btm_h, _ptr(child), _ptr(fill),
            _dtype_code(data_in), _stream())
  return out


def octree_depad(data_in, octree, depth):
  """pytorch/cpp/octree_pad.cpp:34-60."""
  octree = _to_dev(octree)
  info = octree_info(octree)
  if depth < 1:
    raise OcnnError(-1, "Depth should be larger than 1")
  data_in = data_in.contiguous()
  channel, top_h = data_in.size(1), data_in.size(2)
  if top_h != info.nnum(depth):
    raise OcnnError(-3, "depad, d = %d, channel = %d: height %d != %d" %
                    (depth, channel, top_h, info.nnum(depth)))
  btm_h = info.nnum_nempty(depth)
  child = _prop_view(octree, info, CHILD, depth, top_h, torch.int32)
  out = torch.zeros(1, channel, btm_h, 1, dtype=data_in.dtype, device=data_in.device)
  _lib.call("ocnn_pad_backward", _ptr(out), btm_h, channel, _ptr(data_in), top_h, _ptr(child),
            _dtype_code(data_in), _stream())
  return out


def octree_max_pool(data_in, octree, depth):
  """pytorch/cpp/octree_pool.cpp:6-34: `depth` is the input depth; returns (pooled, mask)."""
  info = octree_info(octree)
  data_in = data_in.contiguous()
  channel, btm_h = data_in.size(1), data_in.size(2)
  if info.nnum(depth) != btm_h:
    raise OcnnError(-3, "max_pool: height %d != node_num(%d) = %d" % (btm_h, depth, info.nnum(depth)))
  if depth <= 1:
    raise OcnnError(-1, "Depth should be larger than 1")
  top_h = btm_h >> 3
  top = torch.empty(1, channel, top_h, 1, dtype=data_in.dtype, device=data_in.device)
  mask = torch.empty(1, channel, top_h, 1, dtype=torch.int32, device=data_in.device)
  _lib.call("ocnn_octree_max_pool", _ptr(top), top_h, _ptr(mask), _ptr(data_in), btm_h, channel,
            _dtype_code(data_in), _stream())
  return top, mask


def octree_max_unpool(data_in, mask, octree, depth):
  """pytorch/cpp/octree_pool.cpp:36-62: `depth` is the output depth."""
  info = octree_info(octree)
  data_in = data_in.contiguous()
  mask = mask.contiguous()
  channel, top_h = data_in.size(1), data_in.size(2)
  if top_h != info.nnum_nempty(depth - 1):
    raise OcnnError(-3, "max_unpool: height %d != node_num_nempty(%d)" % (top_h, depth - 1))
  if mask.size(1) != channel or mask.size(2) != top_h:
    raise OcnnError(-3, "max_unpool: mask shape")
  btm_h = top_h << 3
  btm = torch.empty(1, channel, btm_h, 1, dtype=data_in.dtype, device=data_in.device)
  _lib.call("ocnn_octree_max_unpool", _ptr(data_in), top_h, _ptr(mask), _ptr(btm), btm_h, channel,
            _dtype_code(data_in), _stream())
  return btm


def octree_mask_pool(data_in, mask, octree, depth):
  """pytorch/cpp/octree_pool.cpp:64-90."""
  info = octree_info(octree)
  data_in = data_in.contiguous()
  mask = mask.contiguous()
  channel, btm_h = data_in.size(1), data_in.size(2)
  top_h = mask.size(2)
  if info.nnum(depth) != btm_h or top_h != btm_h >> 3:
    raise OcnnError(-3, "mask_pool: height mismatch")
  top = torch.empty(1, channel, top_h, 1, dtype=data_in.dtype, device=data_in.device)
  _lib.call("ocnn_octree_mask_pool", _ptr(top), top_h, _ptr(mask), _ptr(data_in), btm_h, channel,
            _dtype_code(data_in), _stream())
  return top


# ---- keys ----------------------------------------------------------------------------------------------
def octree_encode_key(xyz):
  """pytorch/cpp/octree_key.cpp:11-29: int16 [N,4] (x,y,z,id) -> int64 [N] (bit copy)."""
  if xyz.dim() != 2 or xyz.size(1) != 4:
    raise OcnnError(-1, "The input must be [N, 4]")
  return xyz.contiguous().to(torch.int16).view(torch.int64).reshape(-1).clone()


def octree_decode_key(key):
  """pytorch/cpp/octree_key.cpp:31-47."""
  if key.dim() != 1:
    raise OcnnError(-1, "The dim of input tensor must be 1.")
  return key.contiguous().view(torch.int16).reshape(-1, 4).clone()


def _key_op(fn, t, depth):
  t = t.contiguous()
  if t.numel() < 1:
    raise OcnnError(-1, "The numel of the input tensor must be larger than 1.")
  src = _to_dev(t)
  out = torch.empty_like(src)
  _lib.call(fn, _ptr(out), _ptr(src), src.numel(), depth, _stream())
  return out.to(t.device)


def octree_xyz2key(xyz, depth):
  """pytorch/cpp/octree_key.cpp:49-64."""
  return _key_op("ocnn_xyz2key", xyz, depth)


def octree_key2xyz(key, depth):
  """pytorch/cpp/octree_key.cpp:66-81."""
  return _key_op("ocnn_key2xyz", key, depth)


def _morton_keys(octree, info, depth, nempty=False):
  """(sorted Morton keys of a depth as int64 tensor, their number); de-padded for nempty and
  converted from packed xyz where the octree stores those (pytorch/cpp/octree_key.cpp:95-124)."""
  des_h = info.nnum(depth)
  des = _prop_view(octree, info, KEY, depth, des_h, torch.int64)
  if nempty:
    ne = info.nnum_nempty(depth)
    child = _prop_view(octree, info, CHILD, depth, des_h, torch.int32)
    # keys of the non-empty nodes, in node order (the reference depads the key array)
    tmp = torch.zeros(max(ne, 1), dtype=torch.int64, device=octree.device)
    tmp[:ne] = des[child >= 0]
    des, des_h = tmp, ne
  if info.key2xyz:
    tmp = torch.empty_like(des)
    if des_h:
      _lib.call("ocnn_xyz2key", _ptr(tmp), _ptr(des), des_h, depth, _stream())
    des = tmp
  return des, des_h


def _search_key(out, keys, n_key, query, n_query, sorted_queries=False):
  """Position of each query in the sorted `keys`, -1 on a miss; many queries in a large array go
  through sample tables in the workspace (ocnn_search_key_indexed decides).  Queries that are
  sorted themselves (the keys of another octree) walk the same cache lines lane by lane and take
  the plain search, which is then the faster one."""
  if sorted_queries:
    _lib.call("ocnn_search_key", _ptr(out), _ptr(keys), n_key, _ptr(query), n_query, _stream())
    return
  L = _lib.get()
  nbytes = L.ocnn_search_key_workspace_bytes(n_key)
  ws = _workspace(nbytes + 128, "search")
  base = (ws.data_ptr() + 127) & ~127
  _lib.call("ocnn_search_key_indexed", _ptr(out), _ptr(keys), n_key, _ptr(query), n_query, C.c_void_p(base),
            C.c_size_t(nbytes), _stream())


def octree_search_key(key, octree, depth, key_is_xyz, nempty):
  """pytorch/cpp/octree_key.cpp:83-132: index of each query key at `depth`, -1 on a miss."""
  octree = _to_dev(octree)
  info = octree_info(octree)
  key = _to_dev(key.contiguous())
  n_query = key.numel()
  if n_query < 1:
    raise OcnnError(-1, "The numel of the input tensor must be larger than 1.")
  if key_is_xyz:
    tmp = torch.empty_like(key)
    _lib.call("ocnn_xyz2key", _ptr(tmp), _ptr(key), n_query, depth, _stream())
    key = tmp
  des, des_h = _morton_keys(octree, info, depth, nempty)
  out = torch.empty(n_query, dtype=torch.int32, device=octree.device)
  _search_key(out, des, des_h, key, n_query)
  return out


# ---- row gathers and trilinear stencils ---------------------------------------------------------
def octree_gather(data, index):
  """octree_gather_gpu (octree/octree/octree_nn.h:204-207): data [1,C,H,1], index int32 [H'] ->
  [1,C,H',1] with row h = data row index[h], or zero where index[h] is -1."""
  data, index = data.contiguous(), _to_dev(index.contiguous().int())
  out = torch.empty((1, data.size(1), index.numel(), 1), dtype=data.dtype, device=data.device)
  _lib.call("ocnn_octree_gather", _ptr(out), index.numel(), data.size(1), _ptr(data), data.size(2), _ptr(index),
            _dtype_code(data), _stream())
  return out


def octree_gatherbk(grad, index, height):
  """octree_gatherbk_gpu (octree_nn.h:208-211), the adjoint of octree_gather: grad [1,C,H',1] is
  added into [1,C,height,1] at the rows `index` names (a row may be named many times)."""
  grad, index = grad.contiguous(), _to_dev(index.contiguous().int())
  if grad.dtype != torch.float32:
    raise TypeError("octree_gatherbk is fp32")
  channel, top_h = grad.size(1), grad.size(2)
  out = torch.empty((1, channel, height, 1), dtype=grad.dtype, device=grad.device)
  ws_bytes = _lib.get().ocnn_octree_gatherbk_workspace_bytes(channel, height, top_h)
  ws = _workspace(ws_bytes + 256, "gather") if ws_bytes else None
  base = ((ws.data_ptr() + 255) & ~255) if ws is not None else 0
  _lib.call("ocnn_octree_gatherbk", _ptr(grad), top_h, channel, _ptr(out), height, _ptr(index), C.c_void_p(base),
            C.c_size_t(ws_bytes), _stream())
  return out


def octree_mask(data, label, mask):
  """octree_mask_gpu (octree_nn.h:217-218): the rows of data [1,C,H,1] whose label equals `mask`
  become zero."""
  data, label = data.contiguous(), _to_dev(label.contiguous().int())
  if data.dtype != torch.float32:
    raise TypeError("octree_mask is fp32")
  if label.numel() != data.size(2):
    raise OcnnError(-3, "octree_mask: %d labels for %d rows" % (label.numel(), data.size(2)))
  out = torch.empty_like(data)
  _lib.call("ocnn_octree_mask", _ptr(out), _ptr(data), _ptr(label), data.size(2), int(mask), C.c_int64(data.numel()),
            _stream())
  return out


def octree_bilinear_neigh(octree, depth):
  """bilinear_neigh_gpu (octree_nn.h:170-173): int32 [nnum(depth + 1), 8], for every node of
  level depth + 1 the nodes of level `depth` in the 8 cells around its centre, nearest first
  (weights 27, 9, 9, 9, 3, 3, 3, 1 of 64), -1 where there is none."""
  octree = _to_dev(octree)
  info = octree_info(octree)
  if not 1 <= depth < info.depth:
    raise ValueError("depth %d outside [1, %d)" % (depth, info.depth))
  out = torch.empty((info.nnum(depth + 1), 8), dtype=torch.int32, device=octree.device)
  neigh = _prop_view(octree, info, NEIGH, depth, info.nnum(depth) * 8, torch.int32)
  child = _prop_view(octree, info, CHILD, depth, info.nnum(depth), torch.int32)
  _lib.call("ocnn_bilinear_neigh", _ptr(out), _ptr(neigh), _ptr(child), info.nnum(depth), _stream())
  return out


def octree_bilinear_xyz(xyz, depth_from, depth_to):
  """bilinear_xyz_gpu (octree_nn.h:174-177): packed coordinates int64 [N] of cells of level
  `depth_from` -> (int64 [N, 8] cells of the coarser level `depth_to` around each centre,
  nearest first; float32 [N, 3] weight of the nearer cell per axis)."""
  xyz = _to_dev(xyz.contiguous())
  n = xyz.numel()
  cells = torch.empty((n, 8), dtype=torch.int64, device=xyz.device)
  fracs = torch.empty((n, 3), dtype=torch.float32, device=xyz.device)
  _lib.call("ocnn_bilinear_xyz", _ptr(cells), _ptr(fracs), depth_to, _ptr(xyz), depth_from, n, _stream())
  return cells, fracs


# ---- feature transfer ---------------------------------------------------------------------------
def octree_align(src_data, src_octree, des_octree, depth, add_to=None):
  """pytorch/cpp/octree_align.cpp:9-61 -> [des_data [1,C,des_h,1], idx int32 [src_h]]: the
  features of `src_octree`'s nodes moved to the nodes of `des_octree` with the same key.
  add_to: a contiguous fp32 [1,C,des_h,1] tensor that the moved features are added to in place
  (`x + octree_align(...)[0]` of the decoder loop, pytorch/ocnn/ounet.py:109-111, in one pass);
  it is returned as des_data."""
  src_octree, des_octree = _to_dev(src_octree), _to_dev(des_octree)
  sinfo, dinfo = octree_info(src_octree), octree_info(des_octree)
  src_data = src_data.contiguous()
  if src_data.dtype != torch.float32:
    raise TypeError("octree_align is fp32")
  channel, src_h = src_data.size(1), src_data.size(2)
  if sinfo.nnum(depth) != src_h:
    raise OcnnError(-3, "octree_align: %d rows, the source octree has %d nodes at depth %d"
                    % (src_h, sinfo.nnum(depth), depth))
  src_key, _ = _morton_keys(src_octree, sinfo, depth)
  des_key, des_h = _morton_keys(des_octree, dinfo, depth)
  idx = torch.empty(src_h, dtype=torch.int32, device=src_data.device)
  _search_key(idx, des_key, des_h, src_key, src_h, sorted_queries=True)
  if add_to is not None:
    if (add_to.dtype != torch.float32 or not add_to.is_contiguous() or add_to.device != src_data.device
        or add_to.numel() != channel * des_h or add_to.dim() < 2 or add_to.size(1) != channel):
      raise OcnnError(-3, "octree_align: add_to must be a contiguous fp32 [1, %d, %d, 1] tensor" % (channel, des_h))
    _lib.call("ocnn_align_forward_add", _ptr(add_to), des_h, channel, _ptr(src_data), src_h, _ptr(idx), _stream())
    return [add_to, idx]
  out = torch.empty(1, channel, des_h, 1, dtype=torch.float32, device=src_data.device)
  inverse = torch.empty(max(des_h, 1), dtype=torch.int32, device=src_data.device)
  _lib.call("ocnn_align_forward_ws", _ptr(out), des_h, channel, _ptr(src_data), src_h, _ptr(idx), _ptr(inverse),
            _stream())
  return [out, idx]


def octree_align_grad(des_grad, idx):
  """pytorch/cpp/octree_align.cpp:63-83."""
  des_grad = des_grad.contiguous()
  channel, des_h, src_h = des_grad.size(1), des_grad.size(2), idx.numel()
  out = torch.empty(1, channel, src_h, 1, dtype=torch.float32, device=des_grad.device)
  _lib.call("ocnn_align_backward", _ptr(des_grad), des_h, channel, _ptr(out), src_h, _ptr(idx.contiguous()),
            _stream())
  return out


def octree_interp_pts(data, octree, depth, pts, method="linear", nempty=False):
  """octree_nearest_pts / octree_trilinear_pts (pytorch/ocnn/modules.py:209-275) fused:
  data [1,C,H,1] at `depth`, pts [N,4] = (x, y, z in [0, 2^depth], batch id)
  -> ([1,C,N,1], idx int32 [N,K], weight fp32 [N,K]) with K = 1 (nearest) or 8 (linear)."""
  if method not in ("nearest", "linear"):
    raise ValueError(method)
  octree = _to_dev(octree)
  info = octree_info(octree)
  data = data.contiguous()
  pts = _to_dev(pts).to(torch.float32).contiguous()
  if data.dtype != torch.float32 or pts.dim() != 2 or pts.size(1) != 4:
    raise TypeError("fp32 data [1,C,H,1] and points [N,4] expected")
  channel, H, n = data.size(1), data.size(2), pts.size(0)
  key, n_key = _morton_keys(octree, info, depth, nempty)
  if H != n_key:
    raise OcnnError(-3, "interpolation: %d rows, the octree has %d %snodes at depth %d"
                    % (H, n_key, "non-empty " if nempty else "", depth))
  K = 1 if method == "nearest" else 8
  out = torch.empty(1, channel, n, 1, dtype=torch.float32, device=data.device)
  idx = torch.empty(n, K, dtype=torch.int32, device=data.device)
  weight = torch.empty(n, K, dtype=torch.float32, device=data.device)
  ws_bytes = _lib.get().ocnn_octree_interp_workspace_bytes(channel, H) if n * K >= H // 2 else 0
  ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=data.device)
  _lib.call("ocnn_octree_interp_ws", _ptr(out), _ptr(data), channel, H, _ptr(key), n_key, _ptr(pts), n, depth,
            int(method == "linear"), _ptr(idx), _ptr(weight), _ptr(ws) if ws_bytes else C.c_void_p(0),
            C.c_size_t(ws_bytes), _stream())
  return out, idx, weight


def octree_interp_pts_grad(grad_out, idx, weight, H, method="linear"):
  grad_out = grad_out.contiguous()
  channel, n = grad_out.size(1), grad_out.size(2)
  out = torch.empty(1, channel, H, 1, dtype=torch.float32, device=grad_out.device)
  K = 1 if method == "nearest" else 8
  ws_bytes = (_lib.get().ocnn_octree_interp_backward_workspace_bytes(channel, H, n, int(method == "linear"))
              if n * K >= H // 2 else 0)
  ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=grad_out.device)
  _lib.call("ocnn_octree_interp_backward_ws", _ptr(out), _ptr(grad_out), channel, H, n, int(method == "linear"),
            _ptr(idx), _ptr(weight), _ptr(ws) if ws_bytes else C.c_void_p(0), C.c_size_t(ws_bytes), _stream())
  return out


# ---- point-cloud properties (pytorch/cpp/points_property.cpp) ----------------------------------
_PT_PROPS = {"xyz": 0, "xyzi": 0, "normal": 1, "feature": 2, "label": 3}


def _points_array(points, prop):
  hdr = _points_hdr(points)
  ints = hdr[16:].view(np.int32)
  t = _PT_PROPS[prop]
  npt, flags, ch, off = int(ints[0]), int(ints[1]), int(ints[2 + t]), int(ints[10 + t])
  if not (flags & (1 << t)) or ch == 0:
    return None, npt, 0, off
  return points[off:off + 4 * npt * ch].view(torch.float32).view(npt, ch), npt, ch, off


def points_property(points, property):
  """pytorch/cpp/points_property.cpp:92-109 -> float32 [pt_num, channel] (None if absent)."""
  arr, _, _, _ = _points_array(points, property)
  return None if arr is None else arr.clone()


def points_batch_property(points_list, property):
  """pytorch/cpp/points_property.cpp:111-160: the property of several clouds stacked; 'xyzi'
  appends the index of the cloud as a fourth column."""
  parts = []
  for i, p in enumerate(points_list):
    arr, npt, _, _ = _points_array(p, property)
    if arr is None:
      raise OcnnError(-1, "The specified property does not exist.")
    if property == "xyzi":
      arr = torch.cat([arr, torch.full((npt, 1), float(i), dtype=torch.float32, device=arr.device)], dim=1)
    parts.append(arr)
  return torch.cat(parts, dim=0)


def points_set_property(points, data, property):
  """pytorch/cpp/points_property.cpp:58-90: a copy of the cloud with one property replaced."""
  arr, npt, ch, off = _points_array(points, property)
  if arr is None:
    raise OcnnError(-1, "The property does not exist.")
  if data.dim() != 2 or data.size(0) != npt or data.size(1) != ch:
    raise OcnnError(-3, "points_set_property: [%d, %d] expected" % (npt, ch))
  out = points.clone()
  out[off:off + 4 * npt * ch] = data.to(torch.float32).contiguous().view(-1).view(torch.uint8).to(points.device)
  out._ocnn_points_info = _points_hdr(points)
  return out


# ---- growth ----------------------------------------------------------------------------------------------
def octree_new(batch_size, channel, node_dis, adaptive_layer=0):
  """pytorch/cpp/octree_grow.cpp:110-153."""
  raw = np.zeros(INFO_BYTES, np.uint8)
  _lib.call("ocnn_octree_new_info", batch_size, channel, int(node_dis), adaptive_layer,
            C.c_void_p(raw.ctypes.data))
  info = _Info(raw)
  out = torch.empty(info.size(), dtype=torch.uint8, device=_dev())
  _lib.call("ocnn_octree_new", _ptr(out), info.p, _stream())
  out._ocnn_info = info
  return out


def octree_grow(octree_in, target_depth, full_octree):
  """pytorch/cpp/octree_grow.cpp:13-54."""
  octree_in = _to_dev(octree_in)
  iin = octree_info(octree_in)
  raw = np.zeros(INFO_BYTES, np.uint8)
  _lib.call("ocnn_octree_grow_info", iin.p, target_depth, int(full_octree), C.c_void_p(raw.ctypes.data))
  info = _Info(raw)
  out = torch.empty(info.size(), dtype=torch.uint8, device=octree_in.device)
  _lib.call("ocnn_octree_grow", _ptr(out), info.p, _ptr(octree_in), iin.p, target_depth,
            int(full_octree), _stream())
  out._ocnn_info = info
  return out


def octree_update(octree_in, label_in, depth, split, inplace=False):
  """pytorch/cpp/octree_grow.cpp:164-190: children[depth] from the split labels.
  inplace=True rewrites `octree_in` itself and returns it (for a caller that owns the tensor and
  drops the old state anyway, as the decoder loop does with what octree_grow just returned): the
  clone of the whole blob is saved.  What this module keeps with the tensor is dropped."""
  octree_in = _to_dev(octree_in)
  iin = octree_info(octree_in)
  info = _Info(iin.raw)
  if inplace:
    label = _to_dev(label_in.contiguous().to(torch.int32))
    n = label.numel()
    sb = _lib.get().ocnn_octree_update_scratch_bytes(n)
    ws = _workspace(sb + 256, "update")
    base = (ws.data_ptr() + 255) & ~255
    _lib.call("ocnn_octree_update", _ptr(octree_in), info.p, _ptr(label), n, depth, split, C.c_void_p(base),
              C.c_size_t(sb), _stream())
    forget_cached(octree_in)
    octree_in._ocnn_info = _Info(info.raw)
    return octree_in
  out = torch.empty_like(octree_in)     # (the library copies the blob while the host waits for the count)
  label = _to_dev(label_in.contiguous().to(torch.int32))
  n = label.numel()
  sb = _lib.get().ocnn_octree_update_scratch_bytes(n)
  ws = _workspace(sb + 256, "update")
  base = (ws.data_ptr() + 255) & ~255
  _lib.call("ocnn_octree_update_copy", _ptr(out), _ptr(octree_in), info.p, _ptr(label), n, depth, split,
            C.c_void_p(base), C.c_size_t(sb), _stream())
  out._ocnn_info = _Info(info.raw)
  return out
