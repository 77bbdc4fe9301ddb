"""TEST INFRASTRUCTURE -- not part of the shipped library.

numpy restatement of the reference's feature-transfer compositions, for the parity tests:
  octree_align          pytorch/cpp/octree_align.cpp:9-83 (+ align_forward/backward kernels,
                        octree/octree/octree_nn.cu:710-752)
  octree_nearest_pts    pytorch/ocnn/modules.py:209-221
  octree_trilinear_pts  pytorch/ocnn/modules.py:224-268
  octree_trilinear      pytorch/ocnn/modules.py:271-281
Key conversion and search go through the C restatement (oracle/ocnn_oracle.c).
Pinned by: the three literal cases of pytorch/test/test_octree_align.py, the literal case of
pytorch/test/test_octree_trilinear.py, reproduction of affine functions in the interior of a
full layer (closed form), and nearest == the voxel's own value at voxel centres.
"""
import numpy as np

from .checker import OctreeBlob


def morton_keys(orc, blob, depth, nempty=False):
  b = OctreeBlob(blob)
  key = b.prop("key", depth).copy()
  if nempty:
    key = key[b.prop("child", depth) >= 0]
  if b.key2xyz:
    key = orc.xyz2key(key, depth)
  return key


def octree_align(orc, src_data, src_blob, des_blob, depth):
  src_key = morton_keys(orc, src_blob, depth)
  des_key = morton_keys(orc, des_blob, depth)
  assert src_data.shape[1] == src_key.size
  idx = orc.search_key(des_key, src_key)
  des = np.zeros((src_data.shape[0], des_key.size), np.float32)
  ok = idx != -1
  des[:, idx[ok]] = src_data[:, ok]
  return des, idx


def octree_align_grad(des_grad, idx):
  out = np.zeros((des_grad.shape[0], idx.size), np.float32)
  ok = idx != -1
  out[:, ok] = des_grad[:, idx[ok]]
  return out


def _encode(xyzi):  # octree_encode_key: int16 [N,4] -> int64 (bit copy)
  return np.ascontiguousarray(xyzi.astype(np.int16)).view(np.int64).reshape(-1)


def _search(orc, key_packed, blob, depth, nempty):
  """octree_search_key(key, octree, depth, key_is_xyz=True, nempty), octree_key.cpp:83-132."""
  q = orc.xyz2key(key_packed.view(np.uint64), depth)
  return orc.search_key(morton_keys(orc, blob, depth, nempty), q)


def octree_nearest_pts(orc, data, blob, depth, pts, nempty=False):
  key = _encode(np.float32(pts))
  idx = _search(orc, key, blob, depth, nempty)
  flg = idx > -1
  out = data[:, idx * flg] * flg[None, :]
  return out.astype(np.float32)


def octree_trilinear_pts(orc, data, blob, depth, pts, nempty=False):
  pts = np.float32(pts)
  mask = np.float32([[0, 0, 0], [0, 0, 1], [0, 1, 0], [0, 1, 1], [1, 0, 0], [1, 0, 1], [1, 1, 0], [1, 1, 1]])
  masku = np.int64([0, 4294967296, 65536, 4295032832, 1, 4294967297, 65537, 4295032833])
  xyzf = pts[:, :3] - np.float32(0.5)
  xyzi = np.floor(xyzf)
  frac = xyzf - xyzi
  key = _encode(np.concatenate([xyzi, pts[:, 3:]], axis=1))
  key = (key[:, None] + masku[None, :]).reshape(-1)
  idx = _search(orc, key, blob, depth, nempty)
  flg = idx > -1
  npt = pts.shape[0]
  f = (1 - mask)[None, :, :] - frac[:, None, :]
  weight = np.abs(np.prod(f, axis=2, dtype=np.float32)).reshape(-1)
  out = np.zeros((data.shape[0], npt), np.float64)
  norm = np.zeros(npt, np.float64)
  rows = np.repeat(np.arange(npt), 8)[flg]
  np.add.at(norm, rows, weight[flg].astype(np.float64))
  for c in range(data.shape[0]):
    np.add.at(out[c], rows, weight[flg].astype(np.float64) * data[c, idx[flg]])
  return (out / (norm + 1e-10)[None, :]).astype(np.float32)


def octree_trilinear(orc, data, blob, depth, target_depth):
  b = OctreeBlob(blob)
  key = b.prop("key", target_depth).copy()
  xyz = key if b.key2xyz else orc.key2xyz(key, target_depth)
  xyz = np.ascontiguousarray(xyz).view(np.int16).reshape(-1, 4).astype(np.float32)
  scale = np.float32(2.0 ** (depth - target_depth))
  xyz = (xyz + np.float32([0.5, 0.5, 0.5, 0.0])) * np.float32([scale, scale, scale, 1.0])
  return octree_trilinear_pts(orc, data, blob, depth, xyz)
