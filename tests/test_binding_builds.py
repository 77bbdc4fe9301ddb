"""The ATen side of the operators (o-cnn_amd/binding/ocnn_aten.cpp, the bodies that replace
pytorch/cpp/*.cpp) is a real Python module, linked against libocnn_hip.so.  Without a GPU: it
loads, registers the reference's names (pytorch/cpp/pybind.cpp:3-49), and keeps one host copy of
an octree's header per blob TENSOR: not per address (the allocator hands addresses out again)
and not across in-place rewrites."""
import importlib

import numpy as np
import pytest
import torch


@pytest.fixture(scope="module")
def aten():
  lib = importlib.import_module("o-cnn_amd.lib")
  try:
    return lib.aten()
  except ImportError:
    import subprocess, os
    subprocess.check_call(["make", "-s", "-C", os.path.join(lib.HERE, "binding")])
    return lib.aten()


def test_registers_the_reference_names(aten):
  for name in ("octree_conv", "octree_deconv", "octree_conv_grad", "octree_deconv_grad", "octree2col", "col2octree",
               "octree_pad", "octree_depad", "octree_max_pool", "octree_max_unpool", "octree_mask_pool",
               "octree_xyz2key", "octree_key2xyz", "octree_search_key", "octree_new", "octree_grow", "octree_update",
               "octree_property", "octree_batch", "octree_samples", "points2octree", "octree_set_property",
               "transform_points", "clip_points", "normalize_points", "bounding_sphere", "octree_encode_key",
               "octree_decode_key", "octree_scan", "octree_align", "octree_align_grad", "points_batch_property",
               "points_property", "points_set_property", "points_new"):
    assert callable(getattr(aten, name)), name


def test_header_copy_follows_the_tensor_not_the_address(aten, samples):
  a, b = samples["octree_1"], samples["octree_2"]
  assert not np.array_equal(a[:716], b[:716])
  n = max(a.size, b.size)
  buf = np.zeros(n, np.uint8)
  buf[:a.size] = a
  t1 = torch.from_numpy(buf)
  assert np.array_equal(aten.octree_header(t1).numpy(), a[:716])
  # another tensor object over the very same bytes' address, with another octree in them
  del t1
  buf[:] = 0
  buf[:b.size] = b
  t2 = torch.from_numpy(buf)
  assert np.array_equal(aten.octree_header(t2).numpy(), b[:716])
  # an in-place rewrite through torch (version counter) is seen as well
  t2.copy_(torch.from_numpy(np.concatenate([a, np.zeros(n - a.size, np.uint8)])))
  assert np.array_equal(aten.octree_header(t2).numpy(), a[:716])
  # repeated calls hit the copy
  assert np.array_equal(aten.octree_header(t2).numpy(), a[:716])


def test_header_copies_of_dead_tensors_are_dropped(aten, samples):
  blob = samples["octree_3"]
  base = aten.octree_header_copies()
  live = [torch.from_numpy(blob.copy()) for _ in range(5)]
  for t in live:
    aten.octree_header(t)
  assert aten.octree_header_copies() == base + 5
  del live, t
  assert aten.octree_header_copies() == base


def test_rejects_what_is_not_an_octree(aten):
  with pytest.raises(RuntimeError):
    aten.octree_header(torch.zeros(100, dtype=torch.uint8))
  with pytest.raises(RuntimeError):
    aten.octree_header(torch.zeros(2000, dtype=torch.uint8))   # no magic string


def test_host_side_operators_without_a_gpu(aten, samples):
  """The operators of the binding that move bytes only (point-cloud arrays, key bit copies, the
  sample octrees, octree_set_property) work on host tensors as the reference's do
  (pytorch/cpp/points_property.cpp:38-165, octree_key.cpp:11-47, octree_samples.cpp:5-18,
  octree_property.cpp:308-325)."""
  from oracle.checker import OctreeBlob, make_points_blob
  rng = np.random.default_rng(3)
  n = 257
  pts, nrm = rng.standard_normal((n, 3)).astype(np.float32), rng.standard_normal((n, 3)).astype(np.float32)
  feat, lab = rng.standard_normal((n, 4)).astype(np.float32), rng.integers(0, 9, (n, 1)).astype(np.float32)
  T = torch.from_numpy
  p = aten.points_new(T(pts), T(nrm), T(feat), T(lab))
  assert np.array_equal(p.numpy(), make_points_blob(pts, nrm, feat, lab))
  q = aten.points_new(T(pts), torch.zeros(0), torch.zeros(0), T(lab))
  assert np.array_equal(q.numpy(), make_points_blob(pts, labels=lab))
  assert np.array_equal(aten.points_property(p, "feature").numpy(), feat)
  assert np.array_equal(aten.points_property(q, "label").numpy(), lab) and aten.points_property(q, "normal") is None
  xyzi = aten.points_batch_property([p, q], "xyzi").numpy()
  assert xyzi.shape == (2 * n, 4) and np.array_equal(xyzi[:, :3], np.concatenate([pts, pts]))
  assert np.array_equal(xyzi[:, 3], np.repeat([0.0, 1.0], n).astype(np.float32))
  with pytest.raises(RuntimeError):
    aten.points_batch_property([p, q], "normal")
  with pytest.raises(RuntimeError):
    aten.points_property(p, "colour")
  p2 = aten.points_set_property(p, T(2 * feat), "feature")
  assert np.array_equal(p2.numpy(), make_points_blob(pts, nrm, 2 * feat, lab)) and np.array_equal(
      aten.points_property(p, "feature").numpy(), feat)
  xyz = T(rng.integers(0, 1 << 15, (100, 4)).astype(np.int16))
  key = aten.octree_encode_key(xyz)
  x = xyz.numpy().astype(np.int64) & 0xffff
  assert np.array_equal(key.numpy(), x[:, 0] | x[:, 1] << 16 | x[:, 2] << 32 | x[:, 3] << 48)
  assert torch.equal(aten.octree_decode_key(key), xyz)
  names = sorted(samples)
  for t, name in zip(aten.octree_samples(names), names):
    assert np.array_equal(t.numpy(), samples[name]), name
  with pytest.raises(RuntimeError):
    aten.octree_samples(["octree_0"])
  blob = samples["octree_1"]
  b = OctreeBlob(blob)
  d = b.depth
  old = b.prop("feature", d) if hasattr(b, "prop") else None
  count = aten.octree_property(T(blob.copy()), "feature", d).numel()
  new = torch.arange(count, dtype=torch.float32)
  out = aten.octree_set_property(T(blob.copy()), new, d)
  assert torch.equal(aten.octree_property(out, "feature", d).reshape(-1), new)
  diff = np.nonzero(out.numpy() != blob)[0]
  assert diff.size and diff.max() - diff.min() < 4 * count   # only the feature array of that depth changed
  with pytest.raises(RuntimeError):
    aten.octree_set_property(T(blob.copy()), new[:-1], d)
