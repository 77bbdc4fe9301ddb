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
               "octree_property"):
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
