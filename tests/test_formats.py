"""File formats around the path: `.octree` / `.points` files are the serialized blobs, and a file
from a 32-bit-key build is upgraded (upgrade_key64, octree/octree/transform_octree.cpp:433-497).
The conversion is host code, so the library's version is tested here without a GPU."""
import importlib
import os

import numpy as np
import pytest

from conftest import GOLDEN
from oracle.checker import OctreeBlob, make_points_blob


@pytest.fixture(scope="module")
def samples32():
  z = np.load(os.path.join(GOLDEN, "octree_samples_key32.npz"))
  return {k: z[k] for k in z.files}


@pytest.fixture(scope="module")
def nn():
  lib = importlib.import_module("o-cnn_amd.lib")
  if not os.path.exists(lib.SO_PATH):
    lib.build()
  return importlib.import_module("o-cnn_amd.nn")


def downgrade(blob64):
  """The 32-bit-key layout of a 64-bit blob without neighbours whose keys fit (the inverse of the
  upgrade, written from the format description octree_info.cpp:254-268); like the reference's
  own 32-bit samples, the payload follows the 716-byte header without padding."""
  b = OctreeBlob(blob64)
  hdr = blob64[:716].copy()
  hdr[:12] = np.frombuffer(b"_OCTREE_1.0_", np.uint8)
  dis = b.ptr_dis.copy()
  nkeys = (int(dis[1]) - 720) // 8
  keys = blob64[720:720 + 8 * nkeys].view(np.uint64)
  if b.key2xyz:
    k32 = keys.view(np.uint16).reshape(-1, 4).astype(np.uint8).reshape(-1).view(np.uint32)
  else:
    assert keys.max() < 2 ** 32
    k32 = keys.astype(np.uint32)
  shrink = 4 * nkeys
  new_dis = dis.copy()
  new_dis[0:7] -= 4
  new_dis[1:7] -= shrink
  hdr[652:716] = new_dis.view(np.uint8)
  return np.concatenate([hdr, k32.view(np.uint8), blob64[int(dis[1]):]])


def test_oracle_upgrades_the_reference_samples(orc, samples, samples32):
  for name, raw in samples32.items():
    assert bytes(raw[:12]) == b"_OCTREE_1.0_"
    assert np.array_equal(orc.upgrade_key64(raw), samples[name]), name
    assert np.array_equal(downgrade(samples[name]), raw), name   # pins the test's own helper


@pytest.mark.parametrize("kw", [dict(), dict(key2xyz=True), dict(node_dis=True, split_label=True),
                                dict(adaptive=True, node_dis=True, split_label=True, adp_depth=3)])
def test_oracle_upgrade_vs_compiled_reference(orc, ref, synthetic, kw):
  p, n, _ = synthetic.shape_cloud(3000, 7)
  lab = (np.arange(3000) % 5).astype(np.float32)
  blob = orc.points2octree(make_points_blob(p, n, None, lab), 6, 2, **kw)
  raw = downgrade(blob)
  assert np.array_equal(orc.upgrade_key64(raw), blob)
  assert np.array_equal(ref.upgrade_key64(raw), blob)


def test_library_upgrade_and_files(orc, nn, samples, samples32, synthetic, tmp_path):
  for name, raw in samples32.items():
    assert np.array_equal(nn.upgrade_key64(raw).numpy(), samples[name]), name
  # a .octree file from a 32-bit build is upgraded on the way in; a 64-bit one is returned as is
  f32, f64 = str(tmp_path / "a.octree"), str(tmp_path / "b.octree")
  samples32["octree_2"].tofile(f32)
  assert np.array_equal(nn.read_octree(f32).numpy(), samples["octree_2"])
  import torch
  nn.write_octree(torch.from_numpy(samples["octree_3"]), f64)
  assert np.array_equal(nn.read_octree(f64).numpy(), samples["octree_3"])
  p, n, _ = synthetic.shape_cloud(500, 1)
  pb = make_points_blob(p, n)
  fp = str(tmp_path / "c.points")
  nn.write_points(torch.from_numpy(pb), fp)
  back = nn.read_points(fp)
  assert np.array_equal(back.numpy(), pb) and np.array_equal(back._ocnn_points_info, pb[:88])
  # errors are codes, not aborts
  bad = samples32["octree_1"].copy()
  bad[0] = ord("X")
  with pytest.raises(nn.OcnnError) as e:
    nn.upgrade_key64(bad)
  assert e.value.code == -6
  with pytest.raises(nn.OcnnError):
    nn.upgrade_key64(samples32["octree_1"][:800])
  open(str(tmp_path / "d.points"), "wb").write(b"nope")
  with pytest.raises(nn.OcnnError):
    nn.read_points(str(tmp_path / "d.points"))


def test_octree_samples_match_the_reference_blobs(nn, samples):
  """nn.octree_samples (pytorch/cpp/octree_samples.cpp:5-18): the package's data file holds the
  six blobs of the fixture; an unknown name raises."""
  got = nn.octree_samples(["octree_%d" % i for i in range(1, 7)])
  for i, t in enumerate(got):
    assert t.dtype.is_floating_point is False and np.array_equal(t.numpy(), samples["octree_%d" % (i + 1)])
  with pytest.raises(RuntimeError):
    nn.octree_samples(["octree_7"])
