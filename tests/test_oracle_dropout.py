"""octree_dropout (octree/octree/transform_octree.cpp:286-431): the C restatement against the
compiled reference on the very flags the reference drew (its engine is seeded with the clock's
second; the shim replays engine and distribution for that second), plus what the definition
fixes without either."""
import numpy as np
import pytest

from oracle.checker import OctreeBlob
from test_oracle_scan import CASES, sphere_octree


@pytest.mark.parametrize("case", range(len(CASES)))
def test_dropout_vs_compiled_reference(orc, ref, case):
  rng = np.random.default_rng(1200 + case)
  for trial in range(5):
    depth = int(rng.integers(4, 7))
    blob = sphere_octree(orc, int(rng.integers(500, 6000)), 10 * case + trial, depth, **CASES[case])
    if trial == 3:
      blob = orc.octree_batch([blob, sphere_octree(orc, 900, 77 + case, depth, **CASES[case])])
    dd = int(rng.integers(1, depth + 1))
    ratio = float(rng.choice([0.0, 0.2, 0.5, 0.9, 1.0]))
    b, flags = ref.octree_dropout_drawn(blob, dd, ratio)
    a = orc.octree_dropout(blob, flags, dd)
    assert np.array_equal(a, b), (case, trial, dd, ratio)
    if 0.0 < ratio < 1.0:
      assert 0 < flags.sum() < flags.size


def test_dropout_definition(orc):
  """No flag set: the octree comes back unchanged.  Every flag set at level dd: nothing is left
  below, the dropped nodes keep their child entries (transform_octree.cpp:422-425) and the
  non-empty count of level dd is zero.  Mixed flags: level d+1 holds exactly the children of
  the kept non-empty nodes, in order, with their keys, features and labels."""
  blob = sphere_octree(orc, 4000, 5, 5, node_feature=True, split_label=True)
  src = OctreeBlob(blob)
  for dd in (2, 3, 5):
    same = orc.octree_dropout(blob, np.zeros(src.nnum[dd], np.uint8), dd)
    assert np.array_equal(same, blob)
    none = OctreeBlob(orc.octree_dropout(blob, np.ones(src.nnum[dd], np.uint8), dd))
    assert list(none.nnum[:dd + 1]) == list(src.nnum[:dd + 1]) and not any(none.nnum[dd + 1:6])
    assert np.array_equal(none.prop("child", dd), src.prop("child", dd)) and none.nnum_nempty[dd] == 0
  rng = np.random.default_rng(0)
  dd = 3
  flags = (rng.uniform(size=src.nnum[dd]) < 0.4).astype(np.uint8)
  out = OctreeBlob(orc.octree_dropout(blob, flags, dd))
  keep = {dd: flags == 0}
  for d in range(dd + 1, 6):
    parent = np.full(src.nnum[d], -1)
    c = src.prop("child", d - 1)
    parent[(c[c >= 0][:, None] * 8 + np.arange(8)).reshape(-1)] = np.repeat(np.nonzero(c >= 0)[0], 8)
    keep[d] = keep[d - 1][parent]
    assert out.nnum[d] == keep[d].sum()
    assert np.array_equal(out.prop("key", d), src.prop("key", d)[keep[d]])
    assert np.array_equal(out.prop("feature", d), src.prop("feature", d)[:, keep[d]])
    assert np.array_equal(out.prop("split", d), src.prop("split", d)[keep[d]])
    oc_, sc = out.prop("child", d), src.prop("child", d)[keep[d]]
    assert np.array_equal(oc_ >= 0, sc >= 0) and np.array_equal(oc_[oc_ >= 0], np.arange((sc >= 0).sum()))
    assert out.nnum_nempty[d] == (sc >= 0).sum()
  cd, sd = out.prop("child", dd), src.prop("child", dd)
  live = (flags == 0) & (sd >= 0)
  assert np.array_equal(cd[live], np.arange(live.sum())) and np.array_equal(cd[~live], sd[~live])
  assert out.nnum_nempty[dd] == live.sum() and out.nnum[dd + 1] == 8 * live.sum()
