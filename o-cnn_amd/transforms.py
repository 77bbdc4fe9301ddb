"""Input pipeline of the reference on the device (pytorch/ocnn/transforms.py:6-148): bounding
sphere -> normalisation into [-1, 1] -> random rotation / scale / jitter -> clipping -> octree,
and the batch merge.  Class names, constructor arguments and results follow the reference; the
point cloud stays on the GPU from the first step to the last, and `collate_octrees` builds the
octrees of a plain batch in one device pass when the samples carry their points instead of
octrees (`build_in_collate=True`).

The random draws are the reference's (numpy's global generator: an integer number of rotation
steps per axis, three uniform scales, three uniform jitters), isolated in `draw_distortion` so a
caller or a test can fix them."""
import numpy as np
import torch

from . import nn as F

_DEG = 3.14159265 / 180.0       # the reference's constant (transforms.py:83)


class Points2Octree:
  """transforms.py:6-32."""

  def __init__(self, depth, full_depth=2, node_dis=False, node_feature=False, split_label=False,
               adaptive=False, adp_depth=4, th_normal=0.1, th_distance=2.0, extrapolate=False,
               save_pts=False, key2xyz=False, **kwargs):
    self.args = (depth, full_depth, node_dis, node_feature, split_label, adaptive, adp_depth,
                 th_normal, th_distance, extrapolate, save_pts, key2xyz)

  def __call__(self, points):
    return F.points2octree(points, *self.args)

  def batch(self, points_list):
    """The octrees of several clouds, merged: one device pass for plain octrees."""
    return F.points2octree_batch(points_list, *self.args)


class NormalizePoints:
  """transforms.py:35-58: scale by the bounding sphere (computed, or given by radius / center)."""

  def __init__(self, bsphere="sphere", radius=-1.0, center=(-1.0,), **kwargs):
    self.bsphere, self.radius, self.center = bsphere, radius, center

  def __call__(self, points):
    if self.radius < 0:
      sphere = F.bounding_sphere(points, self.bsphere)
      radius, center = sphere[0], sphere[1:]
    else:
      radius, center = self.radius, self.center
    return F.normalize_points(points, radius, center)


class Distortion(tuple):
  """(rotation angles in radians, per-axis scale, per-axis shift) of one augmentation."""
  identity = None

  def __new__(cls, rotation, scale, shift):
    return super().__new__(cls, (list(rotation), list(scale), list(shift)))


Distortion.identity = Distortion([0.0] * 3, [1.0] * 3, [0.0] * 3)


def draw_distortion(angle, scale, jitter, angle_interval, uniform_scale):
  """One random augmentation.  It consumes numpy's global generator exactly as the reference
  does (transforms.py:80-98), so a seeded run reproduces the reference's clouds: one int32
  `randint` per axis (a whole number of `angle_interval` steps within +-angle degrees), one
  `uniform` of three scales in [1 - scale, 1 + scale] (only the first is used when the scale is
  uniform), one `uniform` of three shifts in [-jitter, jitter]."""
  def steps(axis):
    reach = angle[axis] // angle_interval[axis]
    return int(np.random.randint(low=-reach, high=reach + 1, dtype=np.int32))
  rotation = [steps(axis) * angle_interval[axis] * _DEG for axis in range(3)]
  scales = np.random.uniform(low=1 - scale, high=1 + scale, size=3).tolist()
  shifts = np.random.uniform(low=-jitter, high=jitter, size=3).tolist()
  return Distortion(rotation, scales[:1] * 3 if uniform_scale else scales, shifts)


class TransformPoints:
  """transforms.py:61-108: the augmentation of a cloud that lies in [-1, 1]^3 and the clip back
  into that box.  Returns (points, inbox_mask).  `drawn` fixes the augmentation."""

  def __init__(self, distort, angle=(0, 180, 0), scale=0.25, jitter=0.25, offset=0.0,
               angle_interval=(1, 1, 1), uniform_scale=False, normal_axis="", **kwargs):
    self.distort, self.offset, self.normal_axis = distort, offset, normal_axis
    self.ranges = (list(angle), scale, jitter, list(angle_interval), uniform_scale)

  def __call__(self, points, drawn=None):
    if drawn is None:
      drawn = draw_distortion(*self.ranges) if self.distort else Distortion.identity
    moved = F.transform_points(points, *drawn, self.offset, self.normal_axis)
    return tuple(F.clip_points(moved, [-1.0] * 3, [1.0] * 3))


class TransformCompose:
  """transforms.py:111-130: normalise -> transform + clip -> octree.  With `octree=False` a
  sample keeps its points only and `collate_octrees(..., points2octree=...)` builds the whole
  batch in one pass."""

  def __init__(self, flags, octree=True):
    self.flags, self.octree = flags, octree
    self.normalize_points = NormalizePoints(**flags)
    self.transform_points = TransformPoints(**flags)
    self.points2octree = Points2Octree(**flags)

  def __call__(self, points, idx=0):
    points, inbox_mask = self.transform_points(self.normalize_points(points))
    sample = {"points": points, "inbox_mask": inbox_mask}
    if self.octree:
      sample["octree"] = self.points2octree(points)
    return sample


def collate_octrees(batch, points2octree=None):
  """transforms.py:133-148: a list of samples -> one dict of lists; every entry whose key names
  an octree is merged with octree_batch, labels additionally become the tensor `label`.  If the
  samples carry no octree and `points2octree` (a Points2Octree) is given, the merged octree is
  built from the samples' points in one pass."""
  if not isinstance(batch, list):
    raise TypeError("collate_octrees takes the list of samples of one batch")
  merged = {key: [sample[key] for sample in batch] for key in batch[0]}
  for key in list(merged):
    if "octree" in key:
      merged[key] = F.octree_batch(merged[key])
    if "label" in key:
      merged["label"] = torch.tensor(merged[key])
  if points2octree is not None and "octree" not in merged:
    merged["octree"] = points2octree.batch(merged["points"])
  return merged
