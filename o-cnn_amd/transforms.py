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


def draw_distortion(angle, scale, jitter, angle_interval, uniform_scale):
  """The random part of TransformPoints (transforms.py:80-98), in the reference's order of
  draws: per axis a whole number of `angle_interval` steps within +-angle (radians returned),
  then three scales in [1 - scale, 1 + scale] (the first one three times if uniform), then three
  jitters in [-jitter, jitter]."""
  rnd_angle = [0.0, 0.0, 0.0]
  for i in range(3):
    steps = angle[i] // angle_interval[i]
    rnd_angle[i] = int(np.random.randint(low=-steps, high=steps + 1, dtype=np.int32)) * angle_interval[i] * _DEG
  rnd_scale = np.random.uniform(low=1 - scale, high=1 + scale, size=(3)).tolist()
  if uniform_scale:
    rnd_scale = [rnd_scale[0]] * 3
  rnd_jitter = np.random.uniform(low=-jitter, high=jitter, size=(3)).tolist()
  return rnd_angle, rnd_scale, rnd_jitter


class TransformPoints:
  """transforms.py:61-108: the augmentation of a cloud that lies in [-1, 1], and the clip back
  into that box.  Returns (points, inbox_mask)."""

  def __init__(self, distort, angle=(0, 180, 0), scale=0.25, jitter=0.25, offset=0.0,
               angle_interval=(1, 1, 1), uniform_scale=False, normal_axis="", **kwargs):
    self.distort = distort
    self.angle, self.scale, self.jitter, self.offset = list(angle), scale, jitter, offset
    self.angle_interval, self.uniform_scale, self.normal_axis = list(angle_interval), uniform_scale, normal_axis

  def __call__(self, points, drawn=None):
    if drawn is None:
      drawn = (draw_distortion(self.angle, self.scale, self.jitter, self.angle_interval, self.uniform_scale)
               if self.distort else ([0.0] * 3, [1.0] * 3, [0.0] * 3))
    rnd_angle, rnd_scale, rnd_jitter = drawn
    points = F.transform_points(points, rnd_angle, rnd_scale, rnd_jitter, self.offset, self.normal_axis)
    return tuple(F.clip_points(points, [-1.0] * 3, [1.0] * 3))


class TransformCompose:
  """transforms.py:111-130: normalise -> transform + clip -> octree.  With `octree=False` the
  sample keeps its points only and `collate_octrees(..., points2octree=...)` builds the whole
  batch at once."""

  def __init__(self, flags, octree=True):
    self.flags = flags
    self.normalize_points = NormalizePoints(**flags)
    self.transform_points = TransformPoints(**flags)
    self.points2octree = Points2Octree(**flags)
    self.octree = octree

  def __call__(self, points, idx=0):
    points = self.normalize_points(points)
    points, inbox_mask = self.transform_points(points)
    out = {"points": points, "inbox_mask": inbox_mask}
    if self.octree:
      out["octree"] = self.points2octree(points)
    return out


def collate_octrees(batch, points2octree=None):
  """transforms.py:133-148: lists per key, octrees merged with octree_batch, labels as a tensor.
  If the samples carry no octree and `points2octree` (a Points2Octree) is given, the merged
  octree is built from the samples' points in one pass."""
  assert type(batch) == list
  outputs = {}
  for key in batch[0].keys():
    outputs[key] = [b[key] for b in batch]
    if "octree" in key:
      outputs[key] = F.octree_batch(outputs[key])
    if "label" in key:
      outputs["label"] = torch.tensor(outputs[key])
  if points2octree is not None and "octree" not in outputs:
    outputs["octree"] = points2octree.batch(outputs["points"])
  return outputs
