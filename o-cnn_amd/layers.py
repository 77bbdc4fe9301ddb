"""Mirrors of the thin Python modules of the reference
(pytorch/ocnn/octree_conv.py:75-158, octree_pool.py:69-103, octree_pad.py:47-72).
They add exactly the compositions the reference adds around the extension calls:
`octree_pad` after a stride-2 convolution, `octree_depad` before a stride-2
deconvolution, pad / depad around pooling.  Every call goes through the autograd
functions, so the modules train (fp32) as well as infer."""
import torch
from torch import nn

from . import autograd as F


def resize_with_last_val(list_in, num=3):
  out = list(list_in)
  while len(out) < num:
    out.append(out[-1])
  return out


class OctreeConvBase(nn.Module):
  def __init__(self, depth, channel_in, channel_out, kernel_size=[3], stride=1, nempty=False):
    super().__init__()
    self.depth = depth
    self.channel_in = channel_in
    self.channel_out = channel_out
    self.kernel_size = resize_with_last_val(kernel_size)
    self.stride = stride
    self.nempty = nempty
    self.kdim = self.kernel_size[0] * self.kernel_size[1] * self.kernel_size[2]
    conv_in = channel_in if self.is_conv_layer() else channel_out
    conv_out = channel_out if self.is_conv_layer() else channel_in
    self.cdim = conv_in * self.kdim
    self.weights = nn.Parameter(torch.empty(conv_out, self.cdim))
    nn.init.xavier_uniform_(self.weights)

  def is_conv_layer(self):
    raise NotImplementedError

  def extra_repr(self):
    return ('depth={}, channel_in={}, channel_out={}, kernel_size={}, stride={}, nempty={}'
            .format(self.depth, self.channel_in, self.channel_out, self.kernel_size,
                    self.stride, self.nempty))


class OctreeConv(OctreeConvBase):
  def is_conv_layer(self):
    return True

  def forward(self, data, octree):
    assert data.size(1) == self.channel_in
    conv = F.octree_conv(data, self.weights, octree, self.depth, self.channel_out,
                         self.kernel_size, self.stride, self.nempty)
    if self.stride == 2 and not self.nempty:
      conv = F.octree_pad(conv, octree, self.depth - 1)
    return conv


class OctreeDeconv(OctreeConvBase):
  def is_conv_layer(self):
    return False

  def forward(self, data, octree):
    assert data.size(1) == self.channel_in
    if self.stride == 2 and not self.nempty:
      data = F.octree_depad(data, octree, self.depth)
    return F.octree_deconv(data, self.weights, octree, self.depth, self.channel_out,
                           self.kernel_size, self.stride, self.nempty)


class OctreeConvFast(OctreeConvBase):
  """octree2col + matrix product: the explicit form the implicit-GEMM kernel replaces."""

  def is_conv_layer(self):
    return True

  def forward(self, data, octree):
    col = F.octree2col(data, octree, self.depth, self.kernel_size, self.stride, False)
    col = col.view([self.cdim, -1])
    conv = torch.mm(self.weights, col)
    conv = torch.unsqueeze(torch.unsqueeze(conv, 0), -1)
    if self.stride == 2:
      conv = F.octree_pad(conv, octree, self.depth - 1)
    return conv


class OctreeDeconvFast(OctreeConvBase):
  def is_conv_layer(self):
    return False

  def forward(self, data, octree):
    depth = self.depth
    if self.stride == 2:
      data = F.octree_depad(data, octree, depth)
      depth = depth + 1
    data = torch.squeeze(torch.squeeze(data, dim=0), dim=-1)
    col = torch.mm(self.weights.t(), data)
    col = col.view(self.channel_out, self.kdim, -1)
    return F.col2octree(col, octree, depth, self.kernel_size, self.stride, False)


class OctreePoolBase(nn.Module):
  def __init__(self, depth):
    super().__init__()
    self.depth = depth

  def extra_repr(self):
    return 'depth={}'.format(self.depth)


class OctreeMaxPool(OctreePoolBase):
  def __init__(self, depth, return_indices=False):
    super().__init__(depth)
    self.return_indices = return_indices

  def forward(self, data, octree):
    pool, mask = F.octree_max_pool(data, octree, self.depth)
    output = F.octree_pad(pool, octree, self.depth - 1)
    return output if not self.return_indices else (output, mask)


class OctreeMaxUnpool(OctreePoolBase):
  def forward(self, data, mask, octree):
    pool = F.octree_depad(data, octree, self.depth)
    return F.octree_max_unpool(pool, mask, octree, self.depth + 1)


class OctreeAvgPool(OctreePoolBase):
  def forward(self, data, octree):
    channel = data.shape[1]
    pool = data.view(1, channel, -1, 8).mean(dim=3, keepdims=True)
    return F.octree_pad(pool, octree, self.depth - 1)


class OctreePad(nn.Module):
  def __init__(self, depth, val=0.0):
    super().__init__()
    self.depth, self.val = depth, val

  def forward(self, data_in, octree):
    return F.octree_pad(data_in, octree, self.depth, self.val)


class OctreeDepad(nn.Module):
  def __init__(self, depth):
    super().__init__()
    self.depth = depth

  def forward(self, data_in, octree):
    return F.octree_depad(data_in, octree, self.depth)


def octree_nearest_pts(data, octree, depth, pts, nempty=False):
  """pytorch/ocnn/modules.py:209-221."""
  return F.octree_interp_pts(data, octree, depth, pts, "nearest", nempty)


def octree_trilinear_pts(data, octree, depth, pts, nempty=False):
  """pytorch/ocnn/modules.py:224-268; pts must be scaled into [0, 2^depth]."""
  return F.octree_interp_pts(data, octree, depth, pts, "linear", nempty)


def octree_trilinear(data, octree, depth, target_depth):
  """Interpolate from `depth` to the node centres of `target_depth` (modules.py:271-281)."""
  from . import nn as ops
  xyz = ops.octree_property(octree, "xyz", target_depth)
  xyz = ops.octree_decode_key(xyz).float()
  scale = 2.0 ** (depth - target_depth)
  xyz = (xyz + torch.tensor([0.5, 0.5, 0.5, 0.0], device=xyz.device)) * \
      torch.tensor([scale, scale, scale, 1.0], device=xyz.device)
  return octree_trilinear_pts(data, octree, depth, xyz)


class OctreeTrilinear(nn.Module):
  def __init__(self, depth):
    super().__init__()
    self.depth = depth

  def forward(self, data, octree):
    return octree_trilinear(data, octree, self.depth, self.depth + 1)


class OctreeInterp(nn.Module):
  """pytorch/ocnn/modules.py:294-318: points in [-1, 1] (+ batch id) -> [0, 2^depth]."""

  def __init__(self, depth, method='linear', nempty=False):
    super().__init__()
    self.depth, self.method, self.nempty = depth, method, nempty

  def forward(self, data, octree, pts):
    xyz = (pts[:, :3] + 1.0) * (2 ** (self.depth - 1))
    pts = torch.cat([xyz, pts[:, 3:]], dim=1)
    if self.method not in ('nearest', 'linear'):
      raise ValueError
    return F.octree_interp_pts(data, octree, self.depth, pts, self.method, self.nempty)

  def extra_repr(self):
    return 'depth={}, method={}, nempty={}'.format(self.depth, self.method, self.nempty)


class OctreeAlign(nn.Module):
  def __init__(self, depth):
    super().__init__()
    self.depth = depth

  def forward(self, data, src_octree, des_octree):
    return F.octree_align(data, src_octree, des_octree, self.depth)


class Octree2ColBase(nn.Module):
  """pytorch/ocnn/octree2col.py:59-69."""

  def __init__(self, depth, kernel_size, stride, nempty=False):
    super().__init__()
    self.depth, self.stride, self.nempty = depth, stride, nempty
    self.kernel_size = resize_with_last_val(kernel_size)

  def extra_repr(self):
    return 'depth={}, kernel_size={}, stride={}, nempty={}'.format(self.depth, self.kernel_size, self.stride,
                                                                   self.nempty)


class Octree2Col(Octree2ColBase):
  """pytorch/ocnn/octree2col.py:72-75."""

  def forward(self, data_in, octree):
    return F.octree2col(data_in, octree, self.depth, self.kernel_size, self.stride, self.nempty)


class Col2Octree(Octree2ColBase):
  """pytorch/ocnn/octree2col.py:78-81."""

  def forward(self, data_in, octree):
    return F.col2octree(data_in, octree, self.depth, self.kernel_size, self.stride, self.nempty)


class OctreeTile(nn.Module):
  """pytorch/ocnn/modules.py:193-206: every non-empty node hands its feature to its eight
  children (nearest-neighbour upsampling to the next level)."""

  def __init__(self, depth):
    super().__init__()
    self.depth = depth

  def forward(self, data_in, octree):
    out = F.octree_depad(data_in, octree, self.depth)
    out = out.repeat(1, 1, 1, 8)
    return out.view(1, out.shape[1], -1, 1)


class FullOctree2Voxel(nn.Module):
  """pytorch/ocnn/octree2voxel.py:5-16: [1, C, B * 8^depth, 1] of a full level -> [B, C, 8^depth]
  (Morton order within a sample)."""

  def __init__(self, depth):
    super().__init__()
    self.depth = depth

  def forward(self, data):
    height = 2 ** (3 * self.depth)
    return data.view(data.size(1), -1, height).permute(1, 0, 2)

  def extra_repr(self):
    return 'depth={}'.format(self.depth)


class FullOctreeGlobalPool(OctreePoolBase):
  """pytorch/ocnn/octree_pool.py:106-115: mean over a full level, per sample."""

  def __init__(self, depth):
    super().__init__(depth)
    self.octree2voxel = FullOctree2Voxel(depth)

  def forward(self, data):
    return self.octree2voxel(data).mean(dim=2)


def octree_feature(octree, depth, nempty=False):
  """pytorch/ocnn/modules.py:333-337."""
  from . import nn as ops
  output = ops.octree_property(octree, 'feature', depth)
  return ops.octree_depad(output, octree, depth) if nempty else output
