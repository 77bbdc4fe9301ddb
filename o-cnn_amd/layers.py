"""Module front ends of the hot-path operators, with the class names and constructor
signatures a user of the reference's `ocnn` package expects (pytorch/ocnn/octree_conv.py:75-158,
octree_pool.py:69-103, octree_pad.py:47-72, octree2col.py:59-81, modules.py:209-318).

The reference writes one class per (direction, implementation) pair.  Here one module,
`OctreeConvolution`, carries the whole rule set of the operator:

  * what the level conventions are (a stride-2 convolution reads level `depth` and writes level
    `depth - 1`; a stride-2 deconvolution reads the non-empty nodes of `depth` and writes
    `depth + 1`),
  * which re-indexing surrounds the kernel when all nodes are convolved (`octree_pad` after a
    stride-2 convolution, `octree_depad` before a stride-2 deconvolution; the non-empty mode
    needs neither),
  * how the weight matrix is laid out (`[rows, columns * taps]`, rows = the channel count on the
    output side of the equivalent convolution).

and the four public names only choose its two switches.  Pooling and padding modules are
table driven in the same way.  Every call goes through `autograd`, so the modules train (fp32)
as well as infer."""
import torch
from torch import nn

from . import autograd as F


def _three(kernel_size):
  """`[3]` -> `[3, 3, 3]`, `[3, 1]` -> `[3, 1, 1]`: the last entry repeats."""
  ks = list(kernel_size)
  return (ks + [ks[-1]] * 3)[:3]


class OctreeConvolution(nn.Module):
  """Octree convolution or its transpose, through the implicit-GEMM operator or through the
  explicit column matrix (`explicit=True`: octree2col / col2octree around a plain matrix
  product, the form the reference's *Fast classes spell out and the operator replaces)."""

  def __init__(self, depth, channel_in, channel_out, kernel_size=[3], stride=1, nempty=False,
               transposed=False, explicit=False):
    super().__init__()
    self.depth, self.stride, self.nempty = depth, stride, nempty
    self.channel_in, self.channel_out = channel_in, channel_out
    self.kernel_size = _three(kernel_size)
    self.transposed, self.explicit = transposed, explicit
    self.taps = self.kernel_size[0] * self.kernel_size[1] * self.kernel_size[2]
    rows, cols = (channel_in, channel_out) if transposed else (channel_out, channel_in)
    self.weights = nn.Parameter(torch.empty(rows, cols * self.taps))
    nn.init.xavier_uniform_(self.weights)

  # The reference's attribute names for the matrix shape, kept for code that reads them.
  @property
  def kdim(self):
    return self.taps

  @property
  def cdim(self):
    return self.weights.shape[1]

  def _reindexes(self):
    return self.stride == 2 and (self.explicit or not self.nempty)

  def forward(self, data, octree):
    if data.size(1) != self.channel_in:
      raise ValueError("expected %d input channels, got %d" % (self.channel_in, data.size(1)))
    geometry = (self.kernel_size, self.stride)
    if not self.transposed:
      if self.explicit:
        cols = F.octree2col(data, octree, self.depth, *geometry, False)
        out = (self.weights @ cols.reshape(self.cdim, -1))[None, :, :, None]
      else:
        out = F.octree_conv(data, self.weights, octree, self.depth, self.channel_out, *geometry, self.nempty)
      return F.octree_pad(out, octree, self.depth - 1) if self._reindexes() else out
    if self._reindexes():
      data = F.octree_depad(data, octree, self.depth)
    if not self.explicit:
      return F.octree_deconv(data, self.weights, octree, self.depth, self.channel_out, *geometry, self.nempty)
    cols = self.weights.t() @ data[0, :, :, 0]
    level = self.depth + (1 if self.stride == 2 else 0)
    return F.col2octree(cols.reshape(self.channel_out, self.taps, -1), octree, level, *geometry, False)

  def extra_repr(self):
    return ('depth={}, channel_in={}, channel_out={}, kernel_size={}, stride={}, nempty={}'
            .format(self.depth, self.channel_in, self.channel_out, self.kernel_size, self.stride, self.nempty))


def _convolution_class(name, transposed, explicit, doc):
  def __init__(self, depth, channel_in, channel_out, kernel_size=[3], stride=1, nempty=False):
    OctreeConvolution.__init__(self, depth, channel_in, channel_out, kernel_size, stride, nempty,
                               transposed=transposed, explicit=explicit)
  return type(name, (OctreeConvolution,), {"__init__": __init__, "__doc__": doc})


OctreeConv = _convolution_class("OctreeConv", False, False, "pytorch/ocnn/octree_conv.py:102-113")
OctreeDeconv = _convolution_class("OctreeDeconv", True, False, "pytorch/ocnn/octree_conv.py:116-127")
OctreeConvFast = _convolution_class("OctreeConvFast", False, True, "pytorch/ocnn/octree_conv.py:130-142")
OctreeDeconvFast = _convolution_class("OctreeDeconvFast", True, True, "pytorch/ocnn/octree_conv.py:145-158")


class _LevelModule(nn.Module):
  """A module whose only state is the octree level it works on."""

  def __init__(self, depth):
    super().__init__()
    self.depth = depth

  def extra_repr(self):
    return 'depth={}'.format(self.depth)


class OctreeMaxPool(_LevelModule):
  """Maximum over the 8 children of every parent, re-indexed to all nodes of level depth - 1
  (pytorch/ocnn/octree_pool.py:79-87)."""

  def __init__(self, depth, return_indices=False):
    super().__init__(depth)
    self.return_indices = return_indices

  def forward(self, data, octree):
    reduced, argmax = F.octree_max_pool(data, octree, self.depth)
    padded = F.octree_pad(reduced, octree, self.depth - 1)
    return (padded, argmax) if self.return_indices else padded


class OctreeMaxUnpool(_LevelModule):
  """The adjoint routing: level `depth` back to the argmax positions of level depth + 1
  (pytorch/ocnn/octree_pool.py:90-95)."""

  def forward(self, data, mask, octree):
    return F.octree_max_unpool(F.octree_depad(data, octree, self.depth), mask, octree, self.depth + 1)


class OctreeAvgPool(_LevelModule):
  """Mean over the 8 children (pytorch/ocnn/octree_pool.py:98-103)."""

  def forward(self, data, octree):
    groups = data.unflatten(2, (-1, 8))[..., 0]          # [1, C, H / 8, 8]
    return F.octree_pad(groups.mean(dim=3, keepdim=True), octree, self.depth - 1)


class OctreePad(_LevelModule):
  """Non-empty rows -> all rows of the level (pytorch/ocnn/octree_pad.py:47-58)."""

  def __init__(self, depth, val=0.0):
    super().__init__(depth)
    self.val = val

  def forward(self, data_in, octree):
    return F.octree_pad(data_in, octree, self.depth, self.val)


class OctreeDepad(_LevelModule):
  """All rows -> non-empty rows (pytorch/ocnn/octree_pad.py:61-72)."""

  def forward(self, data_in, octree):
    return F.octree_depad(data_in, octree, self.depth)


class _ColumnModule(nn.Module):
  """pytorch/ocnn/octree2col.py:59-69: the column matrix as an operator of its own."""
  direction = None

  def __init__(self, depth, kernel_size, stride, nempty=False):
    super().__init__()
    self.depth, self.stride, self.nempty = depth, stride, nempty
    self.kernel_size = _three(kernel_size)

  def forward(self, data_in, octree):
    op = F.octree2col if self.direction == "gather" else F.col2octree
    return op(data_in, octree, self.depth, self.kernel_size, self.stride, self.nempty)

  def extra_repr(self):
    return 'depth={}, kernel_size={}, stride={}, nempty={}'.format(self.depth, self.kernel_size, self.stride,
                                                                   self.nempty)


class Octree2Col(_ColumnModule):
  direction = "gather"


class Col2Octree(_ColumnModule):
  direction = "scatter"


# ---- transfer of features to free points and between levels ----------------------------------
def octree_nearest_pts(data, octree, depth, pts, nempty=False):
  """pytorch/ocnn/modules.py:209-221: the feature of the node that holds each point."""
  return F.octree_interp_pts(data, octree, depth, pts, "nearest", nempty)


def octree_trilinear_pts(data, octree, depth, pts, nempty=False):
  """pytorch/ocnn/modules.py:224-268; `pts` = (x, y, z in [0, 2^depth], batch id)."""
  return F.octree_interp_pts(data, octree, depth, pts, "linear", nempty)


def octree_trilinear(data, octree, depth, target_depth):
  """Level `depth` interpolated at the node centres of `target_depth` (modules.py:271-281)."""
  from . import nn as ops
  cells = ops.octree_decode_key(ops.octree_property(octree, "xyz", target_depth)).float()
  centres = cells.clone()
  centres[:, :3] = (cells[:, :3] + 0.5) * 2.0 ** (depth - target_depth)
  return octree_trilinear_pts(data, octree, depth, centres)


class OctreeTrilinear(_LevelModule):
  def forward(self, data, octree):
    return octree_trilinear(data, octree, self.depth, self.depth + 1)


class OctreeInterp(nn.Module):
  """pytorch/ocnn/modules.py:294-318: query points in [-1, 1]^3 (+ batch id)."""

  def __init__(self, depth, method='linear', nempty=False):
    super().__init__()
    if method not in ('nearest', 'linear'):
      raise ValueError("method must be 'nearest' or 'linear'")
    self.depth, self.method, self.nempty = depth, method, nempty

  def forward(self, data, octree, pts):
    cells = torch.cat([(pts[:, :3] + 1.0) * 2.0 ** (self.depth - 1), pts[:, 3:]], dim=1)
    return F.octree_interp_pts(data, octree, self.depth, cells, self.method, self.nempty)

  def extra_repr(self):
    return 'depth={}, method={}, nempty={}'.format(self.depth, self.method, self.nempty)


class OctreeAlign(_LevelModule):
  """Features of one octree re-indexed to the nodes of another (pytorch/ocnn/modules.py:284-291)."""

  def forward(self, data, src_octree, des_octree):
    return F.octree_align(data, src_octree, des_octree, self.depth)
