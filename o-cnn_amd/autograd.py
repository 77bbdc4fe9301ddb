"""torch.autograd wiring of the operators, the counterpart of the Function classes in
pytorch/ocnn/octree_conv.py:15-68, octree_pool.py:7-61, octree_pad.py:7-41 and
octree2col.py: each backward is the reference's choice of adjoint operator
(conv <-> conv_grad, pool <-> unpool, unpool <-> mask_pool, pad <-> depad, octree2col <-> col2octree).
Gradients are fp32, like every reference operator."""
import torch
from torch.autograd import Function

from . import nn as F


def _ks3(kernel_size):
  ks = list(kernel_size)
  while len(ks) < 3:
    ks.append(ks[-1])
  return ks


class OctreeConvFunction(Function):
  @staticmethod
  def forward(ctx, data_in, weights, octree, depth, channel_out, kernel_size, stride, nempty):
    data_in = data_in.contiguous()
    ctx.save_for_backward(data_in, weights, octree)
    ctx.cfg = (depth, channel_out, _ks3(kernel_size), stride, nempty)
    return F.octree_conv(data_in, weights, octree, *ctx.cfg)

  @staticmethod
  def backward(ctx, grad_in):
    data_in, weights, octree = ctx.saved_tensors
    grad_data, grad_w = F.octree_conv_grad(data_in, weights, octree, grad_in.contiguous(), *ctx.cfg,
                                           need_data=ctx.needs_input_grad[0], need_weights=ctx.needs_input_grad[1])
    return (grad_data, grad_w) + (None,) * 6


class OctreeDeconvFunction(Function):
  @staticmethod
  def forward(ctx, data_in, weights, octree, depth, channel_out, kernel_size, stride, nempty):
    data_in = data_in.contiguous()
    ctx.save_for_backward(data_in, weights, octree)
    ctx.cfg = (depth, channel_out, _ks3(kernel_size), stride, nempty)
    return F.octree_deconv(data_in, weights, octree, *ctx.cfg)

  @staticmethod
  def backward(ctx, grad_in):
    data_in, weights, octree = ctx.saved_tensors
    grad_data, grad_w = F.octree_deconv_grad(data_in, weights, octree, grad_in.contiguous(), *ctx.cfg,
                                             need_data=ctx.needs_input_grad[0], need_weights=ctx.needs_input_grad[1])
    return (grad_data, grad_w) + (None,) * 6


class OctreeMaxPoolFunction(Function):
  @staticmethod
  def forward(ctx, data_in, octree, depth):
    data_out, mask = F.octree_max_pool(data_in.contiguous(), octree, depth)
    ctx.depth = depth
    ctx.save_for_backward(mask, octree)
    ctx.mark_non_differentiable(mask)
    return data_out, mask

  @staticmethod
  def backward(ctx, grad_in, _mask_grad):
    mask, octree = ctx.saved_tensors
    return F.octree_max_unpool(grad_in.contiguous(), mask, octree, ctx.depth), None, None


class OctreeMaxUnpoolFunction(Function):
  @staticmethod
  def forward(ctx, data_in, mask, octree, depth):
    mask = mask.contiguous()
    ctx.depth = depth
    ctx.save_for_backward(mask, octree)
    return F.octree_max_unpool(data_in.contiguous(), mask, octree, depth)

  @staticmethod
  def backward(ctx, grad_in):
    mask, octree = ctx.saved_tensors
    return F.octree_mask_pool(grad_in.contiguous(), mask, octree, ctx.depth), None, None, None


class OctreeMaskPoolFunction(Function):
  @staticmethod
  def forward(ctx, data_in, mask, octree, depth):
    mask = mask.contiguous()
    ctx.depth = depth
    ctx.save_for_backward(mask, octree)
    return F.octree_mask_pool(data_in.contiguous(), mask, octree, depth)

  @staticmethod
  def backward(ctx, grad_in):
    mask, octree = ctx.saved_tensors
    return F.octree_max_unpool(grad_in.contiguous(), mask, octree, ctx.depth), None, None, None


class OctreePadFunction(Function):
  @staticmethod
  def forward(ctx, data_in, octree, depth, val=0.0):
    ctx.save_for_backward(octree)
    ctx.depth = depth
    return F.octree_pad(data_in.contiguous(), octree, depth, val)

  @staticmethod
  def backward(ctx, grad_in):
    octree, = ctx.saved_tensors
    return F.octree_depad(grad_in.contiguous(), octree, ctx.depth), None, None, None


class OctreeDepadFunction(Function):
  @staticmethod
  def forward(ctx, data_in, octree, depth):
    ctx.save_for_backward(octree)
    ctx.depth = depth
    return F.octree_depad(data_in.contiguous(), octree, depth)

  @staticmethod
  def backward(ctx, grad_in):
    octree, = ctx.saved_tensors
    return F.octree_pad(grad_in.contiguous(), octree, ctx.depth, 0.0), None, None


class Octree2ColFunction(Function):
  @staticmethod
  def forward(ctx, data_in, octree, depth, kernel_size, stride, nempty):
    ctx.save_for_backward(octree)
    ctx.cfg = (depth, _ks3(kernel_size), stride, nempty)
    return F.octree2col(data_in.contiguous(), octree, *ctx.cfg)

  @staticmethod
  def backward(ctx, grad_in):
    octree, = ctx.saved_tensors
    return (F.col2octree(grad_in.contiguous(), octree, *ctx.cfg),) + (None,) * 5


class Col2OctreeFunction(Function):
  @staticmethod
  def forward(ctx, data_in, octree, depth, kernel_size, stride, nempty):
    ctx.save_for_backward(octree)
    ctx.cfg = (depth, _ks3(kernel_size), stride, nempty)
    return F.col2octree(data_in.contiguous(), octree, *ctx.cfg)

  @staticmethod
  def backward(ctx, grad_in):
    octree, = ctx.saved_tensors
    return (F.octree2col(grad_in.contiguous(), octree, *ctx.cfg),) + (None,) * 5


class OctreeAlignFunction(Function):
  """pytorch/ocnn/octree_align.py: (data, src_octree, des_octree, depth) -> (aligned, idx)."""

  @staticmethod
  def forward(ctx, src_data, src_octree, des_octree, depth):
    out, idx = F.octree_align(src_data.contiguous(), src_octree, des_octree, depth)
    ctx.save_for_backward(idx)
    ctx.mark_non_differentiable(idx)
    return out, idx

  @staticmethod
  def backward(ctx, grad_out, _idx_grad):
    idx, = ctx.saved_tensors
    return F.octree_align_grad(grad_out.contiguous(), idx), None, None, None


class OctreeInterpFunction(Function):
  """Nearest / trilinear interpolation of node features at free points
  (pytorch/ocnn/modules.py:209-275); differentiable in the features."""

  @staticmethod
  def forward(ctx, data, octree, depth, pts, method, nempty):
    out, idx, weight = F.octree_interp_pts(data, octree, depth, pts, method, nempty)
    ctx.save_for_backward(idx, weight)
    ctx.cfg = (data.size(2), method)
    return out

  @staticmethod
  def backward(ctx, grad_out):
    idx, weight = ctx.saved_tensors
    H, method = ctx.cfg
    return (F.octree_interp_pts_grad(grad_out.contiguous(), idx, weight, H, method),) + (None,) * 5


octree_conv = OctreeConvFunction.apply
octree_deconv = OctreeDeconvFunction.apply
octree_max_pool = OctreeMaxPoolFunction.apply
octree_max_unpool = OctreeMaxUnpoolFunction.apply
octree_mask_pool = OctreeMaskPoolFunction.apply
octree_pad = OctreePadFunction.apply
octree_depad = OctreeDepadFunction.apply
octree2col = Octree2ColFunction.apply
col2octree = Col2OctreeFunction.apply
octree_align = OctreeAlignFunction.apply
octree_interp_pts = OctreeInterpFunction.apply
