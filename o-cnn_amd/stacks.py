"""Operator sequences of the benchmark configurations, issued in the reference's order.

The reference wraps every convolution as conv -> BatchNorm2d(eps = 1e-3) -> ReLU
(`OctreeConvBnRelu`, pytorch/ocnn/modules.py:23-36).  At inference the BatchNorm is an
affine map per output channel, so it folds into the weights and a bias; the fused kernel
applies bias and ReLU to the accumulator before the store.

  lenet_trunk  conv -> BN -> ReLU -> max_pool (+pad) per depth, as pytorch/ocnn/lenet.py:24-32
               (lenet_trunk_rows: the same in bf16 on row-major activations)
  unet_trunk   encoder / decoder with 2x2x2 stride-2 down-convolutions and deconvolutions and
               skip concatenations, the op order of pytorch/ocnn/unet.py:61-92 with one
               convolution per stage
"""
import torch

from . import nn as F

BN_EPS = 1e-3  # pytorch/ocnn/modules.py:5


def fold_bn(weights, gamma, beta, mean, var, eps=BN_EPS, deconv=False, kdim=None):
  """(W', b') with  BN(conv(x, W)) == conv(x, W') + b'.
  conv weights are [Cout, Cin*K]; deconv weights are [Cin, Cout*K] (column co*K + k)."""
  scale = gamma / torch.sqrt(var + eps)
  if not deconv:
    w = weights * scale[:, None]
  else:
    cout = scale.numel()
    w = (weights.view(weights.shape[0], cout, kdim) * scale[None, :, None]).reshape(weights.shape)
  return w.contiguous(), (beta - mean * scale).contiguous()


def conv_bn_relu(data, w, b, octree, depth, cout, kernel_size=(3, 3, 3), stride=1, nempty=False,
                 deconv=False, relu=True, out=None):
  """OctreeConvBnRelu / OctreeDeConvBnRelu with folded BatchNorm, including the pad / depad the
  reference modules add around stride-2 layers (pytorch/ocnn/octree_conv.py:102-127)."""
  ks = list(kernel_size)
  if deconv and stride == 2 and not nempty:
    data = F.octree_depad(data, octree, depth)
  padded_after = (not deconv) and stride == 2 and not nempty
  out = F.octree_conv_fused(data, w.to(data.dtype), b, relu, octree, depth, cout, ks, stride, nempty,
                            deconv=deconv, out=None if padded_after else out)
  if padded_after:
    # a padded (empty) node holds 0 in the reference because the pad comes after conv but
    # before BatchNorm; after folding the empty nodes must receive relu(b) instead of 0:
    # the reference order is conv -> pad -> BN -> ReLU.
    # (one pass: the pad writes the per-channel value where a node has no source row)
    out = F.octree_pad_fill(out, octree, depth - 1, torch.relu(b) if relu else b)
  return out


def lenet_trunk(octree, depth, params, data=None, to_depth=2):
  """params[d] = (w, b) for the conv at depth d (3x3x3, stride 1); returns the features at
  `to_depth` after the last pool."""
  if data is None:
    data = F.octree_property(octree, "feature", depth)
  for d in range(depth, to_depth, -1):
    w, b = params[d]
    data = conv_bn_relu(data, w, b, octree, d, w.shape[0])
    pool, _ = F.octree_max_pool(data, octree, d)
    data = F.octree_pad(pool, octree, d - 1)
  return data


def lenet_trunk_rows(octree, depth, params, data=None, to_depth=2, constant_weights=True):
  """lenet_trunk in bf16 with row-major activations between the operators: the input is converted
  once, every convolution and every pooling step (max_pool with the pad behind it) reads and
  writes the layout the convolution kernels gather from, the result is converted back once."""
  if data is None:
    data = F.octree_property(octree, "feature", depth).bfloat16()
  x, cin = F.to_rows(data), data.size(1)
  for d in range(depth, to_depth, -1):
    w, b = params[d]
    x = F.octree_conv_rows(x, cin, w, octree, d, w.shape[0], bias=b, relu=True, constant_weights=constant_weights)
    cin = w.shape[0]
    x = F.octree_max_pool_rows(x, cin, octree, d)
  return F.from_rows(x, cin)


def unet_trunk(octree, depth, params, data=None, stages=3, nempty=False):
  """params: dict with keys ('conv', d), ('down', d), ('up', d), ('dec', d) -> (w, b).
  Encoder: conv at `depth`, then per stage a 2x2x2 stride-2 conv to depth-1 and a 3x3x3 conv;
  decoder: per stage a 2x2x2 stride-2 deconv to depth+1, concatenation with the encoder
  feature of that depth, and a 3x3x3 conv."""
  if data is None:
    data = F.octree_property(octree, "feature", depth)
    if nempty:
      data = F.octree_depad(data, octree, depth)
  # The decoder reads [encoder feature of depth d | upsampled feature] as one tensor.  That tensor
  # is allocated when the encoder reaches depth d, and both producers write their channel slice
  # of it directly: no concatenation copy.
  info = F.octree_info(octree)
  feats, joined = {}, {}

  def encoder_conv(x, d, skip):
    w, b = params[("conv", d)]
    c_skip = w.shape[0]
    if not skip:
      return conv_bn_relu(x, w, b, octree, d, c_skip, nempty=nempty)
    c_up = params[("up", d - 1)][0].shape[1] // 8
    rows = info.nnum_nempty(d) if nempty else info.nnum(d)
    joined[d] = torch.empty(1, c_skip + c_up, rows, 1, dtype=x.dtype, device=x.device)
    return conv_bn_relu(x, w, b, octree, d, c_skip, nempty=nempty, out=joined[d][:, :c_skip])

  feats[depth] = encoder_conv(data, depth, stages > 0)
  d = depth
  for i in range(stages):
    w, b = params[("down", d)]
    x = conv_bn_relu(feats[d], w, b, octree, d, w.shape[0], (2, 2, 2), 2, nempty)
    d -= 1
    feats[d] = encoder_conv(x, d, i + 1 < stages)
  x = feats[d]
  for _ in range(stages):
    w, b = params[("up", d)]
    cout = w.shape[1] // 8
    d += 1
    c_skip = feats[d].shape[1]
    conv_bn_relu(x, w, b, octree, d - 1, cout, (2, 2, 2), 2, nempty, deconv=True, out=joined[d][:, c_skip:])
    w, b = params[("dec", d)]
    x = conv_bn_relu(joined[d], w, b, octree, d, w.shape[0], nempty=nempty)
  return x


def unet_trunk_rows(octree, depth, params, data=None, stages=3, nempty=False, constant_weights=True):
  """unet_trunk in bf16 with row-major activations between the operators: the input is converted
  once, every convolution reads the layout its kernel gathers from and writes it for the next one
  (over all nodes the pad and depad around the stride-2 layers are part of those operators; both
  halves of a concatenation are written in place), and the result is converted back once.
  Same operators in the same order as unet_trunk (pytorch/ocnn/unet.py:61-92 with one
  convolution per stage); channel counts of the concatenated features must be multiples of 16.
  constant_weights (the inference case): packed weights and inverted child links are kept between
  calls, see octree_conv_rows."""
  if data is None:
    data = F.octree_property(octree, "feature", depth).bfloat16()
    if nempty:
      data = F.octree_depad(data, octree, depth)
  info = F.octree_info(octree)
  x, cin = F.to_rows(data), data.size(1)
  feats, joined = {}, {}

  def conv(x, cin, w, b, d, cout, out=None, **kw):
    return F.octree_conv_rows(x, cin, w, octree, d, cout, bias=b, relu=True, out=out, nempty=nempty,
                              constant_weights=constant_weights, **kw)

  def encoder_conv(x, cin, d, skip):
    w, b = params[("conv", d)]
    c_skip = w.shape[0]
    if not skip:
      return conv(x, cin, w, b, d, c_skip), c_skip
    c_up = params[("up", d - 1)][0].shape[1] // 8
    if c_skip % 16 or c_up % 16:
      raise ValueError("concatenated features need channel counts that are multiples of 16")
    rows = info.nnum_nempty(d) if nempty else info.nnum(d)
    joined[d] = torch.empty(rows + 1, c_skip + c_up, dtype=x.dtype, device=x.device)
    return conv(x, cin, w, b, d, c_skip, out=joined[d][:, :c_skip]), c_skip

  feats[depth] = encoder_conv(x, cin, depth, stages > 0)
  d = depth
  for i in range(stages):
    w, b = params[("down", d)]
    x, cin = feats[d]
    x = conv(x, cin, w, b, d, w.shape[0], kernel_size=(2, 2, 2), stride=2)
    d -= 1
    feats[d] = encoder_conv(x, w.shape[0], d, i + 1 < stages)
  x, cin = feats[d]
  for _ in range(stages):
    w, b = params[("up", d)]
    cout = w.shape[1] // 8
    c_skip = feats[d + 1][1]
    conv(x, cin, w, b, d, cout, out=joined[d + 1][:, c_skip:], deconv=True, kernel_size=(2, 2, 2), stride=2)
    d += 1
    w, b = params[("dec", d)]
    x, cin = conv(joined[d], c_skip + cout, w, b, d, w.shape[0]), w.shape[0]
  return F.from_rows(x, cin)


def create_full_octree(depth, channel, batch_size=1, node_dis=True):
  """pytorch/ocnn/modules.py:325-330."""
  octree = F.octree_new(batch_size, channel, node_dis)
  for target_depth in range(1, depth + 1):
    octree = F.octree_grow(octree, target_depth, True)
  return octree


def predict_head(x, head, octree, depth, return_label=False):
  """The prediction module of pytorch/ocnn/ounet.py:46-49: a 1x1x1 conv -> BN -> ReLU to the hidden
  width and a 1x1x1 convolution with bias; head = ((w1, b1), (w2, b2)) with the BatchNorm folded
  into (w1, b1).  Returns the logits [1, n_out, H, 1] (with return_label also their argmax over
  the channels, int32 [H]).  fp32 heads of at most 32 hidden and 8 output channels run as one
  kernel that keeps the hidden channels in registers."""
  (w1, b1), (w2, b2) = head
  if x.dtype == torch.float32 and w1.shape[0] <= 32 and w2.shape[0] <= 8:
    return F.conv1x1_pair(x, w1, b1, w2, b2, relu=True, return_label=return_label)
  hidden = conv_bn_relu(x, w1, b1, octree, depth, w1.shape[0], (1, 1, 1))
  logit = conv_bn_relu(hidden, w2, b2, octree, depth, w2.shape[0], (1, 1, 1), relu=False)
  if return_label:
    return logit, logit.view(logit.shape[1], -1).argmax(0).to(torch.int32)
  return logit


def completion_decoder(code, params, split_labels, depth, full_depth, batch_size=1, channel_out=4,
                       signal=None, skips=None, octree_in=None):
  """The shape-decoding loop of pytorch/ocnn/ounet.py:72-131 (`ocnn_decoder` / `decode_shape`):
  starting from a full octree at `full_depth`, per depth a 2x2x2 stride-2 deconvolution up, the
  encoder's feature of that depth moved onto the growing octree (`octree_align`) and added, a
  3x3x3 convolution, the split prediction (1x1x1 head -> argmax), `octree_update` (child links from
  the labels) and `octree_grow` (keys / children / neighbours of the next depth).

  code          features at full_depth, [1, C, batch*8^full_depth, 1]
  params        {('up', d): (w, b), ('conv', d): (w, b)} for d in full_depth+1 .. depth, and
                optionally {('predict', d): ((w1, b1), (w2, b2))} for d in full_depth .. depth
  split_labels  {d: int32[H_d]}; label 1 = split: the labels that decide the structure (the
                ground truth's when training, ounet.py:89-90).  A callable `f(d, features) ->
                labels` may stand for them; None takes the predicted labels (`decode_shape`,
                ounet.py:118-119).  With a prediction head the logits and their argmax are
                computed at every depth either way.
  skips, octree_in  optional encoder features {d: [1, C_d, H_d(octree_in), 1]} and the octree
                they live on (ounet.py:109-111)
  signal        optional callable `f(features) -> [1, channel_out, H_depth, 1]` written as the
                finest-level feature of the result
  Returns (octree, feats): feats[d] = decoder features, feats[('logit', d)] / feats[('label', d)]
  = the head's output and its argmax (int32 [H_d]) where a head was given.
  """
  octree = create_full_octree(full_depth, channel_out, batch_size)
  feats = {full_depth: code}
  for d in range(full_depth, depth + 1):
    if d > full_depth:
      w, b = params[("up", d)]
      x = conv_bn_relu(feats[d - 1], w, b, octree, d - 1, w.shape[1] // 8, (2, 2, 2), 2, deconv=True)
      if skips is not None and d in skips:
        if x.dtype == torch.float32:
          x, _ = F.octree_align(skips[d], octree_in, octree, d, add_to=x.contiguous())
        else:
          x = x + F.octree_align(skips[d], octree_in, octree, d)[0]
      w, b = params[("conv", d)]
      feats[d] = conv_bn_relu(x, w, b, octree, d, w.shape[0])
    predicted = None
    if ("predict", d) in params:
      logit, predicted = predict_head(feats[d], params[("predict", d)], octree, d, return_label=True)
      feats[("logit", d)], feats[("label", d)] = logit, predicted
    if split_labels is None:
      if predicted is None:
        raise ValueError("no split labels and no prediction head at depth %d" % d)
      label = predicted
    else:
      label = split_labels(d, feats[d]) if callable(split_labels) else split_labels[d]
    # (the octree of this depth is the loop's own, fresh from octree_grow: updated in place)
    octree = F.octree_update(octree, label.to(torch.int32), d, 1, inplace=True)
    if d < depth:
      octree = F.octree_grow(octree, d + 1, False)
    elif signal is not None:
      octree = F.octree_set_property(octree, signal(feats[d]), d)
  return octree, feats
