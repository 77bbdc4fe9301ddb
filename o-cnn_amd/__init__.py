"""MI355X-native octree hot path of O-CNN.

The directory name is not a Python identifier; load the package with
`importlib.import_module("o-cnn_amd")` (the repository root on sys.path).

  nn        -- mirror of the reference's `ocnn.nn` extension functions
               (pytorch/cpp/pybind.cpp:3-49) over libocnn_hip.so
  autograd  -- torch.autograd functions pairing every operator with its adjoint, as the
               Function classes of pytorch/ocnn do
  layers    -- module front ends of the operators under the reference's class names
               (pytorch/ocnn/octree_conv.py, octree_pool.py, octree_pad.py)
  stacks    -- conv -> BatchNorm -> ReLU (folded) operator sequences of the benchmark
               configurations (LeNet trunk, U-Net encoder / decoder)
  synthetic -- seeded synthetic point clouds of the benchmark configurations
  transforms -- NormalizePoints / TransformPoints / Points2Octree / TransformCompose / collate_octrees
"""
from . import lib, nn, autograd, layers, stacks, synthetic, transforms  # noqa: F401
from .nn import *  # noqa: F401,F403
from .layers import (OctreeConvolution, OctreeConv, OctreeDeconv, OctreeConvFast,  # noqa: F401
                     OctreeDeconvFast, OctreeMaxPool, OctreeMaxUnpool, OctreeAvgPool, OctreePad,
                     OctreeDepad, OctreeTrilinear, OctreeInterp, OctreeAlign, octree_nearest_pts,
                     octree_trilinear_pts, octree_trilinear, Octree2Col, Col2Octree)
