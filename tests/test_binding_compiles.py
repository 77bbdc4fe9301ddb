"""The ATen side of the convolution operators (o-cnn_amd/binding/octree_conv_aten.cpp, the
bodies that replace pytorch/cpp/octree_conv.cpp:131-283) must compile against the C interface
(include/ocnn_hip.h) and PyTorch's headers: syntax and types only, nothing is linked or run."""
import os
import shutil
import subprocess
import sysconfig

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_aten_binding_compiles_against_the_header():
  cxx = shutil.which("g++")
  if cxx is None:
    pytest.skip("no g++")
  from torch.utils import cpp_extension as ce
  inc = [os.path.join(ROOT, "include"), "/opt/rocm/include", sysconfig.get_paths()["include"]] + ce.include_paths()
  src = os.path.join(ROOT, "o-cnn_amd", "binding", "octree_conv_aten.cpp")
  cmd = [cxx, "-std=c++17", "-fsyntax-only", "-D__HIP_PLATFORM_AMD__", "-DTORCH_EXTENSION_NAME=ocnn_conv_aten"]
  cmd += ["-I" + p for p in inc] + [src]
  r = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
  assert r.returncode == 0, r.stderr[-4000:]
