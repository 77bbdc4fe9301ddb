import hashlib
import importlib
import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
  sys.path.insert(0, ROOT)
GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
  config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
  """The C restatement of the reference path (oracle/ocnn_oracle.c)."""
  from oracle.checker import Checker, build_oracle
  build_oracle()
  return Checker("orc")


@pytest.fixture(scope="session")
def ref():
  """The real reference compiled from its own sources; absent -> skip."""
  from oracle.checker import Checker, have_ref
  if not have_ref():
    pytest.skip("oracle/_ref/libocnn_ref.so not built (needs the reference checkout)")
  return Checker("ref")


@pytest.fixture(scope="session")
def samples():
  """octree_1 .. octree_6: the blobs embedded in the reference's octree_samples.cpp."""
  z = np.load(os.path.join(GOLDEN, "octree_samples.npz"))
  return {k: z[k] for k in z.files}


@pytest.fixture(scope="session")
def hashes():
  with open(os.path.join(GOLDEN, "config_hashes.json")) as fh:
    return json.load(fh)


@pytest.fixture(scope="session")
def synthetic():
  return importlib.import_module("o-cnn_amd.synthetic")


@pytest.fixture(scope="session")
def oc():
  """The package under test; GPU tests only."""
  import torch
  if not torch.cuda.is_available():
    pytest.skip("no GPU")
  pkg = importlib.import_module("o-cnn_amd")
  pkg.lib.call("ocnn_device_check", 0)
  return pkg


def sha(a):
  return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()
