"""ctypes loader of libocnn_hip.so.  There is no fallback: if the library is
missing or a call fails, an exception is raised."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(HERE, "libocnn_hip.so")

F32, BF16 = 0, 1
KEY, CHILD, NEIGH, FEATURE, LABEL, SPLIT = 1, 2, 4, 8, 16, 32
INFO_BYTES, HEADER_BYTES, POINTS_INFO_BYTES = 716, 720, 88

_SIZE_T = ("ocnn_generate_label_scratch_bytes", "ocnn_points2octree_workspace_bytes",
           "ocnn_octree_batch_workspace_bytes", "ocnn_octree_update_scratch_bytes",
           "ocnn_points_workspace_bytes", "ocnn_octree_interp_workspace_bytes", "ocnn_octree_interp_backward_workspace_bytes",
           "ocnn_octree_gatherbk_workspace_bytes", "ocnn_search_key_workspace_bytes")
_INT64 = ("ocnn_info_ptr_dis", "ocnn_info_sizeof_octree")


class OcnnError(RuntimeError):
  def __init__(self, code, msg):
    super().__init__("libocnn_hip error %d: %s" % (code, msg))
    self.code = code


class BuildParams(C.Structure):
  _fields_ = [("depth", C.c_int), ("full_depth", C.c_int), ("node_dis", C.c_int),
              ("node_feature", C.c_int), ("split_label", C.c_int), ("adaptive", C.c_int),
              ("adp_depth", C.c_int), ("th_normal", C.c_float), ("th_distance", C.c_float),
              ("extrapolate", C.c_int), ("save_pts", C.c_int), ("key2xyz", C.c_int),
              ("merged", C.c_int), ("has_bbox", C.c_int), ("bbmin", C.c_float * 3),
              ("bbmax", C.c_float * 3)]


_lib = None
_aten = None
ATEN_PATH = os.path.join(HERE, "binding", "ocnn_aten.so")


def aten():
  """The ATen binding (binding/ocnn_aten.cpp built by binding/Makefile): the reference's operator
  signatures over the same C interface, as a compiled Python module."""
  global _aten
  if _aten is None:
    if not os.path.exists(ATEN_PATH):
      raise ImportError("%s is missing: run `make -C o-cnn_amd/binding` (or __graft_entry__.build())" % ATEN_PATH)
    import importlib.util
    import torch  # noqa: F401  (the module links against PyTorch's libraries)
    get()
    spec = importlib.util.spec_from_file_location("ocnn_aten", ATEN_PATH)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    _aten = mod
  return _aten


def build():
  """Compile the library in-tree with hipcc for gfx950."""
  import subprocess
  subprocess.check_call(["make", "-s", "-C", os.path.join(HERE, "csrc"), "-j8"])


def get():
  global _lib
  if _lib is None:
    if not os.path.exists(SO_PATH):
      raise ImportError("%s is missing: run `make -C o-cnn_amd/csrc` (or __graft_entry__.build())"
                        % SO_PATH)
    lib = C.CDLL(SO_PATH)
    lib.ocnn_last_error.restype = C.c_char_p
    for n in _SIZE_T:
      getattr(lib, n).restype = C.c_size_t
    for n in _INT64:
      getattr(lib, n).restype = C.c_int64
    lib.ocnn_points2octree_workspace_bytes.argtypes = [C.c_int64, C.c_int, C.c_int]
    _lib = lib
  return _lib


def check(code):
  if code != 0:
    raise OcnnError(code, get().ocnn_last_error().decode())


def call(name, *args):
  """Call an int-status entry point; raise OcnnError on failure."""
  check(getattr(get(), name)(*args))
