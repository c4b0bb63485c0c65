"""ctypes binding of libmplayers_probe.so (csrc/mp_probe.h): the bandwidth and issue probes and the
wavefront self test.  Measurement tools of bench.py and the tests; no operator uses them."""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("MPLAYERS_PROBE_LIB", os.path.join(HERE, "libmplayers_probe.so"))

ROWS, COLUMNS, STREAM = 0, 1, 2

_lib = None


def load():
  global _lib
  if _lib is not None:
    return _lib
  if not os.path.exists(LIB_PATH):
    raise RuntimeError("libmplayers_probe.so is missing: build it with `python -m mplayers_amd._build`")
  lib = ctypes.CDLL(LIB_PATH)
  vp, ci = ctypes.c_void_p, ctypes.c_int
  lib.mplp_copy.argtypes = [ci, ci, ci, vp, vp, ci, ci, ci, vp]
  lib.mplp_issue.argtypes = [vp, ci, vp]
  lib.mplp_issue_count.argtypes = []
  lib.mplp_issue_name.argtypes = [ci]
  lib.mplp_issue_slots.argtypes = [ci]
  lib.mplp_selftest_wave_ops.argtypes = [vp, vp]
  for name in ("mplp_copy", "mplp_issue", "mplp_issue_count", "mplp_issue_slots",
               "mplp_selftest_wave_ops"):
    getattr(lib, name).restype = ci
  lib.mplp_issue_name.restype = ctypes.c_char_p
  lib.mplp_last_error.restype = ctypes.c_char_p
  _lib = lib
  return lib


def check(rc, what):
  if rc != 0:
    raise RuntimeError("%s failed (%d): %s" % (what, rc, load().mplp_last_error().decode()))
