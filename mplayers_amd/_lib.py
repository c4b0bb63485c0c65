"""ctypes binding of libmplayers_hip.so (the C ABI declared in include/mplayers_amd.h)."""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("MPLAYERS_HIP_LIB", os.path.join(HERE, "libmplayers_hip.so"))

SYMBOLS = ("mpl_trwp_forward", "mpl_trwp_backward", "mpl_isgmr_forward", "mpl_isgmr_backward",
           "mpl_trwp_forward_cpu", "mpl_isgmr_forward_cpu",
           "mpl_profile_begin", "mpl_profile_end", "mpl_n_chains", "mpl_table_is_dense",
           "mpl_last_error", "mpl_version", "mpl_edge_shift", "mpl_edge_shift_static",
           "mpl_trwp_soft_forward",
           "mpl_trwp_soft_backward", "mpl_soft_weighted_message", "mpl_soft_weighted_message_back", "mpl_set_option",
           "mpl_stereo_data_cost", "mpl_gradient_cues", "mpl_mrf_energy", "mpl_transpose")

KERNEL_KINDS = ("fwd_sweep", "bwd_sweep", "belief", "aggregate", "label", "combine", "other",
                "fwd_sweep_all", "bwd_sweep_all", "unary_all")


class Shape(ctypes.Structure):
  """struct mpl_shape"""
  _fields_ = [("n_dir", ctypes.c_int), ("batch", ctypes.c_int), ("height", ctypes.c_int),
              ("width", ctypes.c_int), ("n_disp", ctypes.c_int), ("ctx2d", ctypes.c_int)]


# per-call flags (MPL_F_* of include/mplayers_amd.h)
F_MSG_UNINIT = 0x01
F_PACKED_OFF = 0x02
F_PACKED_ALWAYS = 0x04
F_FUSED_U_OFF = 0x08
F_DCONTEXT_SAME_LABEL = 0x10
F_FUSED_PAIRS_OFF = 0x20
F_DENSE_TABLE = 0x40


class KernelStat(ctypes.Structure):
  """struct mpl_kernel_stat"""
  _fields_ = [("launches", ctypes.c_int), ("total_ms", ctypes.c_double)]


_lib = None


def load():
  """Loads the HIP library; raises if it has not been built (there is no fallback path)."""
  global _lib
  if _lib is not None:
    return _lib
  if not os.path.exists(LIB_PATH):
    raise RuntimeError(
        "libmplayers_hip.so is missing: build it with `python -m mplayers_amd._build` "
        "(hipcc --offload-arch=gfx950); there is no CPU or PyTorch fallback for these operators")
  lib = ctypes.CDLL(LIB_PATH)
  vp, ci, cf, cu = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_uint
  sp = ctypes.POINTER(Shape)
  lib.mpl_trwp_forward.argtypes = [sp, cu, cf, ci, ci] + [vp] * 10
  lib.mpl_trwp_backward.argtypes = [sp, cu, cf, ci] + [vp] * 11
  lib.mpl_isgmr_forward.argtypes = [sp, cu, ci, cf, ci, ci] + [vp] * 11
  lib.mpl_isgmr_backward.argtypes = [sp, cu, ci, cf, ci] + [vp] * 12
  lib.mpl_trwp_forward_cpu.argtypes = [sp, cf, ci] + [vp] * 5
  lib.mpl_isgmr_forward_cpu.argtypes = [sp, ci, cf, ci] + [vp] * 6
  lib.mpl_trwp_soft_forward.argtypes = [sp, cu, cf, ci] + [vp] * 10
  lib.mpl_trwp_soft_backward.argtypes = [sp, cu, cf, ci] + [vp] * 11
  lib.mpl_soft_weighted_message.argtypes = [ci, ci, vp, vp, vp, vp]
  lib.mpl_soft_weighted_message_back.argtypes = [ci, ci, vp, vp, vp, vp, vp]
  lib.mpl_set_option.argtypes = [ci, ci]
  lib.mpl_edge_shift.argtypes = [ci, vp, ci, ci, ci, ci, ci, cf, cf, cf, vp, vp, vp]
  lib.mpl_edge_shift_static.argtypes = [ci, vp, ci, ci, ci, ci, ci, cf, cf, cf, vp, vp]
  lib.mpl_stereo_data_cost.argtypes = [vp, vp, ci, ci, ci, ci, ci, ci, ci, vp, vp]
  lib.mpl_gradient_cues.argtypes = [vp, ci, ci, ci, ci, cf, vp, vp, vp]
  lib.mpl_mrf_energy.argtypes = [sp, ci, vp, vp, vp, vp, vp, vp]
  lib.mpl_transpose.argtypes = [vp, vp, ci, ctypes.c_int64, ctypes.c_int64, vp]
  lib.mpl_n_chains.argtypes = [ci, ci, ci]
  lib.mpl_table_is_dense.argtypes = [vp, ci]
  lib.mpl_profile_begin.argtypes = []
  lib.mpl_profile_end.argtypes = [ctypes.POINTER(KernelStat), ci]
  for name in SYMBOLS:
    getattr(lib, name).restype = ci
  lib.mpl_last_error.restype = ctypes.c_char_p
  if lib.mpl_version() // 100 != 2:
    raise RuntimeError("libmplayers_hip.so has ABI version %d, this package needs 2xx: rebuild it "
                       "with `python -m mplayers_amd._build`" % lib.mpl_version())
  _lib = lib
  policy = os.environ.get("MPLAYERS_PACKED_SCANS")  # 0 | 1 | 2, see mpl_set_option
  if policy is not None:
    check(lib.mpl_set_option(OPT_PACKED_SCANS, int(policy)), "set_option")
  fused = os.environ.get("MPLAYERS_FUSED_U")  # 0 | 1, see mpl_set_option
  if fused is not None:
    check(lib.mpl_set_option(OPT_FUSED_U, int(fused)), "set_option")
  return lib


OPT_PACKED_SCANS = 0
OPT_FUSED_U = 1
OPT_BELIEF_REBUILD = 2
OPT_CPU_THREADS = 3
OPT_DENSE_SPLIT_WAVES = 4
BELIEF_REBUILD_DEFAULT = -1


def set_option(option, value):
  check(load().mpl_set_option(int(option), int(value)), "set_option")


def profile_begin():
  check(load().mpl_profile_begin(), "profile_begin")


def profile_end():
  """Returns {kind: (launches, total_ms)} for the kernels launched since profile_begin()."""
  stats = (KernelStat * len(KERNEL_KINDS))()
  check(load().mpl_profile_end(stats, len(KERNEL_KINDS)), "profile_end")
  return {k: (stats[i].launches, stats[i].total_ms) for i, k in enumerate(KERNEL_KINDS)}


def table_is_dense(table):
  """mpl_table_is_dense on a 1-D table given as a sequence, numpy array or tensor of floats (copied
  to host memory): True when the forward scans take their O(L^2) step on it."""
  import numpy as np
  if hasattr(table, "detach"):
    table = table.detach().cpu().numpy()
  row = np.ascontiguousarray(table, dtype=np.float32).reshape(-1)
  rc = load().mpl_table_is_dense(row.ctypes.data, int(row.size))
  if rc < 0:
    raise ValueError("table_is_dense: an empty table")
  return bool(rc)


def check(rc, what):
  if rc != 0:
    raise RuntimeError("%s failed (%d): %s" % (what, rc, load().mpl_last_error().decode()))
