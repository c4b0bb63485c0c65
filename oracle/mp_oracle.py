"""TEST INFRASTRUCTURE ONLY: numpy front end of the CPU oracle (libmp_oracle.so).

Only tests, the smoke check and the benchmark's cpu_baseline leg may import this module; the
product package never does.  Shapes follow the reference's autograd Functions
(pytorch/MP_module.py:17-161): unary (B, cv, H, W, L), messages (n_dir, B, cv, H, W, L),
edge weights (n_dir, B, cv, H, W), indices uint8 (n_iter, n_dir, B, cv, H, W[, L]).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmp_oracle.so")
_lib = None


class _Geom(ctypes.Structure):
  _fields_ = [("n_dir", ctypes.c_int), ("B", ctypes.c_int), ("H", ctypes.c_int),
              ("W", ctypes.c_int), ("L", ctypes.c_int), ("ctx2d", ctypes.c_int)]


def build(force=False):
  """Compile the oracle with gcc (a checker is being built, not used)."""
  if force or not os.path.exists(_LIB_PATH):
    subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libmp_oracle.so"])
  return _LIB_PATH


def lib():
  global _lib
  if _lib is None:
    if not os.path.exists(_LIB_PATH):
      build()
    _lib = ctypes.CDLL(_LIB_PATH)
    assert _lib.mpo_geom_size() == ctypes.sizeof(_Geom)
  return _lib


def _ptr(a):
  return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _real(dtype):
  dtype = np.dtype(dtype)
  if dtype == np.float32:
    return "f32", ctypes.c_float
  if dtype == np.float64:
    return "f64", ctypes.c_double
  raise TypeError(dtype)


def _geom(n_dir, shape5, ctx2d):
  b, cv, h, w, L = shape5
  if ctx2d is None:
    ctx2d = (L == 21)  # the reference selects the (L, L) table by n_disp == 21
  return _Geom(n_dir, b * cv, h, w, L, int(bool(ctx2d)))


def dir_step(d):
  hs, ws = ctypes.c_int(), ctypes.c_int()
  lib().mpo_dir_step(d, ctypes.byref(hs), ctypes.byref(ws))
  return hs.value, ws.value


def n_trees(d, H, W):
  return lib().mpo_n_trees(d, H, W)


def forward(mode, unary, context, edge_weights, n_dir, n_iter, rho, training=True,
            saving_label=False, enable_min_a_dir=False, enable_sgm=False, ctx2d=None,
            want_gaps=False, msg_init=None):
  """Restated ForwardCUDA of TRWP (TRWP_forward.cu:378-560) or ISGMR (ISGMR_forward.cu:433-665).

  Returns a dict with msg, cost_final, msg_min_index, msg_norm_index, label_all and, when
  want_gaps, gap_min / gap_norm / gap_label (second best minus best of every argmin and of every
  saved label, for tie-aware checks).
  """
  unary = np.ascontiguousarray(unary)
  sfx, creal = _real(unary.dtype)
  dt = unary.dtype
  b, cv, h, w, L = unary.shape
  g = _geom(n_dir, unary.shape, ctx2d)
  context = np.ascontiguousarray(context, dtype=dt)
  if edge_weights is None:
    edge_weights = np.ones((n_dir, b, cv, h, w), dtype=dt)
  edge_weights = np.ascontiguousarray(edge_weights, dtype=dt)
  assert edge_weights.shape == (n_dir, b, cv, h, w)
  msg = np.zeros((n_dir, b, cv, h, w, L), dtype=dt) if msg_init is None else \
      np.array(msg_init, dtype=dt, order="C")
  cost = np.zeros((b, cv, h, w, L), dtype=dt)
  imin = np.zeros((n_iter, n_dir, b, cv, h, w, L), dtype=np.uint8) if training else None
  inorm = np.zeros((n_iter, n_dir, b, cv, h, w), dtype=np.uint8) if training else None
  label = np.zeros((n_iter, b, cv, h, w), dtype=np.uint8) if saving_label else None
  gmin = np.full((n_iter, n_dir, b, cv, h, w, L), np.inf, dtype=dt) if want_gaps else None
  gnorm = np.full((n_iter, n_dir, b, cv, h, w), np.inf, dtype=dt) if want_gaps else None
  glabel = np.full((n_iter, b, cv, h, w), np.inf, dtype=dt) if (want_gaps and saving_label) \
      else None
  out = dict(msg=msg, cost_final=cost, msg_min_index=imin, msg_norm_index=inorm, label_all=label,
             gap_min=gmin, gap_norm=gnorm, gap_label=glabel)
  if mode == "TRWP":
    fn = getattr(lib(), "mpo_trwp_forward_" + sfx)
    fn(ctypes.byref(g), creal(rho), int(n_iter), int(enable_min_a_dir), _ptr(unary),
       _ptr(context), _ptr(edge_weights), _ptr(msg), _ptr(cost), _ptr(imin), _ptr(inorm),
       _ptr(label), _ptr(gmin), _ptr(gnorm), _ptr(glabel))
  elif mode in ("ISGMR", "SGM"):
    fn = getattr(lib(), "mpo_isgmr_forward_" + sfx)
    msg_update = np.zeros_like(msg)
    fn(ctypes.byref(g), int(enable_sgm), creal(rho), int(n_iter), int(enable_min_a_dir),
       _ptr(unary), _ptr(context), _ptr(edge_weights), _ptr(msg), _ptr(msg_update), _ptr(cost),
       _ptr(imin), _ptr(inorm), _ptr(label), _ptr(gmin), _ptr(gnorm), _ptr(glabel))
  else:
    raise ValueError(mode)
  return out


def backward(mode, context, edge_weights, dcost_final, msg_min_index, msg_norm_index, rho,
             enable_sgm=False, ctx2d=None, same_label=False):
  """Restated BackwardCUDA (TRWP_backward.cu:277-433, ISGMR_backward.cu:290-493).

  Returns (dunary, dcontext, dedge_weights); dcontext is (L, L) when ctx2d else (L,), as
  allocated by the reference's Function.backward (MP_module.py:65-74).
  same_label (TRWP only): the hard backward of the TRWP_hard_soft build, whose dcontext also
  collects the pairs with current_d == front_d (TRWP_hard_soft/TRWP_backward.cu:110,194,264).
  """
  dcost_final = np.ascontiguousarray(dcost_final)
  sfx, creal = _real(dcost_final.dtype)
  dt = dcost_final.dtype
  n_iter, n_dir, b, cv, h, w, L = msg_min_index.shape
  g = _geom(n_dir, (b, cv, h, w, L), ctx2d)
  context = np.ascontiguousarray(context, dtype=dt)
  if edge_weights is None:
    edge_weights = np.ones((n_dir, b, cv, h, w), dtype=dt)
  edge_weights = np.ascontiguousarray(edge_weights, dtype=dt)
  msg_min_index = np.ascontiguousarray(msg_min_index)
  msg_norm_index = np.ascontiguousarray(msg_norm_index)
  dunary = np.zeros((b, cv, h, w, L), dtype=dt)
  dcontext = np.zeros((L, L) if g.ctx2d else (L,), dtype=dt)
  dedge = np.zeros((n_dir, b, cv, h, w), dtype=dt)
  if mode == "TRWP":
    fn = getattr(lib(), "mpo_trwp_backward_" + sfx)
    fn(ctypes.byref(g), creal(rho), int(n_iter), _ptr(context), _ptr(edge_weights),
       _ptr(dcost_final), _ptr(msg_min_index), _ptr(msg_norm_index), _ptr(dunary),
       _ptr(dcontext), _ptr(dedge), int(bool(same_label)))
  elif mode in ("ISGMR", "SGM"):
    assert not same_label
    fn = getattr(lib(), "mpo_isgmr_backward_" + sfx)
    fn(ctypes.byref(g), int(enable_sgm), creal(rho), int(n_iter), _ptr(context),
       _ptr(edge_weights), _ptr(dcost_final), _ptr(msg_min_index), _ptr(msg_norm_index),
       _ptr(dunary), _ptr(dcontext), _ptr(dedge))
  else:
    raise ValueError(mode)
  return dunary, dcontext, dedge


def refcpu_forward(mode, unary, context, n_dir, n_iter, rho, n_threads=16, ctx2d=None,
                   context_per_dir=False):
  """The reference's CPU ForwardCPU loop nest (TRWP.cpp:172-243 / ISGMR.cpp:190-298), fp32.

  context_per_dir: context is a (n_dir, L, L)-strided table as the reference's CPU path
  indexes it (`context + dir * L * L`); otherwise one table is shared by all directions.
  """
  unary = np.ascontiguousarray(unary, dtype=np.float32)
  b, cv, h, w, L = unary.shape
  g = _geom(n_dir, unary.shape, ctx2d)
  context = np.ascontiguousarray(context, dtype=np.float32)
  stride = L * L if context_per_dir else 0
  if context_per_dir:
    assert context.size >= n_dir * L * L
  msg = np.zeros((n_dir, b, cv, h, w, L), dtype=np.float32)
  cost = np.zeros((b, cv, h, w, L), dtype=np.float32)
  if mode == "TRWP":
    lib().mpo_refcpu_trwp_forward(ctypes.byref(g), ctypes.c_float(rho), int(n_iter), _ptr(unary),
                                  _ptr(context), ctypes.c_int64(stride), _ptr(msg), _ptr(cost),
                                  int(n_threads))
  else:
    msg_update = np.zeros_like(msg)
    lib().mpo_refcpu_isgmr_forward(ctypes.byref(g), ctypes.c_float(rho), int(n_iter),
                                   _ptr(unary), _ptr(context), ctypes.c_int64(stride), _ptr(msg),
                                   _ptr(msg_update), _ptr(cost), int(n_threads))
  return dict(msg=msg, cost_final=cost)


def forward_soft(unary, context, edge_weights, n_dir, n_iter, rho, training=True,
                 saving_label=False, ctx2d=None, want_gaps=False):
  """Restated ForwardCUDASoft (TRWP_hard_soft/TRWP_forward_soft.cu:378-559).

  Returns a dict with msg, cost_final, msg_edge_label (n_iter, n_dir, B, cv, H, W, L, L),
  msg_norm_index and label_all (None where switched off)."""
  unary = np.ascontiguousarray(unary)
  sfx, creal = _real(unary.dtype)
  dt = unary.dtype
  b, cv, h, w, L = unary.shape
  g = _geom(n_dir, unary.shape, ctx2d)
  context = np.ascontiguousarray(context, dtype=dt)
  if edge_weights is None:
    edge_weights = np.ones((n_dir, b, cv, h, w), dtype=dt)
  edge_weights = np.ascontiguousarray(edge_weights, dtype=dt)
  msg = np.zeros((n_dir, b, cv, h, w, L), dtype=dt)
  cost = np.zeros((b, cv, h, w, L), dtype=dt)
  mel = np.zeros((n_iter, n_dir, b, cv, h, w, L, L), dtype=dt) if training else None
  inorm = np.zeros((n_iter, n_dir, b, cv, h, w), dtype=np.uint8) if training else None
  label = np.zeros((n_iter, b, cv, h, w), dtype=np.uint8) if saving_label else None
  glabel = np.full((n_iter, b, cv, h, w), np.inf, dtype=dt) if (want_gaps and saving_label) \
      else None
  fn = getattr(lib(), "mpo_trwp_soft_forward_" + sfx)
  fn(ctypes.byref(g), creal(rho), int(n_iter), _ptr(unary), _ptr(context), _ptr(edge_weights),
     _ptr(msg), _ptr(cost), _ptr(mel), _ptr(inorm), _ptr(label), _ptr(glabel))
  return dict(msg=msg, cost_final=cost, msg_edge_label=mel, msg_norm_index=inorm, label_all=label,
              gap_label=glabel)


def backward_soft(context, edge_weights, dcost_final, msg_edge_label, msg_norm_index, rho,
                  ctx2d=None):
  """Restated BackwardCUDASoft (TRWP_hard_soft/TRWP_backward_soft.cu:422-548).
  Returns (dunary, dcontext, dedge_weights)."""
  dcost_final = np.ascontiguousarray(dcost_final)
  sfx, creal = _real(dcost_final.dtype)
  dt = dcost_final.dtype
  n_iter, n_dir, b, cv, h, w, L, _ = msg_edge_label.shape
  g = _geom(n_dir, (b, cv, h, w, L), ctx2d)
  context = np.ascontiguousarray(context, dtype=dt)
  if edge_weights is None:
    edge_weights = np.ones((n_dir, b, cv, h, w), dtype=dt)
  edge_weights = np.ascontiguousarray(edge_weights, dtype=dt)
  msg_edge_label = np.ascontiguousarray(msg_edge_label, dtype=dt)
  msg_norm_index = np.ascontiguousarray(msg_norm_index)
  dunary = np.zeros((b, cv, h, w, L), dtype=dt)
  dcontext = np.zeros((L, L) if g.ctx2d else (L,), dtype=dt)
  dedge = np.zeros((n_dir, b, cv, h, w), dtype=dt)
  fn = getattr(lib(), "mpo_trwp_soft_backward_" + sfx)
  fn(ctypes.byref(g), creal(rho), int(n_iter), _ptr(context), _ptr(edge_weights),
     _ptr(dcost_final), _ptr(msg_edge_label), _ptr(msg_norm_index), _ptr(dunary), _ptr(dcontext),
     _ptr(dedge))
  return dunary, dcontext, dedge


def soft_weighted_message(message):
  """Restated SoftWeightedMessageKernel (TRWP_hard_soft/TRWP_swbp.cu:131-200): message
  (n_trees, L, L) laid out [fd][cd].  Returns (message_soft_sum_norm (n_trees, L),
  message_soft_sum_min_ind (n_trees,) uint8, largest label on ties)."""
  m = np.asarray(message)
  e = np.exp(-(m - m.min(axis=1, keepdims=True)))       # :170-172
  prob = e / e.sum(axis=1, keepdims=True)               # :175
  soft = (m * prob).sum(axis=1)                         # :176-180
  L = m.shape[1]
  ind = (L - 1 - np.argmin(soft[:, ::-1], axis=1)).astype(np.uint8)  # :95-101
  return soft - soft.min(axis=1, keepdims=True), ind


def soft_weighted_message_back(dnorm, message, min_ind):
  """Restated SoftWeightedMessageBackKernel (TRWP_swbp.cu:203-254): gradient w.r.t. message."""
  m = np.asarray(message)
  g = np.array(dnorm, dtype=m.dtype, copy=True)
  rows = np.arange(m.shape[0])
  g[rows, min_ind] -= g.sum(axis=1)                     # :224-231
  e = np.exp(-(m - m.min(axis=1, keepdims=True)))
  prob = e / e.sum(axis=1, keepdims=True)
  soft = (m * prob).sum(axis=1, keepdims=True)
  return g[:, None, :] * prob * (1 - m + soft)          # :250
