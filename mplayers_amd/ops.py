"""Operator layer with the reference's extension signatures (lib_stereo / lib_seg modules).

`TRWP.forward/backward` and `ISGMR.forward/backward` take exactly the positional arguments of
the reference's pybind11 modules (MPLayers/TRWP/TRWP.cpp:245-256, 285-295, 324-325 and
MPLayers/ISGMR/ISGMR.cpp:300-313, 344-356, 400-401): caller-allocated, zero-filled tensors that
are filled in place; an empty index / label tensor switches that output off.  They hand raw device
pointers and the current HIP stream to the C ABI of libmplayers_hip.so.

CPU tensors take the CPU forward of the library (mpl_trwp_forward_cpu / mpl_isgmr_forward_cpu), as
the reference's operators run ForwardCPU for them (TRWP.cpp:275-282, ISGMR.cpp:330-339), with
that path's own semantics: no edge weights, no indices, the table of direction d at
context + d * L * L.

Deviations from the reference, all towards failing loudly: more labels than 256 (the reference
prints a message and returns zero-filled outputs, TRWP.cpp:269-273), a backward call on CPU tensors
(the reference prints "Does not support CPU backward" and returns, :315-316), tensors on different
devices and non-contiguous tensors raise RuntimeError.
"""
import torch

from . import _lib


def _ptr(t):
  return None if t is None or t.numel() == 0 else t.data_ptr()


def _check(name, t, dtype, numel=None, cuda=True):
  if not isinstance(t, torch.Tensor):
    raise TypeError("%s must be a tensor" % name)
  if cuda and not t.is_cuda:
    raise RuntimeError("%s is not on the GPU like the other tensors of the call" % name)
  if not cuda and t.is_cuda:
    raise RuntimeError("%s is on the GPU, the other tensors of the call are not" % name)
  if not t.is_contiguous():
    raise RuntimeError("%s must be contiguous" % name)  # CHECK_CONTIGUOUS, cudaUtils.hpp:10
  if t.dtype != dtype:
    raise RuntimeError("%s must be %s, got %s" % (name, dtype, t.dtype))
  if numel is not None and t.numel() < numel:
    raise RuntimeError("%s has %d elements, %d needed" % (name, t.numel(), numel))


def _context_numel(L, ctx2d):
  return L * L if ctx2d else L


def _wanted(t):
  """An output gradient the caller has no use for is passed as None or as an empty tensor, the
  reference's way of switching an output off (TRWP_forward.cu:406-408)."""
  return t is not None and t.numel() > 0


class _Op(object):
  """Shared plumbing of the two operator namespaces."""

  @staticmethod
  def _shape_from_msg(msg):
    if msg.dim() != 6:
      raise RuntimeError("msg must be (n_dir, batch, cv, h, w, n_disp)")
    n_dir, b, cv, h, w, L = msg.shape
    ctx2d = (L == 21)  # the reference switches to the (L, L) table by n_disp == 21
    return _lib.Shape(n_dir, b * cv, h, w, L, int(ctx2d)), b * cv * h * w, L, ctx2d

  @staticmethod
  def _shape_from_index(msg_min_index):
    if msg_min_index.dim() != 7:
      raise RuntimeError("msg_min_index must be (n_iter, n_dir, batch, cv, h, w, n_disp)")
    n_iter, n_dir, b, cv, h, w, L = msg_min_index.shape
    ctx2d = (L == 21)
    return _lib.Shape(n_dir, b * cv, h, w, L, int(ctx2d)), n_iter, b * cv * h * w, L, ctx2d

  @staticmethod
  def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream

  @staticmethod
  def _check_forward(unary, context, edge_weights, msg, cost_final, msg_min_index,
                     msg_norm_index, unary_update, label_all, n_iter):
    shape, P, L, ctx2d = _Op._shape_from_msg(msg)
    N = P * L
    f32, u8 = torch.float32, torch.uint8
    _check("unary", unary, f32, N)
    _check("context", context, f32, _context_numel(L, ctx2d))
    _check("edge_weights", edge_weights, f32, shape.n_dir * P)
    _check("msg", msg, f32, shape.n_dir * N)
    _check("cost_final", cost_final, f32, N)
    _check("unary_update", unary_update, f32, N)
    training = msg_min_index.numel() > 0
    if training:
      _check("msg_min_index", msg_min_index, u8, n_iter * shape.n_dir * N)
      _check("msg_norm_index", msg_norm_index, u8, n_iter * shape.n_dir * P)
    if label_all.numel() > 0:
      _check("label_all", label_all, u8, n_iter * P)
    return shape, P, N


def _no_cpu_backward(t):
  if isinstance(t, torch.Tensor) and not t.is_cuda:
    raise RuntimeError("Does not support CPU backward.")  # TRWP.cpp:315-316, ISGMR.cpp:377-378


def _forward_cpu(mode, enable_sgm, rho, n_iter, unary, context, msg, cost_final, msg_update,
                 label_all):
  """ForwardCPU of the reference (TRWP.cpp:172-243, ISGMR.cpp:190-298) through the library's CPU
  entry points.  edge_weights, the index tensors and unary_update play no part in that path."""
  lib = _lib.load()
  shape, P, L, ctx2d = _Op._shape_from_msg(msg)
  N = P * L
  f32 = torch.float32
  _check("unary", unary, f32, N, cuda=False)
  # the table of direction d is read at context + d * L * L
  _check("context", context, f32, (shape.n_dir - 1) * L * L + _context_numel(L, ctx2d), cuda=False)
  _check("msg", msg, f32, shape.n_dir * N, cuda=False)
  _check("cost_final", cost_final, f32, N, cuda=False)
  if label_all.numel() > 0:
    _check("label_all", label_all, torch.uint8, n_iter * P, cuda=False)
  if mode == "TRWP":
    rc = lib.mpl_trwp_forward_cpu(shape, float(rho), int(n_iter), _ptr(unary), _ptr(context),
                                  _ptr(msg), _ptr(cost_final), _ptr(label_all))
  else:
    _check("msg_update", msg_update, f32, shape.n_dir * N, cuda=False)
    rc = lib.mpl_isgmr_forward_cpu(shape, int(enable_sgm), float(rho), int(n_iter), _ptr(unary),
                                   _ptr(context), _ptr(msg), _ptr(cost_final), _ptr(msg_update),
                                   _ptr(label_all))
  _lib.check(rc, mode + ".forward (CPU)")


class TRWP(object):
  """Drop-in for the reference's `lib_stereo.TRWP` / `lib_seg.TRWP` extension modules."""

  @staticmethod
  def forward(rho, n_iter, enable_min_a_dir, unary, context, edge_weights, msg, cost_final,
              msg_min_index, msg_norm_index, unary_update, label_all, msg_uninit=False, flags=0):
    """msg_uninit (not in the reference): True declares that `msg` holds no initial messages --
    they start at zero and the library writes every element, so the caller need not clear it.
    flags (not in the reference): further per-call MPL_F_* bits of the C ABI."""
    if isinstance(unary, torch.Tensor) and not unary.is_cuda:
      if msg_uninit:
        msg.zero_()
      return _forward_cpu("TRWP", 0, rho, n_iter, unary, context, msg, cost_final, None, label_all)
    lib = _lib.load()
    shape, _, _ = _Op._check_forward(unary, context, edge_weights, msg, cost_final, msg_min_index,
                                     msg_norm_index, unary_update, label_all, n_iter)
    flags = int(flags) | (_lib.F_MSG_UNINIT if msg_uninit else 0)
    with torch.cuda.device(unary.device):
      rc = lib.mpl_trwp_forward(shape, flags, float(rho), int(n_iter), int(enable_min_a_dir),
                                _ptr(unary), _ptr(context), _ptr(edge_weights), _ptr(msg),
                                _ptr(cost_final), _ptr(msg_min_index), _ptr(msg_norm_index),
                                _ptr(unary_update), _ptr(label_all), _Op._stream(unary))
    _lib.check(rc, "TRWP.forward")

  @staticmethod
  def backward(rho, context, edge_weights, dcost_final, msg_min_index, msg_norm_index, dunary,
               dcontext, dedge_weights, dmsg, dunary_update, flags=0):
    """dcontext / dedge_weights: None or an empty tensor when that gradient is not wanted (not in
    the reference, which always computes both); flags: per-call MPL_F_* bits of the C ABI."""
    _no_cpu_backward(dcost_final)
    lib = _lib.load()
    shape, n_iter, P, L, ctx2d = _Op._shape_from_index(msg_min_index)
    N = P * L
    f32, u8 = torch.float32, torch.uint8
    _check("context", context, f32, _context_numel(L, ctx2d))
    _check("edge_weights", edge_weights, f32, shape.n_dir * P)
    _check("dcost_final", dcost_final, f32, N)
    _check("msg_min_index", msg_min_index, u8, n_iter * shape.n_dir * N)
    _check("msg_norm_index", msg_norm_index, u8, n_iter * shape.n_dir * P)
    _check("dunary", dunary, f32, N)
    if _wanted(dcontext):
      _check("dcontext", dcontext, f32, _context_numel(L, ctx2d))
    if _wanted(dedge_weights):
      _check("dedge_weights", dedge_weights, f32, shape.n_dir * P)
    _check("dmsg", dmsg, f32, shape.n_dir * N)
    with torch.cuda.device(dcost_final.device):
      rc = lib.mpl_trwp_backward(shape, int(flags), float(rho), int(n_iter), _ptr(context),
                                 _ptr(edge_weights), _ptr(dcost_final), _ptr(msg_min_index),
                                 _ptr(msg_norm_index), _ptr(dunary), _ptr(dcontext),
                                 _ptr(dedge_weights), _ptr(dmsg), _ptr(dunary_update),
                                 _Op._stream(dcost_final))
    _lib.check(rc, "TRWP.backward")


class ISGMR(object):
  """Drop-in for the reference's `lib_stereo.ISGMR` / `lib_seg.ISGMR` extension modules."""

  @staticmethod
  def forward(enable_sgm, rho, n_iter, enable_min_a_dir, unary, context, edge_weights, msg,
              cost_final, msg_min_index, msg_norm_index, unary_update, msg_update, label_all,
              msg_uninit=False, flags=0):
    """msg_uninit, flags (not in the reference): see TRWP.forward."""
    if isinstance(unary, torch.Tensor) and not unary.is_cuda:
      if msg_uninit:
        msg.zero_()
        msg_update.zero_()
      return _forward_cpu("ISGMR", enable_sgm, rho, n_iter, unary, context, msg, cost_final,
                          msg_update, label_all)
    lib = _lib.load()
    shape, _, N = _Op._check_forward(unary, context, edge_weights, msg, cost_final, msg_min_index,
                                     msg_norm_index, unary_update, label_all, n_iter)
    flags = int(flags) | (_lib.F_MSG_UNINIT if msg_uninit else 0)
    _check("msg_update", msg_update, torch.float32, shape.n_dir * N)
    with torch.cuda.device(unary.device):
      rc = lib.mpl_isgmr_forward(shape, flags, int(enable_sgm), float(rho), int(n_iter),
                                 int(enable_min_a_dir), _ptr(unary), _ptr(context),
                                 _ptr(edge_weights), _ptr(msg), _ptr(cost_final),
                                 _ptr(msg_min_index), _ptr(msg_norm_index), _ptr(unary_update),
                                 _ptr(msg_update), _ptr(label_all), _Op._stream(unary))
    _lib.check(rc, "ISGMR.forward")

  @staticmethod
  def backward(enable_sgm, rho, context, edge_weights, dcost_final, msg_min_index,
               msg_norm_index, dunary, dcontext, dedge_weights, dmsg, dunary_update, dmsg_update,
               flags=0):
    """dcontext / dedge_weights / flags: see TRWP.backward."""
    _no_cpu_backward(dcost_final)
    lib = _lib.load()
    shape, n_iter, P, L, ctx2d = _Op._shape_from_index(msg_min_index)
    N = P * L
    f32, u8 = torch.float32, torch.uint8
    _check("context", context, f32, _context_numel(L, ctx2d))
    _check("edge_weights", edge_weights, f32, shape.n_dir * P)
    _check("dcost_final", dcost_final, f32, N)
    _check("msg_min_index", msg_min_index, u8, n_iter * shape.n_dir * N)
    _check("msg_norm_index", msg_norm_index, u8, n_iter * shape.n_dir * P)
    _check("dunary", dunary, f32, N)
    if _wanted(dcontext):
      _check("dcontext", dcontext, f32, _context_numel(L, ctx2d))
    if _wanted(dedge_weights):
      _check("dedge_weights", dedge_weights, f32, shape.n_dir * P)
    _check("dmsg_update", dmsg_update, f32, shape.n_dir * N)
    # dmsg is optional scratch: used when it has the reference's full size, ignored otherwise
    if not (isinstance(dmsg, torch.Tensor) and dmsg.is_cuda and dmsg.is_contiguous() and
            dmsg.dtype == f32 and dmsg.numel() >= shape.n_dir * N):
      dmsg = None
    with torch.cuda.device(dcost_final.device):
      rc = lib.mpl_isgmr_backward(shape, int(flags), int(enable_sgm), float(rho), int(n_iter),
                                  _ptr(context),
                                  _ptr(edge_weights), _ptr(dcost_final), _ptr(msg_min_index),
                                  _ptr(msg_norm_index), _ptr(dunary), _ptr(dcontext),
                                  _ptr(dedge_weights), _ptr(dmsg), _ptr(dunary_update),
                                  _ptr(dmsg_update), _Op._stream(dcost_final))
    _lib.check(rc, "ISGMR.backward")


class TRWP_hard_soft(object):
  """Drop-in for the reference's `lib_stereo.TRWP_hard_soft` / `lib_seg.TRWP_hard_soft` extension
  modules (MPLayers/TRWP_hard_soft/TRWP.cpp:428-445): the hard operators under the same names as
  in `TRWP`, plus `forward_soft` / `backward_soft` and the stand-alone softmin of stored blocks,
  `soft_weighted_message` / `soft_weighted_message_back`."""

  forward = TRWP.forward

  @staticmethod
  def backward(rho, context, edge_weights, dcost_final, msg_min_index, msg_norm_index, dunary,
               dcontext, dedge_weights, dmsg, dunary_update, flags=0):
    """The hard backward of this build differs from TRWP.backward in one point: dcontext also
    collects the pairs whose front label equals their own (entry 0 of a 1-D table, the diagonal of
    a 2-D one): TRWP_hard_soft/TRWP_backward.cu:110,194,264 have no `current_d != front_d` guard
    (TRWP/TRWP_backward.cu:111-112 has)."""
    TRWP.backward(rho, context, edge_weights, dcost_final, msg_min_index, msg_norm_index, dunary,
                  dcontext, dedge_weights, dmsg, dunary_update,
                  flags=int(flags) | _lib.F_DCONTEXT_SAME_LABEL)

  @staticmethod
  def forward_soft(rho, n_iter, unary, context, edge_weights, msg, msg_edge_label, msg_norm_index,
                   cost_final, unary_update, label_all, flags=0):
    lib = _lib.load()
    shape, P, L, ctx2d = _Op._shape_from_msg(msg)
    N = P * L
    f32, u8 = torch.float32, torch.uint8
    _check("unary", unary, f32, N)
    _check("context", context, f32, _context_numel(L, ctx2d))
    _check("edge_weights", edge_weights, f32, shape.n_dir * P)
    _check("msg", msg, f32, shape.n_dir * N)
    _check("cost_final", cost_final, f32, N)
    _check("unary_update", unary_update, f32, N)
    if msg_edge_label.numel() > 0:
      _check("msg_edge_label", msg_edge_label, f32, n_iter * shape.n_dir * N * L)
      _check("msg_norm_index", msg_norm_index, u8, n_iter * shape.n_dir * P)
    if label_all.numel() > 0:
      _check("label_all", label_all, u8, n_iter * P)
    with torch.cuda.device(unary.device):
      rc = lib.mpl_trwp_soft_forward(shape, int(flags), float(rho), int(n_iter), _ptr(unary), _ptr(context),
                                     _ptr(edge_weights), _ptr(msg), _ptr(msg_edge_label),
                                     _ptr(msg_norm_index), _ptr(cost_final), _ptr(unary_update),
                                     _ptr(label_all), _Op._stream(unary))
    _lib.check(rc, "TRWP_hard_soft.forward_soft")

  @staticmethod
  def backward_soft(rho, dcost_final, context, edge_weights, msg_edge_label, msg_norm_index,
                    dunary, dcontext, dedge_weights, dmsg, dunary_update, flags=0):
    lib = _lib.load()
    if msg_norm_index.dim() != 6:
      raise RuntimeError("msg_norm_index must be (n_iter, n_dir, batch, cv, h, w)")
    n_iter, n_dir, b, cv, h, w = msg_norm_index.shape
    L = dcost_final.size(-1)
    ctx2d = (L == 21)
    shape = _lib.Shape(n_dir, b * cv, h, w, L, int(ctx2d))
    P = b * cv * h * w
    N = P * L
    f32, u8 = torch.float32, torch.uint8
    _check("dcost_final", dcost_final, f32, N)
    _check("context", context, f32, _context_numel(L, ctx2d))
    _check("edge_weights", edge_weights, f32, n_dir * P)
    _check("msg_edge_label", msg_edge_label, f32, n_iter * n_dir * N * L)
    _check("msg_norm_index", msg_norm_index, u8, n_iter * n_dir * P)
    _check("dunary", dunary, f32, N)
    if _wanted(dcontext):
      _check("dcontext", dcontext, f32, _context_numel(L, ctx2d))
    if _wanted(dedge_weights):
      _check("dedge_weights", dedge_weights, f32, n_dir * P)
    _check("dmsg", dmsg, f32, n_dir * N)
    with torch.cuda.device(dcost_final.device):
      rc = lib.mpl_trwp_soft_backward(shape, int(flags), float(rho), int(n_iter), _ptr(dcost_final),
                                      _ptr(context), _ptr(edge_weights), _ptr(msg_edge_label),
                                      _ptr(msg_norm_index), _ptr(dunary), _ptr(dcontext),
                                      _ptr(dedge_weights), _ptr(dmsg), _ptr(dunary_update),
                                      _Op._stream(dcost_final))
    _lib.check(rc, "TRWP_hard_soft.backward_soft")

  @staticmethod
  def soft_weighted_message(message, message_soft_sum_norm, message_soft_sum_min_ind):
    """message (n_trees, L, L) [fd][cd] -> normalised soft message sums (n_trees, L) and the label
    of their minimum (n_trees) uint8; TRWP.cpp:385-400."""
    lib = _lib.load()
    if message.dim() != 3 or message.size(1) != message.size(2):
      raise RuntimeError("message must be (n_trees, n_disp, n_disp)")
    n_trees, L, _ = message.shape
    _check("message", message, torch.float32)
    _check("message_soft_sum_norm", message_soft_sum_norm, torch.float32, n_trees * L)
    _check("message_soft_sum_min_ind", message_soft_sum_min_ind, torch.uint8, n_trees)
    with torch.cuda.device(message.device):
      rc = lib.mpl_soft_weighted_message(n_trees, L, _ptr(message), _ptr(message_soft_sum_norm),
                                         _ptr(message_soft_sum_min_ind), _Op._stream(message))
    _lib.check(rc, "TRWP_hard_soft.soft_weighted_message")

  @staticmethod
  def soft_weighted_message_back(dmessage_soft_sum_norm, message, message_soft_sum_min_ind,
                                 dmessage):
    """Gradient of soft_weighted_message with respect to message; TRWP.cpp:402-417."""
    lib = _lib.load()
    if message.dim() != 3 or message.size(1) != message.size(2):
      raise RuntimeError("message must be (n_trees, n_disp, n_disp)")
    n_trees, L, _ = message.shape
    _check("dmessage_soft_sum_norm", dmessage_soft_sum_norm, torch.float32, n_trees * L)
    _check("message", message, torch.float32)
    _check("message_soft_sum_min_ind", message_soft_sum_min_ind, torch.uint8, n_trees)
    _check("dmessage", dmessage, torch.float32, n_trees * L * L)
    with torch.cuda.device(message.device):
      rc = lib.mpl_soft_weighted_message_back(n_trees, L, _ptr(dmessage_soft_sum_norm),
                                              _ptr(message), _ptr(message_soft_sum_min_ind),
                                              _ptr(dmessage), _Op._stream(message))
    _lib.check(rc, "TRWP_hard_soft.soft_weighted_message_back")
