"""Python surface of the message-passing layers: TRWPFunction, ISGMRFunction, MPModule.

Same names, arguments, return tuples and `args` namespace handling as the reference's
pytorch/MP_module.py:17-234, so a model written against it runs unchanged; the operators
underneath are the HIP library of this package instead of the CUDA extensions.

Tensor layouts (as in the reference):
  Function.apply(unary (B, cv, H, W, L), label_context (L,) or (21, 21),
                 edge_weights (n_dir, B, cv, H, W) or None, args) -> (cost_final, label_all)
  MPModule.forward(unary (B, cv, L, H, W), edge_weights (B, n_dir, H, W) or None)
                 -> (cost_final (B, cv, L, H, W), label_context[None], label_all, None, None)
"""
import torch
import torch.nn as nn

from . import _lib, lib_seg, lib_stereo
from .label_context import create_label_context
from .layout import labels_first, labels_last


def _ops_for(n_disp):
  # the reference keeps two builds and picks the segmentation one for 21 labels
  # (MP_module.py:24,95); one library backs both names here
  return lib_seg if n_disp == 21 else lib_stereo


_EMPTY_U8 = dict(dtype=torch.uint8)


def _forward_buffers(unary, args, n_dir, n_iter, with_message_tmp):
  """Allocates what the operators fill in place (MP_module.py:26-45, 97-118).  Nothing is
  zero-filled: the library writes every element that is ever read (index bytes of chain-start
  pixels stay unwritten and are never used), and the operators are told that the messages start
  at zero (msg_uninit) instead of being handed a cleared tensor, so the memsets the reference
  pays for are gone."""
  batch, cv, h, w, n_disp = unary.size()
  buf = dict(
      message=unary.new_empty(n_dir, batch, cv, h, w, n_disp),
      cost_final=unary.new_empty(batch, cv, h, w, n_disp),
      unary_update=unary.new_empty(batch, cv, h, w, n_disp))
  if with_message_tmp:
    buf["message_tmp"] = unary.new_empty(n_dir, batch, cv, h, w, n_disp)
  if args.training:
    buf["message_index"] = unary.new_empty(n_iter, n_dir, batch, cv, h, w, n_disp, **_EMPTY_U8)
    buf["cost_index"] = unary.new_empty(n_iter, n_dir, batch, cv, h, w, **_EMPTY_U8)
  else:
    buf["message_index"] = torch.empty(0, **_EMPTY_U8)
    buf["cost_index"] = torch.empty(0, **_EMPTY_U8)
  if args.enable_saving_label:
    buf["label_all"] = unary.new_empty(n_iter, batch, cv, h, w, **_EMPTY_U8)
  else:
    buf["label_all"] = torch.empty(0, **_EMPTY_U8)
  return buf


def _backward_buffers(dcost_final, message_index, with_message_tmp, need_context=True,
                      need_edge_weights=True):
  """Allocates the gradient tensors (MP_module.py:65-74, 139-150).  dedge_weights and
  dlabel_context accumulate and start at zero; dunary is written everywhere and the scratch
  tensors are written before they are read.  A gradient autograd does not ask for (a fixed
  pairwise table, no edge weights or ones that are not learned) is an empty tensor: the operators
  then leave that part of the reverse scan out."""
  n_iter, n_dir, batch, cv, h, w, n_disp = message_index.size()
  buf = dict(
      dunary=dcost_final.new_empty(batch, cv, h, w, n_disp),
      dmessage=dcost_final.new_empty(n_dir, batch, cv, h, w, n_disp),
      dunary_update=dcost_final.new_empty(0))
  if need_edge_weights:
    buf["dedge_weights"] = dcost_final.new_zeros(n_dir, batch, cv, h, w)
  else:
    buf["dedge_weights"] = dcost_final.new_empty(0)
  if with_message_tmp:
    buf["dmessage_tmp"] = dcost_final.new_empty(n_dir, batch, cv, h, w, n_disp)
  if not need_context:
    buf["dlabel_context"] = dcost_final.new_empty(0)
  elif n_disp == 21:
    buf["dlabel_context"] = dcost_final.new_zeros(n_disp, n_disp)
  else:
    buf["dlabel_context"] = dcost_final.new_zeros(n_disp)
  return buf


def _table_flags(args):
  """MPL_F_DENSE_TABLE when the module says its pairwise table is dense (not in the reference: the
  kind of the table is only known on the device otherwise, see include/mplayers_amd.h)."""
  return _lib.F_DENSE_TABLE if getattr(args, "dense_table", False) else 0


class TRWPFunction(torch.autograd.Function):
  """Tree-reweighted message passing, Gauss-Seidel over directions (MP_module.py:17-86)."""

  @staticmethod
  def forward(ctx, unary, label_context, edge_weights, args):
    n_disp = unary.size(4)
    rho, n_iter, n_dir = args.rho, int(args.mpnet_max_iter), int(args.mpnet_n_dirs)
    buf = _forward_buffers(unary, args, n_dir, n_iter, with_message_tmp=False)
    enable_edge_weights = edge_weights is not None
    if not enable_edge_weights:
      edge_weights = unary.new_ones((n_dir,) + tuple(unary.shape[:4]))
    _ops_for(n_disp).TRWP.forward(rho, n_iter, int(args.enable_min_a_dir), unary, label_context,
                                  edge_weights, buf["message"], buf["cost_final"],
                                  buf["message_index"], buf["cost_index"], buf["unary_update"],
                                  buf["label_all"], msg_uninit=True, flags=_table_flags(args))
    ctx.intermediate_results = (rho, buf["message_index"], buf["cost_index"], label_context,
                                edge_weights, enable_edge_weights)
    return buf["cost_final"], buf["label_all"]

  @staticmethod
  def backward(ctx, dcost_final, dmessage_all):
    rho, message_index, cost_index, label_context, edge_weights, enable_edge_weights = \
        ctx.intermediate_results
    del ctx.intermediate_results
    dcost_final = dcost_final.contiguous()
    n_disp = message_index.size(6)
    need_context = ctx.needs_input_grad[1]
    need_edge_weights = enable_edge_weights and ctx.needs_input_grad[2]
    buf = _backward_buffers(dcost_final, message_index, False, need_context, need_edge_weights)
    _ops_for(n_disp).TRWP.backward(rho, label_context, edge_weights, dcost_final, message_index,
                                   cost_index, buf["dunary"], buf["dlabel_context"],
                                   buf["dedge_weights"], buf["dmessage"], buf["dunary_update"])
    return (buf["dunary"], buf["dlabel_context"] if need_context else None,
            buf["dedge_weights"] if need_edge_weights else None, None)


class ISGMRFunction(torch.autograd.Function):
  """Iterative semi-global matching revised, Jacobi over directions (MP_module.py:89-161)."""

  @staticmethod
  def forward(ctx, unary, label_context, edge_weights, args):
    n_disp = unary.size(4)
    rho, n_iter, n_dir = args.rho, int(args.mpnet_max_iter), int(args.mpnet_n_dirs)
    buf = _forward_buffers(unary, args, n_dir, n_iter, with_message_tmp=True)
    enable_edge_weights = edge_weights is not None
    if not enable_edge_weights:
      edge_weights = unary.new_ones((n_dir,) + tuple(unary.shape[:4]))
    _ops_for(n_disp).ISGMR.forward(int(args.enable_sgm), rho, n_iter, int(args.enable_min_a_dir),
                                   unary, label_context, edge_weights, buf["message"],
                                   buf["cost_final"], buf["message_index"], buf["cost_index"],
                                   buf["unary_update"], buf["message_tmp"], buf["label_all"],
                                   msg_uninit=True, flags=_table_flags(args))
    ctx.intermediate_results = (args.enable_sgm, rho, buf["message_index"], buf["cost_index"],
                                label_context, edge_weights, enable_edge_weights)
    return buf["cost_final"], buf["label_all"]

  @staticmethod
  def backward(ctx, dcost_final, dmessage_all):
    enable_sgm, rho, message_index, cost_index, label_context, edge_weights, \
        enable_edge_weights = ctx.intermediate_results
    del ctx.intermediate_results
    dcost_final = dcost_final.contiguous()
    n_disp = message_index.size(6)
    need_context = ctx.needs_input_grad[1]
    need_edge_weights = enable_edge_weights and ctx.needs_input_grad[2]
    buf = _backward_buffers(dcost_final, message_index, True, need_context, need_edge_weights)
    _ops_for(n_disp).ISGMR.backward(int(enable_sgm), rho, label_context, edge_weights,
                                    dcost_final, message_index, cost_index, buf["dunary"],
                                    buf["dlabel_context"], buf["dedge_weights"], buf["dmessage"],
                                    buf["dunary_update"], buf["dmessage_tmp"])
    return (buf["dunary"], buf["dlabel_context"] if need_context else None,
            buf["dedge_weights"] if need_edge_weights else None, None)


class MPModule(torch.nn.Module):
  """nn.Module wrapper (MP_module.py:164-234).

  Reads from `args`: mpnet_mrf_mode ('TRWP' | 'ISGMR' | 'SGM'), mpnet_max_iter, mpnet_n_dirs,
  n_classes, mpnet_term_weight, mpnet_smoothness_train, mpnet_diag_value, enable_symmetric (and the
  fields create_label_context needs); writes rho (0.5 for TRWP, else 1), enable_saving_label,
  enable_min_a_dir, enable_sgm, enable_seg and, per call, training -- as the reference does.
  """

  def __init__(self, args, enable_create_label_context=False, enable_saving_label=False,
               enable_min_a_dir=False):
    super(MPModule, self).__init__()
    self.args = args
    self.args.rho = 0.5 if (args.mpnet_mrf_mode == 'TRWP') else 1
    self.args.enable_saving_label = enable_saving_label
    self.args.enable_min_a_dir = enable_min_a_dir
    self.args.enable_sgm = args.mpnet_mrf_mode == 'SGM'
    self.args.enable_seg = True if (args.n_classes == 21) else False
    if enable_create_label_context:
      self.create_label_context()

  def _fixed_table_is_dense(self, label_context):
    """Whether the forward scans take their O(L^2) step on the 1-D table the kernels read (the
    first n_classes entries of label_context), asked once per table: the answer is kept until the
    stored table is replaced or written to.  It only matters above 64 labels."""
    n_disp = int(self.args.n_classes)
    if n_disp <= 64 or not label_context.is_cuda:
      return False
    key = (self.label_context.data_ptr(), self.label_context._version)
    if getattr(self, "_dense_key", None) != key:
      if torch.cuda.is_current_stream_capturing():
        return False  # no copy to the host inside a capture; the flag is a hint
      self._dense_key = key
      self._dense_answer = _lib.table_is_dense(label_context.reshape(-1)[:n_disp])
    return self._dense_answer

  def get_label_context(self):
    return self.label_context, self.label_context_loc, self.label_context_diag_loc

  def set_label_context(self, label_context, label_context_loc, label_context_diag_loc):
    self.label_context = label_context
    self.label_context_loc = label_context_loc
    self.label_context_diag_loc = label_context_diag_loc

  def create_label_context(self):
    self.label_context, self.label_context_loc, self.label_context_diag_loc = \
        create_label_context(self.args, enable_seg=self.args.enable_seg,
                             enable_symmetric=self.args.enable_symmetric)

  def _effective_label_context(self, weight_first=False):
    """Re-parameterisation of the learned context (MP_module.py:207-220).  weight_first: the term
    weight scales the stored parameter before the re-parameterisation instead of the sigmoid's
    output (the hard/soft module, MP_module_hard_soft.py:148-163)."""
    term_weight = self.args.mpnet_term_weight
    label_context = self.label_context * (term_weight if weight_first else 1)
    mode = self.args.mpnet_smoothness_train
    if mode == 'sigmoid':
      valid = label_context[self.label_context_loc].flatten()
      scale = 2 if weight_first else 2 * term_weight
      label_context[self.label_context_loc] = scale * torch.sigmoid(valid)
    elif mode == 'softmax':
      valid = label_context[self.label_context_loc].flatten()
      norm = nn.Softmax(dim=0)(valid)
      label_context[self.label_context_loc] = norm * valid.max() / norm.max()
    if mode in {'sigmoid', 'softmax'}:
      diag = self.label_context_diag_loc
      label_context[tuple(diag) if isinstance(diag, list) else diag] = self.args.mpnet_diag_value
    return label_context

  def forward(self, unary, edge_weights=None):
    # label axis innermost for the kernels; direction axis outermost for the edge weights
    unary = labels_last(unary)
    if edge_weights is not None:
      edge_weights = edge_weights.unsqueeze(1).permute(2, 0, 1, 3, 4).contiguous()
      assert unary.size()[-3:-1] == edge_weights.size()[-2:]
    if unary.is_cuda and (self.args.mpnet_mrf_mode == 'SGM'):
      assert self.args.mpnet_max_iter == 1
    label_context = self._effective_label_context()
    self.args.training = self.training
    # a table that is being learned is dense in general and a fixed one is looked at once, on the
    # host; args.mpnet_dense_table overrides both
    dense = getattr(self.args, "mpnet_dense_table", None)
    if dense is None:
      dense = self.label_context.requires_grad or self._fixed_table_is_dense(label_context)
    self.args.dense_table = bool(dense)
    if self.args.mpnet_mrf_mode in {'ISGMR', 'SGM'}:
      cost_final, cost_all = ISGMRFunction.apply(unary, label_context, edge_weights, self.args)
    elif self.args.mpnet_mrf_mode == 'TRWP':
      cost_final, cost_all = TRWPFunction.apply(unary, label_context, edge_weights, self.args)
    else:
      assert False
    cost_final = labels_first(cost_final)
    return cost_final, label_context.unsqueeze(0), cost_all, None, None
