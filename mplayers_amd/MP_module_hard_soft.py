"""Python surface of the hard/soft TRWP layer: TRWPFunction and MPModule with the names, arguments
and return tuples of the reference's pytorch/MP_module_hard_soft.py:13-182 (the module mpnet.py:35
builds its CRF layer from).  `args.mpnet_enable_soft` switches between the min-sum operator and the
soft-weighted one; everything runs in the HIP library of this package.

  TRWPFunction.apply(unary (B, cv, H, W, L), label_context, edge_weights (n_dir, B, cv, H, W) | None,
                     args) -> (cost_final, label_all, message_edge_label, cost_index)
  MPModule.forward(unary (B, cv, L, H, W), edge_weights (B, n_dir, H, W) | None, msg_norm_index=None,
                   pairwise_terms=None)
                   -> (cost_final (B, cv, L, H, W), label_context[None], label_all,
                       message_edge_label, cost_index)
"""
import torch
import torch.nn as nn

from . import lib_seg, lib_stereo
from .label_context import create_label_context


def _ops_for(n_disp):
  # MP_module_hard_soft.py:20: the segmentation build for 21 labels, the stereo build otherwise
  return (lib_seg if n_disp == 21 else lib_stereo).TRWP_hard_soft


class TRWPFunction(torch.autograd.Function):
  """MP_module_hard_soft.py:13-108."""

  @staticmethod
  def forward(ctx, unary, label_context, edge_weights, args):
    batch, cv, h, w, n_disp = unary.size()
    rho, n_iter, n_dir = args.rho, int(args.mpnet_max_iter), int(args.mpnet_n_dirs)
    training = args.training
    ops = _ops_for(n_disp)
    u8 = dict(dtype=torch.uint8)
    # only the initial messages have to be zero; the library writes every element of the other
    # tensors that is read later, except the stored duals of chain-start pixels, which callers
    # can see in the returned tensor and which therefore start at zero as in the reference
    message = unary.new_zeros(n_dir, batch, cv, h, w, n_disp)
    cost_final = unary.new_empty(batch, cv, h, w, n_disp)
    unary_update = unary.new_empty(batch, cv, h, w, n_disp)
    enable_edge_weights = edge_weights is not None
    if not enable_edge_weights:
      edge_weights = unary.new_ones(n_dir, batch, cv, h, w)
    label_all = (unary.new_empty(n_iter, batch, cv, h, w, **u8) if args.enable_saving_label
                 else torch.empty(0, **u8))
    if args.mpnet_enable_soft:
      if training:
        message_edge_label = unary.new_zeros(n_iter, n_dir, batch, cv, h, w, n_disp, n_disp)
        cost_index = unary.new_zeros(n_iter, n_dir, batch, cv, h, w, **u8)
      else:
        message_edge_label = torch.empty(0, dtype=torch.float32)
        cost_index = torch.empty(0, **u8)
      ops.forward_soft(rho, n_iter, unary, label_context, edge_weights, message,
                       message_edge_label, cost_index, cost_final, unary_update, label_all)
      message_index = torch.empty(0, dtype=torch.float32)
    else:
      if training:
        message_index = unary.new_empty(n_iter, n_dir, batch, cv, h, w, n_disp, **u8)
        cost_index = unary.new_zeros(n_iter, n_dir, batch, cv, h, w, **u8)
      else:
        message_index = torch.empty(0, **u8)
        cost_index = torch.empty(0, **u8)
      ops.forward(rho, n_iter, 0, unary, label_context, edge_weights, message, cost_final,
                  message_index, cost_index, unary_update, label_all)
      message_edge_label = torch.empty(0, dtype=torch.float32)
    ctx.intermediate_results = (rho, args, message_edge_label, message_index, cost_index,
                                label_context, edge_weights, enable_edge_weights)
    return cost_final, label_all, message_edge_label, cost_index

  @staticmethod
  def backward(ctx, dcost_final, dlabel_all, dmessage_edge_label, dcost_index):
    dcost_final = dcost_final.contiguous()
    rho, args, message_edge_label, message_index, cost_index, label_context, edge_weights, \
        enable_edge_weights = ctx.intermediate_results
    del ctx.intermediate_results
    # a caller may impose the normalisation indices (MP_module_hard_soft.py:77)
    cost_index = args.msg_norm_index if (args.msg_norm_index is not None) else cost_index
    n_iter, n_dir, batch, cv, h, w = cost_index.size()
    n_disp = args.n_classes
    ops = _ops_for(n_disp)
    dunary = dcost_final.new_empty(batch, cv, h, w, n_disp)
    dmessage = dcost_final.new_empty(n_dir, batch, cv, h, w, n_disp)
    dunary_update = dcost_final.new_empty(0)
    dedge_weights = dcost_final.new_zeros(n_dir, batch, cv, h, w)
    if args.enable_seg:
      dlabel_context = dcost_final.new_zeros(n_disp, n_disp)
    else:
      dlabel_context = dcost_final.new_zeros(n_disp)
    if args.mpnet_enable_soft:
      ops.backward_soft(rho, dcost_final, label_context, edge_weights, message_edge_label,
                        cost_index, dunary, dlabel_context, dedge_weights, dmessage, dunary_update)
    else:
      ops.backward(rho, label_context, edge_weights, dcost_final, message_index, cost_index,
                   dunary, dlabel_context, dedge_weights, dmessage, dunary_update)
    dedge_weights = dedge_weights if enable_edge_weights else None
    return dunary, dlabel_context, dedge_weights, None, None, None


class MPModule(torch.nn.Module):
  """MP_module_hard_soft.py:111-182.  Reads from `args`: mpnet_mrf_mode ('TRWP'), mpnet_enable_soft,
  mpnet_max_iter, mpnet_n_dirs, n_classes, mpnet_term_weight, mpnet_smoothness_train / _mode /
  _trunct_value / _trunct_loc, mpnet_diag_value, enable_symmetric; writes rho, enable_saving_label,
  enable_seg and, per call, training and msg_norm_index."""

  def __init__(self, args, enable_create_label_context=False, enable_saving_label=False):
    super(MPModule, self).__init__()
    self.args = args
    self.args.enable_saving_label = enable_saving_label
    self.args.rho = 0.5 if (args.mpnet_mrf_mode == 'TRWP') else 1
    self.args.enable_seg = True if (args.n_classes == 21) else False
    self.smoothness_train = args.mpnet_smoothness_train if args.mpnet_smoothness_train else None
    self.smoothness_mode = args.mpnet_smoothness_mode if args.mpnet_smoothness_mode else None
    self.smoothness_trunct_value = args.mpnet_smoothness_trunct_value
    self.smoothness_trunct_loc = args.mpnet_smoothness_trunct_loc
    if enable_create_label_context:
      self.create_label_context()

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

  def forward(self, unary, edge_weights=None, msg_norm_index=None, pairwise_terms=None):
    unary = unary.permute(0, 1, 3, 4, 2).contiguous()
    if edge_weights is not None:
      edge_weights = edge_weights.unsqueeze(1).permute(2, 0, 1, 3, 4).contiguous()
    # the term weight scales the stored parameter before the re-parameterisation (:148-163)
    label_context = self.label_context * self.args.mpnet_term_weight
    mode = self.args.mpnet_smoothness_train
    if mode == 'sigmoid':
      valid = label_context[self.label_context_loc].flatten()
      label_context[self.label_context_loc] = 2 * torch.sigmoid(valid)
    elif mode == 'softmax':
      valid = label_context[self.label_context_loc].flatten()
      norm = nn.Softmax(dim=0)(valid)
      label_context[self.label_context_loc] = norm * valid.max() / norm.max()
    if mode in {'sigmoid', 'softmax'}:
      diag = self.label_context_diag_loc
      label_context[tuple(diag) if isinstance(diag, list) else diag] = self.args.mpnet_diag_value
    if edge_weights is not None:
      assert unary.size()[-3:-1] == edge_weights.size()[-2:]
    if unary.is_cuda and (msg_norm_index is not None):
      msg_norm_index = msg_norm_index.cuda()
    self.args.msg_norm_index = msg_norm_index
    self.args.training = self.training
    if self.args.mpnet_mrf_mode == 'TRWP':
      cost_final, cost_all, message_vector, message_index = \
          TRWPFunction.apply(unary, label_context, edge_weights, self.args)
    else:
      assert False
    cost_final = cost_final.permute(0, 1, 4, 2, 3).contiguous()
    return cost_final, label_context.unsqueeze(0), cost_all, message_vector, message_index
