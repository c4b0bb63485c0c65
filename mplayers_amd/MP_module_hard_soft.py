"""Hard / soft-weighted TRWP layer behind the surface of the reference's
pytorch/MP_module_hard_soft.py:13-182 (the module mpnet.py:35 builds its CRF layer from): a
`TRWPFunction` with four outputs and an `MPModule` with five.  `args.mpnet_enable_soft` selects the
soft-weighted operator (softmin expectation over the front labels) or the min-sum one; both run in
the HIP library of this package.

  TRWPFunction.apply(unary (B, cv, H, W, L), label_context, edge_weights (n_dir, B, cv, H, W) | None,
                     args) -> (cost_final, label_all, message_edge_label, cost_index)
  MPModule.forward(unary (B, cv, L, H, W), edge_weights (B, n_dir, H, W) | None, msg_norm_index=None,
                   pairwise_terms=None)
                   -> (cost_final (B, cv, L, H, W), label_context[None], label_all,
                       message_edge_label, cost_index)
"""
import torch

from . import lib_seg, lib_stereo
from .layout import labels_first, labels_last
from .MP_module import MPModule as _HardModule

_U8 = dict(dtype=torch.uint8)


def _operators(n_disp):
  # MP_module_hard_soft.py:20: the segmentation build for 21 labels, the stereo build otherwise
  return (lib_seg if n_disp == 21 else lib_stereo).TRWP_hard_soft


def _none_u8():
  return torch.empty(0, **_U8)


class TRWPFunction(torch.autograd.Function):
  """MP_module_hard_soft.py:13-108.  Outputs beyond the cost: per-iteration labels (empty unless
  args.enable_saving_label), the stored duals of the soft operator (empty in hard mode or outside
  training) and the normalisation indices."""

  @staticmethod
  def forward(ctx, unary, label_context, edge_weights, args):
    shape = tuple(unary.shape)                      # (batch, cv, h, w, n_disp)
    n_disp = shape[-1]
    n_iter, n_dir = int(args.mpnet_max_iter), int(args.mpnet_n_dirs)
    soft, training = bool(args.mpnet_enable_soft), bool(args.training)
    per_dir = (n_dir,) + shape
    per_iter = (n_iter, n_dir) + shape[:-1]
    had_weights = edge_weights is not None
    if not had_weights:
      edge_weights = unary.new_ones((n_dir,) + shape[:-1])
    # The initial messages must be zero.  Of the rest, only what a caller can look at is cleared
    # (the operators leave the entries of chain-start pixels untouched); scratch is not.
    message = unary.new_zeros(per_dir)
    cost_final = unary.new_empty(shape)
    scratch = unary.new_empty(shape)
    label_all = (unary.new_empty((n_iter,) + shape[:-1], **_U8) if args.enable_saving_label
                 else _none_u8())
    cost_index = unary.new_zeros(per_iter, **_U8) if training else _none_u8()
    message_edge_label = torch.empty(0, dtype=torch.float32)
    message_index = _none_u8()
    op = _operators(n_disp)
    if soft:
      if training:
        message_edge_label = unary.new_zeros(per_iter + (n_disp, n_disp))
      op.forward_soft(args.rho, n_iter, unary, label_context, edge_weights, message,
                      message_edge_label, cost_index, cost_final, scratch, label_all)
    else:
      if training:
        message_index = unary.new_empty(per_iter + (n_disp,), **_U8)
      op.forward(args.rho, n_iter, 0, unary, label_context, edge_weights, message, cost_final,
                 message_index, cost_index, scratch, label_all)
    ctx.saved = dict(args=args, soft=soft, blocks=message_edge_label, index=message_index,
                     cost_index=cost_index, context=label_context, weights=edge_weights,
                     had_weights=had_weights)
    return cost_final, label_all, message_edge_label, cost_index

  @staticmethod
  def backward(ctx, dcost_final, dlabel_all, dmessage_edge_label, dcost_index):
    saved = ctx.saved
    del ctx.saved
    args = saved["args"]
    dcost_final = dcost_final.contiguous()
    # a caller may impose the normalisation indices (MP_module_hard_soft.py:77)
    cost_index = saved["cost_index"] if args.msg_norm_index is None else args.msg_norm_index
    n_iter, n_dir = cost_index.shape[:2]
    shape = tuple(cost_index.shape[2:]) + (args.n_classes,)
    n_disp = shape[-1]
    dunary = dcost_final.new_empty(shape)
    scratch = dcost_final.new_empty((n_dir,) + shape)
    unused = dcost_final.new_empty(0)
    # a gradient autograd does not ask for is an empty tensor: the operators leave it out
    need_context = ctx.needs_input_grad[1]
    need_edge_weights = saved["had_weights"] and ctx.needs_input_grad[2]
    dedge_weights = (dcost_final.new_zeros((n_dir,) + shape[:-1]) if need_edge_weights
                     else unused)
    dlabel_context = (dcost_final.new_zeros((n_disp, n_disp) if args.enable_seg else (n_disp,))
                      if need_context else unused)
    op = _operators(n_disp)
    if saved["soft"]:
      op.backward_soft(args.rho, dcost_final, saved["context"], saved["weights"], saved["blocks"],
                       cost_index, dunary, dlabel_context, dedge_weights, scratch, unused)
    else:
      op.backward(args.rho, saved["context"], saved["weights"], dcost_final, saved["index"],
                  cost_index, dunary, dlabel_context, dedge_weights, scratch, unused)
    return (dunary, dlabel_context if need_context else None,
            dedge_weights if need_edge_weights else None, None)


class MPModule(_HardModule):
  """MP_module_hard_soft.py:111-182.  Shares the label-context handling with the hard module; the
  differences are the constructor (no min-over-directions switch; only TRWP), the place of the term
  weight (it scales the stored parameter before the re-parameterisation, :148-163) and the two
  extra inputs / outputs of forward."""

  def __init__(self, args, enable_create_label_context=False, enable_saving_label=False):
    super(MPModule, self).__init__(args, enable_create_label_context=enable_create_label_context,
                                   enable_saving_label=enable_saving_label)
    self.smoothness_train = args.mpnet_smoothness_train or None
    self.smoothness_mode = args.mpnet_smoothness_mode or None
    self.smoothness_trunct_value = args.mpnet_smoothness_trunct_value
    self.smoothness_trunct_loc = args.mpnet_smoothness_trunct_loc

  def forward(self, unary, edge_weights=None, msg_norm_index=None, pairwise_terms=None):
    assert self.args.mpnet_mrf_mode == 'TRWP'
    unary = labels_last(unary)
    if edge_weights is not None:
      edge_weights = edge_weights.unsqueeze(1).permute(2, 0, 1, 3, 4).contiguous()
      assert unary.size()[-3:-1] == edge_weights.size()[-2:]
    label_context = self._effective_label_context(weight_first=True)
    if msg_norm_index is not None and unary.is_cuda:
      msg_norm_index = msg_norm_index.cuda()
    self.args.msg_norm_index = msg_norm_index
    self.args.training = self.training
    cost_final, label_all, blocks, cost_index = TRWPFunction.apply(unary, label_context,
                                                                   edge_weights, self.args)
    return (labels_first(cost_final), label_context.unsqueeze(0), label_all,
            blocks, cost_index)
