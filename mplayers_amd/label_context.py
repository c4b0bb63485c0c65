"""Label-context (pairwise potential) construction, after utils/label_context.py:6-90.

create_label_context(args, enable_seg=None, enable_symmetric=False) returns
(nn.Parameter, loc, diag_loc): a (n_classes, n_classes) table for segmentation (n_classes == 21)
or a (n_classes,) vector indexed by |label difference| otherwise; `loc` indexes the learnable
entries (upper triangle / k >= 1), `diag_loc` the pinned ones (diagonal / k == 0).

args fields read: n_classes, mpnet_smoothness_mode ('Potts' | 'potts' | 'TL' | 'TQ' | 'NPotts'),
mpnet_smoothness_train, mpnet_smoothness_trunct_value, mpnet_smoothness_trunct_loc,
mpnet_term_weight, enable_cuda.
"""
import numpy as np
import torch
import torch.nn as nn


def _gap_cost(mode, gap):
  if mode in ('Potts', 'potts'):
    return 1.0
  if mode == 'TL':
    return float(gap)
  if mode == 'TQ':
    return float(gap) ** 2
  raise ValueError(mode)


def create_label_context(args, enable_seg=None, enable_symmetric=False):
  n = args.n_classes
  mode = args.mpnet_smoothness_mode
  train = args.mpnet_smoothness_train
  trunc_value = args.mpnet_smoothness_trunct_value
  trunc_loc = args.mpnet_smoothness_trunct_loc
  if enable_seg is None:
    enable_seg = (n == 21)
  potts = mode in ('Potts', 'potts')

  if enable_seg:
    table = np.zeros((n, n), dtype=np.float32)
    if mode == 'NPotts':
      table[np.arange(n), np.arange(n)] = -1
    elif mode in ('TL', 'TQ') or (potts and train != 'sigmoid'):
      for i in range(n):
        for j in range(n):
          gap = abs(j - i) if enable_symmetric else j - i
          if gap > 0:
            table[i, j] = _gap_cost(mode, gap)
    if trunc_value >= 0:
      if trunc_loc >= 0:
        # The reference tests the `gap` left over from the last cell of the construction loops
        # (utils/label_context.py:45-47), which is 0: a location of 0 truncates everything, any
        # positive location truncates nothing.  Kept as is.
        if not (mode in ('TL', 'TQ') or (potts and train != 'sigmoid')):
          raise NameError("name 'gap' is not defined")
        if 0 >= trunc_loc:
          table = np.minimum(table, np.float32(trunc_value))
      else:
        table = np.minimum(table, np.float32(trunc_value))
  else:
    table = np.zeros((n,), dtype=np.float32)
    if mode == 'NPotts':
      table[0] = -1
    elif potts:
      if train != 'sigmoid':
        table[1:] = 1
    elif mode in ('TL', 'TQ'):
      table = np.array([_gap_cost(mode, d) for d in range(n)], dtype=np.float32)
    if trunc_value >= 0:
      lo = trunc_loc if trunc_loc >= 0 else 0
      table[lo:] = np.minimum(table[lo:], np.float32(trunc_value))

  label_context = torch.from_numpy(table) * args.mpnet_term_weight
  if getattr(args, 'enable_cuda', False) and (not label_context.is_cuda):
    label_context = label_context.cuda()
  enable_grad = train in {'softmax', 'sigmoid', 'on'}
  label_context = nn.Parameter(label_context, requires_grad=enable_grad)
  if label_context.dim() == 2:
    loc = np.triu_indices(n, k=1)
    diag_loc = [range(n), range(n)]
  else:
    loc = range(1, n)
    diag_loc = range(1)
  return label_context, loc, diag_loc
