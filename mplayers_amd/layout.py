"""Layout changes of the modules as HIP transposes with autograd support.

The reference's modules move the label axis with permute().contiguous()
(pytorch/MP_module.py:199,203,233, pytorch/MP_module_hard_soft.py); these functions return the same
contiguous tensors through mpl_transpose (a batched 2-D transpose bound by HBM), and their backward
passes are the opposite transposes.
"""
import ctypes

import torch

from . import _lib


def _transpose(src, batch, rows, cols, out_shape):
  dst = src.new_empty(out_shape)
  if src.numel() == 0:
    return dst
  with torch.cuda.device(src.device):
    rc = _lib.load().mpl_transpose(ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(dst.data_ptr()),
                                   int(batch), int(rows), int(cols),
                                   ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
  _lib.check(rc, "transpose")
  return dst


def _usable(t):
  return t.is_cuda and t.dtype == torch.float32 and t.dim() == 5


class _LabelsLast(torch.autograd.Function):
  """(batch, cv, labels, H, W) -> (batch, cv, H, W, labels), contiguous."""

  @staticmethod
  def forward(ctx, x):
    b, cv, n, h, w = x.shape
    return _transpose(x.contiguous(), b * cv, n, h * w, (b, cv, h, w, n))

  @staticmethod
  def backward(ctx, grad):
    b, cv, h, w, n = grad.shape
    return _transpose(grad.contiguous(), b * cv, h * w, n, (b, cv, n, h, w))


class _LabelsFirst(torch.autograd.Function):
  """(batch, cv, H, W, labels) -> (batch, cv, labels, H, W), contiguous."""

  @staticmethod
  def forward(ctx, x):
    b, cv, h, w, n = x.shape
    return _transpose(x.contiguous(), b * cv, h * w, n, (b, cv, n, h, w))

  @staticmethod
  def backward(ctx, grad):
    b, cv, n, h, w = grad.shape
    return _transpose(grad.contiguous(), b * cv, n, h * w, (b, cv, h, w, n))


def labels_last(x):
  """x.permute(0, 1, 3, 4, 2).contiguous() for a (batch, cv, labels, H, W) tensor."""
  if _usable(x):
    return _LabelsLast.apply(x)
  return x.permute(0, 1, 3, 4, 2).contiguous()


def labels_first(x):
  """x.permute(0, 1, 4, 2, 3).contiguous() for a (batch, cv, H, W, labels) tensor."""
  if _usable(x):
    return _LabelsFirst.apply(x)
  return x.permute(0, 1, 4, 2, 3).contiguous()
