"""Helpers of the GPU parity tests: run the HIP operators through the reference-style operator
layer (which calls the C ABI) and compare with the CPU oracle."""
import numpy as np
import torch

from mplayers_amd import lib_stereo

DEV = "cuda:0"


def _t(a, dtype=torch.float32):
  return torch.as_tensor(np.ascontiguousarray(a), dtype=dtype).to(DEV).contiguous()


def gpu_forward(mode, unary, context, edge_weights, n_dir, n_iter, rho, training=True,
                saving_label=False, enable_min_a_dir=False, enable_sgm=False, msg_init=None,
                ops=None):
  """ops: a namespace with TRWP / ISGMR operator modules in the reference's calling convention
  (default: mplayers_amd.lib_stereo, the ctypes operators)."""
  ops = lib_stereo if ops is None else ops
  unary = _t(unary)
  b, cv, h, w, L = unary.shape
  context = _t(context)
  if edge_weights is None:
    edge_weights = np.ones((n_dir, b, cv, h, w), dtype=np.float32)
  edge_weights = _t(edge_weights)
  msg = unary.new_zeros(n_dir, b, cv, h, w, L) if msg_init is None else _t(msg_init)
  cost = unary.new_zeros(b, cv, h, w, L)
  scratch = unary.new_zeros(b, cv, h, w, L)
  u8 = dict(dtype=torch.uint8)
  imin = unary.new_zeros(n_iter, n_dir, b, cv, h, w, L, **u8) if training else torch.empty(0, **u8)
  inorm = unary.new_zeros(n_iter, n_dir, b, cv, h, w, **u8) if training else torch.empty(0, **u8)
  label = unary.new_zeros(n_iter, b, cv, h, w, **u8) if saving_label else torch.empty(0, **u8)
  if mode == "TRWP":
    ops.TRWP.forward(rho, n_iter, int(enable_min_a_dir), unary, context, edge_weights, msg,
                     cost, imin, inorm, scratch, label)
  else:
    msg_update = torch.zeros_like(msg)
    ops.ISGMR.forward(int(enable_sgm), rho, n_iter, int(enable_min_a_dir), unary, context,
                      edge_weights, msg, cost, imin, inorm, scratch, msg_update, label)
  torch.cuda.synchronize()
  return dict(msg=msg.cpu().numpy(), cost_final=cost.cpu().numpy(),
              msg_min_index=imin.cpu().numpy() if training else None,
              msg_norm_index=inorm.cpu().numpy() if training else None,
              label_all=label.cpu().numpy() if saving_label else None,
              _dev=dict(context=context, edge_weights=edge_weights, imin=imin, inorm=inorm))


def gpu_backward(mode, context, edge_weights, dcost, msg_min_index, msg_norm_index, rho,
                 enable_sgm=False, garbage_scratch=False, flags=0, want_dctx=True, want_dedge=True,
                 hard_soft=False, ops=None):
  """want_dctx / want_dedge False: that gradient is passed as an empty tensor (not wanted) and
  comes back as None.  hard_soft: the TRWP_hard_soft namespace's hard backward.  ops: as for
  gpu_forward (such operators take the reference's arguments only: no flags)."""
  kw = dict(flags=flags) if ops is None else {}
  ops = lib_stereo if ops is None else ops
  n_iter, n_dir, b, cv, h, w, L = msg_min_index.shape
  context = _t(context)
  if edge_weights is None:
    edge_weights = np.ones((n_dir, b, cv, h, w), dtype=np.float32)
  edge_weights = _t(edge_weights)
  dcost = _t(dcost)
  imin = _t(msg_min_index, torch.uint8)
  inorm = _t(msg_norm_index, torch.uint8)
  dunary = dcost.new_zeros(b, cv, h, w, L)
  make = (lambda *s: torch.full(s, 7.25, device=DEV)) if garbage_scratch else dcost.new_zeros
  dmsg = make(n_dir, b, cv, h, w, L)
  dunary_update = make(b, cv, h, w, L)
  dedge = dcost.new_zeros(n_dir, b, cv, h, w) if want_dedge else dcost.new_empty(0)
  dctx = (dcost.new_zeros(L, L) if L == 21 else dcost.new_zeros(L)) if want_dctx else \
      dcost.new_empty(0)
  if mode == "TRWP":
    op = ops.TRWP_hard_soft if hard_soft else ops.TRWP
    op.backward(rho, context, edge_weights, dcost, imin, inorm, dunary, dctx, dedge, dmsg,
                dunary_update, **kw)
  else:
    dmsg_update = make(n_dir, b, cv, h, w, L)
    ops.ISGMR.backward(int(enable_sgm), rho, context, edge_weights, dcost, imin, inorm,
                       dunary, dctx, dedge, dmsg, dunary_update, dmsg_update, **kw)
  torch.cuda.synchronize()
  return (dunary.cpu().numpy(), dctx.cpu().numpy() if want_dctx else None,
          dedge.cpu().numpy() if want_dedge else None)


def assert_values_close(got, ref, rel=1e-5, what="", belief=None):
  """|got - ref| <= rel * max(1, max|belief|): the 1e-5 relative bar of the parity contract.

  The bar is relative to the magnitude of the beliefs (unary + all messages), the quantities whose
  fp32 sums and differences produce every message: messages contain exact zeros, so an elementwise
  ratio is meaningless, and the fp32 restatement of the reference itself sits 2-3.5e-5 (absolute,
  beliefs up to 8.3) away from its fp64 evaluation on the scaled-down large configuration, i.e.
  two correct fp32 evaluation orders cannot agree more closely than a few 1e-6 of that magnitude."""
  scale = max(1.0, float(np.abs(ref if belief is None else belief).max()))
  err = float(np.abs(got.astype(np.float64) - ref.astype(np.float64)).max())
  assert err <= rel * scale, "%s: max abs err %.3e > %.1e * %.3g" % (what, err, rel, scale)


def assert_indices_match_off_ties(got, ref, gap, tol, what=""):
  """Indices must be identical except where the oracle's best and second best candidates are
  closer than tol (a tie within tolerance)."""
  bad = got != ref
  if bad.any():
    assert float(gap[bad].max()) <= tol, "%s: %d index mismatches, largest gap %.3e > %.1e" % (
        what, int(bad.sum()), float(gap[bad].max()), tol)
  return int(bad.sum())


def assert_labels_match_off_ties(got, ref, gap, tol, what="label_all"):
  """Labels must be identical except where the oracle's smallest and second smallest cost of the
  pixel are closer than tol (CalLabelKernel picks the smallest label among equal costs,
  TRWP_forward.cu:8-29; a cost within tolerance may fall either side of such a near tie)."""
  return assert_indices_match_off_ties(got, ref, gap, tol, what)
