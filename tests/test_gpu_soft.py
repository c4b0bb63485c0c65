"""Soft-weighted TRWP on the GPU (lib_*.TRWP_hard_soft, MP_module_hard_soft) against the CPU oracle.
Tolerances: values within 2e-5 of the belief magnitude (the kernels use the hardware exponential,
as the reference's __expf does); gradients within 1e-4 of the largest entry."""
import argparse

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

CASES = [
    # n_dir, B, H, W, L, context kind, n_iter
    (4, 1, 5, 7, 5, "tl2", 2),
    (4, 2, 6, 5, 21, "dense2d", 2),     # the segmentation case: 441 duals per pixel, 7 per lane
    (8, 1, 6, 7, 21, "dense2d", 1),
    (8, 1, 5, 6, 16, "tl3", 2),         # 256 duals: exactly 4 per lane
    (4, 1, 4, 5, 30, "dense1d", 1),     # 900 duals: 16-per-lane bucket
    (4, 1, 3, 4, 40, "tl3", 1),         # 1600 duals: 64-per-lane bucket
    (4, 1, 3, 3, 64, "dense1d", 1),     # every lane holds a label
    (16, 1, 7, 6, 6, "dense1d", 2),
    (4, 1, 1, 9, 8, "tl2", 2),
    (4, 1, 9, 1, 8, "tl2", 2),
    (2, 3, 3, 12, 3, "tl2", 3),
    # up to 32 labels the front labels of a pixel are split over 4 / 3 / 2 groups of lanes
    (4, 1, 3, 4, 1, "tl2", 2),          # a single label: every message is 0
    (4, 1, 4, 6, 2, "tl2", 2),          # one front label per group, two groups idle
    (4, 1, 4, 5, 13, "dense2d", 2),     # 4 groups, the last one holds a single front label
    (4, 1, 5, 4, 17, "dense2d", 1),     # smallest 3-group case: 6 + 6 + 5 front labels
    (8, 1, 4, 5, 20, "tl3", 1),         # 7 + 7 + 6
    (4, 1, 3, 4, 22, "dense1d", 1),     # smallest 2-group case
    (4, 1, 3, 3, 32, "dense2d", 1),     # every lane used, 16 front labels each
    # more than 64 labels (the stereo build accepts up to 256, TRWP_hard_soft/TRWP.cpp:336-340):
    # several labels per lane, the duals move through LDS in chunks of 32 front labels
    (4, 1, 4, 5, 65, "tl3", 2),         # one label in the second register, one 1-label chunk
    (4, 2, 3, 4, 96, "dense1d", 1),     # chunks end on a label boundary
    (8, 1, 4, 4, 130, "tl3", 1),        # three labels per lane, diagonals too
    (4, 1, 3, 3, 200, "dense1d", 2),    # four labels per lane, partial last chunk
    (4, 1, 2, 3, 256, "tl3", 1),        # every lane holds four labels
]


def make_ctx(kind, L, rng):
  k = np.arange(L, dtype=np.float32)
  if kind == "tl2":
    return (0.4 * np.minimum(k, 2)).astype(np.float32)
  if kind == "tl3":
    return (0.3 * np.minimum(k, 3)).astype(np.float32)
  if kind == "dense1d":
    return rng.random(L).astype(np.float32)
  if kind == "dense2d":
    return np.triu(rng.random((L, L))).astype(np.float32)
  raise KeyError(kind)


def t(a, dtype=None):
  import torch
  x = torch.as_tensor(np.ascontiguousarray(a)).cuda()
  return x if dtype is None else x.to(dtype)


def gpu_forward_soft(unary, ctx, ew, n_dir, n_iter, rho, training=True, saving_label=False):
  import torch
  from mplayers_amd import lib_stereo
  b, cv, h, w, L = unary.shape
  u = t(unary)
  msg = u.new_zeros(n_dir, b, cv, h, w, L)
  cost = u.new_zeros(b, cv, h, w, L)
  scratch = u.new_zeros(b, cv, h, w, L)
  u8 = dict(dtype=torch.uint8)
  mel = u.new_zeros(n_iter, n_dir, b, cv, h, w, L, L) if training else torch.empty(0)
  inorm = u.new_zeros(n_iter, n_dir, b, cv, h, w, **u8) if training else torch.empty(0, **u8)
  label = u.new_zeros(n_iter, b, cv, h, w, **u8) if saving_label else torch.empty(0, **u8)
  lib_stereo.TRWP_hard_soft.forward_soft(rho, n_iter, u, t(ctx), t(ew), msg, mel, inorm, cost,
                                         scratch, label)
  torch.cuda.synchronize()
  return dict(msg=msg.cpu().numpy(), cost_final=cost.cpu().numpy(),
              msg_edge_label=mel.cpu().numpy() if training else None,
              msg_norm_index=inorm.cpu().numpy() if training else None,
              label_all=label.cpu().numpy() if saving_label else None)


@pytest.mark.parametrize("n_dir,B,H,W,L,kind,n_iter", CASES)
@pytest.mark.parametrize("training", [True, False])
def test_forward_soft_matches_oracle(gpu, oracle, n_dir, B, H, W, L, kind, n_iter, training):
  rng = np.random.default_rng(n_dir * 100 + L)
  unary = rng.random((B, 1, H, W, L)).astype(np.float32)
  ctx = make_ctx(kind, L, rng)
  ew = (0.2 + rng.random((n_dir, B, 1, H, W))).astype(np.float32)
  rho = 0.5
  print("case", n_dir, B, H, W, L, kind, n_iter, training, flush=True)
  ref = oracle.forward_soft(unary, ctx, ew, n_dir, n_iter, rho, training=training, saving_label=True,
                            want_gaps=True)
  got = gpu_forward_soft(unary, ctx, ew, n_dir, n_iter, rho, training=training, saving_label=True)
  belief = ref["cost_final"]
  gpu.assert_values_close(got["msg"], ref["msg"], rel=2e-5, what="msg", belief=belief)
  gpu.assert_values_close(got["cost_final"], ref["cost_final"], rel=2e-5, what="cost")
  gpu.assert_labels_match_off_ties(got["label_all"], ref["label_all"], ref["gap_label"],
                                   4e-5 * max(1.0, float(np.abs(belief).max())))
  if training:
    gpu.assert_values_close(got["msg_edge_label"], ref["msg_edge_label"], rel=2e-5, what="duals",
                            belief=belief)
    # the normalisation index may differ where two soft messages are closer than the tolerance
    ref64 = oracle.forward_soft(unary.astype(np.float64), ctx, ew, n_dir, n_iter, rho)
    bad = got["msg_norm_index"] != ref["msg_norm_index"]
    if bad.any():
      it, d, b, c, hh, ww = np.nonzero(bad)
      for i in range(len(it)):
        m = ref64["msg"][d[i], b[i], c[i], hh[i], ww[i]] if it[i] == n_iter - 1 else None
        if m is not None:
          lo = np.sort(m)[:2]
          assert lo[1] - lo[0] <= 2e-5 * max(1.0, float(np.abs(belief).max()))
      assert bad.mean() <= 0.02


@pytest.mark.parametrize("n_dir,B,H,W,L,kind,n_iter", CASES)
def test_backward_soft_matches_oracle(gpu, oracle, n_dir, B, H, W, L, kind, n_iter):
  import torch
  from mplayers_amd import lib_stereo
  rng = np.random.default_rng(n_dir * 100 + L + 1)
  unary = rng.random((B, 1, H, W, L)).astype(np.float32)
  ctx = make_ctx(kind, L, rng)
  ew = (0.2 + rng.random((n_dir, B, 1, H, W))).astype(np.float32)
  dcost = rng.standard_normal((B, 1, H, W, L)).astype(np.float32)
  rho = 0.5
  print("case", n_dir, B, H, W, L, kind, n_iter, flush=True)
  fwd = oracle.forward_soft(unary, ctx, ew, n_dir, n_iter, rho)
  du, dc, de = oracle.backward_soft(ctx.astype(np.float64), ew.astype(np.float64),
                                    dcost.astype(np.float64),
                                    fwd["msg_edge_label"].astype(np.float64),
                                    fwd["msg_norm_index"], rho)
  g = t(dcost)
  dunary = g.new_zeros(B, 1, H, W, L)
  dmsg = torch.full((n_dir, B, 1, H, W, L), 3.5, device="cuda")  # scratch: any contents
  dctx = g.new_zeros(L, L) if L == 21 else g.new_zeros(L)
  dedge = g.new_zeros(n_dir, B, 1, H, W)
  lib_stereo.TRWP_hard_soft.backward_soft(rho, g, t(ctx), t(ew), t(fwd["msg_edge_label"]),
                                          t(fwd["msg_norm_index"]), dunary, dctx, dedge, dmsg,
                                          g.new_empty(0))
  torch.cuda.synchronize()
  for name, got, ref in (("dunary", dunary, du), ("dcontext", dctx, dc), ("dedge", dedge, de)):
    err = np.abs(got.cpu().numpy().astype(np.float64) - ref).max()
    assert err <= 1e-4 * max(1.0, np.abs(ref).max()), (name, err, np.abs(ref).max())
  # gradient mass: softmin weights sum to one and normalised messages carry no net mass
  assert abs(float(dunary.sum()) - float(dcost.sum())) <= 1e-3 * max(1.0, np.abs(dcost).sum())


@pytest.mark.parametrize("L,train_mode", [(21, "sigmoid"), (9, "")])
def test_module_soft_forward_backward(gpu, oracle, L, train_mode):
  """MP_module_hard_soft.MPModule with mpnet_enable_soft: five outputs, gradients for the unary
  term, the edge weights and the learned context."""
  import torch
  from mplayers_amd.MP_module_hard_soft import MPModule
  rng = np.random.default_rng(L)
  B, H, W, n_dir, n_iter = 2, 6, 7, 4, 2
  args = argparse.Namespace(mpnet_mrf_mode="TRWP", mpnet_enable_soft=True, mpnet_max_iter=n_iter,
                            mpnet_n_dirs=n_dir, n_classes=L, mpnet_term_weight=1.5,
                            mpnet_smoothness_train=train_mode, mpnet_smoothness_mode="TL",
                            mpnet_smoothness_trunct_value=3, mpnet_smoothness_trunct_loc=-1,
                            mpnet_diag_value=0.0, enable_symmetric=True, enable_cuda=True)
  mod = MPModule(args, enable_create_label_context=True, enable_saving_label=True).cuda().train()
  unary = rng.standard_normal((B, 1, L, H, W)).astype(np.float32)
  ew = (0.1 + 0.9 * rng.random((B, n_dir, H, W))).astype(np.float32)
  dcost = rng.standard_normal((B, 1, L, H, W)).astype(np.float32)
  u = torch.from_numpy(unary).cuda().requires_grad_(True)
  e = torch.from_numpy(ew).cuda().requires_grad_(True)
  cost, lc_out, labels, blocks, cost_index = mod(u, e)
  assert cost.shape == (B, 1, L, H, W) and labels.shape == (n_iter, B, 1, H, W)
  assert blocks.shape == (n_iter, n_dir, B, 1, H, W, L, L)
  assert cost_index.shape == (n_iter, n_dir, B, 1, H, W)
  cost.backward(torch.from_numpy(dcost).cuda())
  torch.cuda.synchronize()
  ctx = lc_out[0].detach().cpu().numpy()
  un = np.ascontiguousarray(unary.transpose(0, 1, 3, 4, 2))
  en = np.ascontiguousarray(ew[:, None].transpose(2, 0, 1, 3, 4))
  dn = np.ascontiguousarray(dcost.transpose(0, 1, 3, 4, 2))
  ref = oracle.forward_soft(un, ctx, en, n_dir, n_iter, 0.5, saving_label=True)
  gpu.assert_values_close(cost.detach().cpu().numpy().transpose(0, 1, 3, 4, 2), ref["cost_final"],
                          rel=2e-5, what="module cost")
  du, dc, de = oracle.backward_soft(ctx.astype(np.float64), en.astype(np.float64),
                                    dn.astype(np.float64),
                                    blocks.detach().cpu().numpy().astype(np.float64),
                                    cost_index.cpu().numpy(), 0.5)
  assert np.abs(u.grad.cpu().numpy().transpose(0, 1, 3, 4, 2) - du).max() <= 1e-4 * max(1, np.abs(du).max())
  assert np.abs(e.grad.cpu().numpy()[:, None].transpose(2, 0, 1, 3, 4) - de).max() <= 1e-4 * max(1, np.abs(de).max())
  if train_mode:
    # the learned context: its gradient is the oracle's dcontext pulled back through the
    # re-parameterisation of MP_module_hard_soft.py:148-163 (term weight first, then 2 * sigmoid,
    # the diagonal pinned)
    lc = torch.from_numpy(mod.label_context.detach().cpu().numpy().astype(np.float64)).requires_grad_(True)
    eff = lc * args.mpnet_term_weight
    loc, diag = mod.label_context_loc, mod.label_context_diag_loc
    eff[loc] = 2 * torch.sigmoid(eff[loc].flatten())
    eff[tuple(diag) if isinstance(diag, list) else diag] = args.mpnet_diag_value
    eff.backward(torch.from_numpy(dc))
    got_lc = mod.label_context.grad.cpu().numpy()
    assert np.abs(lc.grad.numpy()).max() > 1e-3
    assert np.abs(got_lc - lc.grad.numpy()).max() <= 1e-4 * max(1, np.abs(lc.grad.numpy()).max())
  else:
    assert mod.label_context.grad is None  # a fixed table: not a learnable parameter
  # hard mode through the same surface equals the plain TRWP module
  args.mpnet_enable_soft = False
  cost_h = mod(u.detach(), e.detach())[0]
  hard = oracle.forward("TRWP", un, ctx, en, n_dir, n_iter, 0.5)
  gpu.assert_values_close(cost_h.detach().cpu().numpy().transpose(0, 1, 3, 4, 2), hard["cost_final"],
                          what="hard mode")


@pytest.mark.parametrize("L,n_dir", [(21, 4), (9, 8), (70, 4), (16, 4), (192, 4)])
def test_module_hard_mode_backward_collects_same_label_terms(gpu, oracle, L, n_dir):
  """mpnet_enable_soft = False with a context learned as it is (mpnet_smoothness_train = 'on'):
  the module calls TRWP_hard_soft.backward (MP_module_hard_soft.py:95), whose dcontext also
  collects the pairs with equal labels (TRWP_hard_soft/TRWP_backward.cu:110,194,264), so entry 0
  of a 1-D table / the diagonal of a 2-D one get their gradient; TRWP.backward leaves them 0."""
  import torch
  from mplayers_amd import lib_stereo
  from mplayers_amd.MP_module_hard_soft import MPModule
  rng = np.random.default_rng(L + n_dir)
  B, H, W, n_iter = 2, 6, 7, 2
  args = argparse.Namespace(mpnet_mrf_mode="TRWP", mpnet_enable_soft=False, mpnet_max_iter=n_iter,
                            mpnet_n_dirs=n_dir, n_classes=L, mpnet_term_weight=1.0,
                            mpnet_smoothness_train="on", mpnet_smoothness_mode="TL",
                            mpnet_smoothness_trunct_value=3, mpnet_smoothness_trunct_loc=-1,
                            mpnet_diag_value=0.0, enable_symmetric=True, enable_cuda=True)
  mod = MPModule(args, enable_create_label_context=True).cuda().train()
  assert mod.label_context.requires_grad
  with torch.no_grad():  # a table whose same-label entries matter
    if L == 21:
      mod.label_context.copy_(torch.from_numpy(
          (np.triu(rng.random((L, L)), 1) + np.diag(0.1 + 0.3 * rng.random(L))).astype(np.float32)))
    else:
      mod.label_context[0] = 0.2
  unary = rng.standard_normal((B, 1, L, H, W)).astype(np.float32)
  ew = (0.1 + 0.9 * rng.random((B, n_dir, H, W))).astype(np.float32)
  dcost = rng.standard_normal((B, 1, L, H, W)).astype(np.float32)
  u = torch.from_numpy(unary).cuda().requires_grad_(True)
  e = torch.from_numpy(ew).cuda().requires_grad_(True)
  print("case", L, n_dir, flush=True)
  cost = mod(u, e)[0]
  cost.backward(torch.from_numpy(dcost).cuda())
  torch.cuda.synchronize()
  ctx = mod.label_context.detach().cpu().numpy()
  un = np.ascontiguousarray(unary.transpose(0, 1, 3, 4, 2))
  en = np.ascontiguousarray(ew[:, None].transpose(2, 0, 1, 3, 4))
  dn = np.ascontiguousarray(dcost.transpose(0, 1, 3, 4, 2))
  ref = oracle.forward("TRWP", un, ctx, en, n_dir, n_iter, 0.5)
  gpu.assert_values_close(cost.detach().cpu().numpy().transpose(0, 1, 3, 4, 2), ref["cost_final"],
                          what="hard mode cost")
  du, dc, de = oracle.backward("TRWP", ctx.astype(np.float64), en.astype(np.float64),
                               dn.astype(np.float64), ref["msg_min_index"], ref["msg_norm_index"],
                               0.5, same_label=True)
  same = np.diag(dc) if L == 21 else dc[:1]
  assert np.abs(same).max() > 1e-2  # the terms the guarded operator drops are not small
  got = mod.label_context.grad.cpu().numpy()
  assert np.abs(got - dc).max() <= 1e-4 * max(1, np.abs(dc).max()), np.abs(got - dc).max()
  assert np.abs(u.grad.cpu().numpy().transpose(0, 1, 3, 4, 2) - du).max() <= 1e-4 * max(1, np.abs(du).max())
  assert np.abs(e.grad.cpu().numpy()[:, None].transpose(2, 0, 1, 3, 4) - de).max() <= 1e-4 * max(1, np.abs(de).max())
  # the two operator namespaces on the oracle's indices: they differ in those entries only
  t8 = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
  res = {}
  for name, op in (("TRWP", lib_stereo.TRWP), ("TRWP_hard_soft", lib_stereo.TRWP_hard_soft)):
    dctx = torch.zeros(ctx.shape, device="cuda")
    dunary = torch.empty(un.shape, device="cuda")
    dedge = torch.zeros(en.shape, device="cuda")
    op.backward(0.5, t8(ctx), t8(en), t8(dn), t8(ref["msg_min_index"]), t8(ref["msg_norm_index"]),
                dunary, dctx, dedge, torch.empty((n_dir,) + un.shape, device="cuda"),
                torch.empty(0, device="cuda"))
    torch.cuda.synchronize()
    res[name] = (dunary.cpu().numpy(), dctx.cpu().numpy(), dedge.cpu().numpy())
  assert np.array_equal(res["TRWP"][0], res["TRWP_hard_soft"][0])
  assert np.array_equal(res["TRWP"][2], res["TRWP_hard_soft"][2])
  guarded, full = res["TRWP"][1], res["TRWP_hard_soft"][1]
  if L == 21:
    assert np.all(np.diag(guarded) == 0)
    off = ~np.eye(L, dtype=bool)
    assert np.abs(guarded[off] - full[off]).max() <= 1e-5 * max(1, np.abs(full).max())
  else:
    assert guarded[0] == 0
    assert np.abs(guarded[1:] - full[1:]).max() <= 1e-5 * max(1, np.abs(full).max())
  assert np.abs(full - dc).max() <= 1e-4 * max(1, np.abs(dc).max())


def test_soft_accepts_what_the_reference_accepts(gpu):
  """Up to 256 labels (MAX_DISPARITY of the stereo build); beyond that the call is refused before
  anything is launched (the reference prints a message and returns zero-filled outputs)."""
  import torch
  from mplayers_amd import lib_stereo
  L = 257
  u = torch.zeros(1, 1, 2, 2, L, device="cuda")
  with pytest.raises(RuntimeError, match="n_disp"):
    lib_stereo.TRWP_hard_soft.forward_soft(
        0.5, 1, u, torch.zeros(L, device="cuda"), torch.ones(4, 1, 1, 2, 2, device="cuda"),
        torch.zeros(4, 1, 1, 2, 2, L, device="cuda"), torch.empty(0), torch.empty(0, dtype=torch.uint8),
        torch.zeros_like(u), torch.zeros_like(u), torch.empty(0, dtype=torch.uint8))


@pytest.mark.parametrize("T,L", [(5, 6), (3, 21), (2, 64), (2, 100), (1, 255)])
def test_soft_weighted_message(gpu, oracle, T, L):
  import torch
  from mplayers_amd import lib_seg
  rng = np.random.default_rng(L)
  m = (rng.random((T, L, L)) * 4).astype(np.float32)
  R = rng.standard_normal((T, L)).astype(np.float32)
  ref_norm, ref_ind = oracle.soft_weighted_message(m.astype(np.float64))
  ref_dm = oracle.soft_weighted_message_back(R.astype(np.float64), m.astype(np.float64), ref_ind)
  msg = t(m)
  norm = msg.new_zeros(T, L)
  ind = torch.zeros(T, dtype=torch.uint8, device="cuda")
  lib_seg.TRWP_hard_soft.soft_weighted_message(msg, norm, ind)
  dm = torch.zeros_like(msg)
  lib_seg.TRWP_hard_soft.soft_weighted_message_back(t(R), msg, t(ref_ind), dm)
  torch.cuda.synchronize()
  assert np.abs(norm.cpu().numpy() - ref_norm).max() <= 1e-5 * max(1.0, np.abs(m).max())
  np.testing.assert_array_equal(ind.cpu().numpy(), ref_ind)
  assert np.abs(dm.cpu().numpy() - ref_dm).max() <= 1e-4 * max(1.0, np.abs(ref_dm).max())


@pytest.mark.parametrize("seed", range(16))
def test_random_soft_case(gpu, oracle, seed):
  """Seeded random shapes: every block bucket, partial lanes, 2 to 16 directions, tiny grids."""
  import torch
  from mplayers_amd import lib_stereo
  rng = np.random.default_rng(500 + seed)
  n_dir = int(rng.choice([2, 4, 8, 16]))
  B, H, W = int(rng.integers(1, 3)), int(rng.integers(1, 8)), int(rng.integers(1, 8))
  L = int(rng.choice([1, 2, 7, 8, 9, 15, 16, 17, 21, 22, 31, 32, 33, 47, 63, 64]))
  n_iter = int(rng.integers(1, 3))
  ctx = make_ctx("dense2d" if L == 21 else ["tl2", "dense1d"][seed % 2], L, rng)
  unary = rng.random((B, 1, H, W, L)).astype(np.float32)
  ew = (0.2 + rng.random((n_dir, B, 1, H, W))).astype(np.float32)
  dcost = rng.standard_normal((B, 1, H, W, L)).astype(np.float32)
  print("case", seed, n_dir, B, H, W, L, n_iter, flush=True)
  ref = oracle.forward_soft(unary, ctx, ew, n_dir, n_iter, 0.5)
  got = gpu_forward_soft(unary, ctx, ew, n_dir, n_iter, 0.5)
  belief = ref["cost_final"]
  gpu.assert_values_close(got["msg"], ref["msg"], rel=2e-5, what="msg", belief=belief)
  gpu.assert_values_close(got["cost_final"], ref["cost_final"], rel=2e-5, what="cost")
  gpu.assert_values_close(got["msg_edge_label"], ref["msg_edge_label"], rel=2e-5, what="duals",
                          belief=belief)
  du, dc, de = oracle.backward_soft(ctx.astype(np.float64), ew.astype(np.float64),
                                    dcost.astype(np.float64),
                                    ref["msg_edge_label"].astype(np.float64),
                                    ref["msg_norm_index"], 0.5)
  g = t(dcost)
  dunary = g.new_zeros(B, 1, H, W, L)
  dmsg = torch.full((n_dir, B, 1, H, W, L), -2.5, device="cuda")
  dctx = g.new_zeros(L, L) if L == 21 else g.new_zeros(L)
  dedge = g.new_zeros(n_dir, B, 1, H, W)
  lib_stereo.TRWP_hard_soft.backward_soft(0.5, g, t(ctx), t(ew), t(ref["msg_edge_label"]),
                                          t(ref["msg_norm_index"]), dunary, dctx, dedge, dmsg,
                                          g.new_empty(0))
  torch.cuda.synchronize()
  for name, a, r in (("dunary", dunary, du), ("dcontext", dctx, dc), ("dedge", dedge, de)):
    err = np.abs(a.cpu().numpy().astype(np.float64) - r).max()
    assert err <= 1e-4 * max(1.0, np.abs(r).max()), (name, err)
