"""Backward entry points with outputs switched off and with the per-call flags of the C ABI.

A caller with a fixed pairwise table or edge weights that are not learned passes no dcontext /
dedge_weights tensor; the reverse scans then run without that part of their step.  What is still
computed must not change: dunary and dedge_weights bit for bit (their summation order is fixed),
dcontext to the tolerance of its float atomics.  MPL_F_DCONTEXT_SAME_LABEL (the hard backward of
the reference's TRWP_hard_soft build) is checked against the oracle for every kernel variant,
the several-chains-per-wavefront one included."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

CASES = [
    # mode, n_dir, B, H, W, L, 2-D context
    ("TRWP", 4, 2, 6, 7, 8, False),      # one label per lane, scatter loop over source labels
    ("ISGMR", 8, 2, 6, 7, 16, False),
    ("TRWP", 4, 2, 6, 5, 21, True),      # 2-D table
    ("ISGMR", 8, 1, 6, 5, 21, True),
    ("TRWP", 8, 1, 7, 6, 40, False),     # one label per lane, register scatter
    ("ISGMR", 4, 1, 5, 6, 96, False),    # two labels per lane
    ("TRWP", 8, 1, 6, 6, 192, False),    # three
    ("ISGMR", 4, 1, 4, 5, 250, False),   # four, partial lanes
    ("TRWP", 16, 1, 6, 7, 12, False),
]


def _problem(oracle, mode, n_dir, B, H, W, L, ctx2d, n_iter=2):
  rng = np.random.default_rng(L * 17 + n_dir)
  rho = 0.5 if mode == "TRWP" else 1.0
  unary = (rng.random((B, 1, H, W, L)) * 3).astype(np.float32)
  if ctx2d:
    ctx = (np.triu(rng.random((L, L)), 1) + np.diag(0.1 + 0.2 * rng.random(L))).astype(np.float32)
  else:
    ctx = (0.3 * np.minimum(np.arange(L), 3)).astype(np.float32)
    ctx[0] = 0.1
  ew = (0.1 + 0.9 * rng.random((n_dir, B, 1, H, W))).astype(np.float32)
  dcost = rng.standard_normal((B, 1, H, W, L)).astype(np.float32)
  ref = oracle.forward(mode, unary, ctx, ew, n_dir, n_iter, rho)
  return rho, ctx, ew, dcost, ref["msg_min_index"], ref["msg_norm_index"]


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("mode,n_dir,B,H,W,L,ctx2d", CASES)
def test_outputs_switched_off_leave_the_rest_unchanged(gpu, oracle, mode, n_dir, B, H, W, L, ctx2d,
                                                       packed):
  from mplayers_amd import _lib
  if packed and L > 32:
    pytest.skip("several chains per wavefront exist for at most 32 labels")
  flags = _lib.F_PACKED_ALWAYS if packed else _lib.F_PACKED_OFF
  rho, ctx, ew, dcost, imin, inorm = _problem(oracle, mode, n_dir, B, H, W, L, ctx2d)
  print("case", mode, n_dir, L, ctx2d, packed, flush=True)
  full = gpu.gpu_backward(mode, ctx, ew, dcost, imin, inorm, rho, flags=flags)
  for want_dctx, want_dedge in ((False, False), (True, False), (False, True)):
    got = gpu.gpu_backward(mode, ctx, ew, dcost, imin, inorm, rho, flags=flags,
                           want_dctx=want_dctx, want_dedge=want_dedge, garbage_scratch=True)
    assert np.array_equal(got[0], full[0]), ("dunary", want_dctx, want_dedge)
    if want_dedge:
      assert np.array_equal(got[2], full[2]), "dedge"
    else:
      assert got[2] is None
    if want_dctx:
      assert np.abs(got[1] - full[1]).max() <= 1e-5 * max(1.0, np.abs(full[1]).max()), "dcontext"
    else:
      assert got[1] is None


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("mode,n_dir,B,H,W,L,ctx2d", [c for c in CASES if c[0] == "TRWP"])
def test_same_label_flag_matches_oracle(gpu, oracle, mode, n_dir, B, H, W, L, ctx2d, packed):
  from mplayers_amd import _lib
  if packed and L > 32:
    pytest.skip("several chains per wavefront exist for at most 32 labels")
  flags = _lib.F_PACKED_ALWAYS if packed else _lib.F_PACKED_OFF
  rho, ctx, ew, dcost, imin, inorm = _problem(oracle, mode, n_dir, B, H, W, L, ctx2d)
  print("case", mode, n_dir, L, ctx2d, packed, flush=True)
  du, dc, de = oracle.backward(mode, ctx.astype(np.float64), ew.astype(np.float64),
                               dcost.astype(np.float64), imin, inorm, rho, same_label=True)
  got = gpu.gpu_backward(mode, ctx, ew, dcost, imin, inorm, rho, flags=flags, hard_soft=True)
  same = np.diag(dc) if ctx2d else dc[:1]
  assert np.abs(same).max() > 1e-3
  for name, g, r in (("dunary", got[0], du), ("dcontext", got[1], dc), ("dedge", got[2], de)):
    err = np.abs(g.astype(np.float64) - r).max()
    assert err <= 1e-4 * max(1.0, np.abs(r).max()), (name, err)
  # without the flag those entries stay exactly zero
  plain = gpu.gpu_backward(mode, ctx, ew, dcost, imin, inorm, rho, flags=flags)
  assert np.all((np.diag(plain[1]) if ctx2d else plain[1][:1]) == 0)


def test_per_call_flags_override_the_process_default(gpu, oracle):
  """MPL_F_PACKED_OFF / MPL_F_PACKED_ALWAYS choose the kernels of one call whatever
  mpl_set_option says (two callers in one process cannot switch each other's kernels): the packed
  and the unpacked reverse scans sum dedge in different orders, which shows which one ran."""
  from mplayers_amd import _lib
  rho, ctx, ew, dcost, imin, inorm = _problem(oracle, "ISGMR", 8, 2, 9, 11, 21, True)
  run = lambda flags: gpu.gpu_backward("ISGMR", ctx, ew, dcost, imin, inorm, rho, flags=flags)
  try:
    _lib.set_option(_lib.OPT_PACKED_SCANS, 0)
    off_default = run(0)
    always_by_flag = run(_lib.F_PACKED_ALWAYS)
    _lib.set_option(_lib.OPT_PACKED_SCANS, 2)
    always_default = run(0)
    off_by_flag = run(_lib.F_PACKED_OFF)
  finally:
    _lib.set_option(_lib.OPT_PACKED_SCANS, 1)
  assert np.array_equal(off_default[2], off_by_flag[2])
  assert np.array_equal(always_default[2], always_by_flag[2])
  assert np.array_equal(off_default[0], off_by_flag[0])
  assert np.array_equal(always_default[0], always_by_flag[0])
  assert not np.array_equal(off_default[2], always_default[2])
  assert np.abs(off_default[2] - always_default[2]).max() <= 1e-4 * np.abs(off_default[2]).max()


@pytest.mark.parametrize("mode,L", [("TRWP", 21), ("ISGMR", 12), ("TRWP", 96)])
@pytest.mark.parametrize("with_edge_weights", [True, False])
def test_module_with_a_frozen_table(gpu, mode, L, with_edge_weights):
  """autograd's needs_input_grad decides which gradients the backward operators are asked for:
  with a table that is not trained and edge weights that need no gradient the module hands the
  operators no dcontext / dedge_weights tensor.  dunary must be the bits of the run that computes
  everything, and the gradients that were not asked for come back as None."""
  import argparse
  import torch
  from mplayers_amd import MPModule
  rng = np.random.default_rng(L + 1)
  B, H, W, n_dir, n_iter = 2, 6, 7, 4, 2
  args = argparse.Namespace(mpnet_mrf_mode=mode, mpnet_max_iter=n_iter, mpnet_n_dirs=n_dir,
                            n_classes=L, mpnet_term_weight=1.0, mpnet_smoothness_train="",
                            mpnet_diag_value=0, enable_symmetric=True)
  if L == 21:
    ctx = np.triu(rng.random((L, L)), 1).astype(np.float32)
    loc, diag = np.triu_indices(L, k=1), [range(L), range(L)]
  else:
    ctx = np.concatenate([[0], rng.random(L - 1)]).astype(np.float32)
    loc, diag = np.arange(1, L), [0]
  unary = torch.from_numpy(rng.standard_normal((B, 1, L, H, W)).astype(np.float32)).cuda()
  ew = torch.from_numpy((0.1 + 0.9 * rng.random((B, n_dir, H, W))).astype(np.float32)).cuda()
  dcost = torch.from_numpy(rng.standard_normal((B, 1, L, H, W)).astype(np.float32)).cuda()

  def run(train_table, train_edges):
    mod = MPModule(args).cuda().train()
    table = torch.nn.Parameter(torch.from_numpy(ctx).cuda(), requires_grad=train_table)
    mod.set_label_context(table, loc, diag)
    u = unary.clone().requires_grad_(True)
    e = ew.clone().requires_grad_(train_edges) if with_edge_weights else None
    cost = mod(u, e)[0]
    cost.backward(dcost)
    torch.cuda.synchronize()
    return cost.detach(), u.grad, table.grad, (e.grad if e is not None else None)

  full = run(True, True)
  frozen = run(False, False)
  assert torch.equal(frozen[0], full[0])
  assert torch.equal(frozen[1], full[1])
  assert frozen[2] is None and frozen[3] is None
  assert full[2] is not None and float(full[2].abs().max()) > 0
  assert (full[3] is not None) == with_edge_weights
  table_only = run(True, False)
  assert torch.equal(table_only[1], full[1]) and table_only[3] is None
  assert float((table_only[2] - full[2]).abs().max()) <= 1e-5 * max(1.0, float(full[2].abs().max()))


def test_hard_soft_module_with_a_frozen_table(gpu):
  """The hard path of the hard/soft module (which asks for the same-label dcontext terms) with
  and without a trained table: the same dunary bits, no table gradient when it is frozen."""
  import argparse
  import torch
  from mplayers_amd.MP_module_hard_soft import MPModule as MPModule_hard_soft
  rng = np.random.default_rng(77)
  B, L, H, W, n_dir, n_iter = 2, 21, 6, 7, 4, 2
  unary = torch.from_numpy(rng.standard_normal((B, 1, L, H, W)).astype(np.float32)).cuda()
  dcost = torch.from_numpy(rng.standard_normal((B, 1, L, H, W)).astype(np.float32)).cuda()
  outs = []
  for smoothness_train in ("on", ""):
    args = argparse.Namespace(mpnet_mrf_mode="TRWP", mpnet_max_iter=n_iter, mpnet_n_dirs=n_dir,
                              n_classes=L, mpnet_term_weight=1.0,
                              mpnet_smoothness_train=smoothness_train, mpnet_smoothness_mode="Potts",
                              mpnet_smoothness_trunct_value=-1, mpnet_smoothness_trunct_loc=-1,
                              mpnet_diag_value=0, enable_symmetric=True, mpnet_enable_soft=False,
                              enable_cuda=True)
    mod = MPModule_hard_soft(args, enable_create_label_context=True).cuda().train()
    u = unary.clone().requires_grad_(True)
    cost = mod(u, None)[0]
    cost.backward(dcost)
    torch.cuda.synchronize()
    outs.append((cost.detach(), u.grad, mod.label_context.grad))
  assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
  assert outs[0][2] is not None and outs[1][2] is None
