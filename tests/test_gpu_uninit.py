"""msg_uninit: the forward operators told that the messages start at zero must ignore the contents
of `msg` on entry (here: NaN) and give bit-identical results to a call on a cleared tensor, on
every code path (one chain per wavefront and packed scans, band and dense contexts, odd and even
iteration counts, rho != 1, 16 directions, degenerate grids)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

CASES = [
    # mode, L, n_dir, B, H, W, n_iter, rho, train
    ("TRWP", 16, 4, 1, 9, 13, 3, 0.5, True),
    ("TRWP", 96, 8, 2, 10, 12, 2, 0.5, True),
    ("TRWP", 21, 4, 2, 17, 15, 1, 0.5, True),     # 2-D context, a single iteration
    ("TRWP", 192, 2, 1, 6, 9, 1, 0.5, False),     # one pair of directions only
    ("TRWP", 7, 16, 1, 9, 9, 2, 0.3, True),
    ("TRWP", 12, 8, 40, 12, 14, 2, 0.5, True),    # packed scans
    ("TRWP", 5, 4, 1, 1, 7, 2, 0.5, True),        # one row
    ("TRWP", 5, 4, 1, 6, 1, 2, 0.5, False),       # one column
    ("ISGMR", 16, 4, 1, 9, 13, 3, 1.0, True),     # odd iteration count
    ("ISGMR", 96, 8, 2, 10, 12, 2, 1.0, True),    # even
    ("ISGMR", 21, 8, 2, 17, 15, 1, 1.0, True),
    ("ISGMR", 33, 4, 1, 8, 9, 2, 0.7, True),      # rho != 1: the library clears the tensor itself
    ("ISGMR", 7, 16, 1, 9, 9, 3, 1.0, False),
    ("ISGMR", 12, 8, 40, 12, 14, 3, 1.0, True),   # packed scans
    ("ISGMR", 4, 4, 1, 1, 1, 2, 1.0, True),       # a single pixel
]


@pytest.mark.parametrize("mode,L,n_dir,B,H,W,n_iter,rho,train", CASES)
def test_uninitialised_messages_match_cleared_ones(gpu, mode, L, n_dir, B, H, W, n_iter, rho, train):
  import torch
  from mplayers_amd import lib_stereo
  g = torch.Generator().manual_seed(1000 * L + n_dir)
  dev = "cuda"
  unary = torch.randn(B, 1, H, W, L, generator=g).to(dev)
  if L == 21:
    context = torch.rand(L, L, generator=g).triu(1).to(dev)
  elif L % 2:
    context = torch.rand(L, generator=g).to(dev)                      # dense path
  else:
    context = (0.3 * torch.arange(L, dtype=torch.float32).clamp(max=3)).to(dev)
  edge = (0.1 + 0.9 * torch.rand(n_dir, B, 1, H, W, generator=g)).to(dev)
  u8 = dict(dtype=torch.uint8, device=dev)

  def run(uninit):
    msg = torch.full((n_dir, B, 1, H, W, L), float("nan"), device=dev) if uninit else \
        torch.zeros(n_dir, B, 1, H, W, L, device=dev)
    msg_tmp = torch.full_like(msg, float("nan"))
    cost = torch.full((B, 1, H, W, L), float("nan"), device=dev)
    scratch = torch.full_like(cost, float("nan"))
    imin = torch.zeros(n_iter, n_dir, B, 1, H, W, L, **u8) if train else torch.empty(0, **u8)
    inorm = torch.zeros(n_iter, n_dir, B, 1, H, W, **u8) if train else torch.empty(0, **u8)
    label = torch.zeros(n_iter, B, 1, H, W, **u8)
    if mode == "TRWP":
      lib_stereo.TRWP.forward(rho, n_iter, 0, unary, context, edge, msg, cost, imin, inorm, scratch,
                              label, msg_uninit=uninit)
    else:
      lib_stereo.ISGMR.forward(0, rho, n_iter, 0, unary, context, edge, msg, cost, imin, inorm,
                               scratch, msg_tmp, label, msg_uninit=uninit)
    torch.cuda.synchronize()
    return dict(msg=msg, cost=cost, imin=imin, inorm=inorm, label=label)

  want, got = run(False), run(True)
  for name in want:
    assert not torch.isnan(got[name].float()).any(), name
    assert torch.equal(got[name], want[name]), name


def test_module_allocates_without_clearing(gpu):
  """MPModule hands the operators an uncleared message tensor; its results equal the operator
  level's on cleared messages."""
  import argparse
  import torch
  from mplayers_amd import lib_stereo
  from mplayers_amd.MP_module import MPModule
  g = torch.Generator().manual_seed(5)
  B, L, H, W, n_dir, n_iter = 2, 12, 11, 9, 8, 3
  unary = torch.randn(B, 1, L, H, W, generator=g).cuda()
  edge = (0.1 + 0.9 * torch.rand(B, n_dir, H, W, generator=g)).cuda()
  context = (0.25 * torch.arange(L, dtype=torch.float32).clamp(max=2)).cuda()
  for mode, rho in (("TRWP", 0.5), ("ISGMR", 1.0)):
    args = argparse.Namespace(n_classes=L, mpnet_n_dirs=n_dir, mpnet_max_iter=n_iter,
                              mpnet_term_weight=1, mpnet_smoothness_train=None,
                              mpnet_mrf_mode=mode)
    module = MPModule(args).eval()
    module.set_label_context(context, None, None)
    # poison the allocator's free blocks so that an uncleared tensor really holds garbage
    junk = torch.full((n_dir, B, 1, H, W, L), float("nan"), device="cuda")
    del junk
    cost = module(unary, edge)[0]
    u = unary.permute(0, 1, 3, 4, 2).contiguous()
    e = edge.unsqueeze(1).permute(2, 0, 1, 3, 4).contiguous()
    msg = torch.zeros(n_dir, B, 1, H, W, L, device="cuda")
    ref = torch.empty_like(u)
    empty = torch.empty(0, dtype=torch.uint8, device="cuda")
    if mode == "TRWP":
      lib_stereo.TRWP.forward(rho, n_iter, 0, u, context, e, msg, ref, empty, empty,
                              torch.empty_like(u), empty)
    else:
      lib_stereo.ISGMR.forward(0, rho, n_iter, 0, u, context, e, msg, ref, empty, empty,
                               torch.empty_like(u), torch.empty_like(msg), empty)
    assert torch.equal(cost, ref.permute(0, 1, 4, 2, 3).contiguous()), mode


@pytest.mark.parametrize("mode,L,n_dir,n_iter", [("TRWP", 96, 4, 2), ("TRWP", 40, 8, 1), ("ISGMR", 96, 8, 2),
                                                 ("ISGMR", 40, 8, 3), ("ISGMR", 70, 4, 3), ("ISGMR", 12, 8, 2)])
def test_given_initial_messages_are_used(gpu, oracle, mode, L, n_dir, n_iter):
  """Under the reference's contract `msg` holds the initial messages.  The library looks at them
  on the device and takes its shortcuts only when they are all zero: messages that are not zero
  (here: the result of an earlier call, and a tensor with a single entry that is not zero) must
  come out as the oracle continues from them."""
  rng = np.random.default_rng(L + n_dir)
  B, H, W = 1, 7, 9
  rho = 0.5 if mode == "TRWP" else 1.0
  unary = (rng.random((B, 1, H, W, L)) * 3).astype(np.float32)
  ctx = (0.3 * np.minimum(np.arange(L), 3)).astype(np.float32)
  ew = (0.1 + 0.9 * rng.random((n_dir, B, 1, H, W))).astype(np.float32)
  first = oracle.forward(mode, unary, ctx, ew, n_dir, 1, rho)["msg"]
  single = np.zeros_like(first)
  single[n_dir - 1, 0, 0, H - 1, W - 1, L - 1] = 0.75  # the last element of the last plane
  for init in (first, single):
    ref = oracle.forward(mode, unary, ctx, ew, n_dir, n_iter, rho, msg_init=init, saving_label=True,
                         want_gaps=True)
    got = gpu.gpu_forward(mode, unary, ctx, ew, n_dir, n_iter, rho, msg_init=init,
                          saving_label=True)
    gpu.assert_values_close(got["msg"], ref["msg"], what="msg", belief=ref["cost_final"])
    gpu.assert_values_close(got["cost_final"], ref["cost_final"], what="cost_final")
    tol = 2e-5 * max(1.0, float(np.abs(ref["cost_final"]).max()))
    gpu.assert_indices_match_off_ties(got["msg_min_index"], ref["msg_min_index"], ref["gap_min"],
                                      tol, "msg_min_index")
    gpu.assert_labels_match_off_ties(got["label_all"], ref["label_all"], ref["gap_label"], tol)
