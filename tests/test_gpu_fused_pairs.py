"""TRWP launches with at most 1024 chains run both sweeps of a pair of opposite directions in one
launch (the wavefront of a chain sweeps it forth and then back).  Nothing about the arithmetic
changes, so every output must be bit-identical to the one-launch-per-direction path that
MPL_F_FUSED_PAIRS_OFF selects: band, scan and dense contexts, 1 to 4 labels per lane, training and
inference, cleared and undeclared initial messages, non-zero initial messages, degenerate grids."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

CASES = [
    # L, n_dir, B, H, W, n_iter, rho, train, context kind
    (16, 4, 1, 9, 13, 3, 0.5, True, "tl3"),
    (96, 8, 2, 10, 12, 2, 0.5, True, "tl2"),        # two labels per lane, band of 2
    (21, 4, 4, 33, 31, 2, 0.5, True, "dense2d"),    # the segmentation case, 21-label dense step
    (21, 8, 1, 12, 9, 2, 0.5, False, "dense2d"),
    (192, 2, 1, 6, 9, 1, 0.5, False, "tl4"),        # one pair of directions only, three labels per lane
    (192, 4, 1, 5, 7, 2, 0.5, True, "tq"),
    (256, 4, 1, 4, 6, 2, 0.5, True, "tl12"),        # wide truncated linear: label-scan step
    (7, 16, 1, 9, 9, 2, 0.3, True, "dense1d"),
    (33, 8, 2, 8, 9, 2, 0.5, True, "dense1d"),
    (100, 4, 1, 6, 7, 2, 0.5, True, "dense1d"),     # dense 1-D table, two labels per lane
    (5, 4, 1, 1, 7, 2, 0.5, True, "tl2"),           # one row
    (5, 4, 1, 6, 1, 2, 0.5, False, "tl2"),          # one column
    (4, 4, 1, 1, 1, 2, 0.5, True, "tl2"),           # a single pixel
    (12, 8, 3, 12, 14, 2, 0.5, True, "negw"),       # negative edge weights: dense fallback per pixel
]


def make_context(kind, L, g):
  import torch
  k = torch.arange(L, dtype=torch.float32)
  if kind.startswith("tl"):
    return 0.3 * k.clamp(max=float(kind[2:]))
  if kind == "tq":
    return 0.05 * (k * k).clamp(max=9.0)
  if kind == "dense2d":
    return torch.rand(L, L, generator=g).triu(1)
  return torch.rand(L, generator=g)


PACKED_CASES = [
    # several chains per wavefront (forced for these sizes): the packed scans fuse pairs, too
    (21, 4, 3, 14, 15, 2, 0.5, True, "dense2d"),
    (12, 8, 5, 9, 11, 2, 0.5, True, "tl3"),
    (32, 4, 2, 8, 9, 2, 0.5, False, "dense1d"),
    (5, 16, 2, 7, 9, 1, 0.5, True, "dense1d"),
]


@pytest.mark.parametrize("L,n_dir,B,H,W,n_iter,rho,train,kind", PACKED_CASES)
@pytest.mark.parametrize("start", ["cleared", "uninit", "given"])
def test_fused_pairs_packed_are_bit_identical(gpu, L, n_dir, B, H, W, n_iter, rho, train, kind, start):
  from mplayers_amd import _lib
  test_fused_pairs_are_bit_identical(gpu, L, n_dir, B, H, W, n_iter, rho, train, kind, start,
                                     base_flags=_lib.F_PACKED_ALWAYS)


@pytest.mark.parametrize("L,n_dir,B,H,W,n_iter,rho,train,kind", CASES)
@pytest.mark.parametrize("start", ["cleared", "uninit", "given"])
def test_fused_pairs_are_bit_identical(gpu, L, n_dir, B, H, W, n_iter, rho, train, kind, start,
                                       base_flags=0):
  import torch
  from mplayers_amd import _lib, lib_stereo
  g = torch.Generator().manual_seed(77 * L + n_dir)
  dev = "cuda"
  unary = torch.randn(B, 1, H, W, L, generator=g).to(dev)
  context = make_context(kind, L, g).to(dev)
  edge = 0.1 + 0.9 * torch.rand(n_dir, B, 1, H, W, generator=g)
  if kind == "negw":
    edge = edge - 0.3
  edge = edge.to(dev)
  msg0 = 0.5 * torch.rand(n_dir, B, 1, H, W, L, generator=g).to(dev)
  dcost = torch.randn(B, 1, H, W, L, generator=g).to(dev)
  u8 = dict(dtype=torch.uint8, device=dev)
  print("case", L, n_dir, B, H, W, n_iter, rho, train, kind, start, flush=True)

  def run(flags):
    if start == "given":
      msg = msg0.clone()
    elif start == "uninit":
      msg = torch.full((n_dir, B, 1, H, W, L), float("nan"), device=dev)
    else:
      msg = torch.zeros(n_dir, B, 1, H, W, L, device=dev)
    cost = torch.full((B, 1, H, W, L), float("nan"), device=dev)
    scratch = torch.full_like(cost, float("nan"))
    imin = torch.zeros(n_iter, n_dir, B, 1, H, W, L, **u8) if train else torch.empty(0, **u8)
    inorm = torch.zeros(n_iter, n_dir, B, 1, H, W, **u8) if train else torch.empty(0, **u8)
    label = torch.zeros(n_iter, B, 1, H, W, **u8)
    lib_stereo.TRWP.forward(rho, n_iter, 0, unary, context, edge, msg, cost, imin, inorm, scratch,
                            label, msg_uninit=(start == "uninit"), flags=flags)
    out = [msg, cost, imin, inorm, label]
    if train:
      dunary = torch.zeros(B, 1, H, W, L, device=dev)
      dctx = torch.zeros_like(context)
      dedge = torch.zeros(n_dir, B, 1, H, W, device=dev)
      dmsg = torch.full((n_dir, B, 1, H, W, L), float("nan"), device=dev)
      lib_stereo.TRWP.backward(rho, context, edge, dcost, imin, inorm, dunary, dctx, dedge, dmsg,
                               scratch, flags=flags)
      out += [dunary, dedge]
      torch.cuda.synchronize()
      return [o.cpu().numpy() for o in out], dctx.cpu().numpy()
    torch.cuda.synchronize()
    return [o.cpu().numpy() for o in out], None

  fused, dc_f = run(base_flags)
  plain, dc_p = run(base_flags | _lib.F_FUSED_PAIRS_OFF)
  names = ["msg", "cost_final", "msg_min_index", "msg_norm_index", "label_all", "dunary", "dedge"]
  for name, a, b in zip(names, fused, plain):
    assert not np.isnan(a.astype(np.float64)).any(), name
    assert np.array_equal(a, b), (name, np.abs(a.astype(np.float64) - b).max())
  if dc_f is not None:  # float atomics across chains: equal up to their order
    assert np.abs(dc_f - dc_p).max() <= 1e-4 * max(1.0, np.abs(dc_p).max())


SOFT_CASES = [
    # L, n_dir, B, H, W, n_iter
    (21, 4, 2, 17, 15, 2),    # three lane groups, 2-D context
    (16, 8, 1, 9, 11, 2),     # four groups
    (30, 4, 1, 6, 7, 1),      # two groups
    (5, 16, 1, 7, 8, 2),
    (3, 4, 1, 1, 9, 2),       # one row
]


@pytest.mark.parametrize("L,n_dir,B,H,W,n_iter", SOFT_CASES)
@pytest.mark.parametrize("train", [True, False])
def test_fused_pairs_soft_are_bit_identical(gpu, L, n_dir, B, H, W, n_iter, train):
  """The soft-weighted scans of at most 32 labels fuse pairs the same way."""
  import torch
  from mplayers_amd import _lib, lib_stereo
  g = torch.Generator().manual_seed(31 * L + n_dir)
  dev = "cuda"
  unary = torch.rand(B, 1, H, W, L, generator=g).to(dev)
  context = (torch.rand(L, L, generator=g).triu() if L == 21 else torch.rand(L, generator=g)).to(dev)
  edge = (0.2 + torch.rand(n_dir, B, 1, H, W, generator=g)).to(dev)
  dcost = torch.randn(B, 1, H, W, L, generator=g).to(dev)
  u8 = dict(dtype=torch.uint8, device=dev)
  print("soft case", L, n_dir, B, H, W, n_iter, train, flush=True)

  def run(flags):
    msg = torch.zeros(n_dir, B, 1, H, W, L, device=dev)
    cost = torch.zeros(B, 1, H, W, L, device=dev)
    scratch = torch.zeros(B, 1, H, W, L, device=dev)
    mel = torch.zeros(n_iter, n_dir, B, 1, H, W, L, L, device=dev) if train else torch.empty(0)
    inorm = torch.zeros(n_iter, n_dir, B, 1, H, W, **u8) if train else torch.empty(0, dtype=torch.uint8)
    label = torch.zeros(n_iter, B, 1, H, W, **u8)
    lib_stereo.TRWP_hard_soft.forward_soft(rho, n_iter, unary, context, edge, msg, mel, inorm, cost,
                                           scratch, label, flags=flags)
    out = [msg, cost, label]
    dctx = None
    if train:
      dunary = torch.zeros(B, 1, H, W, L, device=dev)
      dctx = torch.zeros_like(context)
      dedge = torch.zeros(n_dir, B, 1, H, W, device=dev)
      dmsg = torch.full((n_dir, B, 1, H, W, L), float("nan"), device=dev)
      lib_stereo.TRWP_hard_soft.backward_soft(rho, dcost, context, edge, mel, inorm, dunary, dctx,
                                              dedge, dmsg, torch.empty(0, device=dev), flags=flags)
      out += [mel, inorm, dunary, dedge]
    torch.cuda.synchronize()
    return [o.cpu().numpy() for o in out], (dctx.cpu().numpy() if dctx is not None else None)

  rho = 0.5
  fused, dc_f = run(0)
  plain, dc_p = run(_lib.F_FUSED_PAIRS_OFF)
  for i, (a, b) in enumerate(zip(fused, plain)):
    assert not np.isnan(a.astype(np.float64)).any(), i
    assert np.array_equal(a, b), (i, np.abs(a.astype(np.float64) - b).max())
  if dc_f is not None:
    assert np.abs(dc_f - dc_p).max() <= 1e-4 * max(1.0, np.abs(dc_p).max())
