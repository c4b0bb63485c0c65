"""The two inference configurations at their real shape: TRWP forward on the stereo-shaped
384 x 1248 x 96 problem (4 directions, 5 iterations) and ISGMR forward on the denoise-shaped
256 x 256 x 256 one (4 directions, 50 iterations).

  * the denoise problem is integer valued (squared differences to an 8-bit image, a truncated
    quadratic table of integers, unit weights, rho = 1), so fp32 arithmetic is exact and all 50
    Jacobi iterations must agree with the oracle bit for bit -- messages, costs and labels, ties
    included -- on a crop the CPU finishes in seconds;
  * at full size one TRWP iteration is within the oracle's reach, all iterations are checked
    through properties that hold at any size, and single rows / columns of a two-direction run
    (rows do not interact then) are checked exactly over all iterations.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _np(cfg):
  return cfg["unary"].numpy(), cfg["context"].numpy(), cfg["edge_weights"].numpy()


def test_denoise_config_all_50_iterations_bit_exact(gpu, oracle):
  from mplayers_amd import synthetic
  cfg = synthetic.make_config("C3", seed=0, scale=0.12)
  unary, ctx, ew = _np(cfg)
  assert cfg["n_iter"] == 50 and cfg["L"] == 256 and unary.shape[2:4] == (31, 31)
  assert np.array_equal(unary, np.round(unary)) and np.array_equal(ctx, np.round(ctx))
  print("C3 crop", unary.shape, flush=True)
  ref = oracle.forward("ISGMR", unary, ctx, ew, 4, 50, 1.0, training=False, saving_label=True)
  assert float(np.abs(ref["cost_final"]).max()) < 2 ** 24  # every sum is an exact fp32 integer
  got = gpu.gpu_forward("ISGMR", unary, ctx, ew, 4, 50, 1.0, training=False, saving_label=True)
  for k in ("msg", "cost_final", "label_all"):
    assert np.array_equal(got[k], ref[k]), k
  # the labelling still changes late in the run: the iterations are not idle
  assert (ref["label_all"][10] != ref["label_all"][-1]).any()
  # training mode writes the indices and must not change the values
  ref_t = oracle.forward("ISGMR", unary, ctx, ew, 4, 50, 1.0, training=True)
  got_t = gpu.gpu_forward("ISGMR", unary, ctx, ew, 4, 50, 1.0, training=True)
  for k in ("msg", "cost_final", "msg_min_index", "msg_norm_index"):
    assert np.array_equal(got_t[k], ref_t[k]), k


def test_stereo_config_full_size_one_iteration_matches_oracle(gpu, oracle):
  """384 x 1248 x 96, 4 directions: one full-size TRWP iteration against the oracle."""
  from mplayers_amd import synthetic
  cfg = synthetic.make_config("C2", seed=0)
  unary, ctx, ew = _np(cfg)
  print("C2 full size, 1 iteration", unary.shape, flush=True)
  ref = oracle.forward("TRWP", unary, ctx, ew, 4, 1, 0.5, training=False, saving_label=True,
                       want_gaps=True)
  got = gpu.gpu_forward("TRWP", unary, ctx, ew, 4, 1, 0.5, training=False, saving_label=True)
  gpu.assert_values_close(got["msg"], ref["msg"], what="msg", belief=ref["cost_final"])
  gpu.assert_values_close(got["cost_final"], ref["cost_final"], what="cost_final")
  tol = 2e-5 * max(1.0, float(np.abs(ref["cost_final"]).max()))
  n_bad = gpu.assert_labels_match_off_ties(got["label_all"], ref["label_all"], ref["gap_label"], tol)
  assert n_bad <= 1e-4 * ref["label_all"].size


def _forward_on_gpu(cfg, n_dir, edge, n_iter, labels=True):
  import torch
  from mplayers_amd import lib_stereo
  dev = "cuda:0"
  B, H, W, L = cfg["B"], cfg["H"], cfg["W"], cfg["L"]
  unary = cfg["unary"].to(dev)
  ctx = cfg["context"].to(dev)
  ew = edge.contiguous().to(dev)
  msg = torch.zeros(n_dir, B, 1, H, W, L, device=dev)
  cost = torch.zeros(B, 1, H, W, L, device=dev)
  scratch = torch.zeros(B, 1, H, W, L, device=dev)
  empty = torch.empty(0, dtype=torch.uint8)
  lab = torch.zeros(n_iter, B, 1, H, W, dtype=torch.uint8, device=dev) if labels else empty
  if cfg["mode"] == "TRWP":
    lib_stereo.TRWP.forward(cfg["rho"], n_iter, 0, unary, ctx, ew, msg, cost, empty, empty, scratch,
                            lab)
  else:
    tmp = torch.zeros_like(msg)
    lib_stereo.ISGMR.forward(0, cfg["rho"], n_iter, 0, unary, ctx, ew, msg, cost, empty, empty,
                             scratch, tmp, lab)
  torch.cuda.synchronize()
  return unary, msg, cost, lab


@pytest.mark.parametrize("name", ["C2", "C3"])
def test_inference_config_properties_at_full_size(gpu, name):
  """All iterations at the real shape, through what must hold at any size."""
  import torch
  from mplayers_amd import synthetic
  cfg = synthetic.make_config(name, seed=0)
  n_dir, n_iter, L = cfg["n_dir"], cfg["n_iter"], cfg["L"]
  print("full size", name, cfg["mode"], cfg["unary"].shape, n_iter, flush=True)
  unary, msg, cost, lab = _forward_on_gpu(cfg, n_dir, cfg["edge_weights"], n_iter)
  assert bool(torch.isfinite(msg).all())
  # every message vector is normalised: its minimum is exactly 0; chain starts stay all zero
  assert float(msg.amin(dim=-1).abs().max()) == 0.0
  assert float(msg[0, 0, 0, :, 0].abs().max()) == 0.0   # direction 0 starts at the left column
  assert float(msg[1, 0, 0, :, -1].abs().max()) == 0.0  # direction 1 at the right column
  assert float(msg[2, 0, 0, 0].abs().max()) == 0.0      # direction 2 at the top row
  assert float(msg[3, 0, 0, -1].abs().max()) == 0.0     # direction 3 at the bottom row
  assert float(msg[0, 0, 0, :, 1:].amax(dim=-1).min()) > 0.0
  # cost_final = unary + sum_k msg_k in direction order, bit for bit; labels = its argmin
  acc = unary.clone()
  for k in range(n_dir):
    acc += msg[k]
  assert torch.equal(acc, cost)
  assert torch.equal(cost.argmin(dim=-1).to(torch.uint8), lab[-1])
  assert int(lab.max()) < L
  # message passing changes the labelling of the data term, and keeps refining it
  data_only = unary.argmin(dim=-1).to(torch.uint8)
  assert float((lab[-1] != data_only).float().mean()) > 0.01
  assert bool((lab[0] != lab[-1]).any())


@pytest.mark.parametrize("name", ["C2", "C3"])
def test_inference_config_rows_and_columns_match_oracle(gpu, oracle, name):
  """Two horizontal directions only: rows do not interact, so single rows of a full-size run with
  all iterations are small problems for the oracle.  The same with the vertical pair (the
  horizontal one switched off by zero weights) for single columns."""
  import torch
  from mplayers_amd import synthetic
  cfg = synthetic.make_config(name, seed=0)
  mode, rho, n_iter = cfg["mode"], cfg["rho"], cfg["n_iter"]
  H, W = cfg["H"], cfg["W"]
  ctx = cfg["context"].numpy()
  exact = name == "C3"  # integer-valued problem
  print("rows", name, flush=True)
  unary, msg, cost, _ = _forward_on_gpu(cfg, 2, cfg["edge_weights"][:2], n_iter, labels=False)
  rows = torch.tensor([0, H // 2, H - 1])
  un = cfg["unary"].index_select(2, rows).numpy()
  en = cfg["edge_weights"][:2].index_select(3, rows).contiguous().numpy()
  ref = oracle.forward(mode, un, ctx, en, 2, n_iter, rho, training=False)
  got_msg = msg.index_select(3, rows.cuda()).cpu().numpy()
  got_cost = cost.index_select(2, rows.cuda()).cpu().numpy()
  if exact:
    assert np.array_equal(got_msg, ref["msg"]) and np.array_equal(got_cost, ref["cost_final"])
  else:
    gpu.assert_values_close(got_msg, ref["msg"], what="row msg", belief=ref["cost_final"])
    gpu.assert_values_close(got_cost, ref["cost_final"], what="row cost")
  del unary, msg, cost
  print("columns", name, flush=True)
  ew = cfg["edge_weights"].clone()
  ew[:2] = 0
  unary, msg, cost, _ = _forward_on_gpu(cfg, 4, ew, n_iter, labels=False)
  assert float(msg[:2].abs().max()) == 0.0
  cols = torch.tensor([0, W // 3, W - 1])
  # a column as a 1 x H image scanned by the horizontal pair
  un = cfg["unary"].index_select(3, cols).permute(0, 1, 3, 2, 4).contiguous().numpy()   # (1,1,3,H,L)
  en = ew[2:4].index_select(4, cols).permute(0, 1, 2, 4, 3).contiguous().numpy()         # (2,1,1,3,H)
  ref = oracle.forward(mode, un, ctx, en, 2, n_iter, rho, training=False)
  got_msg = msg[2:4].index_select(4, cols.cuda()).permute(0, 1, 2, 4, 3, 5).contiguous().cpu().numpy()
  got_cost = cost.index_select(3, cols.cuda()).permute(0, 1, 3, 2, 4).contiguous().cpu().numpy()
  if exact:
    assert np.array_equal(got_msg, ref["msg"]) and np.array_equal(got_cost, ref["cost_final"])
  else:
    gpu.assert_values_close(got_msg, ref["msg"], what="column msg", belief=ref["cost_final"])
    gpu.assert_values_close(got_cost, ref["cost_final"], what="column cost")
