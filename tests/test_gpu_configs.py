"""GPU parity on the benchmark configurations (scaled to sizes the CPU oracle finishes in seconds),
on the reference-built fixtures, through the nn.Module surface, and -- at the full size of the large
configuration -- through size-independent properties."""
import argparse
import glob
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
# (the fixtures of the SGM flag pin the CPU forward alone, tests/test_cpu_forward.py: that flag
# rewrites the unary tensor on the reference's CPU path, which neither the GPU semantics nor the
# oracle's restatement of the CPU loop nest do)
REFCPU_FIXTURES = [p for p in sorted(glob.glob(os.path.join(GOLDEN, "refcpu_*.npz")))
                   if "refcpu_sgm" not in p]


CONFIG_CASES = [
    # config, mode, scale, n_iter override
    ("C1", "ISGMR", 1.0, None),
    ("C2", "TRWP", 0.1, None),
    ("C3", "ISGMR", 0.12, 5),
    ("C4", "TRWP", 1.0, None),
    ("C4", "ISGMR", 1.0, None),
    ("C5", "TRWP", 0.02, None),
    ("C5", "ISGMR", 0.02, None),
]


@pytest.mark.parametrize("name,mode,scale,n_iter", CONFIG_CASES)
def test_config_matches_oracle(gpu, oracle, name, mode, scale, n_iter):
  from mplayers_amd import synthetic
  cfg = synthetic.make_config(name, seed=0, scale=scale, mode=mode)
  n_iter = n_iter or cfg["n_iter"]
  unary, ctx, ew = cfg["unary"].numpy(), cfg["context"].numpy(), cfg["edge_weights"].numpy()
  train = cfg["training"]
  print("config", name, mode, unary.shape, "n_iter", n_iter, flush=True)
  ref = oracle.forward(mode, unary, ctx, ew, cfg["n_dir"], n_iter, cfg["rho"], training=train,
                       want_gaps=True, saving_label=True)
  got = gpu.gpu_forward(mode, unary, ctx, ew, cfg["n_dir"], n_iter, cfg["rho"], training=train,
                        saving_label=True)
  gpu.assert_values_close(got["msg"], ref["msg"], what="msg", belief=ref["cost_final"])
  gpu.assert_values_close(got["cost_final"], ref["cost_final"], what="cost_final")
  tol = 2e-5 * max(1.0, float(np.abs(ref["cost_final"]).max()))
  n_bad = gpu.assert_labels_match_off_ties(got["label_all"], ref["label_all"], ref["gap_label"], tol)
  assert n_bad <= 1e-3 * ref["label_all"].size
  if not train:
    return
  n_bad = gpu.assert_indices_match_off_ties(got["msg_min_index"], ref["msg_min_index"],
                                            ref["gap_min"], tol, "msg_min_index")
  assert n_bad <= 1e-3 * ref["msg_min_index"].size
  gpu.assert_indices_match_off_ties(got["msg_norm_index"], ref["msg_norm_index"], ref["gap_norm"],
                                    tol, "msg_norm_index")
  # backward on the oracle's indices, against the fp64 oracle
  dcost = synthetic.upstream_grad(cfg).numpy()
  r = oracle.backward(mode, ctx.astype(np.float64), ew.astype(np.float64), dcost.astype(np.float64),
                      ref["msg_min_index"], ref["msg_norm_index"], cfg["rho"])
  g = gpu.gpu_backward(mode, ctx, ew, dcost, ref["msg_min_index"], ref["msg_norm_index"],
                       cfg["rho"])
  for a, b, what in zip(g, r, ("dunary", "dcontext", "dedge_weights")):
    scale_ = max(1.0, float(np.abs(b).max()))
    assert np.abs(a - b).max() <= 1e-4 * scale_, (what, float(np.abs(a - b).max()), scale_)
  assert abs(g[0].astype(np.float64).sum() - dcost.astype(np.float64).sum()) <= 1e-3 * np.abs(dcost).sum() ** 0.5 + 1e-2


@pytest.mark.parametrize("path", REFCPU_FIXTURES,
                         ids=lambda p: os.path.basename(p)[7:-4])
def test_reference_cpu_fixtures(gpu, path):
  """Outputs of the reference's own compiled CPU forward (tests/golden/make_refcpu_golden.py).
  The GPU operator reads one context for all directions, so only the fixtures whose per-direction
  tables are one shared symmetric Toeplitz table apply; unit edge weights as on that CPU path."""
  z = np.load(path)
  ctx = z["context"]
  n_dir, L, _ = ctx.shape
  ii = np.abs(np.arange(L)[:, None] - np.arange(L)[None, :])
  shared = all(np.array_equal(ctx[0], ctx[d]) for d in range(n_dir)) and \
      np.array_equal(ctx[0], ctx[0][0][ii])
  if not shared:
    pytest.skip("per-direction context tables exist only on the reference's CPU path")
  mode, rho, n_iter = str(z["mode"]), float(z["rho"]), int(z["n_iter"])
  c = ctx[0] if L == 21 else ctx[0, 0]
  got = gpu.gpu_forward(mode, z["unary"], c, None, n_dir, n_iter, rho, saving_label=True)
  gpu.assert_values_close(got["msg"], z["msg"], what="msg", belief=z["cost_final"])
  gpu.assert_values_close(got["cost_final"], z["cost_final"], what="cost_final")
  if "int" in path and mode == "ISGMR":
    assert np.array_equal(got["msg"], z["msg"]) and np.array_equal(got["label_all"], z["label_all"])


@pytest.mark.parametrize("mode,L,train_mode", [("TRWP", 21, "sigmoid"), ("ISGMR", 21, ""),
                                               ("ISGMR", 12, "softmax"), ("TRWP", 40, "")])
def test_module_forward_backward(gpu, oracle, mode, L, train_mode):
  """The drop-in surface: MPModule -> autograd Function -> operators -> C ABI."""
  import torch
  from mplayers_amd import MPModule
  rng = np.random.default_rng(L)
  B, H, W, n_dir, n_iter = 2, 7, 9, 4 if mode == "TRWP" else 8, 2
  args = argparse.Namespace(mpnet_mrf_mode=mode, mpnet_max_iter=n_iter, mpnet_n_dirs=n_dir,
                            n_classes=L, mpnet_term_weight=1.5, mpnet_smoothness_train=train_mode,
                            mpnet_smoothness_mode="TL", mpnet_smoothness_trunct_value=3,
                            mpnet_smoothness_trunct_loc=-1, mpnet_diag_value=0.0,
                            enable_symmetric=True, enable_cuda=True)
  mod = MPModule(args, enable_create_label_context=True, enable_saving_label=True).cuda().train()
  unary = rng.standard_normal((B, 1, L, H, W)).astype(np.float32)
  ew = (0.1 + 0.9 * rng.random((B, n_dir, H, W))).astype(np.float32)
  dcost = rng.standard_normal((B, 1, L, H, W)).astype(np.float32)
  u = torch.from_numpy(unary).cuda().requires_grad_(True)
  e = torch.from_numpy(ew).cuda().requires_grad_(True)
  cost, lc_out, labels, _, _ = mod(u, e)
  assert cost.shape == (B, 1, L, H, W) and labels.shape == (n_iter, B, 1, H, W)
  assert lc_out.shape[0] == 1
  cost.backward(torch.from_numpy(dcost).cuda())
  torch.cuda.synchronize()
  ctx = lc_out[0].detach().cpu().numpy()
  un = np.ascontiguousarray(unary.transpose(0, 1, 3, 4, 2))
  en = np.ascontiguousarray(ew[:, None].transpose(2, 0, 1, 3, 4))
  dn = np.ascontiguousarray(dcost.transpose(0, 1, 3, 4, 2))
  rho = 0.5 if mode == "TRWP" else 1.0
  ref = oracle.forward(mode, un, ctx, en, n_dir, n_iter, rho, saving_label=True, want_gaps=True)
  gpu.assert_values_close(cost.detach().cpu().numpy().transpose(0, 1, 3, 4, 2), ref["cost_final"],
                          what="module cost")
  gpu.assert_labels_match_off_ties(labels.cpu().numpy(), ref["label_all"], ref["gap_label"],
                                   2e-5 * max(1.0, float(np.abs(ref["cost_final"]).max())))
  du, dc, de = oracle.backward(mode, ctx.astype(np.float64), en.astype(np.float64),
                               dn.astype(np.float64), ref["msg_min_index"], ref["msg_norm_index"], rho)
  assert np.abs(u.grad.cpu().numpy().transpose(0, 1, 3, 4, 2) - du).max() <= 1e-4 * max(1, np.abs(du).max())
  assert np.abs(e.grad.cpu().numpy()[:, None].transpose(2, 0, 1, 3, 4) - de).max() <= 1e-4 * max(1, np.abs(de).max())
  if train_mode:  # the context parameter is learnable: its gradient flows through the re-parameterisation
    lc = torch.from_numpy(mod.label_context.detach().cpu().numpy().astype(np.float64)).requires_grad_(True)
    loc, diag = mod.label_context_loc, mod.label_context_diag_loc
    eff = lc * 1
    if train_mode == "sigmoid":
      eff[loc] = 2 * args.mpnet_term_weight * torch.sigmoid(eff[loc].flatten())
    else:
      v = eff[loc].flatten()
      sm = torch.softmax(v, 0)
      eff[loc] = sm * v.max() / sm.max()
    eff[tuple(diag) if isinstance(diag, list) else diag] = args.mpnet_diag_value
    eff.backward(torch.from_numpy(dc))
    got = mod.label_context.grad.cpu().numpy()
    assert np.abs(got - lc.grad.numpy()).max() <= 1e-4 * max(1, np.abs(lc.grad.numpy()).max())
  # evaluation mode: no indices are kept, same values
  mod.eval()
  with torch.no_grad():
    cost2, _, _, _, _ = mod(torch.from_numpy(unary).cuda(), torch.from_numpy(ew).cuda())
  assert torch.equal(cost2, cost.detach())
  # without edge weights the third gradient is None (MP_module.py:80-81)
  mod.train()
  u2 = torch.from_numpy(unary).cuda().requires_grad_(True)
  cost3, _, _, _, _ = mod(u2)
  cost3.sum().backward()
  assert u2.grad is not None


def test_operator_error_behaviour(gpu):
  import torch
  from mplayers_amd import lib_stereo
  dev = "cuda:0"
  e = torch.empty(0, dtype=torch.uint8)

  def call(L=5, contiguous=True):
    u = torch.zeros(1, 1, 3, 4, L, device=dev)
    if not contiguous:
      u = torch.zeros(1, 1, 3, L, 4, device=dev).transpose(3, 4)
    msg = torch.zeros(4, 1, 1, 3, 4, L, device=dev)
    lib_stereo.TRWP.forward(0.5, 1, 0, u, torch.zeros(L, device=dev),
                            torch.ones(4, 1, 1, 3, 4, device=dev), msg, torch.zeros(1, 1, 3, 4, L, device=dev),
                            e, e, torch.zeros(1, 1, 3, 4, L, device=dev), e)

  call()
  with pytest.raises(RuntimeError, match="contiguous"):
    call(contiguous=False)
  # the reference prints and returns zero-filled outputs above MAX_DISPARITY (TRWP.cpp:269-273)
  with pytest.raises(RuntimeError, match="n_disp"):
    call(L=300)


def test_runs_are_deterministic_and_batch_items_independent(gpu):
  from mplayers_amd import synthetic
  cfg = synthetic.make_config("C4", seed=3, scale=0.25, mode="TRWP")
  unary, ctx, ew = cfg["unary"].numpy(), cfg["context"].numpy(), cfg["edge_weights"].numpy()
  a = gpu.gpu_forward("TRWP", unary, ctx, ew, 4, 3, 0.5)
  b = gpu.gpu_forward("TRWP", unary, ctx, ew, 4, 3, 0.5)
  for k in ("msg", "cost_final", "msg_min_index", "msg_norm_index"):
    assert np.array_equal(a[k], b[k]), k
  one = gpu.gpu_forward("TRWP", unary[2:3], ctx, ew[:, 2:3], 4, 3, 0.5)
  assert np.array_equal(a["cost_final"][2:3], one["cost_final"])
  assert np.array_equal(a["msg_min_index"][:, :, 2:3], one["msg_min_index"])
  # twelve identical samples give identical per-sample results (pytorch/test_multi_batch.py:61-63)
  rep = np.repeat(unary[:1], 12, axis=0)
  rew = np.repeat(ew[:, :1], 12, axis=1)
  r = gpu.gpu_forward("ISGMR", rep, ctx, rew, 4, 2, 1.0)
  assert all(np.array_equal(r["cost_final"][0], r["cost_final"][i]) for i in range(12))


@pytest.mark.parametrize("mode", ["TRWP", "ISGMR"])
def test_large_config_properties_at_full_size(gpu, mode):
  """1500 x 2000, 192 labels, 8 directions, training mode: too large for the CPU oracle, so the
  full-size run is checked through what must hold at any size."""
  import torch
  from mplayers_amd import lib_stereo, synthetic
  cfg = synthetic.make_config("C5", seed=0, mode=mode)
  B, H, W, L, n_dir = cfg["B"], cfg["H"], cfg["W"], cfg["L"], cfg["n_dir"]
  n_iter, rho = cfg["n_iter"], cfg["rho"]  # the 5 iterations the configuration states
  dev = "cuda:0"
  unary = cfg["unary"].to(dev)
  ctx = cfg["context"].to(dev)
  ew = cfg["edge_weights"].to(dev)
  msg = torch.zeros(n_dir, B, 1, H, W, L, device=dev)
  cost = torch.zeros(B, 1, H, W, L, device=dev)
  scratch = torch.zeros(B, 1, H, W, L, device=dev)
  imin = torch.zeros(n_iter, n_dir, B, 1, H, W, L, dtype=torch.uint8, device=dev)
  inorm = torch.zeros(n_iter, n_dir, B, 1, H, W, dtype=torch.uint8, device=dev)
  labels = torch.zeros(n_iter, B, 1, H, W, dtype=torch.uint8, device=dev)
  print("full size", mode, flush=True)
  if mode == "TRWP":
    lib_stereo.TRWP.forward(rho, n_iter, 0, unary, ctx, ew, msg, cost, imin, inorm, scratch, labels)
  else:
    msg_tmp = torch.zeros_like(msg)
    lib_stereo.ISGMR.forward(0, rho, n_iter, 0, unary, ctx, ew, msg, cost, imin, inorm, scratch,
                             msg_tmp, labels)
    del msg_tmp
  torch.cuda.synchronize()
  # every message vector is normalised: min exactly 0 (all-zero where the chain starts)
  assert float(msg.min()) == 0.0
  mins = msg.amin(dim=-1)
  assert float(mins.abs().max()) == 0.0
  assert float(msg[0, 0, 0, :, 0].abs().max()) == 0.0   # direction 0 starts at the left column
  assert float(msg[3, 0, 0, -1].abs().max()) == 0.0     # direction 3 starts at the bottom row
  assert float(msg[4, 0, 0, 0].abs().max()) == 0.0      # direction 4 (down-right) at the top row
  assert float(msg[0, 0, 0, :, 1:].amax(dim=-1).min()) > 0.0
  # cost_final = unary + sum_k msg_k, summed in direction order (bitwise)
  acc = unary.clone()
  for k in range(n_dir):
    acc += msg[k]
  assert torch.equal(acc, cost)
  del acc
  # labels = argmin of the cost (smallest label on ties); indices are valid labels
  assert torch.equal(cost.argmin(dim=-1).to(torch.uint8), labels[-1])
  assert int(imin.max()) < L and int(inorm.max()) < L
  # the argmin of a message's own argmin index row is where it is zero
  sel = msg[1, 0, 0].gather(-1, inorm[-1, 1, 0, 0].long().unsqueeze(-1)).squeeze(-1)
  assert float(sel[:, :-1].abs().max()) == 0.0
  # backward: gradient mass is conserved (every normalised message has zero net gradient)
  dcost = torch.randn(B, 1, H, W, L, device=dev, generator=torch.Generator(dev).manual_seed(1))
  dunary = torch.zeros_like(dcost)
  dmsg = msg  # reuse as scratch
  dedge = torch.zeros(n_dir, B, 1, H, W, device=dev)
  dctx = torch.zeros(L, device=dev)
  if mode == "TRWP":
    lib_stereo.TRWP.backward(rho, ctx, ew, dcost, imin, inorm, dunary, dctx, dedge, dmsg, scratch)
  else:
    lib_stereo.ISGMR.backward(0, rho, ctx, ew, dcost, imin, inorm, dunary, dctx, dedge, scratch,
                              scratch, dmsg)
  torch.cuda.synchronize()
  total = float(dcost.double().sum())
  assert abs(float(dunary.double().sum()) - total) <= 1e-6 * float(dcost.double().abs().sum())
  assert float(dctx[0]) == 0.0 and bool(torch.isfinite(dctx).all()) and bool(torch.isfinite(dedge).all())
  # edge-weight gradients exist only where a pixel has a front neighbour
  assert float(dedge[0, 0, 0, :, 0].abs().max()) == 0.0
  assert float(dedge[0, 0, 0, :, 1:].abs().max()) > 0.0


def _check_rows_inference(gpu, oracle, mode, unary, ctx, ew, n_iter, rho, what):
  """The forward pass without argmin labels (the kernels compiled for inference), the two horizontal
  directions on device tensors: first rows, a middle row and the last rows against the oracle."""
  import torch
  from mplayers_amd import lib_stereo
  B, _, H, W, L = unary.shape
  n_dir = 2
  dev = unary.device
  msg = torch.zeros(n_dir, B, 1, H, W, L, device=dev)
  cost = torch.zeros(B, 1, H, W, L, device=dev)
  scratch = torch.zeros(B, 1, H, W, L, device=dev)
  empty = torch.empty(0, dtype=torch.uint8)
  print(what, mode, "inference", flush=True)
  if mode == "TRWP":
    lib_stereo.TRWP.forward(rho, n_iter, 0, unary, ctx, ew, msg, cost, empty, empty, scratch, empty)
  else:
    msg_tmp = torch.zeros_like(msg)
    lib_stereo.ISGMR.forward(0, rho, n_iter, 0, unary, ctx, ew, msg, cost, empty, empty, scratch,
                             msg_tmp, empty)
    del msg_tmp
  torch.cuda.synchronize()
  rows = [0, 1, H // 2, H - 2, H - 1]
  sub = lambda t, ax: t.index_select(ax, torch.tensor(rows, device=t.device)).cpu().numpy()
  ref = oracle.forward(mode, sub(unary, 2), ctx.cpu().numpy(), sub(ew, 3), n_dir, n_iter, rho,
                       training=False)
  gpu.assert_values_close(sub(msg, 3), ref["msg"], what="msg rows", belief=ref["cost_final"])
  gpu.assert_values_close(sub(cost, 2), ref["cost_final"], what="cost rows")


def _check_rows(gpu, oracle, mode, unary, ctx, ew, dcost, n_iter, rho, what):
  """Runs forward and backward with the two horizontal directions on device tensors and checks the
  first rows, a middle row and the last rows against the oracle."""
  import torch
  from mplayers_amd import lib_stereo
  B, _, H, W, L = unary.shape
  n_dir = 2
  dev = unary.device
  msg = torch.zeros(n_dir, B, 1, H, W, L, device=dev)
  cost = torch.zeros(B, 1, H, W, L, device=dev)
  scratch = torch.zeros(B, 1, H, W, L, device=dev)
  imin = torch.zeros(n_iter, n_dir, B, 1, H, W, L, dtype=torch.uint8, device=dev)
  inorm = torch.zeros(n_iter, n_dir, B, 1, H, W, dtype=torch.uint8, device=dev)
  empty = torch.empty(0, dtype=torch.uint8)
  dunary = torch.zeros_like(cost)
  dedge = torch.zeros(n_dir, B, 1, H, W, device=dev)
  dctx = torch.zeros(L, device=dev)
  dmsg = torch.empty_like(msg)
  print(what, mode, flush=True)
  if mode == "TRWP":
    lib_stereo.TRWP.forward(rho, n_iter, 0, unary, ctx, ew, msg, cost, imin, inorm, scratch, empty)
    lib_stereo.TRWP.backward(rho, ctx, ew, dcost, imin, inorm, dunary, dctx, dedge, dmsg, scratch)
  else:
    msg_tmp = torch.zeros_like(msg)
    lib_stereo.ISGMR.forward(0, rho, n_iter, 0, unary, ctx, ew, msg, cost, imin, inorm, scratch,
                             msg_tmp, empty)
    lib_stereo.ISGMR.backward(0, rho, ctx, ew, dcost, imin, inorm, dunary, dctx, dedge, scratch,
                              scratch, dmsg)
    del msg_tmp
  torch.cuda.synchronize()
  rows = [0, 1, H // 2, H - 2, H - 1]
  sub = lambda t, ax: t.index_select(ax, torch.tensor(rows, device=t.device)).cpu().numpy()
  un, en, dn = sub(unary, 2), sub(ew, 3), sub(dcost, 2)
  ref = oracle.forward(mode, un, ctx.cpu().numpy(), en, n_dir, n_iter, rho, want_gaps=True)
  belief = ref["cost_final"]
  tol = 1e-5 * max(1.0, float(np.abs(belief).max()))
  gpu.assert_values_close(sub(msg, 3), ref["msg"], what="msg rows", belief=belief)
  gpu.assert_values_close(sub(cost, 2), ref["cost_final"], what="cost rows")
  gpu.assert_indices_match_off_ties(sub(imin, 4), ref["msg_min_index"], ref["gap_min"], 4 * tol,
                                    "min index rows")
  gpu.assert_indices_match_off_ties(sub(inorm, 4), ref["msg_norm_index"], ref["gap_norm"], 4 * tol,
                                    "norm index rows")
  # backward on the GPU's own indices of those rows
  du, _, de = oracle.backward(mode, ctx.cpu().numpy().astype(np.float64), en.astype(np.float64),
                              dn.astype(np.float64), sub(imin, 4), sub(inorm, 4), rho)
  assert np.abs(sub(dunary, 2) - du).max() <= 1e-4 * max(1.0, np.abs(du).max())
  assert np.abs(sub(dedge, 3) - de).max() <= 1e-4 * max(1.0, np.abs(de).max())


@pytest.mark.parametrize("mode", ["TRWP", "ISGMR"])
def test_full_size_rows_match_oracle(gpu, oracle, mode):
  """With only the two horizontal directions the rows of an image do not interact, so the oracle
  can check a few rows of a full-size (1500 x 2000 x 192) run exactly as it checks small images:
  first rows, a middle row and the last rows, whose byte offsets lie beyond 2^31."""
  from mplayers_amd import synthetic
  cfg = synthetic.make_config("C5", seed=0, mode=mode)
  dev = "cuda:0"
  unary, ctx, ew = cfg["unary"].to(dev), cfg["context"].to(dev), cfg["edge_weights"][:2].contiguous().to(dev)
  _check_rows(gpu, oracle, mode, unary, ctx, ew, synthetic.upstream_grad(cfg).to(dev), cfg["n_iter"],
              cfg["rho"], "full-size rows")
  _check_rows_inference(gpu, oracle, mode, unary, ctx, ew, cfg["n_iter"], cfg["rho"], "full-size rows")


@pytest.mark.parametrize("mode", ["TRWP", "ISGMR"])
def test_rows_of_the_largest_image_match_oracle(gpu, oracle, mode):
  """2684 x 2000 pixels of 200 labels: 4 294 400 000 bytes per plane, 567 232 below the largest
  image the library accepts, so the vector offsets of the last rows use all 32 bits."""
  import torch
  H, W, L = 2684, 2000, 200
  dev = "cuda:0"
  g = torch.Generator(device=dev)
  g.manual_seed(11)
  unary = torch.rand(1, 1, H, W, L, device=dev, generator=g)
  ew = 0.2 + torch.rand(2, 1, 1, H, W, device=dev, generator=g)
  dcost = torch.randn(1, 1, H, W, L, device=dev, generator=g)
  ctx = (0.25 * torch.clamp(torch.arange(L, dtype=torch.float32), max=3.0)).to(dev)
  rho = 0.5 if mode == "TRWP" else 1.0
  _check_rows(gpu, oracle, mode, unary, ctx, ew, dcost, 1, rho, "largest image rows")
  del dcost
  # the kernels compiled for inference, and with them a negative weight in the last row
  _check_rows_inference(gpu, oracle, mode, unary, ctx, ew, 1, rho, "largest image rows")
  ew[:, :, :, H - 1, 700] = -0.3
  _check_rows_inference(gpu, oracle, mode, unary, ctx, ew, 1, rho, "largest image rows, a negative weight")


@pytest.mark.parametrize("mode", ["TRWP", "ISGMR"])
def test_rows_of_a_batch_beyond_2_31_elements(gpu, oracle, mode):
  """Four 1500 x 2000 images of 192 labels: 2.304 G elements per plane, more than a 32-bit element
  index holds (the scans address per batch item, the element-wise kernels over the whole plane)."""
  import torch
  B, H, W, L = 4, 1500, 2000, 192
  dev = "cuda:0"
  g = torch.Generator(device=dev)
  g.manual_seed(12)
  unary = torch.rand(B, 1, H, W, L, device=dev, generator=g)
  ew = 0.2 + torch.rand(2, B, 1, H, W, device=dev, generator=g)
  dcost = torch.randn(B, 1, H, W, L, device=dev, generator=g)
  ctx = (0.25 * torch.clamp(torch.arange(L, dtype=torch.float32), max=4.0)).to(dev)
  rho = 0.5 if mode == "TRWP" else 1.0
  _check_rows(gpu, oracle, mode, unary, ctx, ew, dcost, 1, rho, "batch of four rows")
  torch.cuda.empty_cache()


@pytest.mark.parametrize("mode,pair", [("TRWP", 2), ("ISGMR", 2), ("TRWP", 4), ("ISGMR", 6)])
def test_full_size_chains_match_oracle(gpu, oracle, mode, pair):
  """Zero edge weights make a direction's messages vanish, so with every direction but one
  opposite pair switched off the chains of that pair do not interact: single columns (pair 2/3)
  or diagonals (4/5, 6/7) of a full-size run are then two-direction problems on a 1 x n image,
  which the oracle checks exactly, forward and backward."""
  import torch
  from mplayers_amd import lib_stereo, synthetic
  cfg = synthetic.make_config("C5", seed=0, mode=mode)
  B, H, W, L = cfg["B"], cfg["H"], cfg["W"], cfg["L"]
  n_dir = 4 if pair < 4 else 8
  n_iter, rho = cfg["n_iter"], cfg["rho"]
  dev = "cuda:0"
  unary = cfg["unary"].to(dev)
  ctx = cfg["context"].to(dev)
  ew = cfg["edge_weights"][:n_dir].clone()
  for d in range(n_dir):
    if d not in (pair, pair + 1):
      ew[d] = 0
  ew = ew.contiguous().to(dev)
  dcost = synthetic.upstream_grad(cfg).to(dev)
  msg = torch.zeros(n_dir, B, 1, H, W, L, device=dev)
  cost = torch.zeros(B, 1, H, W, L, device=dev)
  scratch = torch.zeros(B, 1, H, W, L, device=dev)
  imin = torch.zeros(n_iter, n_dir, B, 1, H, W, L, dtype=torch.uint8, device=dev)
  inorm = torch.zeros(n_iter, n_dir, B, 1, H, W, dtype=torch.uint8, device=dev)
  empty = torch.empty(0, dtype=torch.uint8)
  dunary = torch.zeros_like(cost)
  dedge = torch.zeros(n_dir, B, 1, H, W, device=dev)
  dctx = torch.zeros(L, device=dev)
  dmsg = torch.empty_like(msg)
  print("full-size chains", mode, pair, flush=True)
  if mode == "TRWP":
    lib_stereo.TRWP.forward(rho, n_iter, 0, unary, ctx, ew, msg, cost, imin, inorm, scratch, empty)
    lib_stereo.TRWP.backward(rho, ctx, ew, dcost, imin, inorm, dunary, dctx, dedge, dmsg, scratch)
  else:
    msg_tmp = torch.zeros_like(msg)
    lib_stereo.ISGMR.forward(0, rho, n_iter, 0, unary, ctx, ew, msg, cost, imin, inorm, scratch,
                             msg_tmp, empty)
    lib_stereo.ISGMR.backward(0, rho, ctx, ew, dcost, imin, inorm, dunary, dctx, dedge, scratch,
                              scratch, dmsg)
    del msg_tmp
  # the same run through the kernels compiled for inference (no argmin labels)
  msg_inf, cost_inf = torch.zeros_like(msg), torch.zeros_like(cost)
  if mode == "TRWP":
    lib_stereo.TRWP.forward(rho, n_iter, 0, unary, ctx, ew, msg_inf, cost_inf, empty, empty, scratch, empty)
  else:
    msg_tmp = torch.zeros_like(msg)
    lib_stereo.ISGMR.forward(0, rho, n_iter, 0, unary, ctx, ew, msg_inf, cost_inf, empty, empty, scratch,
                             msg_tmp, empty)
    del msg_tmp
  torch.cuda.synchronize()
  # messages of the switched-off directions vanish
  for d in range(n_dir):
    if d not in (pair, pair + 1):
      assert float(msg[d].abs().max()) == 0.0
  hs, ws = oracle.dir_step(pair)
  if pair == 2:
    starts = [(0, 0), (0, 1), (0, W // 2), (0, W - 1)]
  elif pair == 4:   # down-right: chains start on the top row and on the left column
    starts = [(0, 0), (0, 700), (0, W - 3), (H - 5, 0), (600, 0)]
  else:             # pair 6, down-left: top row and right column
    starts = [(0, W - 1), (0, 900), (0, 2), (H - 4, W - 1), (400, W - 1)]
  ctx_np = ctx.cpu().numpy()
  for (h0, w0) in starts:
    n = 1 + min((H - 1 - h0) // hs if hs else 10**9,
                ((W - 1 - w0) // ws if ws > 0 else (w0 // -ws if ws < 0 else 10**9)))
    hh = torch.arange(n, device=dev) * hs + h0
    ww = torch.arange(n, device=dev) * ws + w0
    pick = lambda t: t[..., hh, ww, :] if t.shape[-1] == L else t[..., hh, ww]
    un = unary[:, :, hh, ww, :].cpu().numpy()[:, :, None]                 # (1, 1, 1, n, L)
    en = ew[[pair, pair + 1]][:, :, :, hh, ww].cpu().numpy()[:, :, :, None]  # (2, 1, 1, 1, n)
    dn = dcost[:, :, hh, ww, :].cpu().numpy()[:, :, None]
    ref = oracle.forward(mode, un, ctx_np, en, 2, n_iter, rho, want_gaps=True)
    belief = ref["cost_final"]
    tol = 1e-5 * max(1.0, float(np.abs(belief).max()))
    got_msg = msg[[pair, pair + 1]][:, :, :, hh, ww, :].cpu().numpy()[:, :, :, None]
    gpu.assert_values_close(got_msg, ref["msg"], what="chain msg", belief=belief)
    gpu.assert_values_close(cost[:, :, hh, ww, :].cpu().numpy()[:, :, None], ref["cost_final"],
                            what="chain cost")
    gpu.assert_values_close(msg_inf[[pair, pair + 1]][:, :, :, hh, ww, :].cpu().numpy()[:, :, :, None],
                            ref["msg"], what="chain msg, inference", belief=belief)
    gpu.assert_values_close(cost_inf[:, :, hh, ww, :].cpu().numpy()[:, :, None], ref["cost_final"],
                            what="chain cost, inference")
    gi = imin[:, [pair, pair + 1]][:, :, :, :, hh, ww, :].cpu().numpy()[:, :, :, :, None]
    gn = inorm[:, [pair, pair + 1]][:, :, :, :, hh, ww].cpu().numpy()[:, :, :, :, None]
    gpu.assert_indices_match_off_ties(gi, ref["msg_min_index"], ref["gap_min"], 4 * tol, "min idx")
    gpu.assert_indices_match_off_ties(gn, ref["msg_norm_index"], ref["gap_norm"], 4 * tol, "norm idx")
    du, _, de = oracle.backward(mode, ctx_np.astype(np.float64), en.astype(np.float64),
                                dn.astype(np.float64), gi, gn, rho)
    got_du = dunary[:, :, hh, ww, :].cpu().numpy()[:, :, None]
    got_de = dedge[[pair, pair + 1]][:, :, :, hh, ww].cpu().numpy()[:, :, :, None]
    assert np.abs(got_du - du).max() <= 1e-4 * max(1.0, np.abs(du).max()), (h0, w0)
    assert np.abs(got_de - de).max() <= 1e-4 * max(1.0, np.abs(de).max()), (h0, w0)


@pytest.mark.parametrize("mode", ["TRWP", "ISGMR"])
def test_module_at_full_size_equals_the_operators(gpu, mode):
  """The large configuration as stated (1500 x 2000, 192 labels, 8 directions, 5 iterations)
  through MPModule, the path a user of the layer takes: uninitialised buffers and messages that
  start at zero by declaration.  Its cost and its gradients must be the ones the operators give
  on zero-filled tensors under the reference's contract, bit for bit (dcontext, summed with float
  atomics, to 1e-4), and the size-independent properties must hold."""
  import torch
  from mplayers_amd import MPModule, lib_stereo, synthetic
  cfg = synthetic.make_config("C5", seed=0, mode=mode)
  B, H, W, L, n_dir, n_iter, rho = (cfg[k] for k in ("B", "H", "W", "L", "n_dir", "n_iter", "rho"))
  dev = "cuda:0"
  args = argparse.Namespace(mpnet_mrf_mode=mode, mpnet_max_iter=n_iter, mpnet_n_dirs=n_dir,
                            n_classes=L, mpnet_term_weight=1.0, mpnet_smoothness_train="",
                            mpnet_diag_value=0, enable_symmetric=True)
  mod = MPModule(args, enable_saving_label=True).cuda().train()
  table = torch.nn.Parameter(cfg["context"].to(dev))
  mod.set_label_context(table, np.arange(1, L), [0])
  print("module at full size", mode, flush=True)
  u = cfg["unary"].to(dev).permute(0, 1, 4, 2, 3).contiguous().requires_grad_(True)  # (B, cv, L, H, W)
  e = cfg["edge_weights"][:, :, 0].permute(1, 0, 2, 3).contiguous().to(dev).requires_grad_(True)
  g = synthetic.upstream_grad(cfg).to(dev)
  cost, _, labels, _, _ = mod(u, e)
  cost.backward(g.permute(0, 1, 4, 2, 3))
  torch.cuda.synchronize()
  cost_m = cost.detach().permute(0, 1, 3, 4, 2).contiguous()
  du_m = u.grad.permute(0, 1, 3, 4, 2).contiguous()
  de_m = e.grad.permute(1, 0, 2, 3).unsqueeze(2).contiguous()
  dc_m = table.grad.clone()
  assert torch.equal(cost_m.argmin(dim=-1).to(torch.uint8), labels[-1])
  total = float(g.double().sum())
  assert abs(float(du_m.double().sum()) - total) <= 1e-6 * float(g.double().abs().sum())
  assert float(dc_m[0]) == 0.0 and bool(torch.isfinite(dc_m).all())
  del cost, u, mod
  torch.cuda.empty_cache()
  # the operators on zero-filled tensors, flags = 0
  unary = cfg["unary"].to(dev)
  ctx = cfg["context"].to(dev)
  ew = cfg["edge_weights"].to(dev)
  msg = torch.zeros(n_dir, B, 1, H, W, L, device=dev)
  cost = torch.zeros(B, 1, H, W, L, device=dev)
  scratch = torch.zeros(B, 1, H, W, L, device=dev)
  imin = torch.zeros(n_iter, n_dir, B, 1, H, W, L, dtype=torch.uint8, device=dev)
  inorm = torch.zeros(n_iter, n_dir, B, 1, H, W, dtype=torch.uint8, device=dev)
  empty = torch.empty(0, dtype=torch.uint8)
  dunary = torch.zeros_like(cost)
  dedge = torch.zeros(n_dir, B, 1, H, W, device=dev)
  dctx = torch.zeros(L, device=dev)
  if mode == "TRWP":
    lib_stereo.TRWP.forward(rho, n_iter, 0, unary, ctx, ew, msg, cost, imin, inorm, scratch, empty)
    lib_stereo.TRWP.backward(rho, ctx, ew, g, imin, inorm, dunary, dctx, dedge, msg, scratch)
  else:
    msg_tmp = torch.zeros_like(msg)
    lib_stereo.ISGMR.forward(0, rho, n_iter, 0, unary, ctx, ew, msg, cost, imin, inorm, scratch,
                             msg_tmp, empty)
    lib_stereo.ISGMR.backward(0, rho, ctx, ew, g, imin, inorm, dunary, dctx, dedge, msg, scratch,
                              msg_tmp)
  torch.cuda.synchronize()
  assert torch.equal(cost_m, cost)
  assert torch.equal(du_m, dunary)
  assert torch.equal(de_m, dedge)
  assert float((dc_m - dctx).abs().max()) <= 1e-4 * max(1.0, float(dctx.abs().max()))
  print("peak memory %.1f GB" % (torch.cuda.max_memory_allocated() / 1e9), flush=True)
  assert torch.cuda.max_memory_allocated() < 288e9


@pytest.mark.parametrize("mode,L", [("TRWP", 21), ("ISGMR", 12), ("TRWP", 70)])
def test_module_with_two_cost_volumes(gpu, oracle, mode, L):
  """cv = 2: two cost volumes per batch item share the pairwise table and run as independent
  problems (batch * cv of them, MP_module.py:36).  The module passes edge weights per batch item,
  so they are left out here (the reference's (B, n_dir, H, W) maps do not cover a second volume);
  the autograd Function takes them per volume."""
  import torch
  from mplayers_amd import MPModule
  from mplayers_amd.MP_module import ISGMRFunction, TRWPFunction
  rng = np.random.default_rng(L + 5)
  B, cv, H, W, n_dir, n_iter = 2, 2, 6, 7, 4 if mode == "TRWP" else 8, 2
  rho = 0.5 if mode == "TRWP" else 1.0
  args = argparse.Namespace(mpnet_mrf_mode=mode, mpnet_max_iter=n_iter, mpnet_n_dirs=n_dir,
                            n_classes=L, mpnet_term_weight=1.0, mpnet_smoothness_train="",
                            mpnet_diag_value=0, enable_symmetric=True)
  mod = MPModule(args, enable_saving_label=True).cuda().train()
  if L == 21:
    ctx = np.triu(rng.random((L, L)), 1).astype(np.float32)
    loc, diag = np.triu_indices(L, k=1), [range(L), range(L)]
  else:
    ctx = np.concatenate([[0], rng.random(L - 1)]).astype(np.float32)
    loc, diag = np.arange(1, L), [0]
  table = torch.nn.Parameter(torch.from_numpy(ctx).cuda())
  mod.set_label_context(table, loc, diag)
  unary = rng.standard_normal((B, cv, L, H, W)).astype(np.float32)
  dcost = rng.standard_normal((B, cv, L, H, W)).astype(np.float32)
  u = torch.from_numpy(unary).cuda().requires_grad_(True)
  cost, _, labels, _, _ = mod(u, None)
  cost.backward(torch.from_numpy(dcost).cuda())
  torch.cuda.synchronize()
  un = np.ascontiguousarray(unary.transpose(0, 1, 3, 4, 2))
  dn = np.ascontiguousarray(dcost.transpose(0, 1, 3, 4, 2))
  ref = oracle.forward(mode, un, ctx, None, n_dir, n_iter, rho, saving_label=True, want_gaps=True)
  got = cost.detach().cpu().numpy().transpose(0, 1, 3, 4, 2)
  gpu.assert_values_close(got, ref["cost_final"], what="cost_final")
  tol = 2e-5 * max(1.0, float(np.abs(ref["cost_final"]).max()))
  gpu.assert_labels_match_off_ties(labels.cpu().numpy(), ref["label_all"], ref["gap_label"], tol)
  du, dc, _ = oracle.backward(mode, ctx, None, dn, ref["msg_min_index"], ref["msg_norm_index"], rho)
  gu = u.grad.cpu().numpy().transpose(0, 1, 3, 4, 2)
  assert np.abs(gu - du).max() <= 1e-4 * max(1.0, float(np.abs(du).max()))
  assert np.abs(table.grad.cpu().numpy() - dc).max() <= 1e-4 * max(1.0, float(np.abs(dc).max()))
  # the second volume is an independent problem: alone it gives the same numbers
  u1 = torch.from_numpy(unary[:, 1:2]).cuda()
  cost1 = mod(u1, None)[0]
  assert torch.equal(cost1, cost[:, 1:2])
  # the Function with edge weights per volume
  ew = (0.1 + 0.9 * rng.random((n_dir, B, cv, H, W))).astype(np.float32)
  fn = TRWPFunction if mode == "TRWP" else ISGMRFunction
  mod.args.training = True
  uf = torch.from_numpy(un).cuda().requires_grad_(True)
  ef = torch.from_numpy(ew).cuda().requires_grad_(True)
  cf, _ = fn.apply(uf, table.detach(), ef, mod.args)
  cf.backward(torch.from_numpy(dn).cuda())
  torch.cuda.synchronize()
  ref = oracle.forward(mode, un, ctx, ew, n_dir, n_iter, rho)
  gpu.assert_values_close(cf.detach().cpu().numpy(), ref["cost_final"], what="cost_final (ew)")
  du, _, de = oracle.backward(mode, ctx, ew, dn, ref["msg_min_index"], ref["msg_norm_index"], rho)
  assert np.abs(uf.grad.cpu().numpy() - du).max() <= 1e-4 * max(1.0, float(np.abs(du).max()))
  assert np.abs(ef.grad.cpu().numpy() - de).max() <= 1e-4 * max(1.0, float(np.abs(de).max()))
