"""Pins the CPU oracle (oracle/) before anything is compared with it.

What pins what:
  * reference-held fixtures: tests/golden/refcpu_*.npz come from the reference's own compiled CPU
    forward (TRWP.cpp / ISGMR.cpp); the restated CPU loop nest must reproduce them bit for bit,
    and the GPU-semantics restatement must agree with them wherever both semantics coincide
    (unit edge weights, one symmetric context shared by all directions).
  * mathematics: on a chain the min-sum recursion is exact dynamic programming, so one iteration
    with rho = 1 must give brute-force min-marginals (edge weights and a 2-D context included);
    one ISGMR iteration with the SGM flag is textbook semi-global matching; the backward pass must
    agree with central finite differences of the forward pass; flips and transposes of the input
    must permute the directions.
"""
import glob
import itertools
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
# (the fixtures of the SGM flag pin the CPU forward alone, tests/test_cpu_forward.py: that flag
# rewrites the unary tensor on the reference's CPU path, which neither the GPU semantics nor the
# oracle's restatement of the CPU loop nest do)
REFCPU_FIXTURES = [p for p in sorted(glob.glob(os.path.join(GOLDEN, "refcpu_*.npz")))
                   if "refcpu_sgm" not in p]


def _toeplitz_is_shared(context):
  n_dir, L, _ = context.shape
  if not all(np.array_equal(context[0], context[d]) for d in range(n_dir)):
    return False
  ii = np.abs(np.arange(L)[:, None] - np.arange(L)[None, :])
  return np.array_equal(context[0], context[0][0][ii])


@pytest.mark.parametrize("path", REFCPU_FIXTURES,
                         ids=lambda p: os.path.basename(p)[7:-4])
def test_refcpu_port_matches_reference_fixture(oracle, path):
  z = np.load(path)
  mode, rho, n_dir, n_iter = str(z["mode"]), float(z["rho"]), int(z["n_dir"]), int(z["n_iter"])
  out = oracle.refcpu_forward(mode, z["unary"], z["context"], n_dir, n_iter, rho,
                              context_per_dir=True)
  assert np.array_equal(out["msg"], z["msg"])
  assert np.array_equal(out["cost_final"], z["cost_final"])


@pytest.mark.parametrize("path", REFCPU_FIXTURES,
                         ids=lambda p: os.path.basename(p)[7:-4])
def test_gpu_semantics_agree_with_reference_fixture(oracle, path):
  z = np.load(path)
  if not _toeplitz_is_shared(z["context"]):
    pytest.skip("per-direction context: only the CPU semantics define this case")
  mode, rho, n_dir, n_iter = str(z["mode"]), float(z["rho"]), int(z["n_dir"]), int(z["n_iter"])
  L = z["unary"].shape[-1]
  ctx = z["context"][0] if L == 21 else z["context"][0, 0]
  out = oracle.forward(mode, z["unary"], ctx, None, n_dir, n_iter, rho, saving_label=True)
  scale = max(1.0, float(np.abs(z["cost_final"]).max()))
  assert np.abs(out["msg"] - z["msg"]).max() <= 1e-5 * scale
  assert np.abs(out["cost_final"] - z["cost_final"]).max() <= 1e-5 * scale
  if "int" in path and mode == "ISGMR":  # exact arithmetic: values and labels must be identical
    assert np.array_equal(out["msg"], z["msg"])
    assert np.array_equal(out["label_all"], z["label_all"])


def test_reference_build_matches_port_when_present(oracle):
  from oracle import ref_cpu
  if not ref_cpu.available():
    pytest.skip("oracle/_ref not built (reference tree absent)")
  rng = np.random.default_rng(5)
  for mode, rho in (("TRWP", 0.5), ("ISGMR", 1.0)):
    unary = rng.random((1, 2, 5, 6, 7)).astype(np.float32)
    ctx = rng.random((8, 7, 7)).astype(np.float32)
    r = ref_cpu.forward(mode, unary, ctx, 8, 2, rho)
    p = oracle.refcpu_forward(mode, unary, ctx, 8, 2, rho, context_per_dir=True)
    assert np.array_equal(r["msg"], p["msg"]) and np.array_equal(r["cost_final"], p["cost_final"])


# ----------------------------------------------------------------------------------------------
def _chain_min_marginals(unary, pair):
  """unary (n, L); pair[e] (L, L) energy table of edge (e, e+1) indexed [l_e, l_{e+1}]."""
  n, L = unary.shape
  mm = np.full((n, L), np.inf)
  for lab in itertools.product(range(L), repeat=n):
    e = sum(unary[p, lab[p]] for p in range(n)) + sum(pair[p][lab[p], lab[p + 1]] for p in range(n - 1))
    for p in range(n):
      mm[p, lab[p]] = min(mm[p, lab[p]], e)
  return mm


@pytest.mark.parametrize("mode", ["TRWP", "ISGMR"])
@pytest.mark.parametrize("vertical", [False, True])
@pytest.mark.parametrize("ctx2d", [False, True])
def test_chain_is_exact_dynamic_programming(oracle, mode, vertical, ctx2d):
  rng = np.random.default_rng(3)
  n, L = 5, 3
  u = rng.random((n, L))
  if ctx2d:
    table = np.triu(rng.random((L, L)), 1)  # only i <= j is ever read
    sym = table + table.T
    ctx = table
  else:
    c = np.concatenate([[0.0], rng.random(L - 1)])
    sym = c[np.abs(np.arange(L)[:, None] - np.arange(L)[None, :])]
    ctx = c
  we = 0.5 + rng.random(n - 1)
  mm = _chain_min_marginals(u, [we[e] * sym for e in range(n - 1)])
  if vertical:  # W = 1: directions 0/1 have no edge at all, 2/3 carry the chain
    unary = u.reshape(1, 1, n, 1, L)
    ew = np.ones((4, 1, 1, n, 1))
    ew[2, 0, 0, 1:, 0] = we  # weight lives at the receiving pixel; its front is the pixel above
    ew[3, 0, 0, :-1, 0] = we
    n_dir = 4
  else:
    unary = u.reshape(1, 1, 1, n, L)
    ew = np.ones((2, 1, 1, 1, n))
    ew[0, 0, 0, 0, 1:] = we
    ew[1, 0, 0, 0, :-1] = we
    n_dir = 2
  out = oracle.forward(mode, unary, ctx, ew, n_dir, 1, 1.0, ctx2d=ctx2d)
  cf = out["cost_final"].reshape(n, L)
  assert np.abs((cf - cf.min(1, keepdims=True)) - (mm - mm.min(1, keepdims=True))).max() < 1e-12
  # every written message is normalised to min 0; chain-start pixels are never written
  msg = out["msg"].reshape(n_dir, n, L)
  assert np.all(msg.min(-1) == 0)
  first = 2 if vertical else 0
  assert np.all(msg[first, 0] == 0) and np.all(msg[first + 1, -1] == 0)
  assert np.any(msg[first, 1] != 0)


def _textbook_sgm(unary, c, n_dir):
  """Hirschmueller's path recursion L_r(p,d) = C(p,d) + min_d'(L_r(p-r,d') + V(d,d')) - min_k L_r(p-r,k),
  summed over directions.  unary (H, W, L); V(d,d') = c[|d-d'|]."""
  H, W, L = unary.shape
  steps = [(0, 1), (0, -1), (1, 0), (-1, 0), (1, 1), (-1, -1), (1, -1), (-1, 1)][:n_dir]
  V = c[np.abs(np.arange(L)[:, None] - np.arange(L)[None, :])]
  S = np.zeros_like(unary)
  for hs, ws in steps:
    Lr = np.zeros_like(unary)
    hh = range(H) if hs >= 0 else range(H - 1, -1, -1)
    ww = range(W) if ws >= 0 else range(W - 1, -1, -1)
    for h in hh:
      for w in ww:
        fh, fw = h - hs, w - ws
        if 0 <= fh < H and 0 <= fw < W:
          prev = Lr[fh, fw]
          Lr[h, w] = unary[h, w] + (prev[None, :] + V).min(1) - prev.min()
        else:
          Lr[h, w] = unary[h, w]
    S += Lr
  return S


@pytest.mark.parametrize("n_dir", [4, 8])
def test_one_sgm_iteration_is_textbook_sgm(oracle, n_dir):
  rng = np.random.default_rng(11)
  H, W, L = 6, 7, 5
  unary = rng.random((1, 1, H, W, L))
  c = np.minimum(np.arange(L), 2) * 0.3
  out = oracle.forward("SGM", unary, c, None, n_dir, 1, 1.0, enable_sgm=True)
  S = _textbook_sgm(unary[0, 0], c, n_dir)
  cf = out["cost_final"][0, 0]
  assert np.abs((cf - cf.min(-1, keepdims=True)) - (S - S.min(-1, keepdims=True))).max() < 1e-12


# ----------------------------------------------------------------------------------------------
def _rand_problem(rng, n_dir, B, H, W, L, ctx2d):
  unary = rng.random((B, 1, H, W, L))
  if ctx2d:
    ctx = np.triu(rng.random((L, L)), 1)
  else:
    ctx = np.concatenate([[0.0], rng.random(L - 1)])
  ew = 0.1 + 0.9 * rng.random((n_dir, B, 1, H, W))
  return unary, ctx, ew


@pytest.mark.parametrize("mode,rho", [("TRWP", 0.5), ("ISGMR", 1.0), ("SGM", 1.0)])
@pytest.mark.parametrize("n_dir,ctx2d", [(4, False), (8, True), (16, False)])
def test_backward_matches_finite_differences(oracle, mode, rho, n_dir, ctx2d):
  rng = np.random.default_rng(7)
  B, H, W, L = 1, 4, 5, 3
  n_iter = 1 if mode == "SGM" else 2
  sgm = mode == "SGM"
  unary, ctx, ew = _rand_problem(rng, n_dir, B, H, W, L, ctx2d)
  dcost = rng.standard_normal(unary.shape)

  def loss(u, c, e):
    o = oracle.forward(mode, u, c, e, n_dir, n_iter, rho, training=False, enable_sgm=sgm, ctx2d=ctx2d)
    return float((o["cost_final"] * dcost).sum())

  out = oracle.forward(mode, unary, ctx, ew, n_dir, n_iter, rho, enable_sgm=sgm, ctx2d=ctx2d)
  du, dc, de = oracle.backward(mode, ctx, ew, dcost, out["msg_min_index"], out["msg_norm_index"],
                               rho, enable_sgm=sgm, ctx2d=ctx2d)
  eps = 1e-6

  def fd(arr, idx, which):
    args = [unary, ctx, ew]
    hi, lo = arr.copy(), arr.copy()
    hi[idx] += eps
    lo[idx] -= eps
    a_hi, a_lo = list(args), list(args)
    a_hi[which], a_lo[which] = hi, lo
    return (loss(*a_hi) - loss(*a_lo)) / (2 * eps)

  for idx in [tuple(rng.integers(0, s) for s in unary.shape) for _ in range(25)]:
    assert abs(fd(unary, idx, 0) - du[idx]) < 1e-6
  for idx in [tuple(rng.integers(0, s) for s in ew.shape) for _ in range(25)]:
    assert abs(fd(ew, idx, 2) - de[idx]) < 1e-6
  if ctx2d:
    for i in range(L):
      for j in range(i + 1, L):
        assert abs(fd(ctx, (i, j), 1) - dc[i, j]) < 1e-6
    # the diagonal and the lower triangle are never written (TRWP_backward.cu:111-112)
    assert np.all(np.tril(dc) == 0)
  else:
    for k in range(1, L):
      assert abs(fd(ctx, (k,), 1) - dc[k]) < 1e-6
    assert dc[0] == 0
  # every normalised message carries zero net gradient mass
  factor = n_dir if sgm else 1
  assert abs(du.sum() - factor * dcost.sum()) < 1e-9


@pytest.mark.parametrize("n_dir,ctx2d", [(4, False), (8, True), (16, True), (8, False)])
def test_hard_soft_backward_collects_the_same_label_terms(oracle, n_dir, ctx2d):
  """The hard backward of the reference's TRWP_hard_soft build drops the `current_d != front_d`
  guard (TRWP_hard_soft/TRWP_backward.cu:110 against TRWP/TRWP_backward.cu:111-112): entry 0 of a
  1-D table / the diagonal of a 2-D one then receive their true gradient, which finite differences
  of the forward pass pin; every other output is what the guarded backward gives."""
  rng = np.random.default_rng(11)
  B, H, W, L, n_iter, rho = 1, 4, 5, 3, 2, 0.5
  unary, ctx, ew = _rand_problem(rng, n_dir, B, H, W, L, ctx2d)
  if ctx2d:
    ctx = ctx + np.diag(0.2 + rng.random(L))  # a diagonal that matters
  else:
    ctx[0] = 0.3
  dcost = rng.standard_normal(unary.shape)

  def loss(c):
    o = oracle.forward("TRWP", unary, c, ew, n_dir, n_iter, rho, training=False, ctx2d=ctx2d)
    return float((o["cost_final"] * dcost).sum())

  out = oracle.forward("TRWP", unary, ctx, ew, n_dir, n_iter, rho, ctx2d=ctx2d)
  args = ("TRWP", ctx, ew, dcost, out["msg_min_index"], out["msg_norm_index"], rho)
  du0, dc0, de0 = oracle.backward(*args, ctx2d=ctx2d)
  du1, dc1, de1 = oracle.backward(*args, ctx2d=ctx2d, same_label=True)
  assert np.array_equal(du0, du1) and np.array_equal(de0, de1)
  eps = 1e-6
  entries = [(i, j) for i in range(L) for j in range(i, L)] if ctx2d else [(k,) for k in range(L)]
  seen_nonzero = False
  for idx in entries:
    hi, lo = ctx.copy(), ctx.copy()
    hi[idx] += eps
    lo[idx] -= eps
    g = (loss(hi) - loss(lo)) / (2 * eps)
    assert abs(g - dc1[idx]) < 1e-6, idx
    same = (idx[0] == idx[1]) if ctx2d else (idx[0] == 0)
    if same:
      assert dc0[idx] == 0
      seen_nonzero |= abs(dc1[idx]) > 1e-3
    else:
      assert dc0[idx] == dc1[idx]
  assert seen_nonzero  # the guarded operator really loses something
  if ctx2d:
    assert np.all(np.tril(dc1, -1) == 0)


@pytest.mark.parametrize("n_dir", [4, 8])
def test_isgmr_flip_and_transpose_permute_directions(oracle, n_dir):
  rng = np.random.default_rng(21)
  B, H, W, L = 1, 5, 7, 4
  unary, ctx, ew = _rand_problem(rng, n_dir, B, H, W, L, False)
  base = oracle.forward("ISGMR", unary, ctx, ew, n_dir, 2, 1.0)
  # horizontal flip: 0<->1, 4<->6, 5<->7 (steps (h, w) -> (h, -w))
  perm = [1, 0, 2, 3, 6, 7, 4, 5][:n_dir]
  out = oracle.forward("ISGMR", unary[:, :, :, ::-1], ctx, ew[perm][:, :, :, :, ::-1], n_dir, 2, 1.0)
  assert np.array_equal(out["cost_final"][:, :, :, ::-1], base["cost_final"]) or \
      np.abs(out["cost_final"][:, :, :, ::-1] - base["cost_final"]).max() < 1e-12
  assert np.abs(out["msg"][perm][:, :, :, :, ::-1] - base["msg"]).max() < 1e-12
  # transpose: (h, w) -> (w, h): 0<->2, 1<->3, 4->4, 5->5, 6<->7
  perm = [2, 3, 0, 1, 4, 5, 7, 6][:n_dir]
  out = oracle.forward("ISGMR", unary.transpose(0, 1, 3, 2, 4), ctx,
                       ew[perm].transpose(0, 1, 2, 4, 3), n_dir, 2, 1.0)
  assert np.abs(out["cost_final"].transpose(0, 1, 3, 2, 4) - base["cost_final"]).max() < 1e-12
  assert np.array_equal(out["msg_min_index"][:, perm].transpose(0, 1, 2, 3, 5, 4, 6),
                        base["msg_min_index"])


def test_geometry_visits_every_edge_once(oracle):
  """Each pixel whose front neighbour is inside the image is visited exactly once per direction
  by the restated chain enumeration (common.cpp:78-87 + the kernels' start formulas)."""
  import ctypes
  lib = oracle.lib()
  for H, W in [(5, 7), (8, 3), (1, 6), (6, 1), (9, 9)]:
    for d in range(16):
      hs, ws = oracle.dir_step(d)
      seen = np.zeros((H, W), dtype=int)
      for tree in range(oracle.n_trees(d, H, W)):
        h0, w0, nr = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        lib.mpo_tree_start(d, hs, ws, H, W, tree, ctypes.byref(h0), ctypes.byref(w0), ctypes.byref(nr))
        for i in range(nr.value + 1):
          h, w = h0.value + i * hs, w0.value + i * ws
          if 0 <= h < H and 0 <= w < W and 0 <= h - hs < H and 0 <= w - ws < W:
            seen[h, w] += 1
      hh, ww = np.mgrid[0:H, 0:W]
      expect = ((hh - hs >= 0) & (hh - hs < H) & (ww - ws >= 0) & (ww - ws < W)).astype(int)
      assert np.array_equal(seen, expect), (H, W, d)


def test_tie_rules(oracle):
  """All-equal inputs: min index = largest front label, norm index = largest label, label = 0."""
  L = 6
  unary = np.zeros((1, 1, 3, 4, L), dtype=np.float32)
  ctx = np.zeros(L, dtype=np.float32)
  out = oracle.forward("ISGMR", unary, ctx, None, 4, 1, 1.0, saving_label=True)
  hh, ww = np.mgrid[0:3, 0:4]
  valid0 = ww - 1 >= 0
  assert np.all(out["msg_min_index"][0, 0, 0, 0][valid0] == L - 1)
  assert np.all(out["msg_norm_index"][0, 0, 0, 0][valid0] == L - 1)
  assert np.all(out["msg_min_index"][0, 0, 0, 0][~valid0] == 0)  # never written
  assert np.all(out["label_all"] == 0)


def test_batch_items_are_independent(oracle):
  rng = np.random.default_rng(2)
  unary, ctx, ew = _rand_problem(rng, 4, 3, 4, 5, 4, False)
  for mode, rho in (("TRWP", 0.5), ("ISGMR", 1.0)):
    full = oracle.forward(mode, unary, ctx, ew, 4, 2, rho)
    one = oracle.forward(mode, unary[1:2], ctx, ew[:, 1:2], 4, 2, rho)
    assert np.array_equal(full["cost_final"][1:2], one["cost_final"])
    assert np.array_equal(full["msg_min_index"][:, :, 1:2], one["msg_min_index"])
