"""Seeded random shapes against the oracle: label counts from 1 to 256 (every lanes-per-label
variant, partial lanes), 2 to 16 directions, degenerate grids, all context kinds, forward in
training mode followed by the backward pass."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def random_case(seed):
  rng = np.random.default_rng(1000 + seed)
  mode = ["TRWP", "ISGMR"][seed % 2]
  n_dir = int(rng.choice([2, 4, 8, 16]))
  B = int(rng.integers(1, 4))
  H = int(rng.integers(1, 11))
  W = int(rng.integers(1, 11))
  L = int(rng.choice([1, 2, 3, 5, 8, 16, 21, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 191, 192,
                      193, 200, 255, 256]))
  n_iter = int(rng.integers(1, 4))
  k = np.arange(L, dtype=np.float32)
  kind = int(rng.integers(0, 5))
  if L == 21:
    ctx = np.triu(rng.random((L, L)), 1).astype(np.float32)
  elif kind == 0:
    ctx = (0.3 * np.minimum(k, rng.integers(1, 6))).astype(np.float32)          # truncated linear
  elif kind == 1:
    ctx = (0.05 * np.minimum(k * k, rng.integers(1, 200))).astype(np.float32)   # truncated quadratic
  elif kind == 2:
    ctx = (k > 0).astype(np.float32) * np.float32(rng.random() + 0.1)           # Potts
  elif kind == 3:
    ctx = rng.random(L).astype(np.float32)                                      # arbitrary 1-D
  else:
    ctx = np.sort(rng.random(L)).astype(np.float32)                             # monotone, no tail
  unary = rng.random((B, 1, H, W, L)).astype(np.float32)
  ew = (0.1 + rng.random((n_dir, B, 1, H, W))).astype(np.float32)
  if seed % 7 == 3:
    ew[rng.random(ew.shape) < 0.2] *= -1   # negative weights take the dense fallback
  dcost = rng.standard_normal((B, 1, H, W, L)).astype(np.float32)
  return mode, n_dir, n_iter, unary, ctx, ew, dcost


@pytest.mark.parametrize("seed", range(40))
def test_random_case(gpu, oracle, seed):
  mode, n_dir, n_iter, unary, ctx, ew, dcost = random_case(seed)
  rho = 0.5 if mode == "TRWP" else 1.0
  print("case", seed, mode, n_dir, n_iter, unary.shape, flush=True)
  ref = oracle.forward(mode, unary, ctx, ew, n_dir, n_iter, rho, saving_label=True, want_gaps=True)
  got = gpu.gpu_forward(mode, unary, ctx, ew, n_dir, n_iter, rho, saving_label=True)
  belief = ref["cost_final"]
  tol = 1e-5 * max(1.0, float(np.abs(belief).max()))
  gpu.assert_values_close(got["msg"], ref["msg"], what="msg", belief=belief)
  gpu.assert_values_close(got["cost_final"], ref["cost_final"], what="cost")
  gpu.assert_indices_match_off_ties(got["msg_min_index"], ref["msg_min_index"], ref["gap_min"],
                                    4 * tol, "min index")
  gpu.assert_indices_match_off_ties(got["msg_norm_index"], ref["msg_norm_index"], ref["gap_norm"],
                                    4 * tol, "norm index")
  # backward on the oracle's indices, against the fp64 oracle
  du, dc, de = oracle.backward(mode, ctx.astype(np.float64), ew.astype(np.float64),
                               dcost.astype(np.float64), ref["msg_min_index"],
                               ref["msg_norm_index"], rho)
  gu, gc, ge = gpu.gpu_backward(mode, ctx, ew, dcost, ref["msg_min_index"], ref["msg_norm_index"],
                                rho, garbage_scratch=True)
  for name, g, r in (("dunary", gu, du), ("dcontext", gc, dc), ("dedge", ge, de)):
    err = np.abs(g.astype(np.float64) - r).max()
    assert err <= 1e-4 * max(1.0, np.abs(r).max()), (name, err)


@pytest.mark.parametrize("mode,rho", [("ISGMR", 0.7), ("ISGMR", 0.5), ("TRWP", 1.0), ("TRWP", 0.3)])
@pytest.mark.parametrize("L,n_dir", [(21, 8), (96, 4), (7, 16)])
def test_other_rho_values(gpu, oracle, mode, rho, L, n_dir):
  """The nn.Module fixes rho (0.5 for TRWP, 1 for ISGMR) but the operators take any value; ISGMR
  shares planes between opposite directions only at rho == 1, so other values take other paths."""
  rng = np.random.default_rng(int(rho * 100) + L)
  B, H, W, n_iter = 2, 6, 7, 3
  k = np.arange(L, dtype=np.float32)
  ctx = np.triu(rng.random((L, L)), 1).astype(np.float32) if L == 21 else \
      (0.3 * np.minimum(k, 3)).astype(np.float32)
  unary = rng.random((B, 1, H, W, L)).astype(np.float32)
  ew = (0.1 + rng.random((n_dir, B, 1, H, W))).astype(np.float32)
  dcost = rng.standard_normal((B, 1, H, W, L)).astype(np.float32)
  ref = oracle.forward(mode, unary, ctx, ew, n_dir, n_iter, rho, want_gaps=True)
  got = gpu.gpu_forward(mode, unary, ctx, ew, n_dir, n_iter, rho)
  belief = ref["cost_final"]
  tol = 1e-5 * max(1.0, float(np.abs(belief).max()))
  gpu.assert_values_close(got["msg"], ref["msg"], what="msg", belief=belief)
  gpu.assert_values_close(got["cost_final"], ref["cost_final"], what="cost")
  gpu.assert_indices_match_off_ties(got["msg_min_index"], ref["msg_min_index"], ref["gap_min"],
                                    4 * tol, "min index")
  du, dc, de = oracle.backward(mode, ctx.astype(np.float64), ew.astype(np.float64),
                               dcost.astype(np.float64), ref["msg_min_index"],
                               ref["msg_norm_index"], rho)
  gu, gc, ge = gpu.gpu_backward(mode, ctx, ew, dcost, ref["msg_min_index"], ref["msg_norm_index"],
                                rho, garbage_scratch=True)
  for name, g, r in (("dunary", gu, du), ("dcontext", gc, dc), ("dedge", ge, de)):
    err = np.abs(g.astype(np.float64) - r).max()
    assert err <= 1e-4 * max(1.0, np.abs(r).max()), (name, err)
