"""Chains longer than two banks of prefetched pixels (HorizontalKernel / DiagonalKernel*,
TRWP_forward.cu:82-376): the forward scans then run trips of steps that are compiled for the inside
of a chain without negative edge weights, and a chain that has such a weight takes the general loop
from its first step.  Band tables of every compiled width, wide truncated-linear and dense tables,
1 to 4 labels per lane, with and without argmin labels, against the oracle; images in which some
chains have negative weights and their neighbours have none."""
import zlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _table(kind, L, rng):
  k = np.arange(L, dtype=np.float32)
  if kind == "tl2":
    return np.minimum(k, 2) * 0.25
  if kind == "tl3":
    return np.minimum(k, 3) * 0.3
  if kind == "tq4":
    return np.minimum(k * k, 10) * 0.1
  if kind == "tq9":
    return np.minimum(k * k, 70) * 0.02
  if kind == "tq20":
    return np.minimum(k * k, 390) * 0.004
  if kind == "tl40":
    return np.minimum(k, min(40, L - 2)) * 0.05
  if kind == "bump":  # a band whose entry 0 is not its smallest
    c = np.full(L, 0.5, dtype=np.float32)
    c[0], c[1], c[2] = 0.3, 0.1, 0.4
    return c
  if kind == "dense":
    return np.concatenate([[0], rng.random(L - 1)]).astype(np.float32)
  raise KeyError(kind)


def _inputs(kind, n_dir, B, H, W, L, negative):
  rng = np.random.default_rng(zlib.crc32(repr((kind, n_dir, B, H, W, L, negative)).encode()))
  unary = (rng.random((B, 1, H, W, L)) * 3).astype(np.float32)
  ctx = _table(kind, L, rng).astype(np.float32)
  ew = (0.1 + 0.9 * rng.random((n_dir, B, 1, H, W))).astype(np.float32)
  if negative:
    # a few pixels of rows 1 and 3 and of column 5: the chains through them take the general loop,
    # the other rows, columns and diagonals do not
    ew[:, :, :, 1, 7::11] = -0.3
    ew[:, :, :, 3, 20] = -0.6
    ew[:, :, :, 2::3, 5] = -0.2
  return unary, ctx, ew


CASES = [
    # mode, n_dir, B, H, W, L, kind
    ("TRWP", 4, 1, 5, 41, 96, "tl2"), ("TRWP", 8, 1, 6, 38, 96, "tl3"), ("TRWP", 4, 2, 5, 37, 90, "tq4"),
    ("TRWP", 4, 1, 5, 40, 128, "tq9"), ("TRWP", 4, 1, 4, 39, 192, "tl2"), ("TRWP", 8, 1, 5, 36, 192, "tq20"),
    ("TRWP", 4, 1, 4, 37, 200, "tq4"), ("TRWP", 4, 1, 4, 35, 256, "tq9"), ("TRWP", 4, 1, 5, 44, 96, "bump"),
    ("TRWP", 4, 1, 5, 40, 96, "tl40"), ("TRWP", 4, 1, 4, 36, 130, "dense"), ("TRWP", 4, 1, 6, 45, 16, "tl3"),
    ("TRWP", 8, 2, 5, 39, 24, "tq4"), ("TRWP", 4, 1, 5, 40, 48, "bump"), ("ISGMR", 4, 1, 5, 41, 96, "tl2"),
    ("ISGMR", 8, 1, 5, 38, 192, "tl3"), ("ISGMR", 4, 1, 4, 37, 256, "tq9"), ("ISGMR", 4, 1, 6, 43, 16, "tq4"),
    ("ISGMR", 4, 1, 5, 40, 100, "bump"), ("ISGMR", 16, 1, 6, 40, 96, "tl2"),
    # label counts that leave a lane with some of its labels only (a descriptor per access)
    ("TRWP", 4, 1, 5, 40, 97, "tl3"), ("ISGMR", 4, 1, 5, 38, 131, "tq4"), ("TRWP", 8, 1, 5, 37, 203, "tq9"),
]


@pytest.mark.parametrize("mode,n_dir,B,H,W,L,kind", CASES)
@pytest.mark.parametrize("training", [False, True])
@pytest.mark.parametrize("negative", [False, True])
def test_long_chains_match_oracle(gpu, oracle, mode, n_dir, B, H, W, L, kind, training, negative):
  unary, ctx, ew = _inputs(kind, n_dir, B, H, W, L, negative)
  rho = 0.5 if mode == "TRWP" else 1.0
  n_iter = 2
  print("case", mode, n_dir, B, H, W, L, kind, training, negative, flush=True)
  ref = oracle.forward(mode, unary, ctx, ew, n_dir, n_iter, rho, training=training, saving_label=True,
                       want_gaps=True)
  out = gpu.gpu_forward(mode, unary, ctx, ew, n_dir, n_iter, rho, training=training, saving_label=True)
  belief = ref["cost_final"]
  tol = 1e-5 * max(1.0, float(np.abs(belief).max()))
  gpu.assert_values_close(out["msg"], ref["msg"], what="msg", belief=belief)
  gpu.assert_values_close(out["cost_final"], ref["cost_final"], what="cost_final")
  if training:
    gpu.assert_indices_match_off_ties(out["msg_min_index"], ref["msg_min_index"], ref["gap_min"],
                                      4 * tol, "min index")
    gpu.assert_indices_match_off_ties(out["msg_norm_index"], ref["msg_norm_index"], ref["gap_norm"],
                                      4 * tol, "norm index")


@pytest.mark.parametrize("L,kind", [(96, "tl2"), (192, "tq4"), (16, "tl3")])
def test_a_negative_weight_changes_only_what_it_reaches(gpu, L, kind):
  """One horizontal direction pair, TRWP without argmin labels: the rows do not interact, so a
  negative weight in one row (that row's chain takes the general loop) must leave the messages of
  every other row exactly as they are without it."""
  n_dir, B, H, W = 2, 1, 6, 40
  unary, ctx, ew = _inputs(kind, n_dir, B, H, W, L, False)
  base = gpu.gpu_forward("TRWP", unary, ctx, ew, n_dir, 2, 0.5, training=False)
  ew2 = ew.copy()
  ew2[:, :, :, 2, 17] = -0.5
  other = gpu.gpu_forward("TRWP", unary, ctx, ew2, n_dir, 2, 0.5, training=False)
  rows = [0, 1, 3, 4, 5]
  assert np.array_equal(base["msg"][:, :, :, rows].view(np.uint8), other["msg"][:, :, :, rows].view(np.uint8))
  assert not np.array_equal(base["msg"][:, :, :, 2], other["msg"][:, :, :, 2])


def _random_long_case(seed):
  rng = np.random.default_rng(10000 + seed)
  mode = ["TRWP", "ISGMR"][rng.integers(2)]
  n_dir = [4, 8, 16][rng.integers(3)]
  B = int(rng.integers(1, 3))
  a, b = int(rng.integers(3, 9)), int(rng.integers(30, 72))
  H, W = (a, b) if rng.integers(2) else (b, a)
  if rng.integers(4) == 0:
    H, W = int(rng.integers(20, 40)), int(rng.integers(20, 40))
  L = [16, 24, 33, 48, 64, 65, 90, 96, 97, 128, 131, 160, 192, 200, 203, 255, 256][rng.integers(17)]
  kind = ["tl2", "tl3", "tq4", "tq9", "tq20", "tl40", "bump", "dense"][rng.integers(8)]
  if kind == "tq20" and L < 24:
    kind = "tq4"
  training = bool(rng.integers(2))
  # sixteen directions at rho = 0.5 amplify rounding several times per iteration: two iterations there
  n_iter = int(rng.integers(1, 3 if n_dir == 16 else 4))
  unary = (rng.random((B, 1, H, W, L)) * 3).astype(np.float32)
  ctx = _table(kind, L, rng).astype(np.float32)
  ew = (0.1 + 0.9 * rng.random((n_dir, B, 1, H, W))).astype(np.float32)
  negative = int(rng.integers(3))
  if negative == 1:
    ew[rng.random(ew.shape) < 0.01] = -0.4
  elif negative == 2:
    ew[:, :, :, int(rng.integers(H)), int(rng.integers(W))] = -0.7
  msg_init = None
  if rng.integers(3) == 0:
    msg_init = (rng.random((n_dir, B, 1, H, W, L)) * 0.5).astype(np.float32)
  return mode, n_dir, n_iter, unary, ctx, ew, training, msg_init, (B, H, W, L, kind, negative)


@pytest.mark.parametrize("seed", range(64))
def test_random_long_chains(gpu, oracle, seed):
  """Seeded random problems with chains of 20 to 70 pixels: every kind of table, 16 to 256 labels,
  4 / 8 / 16 directions, 1 to 3 iterations, negative weights nowhere, scattered or at one pixel,
  zero or given initial messages, with and without argmin labels."""
  mode, n_dir, n_iter, unary, ctx, ew, training, msg_init, what = _random_long_case(seed)
  rho = 0.5 if mode == "TRWP" else 1.0
  print("case", seed, mode, n_dir, n_iter, training, msg_init is not None, what, flush=True)
  kw = dict(training=training, saving_label=True, msg_init=msg_init)
  ref = oracle.forward(mode, unary, ctx, ew, n_dir, n_iter, rho, want_gaps=True, **kw)
  out = gpu.gpu_forward(mode, unary, ctx, ew, n_dir, n_iter, rho, **kw)
  belief = ref["cost_final"]
  tol = 1e-5 * max(1.0, float(np.abs(belief).max()))
  gpu.assert_values_close(out["msg"], ref["msg"], what="msg", belief=belief)
  gpu.assert_values_close(out["cost_final"], ref["cost_final"], what="cost_final")
  gpu.assert_labels_match_off_ties(out["label_all"], ref["label_all"], ref["gap_label"], 4 * tol)
  if training:
    gpu.assert_indices_match_off_ties(out["msg_min_index"], ref["msg_min_index"], ref["gap_min"],
                                      4 * tol, "min index")
    gpu.assert_indices_match_off_ties(out["msg_norm_index"], ref["msg_norm_index"], ref["gap_norm"],
                                      4 * tol, "norm index")
