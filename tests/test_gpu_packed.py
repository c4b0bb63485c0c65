"""Scans with several chains per wavefront (at most 32 labels).  By default only launches with a
2-D table and more than 1024 chains (2048 with 21 labels), or with a 1-D table of at most 8 / 16
labels and more than 6144 / 10000 chains, take them, so the small cases are run with the policy forced (option value 2)
and one case is large enough to take them on its own; every result is checked against the oracle
exactly like the one-chain-per-wavefront kernels."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture
def always_packed(gpu):
  from mplayers_amd import _lib
  _lib.set_option(_lib.OPT_PACKED_SCANS, 2)
  yield
  _lib.set_option(_lib.OPT_PACKED_SCANS, 1)


def small_case(seed):
  rng = np.random.default_rng(7000 + seed)
  mode = ["TRWP", "ISGMR"][seed % 2]
  n_dir = int(rng.choice([2, 4, 8, 16]))
  B = int(rng.integers(1, 5))
  H = int(rng.integers(1, 12))
  W = int(rng.integers(1, 12))
  L = int(rng.choice([1, 2, 3, 5, 8, 10, 11, 16, 17, 21, 22, 31, 32]))
  n_iter = int(rng.integers(1, 4))
  k = np.arange(L, dtype=np.float32)
  if L == 21:
    ctx = np.triu(rng.random((L, L)), 1).astype(np.float32)
  elif seed % 3 == 0:
    ctx = (0.3 * np.minimum(k, 2)).astype(np.float32)
  else:
    ctx = rng.random(L).astype(np.float32)
  unary = rng.random((B, 1, H, W, L)).astype(np.float32)
  ew = (0.1 + rng.random((n_dir, B, 1, H, W))).astype(np.float32)
  if seed % 5 == 2:
    ew[rng.random(ew.shape) < 0.2] *= -1
  dcost = rng.standard_normal((B, 1, H, W, L)).astype(np.float32)
  return mode, n_dir, n_iter, unary, ctx, ew, dcost


def check_against_oracle(gpu, oracle, mode, n_dir, n_iter, unary, ctx, ew, dcost, msg_init=None):
  rho = 0.5 if mode == "TRWP" else 1.0
  ref = oracle.forward(mode, unary, ctx, ew, n_dir, n_iter, rho, saving_label=True, want_gaps=True,
                       msg_init=msg_init)
  got = gpu.gpu_forward(mode, unary, ctx, ew, n_dir, n_iter, rho, saving_label=True,
                        msg_init=msg_init)
  belief = ref["cost_final"]
  tol = 1e-5 * max(1.0, float(np.abs(belief).max()))
  gpu.assert_values_close(got["msg"], ref["msg"], what="msg", belief=belief)
  gpu.assert_values_close(got["cost_final"], ref["cost_final"], what="cost")
  gpu.assert_indices_match_off_ties(got["msg_min_index"], ref["msg_min_index"], ref["gap_min"],
                                    4 * tol, "min index")
  gpu.assert_indices_match_off_ties(got["msg_norm_index"], ref["msg_norm_index"], ref["gap_norm"],
                                    4 * tol, "norm index")
  inf = gpu.gpu_forward(mode, unary, ctx, ew, n_dir, n_iter, rho, training=False, msg_init=msg_init)
  gpu.assert_values_close(inf["cost_final"], ref["cost_final"], what="inference cost")
  du, dc, de = oracle.backward(mode, ctx.astype(np.float64), ew.astype(np.float64),
                               dcost.astype(np.float64), ref["msg_min_index"],
                               ref["msg_norm_index"], rho)
  gu, gc, ge = gpu.gpu_backward(mode, ctx, ew, dcost, ref["msg_min_index"], ref["msg_norm_index"],
                                rho, garbage_scratch=True)
  for name, g, r in (("dunary", gu, du), ("dcontext", gc, dc), ("dedge", ge, de)):
    err = np.abs(g.astype(np.float64) - r).max()
    assert err <= 1e-4 * max(1.0, np.abs(r).max()), (name, err)
  return got


@pytest.mark.parametrize("seed", range(36))
def test_small_cases_forced_packed(gpu, oracle, always_packed, seed):
  mode, n_dir, n_iter, unary, ctx, ew, dcost = small_case(seed)
  print("case", seed, mode, n_dir, n_iter, unary.shape, flush=True)
  msg_init = None
  if seed % 4 == 1:  # non-zero initial messages
    rng = np.random.default_rng(seed)
    msg_init = rng.random((n_dir,) + unary.shape).astype(np.float32)
    msg_init -= msg_init.min(axis=-1, keepdims=True)
  check_against_oracle(gpu, oracle, mode, n_dir, n_iter, unary, ctx, ew, dcost, msg_init)


@pytest.mark.parametrize("mode", ["TRWP", "ISGMR"])
def test_segmentation_batch_takes_packed_scans(gpu, oracle, mode):
  """8 x 65 x 64 pixels, 21 labels: more than 2048 chains per launch, so the default policy packs;
  the same call with packing switched off must agree with it to the tolerance."""
  from mplayers_amd import _lib
  rng = np.random.default_rng(11)
  B, H, W, L, n_iter = 8, 65, 64, 21, 2
  n_dir = 8 if mode == "ISGMR" else 4
  if mode == "TRWP":
    B, W = 32, 64   # one direction per launch: 32 x 65 rows = 2080 chains
  ctx = np.triu(rng.random((L, L)), 1).astype(np.float32)
  unary = rng.standard_normal((B, 1, H, W, L)).astype(np.float32)
  ew = (0.1 + 0.9 * rng.random((n_dir, B, 1, H, W))).astype(np.float32)
  dcost = rng.standard_normal((B, 1, H, W, L)).astype(np.float32)
  got = check_against_oracle(gpu, oracle, mode, n_dir, n_iter, unary, ctx, ew, dcost)
  _lib.set_option(_lib.OPT_PACKED_SCANS, 0)
  try:
    rho = 0.5 if mode == "TRWP" else 1.0
    plain = gpu.gpu_forward(mode, unary, ctx, ew, n_dir, n_iter, rho, saving_label=True)
  finally:
    _lib.set_option(_lib.OPT_PACKED_SCANS, 1)
  gpu.assert_values_close(got["cost_final"], plain["cost_final"], what="packed vs plain")
  assert (got["msg_min_index"] != plain["msg_min_index"]).mean() < 1e-3


def test_band_table_of_many_chains_stays_unpacked(gpu, oracle):
  """A 1-D table is nearly always a band, whose step the one-chain-per-wavefront scans do in a few
  taps while the packed step scans every front label: 16 labels and 1344 chains per launch are not
  packed by default.  The two kinds of reverse scan sum dedge_weights in different orders, which
  shows which one ran."""
  from mplayers_amd import _lib
  rng = np.random.default_rng(5)
  B, H, W, L, n_dir, n_iter = 2, 160, 176, 16, 4, 1
  ctx = (0.3 * np.minimum(np.arange(L), 3)).astype(np.float32)
  unary = rng.random((B, 1, H, W, L)).astype(np.float32)
  ew = (0.1 + 0.9 * rng.random((n_dir, B, 1, H, W))).astype(np.float32)
  dcost = rng.standard_normal((B, 1, H, W, L)).astype(np.float32)
  fwd = gpu.gpu_forward("ISGMR", unary, ctx, ew, n_dir, n_iter, 1.0)
  run = lambda flags: gpu.gpu_backward("ISGMR", ctx, ew, dcost, fwd["msg_min_index"],
                                       fwd["msg_norm_index"], 1.0, flags=flags)
  default, off, always = run(0), run(_lib.F_PACKED_OFF), run(_lib.F_PACKED_ALWAYS)
  assert np.array_equal(default[2], off[2])
  assert not np.array_equal(default[2], always[2])
  assert np.abs(default[2] - always[2]).max() <= 1e-4 * np.abs(default[2]).max()
  assert np.array_equal(default[0], off[0])


def test_few_labels_and_many_chains_pack_by_default(gpu, oracle):
  """8 labels, 6528 chains in the launch: with at most 8 labels a 1-D table costs the packed step
  little more than a band would, and 8 chains share a wavefront."""
  from mplayers_amd import _lib
  rng = np.random.default_rng(9)
  B, H, W, L, n_dir, n_iter = 16, 200, 4, 8, 4, 2
  ctx = (0.4 * np.minimum(np.arange(L), 2)).astype(np.float32)
  unary = rng.random((B, 1, H, W, L)).astype(np.float32)
  ew = (0.1 + 0.9 * rng.random((n_dir, B, 1, H, W))).astype(np.float32)
  dcost = rng.standard_normal((B, 1, H, W, L)).astype(np.float32)
  check_against_oracle(gpu, oracle, "ISGMR", n_dir, n_iter, unary, ctx, ew, dcost)
  fwd = gpu.gpu_forward("ISGMR", unary, ctx, ew, n_dir, n_iter, 1.0)
  run = lambda flags: gpu.gpu_backward("ISGMR", ctx, ew, dcost, fwd["msg_min_index"],
                                       fwd["msg_norm_index"], 1.0, flags=flags)
  default, always = run(0), run(_lib.F_PACKED_ALWAYS)
  assert np.array_equal(default[2], always[2])  # (8-term sums: both kinds of scan give these bits)
  assert np.array_equal(default[0], always[0])


def test_set_option_rejects_unknown(gpu):
  from mplayers_amd import _lib
  with pytest.raises(RuntimeError):
    _lib.set_option(99, 1)
  with pytest.raises(RuntimeError):
    _lib.set_option(_lib.OPT_PACKED_SCANS, 3)
