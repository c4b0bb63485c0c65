"""Wide truncated-linear contexts c[k] = s * min(k, tau) (the stereo settings of the reference's
energy-minimisation runs: tau = L - 1 for 96 and 32 labels, MPLayers/run_all.sh:11-15) take the
label-scan step instead of the dense one.  Values against the oracle within the parity tolerance,
indices off ties; on integer-valued problems everything is exact, ties included."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

CASES = [
    # mode, L, tau, slope, n_dir, B, H, W, n_iter
    ("TRWP", 96, 95, 10.0, 4, 1, 9, 11, 3),      # KITTI setting: untruncated, integer slope
    ("ISGMR", 96, 95, 0.37, 8, 2, 7, 9, 2),
    ("TRWP", 32, 31, 0.25, 8, 1, 8, 8, 2),       # one label per lane
    ("ISGMR", 32, 31, 1.0, 16, 1, 9, 9, 2),
    ("TRWP", 60, 59, 0.4, 4, 1, 10, 7, 2),       # partial last lane
    ("TRWP", 192, 191, 0.3, 8, 1, 6, 8, 2),      # three labels per lane
    ("ISGMR", 192, 40, 0.3, 4, 1, 6, 8, 3),      # truncation inside the label range, beyond the band path
    ("TRWP", 256, 255, 0.05, 4, 1, 5, 6, 2),     # four labels per lane
    ("ISGMR", 200, 120, 0.11, 4, 2, 5, 6, 2),
    ("TRWP", 129, 9, 0.7, 4, 1, 7, 7, 2),        # moderate band (K = 10): also the scan step
    ("ISGMR", 17, 16, 0.5, 4, 1, 9, 9, 2),
    ("TRWP", 3, 2, 0.5, 4, 1, 5, 5, 2),
]


@pytest.mark.parametrize("mode,L,tau,slope,n_dir,B,H,W,n_iter", CASES)
@pytest.mark.parametrize("train", [True, False])
def test_linear_context_matches_oracle(gpu, oracle, mode, L, tau, slope, n_dir, B, H, W, n_iter, train):
  rng = np.random.default_rng(L * 31 + tau)
  rho = 0.5 if mode == "TRWP" else 1.0
  k = np.arange(L, dtype=np.float32)
  ctx = (np.float32(slope) * np.minimum(k, tau)).astype(np.float32)
  unary = (rng.random((B, 1, H, W, L)) * slope * 6).astype(np.float32)
  ew = (0.1 + rng.random((n_dir, B, 1, H, W))).astype(np.float32)
  if L == 60:
    ew[rng.random(ew.shape) < 0.15] *= -1        # negative weights: dense fallback inside the kernel
  ref = oracle.forward(mode, unary, ctx, ew, n_dir, n_iter, rho, saving_label=True, want_gaps=True)
  got = gpu.gpu_forward(mode, unary, ctx, ew, n_dir, n_iter, rho, training=train, saving_label=True)
  belief = ref["cost_final"]
  tol = 1e-5 * max(1.0, float(np.abs(belief).max()))
  gpu.assert_values_close(got["msg"], ref["msg"], what="msg", belief=belief)
  gpu.assert_values_close(got["cost_final"], ref["cost_final"], what="cost")
  assert (np.abs(got["msg"].min(axis=-1)) == 0).all()          # every message vector has minimum 0
  if train:
    gpu.assert_indices_match_off_ties(got["msg_min_index"], ref["msg_min_index"], ref["gap_min"],
                                      4 * tol, "min index")
    gpu.assert_indices_match_off_ties(got["msg_norm_index"], ref["msg_norm_index"], ref["gap_norm"],
                                      4 * tol, "norm index")


@pytest.mark.parametrize("mode,L,tau,n_dir", [("TRWP", 96, 95, 4), ("ISGMR", 32, 31, 8),
                                              ("TRWP", 192, 100, 8), ("ISGMR", 60, 59, 16)])
def test_integer_problem_is_exact_with_ties(gpu, oracle, mode, L, tau, n_dir):
  """Integer costs, integer slope, unit weights (an energy-minimisation instance): all arithmetic
  is exact and ties are everywhere, so messages, costs, labels and both index tensors must equal
  the oracle's bit for bit -- the scan step reproduces the largest-label tie rule."""
  rng = np.random.default_rng(L + n_dir)
  B, H, W, n_iter = 1, 8, 9, 3
  rho = 1.0                                        # rho = 0.5 would halve odd integers: keep it exact
  k = np.arange(L, dtype=np.float32)
  ctx = (3.0 * np.minimum(k, tau)).astype(np.float32)
  unary = rng.integers(0, 40, size=(B, 1, H, W, L)).astype(np.float32)
  ew = np.ones((n_dir, B, 1, H, W), dtype=np.float32)
  ref = oracle.forward(mode, unary, ctx, ew, n_dir, n_iter, rho, saving_label=True)
  got = gpu.gpu_forward(mode, unary, ctx, ew, n_dir, n_iter, rho, saving_label=True)
  for name in ("msg", "cost_final", "msg_min_index", "msg_norm_index", "label_all"):
    assert np.array_equal(got[name], ref[name]), name
