"""Pins of oracle/terms_oracle.py (stereo data cost, gradient cues, MRF energy) and the host-side
pieces of mplayers_amd.compute_terms / energy_min that need no GPU.

The reference's own build of this code needs OpenCV or imageLib, neither of which exists here, so
nothing below runs reference code: the matching cost is pinned by hand-computed values, by the
continuous definition of the Birchfield-Tomasi measure on even-valued images (where the integer
halves are exact), and by closed forms; the energy by explicit edge lists, edge counts and the
exact MAP labelling of a chain."""
import itertools

import numpy as np
import pytest

from oracle import mp_oracle, terms_oracle

STEPS = terms_oracle.STEPS


# ---------------------------------------------------------------------------------------------
# data cost
# ---------------------------------------------------------------------------------------------

def test_dsi_hand_computed_row():
  # one row, one band.  Half-way interpolants: im1 -> [10,15] [15,30] [30,40]; im2 -> [10,20] [20,35] [35,40]
  im1 = np.array([[10, 20, 40]], dtype=np.uint8)
  im2 = np.array([[10, 30, 40]], dtype=np.uint8)
  dsi = terms_oracle.compute_dsi(im1, im2, 3)
  assert dsi.shape == (1, 3, 3) and dsi.dtype == np.float32
  # x=0: d=0 -> 10 lies in [10,20]: 0; d=1,2 leave the image: min(255, 255)
  assert dsi[0, 0].tolist() == [0.0, 255.0, 255.0]
  # x=1: d=0 -> 20 in [20,35]: 0 (the plain difference would be 10); d=1 -> 20 in [10,20]: 0
  assert dsi[0, 1].tolist() == [0.0, 0.0, 255.0]
  # x=2: d=0 -> 40 in [35,40]: 0; d=1 -> 40 vs [20,35]: 5, but 30 lies in [30,40]: min(5, 0) = 0;
  #      d=2 -> 40 vs [10,20]: 20, and 10 vs [30,40]: 20
  assert dsi[0, 2].tolist() == [0.0, 0.0, 20.0]
  plain = terms_oracle.compute_dsi(im1, im2, 3, birchfield=0)
  assert plain[0, 1].tolist() == [10.0, 10.0, 255.0]
  assert plain[0, 2].tolist() == [0.0, 10.0, 30.0]


def continuous_bt(row1, row2, x, x2):
  """Definition of the sampling-insensitive measure: the smaller of the two one-sided distances
  min_t |I1(x) - I2lin(x2 + t)|, |t| <= 1/2, with I2lin the piecewise-linear interpolant (clamped
  at the row ends).  I2lin is continuous, so over the interval it takes every value between its
  smallest and largest sample of a dense grid of t (which holds the kinks t = 0, +-1/2): the
  distance of I1(x) to that range."""
  def one_sided(a, xa, b, xb):
    n = len(b)
    ts = np.linspace(-0.5, 0.5, 201)
    pos = np.clip(xb + ts, 0, n - 1)
    lo = np.floor(pos).astype(int)
    hi = np.minimum(lo + 1, n - 1)
    val = b[lo] * (1 - (pos - lo)) + b[hi] * (pos - lo)
    return max(0.0, a[xa] - val.max(), val.min() - a[xa])
  a, b = row1.astype(np.float64), row2.astype(np.float64)
  return min(one_sided(a, x, b, x2), one_sided(b, x2, a, x))


def test_dsi_equals_continuous_definition_on_even_images():
  rng = np.random.default_rng(1)
  H, W, L = 3, 12, 6
  im1 = (rng.integers(0, 128, size=(H, W, 3)) * 2).astype(np.uint8)
  im2 = (rng.integers(0, 128, size=(H, W, 3)) * 2).astype(np.uint8)
  dsi = terms_oracle.compute_dsi(im1, im2, L, trunc_diffs=10 ** 6)
  for y in range(H):
    for x in range(W):
      for d in range(L):
        if x - d < 0:
          assert dsi[y, x, d] == 3 * 255
        else:
          want = sum(continuous_bt(im1[y, :, c], im2[y, :, c], x, x - d) for c in range(3))
          assert dsi[y, x, d] == pytest.approx(want, abs=1e-9), (y, x, d)


def test_dsi_closed_forms():
  rng = np.random.default_rng(2)
  H, W, L = 5, 17, 7
  im = rng.integers(0, 256, size=(H, W, 3), dtype=np.uint8)
  # identical images: zero cost at zero disparity; Birchfield-Tomasi never exceeds the plain cost
  same = terms_oracle.compute_dsi(im, im, L)
  assert (same[:, :, 0] == 0).all()
  other = rng.integers(0, 256, size=(H, W, 3), dtype=np.uint8)
  bt = terms_oracle.compute_dsi(im, other, L)
  plain = terms_oracle.compute_dsi(im, other, L, birchfield=0)
  assert (bt <= plain).all() and (bt < plain).any()
  # right image = left image moved s pixels to the left: zero cost at d = s wherever x - s exists
  s = 3
  shifted = np.zeros_like(im)
  shifted[:, :W - s] = im[:, s:]
  moved = terms_oracle.compute_dsi(im, shifted, L, birchfield=0)
  assert (moved[:, s:, s] == 0).all()
  assert (moved[:, :s, s] == 3 * 255).all()           # match outside the image
  # constant images k apart: interpolation changes nothing -> colours * k, truncated, squared
  a = np.full((2, 6, 3), 100, dtype=np.uint8)
  b = np.full((2, 6, 3), 130, dtype=np.uint8)
  for bf in (0, 1):
    assert (terms_oracle.compute_dsi(a, b, 1, birchfield=bf)[:, :, 0] == 90).all()
    assert (terms_oracle.compute_dsi(a, b, 1, birchfield=bf, trunc_diffs=20)[:, :, 0] == 60).all()
    sq = terms_oracle.compute_dsi(a, b, 2, birchfield=bf, squared_diffs=1, trunc_diffs=50)
    assert (sq[:, :, 0] == 2500).all()                # 3 * 900 = 2700 truncated at 50^2
    assert (sq[:, 0, 1] == 2500).all()                # outside: min(3 * 255^2, 50^2)
  # only the first three bands count; one or two bands are summed as they are
  four = np.concatenate([im, rng.integers(0, 256, size=(H, W, 1), dtype=np.uint8)], axis=2)
  four2 = np.concatenate([other, rng.integers(0, 256, size=(H, W, 1), dtype=np.uint8)], axis=2)
  assert (terms_oracle.compute_dsi(four, four2, L) == bt).all()
  per_band = sum(terms_oracle.compute_dsi(im[:, :, c], other[:, :, c], L, trunc_diffs=10 ** 6)
                 for c in range(3))
  full = terms_oracle.compute_dsi(im, other, L, trunc_diffs=10 ** 6)
  inside = np.arange(W)[:, None] >= np.arange(L)[None, :]
  assert (full[:, inside] == per_band[:, inside]).all()
  # more labels than columns: everything beyond the image is the out-of-image cost
  wide = terms_oracle.compute_dsi(im[:, :4], other[:, :4], 9)
  assert (wide[:, :, 4:] == 765).all()


def test_cues_hand_computed_and_closed_forms():
  im = np.array([[[10, 10, 10], [13, 10, 10], [40, 40, 40]],
                 [[10, 14, 10], [13, 10, 10], [40, 40, 41]]], dtype=np.uint8)
  # threshold 2 -> squared sum below 3 * 2 * 2 = 12 earns the penalty
  h_cue, v_cue = terms_oracle.compute_cues(im, 2, 5)
  assert h_cue.shape == (2, 2) and v_cue.shape == (3, 1)
  assert h_cue.tolist() == [[5.0, 1.0], [1.0, 1.0]]   # 9 | 3*30^2 ; 9+16=25 | 27^2+30^2+31^2
  assert v_cue.tolist() == [[1.0], [5.0], [5.0]]      # 16 | 0 | 1  (column-major: one row per x)
  const = np.full((4, 5, 3), 77, dtype=np.uint8)
  h_cue, v_cue = terms_oracle.compute_cues(const, 1, 3)
  assert (h_cue == 3).all() and (v_cue == 3).all()
  h_cue, v_cue = terms_oracle.compute_cues(const, 0, 3)  # nothing is below a zero threshold
  assert (h_cue == 1).all() and (v_cue == 1).all()
  gray = np.array([[0, 3, 3], [0, 0, 9]], dtype=np.uint8)
  h_cue, v_cue = terms_oracle.compute_cues(gray, 3, 2)   # one band: below 9
  assert h_cue.tolist() == [[1.0, 2.0], [2.0, 1.0]]
  assert v_cue.tolist() == [[2.0], [1.0], [1.0]]


# ---------------------------------------------------------------------------------------------
# energy
# ---------------------------------------------------------------------------------------------

def energy_by_edge_list(unary, context, lab, edge, n_dir, ctx2d):
  B, H, W, L = unary.shape
  eu = sum(float(unary[b, h, w, lab[b, h, w]]) for b in range(B) for h in range(H) for w in range(W))
  ep = 0.0
  for d in range(0, n_dir, 2):
    hs, ws = STEPS[d]
    for b in range(B):
      for h in range(H):
        for w in range(W):
          qh, qw = h - hs, w - ws
          if 0 <= qh < H and 0 <= qw < W:
            xp, xq = int(lab[b, h, w]), int(lab[b, qh, qw])
            c = context[min(xp, xq)][max(xp, xq)] if ctx2d else context[abs(xp - xq)]
            ep += float(c) * (1.0 if edge is None else float(edge[d, b, h, w]))
  return eu, ep


@pytest.mark.parametrize("n_dir,L,ctx2d", [(4, 5, False), (8, 21, True), (16, 4, False), (2, 3, False)])
def test_energy_matches_explicit_edge_list(n_dir, L, ctx2d):
  rng = np.random.default_rng(n_dir + L)
  B, H, W = 2, 5, 6
  unary = rng.standard_normal((B, H, W, L)).astype(np.float32)
  context = (rng.random((L, L)) if ctx2d else rng.random(L)).astype(np.float32)
  edge = rng.random((n_dir, B, H, W)).astype(np.float32)
  labels = rng.integers(0, L, size=(3, B, H, W)).astype(np.uint8)
  for ew in (None, edge):
    got = terms_oracle.mrf_energy(unary, context, labels, ew, n_dir, ctx2d)
    for i in range(3):
      assert got[i] == pytest.approx(energy_by_edge_list(unary, context, labels[i], ew, n_dir, ctx2d),
                                     rel=1e-12, abs=1e-12)


def test_energy_counts_every_edge_once():
  H, W = 6, 7
  unary = np.zeros((1, H, W, 3), dtype=np.float32)
  ones = np.ones(3, dtype=np.float32)              # ctx == 1 everywhere: pairwise energy = #edges
  labels = np.zeros((1, 1, H, W), dtype=np.uint8)
  n4 = H * (W - 1) + (H - 1) * W
  n8 = n4 + 2 * (H - 1) * (W - 1)
  n16 = n8 + 2 * (H - 1) * (W - 2) + 2 * (H - 2) * (W - 1)
  for n_dir, want in ((2, H * (W - 1)), (4, n4), (8, n8), (16, n16)):
    assert terms_oracle.mrf_energy(unary, ones, labels, None, n_dir)[0, 1] == want
  # Potts: the number of label discontinuities of a half/half image
  potts = np.array([0, 1, 1], dtype=np.float32)
  labels[0, 0, :, 4:] = 2
  assert terms_oracle.mrf_energy(unary, potts, labels, None, 4)[0, 1] == H
  assert terms_oracle.mrf_energy(unary, potts, labels, None, 8)[0, 1] == H + 2 * (H - 1)


@pytest.mark.parametrize("vertical", [False, True])
def test_layer_labels_minimise_the_energy_on_a_chain(vertical):
  """On a chain one ISGMR iteration with rho = 1 gives exact min-marginals, so the argmin labelling
  is the MAP one: its energy must equal the minimum over all labellings.  This ties the energy's
  edge-weight placement (weight at the receiving pixel of the even direction) to the layers'."""
  rng = np.random.default_rng(5 + vertical)
  n, L = 6, 3
  shape = (1, 1, n, 1, L) if vertical else (1, 1, 1, n, L)
  n_dir = 4 if vertical else 2
  unary = rng.standard_normal(shape).astype(np.float32)
  context = np.array([0.0, 0.6, 1.1], dtype=np.float32)
  edge = (0.2 + rng.random((n_dir,) + shape[:4])).astype(np.float32)
  d = 2 if vertical else 0
  edge[d + 1] = 0                                  # the odd direction reads the weight of its own
  if vertical:                                     # plane at the other end point of every edge:
    edge[d + 1][:, :, :-1] = edge[d][:, :, 1:]     # make both planes describe the same edges
  else:
    edge[d + 1][:, :, :, :-1] = edge[d][:, :, :, 1:]
  out = mp_oracle.forward("ISGMR", unary, context, edge, n_dir, 1, 1.0, training=False,
                          saving_label=True)
  labels = out["label_all"].reshape(1, 1, *shape[2:4])
  u4 = unary.reshape(1, *shape[2:])
  e4 = edge.reshape(n_dir, 1, *shape[2:4])
  got = terms_oracle.mrf_energy(u4, context, labels, e4, n_dir).sum()
  best = min(terms_oracle.mrf_energy(u4, context, np.array(x, dtype=np.uint8).reshape(labels.shape),
                                     e4, n_dir).sum()
             for x in itertools.product(range(L), repeat=n))
  assert got == pytest.approx(best, abs=1e-5)


# ---------------------------------------------------------------------------------------------
# host code of the product that needs no GPU
# ---------------------------------------------------------------------------------------------

def test_smoothness_context_tables():
  from mplayers_amd.compute_terms import smoothness_context
  L = 6
  k = np.abs(np.arange(L)[:, None] - np.arange(L)[None, :]).astype(np.float64)
  assert (smoothness_context(L, "L", 3).numpy() == k).all()
  assert (smoothness_context(L, "Q", 3).numpy() == k * k).all()
  assert (smoothness_context(L, "TL", 3).numpy() == np.minimum(k, 3)).all()
  assert (smoothness_context(L, "TQ", 2).numpy() == np.minimum(k * k, 4)).all()
  np.testing.assert_allclose(smoothness_context(L, "Cauchy", 2).numpy(),
                             0.5 * 4 * np.log(1 + (k / 2) ** 2), rtol=1e-6)
  huber = smoothness_context(L, "Huber", 2).numpy()
  assert huber[0].tolist() == [0.0, 1.0, 4.0, 8.0, 12.0, 16.0]   # k^2 up to 2, then 4k - 4
  with pytest.raises(RuntimeError):
    smoothness_context(L, "nope", 2)


def test_unary_csv_and_synthetic_pair(tmp_path):
  from mplayers_amd import energy_min
  path = tmp_path / "toy_unary.csv"
  cost = np.arange(2 * 3 * 4, dtype=np.float32).reshape(2, 3, 4) / 4
  with open(path, "w") as f:
    f.write("2,3,4\n")
    for row in cost.reshape(-1, 4):
      f.write(",".join(repr(float(v)) for v in row) + "\n")
  h, w, n, t = energy_min.parse_unary_cost(str(path))
  assert (h, w, n) == (2, 3, 4) and (t.numpy() == cost).all()
  left, right, disp = energy_min.synthetic_stereo_pair(20, 30, 8)
  assert left.shape == right.shape == (20, 30, 3) and left.dtype == np.uint8
  ys, xs = np.nonzero(np.arange(30)[None, :] - disp >= 0)
  assert (left[ys, xs] == right[ys, xs - disp[ys, xs]]).all()
  # the true disparity has zero plain matching cost wherever the match is inside the image
  dsi = terms_oracle.compute_dsi(left, right, 8, birchfield=0)
  assert (dsi[ys, xs, disp[ys, xs]] == 0).all()


def test_denoising_terms_follow_the_label_context_builder(tmp_path):
  """house / penguin: unary from the CSV file, pairwise table from create_label_context with the
  truncation acting on the squared cost and the term weight applied (MPLayers/main.py:112-127)."""
  import argparse
  from mplayers_amd import energy_min
  from mplayers_amd.label_context import create_label_context
  n = 9
  ns = argparse.Namespace(n_classes=n, mpnet_smoothness_mode="TQ", mpnet_smoothness_train=None,
                          mpnet_smoothness_trunct_loc=-1, mpnet_smoothness_trunct_value=20,
                          mpnet_term_weight=5, enable_cuda=False)
  table, _, _ = create_label_context(ns, enable_seg=True, enable_symmetric=True)
  k = np.abs(np.arange(n)[:, None] - np.arange(n)[None, :])
  assert (table.detach().numpy() == 5 * np.minimum(k * k, 20)).all()
  ns.mpnet_smoothness_trunct_value = -1
  table, _, _ = create_label_context(ns, enable_seg=True, enable_symmetric=True)
  assert (table.detach().numpy() == 5 * k * k).all()
