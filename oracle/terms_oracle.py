"""CPU restatement (numpy) of the MRF terms around the message-passing layers.

TEST INFRASTRUCTURE ONLY: imported by tests/ (and nothing else); the product path is the HIP
kernels behind mpl_stereo_data_cost, mpl_gradient_cues and mpl_mrf_energy.

compute_dsi   follows computeDSI, MPLayers/aux/aux.cpp:5-98 (Birchfield-Tomasi matching cost of the
              Middlebury MRF benchmark code), vectorised over the image, one disparity at a time.
compute_cues  follows computeCues, MPLayers/aux/aux.cpp:100-170, with the output layout of
              MPLayers/aux/auxPy.cpp:83-99.
mrf_energy    follows calEnergy, tools/matlab/MRF/calEnergy.m:2-48, generalised to the layers'
              direction table (every undirected edge once, weight stored at the receiving pixel).

The reference cannot build these here (OpenCV / imageLib are absent), so the pins are
mathematical (tests/test_oracle_terms.py): hand-computed costs, the continuous definition of the
Birchfield-Tomasi measure sampled densely on even-valued images, shift and constant-image closed
forms, truncation and band handling; energies against explicit edge lists, edge counts per
connectivity, and the exact MAP labelling of a chain found by enumeration.
"""
import numpy as np

STEPS = ((0, 1), (0, -1), (1, 0), (-1, 0), (1, 1), (-1, -1), (1, -1), (-1, 1),
         (1, 2), (-1, -2), (2, 1), (-2, -1), (2, -1), (-2, 1), (1, -2), (-1, 2))


def _as_bands(im):
  im = np.asarray(im)
  assert im.dtype == np.uint8
  return im[:, :, None] if im.ndim == 2 else im


def _interval(im):
  """Per pixel and band: the range spanned by the value and its half-way interpolants to the left
  and right neighbour in the row (aux.cpp:58-66); integer halves truncate."""
  c = im.astype(np.int64)
  left = c.copy()
  left[:, 1:] = (c[:, 1:] + c[:, :-1]) // 2
  right = c.copy()
  right[:, :-1] = (c[:, :-1] + c[:, 1:]) // 2
  lo = np.minimum(c, np.minimum(left, right))
  hi = np.maximum(c, np.maximum(left, right))
  return c, lo, hi


def compute_dsi(im1, im2, n_labels, birchfield=1, squared_diffs=0, trunc_diffs=255):
  """im1 (reference/left), im2 (match/right): (H, W[, bands]) uint8 -> (H, W, n_labels) float32."""
  im1, im2 = _as_bands(im1), _as_bands(im2)
  H, W, bands = im1.shape
  colors = min(3, bands)
  worst = colors * (255 * 255 if squared_diffs else 255)            # aux.cpp:24
  max_sum = trunc_diffs * trunc_diffs if squared_diffs else colors * abs(trunc_diffs)  # :27-28
  bad = min(worst, max_sum)                                          # :30
  c1, lo1, hi1 = _interval(im1[:, :, :colors])
  c2, lo2, hi2 = _interval(im2[:, :, :colors])
  out = np.full((H, W, n_labels), bad, dtype=np.int64)
  for d in range(min(n_labels, W)):
    a = slice(d, W)        # x in the left image
    b = slice(0, W - d)    # x - d in the right image
    if birchfield:
      d1 = np.maximum(0, np.maximum(c1[:, a] - hi2[:, b], lo2[:, b] - c1[:, a]))
      d2 = np.maximum(0, np.maximum(c2[:, b] - hi1[:, a], lo1[:, a] - c2[:, b]))
      diff = np.minimum(d1, d2)
    else:
      diff = np.abs(c1[:, a] - c2[:, b])
    if squared_diffs:
      diff = diff * diff
    out[:, a, d] = np.minimum(diff.sum(axis=2), max_sum)
  return out.astype(np.float32)


def compute_cues(im, grad_thresh, grad_penalty):
  """-> h_cue (H, W-1), v_cue (W, H-1) float32 (auxPy.cpp:88-96: vCueId = w * (H-1) + h)."""
  im = _as_bands(im)
  c = im[:, :, :min(3, im.shape[2])].astype(np.int64)
  thresh = grad_thresh * c.shape[2] * grad_thresh                   # aux.cpp:118
  sx = ((c[:, :-1] - c[:, 1:]) ** 2).sum(axis=2)
  sy = ((c[:-1, :] - c[1:, :]) ** 2).sum(axis=2)
  h_cue = np.where(sx < thresh, grad_penalty, 1).astype(np.float32)
  v_cue = np.where(sy < thresh, grad_penalty, 1).astype(np.float32).T
  return h_cue, np.ascontiguousarray(v_cue)


def mrf_energy(unary, context, labels, edge_weights=None, n_dir=4, ctx2d=False):
  """unary (B, H, W, L), labels (n_lab, B, H, W) uint8, edge_weights (n_dir, B, H, W) or None,
  context (L,) [ctx(a, b) = context[|a - b|]] or (L, L) [ctx2d: context[min, max]]
  -> (n_lab, 2) float64: unary energy, pairwise energy."""
  unary = np.asarray(unary, dtype=np.float64)
  labels = np.asarray(labels).astype(np.int64)
  context = np.asarray(context, dtype=np.float64)
  B, H, W, L = unary.shape
  out = np.zeros((labels.shape[0], 2))
  for i, lab in enumerate(labels):
    out[i, 0] = np.take_along_axis(unary, lab[..., None], axis=3).sum()
    for d in range(0, n_dir, 2):
      hs, ws = STEPS[d]
      # receiving pixels p = (h, w) with q = (h - hs, w - ws) inside the image
      h0, h1 = max(0, hs), min(H, H + hs)
      w0, w1 = max(0, ws), min(W, W + ws)
      if h0 >= h1 or w0 >= w1:
        continue
      xp = lab[:, h0:h1, w0:w1]
      xq = lab[:, h0 - hs:h1 - hs, w0 - ws:w1 - ws]
      if ctx2d:
        c = context.reshape(L, L)[np.minimum(xp, xq), np.maximum(xp, xq)]
      else:
        c = context.reshape(-1)[np.abs(xp - xq)]
      wt = 1.0 if edge_weights is None else np.asarray(edge_weights, dtype=np.float64)[d][:, h0:h1, w0:w1]
      out[i, 1] += (wt * c).sum()
  return out
