"""CPU restatement (numpy) of the reference's edge-weight producer, utils/edge_weights.py.

TEST INFRASTRUCTURE ONLY: imported by tests/ (and nothing else); the product path is the HIP kernel
behind mpl_edge_shift.

get_steps follows utils/edge_weights.py:5-42 (the direction table of MPLayers/common.cpp:28-76);
edge_shift follows getEdgeShift, utils/edge_weights.py:45-111: for direction d with step r and every
pixel p whose front neighbour q = p - r is inside the image, out[d, p] = f(|I(p) - I(q)|), and 0
where q is outside.  Written with coordinate grids and a gather instead of the reference's slice
pairs; tests/test_edge_weights.py pins it with per-pixel loops and closed forms.
"""
import numpy as np

STEPS = ((0, 1), (0, -1), (1, 0), (-1, 0), (1, 1), (-1, -1), (1, -1), (-1, 1),
         (1, 2), (-1, -2), (2, 1), (-2, -1), (2, -1), (-2, 1), (1, -2), (-1, 2))

REDUCING = ("superpixel_edge", "kernel_cue_real", "kernel_cue_binary", "threshold")


def get_steps(d):
  """utils/edge_weights.py:5-42: (h_step, w_step); (0, 0) outside the table."""
  return STEPS[d] if 0 <= d < len(STEPS) else (0, 0)


def edge_shift(edge_mode, image, n_dirs, sigma=10.0, threshold=0.0, penalty=0.0):
  """image (B, C, H, W) float32 -> (n_dirs, B, C, H, W) float32; getEdgeShift for a 4-D image.
  The channel-reducing modes follow the reference's broadcasting for one image (B == 1)."""
  image = np.asarray(image, dtype=np.float32)
  B, C, H, W = image.shape
  if edge_mode in REDUCING and B != 1:
    raise ValueError("channel-reducing modes take one image")
  out = np.zeros((n_dirs, B, C, H, W), dtype=np.float32)
  hh, ww = np.meshgrid(np.arange(H), np.arange(W), indexing="ij")
  for d in range(n_dirs):
    hs, ws = get_steps(d)
    qh, qw = hh - hs, ww - ws
    valid = (qh >= 0) & (qh < H) & (qw >= 0) & (qw < W)
    if not valid.any():
      continue
    front = image[:, :, np.clip(qh, 0, H - 1), np.clip(qw, 0, W - 1)]  # I(q), garbage where invalid
    diff = np.abs(image - front)
    if edge_mode == "gt_edge":  # :80-81, :86-87
      diff = np.where(image == 255, np.float32(1), diff)
      val = (diff == 0).astype(np.float32)
    elif edge_mode == "canny":  # :82-83, :90-91
      diff = np.where(image == 1, np.float32(1), diff)
      val = 1 - diff
    elif edge_mode in ("sobel", "edge_net_sigmoid"):  # :90-93
      val = 1 - diff
    elif edge_mode == "edge_net":  # :94-95
      val = np.exp(-diff)
    elif edge_mode == "superpixel_edge":  # :88-89
      val = np.broadcast_to((diff.sum(axis=1, keepdims=True) == 0).astype(np.float32), diff.shape)
    elif edge_mode in ("kernel_cue_real", "kernel_cue_binary"):  # :96-99
      g = np.exp(np.mean(diff * diff, axis=1, keepdims=True, dtype=np.float32)
                 / np.float32(-2.0 * sigma ** 2)).astype(np.float32)
      if edge_mode == "kernel_cue_binary":
        mean = g[:, :, valid].mean(dtype=np.float64)
        g = (g >= np.float32(0.8) * np.float32(mean)).astype(np.float32)
      val = np.broadcast_to(g, diff.shape)
    elif edge_mode == "threshold":  # :100-101
      m = np.mean(diff * diff, axis=1, keepdims=True, dtype=np.float32)
      val = np.broadcast_to((m < threshold).astype(np.float32) * np.float32(penalty), diff.shape)
    else:  # :102-103: the shifted image itself
      val = front
    out[d] = np.where(valid, val, np.float32(0))
  return out
