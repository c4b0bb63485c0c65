"""Edge-weight producers of the reference (utils/edge_weights.py) on top of the HIP kernel
mpl_edge_shift: same function names, arguments and result shapes.

    get_steps(dir)                                   utils/edge_weights.py:5-42
    getEdgeShift(edge_mode, image, n_dirs, ...)      utils/edge_weights.py:45-111
    multi_edge_weights(edge_mode, img, n_dirs, ...)  utils/edge_weights.py:115-180

The image must live on the GPU; there is no CPU path.
"""
import ctypes

import torch
import torch.nn.functional as F

from . import _lib

_STEPS = ((0, 1), (0, -1), (1, 0), (-1, 0), (1, 1), (-1, -1), (1, -1), (-1, 1),
          (1, 2), (-1, -2), (2, 1), (-2, -1), (2, -1), (-2, 1), (1, -2), (-1, 2))

# edge_mode string -> MPL_EDGE_* of include/mplayers_amd.h; anything else is the plain shift
_MODES = {"gt_edge": 0, "superpixel_edge": 1, "sobel": 2, "edge_net_sigmoid": 2, "canny": 3,
          "edge_net": 4, "kernel_cue_real": 5, "kernel_cue_binary": 6, "threshold": 7}
_MODE_SHIFT = 8
_REDUCING = (1, 5, 6, 7)


def get_steps(dir):
  """(h_step, w_step) of a direction; (0, 0) and a warning outside the 16-direction table."""
  if 0 <= dir < len(_STEPS):
    return _STEPS[dir]
  print('Warning, edge weights support only 16 directions by far')
  return 0, 0


def getEdgeShift(edge_mode, image, n_dirs, sigma=10, threshold=0, penalty=0):
  """image (batch, channels, h, w), (channels, h, w) or (h, w) -> edge weights
  (n_dirs, batch, channels, h, w) with the leading singleton axes of a 3-D / 2-D image removed
  again, as the reference does."""
  ndim = image.dim()
  if ndim == 2:
    image = image[None, None]
  elif ndim == 3:
    image = image[None]
  assert image.dim() == 4, image.size()
  if not image.is_cuda:
    raise RuntimeError("getEdgeShift: the image must be a GPU tensor (no CPU path in this build)")
  if n_dirs > len(_STEPS):
    raise RuntimeError("getEdgeShift: at most 16 directions")
  mode = _MODES.get(edge_mode, _MODE_SHIFT)
  batch, channels, height, width = image.size()
  if mode in _REDUCING and batch != 1:
    # the reference's broadcasting assignment only has a meaning for one image
    raise RuntimeError("getEdgeShift: edge_mode %r takes one image (batch == 1)" % edge_mode)
  src = image.contiguous().float()
  out = torch.empty((n_dirs, batch, channels, height, width), dtype=torch.float32,
                    device=image.device)
  sums = (torch.empty(16, dtype=torch.float64, device=image.device)
          if edge_mode == "kernel_cue_binary" else None)
  with torch.cuda.device(image.device):
    stream = torch.cuda.current_stream().cuda_stream
    rc = _lib.load().mpl_edge_shift(
        mode, ctypes.c_void_p(src.data_ptr()), batch, channels, height, width, n_dirs,
        ctypes.c_float(sigma), ctypes.c_float(threshold), ctypes.c_float(penalty),
        ctypes.c_void_p(out.data_ptr()),
        ctypes.c_void_p(sums.data_ptr() if sums is not None else None), ctypes.c_void_p(stream))
  _lib.check(rc, "edge_shift")
  out = out.to(image.dtype) if image.dtype.is_floating_point else out
  if ndim == 2:
    out = out[:, 0, 0]
  elif ndim == 3:
    out = out[:, 0]
  return out


def multi_edge_weights(edge_mode, img, n_dirs, scale_list=None, sigma=5, threshold=10, penalty=2,
                       padding_mask=None):
  """Edge weights of one (channels, h, w) image at every scale of scale_list: a list of
  (n_dirs, channels, h_s, w_s) tensors (superpixel_edge: (n_dirs, h_s, w_s)).  Resampling follows
  the reference: nearest for label-like inputs, bilinear with aligned corners otherwise; the
  padding mask is resampled on a regular [-1, 1] grid and re-binarised at 0.5."""
  _, height, width = img.size()
  nearest = edge_mode in ('gt_edge', 'edge_net', 'edge_net_sigmoid', 'superpixel_edge')
  results = []
  for scale in scale_list:
    if scale == 1:
      scaled, mask = img, padding_mask
    else:
      if nearest:
        scaled = F.interpolate(img[None], scale_factor=(scale, scale), mode='nearest')[0]
      else:
        scaled = F.interpolate(img[None], scale_factor=(scale, scale), mode='bilinear',
                               align_corners=True)[0]
      mask = None
      if padding_mask is not None:
        h_s, w_s = int(height * scale), int(width * scale)
        xs = torch.linspace(-1, 1, w_s, device=padding_mask.device).expand(h_s, w_s)
        ys = torch.linspace(-1, 1, h_s, device=padding_mask.device)[:, None].expand(h_s, w_s)
        grid = torch.stack((xs, ys), dim=2)[None]
        mask = (F.grid_sample(padding_mask[None], grid, align_corners=False)[0] > 0.5).float()
    if n_dirs > 0:
      weights = getEdgeShift(edge_mode, scaled, n_dirs, sigma=sigma, threshold=threshold,
                             penalty=penalty)
      weights = weights.squeeze(1)
    else:
      weights = scaled
    if mask is not None:
      weights = weights * mask
    if edge_mode == 'superpixel_edge':
      weights = weights[:, 0]
    results.append(weights)
  return results
