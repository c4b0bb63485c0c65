"""MRF terms of the reference's energy-minimisation driver on top of the HIP kernels
mpl_stereo_data_cost, mpl_gradient_cues and mpl_mrf_energy.

    compute_all_terms(...)        lib_stereo.compute_terms.compute_all_terms, MPLayers/aux/auxPy.cpp:7-111
    MRFParams, compute_terms_py   MPLayers/test_compute_terms.py:13-57
    smoothness_context(...)       computeSmoothnessContext, MPLayers/aux/aux.cpp:172-226
    stereo_data_cost, gradient_cues, mrf_energy   tensor-level functions over the C ABI

Images are decoded on the host (PIL) and everything else runs on the GPU; there is no CPU path.
"""
import ctypes

import numpy as np
import torch

from . import _lib


def _device():
  if not torch.cuda.is_available():
    raise RuntimeError("compute_terms: needs a GPU (there is no CPU path in this build)")
  return torch.device("cuda", torch.cuda.current_device())


def read_image(path_or_array):
  """-> (H, W, bands) uint8 numpy array.  A colour file comes back in B, G, R band order, as the
  reference's OpenCV reader delivers it (auxPy.cpp:28); arrays are taken as they are."""
  if isinstance(path_or_array, (str, bytes)) or hasattr(path_or_array, "__fspath__"):
    from PIL import Image
    with Image.open(path_or_array) as img:
      if img.mode not in ("L", "RGB"):
        img = img.convert("RGB" if img.mode in ("RGBA", "P", "CMYK") else "L")
      arr = np.array(img, dtype=np.uint8)
    if arr.ndim == 3:
      arr = arr[:, :, ::-1]
  else:
    arr = np.asarray(path_or_array)
    if arr.dtype != np.uint8:
      raise RuntimeError("compute_terms: images must be uint8")
  if arr.ndim == 2:
    arr = arr[:, :, None]
  if arr.ndim != 3:
    raise RuntimeError("compute_terms: an image is (H, W) or (H, W, bands)")
  return np.ascontiguousarray(arr)


def _image_tensor(img, device):
  if torch.is_tensor(img):
    if img.dtype != torch.uint8:
      raise RuntimeError("compute_terms: images must be uint8")
    t = img if img.dim() == 3 else img[:, :, None]
    return t.to(device).contiguous()
  return torch.from_numpy(read_image(img)).to(device)


def stereo_data_cost(left, right, n_disp, birchfield=True, squared_diffs=False, trunc_diffs=255):
  """left, right: (H, W[, bands]) uint8 (paths, arrays or tensors) -> (H, W, n_disp) fp32 GPU
  tensor, the `unary` layout of the layers (label axis innermost)."""
  dev = _device()
  im1, im2 = _image_tensor(left, dev), _image_tensor(right, dev)
  if im1.shape != im2.shape:
    raise RuntimeError("compute_terms: image shapes don't match")  # auxPy.cpp:42-43
  height, width, bands = im1.shape
  out = torch.empty((height, width, n_disp), dtype=torch.float32, device=dev)
  with torch.cuda.device(dev):
    rc = _lib.load().mpl_stereo_data_cost(
        ctypes.c_void_p(im1.data_ptr()), ctypes.c_void_p(im2.data_ptr()), height, width, bands,
        n_disp, int(bool(birchfield)), int(bool(squared_diffs)), int(trunc_diffs),
        ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
  _lib.check(rc, "stereo_data_cost")
  return out


def gradient_cues(image, grad_thresh, grad_penalty):
  """-> h_cue (H, W-1), v_cue (W, H-1) fp32 GPU tensors."""
  dev = _device()
  im = _image_tensor(image, dev)
  height, width, bands = im.shape
  h_cue = torch.empty((height, width - 1), dtype=torch.float32, device=dev)
  v_cue = torch.empty((width, height - 1), dtype=torch.float32, device=dev)
  with torch.cuda.device(dev):
    rc = _lib.load().mpl_gradient_cues(
        ctypes.c_void_p(im.data_ptr()), height, width, bands, int(grad_thresh),
        ctypes.c_float(grad_penalty), ctypes.c_void_p(h_cue.data_ptr() if h_cue.numel() else None),
        ctypes.c_void_p(v_cue.data_ptr() if v_cue.numel() else None),
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
  _lib.check(rc, "gradient_cues")
  return h_cue, v_cue


def smoothness_context(n_labels, method, smoothness_max):
  """(n_labels, n_labels) fp32 CPU tensor of the pairwise function of |xi - xj| (aux.cpp:172-226):
  'L', 'Q', 'TL', 'TQ' (truncated at smoothness_max, squared for TQ), 'Cauchy', 'Huber'."""
  delta = torch.arange(n_labels, dtype=torch.float32)
  delta = (delta[:, None] - delta[None, :]).abs()
  smax = float(smoothness_max)
  if method == "L":
    table = delta
  elif method == "Q":
    table = delta * delta
  elif method == "TL":
    table = delta.clamp(max=smax)
  elif method == "TQ":
    table = (delta * delta).clamp(max=smax * smax)
  elif method == "Cauchy":
    table = (0.5 * smax * smax * torch.log1p((delta.double() / smax) ** 2)).float()
  elif method == "Huber":
    table = torch.where(delta <= smax, delta * delta, 2 * smax * delta - smax * smax)
  else:
    raise RuntimeError("smoothness_context: unknown method %r" % (method,))
  return table.contiguous()


def compute_all_terms(left_img_path, right_img_path, context, grad_thresh, grad_penalty, truncated,
                      height, width, n_channels, n_disp, data_cost, RGB, h_cue, v_cue,
                      smoothness_context_out):
  """Fills the caller's tensors, as the reference extension does: data_cost (H*W, n_disp),
  RGB (H*W, n_channels), h_cue (1, H*(W-1)), v_cue (1, (H-1)*W), smoothness_context (n_disp,
  n_disp); they may live on the CPU (the reference's case) or on the GPU."""
  left, right = read_image(left_img_path), read_image(right_img_path)
  if left.shape != right.shape:
    raise RuntimeError("compute_terms: image shapes don't match")
  if (height, width) != left.shape[:2]:
    raise RuntimeError("compute_terms: size does not match, extern h:%d, w:%d, intern h:%d, w:%d"
                       % (height, width, left.shape[0], left.shape[1]))
  if n_channels > left.shape[2]:
    raise RuntimeError("compute_terms: the image has %d bands, %d asked for" % (left.shape[2], n_channels))
  dev = _device()
  im1 = torch.from_numpy(left).to(dev)
  cost = stereo_data_cost(im1, torch.from_numpy(right).to(dev), n_disp)
  data_cost.view(-1).copy_(cost.view(-1))
  RGB.view(-1).copy_(im1[:, :, :n_channels].float().reshape(-1))
  hc, vc = gradient_cues(im1, grad_thresh, grad_penalty)
  h_cue.view(-1).copy_(hc.view(-1))
  v_cue.view(-1).copy_(vc.view(-1))
  smoothness_context_out.view(-1).copy_(smoothness_context(n_disp, context, truncated).view(-1))


class MRFParams():
  """MPLayers/test_compute_terms.py:13-27."""

  def __init__(self, left_img_path, right_img_path, context, n_disp, grad_thresh, grad_penalty,
               truncated):
    self.left_img_path = left_img_path
    self.right_img_path = right_img_path
    self.context = context
    self.grad_thresh = grad_thresh
    self.grad_penalty = grad_penalty
    self.truncated = truncated
    self.n_disp = n_disp
    self.height = 0
    self.width = 0
    self.n_channels = 0
    self.data_type = torch.float32


def compute_terms_py(param, device=None):
  """-> data_cost (H, W, n_disp), RGB (H, W, bands), smoothness_context (n_disp, n_disp), param
  (MPLayers/test_compute_terms.py:30-57).  The tensors stay on the GPU unless device says
  otherwise."""
  left = read_image(param.left_img_path)
  param.height, param.width, param.n_channels = left.shape
  dev = _device()
  im1 = torch.from_numpy(left).to(dev)
  data_cost = stereo_data_cost(im1, param.right_img_path, param.n_disp)
  rgb = im1.to(param.data_type)
  table = smoothness_context(param.n_disp, param.context, param.truncated).to(dev)
  if device is not None:
    data_cost, rgb, table = data_cost.to(device), rgb.to(device), table.to(device)
  return data_cost, rgb, table, param


def mrf_energy(unary, label_context, labels, edge_weights=None, n_dir=4):
  """Energies of labellings.  unary (B, H, W, L) fp32 [the operators' layout], labels
  (n, B, H, W) or (B, H, W) uint8, label_context as the operators take it (a (21, 21) table when
  L == 21, else at least L floats indexed by |xi - xj|), edge_weights (n_dir, B, H, W) or None
  -> (n, 2) fp64 GPU tensor: unary energy, pairwise energy (every undirected edge once)."""
  for name, t in (("unary", unary), ("label_context", label_context), ("labels", labels)):
    if not t.is_cuda:
      raise RuntimeError("mrf_energy: %s must be a GPU tensor" % name)
    if not t.is_contiguous():
      raise RuntimeError("mrf_energy: %s must be contiguous" % name)
  if unary.dtype != torch.float32 or label_context.dtype != torch.float32:
    raise RuntimeError("mrf_energy: unary and label_context must be float32")
  if labels.dtype != torch.uint8:
    raise RuntimeError("mrf_energy: labels must be uint8")
  batch, height, width, n_disp = unary.shape
  if labels.dim() == 3:
    labels = labels[None]
  if tuple(labels.shape[1:]) != (batch, height, width):
    raise RuntimeError("mrf_energy: labels must be (n, batch, height, width)")
  ctx2d = int(n_disp == 21)
  if label_context.numel() < (n_disp * n_disp if ctx2d else n_disp):
    raise RuntimeError("mrf_energy: label_context is too small")
  if edge_weights is not None:
    if (not edge_weights.is_cuda or not edge_weights.is_contiguous()
        or edge_weights.dtype != torch.float32
        or tuple(edge_weights.shape) != (n_dir, batch, height, width)):
      raise RuntimeError("mrf_energy: edge_weights must be a contiguous float32 GPU tensor "
                         "(n_dir, batch, height, width)")
  out = torch.empty((labels.shape[0], 2), dtype=torch.float64, device=unary.device)
  shape = _lib.Shape(n_dir, batch, height, width, n_disp, ctx2d)
  with torch.cuda.device(unary.device):
    rc = _lib.load().mpl_mrf_energy(
        ctypes.byref(shape), labels.shape[0], ctypes.c_void_p(unary.data_ptr()),
        ctypes.c_void_p(label_context.data_ptr()),
        ctypes.c_void_p(edge_weights.data_ptr() if edge_weights is not None else None),
        ctypes.c_void_p(labels.data_ptr()), ctypes.c_void_p(out.data_ptr()),
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
  _lib.check(rc, "mrf_energy")
  return out
