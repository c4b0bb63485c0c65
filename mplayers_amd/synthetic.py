"""Seeded synthetic inputs of the benchmark configurations (stereo-, denoise-, segmentation-shaped).

All random draws come from one CPU torch.Generator, so CPU and GPU runs see identical bits.
Returned tensors are CPU tensors in the layouts of the autograd Functions:
  unary (B, 1, H, W, L), context (L,) or (21, 21), edge_weights (n_dir, B, 1, H, W) or None.
"""
import math

import torch

_STEPS = [(0, 1), (0, -1), (1, 0), (-1, 0), (1, 1), (-1, -1), (1, -1), (-1, 1),
          (1, 2), (-1, -2), (2, 1), (-2, -1), (2, -1), (-2, 1), (1, -2), (-1, 2)]


def truncated_linear(n_labels, trunc, scale):
  k = torch.arange(n_labels, dtype=torch.float32)
  return torch.clamp(k, max=float(trunc)) * scale


def truncated_quadratic(n_labels, trunc, scale):
  k = torch.arange(n_labels, dtype=torch.float32)
  return torch.clamp(k * k, max=float(trunc)) * scale


def _gaussian_blur(img, sigma, radius):
  x = torch.arange(-radius, radius + 1, dtype=torch.float32)
  k = torch.exp(-x * x / (2 * sigma * sigma))
  k = k / k.sum()
  t = img[None, None]
  t = torch.nn.functional.pad(t, (radius, radius, radius, radius), mode="reflect")
  t = torch.nn.functional.conv2d(t, k.view(1, 1, 1, -1))
  t = torch.nn.functional.conv2d(t, k.view(1, 1, -1, 1))
  return t[0, 0]


def image_edge_weights(H, W, n_dir, gen):
  """exp(-|I(p) - I(p - r_d)|) from a blurred random image; 1 where p - r_d is outside.
  The weight of an edge is stored at the pixel that receives the message."""
  img = _gaussian_blur(torch.rand(H, W, generator=gen), sigma=2.0, radius=6)
  out = torch.ones(n_dir, 1, 1, H, W)
  for d in range(n_dir):
    hs, ws = _STEPS[d]
    h0, h1 = max(hs, 0), H + min(hs, 0)
    w0, w1 = max(ws, 0), W + min(ws, 0)
    if h1 <= h0 or w1 <= w0:
      continue
    cur = img[h0:h1, w0:w1]
    front = img[h0 - hs:h1 - hs, w0 - ws:w1 - ws]
    out[d, 0, 0, h0:h1, w0:w1] = torch.exp(-(cur - front).abs())
  return out


def stereo_unary(H, W, L, gen):
  """|l - d*(p)| / L + N(0, 0.05), d* piecewise constant: a background plus 20 random rectangles."""
  disp = torch.full((H, W), int(torch.randint(0, L, (1,), generator=gen)), dtype=torch.float32)
  for _ in range(20):
    hh = sorted(int(v) for v in torch.randint(0, H, (2,), generator=gen))
    ww = sorted(int(v) for v in torch.randint(0, W, (2,), generator=gen))
    disp[hh[0]:hh[1] + 1, ww[0]:ww[1] + 1] = float(torch.randint(0, L, (1,), generator=gen))
  lab = torch.arange(L, dtype=torch.float32)
  unary = (lab.view(1, 1, L) - disp.view(H, W, 1)).abs() / L
  unary = unary + 0.05 * torch.randn(H, W, L, generator=gen)
  return unary.view(1, 1, H, W, L).contiguous()


def denoise_unary(H, W, L, gen):
  """(l - y(p))^2 with y a smooth random uint8 image (8 Gaussian bumps) plus N(0, 20) noise."""
  hh, ww = torch.meshgrid(torch.arange(H, dtype=torch.float32),
                          torch.arange(W, dtype=torch.float32), indexing="ij")
  img = torch.zeros(H, W)
  for _ in range(8):
    a = 0.3 + 0.7 * float(torch.rand(1, generator=gen))
    ch = float(torch.rand(1, generator=gen)) * H
    cw = float(torch.rand(1, generator=gen)) * W
    s = 20 + 40 * float(torch.rand(1, generator=gen))
    img = img + a * torch.exp(-((hh - ch) ** 2 + (ww - cw) ** 2) / (2 * s * s))
  img = (img - img.min()) / (img.max() - img.min() + 1e-12) * 255
  y = torch.clamp(img + 20 * torch.randn(H, W, generator=gen), 0, 255).round()
  lab = torch.arange(L, dtype=torch.float32)
  return ((lab.view(1, 1, L) - y.view(H, W, 1)) ** 2).view(1, 1, H, W, L).contiguous()


CONFIGS = {
    # name: mode, rho, B, H, W, L, n_dir, n_iter, training
    "C1": dict(mode="ISGMR", rho=1.0, B=1, H=64, W=96, L=16, n_dir=4, n_iter=3, training=True),
    "C2": dict(mode="TRWP", rho=0.5, B=1, H=384, W=1248, L=96, n_dir=4, n_iter=5, training=False),
    "C3": dict(mode="ISGMR", rho=1.0, B=1, H=256, W=256, L=256, n_dir=4, n_iter=50, training=False),
    "C4": dict(mode="TRWP", rho=0.5, B=4, H=129, W=129, L=21, n_dir=4, n_iter=5, training=True),
    "C5": dict(mode="TRWP", rho=0.5, B=1, H=1500, W=2000, L=192, n_dir=8, n_iter=5, training=True),
}


def make_config(name, seed=0, scale=1.0, mode=None, n_dir=None, context=None, n_labels=None,
                batch=None, n_iter=None):
  """Builds the inputs of configuration `name` (C1..C5).  scale < 1 shrinks H and W (parity tests
  at sizes a CPU checker finishes in seconds); mode overrides TRWP/ISGMR for the two-algorithm
  configurations.  n_labels, batch, n_iter run the same problem at another size; context
  ("dense1d" / "dense2d") replaces the pairwise table by a learned-style dense one: random entries
  in [0, 1), zero at offset 0 / on the diagonal (2-D: upper triangle, the part that is read).
  Returns a dict with the config fields plus unary, context, edge_weights."""
  cfg = dict(CONFIGS[name])
  if n_labels is not None:
    cfg["L"] = int(n_labels)
  if batch is not None:
    cfg["B"] = int(batch)
  if n_iter is not None:
    cfg["n_iter"] = int(n_iter)
  if mode is not None:
    cfg["mode"] = mode
    cfg["rho"] = 0.5 if mode == "TRWP" else 1.0
  cfg["name"] = name
  if n_dir is not None:
    cfg["n_dir"] = int(n_dir)  # the same problem on another connectivity (2, 4, 8 or 16 directions)
  H = cfg["H"] = max(2, int(round(cfg["H"] * scale)))
  W = cfg["W"] = max(2, int(round(cfg["W"] * scale)))
  B, L, n_dir = cfg["B"], cfg["L"], cfg["n_dir"]
  gen = torch.Generator(device="cpu").manual_seed(seed)
  if name == "C1":
    cfg["unary"] = torch.rand(B, 1, L, H, W, generator=gen).permute(0, 1, 3, 4, 2).contiguous()
    cfg["context"] = truncated_linear(L, 4, 0.5)
    cfg["edge_weights"] = torch.ones(n_dir, B, 1, H, W)
  elif name in ("C2", "C5"):
    cfg["unary"] = torch.cat([stereo_unary(H, W, L, gen) for _ in range(B)], 0)
    cfg["context"] = truncated_linear(L, 2, 0.25) if name == "C2" else truncated_linear(L, 3, 0.3)
    cfg["edge_weights"] = torch.cat([image_edge_weights(H, W, n_dir, gen) for _ in range(B)], 1)
  elif name == "C3":
    cfg["unary"] = denoise_unary(H, W, L, gen)
    cfg["context"] = truncated_quadratic(L, 200, 25.0)
    cfg["edge_weights"] = torch.ones(n_dir, B, 1, H, W)
  elif name == "C4":
    cfg["unary"] = torch.randn(B, 1, L, H, W, generator=gen).permute(0, 1, 3, 4, 2).contiguous()
    cfg["context"] = torch.triu(torch.rand(L, L, generator=gen), diagonal=1)
    ew = 0.1 + 0.9 * torch.rand(B, n_dir, H, W, generator=gen)
    cfg["edge_weights"] = ew.unsqueeze(1).permute(2, 0, 1, 3, 4).contiguous()
  else:
    raise KeyError(name)
  if context == "dense1d":
    c = torch.rand(L, generator=gen)
    c[0] = 0.0
    cfg["context"] = c
  elif context == "dense2d":
    if L != 21:
      raise ValueError("the operators take a 2-D table with 21 labels only, as the reference does")
    cfg["context"] = torch.triu(torch.rand(L, L, generator=gen), diagonal=1)
  elif context is not None:
    raise KeyError(context)
  cfg["units"] = B * H * W * L * cfg["n_iter"]
  return cfg


def upstream_grad(cfg, seed=1):
  gen = torch.Generator(device="cpu").manual_seed(seed)
  return torch.randn(cfg["unary"].shape, generator=gen)
