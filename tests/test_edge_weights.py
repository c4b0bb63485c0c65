"""Edge-weight producer (utils/edge_weights.py:45-180 of the reference): the numpy oracle is pinned
with per-pixel loops written from the definition and with closed forms; the HIP kernel is then
compared with the oracle through the reference-style Python surface."""
import math

import numpy as np
import pytest

from oracle import edge_oracle

STEPS = [(0, 1), (0, -1), (1, 0), (-1, 0), (1, 1), (-1, -1), (1, -1), (-1, 1),
         (1, 2), (-1, -2), (2, 1), (-2, -1), (2, -1), (-2, 1), (1, -2), (-1, 2)]


def loops(edge_mode, image, n_dirs, sigma=10.0, threshold=0.0, penalty=0.0):
  """Definition, pixel by pixel, in float64 where it matters: weight of direction d at pixel p
  compares p with its front neighbour p - step(d); pixels without one keep 0."""
  B, C, H, W = image.shape
  out = np.zeros((n_dirs, B, C, H, W), dtype=np.float64)
  for d in range(n_dirs):
    hs, ws = STEPS[d]
    pairs = [(h, w, h - hs, w - ws) for h in range(H) for w in range(W)
             if 0 <= h - hs < H and 0 <= w - ws < W]
    cue = {}
    for b in range(B):
      for (h, w, qh, qw) in pairs:
        diffs = [abs(float(image[b, c, h, w]) - float(image[b, c, qh, qw])) for c in range(C)]
        for c in range(C):
          cur, diff = float(image[b, c, h, w]), diffs[c]
          if edge_mode == "gt_edge":
            v = 1.0 if (diff == 0 and cur != 255) else 0.0
          elif edge_mode == "canny":
            v = 1.0 - (1.0 if cur == 1 else diff)
          elif edge_mode in ("sobel", "edge_net_sigmoid"):
            v = 1.0 - diff
          elif edge_mode == "edge_net":
            v = math.exp(-diff)
          elif edge_mode == "superpixel_edge":
            v = 1.0 if sum(diffs) == 0 else 0.0
          elif edge_mode in ("kernel_cue_real", "kernel_cue_binary"):
            v = math.exp(-(sum(x * x for x in diffs) / C) / (2 * sigma ** 2))
            cue[(b, h, w)] = v
          elif edge_mode == "threshold":
            v = penalty if (sum(x * x for x in diffs) / C) < threshold else 0.0
          else:
            v = float(image[b, c, qh, qw])
          out[d, b, c, h, w] = v
    if edge_mode == "kernel_cue_binary" and cue:
      mean = sum(cue.values()) / len(cue)
      for (b, h, w), v in cue.items():
        out[d, b, :, h, w] = 1.0 if v >= 0.8 * mean else 0.0
  return out


def rand_image(rng, B, C, H, W, kind):
  if kind == "labels":  # label map with void pixels
    img = rng.integers(0, 3, size=(B, C, H, W)).astype(np.float32)
    img[rng.random((B, C, H, W)) < 0.1] = 255
    return img
  if kind == "binary":
    return (rng.random((B, C, H, W)) < 0.3).astype(np.float32)
  return rng.random((B, C, H, W)).astype(np.float32)


MODES = [("gt_edge", "labels"), ("canny", "binary"), ("sobel", "float"), ("edge_net_sigmoid", "float"),
         ("edge_net", "float"), ("superpixel_edge", "labels"), ("kernel_cue_real", "float"),
         ("kernel_cue_binary", "float"), ("threshold", "float"), ("shift", "float")]


@pytest.mark.parametrize("mode,kind", MODES)
def test_oracle_matches_definition(mode, kind):
  rng = np.random.default_rng(3)
  B = 1 if mode in edge_oracle.REDUCING else 2
  img = rand_image(rng, B, 3, 5, 6, kind)
  kw = dict(sigma=0.4, threshold=0.15, penalty=2.5)
  got = edge_oracle.edge_shift(mode, img, 16, **kw)
  want = loops(mode, img, 16, **kw)
  assert got.shape == (16, B, 3, 5, 6)
  np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-7)


def test_oracle_closed_forms():
  # constant image: every comparable pair is equal; pixels without a front neighbour keep 0
  img = np.full((1, 2, 4, 5), 7.0, np.float32)
  for mode, inside in (("gt_edge", 1.0), ("sobel", 1.0), ("edge_net", 1.0), ("superpixel_edge", 1.0),
                       ("kernel_cue_real", 1.0), ("kernel_cue_binary", 1.0), ("shift", 7.0)):
    out = edge_oracle.edge_shift(mode, img, 8, sigma=1.0)
    assert out[0, 0, 0, :, 1:].min() == inside and out[0, 0, 0, :, 1:].max() == inside
    assert (out[0, 0, 0, :, 0] == 0).all()        # dir 0 = (0, +1): column 0 has no front
    assert (out[1, 0, 0, :, -1] == 0).all()       # dir 1 = (0, -1): last column
    assert (out[2, 0, 0, 0, :] == 0).all()        # dir 2 = (+1, 0): first row
    assert (out[5, 0, 0, -1, :] == 0).all() and (out[5, 0, 0, :, -1] == 0).all()  # (-1, -1)
  # one step edge between columns 1 and 2: only the pixel that receives across it changes
  img = np.zeros((1, 1, 2, 4), np.float32)
  img[..., 2:] = 0.25
  out = edge_oracle.edge_shift("edge_net", img, 2)
  np.testing.assert_allclose(out[0, 0, 0, 0], [0, 1, math.exp(-0.25), 1], rtol=1e-6)
  np.testing.assert_allclose(out[1, 0, 0, 0], [1, math.exp(-0.25), 1, 0], rtol=1e-6)
  out = edge_oracle.edge_shift("shift", img, 2)
  np.testing.assert_allclose(out[0, 0, 0, 0], [0, 0, 0, 0.25])   # value of the left neighbour
  np.testing.assert_allclose(out[1, 0, 0, 0], [0, 0.25, 0.25, 0])  # value of the right neighbour
  # 255 marks void in a label map; an edge pixel (1) of a binary map always cuts
  lab = np.zeros((1, 1, 1, 4), np.float32)
  lab[..., 2] = 255
  np.testing.assert_array_equal(edge_oracle.edge_shift("gt_edge", lab, 1)[0, 0, 0, 0], [0, 1, 0, 0])
  edge = np.zeros((1, 1, 1, 4), np.float32)
  edge[..., 1:3] = 1
  np.testing.assert_array_equal(edge_oracle.edge_shift("canny", edge, 1)[0, 0, 0, 0], [0, 0, 0, 0])
  np.testing.assert_array_equal(edge_oracle.edge_shift("sobel", edge, 1)[0, 0, 0, 0], [0, 0, 1, 0])
  # colour cue: diff (0.3, 0.4, 0) -> mean square 0.25/3
  rgb = np.zeros((1, 3, 1, 2), np.float32)
  rgb[0, :, 0, 1] = (0.3, 0.4, 0.0)
  out = edge_oracle.edge_shift("kernel_cue_real", rgb, 1, sigma=0.5)
  np.testing.assert_allclose(out[0, 0, :, 0, 1], math.exp(-(0.25 / 3) / 0.5), rtol=1e-6)
  out = edge_oracle.edge_shift("threshold", rgb, 1, threshold=0.1, penalty=3.0)
  np.testing.assert_array_equal(out[0, 0, :, 0, 1], [3.0, 3.0, 3.0])
  out = edge_oracle.edge_shift("threshold", rgb, 1, threshold=0.05, penalty=3.0)
  np.testing.assert_array_equal(out[0, 0, :, 0, 1], [0.0, 0.0, 0.0])


def test_oracle_steps_match_scan_geometry(oracle):
  # the producer and the scan kernels must agree on which neighbour a weight belongs to
  for d in range(16):
    assert tuple(oracle.dir_step(d)) == edge_oracle.get_steps(d) == STEPS[d]
  assert edge_oracle.get_steps(16) == (0, 0)


def test_reducing_modes_take_one_image():
  with pytest.raises(ValueError):
    edge_oracle.edge_shift("threshold", np.zeros((2, 3, 4, 4), np.float32), 4)


def test_surface_refuses_cpu_tensors():
  import torch
  from mplayers_amd import edge_weights
  assert edge_weights.get_steps(10) == (2, 1)
  with pytest.raises(RuntimeError):
    edge_weights.getEdgeShift("sobel", torch.zeros(1, 1, 4, 4), 4)


# ------------------------------------------------------------------------------------------------
# GPU parity
# ------------------------------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("mode,kind", MODES)
@pytest.mark.parametrize("shape", [(2, 3, 7, 9), (1, 1, 33, 70), (3, 2, 1, 5), (1, 4, 130, 67)])
def test_gpu_matches_oracle(mode, kind, shape):
  import torch
  from mplayers_amd import edge_weights
  B, C, H, W = shape
  if mode in edge_oracle.REDUCING:
    B = 1
  rng = np.random.default_rng(B * 1000 + H)
  img = rand_image(rng, B, C, H, W, kind)
  kw = dict(sigma=0.4, threshold=0.15, penalty=2.5)
  print("case", mode, (B, C, H, W), flush=True)
  want = edge_oracle.edge_shift(mode, img, 16, **kw)
  got = edge_weights.getEdgeShift(mode, torch.from_numpy(img).cuda(), 16, **kw).cpu().numpy()
  assert got.shape == want.shape
  if mode == "kernel_cue_binary":
    # the mean is summed in a different order: values within 1e-6 of the cut may fall either way
    real = edge_oracle.edge_shift("kernel_cue_real", img, 16, **kw)
    for d in range(16):
      hs, ws = STEPS[d]
      valid = real[d][:, :, max(hs, 0):H + min(hs, 0), max(ws, 0):W + min(ws, 0)]
      if valid.size == 0:
        continue
      cut = 0.8 * valid.mean(dtype=np.float64)
      clear = np.abs(real[d] - cut) > 1e-5
      np.testing.assert_array_equal(got[d][clear], want[d][clear])
  else:
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-7)


@pytest.mark.gpu
def test_gpu_lower_rank_images_and_errors():
  import torch
  from mplayers_amd import edge_weights
  rng = np.random.default_rng(0)
  img = rng.random((3, 6, 8)).astype(np.float32)
  want = edge_oracle.edge_shift("edge_net", img[None], 8)
  got = edge_weights.getEdgeShift("edge_net", torch.from_numpy(img).cuda(), 8)
  assert tuple(got.shape) == (8, 3, 6, 8)
  np.testing.assert_allclose(got.cpu().numpy(), want[:, 0], rtol=2e-6, atol=1e-7)
  got2 = edge_weights.getEdgeShift("edge_net", torch.from_numpy(img[0]).cuda(), 4)
  assert tuple(got2.shape) == (4, 6, 8)
  np.testing.assert_allclose(got2.cpu().numpy(), want[:4, 0, 0], rtol=2e-6, atol=1e-7)
  with pytest.raises(RuntimeError):
    edge_weights.getEdgeShift("threshold", torch.zeros(2, 3, 4, 4).cuda(), 4)
  with pytest.raises(RuntimeError):
    edge_weights.getEdgeShift("sobel", torch.zeros(1, 3, 4, 4).cuda(), 17)


@pytest.mark.gpu
def test_gpu_multi_scale_and_layer_input():
  """multi_edge_weights at scale 1 equals getEdgeShift; at other scales it equals the oracle on
  the resampled image; the result feeds the layer in its (B, n_dir, H, W) layout."""
  import torch
  import torch.nn.functional as F
  from mplayers_amd import edge_weights
  rng = np.random.default_rng(1)
  img = torch.from_numpy(rng.random((3, 16, 20)).astype(np.float32)).cuda()
  mask = torch.ones(1, 16, 20).cuda()
  mask[:, :, 15:] = 0
  outs = edge_weights.multi_edge_weights("kernel_cue_real", img, 4, scale_list=[1, 0.5], sigma=0.3,
                                         padding_mask=mask)
  assert tuple(outs[0].shape) == (4, 3, 16, 20) and tuple(outs[1].shape) == (4, 3, 8, 10)
  want0 = edge_oracle.edge_shift("kernel_cue_real", img.cpu().numpy()[None], 4, sigma=0.3)[:, 0]
  want0 = want0 * mask.cpu().numpy()
  np.testing.assert_allclose(outs[0].cpu().numpy(), want0, rtol=2e-6, atol=1e-7)
  half = F.interpolate(img[None], scale_factor=(0.5, 0.5), mode="bilinear", align_corners=True)[0]
  want1 = edge_oracle.edge_shift("kernel_cue_real", half.cpu().numpy()[None], 4, sigma=0.3)[:, 0]
  got1 = outs[1].cpu().numpy()
  keep = got1 != 0  # the resampled mask removes the padded columns
  np.testing.assert_allclose(got1[keep], want1[keep], rtol=2e-6, atol=1e-7)
  assert (got1[:, :, :, -2:] == 0).all()
  sp = edge_weights.multi_edge_weights("superpixel_edge", torch.round(img * 2), 8, scale_list=[1])
  assert tuple(sp[0].shape) == (8, 16, 20)
