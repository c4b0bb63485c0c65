"""GPU parity of the MRF terms around the layers (mpl_stereo_data_cost, mpl_gradient_cues,
mpl_mrf_energy) against oracle/terms_oracle.py, through the reference-style Python surface
(mplayers_amd.compute_terms), and the energy-minimisation driver end to end.

Data cost and cues are integer work: bit-exact.  Energies are fp64 sums of fp32 terms accumulated
in an order that is not fixed: 1e-12 relative."""
import itertools

import numpy as np
import pytest

from oracle import terms_oracle

pytestmark = pytest.mark.gpu


def _torch():
  import torch
  return torch


@pytest.mark.parametrize("H,W,bands,L", [(5, 17, 3, 7), (3, 9, 1, 4), (4, 6, 4, 9), (2, 5, 2, 13),
                                         (37, 53, 3, 21), (1, 1, 3, 3), (16, 64, 3, 192)])
@pytest.mark.parametrize("flags", [(1, 0, 255), (0, 0, 255), (1, 1, 30), (1, 0, 7), (0, 1, 255)])
def test_data_cost_bit_exact(gpu, H, W, bands, L, flags):
  from mplayers_amd import compute_terms
  rng = np.random.default_rng(H * 131 + W * 7 + L)
  shape = (H, W) if bands == 1 and H % 2 else (H, W, bands)
  im1 = rng.integers(0, 256, size=shape, dtype=np.uint8)
  # a right image that really matches somewhere, plus noise
  im2 = np.roll(im1, -2, axis=1) if W > 2 else im1.copy()
  noise = rng.integers(-6, 7, size=shape)
  im2 = np.clip(im2.astype(np.int64) + noise, 0, 255).astype(np.uint8)
  bf, sq, trunc = flags
  got = compute_terms.stereo_data_cost(im1, im2, L, bf, sq, trunc).cpu().numpy()
  want = terms_oracle.compute_dsi(im1, im2, L, bf, sq, trunc)
  assert got.shape == want.shape == (H, W, L)
  assert (got == want).all()


def test_data_cost_large_image_properties(gpu):
  """Full stereo size (the cost volume of a 1500 x 2000 pair with 192 disparities, 2.3 GB): the
  volume is exact on sampled rows, and shifting both images by one row shifts the volume."""
  torch = _torch()
  from mplayers_amd import compute_terms
  H, W, L = 1500, 2000, 192
  g = torch.Generator().manual_seed(3)
  left = torch.randint(0, 256, (H, W, 3), dtype=torch.uint8, generator=g)
  right = torch.roll(left, -17, dims=1)
  cost = compute_terms.stereo_data_cost(left.cuda(), right.cuda(), L)
  assert cost.shape == (H, W, L)
  for y in (0, 749, H - 1):
    want = terms_oracle.compute_dsi(left[y:y + 1].numpy(), right[y:y + 1].numpy(), L)
    assert (cost[y:y + 1].cpu().numpy() == want).all()
  assert bool((cost[:, 17:, 17] == 0).all())
  assert bool((cost[:, :17, 17] == 765).all())
  moved = compute_terms.stereo_data_cost(torch.roll(left, 1, dims=0).cuda(),
                                         torch.roll(right, 1, dims=0).cuda(), L)
  assert bool((moved[1:] == cost[:-1]).all())


@pytest.mark.parametrize("H,W,bands", [(2, 3, 3), (9, 14, 3), (7, 5, 1), (6, 6, 4), (1, 8, 3), (8, 1, 3)])
def test_gradient_cues_exact(gpu, H, W, bands):
  from mplayers_amd import compute_terms
  rng = np.random.default_rng(H + 10 * W)
  # smooth-ish image so that both outcomes occur
  im = np.clip(128 + np.cumsum(rng.integers(-4, 5, size=(H, W, bands)), axis=1), 0, 255).astype(np.uint8)
  for thresh, penalty in ((3, 2), (8, 5), (0, 4)):
    h_cue, v_cue = compute_terms.gradient_cues(im, thresh, penalty)
    want_h, want_v = terms_oracle.compute_cues(im, thresh, penalty)
    assert (h_cue.cpu().numpy() == want_h).all()
    assert (v_cue.cpu().numpy() == want_v).all()


@pytest.mark.parametrize("n_dir,L,B,H,W", [(4, 5, 2, 5, 6), (8, 21, 1, 9, 7), (16, 4, 2, 6, 9),
                                           (2, 3, 1, 1, 12), (8, 192, 1, 33, 47), (4, 256, 1, 4, 5)])
def test_energy_matches_oracle(gpu, n_dir, L, B, H, W):
  torch = _torch()
  from mplayers_amd import compute_terms
  rng = np.random.default_rng(n_dir * 100 + L)
  ctx2d = L == 21
  unary = rng.standard_normal((B, H, W, L)).astype(np.float32)
  context = (rng.random((L, L)) if ctx2d else rng.random(L)).astype(np.float32)
  edge = rng.random((n_dir, B, H, W)).astype(np.float32)
  labels = rng.integers(0, L, size=(4, B, H, W)).astype(np.uint8)
  dev = lambda a: torch.from_numpy(a).cuda()
  for ew in (None, edge):
    got = compute_terms.mrf_energy(dev(unary), dev(context), dev(labels),
                                   None if ew is None else dev(ew), n_dir).cpu().numpy()
    want = terms_oracle.mrf_energy(unary, context, labels, ew, n_dir, ctx2d)
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)
  # a single labelling may come without the leading axis; repeated calls overwrite the result
  one = compute_terms.mrf_energy(dev(unary), dev(context), dev(labels[2]), dev(edge), n_dir)
  np.testing.assert_allclose(one.cpu().numpy()[0], want[2], rtol=1e-12, atol=1e-12)


def test_energy_errors(gpu):
  torch = _torch()
  from mplayers_amd import compute_terms
  unary = torch.zeros(1, 4, 5, 3, device="cuda")
  ctx = torch.ones(3, device="cuda")
  labels = torch.zeros(2, 1, 4, 5, dtype=torch.uint8, device="cuda")
  with pytest.raises(RuntimeError):
    compute_terms.mrf_energy(unary.cpu(), ctx, labels)
  with pytest.raises(RuntimeError):
    compute_terms.mrf_energy(unary, ctx[:2], labels)
  with pytest.raises(RuntimeError):
    compute_terms.mrf_energy(unary, ctx, labels[:, :, :3])
  with pytest.raises(RuntimeError):
    compute_terms.mrf_energy(unary, ctx, labels, None, 3)
  with pytest.raises(RuntimeError):
    compute_terms.mrf_energy(unary, ctx, labels.float())
  with pytest.raises(RuntimeError):
    compute_terms.stereo_data_cost(np.zeros((3, 4), np.uint8), np.zeros((3, 5), np.uint8), 2)


def test_layer_labels_minimise_the_energy_on_a_chain(gpu):
  """GPU layers + GPU energy on a chain: the labelling of one ISGMR iteration (rho = 1) is the MAP
  one, so its energy equals the minimum over all labellings (enumerated with the oracle)."""
  torch = _torch()
  from mplayers_amd import compute_terms
  rng = np.random.default_rng(11)
  n, L, n_dir = 7, 3, 2
  unary = rng.standard_normal((1, 1, 1, n, L)).astype(np.float32)
  context = np.array([0.0, 0.6, 1.1], dtype=np.float32)
  edge = (0.2 + rng.random((n_dir, 1, 1, 1, n))).astype(np.float32)
  edge[1] = 0
  edge[1][:, :, :, :-1] = edge[0][:, :, :, 1:]
  out = gpu.gpu_forward("ISGMR", unary, context, edge, n_dir, 1, 1.0, training=False,
                        saving_label=True)
  labels = out["label_all"].reshape(1, 1, 1, n)
  dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
  got = compute_terms.mrf_energy(dev(unary.reshape(1, 1, n, L)), dev(context), dev(labels),
                                 dev(edge.reshape(n_dir, 1, 1, n)), n_dir).sum().item()
  every = np.array(list(itertools.product(range(L), repeat=n)), dtype=np.uint8).reshape(-1, 1, 1, n)
  best = terms_oracle.mrf_energy(unary.reshape(1, 1, n, L), context, every,
                                 edge.reshape(n_dir, 1, 1, n), n_dir).sum(axis=1).min()
  assert got == pytest.approx(best, abs=1e-5)


def test_compute_all_terms_from_image_files(gpu, tmp_path):
  """The reference-style surface on image files: PPM/PGM in, caller-allocated CPU tensors filled."""
  torch = _torch()
  from PIL import Image
  from mplayers_amd import compute_terms, energy_min
  left, right, _ = energy_min.synthetic_stereo_pair(24, 31, 6, seed=4)
  Image.fromarray(left).save(tmp_path / "imL.ppm")
  Image.fromarray(right).save(tmp_path / "imR.ppm")
  H, W, L = 24, 31, 6
  data_cost = torch.ones(H * W, L)
  rgb = torch.zeros(H * W, 3)
  h_cue = torch.zeros(1, H * (W - 1))
  v_cue = torch.zeros(1, (H - 1) * W)
  table = torch.zeros(L, L)
  compute_terms.compute_all_terms(str(tmp_path / "imL.ppm"), str(tmp_path / "imR.ppm"), "TL", 8, 2,
                                  2, H, W, 3, L, data_cost, rgb, h_cue, v_cue, table)
  bgr_l, bgr_r = left[:, :, ::-1], right[:, :, ::-1]
  assert (data_cost.view(H, W, L).numpy() == terms_oracle.compute_dsi(bgr_l, bgr_r, L)).all()
  assert (rgb.view(H, W, 3).numpy() == bgr_l.astype(np.float32)).all()
  want_h, want_v = terms_oracle.compute_cues(bgr_l, 8, 2)
  assert (h_cue.view(H, W - 1).numpy() == want_h).all()
  assert (v_cue.view(W, H - 1).numpy() == want_v).all()
  k = np.abs(np.arange(L)[:, None] - np.arange(L)[None, :])
  assert (table.numpy() == np.minimum(k, 2)).all()
  # grey-scale file and the MRFParams route
  Image.fromarray(left[:, :, 0]).save(tmp_path / "imL.pgm")
  Image.fromarray(right[:, :, 0]).save(tmp_path / "imR.pgm")
  param = compute_terms.MRFParams(str(tmp_path / "imL.pgm"), str(tmp_path / "imR.pgm"), "TQ", L, 0,
                                  0, 2)
  cost, rgb1, table1, param = compute_terms.compute_terms_py(param)
  assert (param.height, param.width, param.n_channels) == (H, W, 1)
  assert (cost.cpu().numpy() == terms_oracle.compute_dsi(left[:, :, 0], right[:, :, 0], L)).all()
  assert (rgb1.cpu().numpy()[:, :, 0] == left[:, :, 0]).all()
  assert (table1.cpu().numpy() == np.minimum(k * k, 4)).all()


def test_driver_runs_sgm_as_one_iteration(gpu, tmp_path):
  from mplayers_amd import energy_min
  res = energy_min.main(["--synthetic", "24", "32", "--mode", "SGM", "--n_dir", "8", "--n_iter", "5",
                         "--n_disp", "8", "--context", "TL", "--truncated", "2"])
  assert res["labels"].shape[0] == 1 and res["energy"].shape == (1, 2)


@pytest.mark.parametrize("mode,n_dir", [("TRWP", 4), ("ISGMR", 8), ("TRWP", 16)])
def test_energy_minimisation_driver(gpu, tmp_path, mode, n_dir):
  """End to end on a random-dot stereo pair: the layer's labelling has a far lower energy than the
  data term's own argmin, recovers the true disparity on most pixels, and the .mat file holds the
  reference's keys."""
  import scipy.io as scio
  from mplayers_amd import energy_min
  H, W, L, n_iter = 48, 64, 8, 6
  argv = ["--synthetic", str(H), str(W), "--mode", mode, "--n_dir", str(n_dir), "--n_iter",
          str(n_iter), "--n_disp", str(L), "--context", "TL", "--truncated", "2", "--p_weight", "10",
          "--enable_saving_label", "--save_dir", str(tmp_path)]
  res = energy_min.main(argv)
  energy = res["energy"].cpu().numpy()
  labels = res["labels"].cpu().numpy()
  assert energy.shape == (n_iter, 2) and labels.shape == (n_iter, H, W)
  # the driver's energies are those of the oracle for the saved labellings
  left, right, disparity = energy_min.synthetic_stereo_pair(H, W, L)
  unary = terms_oracle.compute_dsi(left, right, L)
  k = np.arange(L)
  table = 10.0 * np.minimum(k, 2)
  want = terms_oracle.mrf_energy(unary[None], table.astype(np.float32), labels[:, None], None, n_dir)
  np.testing.assert_allclose(energy, want, rtol=1e-12)
  data_only = unary.argmin(axis=2).astype(np.uint8)
  base = terms_oracle.mrf_energy(unary[None], table.astype(np.float32), data_only[None, None], None,
                                 n_dir).sum()
  assert energy[-1].sum() < 0.8 * base
  inside = np.arange(W)[None, :] - disparity >= 0
  assert (labels[-1][inside] == disparity[inside]).mean() > 0.9
  mat = scio.loadmat(res["file_path"])
  for key in ("n_iter", "n_dir", "rho", "p_func", "n_disp", "p_weight", "trunct", "min_a_dir",
              "unary", "label_context", "seg_all", "energy"):
    assert key in mat
  assert mat["seg_all"].shape == (H, W, n_iter) and mat["seg_all"].dtype == np.uint8
  assert mat["unary"].shape == (H, W, L) and mat["label_context"].shape == (L, L, n_dir)
  assert (mat["seg_all"][:, :, -1] == labels[-1]).all()
  # a second run finds the file and does nothing, as the reference's driver does
  assert energy_min.main(argv) is None


def test_driver_declares_a_wide_quadratic_table_dense(gpu):
  """The module looks at a fixed table on the host and declares a dense one to the library, whose
  launches then put several wavefronts on a chain; the labels, energies and costs are those of the
  same run with one wavefront per chain, bit for bit."""
  from mplayers_amd import _lib, energy_min
  argv = ["--synthetic", "20", "44", "--mode", "TRWP", "--n_dir", "4", "--n_iter", "4", "--n_disp",
          "96", "--context", "TQ", "--truncated", "50", "--p_weight", "1"]
  k = np.arange(96, dtype=np.float32)
  assert _lib.table_is_dense(np.minimum(k * k, 2500)) and not _lib.table_is_dense(np.minimum(k, 50))
  res = energy_min.main(argv)
  _lib.set_option(_lib.OPT_DENSE_SPLIT_WAVES, 1)
  try:
    one = energy_min.main(argv)
  finally:
    _lib.set_option(_lib.OPT_DENSE_SPLIT_WAVES, 0)
  assert (res["labels"].cpu().numpy() == one["labels"].cpu().numpy()).all()
  assert (res["energy"].cpu().numpy() == one["energy"].cpu().numpy()).all()
  a, b = res["cost_final"].cpu().numpy(), one["cost_final"].cpu().numpy()
  assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
  assert len(np.unique(res["labels"][-1].cpu().numpy())) > 1
