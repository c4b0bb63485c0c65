"""Dense 1-D tables with more than 64 labels (learned tables, untruncated ones): the O(L^2) scan
of TRWP_forward.cu:127-153 against the oracle, and the launches that MPL_F_DENSE_TABLE splits over
several wavefronts per chain against the one-wavefront scan: the same bits for every count."""
import zlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _inputs(mode, n_dir, B, H, W, L, seed=0):
  rng = np.random.default_rng(zlib.crc32(repr((mode, n_dir, B, H, W, L, seed)).encode()))
  unary = (rng.random((B, 1, H, W, L)) * 3).astype(np.float32)
  ctx = np.concatenate([[0], rng.random(L - 1)]).astype(np.float32)
  ew = (0.1 + 0.9 * rng.random((n_dir, B, 1, H, W))).astype(np.float32)
  if seed == 1:
    ew[0, :, :, :, 2] = -0.5  # negative weights take the same scan
  return unary, ctx, ew


def _forward(gpu, mode, unary, ctx, ew, n_dir, n_iter, rho, training, flags, waves=0, **kw):
  from mplayers_amd import _lib
  _lib.set_option(_lib.OPT_DENSE_SPLIT_WAVES, waves)
  try:
    return _forward_flags(gpu, mode, unary, ctx, ew, n_dir, n_iter, rho, training, flags, **kw)
  finally:
    _lib.set_option(_lib.OPT_DENSE_SPLIT_WAVES, 0)


def _forward_flags(gpu, mode, unary, ctx, ew, n_dir, n_iter, rho, training, flags, msg_uninit=False):
  """gpu_forward of tests/_gpu_util.py with per-call flags."""
  import torch
  from mplayers_amd import lib_stereo
  t = gpu._t
  u = t(unary)
  b, cv, h, w, L = u.shape
  c, e = t(ctx), t(ew)
  fill = (lambda *s, **k: torch.full(s, float("nan"), device=gpu.DEV)) if msg_uninit else u.new_zeros
  msg = fill(n_dir, b, cv, h, w, L)
  cost = u.new_zeros(b, cv, h, w, L)
  scratch = u.new_zeros(b, cv, h, w, L)
  u8 = dict(dtype=torch.uint8)
  imin = u.new_zeros(n_iter, n_dir, b, cv, h, w, L, **u8) if training else torch.empty(0, **u8)
  inorm = u.new_zeros(n_iter, n_dir, b, cv, h, w, **u8) if training else torch.empty(0, **u8)
  label = u.new_zeros(n_iter, b, cv, h, w, **u8)
  if mode == "TRWP":
    lib_stereo.TRWP.forward(rho, n_iter, 0, u, c, e, msg, cost, imin, inorm, scratch, label,
                            msg_uninit=msg_uninit, flags=flags)
  else:
    tmp = fill(n_dir, b, cv, h, w, L)
    lib_stereo.ISGMR.forward(0, rho, n_iter, 0, u, c, e, msg, cost, imin, inorm, scratch, tmp, label,
                             msg_uninit=msg_uninit, flags=flags)
  torch.cuda.synchronize()
  return dict(msg=msg.cpu().numpy(), cost_final=cost.cpu().numpy(), label_all=label.cpu().numpy(),
              msg_min_index=imin.cpu().numpy(), msg_norm_index=inorm.cpu().numpy())


CASES = [
    # mode, n_dir, B, H, W, L
    ("TRWP", 4, 1, 6, 7, 65), ("ISGMR", 4, 1, 5, 6, 65), ("TRWP", 8, 2, 5, 6, 130),
    ("ISGMR", 8, 1, 6, 5, 130), ("TRWP", 4, 1, 7, 9, 192), ("ISGMR", 4, 2, 5, 7, 192),
    ("TRWP", 4, 1, 5, 5, 256), ("ISGMR", 16, 1, 6, 6, 256), ("TRWP", 4, 1, 6, 6, 97),
]


@pytest.mark.parametrize("mode,n_dir,B,H,W,L", CASES)
@pytest.mark.parametrize("training", [True, False])
def test_dense_scan_matches_oracle_and_split_scan_matches_it_bitwise(gpu, oracle, mode, n_dir, B, H,
                                                                     W, L, training):
  from mplayers_amd import _lib
  unary, ctx, ew = _inputs(mode, n_dir, B, H, W, L)
  rho = 0.5 if mode == "TRWP" else 1.0
  n_iter = 2
  print("case", mode, n_dir, B, H, W, L, training, flush=True)
  ref = oracle.forward(mode, unary, ctx, ew, n_dir, n_iter, rho, training=training,
                       saving_label=True, want_gaps=True)
  one = _forward(gpu, mode, unary, ctx, ew, n_dir, n_iter, rho, training, 0)
  gpu.assert_values_close(one["msg"], ref["msg"], what="msg", belief=ref["cost_final"])
  gpu.assert_values_close(one["cost_final"], ref["cost_final"], what="cost_final")
  tol = 2e-5 * max(1.0, float(np.abs(ref["cost_final"]).max()))
  if training:
    gpu.assert_indices_match_off_ties(one["msg_min_index"], ref["msg_min_index"], ref["gap_min"],
                                      tol, "msg_min_index")
    gpu.assert_indices_match_off_ties(one["msg_norm_index"], ref["msg_norm_index"],
                                      ref["gap_norm"], tol, "msg_norm_index")
  gpu.assert_labels_match_off_ties(one["label_all"], ref["label_all"], ref["gap_label"], tol)
  for waves in (0, 2, 3, 5, 8):
    got = _forward(gpu, mode, unary, ctx, ew, n_dir, n_iter, rho, training, _lib.F_DENSE_TABLE,
                   waves=waves)
    for k in ("msg", "cost_final", "label_all", "msg_min_index", "msg_norm_index"):
      assert np.array_equal(got[k], one[k]), (k, waves)


@pytest.mark.parametrize("mode", ["TRWP", "ISGMR"])
def test_split_scan_with_negative_weights_and_undefined_messages(gpu, mode):
  from mplayers_amd import _lib
  unary, ctx, ew = _inputs(mode, 4, 1, 6, 8, 192, seed=1)
  rho = 0.5 if mode == "TRWP" else 1.0
  one = _forward(gpu, mode, unary, ctx, ew, 4, 3, rho, True, 0)
  for waves in (0, 4):
    got = _forward(gpu, mode, unary, ctx, ew, 4, 3, rho, True, _lib.F_DENSE_TABLE, waves=waves,
                   msg_uninit=True)
    for k in ("msg", "cost_final", "label_all", "msg_min_index", "msg_norm_index"):
      assert np.array_equal(got[k], one[k]), (k, waves)


def test_flag_changes_nothing_for_a_band_table(gpu):
  """A truncated linear table under the flag: the dense scan gives the band scan's bits."""
  from mplayers_amd import _lib
  rng = np.random.default_rng(4)
  L, n_dir = 96, 4
  unary = (rng.random((1, 1, 6, 9, L)) * 3).astype(np.float32)
  ctx = (0.25 * np.minimum(np.arange(L), 2)).astype(np.float32)
  ew = (0.1 + 0.9 * rng.random((n_dir, 1, 1, 6, 9))).astype(np.float32)
  for mode, rho in (("TRWP", 0.5), ("ISGMR", 1.0)):
    a = _forward(gpu, mode, unary, ctx, ew, n_dir, 2, rho, True, 0)
    b = _forward(gpu, mode, unary, ctx, ew, n_dir, 2, rho, True, _lib.F_DENSE_TABLE)
    for k in ("msg", "cost_final", "label_all", "msg_min_index", "msg_norm_index"):
      if not np.array_equal(a[k], b[k]):
        a2 = _forward(gpu, mode, unary, ctx, ew, n_dir, 2, rho, True, 0)
        b2 = _forward(gpu, mode, unary, ctx, ew, n_dir, 2, rho, True, _lib.F_DENSE_TABLE)
        where = np.argwhere(a[k] != b[k])
        raise AssertionError((mode, k, "band run repeats itself", np.array_equal(a[k], a2[k]),
                              "dense run repeats itself", np.array_equal(b[k], b2[k]),
                              "second runs agree", np.array_equal(a2[k], b2[k]),
                              len(where), where[:4].tolist(),
                              float(np.abs(a[k].astype(np.float64) - b[k]).max())))


def test_flag_on_a_wide_truncated_linear_table(gpu, oracle):
  """A truncated linear table of more than 32 entries takes the O(L) label scan without the flag and
  the dense step in the launches that the flag splits.  The scan picks its candidates from
  products t * slope, so where sums round the two may differ in the last bits: both are held to the
  oracle's values.  Where nothing rounds the bits are the same: ISGMR on an integer-valued problem
  (TRWP halves the message of the pixel before at every step of a chain, so its sums round from some
  twenty pixels on whatever the inputs)."""
  from mplayers_amd import _lib
  rng = np.random.default_rng(11)
  L, n_dir, H, W = 128, 4, 5, 37
  ew = (0.1 + 0.9 * rng.random((n_dir, 1, 1, H, W))).astype(np.float32)
  unary = (rng.random((1, 1, H, W, L)) * 3).astype(np.float32)
  ctx = (0.05 * np.minimum(np.arange(L), 40)).astype(np.float32)
  for mode, rho in (("TRWP", 0.5), ("ISGMR", 1.0)):
    ref = oracle.forward(mode, unary, ctx, ew, n_dir, 2, rho, training=True, want_gaps=True)
    for flags in (0, _lib.F_DENSE_TABLE):
      got = _forward(gpu, mode, unary, ctx, ew, n_dir, 2, rho, True, flags)
      gpu.assert_values_close(got["msg"], ref["msg"], what="msg", belief=ref["cost_final"])
      gpu.assert_values_close(got["cost_final"], ref["cost_final"], what="cost_final")
  unary_i = rng.integers(0, 60, (1, 1, H, W, L)).astype(np.float32)
  ctx_i = (2.0 * np.minimum(np.arange(L), 40)).astype(np.float32)
  ones = np.ones_like(ew)
  a = _forward(gpu, "ISGMR", unary_i, ctx_i, ones, n_dir, 2, 1.0, True, 0)
  b = _forward(gpu, "ISGMR", unary_i, ctx_i, ones, n_dir, 2, 1.0, True, _lib.F_DENSE_TABLE)
  for k in ("msg", "cost_final", "label_all", "msg_min_index", "msg_norm_index"):
    assert np.array_equal(a[k], b[k]), k


def test_split_option_is_validated(gpu):
  from mplayers_amd import _lib
  assert _lib.load().mpl_set_option(_lib.OPT_DENSE_SPLIT_WAVES, 9) != 0


def test_module_asks_once_whether_a_fixed_table_is_dense(gpu):
  """MPModule with a table that is not being trained: above 64 labels it asks the library's rule
  once per table and declares a dense one; a band table, a short table and an explicit
  args.mpnet_dense_table are left alone, and a table written to is asked about again."""
  import argparse
  import torch
  from mplayers_amd.MP_module import MPModule
  B, H, W, n_dir = 1, 6, 9, 4

  def module_for(L, table, **extra):
    args = argparse.Namespace(n_classes=L, mpnet_n_dirs=n_dir, mpnet_max_iter=2, mpnet_term_weight=1,
                              mpnet_smoothness_train=None, mpnet_mrf_mode="TRWP", **extra)
    m = MPModule(args, enable_create_label_context=False).eval()
    m.set_label_context(table.cuda(), None, None)
    return m

  k96 = torch.arange(96, dtype=torch.float32)
  unary = torch.rand(B, 1, 96, H, W, generator=torch.Generator().manual_seed(1)).cuda()
  wide = module_for(96, (k96 * k96).clamp(max=2500.) * 0.01)
  cost_wide = wide(unary)[0]
  assert wide.args.dense_table is True
  band = module_for(96, k96.clamp(max=3.) * 0.3)
  band(unary)
  assert band.args.dense_table is False
  # the same dense table with the declaration switched off: the same bits
  off = module_for(96, (k96 * k96).clamp(max=2500.) * 0.01, mpnet_dense_table=False)
  assert torch.equal(off(unary)[0], cost_wide) and off.args.dense_table is False
  # a table that is written to is looked at again
  band.label_context.copy_((k96 * k96).clamp(max=2500.) * 0.01)
  assert torch.equal(band(unary)[0], cost_wide) and band.args.dense_table is True
  k40 = torch.arange(40, dtype=torch.float32)
  short = module_for(40, k40 * k40 * 0.01)
  short(unary[:, :, :40].contiguous())
  assert short.args.dense_table is False


@pytest.mark.parametrize("mode", ["TRWP", "ISGMR"])
@pytest.mark.parametrize("pair", [0, 2])
def test_split_scans_at_the_measured_size(gpu, oracle, mode, pair):
  """384 x 1248 pixels, 192 labels, a dense table declared dense: the launches of the size whose
  rate is reported (four wavefronts per chain on the 384 rows, two on the 1248 columns for TRWP,
  one for ISGMR's launch of all directions).  Zero edge weights switch the other pair of directions
  off, so single rows / columns are two-direction problems on a 1 x n image for the oracle;
  with and without argmin labels."""
  import torch
  from mplayers_amd import _lib, lib_stereo
  H, W, L, n_dir, n_iter = 384, 1248, 192, 4, 2
  rho = 0.5 if mode == "TRWP" else 1.0
  dev = "cuda:0"
  g = torch.Generator(device=dev)
  g.manual_seed(5)
  unary = torch.rand(1, 1, H, W, L, device=dev, generator=g) * 3
  ew = 0.1 + 0.9 * torch.rand(n_dir, 1, 1, H, W, device=dev, generator=g)
  for d in range(n_dir):
    if d not in (pair, pair + 1):
      ew[d] = 0
  ctx = torch.cat([torch.zeros(1, device=dev), torch.rand(L - 1, device=dev, generator=g)])
  empty = torch.empty(0, dtype=torch.uint8)
  runs = {}
  for training in (True, False):
    msg = torch.zeros(n_dir, 1, 1, H, W, L, device=dev)
    cost = torch.zeros(1, 1, H, W, L, device=dev)
    scratch = torch.zeros(1, 1, H, W, L, device=dev)
    imin = torch.zeros(n_iter, n_dir, 1, 1, H, W, L, dtype=torch.uint8, device=dev) if training else empty
    inorm = torch.zeros(n_iter, n_dir, 1, 1, H, W, dtype=torch.uint8, device=dev) if training else empty
    print("measured size", mode, pair, training, flush=True)
    if mode == "TRWP":
      lib_stereo.TRWP.forward(rho, n_iter, 0, unary, ctx, ew, msg, cost, imin, inorm, scratch, empty,
                              flags=_lib.F_DENSE_TABLE)
    else:
      lib_stereo.ISGMR.forward(0, rho, n_iter, 0, unary, ctx, ew, msg, cost, imin, inorm, scratch,
                               torch.zeros_like(msg), empty, flags=_lib.F_DENSE_TABLE)
    torch.cuda.synchronize()
    runs[training] = (msg, cost, imin, inorm)
  ctx_np = ctx.cpu().numpy()
  for k in ([0, 191, 383] if pair == 0 else [0, 700, 1247]):
    if pair == 0:
      hh, ww = torch.full((W,), k, device=dev), torch.arange(W, device=dev)
    else:
      hh, ww = torch.arange(H, device=dev), torch.full((H,), k, device=dev)
    un = unary[:, :, hh, ww, :].cpu().numpy()[:, :, None]
    en = ew[[pair, pair + 1]][:, :, :, hh, ww].cpu().numpy()[:, :, :, None]
    ref = oracle.forward(mode, un, ctx_np, en, 2, n_iter, rho, want_gaps=True)
    belief = ref["cost_final"]
    tol = 1e-5 * max(1.0, float(np.abs(belief).max()))
    for training, (msg, cost, imin, inorm) in runs.items():
      what = "chain %d, %s" % (k, "training" if training else "inference")
      gpu.assert_values_close(msg[[pair, pair + 1]][:, :, :, hh, ww, :].cpu().numpy()[:, :, :, None],
                              ref["msg"], what="msg, " + what, belief=belief)
      gpu.assert_values_close(cost[:, :, hh, ww, :].cpu().numpy()[:, :, None], ref["cost_final"],
                              what="cost, " + what)
      if training:
        gi = imin[:, [pair, pair + 1]][:, :, :, :, hh, ww, :].cpu().numpy()[:, :, :, :, None]
        gn = inorm[:, [pair, pair + 1]][:, :, :, :, hh, ww].cpu().numpy()[:, :, :, :, None]
        gpu.assert_indices_match_off_ties(gi, ref["msg_min_index"], ref["gap_min"], 4 * tol, "min idx")
        gpu.assert_indices_match_off_ties(gn, ref["msg_norm_index"], ref["gap_norm"], 4 * tol, "norm idx")
