"""CPU-side checks: the C-ABI library loads and exports what include/mplayers_amd.h declares, the
host-side argument validation answers without touching a GPU, and the Python surface mirrors the
reference's (pytorch/MP_module.py, utils/label_context.py)."""
import argparse
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
  text = open(os.path.join(ROOT, "include", "mplayers_amd.h")).read()
  text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
  return sorted(set(re.findall(r"\b(mpl_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
  from mplayers_amd import _lib
  lib = _lib.load()
  names = _declared_functions()
  assert {"mpl_trwp_forward", "mpl_trwp_backward", "mpl_isgmr_forward", "mpl_isgmr_backward"} <= set(names)
  for name in names:
    assert hasattr(lib, name), name
  assert sorted(_lib.SYMBOLS) == names
  assert lib.mpl_version() // 100 == 2


def test_chain_counts_match_reference_tree_counts(oracle):
  from mplayers_amd import _lib
  lib = _lib.load()
  for H, W in [(5, 7), (8, 3), (2, 6), (6, 2), (129, 129), (1500, 2000)]:
    for d in range(16):
      assert lib.mpl_n_chains(d, H, W) == oracle.n_trees(d, H, W), (H, W, d)
  assert lib.mpl_n_chains(16, 4, 4) == -1


def test_table_kind_on_the_host():
  """mpl_table_is_dense: the tables the band and label scans take are not dense, the others are."""
  from mplayers_amd import _lib
  k = np.arange(96, dtype=np.float32)
  rng = np.random.default_rng(3)
  not_dense = {
      "potts": np.minimum(k, 1) * 0.7, "tl2": np.minimum(k, 2) * 0.25, "tq5": np.minimum(k * k, 25) * 0.1,
      "band of 32": np.minimum(k, 32) ** 1.5, "linear": k * 10, "tl95": np.minimum(k, 95) * 10,
      "constant": np.full(96, 0.3), "bump": np.concatenate([[0.3, 0.1, 0.4], np.full(93, 0.5)]),
      "one label": np.zeros(1)}
  dense = {
      "band of 33": np.minimum(k, 33) ** 1.5, "tq40": np.minimum(k * k, 1600) * 0.01,
      "quadratic": k * k, "random": np.concatenate([[0], rng.random(95)]),
      "above its tail": np.concatenate([[0, 2.0], np.ones(94)]),
      "linear from 1": 1 + k, "nan tail": np.concatenate([np.minimum(k[:95], 2), [np.nan]])}
  for name, t in not_dense.items():
    assert _lib.table_is_dense(t) is False, name
  for name, t in dense.items():
    assert _lib.table_is_dense(t) is True, name
  assert _lib.table_is_dense(torch.tensor(dense["tq40"])) is True
  assert _lib.load().mpl_table_is_dense(None, 4) == -1
  with pytest.raises(ValueError):
    _lib.table_is_dense(np.zeros(0))


def test_shape_validation_answers_before_any_launch():
  from mplayers_amd import _lib
  lib = _lib.load()
  one = ctypes.c_void_p(8)  # never dereferenced: validation fails first

  def fwd(shape, n_iter=1):
    return lib.mpl_trwp_forward(shape, flags, 0.5, n_iter, 0, one, one, one, one, one, None, None,
                                one, None, None)

  flags = 0
  assert fwd(_lib.Shape(4, 1, 4, 4, 257, 0)) == -1
  assert b"n_disp" in lib.mpl_last_error()
  assert fwd(_lib.Shape(3, 1, 4, 4, 8, 0)) == -1
  assert b"n_dir" in lib.mpl_last_error()
  assert fwd(_lib.Shape(4, 0, 4, 4, 8, 0)) == -1
  assert fwd(_lib.Shape(4, 1, 4, 4, 65, 1)) == -1
  assert b"2-D context" in lib.mpl_last_error()
  assert fwd(_lib.Shape(4, 1, 4, 4, 8, 0), n_iter=0) == -1
  assert fwd(_lib.Shape(4, 1, 40000, 40000, 8, 0)) == -1  # one image above 4 GiB
  assert lib.mpl_isgmr_backward(_lib.Shape(4, 1, 4, 4, 8, 0), 0, 0, 1.0, 1, one, one, one, one,
                                one, one, one, one, None, None, None, None) == -1
  assert b"null" in lib.mpl_last_error()
  # per-call flags: unknown bits and contradictory choices are refused
  flags = 0x8000
  assert fwd(_lib.Shape(4, 1, 4, 4, 8, 0)) == -1
  assert b"flag" in lib.mpl_last_error()
  flags = _lib.F_PACKED_OFF | _lib.F_PACKED_ALWAYS
  assert fwd(_lib.Shape(4, 1, 4, 4, 8, 0)) == -1
  assert b"exclude" in lib.mpl_last_error()


def test_operator_namespaces_are_shared():
  """One extension backs the reference's four import names (lib_stereo / lib_seg . TRWP / ISGMR)."""
  from mplayers_amd import lib_seg, lib_stereo
  assert lib_seg.TRWP is lib_stereo.TRWP and lib_seg.ISGMR is lib_stereo.ISGMR


def _args(**kw):
  base = dict(mpnet_mrf_mode="TRWP", mpnet_max_iter=5, mpnet_n_dirs=4, n_classes=21,
              mpnet_term_weight=2.0, mpnet_smoothness_train="", mpnet_smoothness_mode="Potts",
              mpnet_smoothness_trunct_value=-1, mpnet_smoothness_trunct_loc=-1, mpnet_diag_value=0,
              enable_symmetric=True, enable_cuda=False)
  base.update(kw)
  return argparse.Namespace(**base)


def test_module_sets_the_argument_namespace_like_the_reference():
  """MP_module.py:170-176: rho 0.5 for TRWP and 1 otherwise, the SGM / segmentation flags."""
  from mplayers_amd import MPModule
  a = _args()
  m = MPModule(a, enable_create_label_context=True, enable_saving_label=True)
  assert a.rho == 0.5 and a.enable_saving_label and not a.enable_min_a_dir
  assert a.enable_seg and not a.enable_sgm
  lc, loc, diag = m.get_label_context()
  assert lc.shape == (21, 21) and not lc.requires_grad
  assert torch.equal(lc, 2.0 * (1 - torch.eye(21)))
  a = _args(mpnet_mrf_mode="SGM", n_classes=16)
  MPModule(a)
  assert a.rho == 1 and a.enable_sgm and not a.enable_seg


def test_label_context_builders():
  """utils/label_context.py:6-90."""
  from mplayers_amd.label_context import create_label_context
  lc, loc, diag = create_label_context(_args(n_classes=8, mpnet_smoothness_mode="TL",
                                             mpnet_smoothness_trunct_value=3, mpnet_term_weight=0.5))
  assert torch.equal(lc, 0.5 * torch.tensor([0, 1, 2, 3, 3, 3, 3, 3.]))
  assert list(loc) == list(range(1, 8)) and list(diag) == [0]
  lc, _, _ = create_label_context(_args(n_classes=6, mpnet_smoothness_mode="TQ",
                                        mpnet_smoothness_trunct_value=5,
                                        mpnet_smoothness_trunct_loc=3, mpnet_term_weight=1.0))
  assert torch.equal(lc, torch.tensor([0, 1, 4, 5, 5, 5.]))
  lc, _, _ = create_label_context(_args(n_classes=5, mpnet_smoothness_mode="NPotts",
                                        mpnet_term_weight=1.0))
  assert torch.equal(lc, torch.tensor([-1, 0, 0, 0, 0.]))
  lc, _, _ = create_label_context(_args(n_classes=5, mpnet_smoothness_mode="Potts",
                                        mpnet_smoothness_train="sigmoid", mpnet_term_weight=1.0))
  assert torch.equal(lc.detach(), torch.zeros(5)) and lc.requires_grad
  # segmentation tables: upper triangle only unless symmetric
  lc, loc, diag = create_label_context(_args(mpnet_smoothness_mode="TL", enable_symmetric=False,
                                             mpnet_smoothness_trunct_value=2, mpnet_term_weight=1.0),
                                       enable_symmetric=False)
  i, j = np.triu_indices(21, k=1)
  expect = np.zeros((21, 21), dtype=np.float32)
  expect[i, j] = np.minimum(j - i, 2)
  assert np.array_equal(lc.numpy(), expect)
  assert np.array_equal(loc[0], i) and np.array_equal(loc[1], j)
  # a positive truncation location truncates nothing for the 2-D table (reference quirk)
  lc, _, _ = create_label_context(_args(mpnet_smoothness_mode="TL", mpnet_smoothness_trunct_value=2,
                                        mpnet_smoothness_trunct_loc=4, mpnet_term_weight=1.0),
                                  enable_symmetric=True)
  assert float(lc.max()) == 20.0


def test_module_reparameterisation_matches_reference_formulas():
  """sigmoid / softmax training modes of MP_module.py:208-220 (no kernel involved)."""
  from mplayers_amd import MPModule
  a = _args(n_classes=6, mpnet_smoothness_mode="TL", mpnet_smoothness_train="sigmoid",
            mpnet_term_weight=3.0, mpnet_diag_value=0.25)
  m = MPModule(a, enable_create_label_context=True)
  raw = m.label_context.detach().clone()
  eff = m._effective_label_context().detach()
  assert torch.allclose(eff[1:], 2 * 3.0 * torch.sigmoid(raw[1:]))
  assert float(eff[0]) == 0.25
  a = _args(n_classes=6, mpnet_smoothness_mode="TL", mpnet_smoothness_train="softmax",
            mpnet_term_weight=1.0, mpnet_diag_value=0.0)
  m = MPModule(a, enable_create_label_context=True)
  raw = m.label_context.detach().clone()
  eff = m._effective_label_context().detach()
  sm = torch.softmax(raw[1:], 0)
  assert torch.allclose(eff[1:], sm * raw[1:].max() / sm.max())


def test_synthetic_configs_are_seeded_and_shaped():
  from mplayers_amd import synthetic
  a = synthetic.make_config("C5", scale=0.02)
  b = synthetic.make_config("C5", scale=0.02)
  assert torch.equal(a["unary"], b["unary"]) and torch.equal(a["edge_weights"], b["edge_weights"])
  assert a["unary"].shape == (1, 1, 30, 40, 192) and a["edge_weights"].shape == (8, 1, 1, 30, 40)
  assert torch.allclose(a["context"][:5], torch.tensor([0, 0.3, 0.6, 0.9, 0.9])) and bool((a["context"][3:] == a["context"][3]).all())
  ew = a["edge_weights"]
  assert float(ew[0, 0, 0, :, 0].min()) == 1.0 and float(ew[1, 0, 0, :, -1].min()) == 1.0
  assert 0 < float(ew.min()) and float(ew.max()) <= 1.0
  c4 = synthetic.make_config("C4", scale=0.1, mode="ISGMR")
  assert c4["rho"] == 1.0 and c4["context"].shape == (21, 21)
  assert torch.equal(torch.tril(c4["context"]), torch.zeros(21, 21))


def test_product_never_touches_the_oracle_or_scratch_files():
  """The package, the bench and the entry points may not import anything from oracle/ (test
  infrastructure; bench.py's cpu_baseline leg and smoke() are the two allowed users) nor read the
  builder's scratch folder."""
  import os
  import re
  root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
  pkg = os.path.join(root, "mplayers_amd")
  offenders = []
  for dirpath, _, files in os.walk(pkg):
    for name in files:
      if not name.endswith((".py", ".hip", ".h", ".cpp")):
        continue
      text = open(os.path.join(dirpath, name)).read()
      if re.search(r"^\s*(from|import)\s+oracle\b", text, re.M) or re.search(r"(^|[\"'/\s])_work/", text):
        offenders.append(os.path.relpath(os.path.join(dirpath, name), root))
  assert offenders == []
  bench = open(os.path.join(root, "bench.py")).read()
  uses = [m.start() for m in re.finditer(r"from oracle|import oracle", bench)]
  body = bench[bench.index("def cpu_baseline"):]
  end = body.index("\ndef ", 1)
  assert all(bench.index("def cpu_baseline") <= u < bench.index("def cpu_baseline") + end for u in uses)
  assert not re.search(r"(^|[\"'/\s])_work/", bench)


def test_probe_library_is_separate_and_validates():
  """The measurement probes live in a library of their own (csrc/mp_probe.h): the product
  library exports none of them, and they answer bad arguments on the host."""
  import ctypes
  from mplayers_amd import _lib, _probe
  product = _lib.load()
  for name in ("mpl_probe_copy", "mpl_probe_issue", "mpl_selftest_wave_ops", "mplp_copy",
               "mplp_issue", "mplp_selftest_wave_ops"):
    assert not hasattr(product, name), name
  lib = _probe.load()
  text = open(os.path.join(ROOT, "mplayers_amd", "csrc", "mp_probe.h")).read()
  text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
  for name in sorted(set(re.findall(r"\b(mplp_[a-z0-9_]+)\s*\(", text))):
    assert hasattr(lib, name), name
  null = ctypes.c_void_p(None)
  one = ctypes.c_void_p(16)   # never dereferenced: every call below fails validation first
  assert lib.mplp_copy(0, 2, 2, one, one, 4, 4, 8, null) != 0
  assert lib.mplp_copy(0, 1, 1, one, one, 4, 4, 6, null) != 0
  assert lib.mplp_issue(null, 64, null) != 0
  assert lib.mplp_issue(one, 1, null) != 0
  assert lib.mplp_issue_count() > 1 and lib.mplp_issue_slots(0) == 0
  assert lib.mplp_issue_slots(lib.mplp_issue_count()) == -1
  assert lib.mplp_issue_name(1) != b"" and lib.mplp_issue_name(-1) == b""
  assert lib.mplp_selftest_wave_ops(null, null) != 0
  assert b"" != lib.mplp_last_error()


def test_new_entry_points_validate_before_launching():
  """Terms and transpose entry points answer bad arguments with MPL_EINVAL on the host."""
  import ctypes
  from mplayers_amd import _lib
  lib = _lib.load()
  null = ctypes.c_void_p(None)
  one = ctypes.c_void_p(16)   # never dereferenced: every call below fails validation first
  assert lib.mpl_stereo_data_cost(null, one, 4, 4, 3, 8, 1, 0, 255, one, null) != 0
  assert lib.mpl_stereo_data_cost(one, one, 0, 4, 3, 8, 1, 0, 255, one, null) != 0
  assert lib.mpl_gradient_cues(null, 4, 4, 3, 8, ctypes.c_float(2), one, one, null) != 0
  assert lib.mpl_gradient_cues(one, 4, 4, 3, 8, ctypes.c_float(2), null, one, null) != 0
  shape = _lib.Shape(3, 1, 4, 4, 8, 0)      # odd direction count
  assert lib.mpl_mrf_energy(ctypes.byref(shape), 1, one, one, null, one, one, null) != 0
  shape = _lib.Shape(4, 1, 4, 4, 8, 0)
  assert lib.mpl_mrf_energy(ctypes.byref(shape), 1, one, one, null, null, one, null) != 0
  assert lib.mpl_mrf_energy(ctypes.byref(shape), 0, one, one, null, one, one, null) == 0  # nothing to do
  assert lib.mpl_transpose(null, one, 1, 4, 4, null) != 0
  assert lib.mpl_transpose(one, one, 1, -1, 4, null) != 0
  assert lib.mpl_transpose(one, one, 0, 4, 4, null) == 0                                  # empty
  assert b"" != lib.mpl_last_error()
