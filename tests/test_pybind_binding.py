"""The C++ boundary made real: the pybind11 modules of tests/binding/mpl_torch_binding.cpp (what a
maintainer of the reference puts in place of MPLayers/TRWP/TRWP.cpp:245-326 and
MPLayers/ISGMR/ISGMR.cpp:300-404) are built against libmplayers_hip.so and take the place of the
ctypes operators in the parity checks of the CPU-runnable and the segmentation-shaped
configurations."""
import importlib
import os
import sys
import types

import numpy as np
import pytest

BUILT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "binding", "_built")


def _load(pkg):
  """`from lib_stereo import TRWP, ISGMR` as pytorch/MP_module.py:4-8 does it, from the directory
  the modules were built into (without leaving it on sys.path)."""
  path = os.path.join(BUILT, pkg)
  assert os.path.exists(os.path.join(path, "TRWP.so")), \
      "pybind11 binding not built: python tests/binding/build_binding.py"
  import torch  # noqa: F401  (libtorch must be loaded before the extension modules)
  ns = types.SimpleNamespace()
  for name in ("TRWP", "ISGMR"):
    spec = importlib.util.spec_from_file_location(name, os.path.join(path, name + ".so"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    setattr(ns, name, mod)
  return ns


def test_binding_modules_load_and_take_cpu_tensors_like_the_reference():
  """CPU tensors run the reference's ForwardCPU semantics through the library's CPU entry points
  (bit-exact against a fixture of the reference's own compiled CPU code); a CPU backward is
  refused with the reference's message."""
  import torch
  for pkg in ("lib_stereo", "lib_seg"):
    ops = _load(pkg)
    for mod in (ops.TRWP, ops.ISGMR):
      assert callable(mod.forward) and callable(mod.backward)
  golden = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
  e8 = torch.empty(0, dtype=torch.uint8)
  for name, mod in (("refcpu_trwp_d8_l21.npz", _load("lib_seg").TRWP),
                    ("refcpu_isgmr_d4_l16.npz", _load("lib_stereo").ISGMR)):
    z = np.load(os.path.join(golden, name))
    u = torch.tensor(z["unary"])
    n_dir, n_iter, rho = int(z["n_dir"]), int(z["n_iter"]), float(z["rho"])
    msg = torch.zeros((n_dir,) + tuple(u.shape))
    cost, scratch = torch.zeros_like(u), torch.zeros_like(u)
    label = torch.zeros((n_iter,) + tuple(u.shape[:-1]), dtype=torch.uint8)
    if str(z["mode"]) == "TRWP":
      mod.forward(rho, n_iter, 0, u, torch.tensor(z["context"]), torch.empty(0), msg, cost, e8, e8,
                  scratch, label)
    else:
      mod.forward(0, rho, n_iter, 0, u, torch.tensor(z["context"]), torch.empty(0), msg, cost, e8,
                  e8, scratch, torch.zeros_like(msg), label)
    assert np.array_equal(msg.numpy(), z["msg"]) and np.array_equal(cost.numpy(), z["cost_final"])
    assert np.array_equal(label.numpy(), z["label_all"])
  ops = _load("lib_stereo")
  L = 4
  u = torch.zeros(1, 1, 2, 2, L)
  # a 1-D table alone is too short for the CPU path (one table per direction)
  with pytest.raises(RuntimeError, match="context"):
    ops.TRWP.forward(0.5, 1, 0, u, torch.zeros(L), torch.ones(4, 1, 1, 2, 2),
                     torch.zeros(4, 1, 1, 2, 2, L), torch.zeros_like(u), e8, e8,
                     torch.zeros_like(u), e8)
  idx = torch.zeros(1, 4, 1, 1, 2, 2, L, dtype=torch.uint8)
  with pytest.raises(RuntimeError, match="Does not support CPU backward"):
    ops.TRWP.backward(0.5, torch.zeros(L), torch.ones(4, 1, 1, 2, 2), u, idx, idx[..., 0].contiguous(),
                      torch.zeros_like(u), torch.zeros(L), torch.zeros(4, 1, 1, 2, 2),
                      torch.zeros(4, 1, 1, 2, 2, L), torch.zeros_like(u))
  # positional arguments only, in the reference's order: a wrong count is a TypeError
  with pytest.raises(TypeError):
    ops.ISGMR.forward(0.5, 1, 0, u)


@pytest.mark.gpu
@pytest.mark.parametrize("name,mode", [("C1", "ISGMR"), ("C4", "TRWP"), ("C4", "ISGMR")])
def test_configs_through_the_pybind_modules(gpu, oracle, name, mode):
  """The same oracle comparisons as tests/test_gpu_configs.py, with the compiled modules in
  place of mplayers_amd/ops.py: forward values, indices, labels; backward on the oracle's
  indices."""
  from mplayers_amd import synthetic
  ops = _load("lib_seg" if name == "C4" else "lib_stereo")
  cfg = synthetic.make_config(name, seed=0, mode=mode)
  unary, ctx, ew = cfg["unary"].numpy(), cfg["context"].numpy(), cfg["edge_weights"].numpy()
  n_dir, n_iter, rho = cfg["n_dir"], cfg["n_iter"], cfg["rho"]
  print("config", name, mode, unary.shape, flush=True)
  ref = oracle.forward(mode, unary, ctx, ew, n_dir, n_iter, rho, want_gaps=True, saving_label=True)
  got = gpu.gpu_forward(mode, unary, ctx, ew, n_dir, n_iter, rho, saving_label=True, ops=ops)
  gpu.assert_values_close(got["msg"], ref["msg"], what="msg", belief=ref["cost_final"])
  gpu.assert_values_close(got["cost_final"], ref["cost_final"], what="cost_final")
  tol = 2e-5 * max(1.0, float(np.abs(ref["cost_final"]).max()))
  gpu.assert_labels_match_off_ties(got["label_all"], ref["label_all"], ref["gap_label"], tol)
  gpu.assert_indices_match_off_ties(got["msg_min_index"], ref["msg_min_index"], ref["gap_min"],
                                    tol, "msg_min_index")
  gpu.assert_indices_match_off_ties(got["msg_norm_index"], ref["msg_norm_index"], ref["gap_norm"],
                                    tol, "msg_norm_index")
  dcost = synthetic.upstream_grad(cfg).numpy()
  r = oracle.backward(mode, ctx.astype(np.float64), ew.astype(np.float64), dcost.astype(np.float64),
                      ref["msg_min_index"], ref["msg_norm_index"], rho)
  g = gpu.gpu_backward(mode, ctx, ew, dcost, ref["msg_min_index"], ref["msg_norm_index"], rho,
                       ops=ops)
  for a, b, what in zip(g, r, ("dunary", "dcontext", "dedge_weights")):
    assert np.abs(a - b).max() <= 1e-4 * max(1.0, float(np.abs(b).max())), what
  # the ctypes operators give the same bits (same library underneath, same flags)
  same = gpu.gpu_forward(mode, unary, ctx, ew, n_dir, n_iter, rho, saving_label=True)
  for k in ("msg", "cost_final", "msg_min_index", "msg_norm_index", "label_all"):
    assert np.array_equal(got[k], same[k]), k


@pytest.mark.gpu
def test_pybind_modules_report_library_errors(gpu):
  import torch
  ops = _load("lib_stereo")
  L = 300  # more labels than uint8 indices can hold: the reference prints and returns zeros
  u = torch.zeros(1, 1, 2, 2, L, device="cuda")
  e8 = torch.empty(0, dtype=torch.uint8)
  with pytest.raises(RuntimeError, match="n_disp"):
    ops.TRWP.forward(0.5, 1, 0, u, torch.zeros(L, device="cuda"),
                     torch.ones(4, 1, 1, 2, 2, device="cuda"),
                     torch.zeros(4, 1, 1, 2, 2, L, device="cuda"), torch.zeros_like(u), e8, e8,
                     torch.zeros_like(u), e8)
  with pytest.raises(RuntimeError, match="contiguous"):
    ops.TRWP.forward(0.5, 1, 0, torch.zeros(1, 1, 2, 8, 2, device="cuda").transpose(3, 4),
                     torch.zeros(8, device="cuda"), torch.ones(4, 1, 1, 2, 2, device="cuda"),
                     torch.zeros(4, 1, 1, 2, 2, 8, device="cuda"),
                     torch.zeros(1, 1, 2, 2, 8, device="cuda"), e8, e8,
                     torch.zeros(1, 1, 2, 2, 8, device="cuda"), e8)
