"""GPU parity: the HIP kernels (called through the C ABI) against the CPU oracle.

Tolerances: messages and beliefs within 1e-5 relative (fp32); argmin indices and labels identical
except at ties within tolerance; bit-exact on integer-valued inputs where fp32 arithmetic is exact.
"""
import zlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_wave_primitives(gpu):
  import ctypes
  import torch
  from mplayers_amd import _probe
  out = torch.zeros(8, dtype=torch.int32, device="cuda")
  _probe.check(_probe.load().mplp_selftest_wave_ops(ctypes.c_void_p(out.data_ptr()), None),
               "selftest")
  torch.cuda.synchronize()
  out = out.cpu().tolist()
  assert out[0] == 1, "lanes failing: %08x %08x" % (out[2] & 0xffffffff, out[1] & 0xffffffff)


def _seed(*parts):
  return zlib.crc32(repr(parts).encode())


def _context(rng, kind, L):
  if kind == "tl2":
    return np.minimum(np.arange(L), 2).astype(np.float32) * 0.25
  if kind == "tl3":
    return np.minimum(np.arange(L), 3).astype(np.float32) * 0.3
  if kind == "tl4":
    return np.minimum(np.arange(L), 4).astype(np.float32) * 0.5
  if kind == "potts":
    c = np.ones(L, dtype=np.float32)
    c[0] = 0
    return c
  if kind == "tq":
    return np.minimum(np.arange(L) ** 2, 40).astype(np.float32) * 0.05
  if kind == "npotts":  # negative centre tap, constant elsewhere
    c = np.zeros(L, dtype=np.float32)
    c[0] = -1
    return c
  if kind == "bump":  # constant tail but c[0] is not the smallest tap
    c = np.full(L, 0.7, dtype=np.float32)
    c[0], c[1], c[2] = 0.3, 0.1, 0.5
    return c
  if kind == "dense1d":  # no constant tail at all
    return np.concatenate([[0], rng.random(L - 1)]).astype(np.float32)
  if kind == "dense2d":
    return np.triu(rng.random((L, L)), 1).astype(np.float32)
  raise KeyError(kind)


CASES = [
    # mode, n_dir, B, H, W, L, context kind, n_iter
    ("ISGMR", 4, 1, 5, 7, 16, "tl4", 2),
    ("TRWP", 4, 1, 5, 7, 16, "tl4", 2),
    ("TRWP", 4, 2, 6, 5, 21, "dense2d", 2),
    ("ISGMR", 8, 2, 6, 5, 21, "dense2d", 2),
    ("TRWP", 8, 1, 7, 9, 96, "tl2", 2),
    ("ISGMR", 8, 1, 7, 9, 192, "tl3", 2),
    ("TRWP", 8, 1, 6, 6, 192, "tl3", 2),
    ("ISGMR", 4, 1, 6, 6, 256, "tq", 2),
    ("TRWP", 4, 1, 5, 6, 65, "tl3", 2),
    ("ISGMR", 4, 1, 5, 6, 97, "potts", 2),
    ("TRWP", 4, 1, 5, 6, 130, "tq", 2),
    ("ISGMR", 4, 1, 4, 5, 200, "bump", 2),
    ("TRWP", 4, 1, 4, 5, 33, "npotts", 2),
    ("ISGMR", 4, 1, 5, 4, 48, "dense1d", 2),
    ("TRWP", 8, 1, 5, 4, 70, "dense1d", 1),
    ("ISGMR", 16, 1, 9, 8, 12, "tl2", 2),
    ("TRWP", 16, 1, 8, 9, 12, "dense1d", 2),
    ("ISGMR", 4, 1, 1, 9, 8, "tl2", 2),
    ("TRWP", 4, 1, 9, 1, 8, "tl2", 2),
    ("TRWP", 8, 3, 2, 2, 5, "tl2", 3),
    ("ISGMR", 2, 1, 3, 40, 3, "potts", 3),
]


@pytest.mark.parametrize("mode,n_dir,B,H,W,L,kind,n_iter", CASES)
@pytest.mark.parametrize("training", [True, False])
def test_forward_matches_oracle(gpu, oracle, mode, n_dir, B, H, W, L, kind, n_iter, training):
  rng = np.random.default_rng(_seed(mode, n_dir, L, kind))
  rho = 0.5 if mode == "TRWP" else 1.0
  unary = rng.random((B, 1, H, W, L)).astype(np.float32) * 3
  ctx = _context(rng, kind, L)
  ew = (0.1 + 0.9 * rng.random((n_dir, B, 1, H, W))).astype(np.float32)
  print("case", mode, n_dir, B, H, W, L, kind, n_iter, training, flush=True)
  ref = oracle.forward(mode, unary, ctx, ew, n_dir, n_iter, rho, training=training,
                       saving_label=True, want_gaps=True)
  got = gpu.gpu_forward(mode, unary, ctx, ew, n_dir, n_iter, rho, training=training,
                        saving_label=True)
  gpu.assert_values_close(got["msg"], ref["msg"], what="msg", belief=ref["cost_final"])
  gpu.assert_values_close(got["cost_final"], ref["cost_final"], what="cost_final")
  tol = 2e-5 * max(1.0, float(np.abs(ref["cost_final"]).max()))
  if training:
    gpu.assert_indices_match_off_ties(got["msg_min_index"], ref["msg_min_index"], ref["gap_min"],
                                      tol, "msg_min_index")
    gpu.assert_indices_match_off_ties(got["msg_norm_index"], ref["msg_norm_index"],
                                      ref["gap_norm"], tol, "msg_norm_index")
  gpu.assert_labels_match_off_ties(got["label_all"], ref["label_all"], ref["gap_label"], tol)


@pytest.mark.parametrize("mode,n_dir,L,kind", [
    ("ISGMR", 8, 16, "int1d"), ("ISGMR", 4, 21, "int2d"), ("TRWP", 4, 70, "int1d"),
    ("ISGMR", 16, 130, "int_tl"), ("TRWP", 4, 21, "int2d"), ("ISGMR", 4, 192, "int_tl"),
])
def test_integer_inputs_are_bit_exact(gpu, oracle, mode, n_dir, L, kind):
  """Integer-valued inputs (the reference's own test inputs, pytorch/test_parallel_grad.py:
  102-110) make every fp32 operation exact and produce many exact ties: values, indices and
  labels must then be identical, tie rules included."""
  rng = np.random.default_rng(L * 31 + n_dir)
  B, H, W = 2, 6, 7
  rho = 0.5 if mode == "TRWP" else 1.0
  n_iter = 1 if mode == "TRWP" else 3  # rho = 0.5 halves the grid every sweep
  unary = rng.integers(0, 16, (B, 1, H, W, L)).astype(np.float32) * (4 if mode == "TRWP" else 1)
  if kind == "int2d":
    ctx = np.triu(rng.integers(0, 5, (L, L)), 1).astype(np.float32)
  elif kind == "int_tl":
    ctx = np.minimum(np.arange(L), 3).astype(np.float32) * 2
  else:
    ctx = np.concatenate([[0], rng.integers(0, 5, L - 1)]).astype(np.float32)
  if mode == "TRWP":
    ctx = ctx * 4
  ew = rng.integers(1, 4, (n_dir, B, 1, H, W)).astype(np.float32)
  print("case", mode, n_dir, L, kind, flush=True)
  ref = oracle.forward(mode, unary, ctx, ew, n_dir, n_iter, rho, saving_label=True)
  got = gpu.gpu_forward(mode, unary, ctx, ew, n_dir, n_iter, rho, saving_label=True)
  for k in ("msg", "cost_final", "msg_min_index", "msg_norm_index", "label_all"):
    assert np.array_equal(got[k], ref[k]), k


def test_negative_edge_weights_take_the_dense_path(gpu, oracle):
  rng = np.random.default_rng(77)
  B, H, W, L, n_dir = 1, 5, 6, 40, 4
  unary = rng.random((B, 1, H, W, L)).astype(np.float32)
  ctx = _context(rng, "tl3", L)
  ew = (rng.random((n_dir, B, 1, H, W)) - 0.3).astype(np.float32)
  for mode, rho in (("TRWP", 0.5), ("ISGMR", 1.0)):
    ref = oracle.forward(mode, unary, ctx, ew, n_dir, 2, rho, want_gaps=True)
    got = gpu.gpu_forward(mode, unary, ctx, ew, n_dir, 2, rho)
    gpu.assert_values_close(got["cost_final"], ref["cost_final"], what="cost_final")
    gpu.assert_indices_match_off_ties(got["msg_min_index"], ref["msg_min_index"], ref["gap_min"],
                                      2e-5, "msg_min_index")


@pytest.mark.parametrize("mode,n_dir,B,H,W,L,kind,n_iter", CASES)
def test_backward_matches_oracle(gpu, oracle, mode, n_dir, B, H, W, L, kind, n_iter):
  rng = np.random.default_rng(_seed(mode, n_dir, L, kind, 1))
  rho = 0.5 if mode == "TRWP" else 1.0
  unary = rng.random((B, 1, H, W, L)).astype(np.float32) * 3
  ctx = _context(rng, kind, L)
  ew = (0.1 + 0.9 * rng.random((n_dir, B, 1, H, W))).astype(np.float32)
  dcost = rng.standard_normal(unary.shape).astype(np.float32)
  print("case", mode, n_dir, B, H, W, L, kind, n_iter, flush=True)
  # same indices on both sides: the backward pass is checked on its own
  fwd = oracle.forward(mode, unary, ctx, ew, n_dir, n_iter, rho)
  ref = oracle.backward(mode, ctx.astype(np.float64), ew.astype(np.float64),
                        dcost.astype(np.float64), fwd["msg_min_index"], fwd["msg_norm_index"], rho)
  got = gpu.gpu_backward(mode, ctx, ew, dcost, fwd["msg_min_index"], fwd["msg_norm_index"], rho,
                         garbage_scratch=True)
  for g, r, name in zip(got, ref, ("dunary", "dcontext", "dedge_weights")):
    scale = max(1.0, float(np.abs(r).max()))
    assert np.abs(g - r).max() <= 1e-4 * scale, (name, float(np.abs(g - r).max()), scale)
  if ctx.ndim == 2:
    assert np.all(np.tril(got[1]) == 0)
  else:
    assert got[1][0] == 0


@pytest.mark.parametrize("mode,L,kind", [("TRWP", 40, "tl3"), ("ISGMR", 64, "tl3"), ("TRWP", 33, "rand1d")])
def test_backward_of_many_short_chains(gpu, oracle, mode, L, kind):
  """33 to 64 labels with a 1-D table: launches of more than 2048 chains take the reverse scan that
  sums popular argmin targets with wave reductions, smaller ones the LDS accumulators.  9 x 240 x 6
  pixels give TRWP 2160 rows of 6 pixels (the first kind) and 54 columns of 240 (the second);
  ISGMR puts all of them into one launch."""
  rng = np.random.default_rng(L)
  n_dir, n_iter, B, H, W = 4, 2, 9, 240, 6
  rho = 0.5 if mode == "TRWP" else 1.0
  unary = rng.random((B, 1, H, W, L)).astype(np.float32) * 3
  k = np.arange(L, dtype=np.float32)
  ctx = (0.3 * np.minimum(k, 3)).astype(np.float32) if kind == "tl3" else rng.random(L).astype(np.float32)
  ew = (0.1 + 0.9 * rng.random((n_dir, B, 1, H, W))).astype(np.float32)
  dcost = rng.standard_normal(unary.shape).astype(np.float32)
  print("case", mode, L, kind, flush=True)
  fwd = oracle.forward(mode, unary, ctx, ew, n_dir, n_iter, rho)
  ref = oracle.backward(mode, ctx.astype(np.float64), ew.astype(np.float64),
                        dcost.astype(np.float64), fwd["msg_min_index"], fwd["msg_norm_index"], rho)
  got = gpu.gpu_backward(mode, ctx, ew, dcost, fwd["msg_min_index"], fwd["msg_norm_index"], rho,
                         garbage_scratch=True)
  for g, r, name in zip(got, ref, ("dunary", "dcontext", "dedge_weights")):
    scale = max(1.0, float(np.abs(r).max()))
    assert np.abs(g - r).max() <= 1e-4 * scale, (name, float(np.abs(g - r).max()), scale)
  assert got[1][0] == 0
  if mode == "TRWP":
    # the hard backward of the TRWP_hard_soft build on the same launches: entry 0 of the table
    # also collects the pairs whose front label is their own (one label per lane, popular-target
    # shortcuts: the accumulator of label 0 is gathered twice and halved at the flush)
    ref = oracle.backward(mode, ctx.astype(np.float64), ew.astype(np.float64),
                          dcost.astype(np.float64), fwd["msg_min_index"], fwd["msg_norm_index"],
                          rho, same_label=True)
    got = gpu.gpu_backward(mode, ctx, ew, dcost, fwd["msg_min_index"], fwd["msg_norm_index"], rho,
                           garbage_scratch=True, hard_soft=True)
    assert abs(ref[1][0]) > 1e-3
    for g, r, name in zip(got, ref, ("dunary", "dcontext", "dedge_weights")):
      scale = max(1.0, float(np.abs(r).max()))
      assert np.abs(g - r).max() <= 1e-4 * scale, (name, float(np.abs(g - r).max()), scale)


def test_sgm_flag(gpu, oracle):
  rng = np.random.default_rng(5)
  B, H, W, L, n_dir = 1, 6, 7, 24, 8
  unary = rng.random((B, 1, H, W, L)).astype(np.float32)
  ctx = _context(rng, "tl2", L)
  ref = oracle.forward("SGM", unary, ctx, None, n_dir, 1, 1.0, enable_sgm=True, want_gaps=True)
  got = gpu.gpu_forward("SGM", unary, ctx, None, n_dir, 1, 1.0, enable_sgm=True)
  gpu.assert_values_close(got["cost_final"], ref["cost_final"], what="cost_final")
  dcost = rng.standard_normal(unary.shape).astype(np.float32)
  r = oracle.backward("SGM", ctx, None, dcost, ref["msg_min_index"], ref["msg_norm_index"], 1.0,
                      enable_sgm=True)
  g = gpu.gpu_backward("SGM", ctx, None, dcost, ref["msg_min_index"], ref["msg_norm_index"], 1.0,
                       enable_sgm=True)
  for a, b in zip(g, r):
    assert np.abs(a - b).max() <= 1e-4 * max(1.0, float(np.abs(b).max()))


def test_min_a_dir_and_initial_messages(gpu, oracle):
  rng = np.random.default_rng(9)
  B, H, W, L, n_dir = 1, 5, 6, 10, 4
  unary = rng.random((B, 1, H, W, L)).astype(np.float32)
  ctx = _context(rng, "tl2", L)
  for mode, rho in (("TRWP", 0.5), ("ISGMR", 1.0)):
    ref = oracle.forward(mode, unary, ctx, None, n_dir, 3, rho, enable_min_a_dir=True,
                         saving_label=True)
    got = gpu.gpu_forward(mode, unary, ctx, None, n_dir, 3, rho, enable_min_a_dir=True,
                          saving_label=True)
    gpu.assert_values_close(got["cost_final"], ref["cost_final"], what="cost_final min_a_dir")
  # TRWP continues from the messages it is given (msg is an in/out tensor in the reference)
  first = oracle.forward("TRWP", unary, ctx, None, n_dir, 1, 0.5)
  ref = oracle.forward("TRWP", unary, ctx, None, n_dir, 2, 0.5)
  got = gpu.gpu_forward("TRWP", unary, ctx, None, n_dir, 1, 0.5, msg_init=first["msg"])
  gpu.assert_values_close(got["msg"], ref["msg"], what="continued msg", belief=ref["cost_final"])


@pytest.mark.gpu
def test_issue_probe_reads_sane_costs(gpu):
  """The probe's rows are read in units of one plain vector instruction: an idle slot costs a
  lone wavefront as much as an instruction (`s_nop 1`, two slots, about twice a dependent add), a
  dependent add no more than an independent one, an LDS round trip several instructions.  Ratios
  only: the absolute clock counts depend on the clock the counter runs on."""
  import ctypes
  import torch
  from mplayers_amd import _probe
  lib = _probe.load()
  n = lib.mplp_issue_count()
  clocks = torch.zeros(n, dtype=torch.int64, device="cuda")
  _probe.check(lib.mplp_issue(ctypes.c_void_p(clocks.data_ptr()), n, None), "probe_issue")
  torch.cuda.synchronize()
  c = clocks.cpu().tolist()
  cost = {lib.mplp_issue_name(i).decode(): (c[i] - c[0]) / lib.mplp_issue_slots(i)
          for i in range(1, n)}
  print(cost, flush=True)
  assert all(v > 0 for v in cost.values())
  add = cost["vop2 add, each needs the one before"]
  assert 0.8 <= cost["vop2 add, independent"] / add <= 1.25
  assert 1.6 <= cost["s_nop 1"] / add <= 2.6
  assert cost["ds_read_b32 and wait (round trip, 2 slots)"] > 3 * add


def test_copy_probe_moves_what_it_claims(gpu):
  """The bandwidth probe's kernels write the sum of their input planes (+ k for output plane k) to
  every element, whatever the access shape, and reject shapes they do not implement."""
  import ctypes
  import torch
  from mplayers_amd import _probe
  lib = _probe.load()
  H, W, L = 13, 21, 44
  n = H * W * L
  src = torch.randn(4 * n, device="cuda")
  stream = torch.cuda.current_stream().cuda_stream
  for shape in (0, 1, 2):
    for n_in, n_out in ((1, 1), (1, 3), (3, 2), (4, 3), (3, 0)):
      dst = torch.full((3 * n,), -7.0, device="cuda")
      rc = lib.mplp_copy(shape, n_in, n_out, ctypes.c_void_p(src.data_ptr()),
                              ctypes.c_void_p(dst.data_ptr()), H, W, L, ctypes.c_void_p(stream))
      assert rc == 0, lib.mplp_last_error()
      want = src.view(4, n)[0].clone()
      for k in range(1, n_in):
        want = want + src.view(4, n)[k]
      for k in range(3):
        got = dst.view(3, n)[k]
        if k < n_out:
          assert torch.equal(got, want + k), (shape, n_in, n_out, k)
        else:
          assert bool((got == -7.0).all()), (shape, n_in, n_out, k)
  dst = torch.empty(3 * n, device="cuda")
  args = (ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(dst.data_ptr()))
  assert lib.mplp_copy(0, 2, 2, *args, H, W, L, ctypes.c_void_p(stream)) != 0
  assert lib.mplp_copy(3, 1, 1, *args, H, W, L, ctypes.c_void_p(stream)) != 0
  assert lib.mplp_copy(0, 1, 1, *args, H, W, 42, ctypes.c_void_p(stream)) != 0
