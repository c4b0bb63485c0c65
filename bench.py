#!/usr/bin/env python3
"""Benchmark of the TRWP / ISGMR message-passing path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config C5] [--alg both|TRWP|ISGMR]

A step is one forward + backward pass of the selected algorithm(s) over one synthetic batch of
the configuration (default: the large 1500x2000, 192-label, 8-direction one), inputs resident in
HBM, every buffer pre-allocated as the reference's operator interface has the caller do it; the
message tensor is re-zeroed inside the timed region (the operators take it as initial messages).
Prints ONE JSON line: throughput in pixel*label*iter/s, the roofline position of the dominant
kernel (HIP-event timings taken inside the library on the launch stream during the timed steps)
and the reference's CPU forward path timed on a bounded crop on this host.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
# plain fp32 vector lane-operations per second: 256 compute units x 64 lanes x 2.4 GHz (the
# published 157.3 TFLOP/s counts a packed multiply-add as four operations; a minimum has no packed
# form, so the dense min-plus step is priced against one operation per lane and clock)
VALU_PEAK_TLANEOPS = 39.3

# HBM bytes per launch of the scan kernels at the full-size large configuration were measured with
# `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` (one counter per run) and scaled by what the
# same counters read for a plain device copy of one plane; counters cannot be read from inside this
# script, so the figure is taken from the committed summary of those runs: the table row whose
# first cell names the kernel kind ("bwd_sweep", ...), column "HBM GB / launch".
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "c5_trwp_isgmr_hbm_traffic.md")


def measured_traffic_bytes(kind, cfg_name, scale, training):
  """HBM bytes per launch of kernel `kind` from the committed counter summary; None when the
  summary is absent or covers another workload."""
  if (cfg_name, scale, training) != ("C5", 1.0, True) or not os.path.exists(TRAFFIC_SUMMARY):
    return None
  col = None
  for line in open(TRAFFIC_SUMMARY):
    cells = [c.strip() for c in line.strip().strip("|").split("|")]
    if col is None:
      if "HBM GB / launch" in cells:
        col = cells.index("HBM GB / launch")
      continue
    if cells and cells[0].strip("`") == kind and col < len(cells):
      try:
        return float(cells[col]) * 1e9
      except ValueError:
        return None
  return None


def parse():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=10)
  ap.add_argument("--warmup", type=int, default=3)
  ap.add_argument("--config", default="C5")
  ap.add_argument("--scale", type=float, default=1.0, help="shrink H and W (debugging only)")
  ap.add_argument("--n-dir", type=int, default=None, choices=[2, 4, 8, 16],
                  help="run the configuration on another connectivity (not the headline workload)")
  ap.add_argument("--context", default=None, choices=["dense1d", "dense2d"],
                  help="replace the configuration's pairwise table by a learned-style dense one: a "
                       "1-D table of random entries, or a 2-D (L, L) table (at most 64 labels); the "
                       "scans then take their O(L^2) step and the roofline reported is the VALU one "
                       "(2 L lane-operations per label and direction sweep); not the headline workload")
  ap.add_argument("--no-dense-flag", action="store_true",
                  help="with --context: do not declare the table dense (one wavefront per chain)")
  ap.add_argument("--split-waves", type=int, default=None,
                  help="with --context: force this many wavefronts per chain (MPL_OPT_DENSE_SPLIT_WAVES)")
  ap.add_argument("--labels", type=int, default=None, help="run the configuration with this many labels")
  ap.add_argument("--batch", type=int, default=None, help="run the configuration at this batch size")
  ap.add_argument("--n-iter", type=int, default=None, help="run this many iterations")
  ap.add_argument("--no-configs", action="store_true",
                  help="leave the four smaller configurations out of the default run (profiler runs)")
  ap.add_argument("--alg", default="both", choices=["both", "TRWP", "ISGMR", "SOFT"],
                  help="SOFT: soft-weighted TRWP (stores n_disp^2 floats per pixel, direction and "
                       "iteration)")
  ap.add_argument("--fwd-only", action="store_true", help="inference forward only (C2/C3 style)")
  ap.add_argument("--no-cpu-baseline", action="store_true")
  ap.add_argument("--copy-probe", action="store_true",
                  help="also run one plain device copy of one fp32 plane (reference point for "
                       "hardware byte counters)")
  ap.add_argument("--peak-probe", action="store_true",
                  help="also time the library's copy probes on planes of the workload's size: one-pass "
                       "streaming kernels and scan-shaped kernels (one long-lived wavefront per row "
                       "or column) for several read:write mixes (\"measured_stream_rates\")")
  ap.add_argument("--no-peak-probe", action="store_true",
                  help="leave the copy probes out of the default large-configuration run (profiler runs)")
  ap.add_argument("--issue-probe", action="store_true",
                  help="also report what instruction patterns cost a lone wavefront, in clocks per "
                       "issue slot (under \"issue_costs\"): the bound of launches with fewer chains "
                       "than the chip has SIMDs")
  ap.add_argument("--module-probe", action="store_true",
                  help="also time forward+backward through the nn.Module surface, which allocates "
                       "its buffers on every call as the reference's does (reported under "
                       "\"module_surface\")")
  ap.add_argument("--edge-probe", action="store_true",
                  help="also time the edge-weight producer on an image of the workload's size "
                       "(reported under \"edge_weights\")")
  ap.add_argument("--msg-uninit", action="store_true",
                  help="headline under the library's MPL_F_MSG_UNINIT extension: the library starts "
                       "the messages at zero itself and the step does not touch `msg` beforehand "
                       "(default: the reference's operator contract, the step zero-fills `msg` "
                       "inside the timed region and the operators read it as initial messages; the "
                       "other contract is timed over the same number of steps and reported beside it)")
  ap.add_argument("--no-fused-pairs", action="store_true",
                  help="TRWP: one launch per direction even for launches of at most 1024 chains "
                       "(MPL_F_FUSED_PAIRS_OFF)")
  ap.add_argument("--dunary-only", action="store_true",
                  help="backward without dcontext and dedge_weights (a fixed pairwise table and "
                       "edge weights that are not learned); not the headline workload")
  ap.add_argument("--graph-probe", action="store_true",
                  help="also capture one step in a HIP graph and time its replays (the library only "
                       "launches kernels, so a step is capturable; reported under \"graph_replay\")")
  ap.add_argument("--terms-probe", action="store_true",
                  help="also time the stereo data cost of an image pair of the workload's size and "
                       "the energies of n_iter labellings (reported under \"mrf_terms\")")
  return ap.parse_args()


def host_cpu():
  """Model name and logical CPU count of this host, and the thread share the harness grants."""
  model = "unknown"
  try:
    for line in open("/proc/cpuinfo"):
      if line.startswith("model name"):
        model = line.split(":", 1)[1].strip()
        break
  except OSError:
    pass
  share = os.environ.get("OMP_NUM_THREADS")
  return model, os.cpu_count(), int(share) if share and share.isdigit() else None


def cpu_baseline(cfg, budget_s=12.0):
  """Times the reference's CPU forward path (built from the reference sources into oracle/_ref)
  or, where that build is absent, the oracle's restatement of the same loop nest, on a crop of
  the workload: full-width rows, one iteration, unit edge weights (that path ignores them),
  forward only (the reference has no CPU backward).  A short calibration run sizes the crop so
  that the timed run takes about budget_s seconds.  The reference hard-codes 16 OpenMP threads;
  the restatement is timed a second time on every core this process may use."""
  import numpy as np
  from oracle import mp_oracle, ref_cpu
  L, n_dir, W = cfg["L"], cfg["n_dir"], cfg["W"]
  mode = "TRWP" if cfg["mode"] == "TRWP" else "ISGMR"
  threads = 16  # NUM_THREADS of the reference (tools/cpp/utils.h:17)
  ctx = cfg["context"].numpy()
  if ctx.ndim == 1:
    ii = np.abs(np.arange(L)[:, None] - np.arange(L)[None, :])
    table = ctx[ii]
  else:
    table = ctx + ctx.T
  table = np.ascontiguousarray(np.broadcast_to(table, (n_dir, L, L)), dtype=np.float32)
  kind = "reference" if ref_cpu.available() else "port"

  def run(rows, which, n_threads):
    unary = cfg["unary"][:1, :, :rows, :, :].contiguous().numpy()
    t0 = time.perf_counter()
    if which == "reference":
      ref_cpu.forward(mode, unary, table, n_dir, 1, cfg["rho"])
    else:
      mp_oracle.refcpu_forward(mode, unary, table, n_dir, 1, cfg["rho"], n_threads=n_threads,
                               context_per_dir=True, ctx2d=(L == 21))
    return time.perf_counter() - t0

  rows0 = min(cfg["H"], 4)
  dt0 = run(rows0, kind, threads)
  rows = int(max(rows0, min(cfg["H"], rows0 * budget_s / max(dt0, 1e-3))))
  dt = run(rows, kind, threads) if rows > rows0 else dt0
  units = rows * W * L * 1
  model, nproc, share = host_cpu()
  # every core this process may use: the affinity mask, capped by the harness's thread share
  try:
    usable = len(os.sched_getaffinity(0))
  except AttributeError:
    usable = nproc or threads
  all_cores = min(usable, share) if share else usable
  dt_all = run(rows, "port", all_cores)
  out = {"value": units / dt, "unit": "pixel*label*iter/s", "cores": threads, "kind": kind,
         "sample": "%s forward only (the reference has no CPU backward), first %d rows x %d "
                   "columns of %s, %d labels, %d directions, 1 iteration, unit edge weights, "
                   "%.1f s" % (mode, rows, W, cfg["name"], L, n_dir, dt),
         "host_cpu": model, "nproc": nproc, "usable_cores": usable, "thread_share": share,
         "all_cores": {"kind": "port", "cores": all_cores, "value": units / dt_all,
                       "seconds": round(dt_all, 2),
                       "note": "the restatement of the same loop nest (oracle/mp_oracle.c) on every "
                               "core this process may use; the reference's own build cannot change "
                               "its 16 threads"},
         "compile_flags": {"reference": "g++ -O2 -std=c++17 -fopenmp (oracle/build_ref.py, the "
                                        "reference's sources compiled in place)",
                           "port": "gcc -O2 -ffp-contract=off -fopenmp (oracle/Makefile)"}}
  return out


def peak_probe(H, W, L, dev, reps=5):
  """What this GPU sustains on planes of the workload's size, in GB/s of bytes moved: one-pass
  streaming kernels (the shape of the element-wise passes) and long-lived one-wavefront-per-chain
  kernels that move n_in planes in and n_out planes out pixel by pixel (the shape of the scans,
  without their arithmetic): mplp_copy of the probe library."""
  import ctypes
  import torch
  from mplayers_amd import _probe
  if L % 4:
    return {"note": "the probe needs a label count that is a multiple of 4"}
  lib = _probe.load()
  n = H * W * L
  src = torch.zeros(4 * n, dtype=torch.float32, device=dev)
  dst = torch.empty(3 * n, dtype=torch.float32, device=dev)
  stream = torch.cuda.current_stream().cuda_stream
  res = {"plane_bytes": 4 * n}
  start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
  for shape, sname in ((2, "stream"), (0, "rows"), (1, "columns")):
    for n_in, n_out in ((1, 1), (3, 0), (1, 3), (3, 2), (4, 3)):
      def run():
        _probe.check(lib.mplp_copy(shape, n_in, n_out, ctypes.c_void_p(src.data_ptr()),
                                   ctypes.c_void_p(dst.data_ptr()), H, W, L,
                                   ctypes.c_void_p(stream)), "probe_copy")
      run()
      torch.cuda.synchronize()
      start.record()
      for _ in range(reps):
        run()
      stop.record()
      torch.cuda.synchronize()
      ms = start.elapsed_time(stop) / reps
      res["%s_%din_%dout_GBs" % (sname, n_in, n_out)] = round((n_in + n_out) * 4 * n / ms / 1e6, 1)
  return res


def issue_probe(dev):
  """Clocks per issue slot of instruction patterns for a wavefront that has its SIMD to itself
  (mplp_issue of the probe library): what bounds the scans of launches with fewer chains than the
  chip has SIMDs."""
  import ctypes
  import torch
  from mplayers_amd import _probe
  lib = _probe.load()
  n = lib.mplp_issue_count()
  clocks = torch.zeros(n, dtype=torch.int64, device=dev)
  stream = torch.cuda.current_stream().cuda_stream
  _probe.check(lib.mplp_issue(ctypes.c_void_p(clocks.data_ptr()), n, ctypes.c_void_p(stream)),
               "probe_issue")
  torch.cuda.synchronize()
  c = clocks.cpu().tolist()
  res = {"empty_region_clocks": c[0]}
  for i in range(1, n):
    slots = lib.mplp_issue_slots(i)
    res[lib.mplp_issue_name(i).decode()] = round((c[i] - c[0]) / slots, 2)
  return res


def module_probe(cfg, algs, unary, edge, dcost, reps=3):
  """forward + backward of MPModule (buffers allocated inside every call, as the reference's
  autograd functions do), per algorithm: wall ms per call."""
  import torch
  from mplayers_amd import MPModule
  res = {}
  u = unary.permute(0, 1, 4, 2, 3).contiguous().requires_grad_(True)        # (B, cv, L, H, W)
  e = edge[:, :, 0].permute(1, 0, 2, 3).contiguous().requires_grad_(True)   # (B, n_dir, H, W)
  g = dcost.permute(0, 1, 4, 2, 3).contiguous()
  for alg in algs:
    ns = argparse.Namespace(mpnet_mrf_mode=alg, mpnet_max_iter=cfg["n_iter"],
                            mpnet_n_dirs=cfg["n_dir"], n_classes=cfg["L"], mpnet_term_weight=1.0,
                            mpnet_smoothness_train="", mpnet_smoothness_mode="TL",
                            mpnet_smoothness_trunct_value=3, mpnet_smoothness_trunct_loc=-1,
                            mpnet_diag_value=0.0, enable_symmetric=True, enable_cuda=True)
    mod = MPModule(ns, enable_create_label_context=True).cuda().train()
    times = []
    for r in range(reps + 1):
      u.grad = e.grad = None
      torch.cuda.synchronize()
      t0 = time.perf_counter()
      cost = mod(u, e)[0]
      cost.backward(g)
      torch.cuda.synchronize()
      times.append((time.perf_counter() - t0) * 1e3)
      del cost
    res[alg] = {"ms_per_call": sum(times[1:]) / reps}
  res["note"] = ("includes the per-call allocation of messages, indices and gradients, the two "
                 "layout permutes of the module and autograd's bookkeeping")
  return res


def edge_probe(B, H, W, n_dir, dev, channels=3, reps=20):
  """exp(-|I(p) - I(q)|) weights of a (B, 3, H, W) image for n_dir directions: reads one image,
  writes n_dir maps of its size."""
  import torch
  from mplayers_amd import edge_weights
  img = torch.rand(B, channels, H, W, device=dev)
  edge_weights.getEdgeShift("edge_net", img, n_dir)
  torch.cuda.synchronize()
  t0 = time.perf_counter()
  for _ in range(reps):
    edge_weights.getEdgeShift("edge_net", img, n_dir)
  torch.cuda.synchronize()
  ms = (time.perf_counter() - t0) / reps * 1e3
  nbytes = B * channels * H * W * 4 * (1 + n_dir)
  return {"mode": "edge_net", "image": [B, channels, H, W], "n_dirs": n_dir, "ms": ms,
          "algorithmic_GBs": nbytes / (ms * 1e-3) / 1e9,
          "note": "wall time per call including the allocation of the result"}


def terms_probe(H, W, L, n_dir, n_iter, dev, reps=10):
  """Stereo data cost of a 3-band H x W pair for L disparities (writes the (H, W, L) fp32 volume
  the layers take as unary) and the energies of n_iter labellings of it."""
  import torch
  from mplayers_amd import compute_terms
  left = torch.randint(0, 256, (H, W, 3), dtype=torch.uint8, device=dev)
  right = torch.roll(left, -5, dims=1)
  labels = torch.randint(0, L, (n_iter, 1, H, W), dtype=torch.uint8, device=dev)
  context = torch.arange(L, dtype=torch.float32, device=dev).clamp(max=3)

  def timed(fn):
    fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
      fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / reps * 1e3

  cost = compute_terms.stereo_data_cost(left, right, L)
  ms_cost = timed(lambda: compute_terms.stereo_data_cost(left, right, L))
  unary = cost.view(1, H, W, L)
  ms_energy = timed(lambda: compute_terms.mrf_energy(unary, context, labels, None, n_dir))
  return {"image": [H, W, 3], "n_disp": L,
          "data_cost_ms": ms_cost, "data_cost_written_GBs": H * W * L * 4 / (ms_cost * 1e-3) / 1e9,
          "energy_labellings": n_iter, "energy_ms": ms_energy,
          "note": "wall time per call including the allocation of the result"}


class Workload(object):
  """The pre-allocated tensors of one configuration and its timed step: one forward (+ backward)
  pass of every selected algorithm through the operators, exactly as the reference's callers
  drive them."""

  def __init__(self, cfg, algs, training, dev, dunary_only=False, trwp_flags=0, fwd_flags=0):
    import torch
    from mplayers_amd import synthetic
    self.cfg, self.algs, self.training = cfg, algs, training
    self.dunary_only, self.trwp_flags, self.fwd_flags = dunary_only, trwp_flags, fwd_flags
    B, H, W, L, n_dir, n_iter = (cfg[k] for k in ("B", "H", "W", "L", "n_dir", "n_iter"))
    self.unary = cfg["unary"].to(dev)
    self.context = cfg["context"].to(dev)
    self.edge = cfg["edge_weights"].to(dev)
    self.dcost = synthetic.upstream_grad(cfg).to(dev) if training else None
    f32 = dict(dtype=torch.float32, device=dev)
    u8 = dict(dtype=torch.uint8, device=dev)
    self.msg = torch.zeros(n_dir, B, 1, H, W, L, **f32)
    self.msg_tmp = torch.zeros(n_dir, B, 1, H, W, L, **f32) if "ISGMR" in algs else None
    self.soft_blocks = (torch.zeros(n_iter, n_dir, B, 1, H, W, L, L, **f32)
                        if ("SOFT" in algs and training) else torch.empty(0))
    self.cost = torch.zeros(B, 1, H, W, L, **f32)
    self.belief = torch.zeros(B, 1, H, W, L, **f32)
    self.empty = torch.empty(0, dtype=torch.uint8)
    if training:
      self.imin = torch.zeros(n_iter, n_dir, B, 1, H, W, L, **u8)
      self.inorm = torch.zeros(n_iter, n_dir, B, 1, H, W, **u8)
      self.dunary = torch.zeros(B, 1, H, W, L, **f32)
      self.dmsg = torch.zeros(n_dir, B, 1, H, W, L, **f32)
      self.dmsg_tmp = torch.zeros(n_dir, B, 1, H, W, L, **f32) if "ISGMR" in algs else None
      self.dscratch = torch.zeros(B, 1, H, W, L, **f32)
      self.dedge = torch.zeros(n_dir, B, 1, H, W, **f32)
      self.dctx = torch.zeros(tuple(cfg["context"].shape), **f32)
      if dunary_only:
        self.dedge = self.dctx = torch.empty(0, **f32)
    else:
      self.imin = self.inorm = self.empty

  def step(self, uninit):
    from mplayers_amd import lib_stereo
    w, n_iter = self, self.cfg["n_iter"]
    for alg in self.algs:
      rho = 1.0 if alg == "ISGMR" else 0.5
      if alg == "SOFT" or not uninit:
        w.msg.zero_()
      if w.training and not w.dunary_only:
        # the accumulating gradients must arrive zero-filled (the reference's caller allocates
        # them with new_zeros on every call, MP_module.py:65-74)
        w.dedge.zero_()
        w.dctx.zero_()
      if alg == "SOFT":
        lib_stereo.TRWP_hard_soft.forward_soft(rho, n_iter, w.unary, w.context, w.edge, w.msg,
                                               w.soft_blocks, w.inorm, w.cost, w.belief, w.empty)
        if w.training:
          lib_stereo.TRWP_hard_soft.backward_soft(rho, w.dcost, w.context, w.edge, w.soft_blocks,
                                                  w.inorm, w.dunary, w.dctx, w.dedge, w.dmsg,
                                                  w.dscratch)
      elif alg == "TRWP":
        lib_stereo.TRWP.forward(rho, n_iter, 0, w.unary, w.context, w.edge, w.msg, w.cost, w.imin,
                                w.inorm, w.belief, w.empty, msg_uninit=uninit,
                                flags=w.trwp_flags | w.fwd_flags)
        if w.training:
          lib_stereo.TRWP.backward(rho, w.context, w.edge, w.dcost, w.imin, w.inorm, w.dunary,
                                   w.dctx, w.dedge, w.dmsg, w.dscratch, flags=w.trwp_flags)
      else:
        lib_stereo.ISGMR.forward(0, rho, n_iter, 0, w.unary, w.context, w.edge, w.msg, w.cost,
                                 w.imin, w.inorm, w.belief, w.msg_tmp, w.empty, msg_uninit=uninit,
                                 flags=w.fwd_flags)
        if w.training:
          lib_stereo.ISGMR.backward(0, rho, w.context, w.edge, w.dcost, w.imin, w.inorm, w.dunary,
                                    w.dctx, w.dedge, w.dmsg, w.dscratch, w.dmsg_tmp)

  def timed(self, steps, warmup, uninit, profile=False):
    """Wall seconds of `steps` steps after `warmup` untimed ones (synchronised on both sides) and,
    with profile, the library's per-kernel HIP-event totals over the timed steps."""
    import torch
    from mplayers_amd import _lib
    for _ in range(warmup):
      self.step(uninit)
    torch.cuda.synchronize()
    if profile:
      _lib.profile_begin()
    t0 = time.perf_counter()
    for _ in range(steps):
      self.step(uninit)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    return dt, (_lib.profile_end() if profile else None)


def contract_bytes(cfg, training, soft=False):
  """Algorithmic bytes per label and direction sweep, forward and backward: forward 20 B (read S,
  m_d, m_inv; write m_d, S) + 1 B argmin index + 1/L B norm index when training; backward
  25 B + 1/L (read index; read+reset h_d; update h_inv; update A)."""
  L = cfg["L"]
  fwd_b = (21.0 + 1.0 / L) if training else 20.0
  bwd_b = 25.0 + 1.0 / L
  if soft:
    # the stored duals replace the argmin index: 4*L bytes per label written forward (training)
    # and read back
    fwd_b = (20.0 + 4.0 * L + 1.0 / L) if training else 20.0
    bwd_b = 24.0 + 4.0 * L + 1.0 / L
  return fwd_b, bwd_b


# the workload of each of the smaller benchmark configurations as the benchmark definition states it
SMALL_CONFIGS = (("C1", ["ISGMR"], True), ("C2", ["TRWP"], False), ("C3", ["ISGMR"], False),
                 ("C4", ["TRWP", "ISGMR"], True))


def small_configs(dev, steps=20, warmup=3):
  """The four smaller configurations as stated (their own algorithm and mode), under the
  reference's operator contract and with the messages declared zero: ms per step, units per
  second, and the fraction of the 8 TB/s roofline on the contract bytes per unit."""
  import torch
  from mplayers_amd import synthetic
  res = {}
  for name, algs, training in SMALL_CONFIGS:
    cfg = synthetic.make_config(name, seed=0)
    w = Workload(cfg, algs, training, dev)
    fwd_b, bwd_b = contract_bytes(cfg, training)
    contract = cfg["n_dir"] * (fwd_b + (bwd_b if training else 0.0))
    units = cfg["units"] * len(algs)
    entry = {"workload": "%s %s, batch %d, grid %dx%d, %d labels, %d directions, %d iterations" % (
        "+".join(algs), "fwd+bwd" if training else "fwd", cfg["B"], cfg["H"], cfg["W"], cfg["L"],
        cfg["n_dir"], cfg["n_iter"]), "steps": steps, "contract_bytes_per_unit": round(contract, 3)}
    for key, uninit in (("reference_contract", False), ("msg_uninit", True)):
      dt, _ = w.timed(steps, warmup, uninit)
      value = units * steps / dt
      entry[key] = {"ms_per_step": round(dt / steps * 1e3, 4), "value": value,
                    "frac_of_hbm_roofline": round(contract * value / 1e9 / HBM_PEAK_GBS, 4)}
    res[name] = entry
    del w
    torch.cuda.empty_cache()
  res["note"] = ("C1 and C4 fit in the caches (their planes are 0.4 and 5.6 MB): their fraction of "
                 "the HBM roofline is informational")
  return res


def main():
  a = parse()
  if a.gpus != 1:
    print("bench.py: this build drives one GPU only (the path shards by batch item or by "
          "direction without any exchange inside the operators); run with --gpus 1", file=sys.stderr)
    return 2
  import torch
  from mplayers_amd import _lib, synthetic
  _lib.load()
  dev = torch.device("cuda:0")
  torch.cuda.set_device(dev)

  cfg = synthetic.make_config(a.config, seed=0, scale=a.scale, n_dir=a.n_dir, context=a.context,
                              n_labels=a.labels, batch=a.batch, n_iter=a.n_iter)
  B, H, W, L, n_dir, n_iter = (cfg[k] for k in ("B", "H", "W", "L", "n_dir", "n_iter"))
  algs = ["TRWP", "ISGMR"] if a.alg == "both" else [a.alg]
  training = not a.fwd_only
  N = B * H * W * L

  uninit = bool(a.msg_uninit)
  trwp_flags = _lib.F_FUSED_PAIRS_OFF if a.no_fused_pairs else 0
  # a dense table is declared to the library (MPL_F_DENSE_TABLE) as a caller who trains one does
  fwd_flags = _lib.F_DENSE_TABLE if (a.context is not None and not a.no_dense_flag) else 0
  if a.split_waves is not None:
    _lib.set_option(_lib.OPT_DENSE_SPLIT_WAVES, a.split_waves)
  work = Workload(cfg, algs, training, dev, dunary_only=a.dunary_only, trwp_flags=trwp_flags,
                  fwd_flags=fwd_flags)
  unary, edge, dcost = work.unary, work.edge, work.dcost

  if a.copy_probe:
    probe = torch.empty_like(work.cost)
    probe.copy_(unary)  # reads N*4 bytes, writes N*4 bytes
    del probe
  dt, stats = work.timed(a.steps, a.warmup, uninit, profile=True)

  units_per_step = cfg["units"] * len(algs)
  value = units_per_step * a.steps / dt

  # roofline of the dominant kernel.  One launch handles N labels of one direction (TRWP) or of
  # all n_dir directions (ISGMR).
  fwd_b, bwd_b = contract_bytes(cfg, training, soft=(a.alg == "SOFT"))
  # kind -> (bytes per label and direction sweep, direction sweeps per launch, companion pass)
  # ISGMR splits the work of a sweep between the scan kernel and one element-wise pass per
  # iteration (forward: U of every direction; backward: gradient recombination); its rate is
  # computed over both, so that it stays comparable with the algorithmic byte count.
  model = {"fwd_sweep": (fwd_b, 1, None), "bwd_sweep": (bwd_b, 1, None),
           "fwd_sweep_all": (fwd_b, n_dir, "unary_all"), "bwd_sweep_all": (bwd_b, n_dir, "combine")}
  kernels = {}
  for kind, (bpl, dirs_per_launch, companion) in model.items():
    n, ms = stats[kind]
    if n == 0:
      continue
    per_launch = bpl * N * dirs_per_launch  # algorithmic bytes one launch moves
    both_ms = ms + (stats[companion][1] if companion else 0.0)
    kernels[kind] = {"launches": n, "avg_ms": ms / n, "total_ms": both_ms,
                     "bytes_per_launch": per_launch,
                     "achieved_GBs": per_launch / (both_ms / n * 1e-3) / 1e9,
                     "bytes_per_label_sweep": bpl}
    if companion:
      kernels[kind]["companion_pass"] = companion
      kernels[kind]["companion_avg_ms"] = stats[companion][1] / n
  dominant = max(kernels, key=lambda k: kernels[k]["total_ms"])
  traffic = None if a.dunary_only else measured_traffic_bytes(dominant, cfg["name"], a.scale,
                                                              training)
  roofline = {"bound": "hbm", "kernel": dominant, "achieved": kernels[dominant]["achieved_GBs"],
              "peak": HBM_PEAK_GBS, "unit": "GB/s",
              "frac": kernels[dominant]["achieved_GBs"] / HBM_PEAK_GBS, "traffic": traffic,
              "algorithmic_bytes_per_launch": kernels[dominant]["bytes_per_launch"],
              "avg_launch_ms": kernels[dominant]["total_ms"] / kernels[dominant]["launches"]}
  if a.context is not None:
    # dense O(L^2) step: the forward scan evaluates L candidates per label, an add and a minimum
    # each (the loop of TRWP_forward.cu:127-153): 2 L lane-operations per label and direction sweep
    fk = "fwd_sweep" if "fwd_sweep" in kernels else "fwd_sweep_all"
    sweeps = n_dir if fk == "fwd_sweep_all" else 1
    lane_ops = 2.0 * L * N * sweeps
    avg_ms = kernels[fk]["avg_ms"]
    achieved = lane_ops / (avg_ms * 1e-3) / 1e12
    roofline = {"bound": "valu", "kernel": fk, "achieved": achieved, "peak": VALU_PEAK_TLANEOPS,
                "unit": "Tlane-op/s", "frac": achieved / VALU_PEAK_TLANEOPS, "traffic": None,
                "algorithmic_lane_ops_per_launch": lane_ops, "avg_launch_ms": avg_ms,
                "hbm_GBs_of_that_kernel": kernels[fk]["achieved_GBs"]}
  # whole-step roofline fraction against the contract bytes per unit (n_dir * (fwd + bwd))
  contract = n_dir * (fwd_b + (bwd_b if training else 0.0))
  whole = contract * value / 1e9 / HBM_PEAK_GBS

  out = {
      "metric": "pixel*label*iter/s, %s %s" % (" & ".join(algs), "fwd+bwd" if training else "fwd"),
      "value": value, "unit": "pixel*label*iter/s", "n_gpus": 1, "steps": a.steps,
      "warmup": a.warmup, "ms_per_step": dt / a.steps * 1e3, "higher_is_better": True,
      "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
      "config": {"workload": "%s: %s %s, batch %d, grid %dx%d, %d labels, %d directions, %d "
                             "iterations" % (cfg["name"], "+".join(algs),
                                             "fwd+bwd" if training else "fwd", B, H, W, L, n_dir,
                                             n_iter),
                 "scale": a.scale,
                 "pairwise_table": (a.context + (", declared dense (MPL_F_DENSE_TABLE)" if fwd_flags
                                                 else "")) if a.context else "as the configuration states",
                 "initial_messages": ("zero by declaration (MPL_F_MSG_UNINIT): the library writes "
                                      "every element itself" if uninit else
                                      "the reference's operator contract: `msg` cleared by the "
                                      "caller inside the timed step and read as initial messages"),
                 "gradients": ("none" if not training else
                               "dunary only" if a.dunary_only else
                               "dunary, dcontext, dedge_weights (the two accumulating ones cleared "
                               "inside the timed step)")},
      "roofline": roofline,
      "whole_step_frac_of_hbm_roofline": whole,
      "contract_bytes_per_unit": contract,
      "kernels": {k: {kk: (round(vv, 4) if isinstance(vv, float) else vv) for kk, vv in v.items()}
                  for k, v in kernels.items()},
      "other_kernels_ms": {k: round(stats[k][1], 3) for k in stats if k not in kernels},

  }
  if "SOFT" not in algs:
    # the same step under the other contract for the initial messages, over the same number of
    # steps: zero by declaration (the library's extension, what its nn.Module passes) when the
    # headline is the reference's operator contract, and the other way round
    alt_dt, _ = work.timed(a.steps, min(2, a.warmup), not uninit)
    alt_ms = alt_dt / a.steps * 1e3
    out["msg_uninit" if not uninit else "caller_cleared_messages"] = {
        "ms_per_step": alt_ms, "steps": a.steps, "value": units_per_step / (alt_ms * 1e-3)}
  if a.peak_probe or (cfg["name"] == "C5" and a.scale == 1.0 and not a.no_peak_probe):
    # what this GPU sustains for traffic of the kernels' shapes, next to the published 8 TB/s
    out["measured_stream_rates"] = peak_probe(H, W, L, dev, reps=5 if a.peak_probe else 2)
  if a.issue_probe:
    out["issue_costs"] = issue_probe(dev)
  if a.module_probe and training:
    out["module_surface"] = module_probe(cfg, algs, unary, edge, dcost)
  if a.edge_probe:
    out["edge_weights"] = edge_probe(B, H, W, n_dir, dev)
  if a.terms_probe:
    out["mrf_terms"] = terms_probe(H, W, L, n_dir, n_iter, dev)
  if a.graph_probe:
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
      work.step(uninit)
    graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
      graph.replay()
    torch.cuda.synchronize()
    g_ms = (time.perf_counter() - t0) / a.steps * 1e3
    out["graph_replay"] = {"ms_per_step": g_ms, "eager_ms_per_step": out["ms_per_step"],
                           "speedup": out["ms_per_step"] / g_ms}
  if cfg["name"] == "C5" and a.scale == 1.0 and a.context is None and not a.no_configs:
    # the other four configurations of the benchmark, each as stated, after this one's buffers are gone
    del work, unary, edge, dcost
    torch.cuda.empty_cache()
    out["configs"] = small_configs(dev)
  if not a.no_cpu_baseline:
    out["cpu_baseline"] = cpu_baseline(cfg)
  print(json.dumps(out))
  return 0


if __name__ == "__main__":
  sys.exit(main())
