"""HIP graph capture of the operators: the library only launches kernels on the caller's stream (no
allocation, no memset, no synchronisation), so a forward + backward call can be captured once and
replayed.  Every replay is checked against the eager result, with eager work and synchronisation
between the replays."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("mode", ["TRWP", "ISGMR"])
@pytest.mark.parametrize("L,n_dir,B,H,W", [(21, 4, 2, 33, 35), (96, 8, 1, 24, 40), (16, 16, 8, 40, 40)])
def test_graph_replay_matches_eager(gpu, mode, L, n_dir, B, H, W):
  import torch
  from mplayers_amd import lib_stereo
  g = torch.Generator().manual_seed(L + n_dir)
  dev = "cuda"
  n_iter = 3
  rho = 0.5 if mode == "TRWP" else 1.0
  f32 = dict(dtype=torch.float32, device=dev)
  u8 = dict(dtype=torch.uint8, device=dev)
  unary = torch.randn(B, 1, H, W, L, generator=g).to(dev)
  if L == 21:
    context = torch.rand(L, L, generator=g).triu(1).to(dev)
  else:
    context = (0.3 * torch.arange(L, dtype=torch.float32).clamp(max=3)).to(dev)
  edge = (0.1 + 0.9 * torch.rand(n_dir, B, 1, H, W, generator=g)).to(dev)
  dcost = torch.randn(B, 1, H, W, L, generator=g).to(dev)
  msg = torch.zeros(n_dir, B, 1, H, W, L, **f32)
  msg_tmp = torch.zeros_like(msg)
  cost = torch.zeros(B, 1, H, W, L, **f32)
  belief = torch.zeros_like(cost)
  imin = torch.zeros(n_iter, n_dir, B, 1, H, W, L, **u8)
  inorm = torch.zeros(n_iter, n_dir, B, 1, H, W, **u8)
  label = torch.zeros(n_iter, B, 1, H, W, **u8)
  dunary = torch.zeros_like(cost)
  dmsg = torch.zeros_like(msg)
  dmsg_tmp = torch.zeros_like(msg)
  dscratch = torch.zeros_like(cost)
  dedge = torch.zeros(n_dir, B, 1, H, W, **f32)
  dctx = torch.zeros((L, L) if L == 21 else (L,), **f32)
  outputs = dict(msg=msg, cost=cost, imin=imin, inorm=inorm, label=label, dunary=dunary,
                 dedge=dedge, dctx=dctx)

  def step():
    # what a caller re-initialises per call: the initial messages and the accumulating gradients
    msg.zero_()
    dedge.zero_()
    dctx.zero_()
    dunary.zero_()
    if mode == "TRWP":
      lib_stereo.TRWP.forward(rho, n_iter, 0, unary, context, edge, msg, cost, imin, inorm, belief,
                              label)
      lib_stereo.TRWP.backward(rho, context, edge, dcost, imin, inorm, dunary, dctx, dedge, dmsg,
                               dscratch)
    else:
      lib_stereo.ISGMR.forward(0, rho, n_iter, 0, unary, context, edge, msg, cost, imin, inorm,
                               belief, msg_tmp, label)
      lib_stereo.ISGMR.backward(0, rho, context, edge, dcost, imin, inorm, dunary, dctx, dedge,
                                dmsg, dscratch, dmsg_tmp)

  step()
  torch.cuda.synchronize()
  eager = {k: v.clone() for k, v in outputs.items()}
  graph = torch.cuda.CUDAGraph()
  with torch.cuda.graph(graph):
    step()
  for replay in range(3):
    # eager work between replays: spoil every output and scratch buffer, then synchronise (the
    # index tensors are re-zeroed instead: chain-start pixels are never written and keep the
    # caller's zeros, as in the reference)
    for name, t in list(outputs.items()) + [("scratch", x) for x in (belief, msg_tmp, dmsg, dmsg_tmp, dscratch)]:
      t.zero_() if name in ("imin", "inorm") else t.fill_(3)
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    for name, want in eager.items():
      got = outputs[name]
      if name == "dctx":  # accumulated with float atomics: the order of the partial sums varies
        scale = max(1.0, float(want.abs().max()))
        assert float((got - want).abs().max()) <= 1e-4 * scale, (replay, name)
      else:
        assert torch.equal(got, want), (replay, name)
