"""Pins of the soft-weighted TRWP oracle (restating MPLayers/TRWP_hard_soft).  The reference has no
CPU build of this operator and no fixtures, so the restatement is checked against what the
mathematics fixes:
  * the soft message is -d/d(beta) log sum_fd exp(-beta * dual) at beta = 1 (independent fp64 chain
    recursion built on scipy's logsumexp and a central difference in beta),
  * with well-separated costs the softmin collapses onto the min: soft TRWP == hard TRWP,
  * the stored (L, L) blocks have the layout of TRWP_forward_soft.cu:64 (even directions [fd][cd],
    odd ones [cd][fd]),
  * the backward pass equals central finite differences of the forward pass in fp64.
"""
import numpy as np
import pytest
from scipy.special import logsumexp


def ctx_table(ctx, L):
  if ctx.ndim == 1:
    return ctx[np.abs(np.arange(L)[:, None] - np.arange(L)[None, :])]
  up = np.triu(ctx)
  return up + np.triu(ctx, 1).T


def soft_expect(dual):
  """sum_fd softmax(-dual) * dual along the last axis, as a derivative of logsumexp."""
  h = 1e-6
  f = lambda beta: logsumexp(-beta * dual, axis=-1)
  return -(f(1 + h) - f(1 - h)) / (2 * h)


def test_single_row_matches_logsumexp_derivative(oracle):
  rng = np.random.default_rng(0)
  L, W = 5, 6
  unary = rng.random((1, 1, 1, W, L))
  ctx = np.array([0.0, 0.3, 0.7, 0.9, 0.9])
  ew = 0.5 + rng.random((2, 1, 1, 1, W))
  rho = 0.7
  out = oracle.forward_soft(unary, ctx, ew, 2, 1, rho)
  tab = ctx_table(ctx, L)
  # direction 0 (left to right), first iteration: U = rho * unary (all messages are zero);
  # recurrence a = U[front] + rho * m[front]
  m0 = np.zeros((W, L))
  for x in range(1, W):
    a = rho * unary[0, 0, 0, x - 1] + rho * m0[x - 1]
    dual = a[None, :] + ew[0, 0, 0, 0, x] * tab          # [cd, fd]
    soft = soft_expect(dual)
    m0[x] = soft - soft.min()
    np.testing.assert_allclose(out["msg"][0, 0, 0, 0, x], m0[x], atol=2e-9)
  assert np.all(out["msg"][0, 0, 0, 0, 0] == 0)
  # direction 1 runs right to left and already sees direction 0's messages:
  # U = rho * (unary + m0 + m1 - m1) - m0 with m1 still zero
  U = rho * (unary[0, 0, 0] + m0) - m0
  m1 = np.zeros((W, L))
  for x in range(W - 2, -1, -1):
    a = U[x + 1] + rho * m1[x + 1]
    dual = a[None, :] + ew[1, 0, 0, 0, x] * tab
    soft = soft_expect(dual)
    m1[x] = soft - soft.min()
    np.testing.assert_allclose(out["msg"][1, 0, 0, 0, x], m1[x], atol=2e-9)
  np.testing.assert_allclose(out["cost_final"], unary + out["msg"].sum(0), atol=1e-12)


@pytest.mark.parametrize("n_dir,L,ctx2d", [(4, 6, False), (8, 5, False), (16, 4, False), (8, 5, True)])
def test_separated_costs_reduce_to_hard_trwp(oracle, n_dir, L, ctx2d):
  rng = np.random.default_rng(n_dir + L)
  B, H, W, n_iter = 2, 5, 6, 2
  scale = 64.0  # integer costs times 64: competing candidates differ by >= 32, exp(-32) ~ 1e-14
  unary = scale * rng.integers(0, 6, (B, 1, H, W, L)).astype(np.float64)
  if ctx2d:
    ctx = scale * np.triu(rng.integers(1, 4, (L, L)), 1).astype(np.float64)
  else:
    ctx = scale * np.minimum(np.arange(L), 2).astype(np.float64)
  ew = rng.integers(1, 3, (n_dir, B, 1, H, W)).astype(np.float64)
  # rho = 1 keeps every intermediate value a multiple of 64 (rho < 1 would shrink the gaps along
  # a chain); the rho terms are covered by the single-row and the layout tests
  soft = oracle.forward_soft(unary, ctx, ew, n_dir, n_iter, 1.0, ctx2d=ctx2d, saving_label=True)
  hard = oracle.forward("TRWP", unary, ctx, ew, n_dir, n_iter, 1.0, ctx2d=ctx2d, saving_label=True)
  np.testing.assert_allclose(soft["msg"], hard["msg"], atol=1e-9)
  np.testing.assert_allclose(soft["cost_final"], hard["cost_final"], atol=1e-9)
  np.testing.assert_array_equal(soft["label_all"], hard["label_all"])
  # exact ties between normalised candidates pick the largest label in both operators
  np.testing.assert_array_equal(soft["msg_norm_index"], hard["msg_norm_index"])


def test_edge_label_layout(oracle):
  rng = np.random.default_rng(2)
  L, H, W, rho = 3, 2, 4, 0.5
  unary = rng.random((1, 1, H, W, L))
  ctx = np.array([0.0, 0.4, 1.0])
  ew = 0.5 + rng.random((4, 1, 1, H, W))
  out = oracle.forward_soft(unary, ctx, ew, 4, 1, rho)
  blocks = out["msg_edge_label"]
  assert blocks.shape == (1, 4, 1, 1, H, W, L, L)
  tab = ctx_table(ctx, L)
  # direction 0, second pixel of a row: its front pixel is a chain start (message 0) and all
  # messages are still zero, so dual[cd, fd] = rho * unary[front, fd] + w * ctx(cd, fd)
  dual = rho * unary[0, 0, 1, 0][None, :] + ew[0, 0, 0, 1, 1] * tab
  np.testing.assert_allclose(blocks[0, 0, 0, 0, 1, 1], dual.T, atol=1e-12)   # [fd][cd]
  assert np.all(blocks[0, 0, 0, 0, :, 0] == 0)                                 # chain starts
  # direction 2 (top to bottom) is even as well; direction 3 (bottom to top) stores [cd][fd]
  m = out["msg"]
  d = 3
  # U of direction 3 when it runs: rho * (unary + m0 + m1 + m2 + m3 - m3) - m2 with m3 still zero
  U = rho * (unary[0, 0] + m[0, 0, 0] + m[1, 0, 0] + m[2, 0, 0]) - m[2, 0, 0]
  dual3 = U[1, 2][None, :] + ew[d, 0, 0, 0, 2] * tab     # pixel (0, 2), front pixel (1, 2)
  np.testing.assert_allclose(blocks[0, d, 0, 0, 0, 2], dual3, atol=1e-12)      # [cd][fd]


@pytest.mark.parametrize("n_dir,ctx2d", [(4, False), (8, True), (16, False)])
def test_backward_matches_finite_differences(oracle, n_dir, ctx2d):
  rng = np.random.default_rng(7 + n_dir)
  B, H, W, L, n_iter, rho = 1, 4, 5, 4, 2, 0.5
  unary = rng.random((B, 1, H, W, L))
  ctx = np.triu(rng.random((L, L))) if ctx2d else np.sort(rng.random(L))
  ew = 0.5 + rng.random((n_dir, B, 1, H, W))
  R = rng.standard_normal((B, 1, H, W, L))

  def loss(u, c, e):
    return float((oracle.forward_soft(u, c, e, n_dir, n_iter, rho, ctx2d=ctx2d)["cost_final"] * R).sum())

  fwd = oracle.forward_soft(unary, ctx, ew, n_dir, n_iter, rho, ctx2d=ctx2d)
  du, dc, de = oracle.backward_soft(ctx, ew, R, fwd["msg_edge_label"], fwd["msg_norm_index"], rho,
                                    ctx2d=ctx2d)
  h = 1e-6

  def fd(arr, idx, which):
    p, m = arr.copy(), arr.copy()
    p[idx] += h
    m[idx] -= h
    args = {"u": unary, "c": ctx, "e": ew}
    ap, am = dict(args), dict(args)
    ap[which], am[which] = p, m
    return (loss(ap["u"], ap["c"], ap["e"]) - loss(am["u"], am["c"], am["e"])) / (2 * h)

  for _ in range(12):
    idx = tuple(rng.integers(0, s) for s in unary.shape)
    assert abs(fd(unary, idx, "u") - du[idx]) < 1e-6 * max(1, abs(du).max())
  for _ in range(8):
    idx = tuple(rng.integers(0, s) for s in ew.shape)
    assert abs(fd(ew, idx, "e") - de[idx]) < 1e-6 * max(1, abs(de).max())
  if ctx2d:
    for i in range(L):
      for j in range(i, L):   # only the upper triangle (diagonal included) is read
        assert abs(fd(ctx, (i, j), "c") - dc[i, j]) < 1e-6 * max(1, abs(dc).max())
    assert np.all(np.tril(dc, -1) == 0)
  else:
    for k in range(L):
      assert abs(fd(ctx, (k,), "c") - dc[k]) < 1e-6 * max(1, abs(dc).max())
  # every normalised message has zero net gradient mass, and the softmin weights sum to one:
  # the gradient mass of cost_final reaches dunary unchanged
  ones = np.ones_like(R)
  du1, _, _ = oracle.backward_soft(ctx, ew, ones, fwd["msg_edge_label"], fwd["msg_norm_index"], rho,
                                   ctx2d=ctx2d)
  np.testing.assert_allclose(du1.sum(), ones.sum(), rtol=1e-9)


def test_soft_weighted_message_oracle():
  """Stand-alone softmin of stored blocks: forward against the logsumexp derivative, backward
  against central finite differences."""
  rng = np.random.default_rng(5)
  T, L = 4, 6
  m = rng.random((T, L, L)) * 3
  norm, ind = soft_oracle().soft_weighted_message(m)
  soft = soft_expect(np.swapaxes(m, 1, 2))                 # [cd][fd] rows
  np.testing.assert_allclose(norm, soft - soft.min(axis=1, keepdims=True), atol=2e-9)
  np.testing.assert_array_equal(ind, soft.argmin(axis=1))
  # ties pick the largest label
  m2 = np.tile(m[:1, :, :1], (1, 1, L))
  assert soft_oracle().soft_weighted_message(m2)[1][0] == L - 1
  R = rng.standard_normal((T, L))
  dm = soft_oracle().soft_weighted_message_back(R, m, ind)
  h = 1e-6
  for _ in range(20):
    idx = tuple(rng.integers(0, s) for s in m.shape)
    p, q = m.copy(), m.copy()
    p[idx] += h
    q[idx] -= h
    fd = ((soft_oracle().soft_weighted_message(p)[0] - soft_oracle().soft_weighted_message(q)[0]) * R).sum() / (2 * h)
    assert abs(fd - dm[idx]) < 1e-6


def soft_oracle():
  from oracle import mp_oracle
  return mp_oracle
