"""Writes tests/golden/refcpu_*.npz: inputs and outputs of the reference's own CPU forward
path (MPLayers/TRWP/TRWP.cpp:172-243, MPLayers/ISGMR/ISGMR.cpp:190-298), produced by the
modules that oracle/build_ref.py compiles from the reference sources.  Run once in the build
container (the reference tree does not travel):

    make -C oracle ref && python3 tests/golden/make_refcpu_golden.py

Each fixture holds: mode, rho, n_dir, n_iter, unary (B,cv,H,W,L), context (n_dir,L,L) and the
reference's msg, cost_final and label_all (the later ones also unary_out, the unary tensor after
the call, which the SGM flag overwrites).  Fixtures that exist are kept unless --all is given.  Inputs are integer valued in half of the cases so
that every fp32 operation is exact and comparisons can be bitwise.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import ref_cpu  # noqa: E402

CASES = [
    # name, mode, rho, n_dir, n_iter, B, H, W, L, integer inputs, symmetric shared 1-D context
    ("trwp_d4_l5", "TRWP", 0.5, 4, 3, 2, 7, 9, 5, False, True),
    ("trwp_d8_l21", "TRWP", 0.5, 8, 2, 1, 6, 8, 21, False, False),
    ("trwp_d16_l4_int", "TRWP", 0.5, 16, 2, 1, 9, 7, 4, True, True),
    ("isgmr_d4_l16", "ISGMR", 1.0, 4, 3, 1, 8, 12, 16, False, True),
    ("isgmr_d8_l21_int", "ISGMR", 1.0, 8, 3, 2, 5, 6, 21, True, False),
    ("isgmr_d16_l6", "ISGMR", 1.0, 16, 2, 1, 10, 11, 6, False, True),
    # the SGM flag of the ISGMR operator (unary read at the current pixel and replaced after
    # every iteration, ISGMR.cpp:72-77, 255-261) and the label loop at 256 labels (common.cpp:152)
    ("sgm_d4_l8", "SGM", 1.0, 4, 2, 2, 6, 7, 8, False, True),
    ("sgm_d8_l21_int", "SGM", 1.0, 8, 3, 1, 5, 6, 21, True, False),
    ("trwp_d4_l256", "TRWP", 0.5, 4, 1, 1, 3, 4, 256, False, True),
]


def main():
  assert ref_cpu.available(), "run `make -C oracle ref` first"
  for i, (name, mode, rho, n_dir, n_iter, B, H, W, L, integer, shared) in enumerate(CASES):
    rng = np.random.default_rng(100 + i)
    if integer:
      unary = rng.integers(0, 255, (B, 1, H, W, L)).astype(np.float32)
    else:
      unary = rng.random((B, 1, H, W, L)).astype(np.float32)
    if shared:
      # one symmetric Toeplitz table repeated for every direction: ctx[d, i, j] = c[|i-j|]
      c = rng.integers(0, 6, L).astype(np.float32) if integer else rng.random(L).astype(np.float32)
      c[0] = 0
      ii = np.abs(np.arange(L)[:, None] - np.arange(L)[None, :])
      context = np.broadcast_to(c[ii], (n_dir, L, L)).copy()
    else:
      context = rng.integers(0, 6, (n_dir, L, L)).astype(np.float32) if integer else \
          rng.random((n_dir, L, L)).astype(np.float32)
    path = os.path.join(HERE, "refcpu_%s.npz" % name)
    if os.path.exists(path) and "--all" not in sys.argv:
      continue  # fixtures already written are kept as they are
    if name == "trwp_d4_l256":
      context = context[:, :1, :].copy()  # one row per direction is all a 1-D table needs ...
      context = np.concatenate([context.reshape(n_dir, L), np.zeros((n_dir, L * L - L), np.float32)],
                               axis=1).reshape(n_dir, L, L)  # ... at the stride of a full table
    out = ref_cpu.forward(mode, unary, context, n_dir, n_iter, rho, saving_label=True,
                          enable_sgm=(mode == "SGM"))
    np.savez_compressed(path, mode=mode, rho=rho,
                        n_dir=n_dir, n_iter=n_iter, unary=unary, context=context,
                        msg=out["msg"], cost_final=out["cost_final"], label_all=out["label_all"],
                        unary_out=out["unary_out"])
    print(name, out["msg"].shape, float(np.abs(out["msg"]).max()))


if __name__ == "__main__":
  main()
