"""mpl_edge_shift_static: the edge-weight producer with library-owned static scratch, for callers
that cannot allocate.  Called through the C ABI and compared bit for bit with mpl_edge_shift
(which takes the scratch as a workspace argument) on two calls in a row, the second one on a
smaller image, so that a call that relied on what the previous one left in the shared array
would show."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

MODE_CUE_BINARY, MODE_CUE_REAL, MODE_EXP = 6, 5, 4


def _call(lib, static, mode, img, n_dirs, sigma, sums):
  import torch
  from mplayers_amd import _lib
  b, c, h, w = img.shape
  out = torch.full((n_dirs, b, c, h, w), -7.0, device=img.device)
  stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
  args = [mode, ctypes.c_void_p(img.data_ptr()), b, c, h, w, n_dirs, ctypes.c_float(sigma),
          ctypes.c_float(0.0), ctypes.c_float(0.0), ctypes.c_void_p(out.data_ptr())]
  if static:
    rc = lib.mpl_edge_shift_static(*args, stream)
  else:
    rc = lib.mpl_edge_shift(*args, ctypes.c_void_p(sums.data_ptr()), stream)
  _lib.check(rc, "edge_shift_static" if static else "edge_shift")
  torch.cuda.synchronize()
  return out.cpu().numpy()


def test_static_scratch_entry_point_matches_the_workspace_one(gpu):
  import torch
  from mplayers_amd import _lib
  lib = _lib.load()
  rng = np.random.default_rng(5)
  sums = torch.empty(16, dtype=torch.float64, device="cuda")
  # two calls in a row, the second on a smaller image with fewer directions
  for (c, h, w, n_dirs) in ((3, 61, 83, 16), (2, 17, 23, 8)):
    img = torch.from_numpy((rng.random((1, c, h, w)) * 40).astype(np.float32)).cuda()
    print("case", c, h, w, n_dirs, flush=True)
    for mode in (MODE_CUE_BINARY, MODE_CUE_REAL):
      want = _call(lib, False, mode, img, n_dirs, 10.0, sums)
      got = _call(lib, True, mode, img, n_dirs, 10.0, sums)
      assert np.array_equal(got, want), (mode, c, h, w)
      if mode == MODE_CUE_BINARY:
        # the threshold (0.8 of the mean held in the scratch) really splits the pixels
        assert set(np.unique(got)) <= {0.0, 1.0} and 0.05 < (got == 1.0).mean() < 0.95
  # a per-channel mode with a batch: no scratch involved, same results
  img = torch.from_numpy(rng.random((2, 3, 9, 11)).astype(np.float32)).cuda()
  assert np.array_equal(_call(lib, True, MODE_EXP, img, 4, 1.0, sums),
                        _call(lib, False, MODE_EXP, img, 4, 1.0, sums))


def test_static_scratch_entry_point_refuses_what_it_cannot_hold(gpu):
  from mplayers_amd import _lib
  lib = _lib.load()
  one = ctypes.c_void_p(256)  # never dereferenced: validation answers first
  f = ctypes.c_float(1.0)
  assert lib.mpl_edge_shift_static(MODE_CUE_BINARY, one, 1, 3, 8, 8, 17, f, f, f, one, None) == -1
  assert b"static scratch" in lib.mpl_last_error()
  assert lib.mpl_edge_shift_static(MODE_CUE_BINARY, one, 2, 3, 8, 8, 4, f, f, f, one, None) == -1
  assert b"batch == 1" in lib.mpl_last_error()
