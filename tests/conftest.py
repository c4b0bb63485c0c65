import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
  sys.path.insert(0, ROOT)


def pytest_configure(config):
  config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
  from oracle import mp_oracle
  mp_oracle.build()
  return mp_oracle


@pytest.fixture(scope="session")
def gpu():
  """Helpers of the GPU parity tests; fails (not skips) without a GPU or without the HIP library."""
  import torch
  assert torch.cuda.is_available(), "these tests need the MI355X"
  from mplayers_amd import _lib
  _lib.load()
  from tests import _gpu_util
  return _gpu_util
