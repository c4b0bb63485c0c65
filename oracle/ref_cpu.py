"""TEST INFRASTRUCTURE ONLY: loader for the reference's compiled CPU forward path (_ref/*.so).

The modules are the reference's own pybind11 extensions built by build_ref.py; they take CPU
torch tensors with the operator signatures of MPLayers/TRWP/TRWP.cpp:245-256 and
MPLayers/ISGMR/ISGMR.cpp:300-313.  available() is False where they were not built.
"""
import importlib.util
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_mods = {}


def _path(name):
  return os.path.join(_HERE, "_ref", name + ".so")


def available():
  return os.path.exists(_path("ref_TRWP")) and os.path.exists(_path("ref_ISGMR"))


def module(name):
  if name not in _mods:
    import torch  # noqa: F401  (libtorch must be loaded first)
    spec = importlib.util.spec_from_file_location(name, _path(name))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    _mods[name] = mod
  return _mods[name]


def forward(mode, unary, context, n_dir, n_iter, rho, saving_label=False, enable_sgm=False):
  """Run the reference ForwardCPU.  unary (B,cv,H,W,L) fp32, context a (n_dir,L,L)-strided
  table (the CPU path reads `context + dir*L*L`, TRWP.cpp:205).  Returns msg, cost_final, label_all
  and unary_out (the SGM flag of ISGMR overwrites the unary tensor, ISGMR.cpp:255-261)."""
  import torch
  unary = torch.tensor(unary, dtype=torch.float32).contiguous()  # (a copy: may be overwritten)
  context = torch.as_tensor(context, dtype=torch.float32).contiguous()
  b, cv, h, w, L = unary.shape
  assert context.numel() >= n_dir * L * L
  msg = unary.new_zeros(n_dir, b, cv, h, w, L)
  cost = unary.new_zeros(b, cv, h, w, L)
  empty_u8 = torch.empty(0, dtype=torch.uint8)
  label = unary.new_zeros(n_iter, b, cv, h, w, dtype=torch.uint8) if saving_label else empty_u8
  edge = torch.empty(0)
  scratch = unary.new_zeros(b, cv, h, w, L)
  if mode == "TRWP":
    module("ref_TRWP").forward(float(rho), int(n_iter), 0, unary, context, edge, msg, cost,
                               empty_u8, empty_u8, scratch, label)
  else:
    msg_update = torch.zeros_like(msg)
    module("ref_ISGMR").forward(int(bool(enable_sgm)), float(rho), int(n_iter), 0, unary, context,
                                edge, msg, cost, empty_u8, empty_u8, scratch, msg_update, label)
  return dict(msg=msg.numpy(), cost_final=cost.numpy(), label_all=label.numpy(),
              unary_out=unary.numpy())
