"""Builds the pybind11 operator modules of mpl_torch_binding.cpp against libmplayers_hip.so:

    tests/binding/_built/lib_stereo/{TRWP,ISGMR}.so     (and the same two under lib_seg/)

which is the directory layout the reference's setup.py leaves under MPLayers/ and
pytorch/MP_module.py:4-8 imports from.  Host code only: g++ with the torch and HIP headers, linked
to the C ABI library (found at run time through an rpath relative to the module).  Usage:

    python3 tests/binding/build_binding.py
"""
import os
import shutil
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
OUT = os.path.join(HERE, "_built")


def build(verbose=True):
  import torch
  from torch.utils import cpp_extension
  libdir = os.path.join(ROOT, "mplayers_amd")
  if not os.path.exists(os.path.join(libdir, "libmplayers_hip.so")):
    raise RuntimeError("build libmplayers_hip.so first: python -m mplayers_amd._build")
  torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
  inc = cpp_extension.include_paths() + [sysconfig.get_paths()["include"],
                                         os.path.join(ROOT, "include"), "/opt/rocm/include"]
  stereo = os.path.join(OUT, "lib_stereo")
  seg = os.path.join(OUT, "lib_seg")
  os.makedirs(stereo, exist_ok=True)
  os.makedirs(seg, exist_ok=True)
  procs = []
  for name in ("TRWP", "ISGMR"):
    cmd = ["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-w",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DMPL_BIND_" + name,
           "-DTORCH_EXTENSION_NAME=" + name, "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
    cmd += ["-I" + p for p in inc] + [os.path.join(HERE, "mpl_torch_binding.cpp")]
    cmd += ["-L" + libdir, "-lmplayers_hip", "-Wl,-rpath,$ORIGIN/../../../../mplayers_amd",
            "-L" + torch_lib, "-Wl,-rpath," + torch_lib, "-lc10", "-lc10_hip", "-ltorch",
            "-ltorch_cpu", "-ltorch_python", "-o", os.path.join(stereo, name + ".so")]
    if verbose:
      print(" ".join(cmd))
    procs.append((name, subprocess.Popen(cmd)))
  for name, proc in procs:
    if proc.wait() != 0:
      raise RuntimeError("building the %s binding failed" % name)
    # the reference builds the same sources a second time with MAX_DISPARITY = 32 for lib_seg
    # (MPLayers/setup.py:58-61); one library backs both here
    shutil.copyfile(os.path.join(stereo, name + ".so"), os.path.join(seg, name + ".so"))
  return OUT


if __name__ == "__main__":
  print(build(verbose="-q" not in sys.argv))
