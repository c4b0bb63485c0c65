"""Compile the reference's own CPU forward path (pybind11 modules) into oracle/_ref/.

TEST INFRASTRUCTURE ONLY.  The reference sources are compiled where they lie (nothing is
copied): MPLayers/TRWP/TRWP.cpp, MPLayers/ISGMR/ISGMR.cpp, MPLayers/common.cpp and
tools/cpp/utils.cpp, with the defines of the reference's MPLayers/setup.py:29,58-61 for a
CPU-only build (no USE_CUDA).  Output: _ref/ref_TRWP.so, _ref/ref_ISGMR.so.  Usage:

    python3 build_ref.py [/root/reference]
"""
import os
import subprocess
import sys
import sysconfig


def main():
  ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
  here = os.path.dirname(os.path.abspath(__file__))
  out = os.path.join(here, "_ref")
  if not os.path.isdir(os.path.join(ref, "MPLayers")):
    print("reference tree not found at %s: nothing built" % ref)
    return 0
  import torch
  from torch.utils import cpp_extension
  os.makedirs(out, exist_ok=True)
  inc = cpp_extension.include_paths() + [sysconfig.get_paths()["include"],
                                         os.path.join(ref, "MPLayers"),
                                         os.path.join(ref, "tools", "cpp")]
  libdir = os.path.join(os.path.dirname(torch.__file__), "lib")
  common = [os.path.join(ref, "MPLayers", "common.cpp"), os.path.join(ref, "tools", "cpp", "utils.cpp")]
  for name, src in (("ref_TRWP", os.path.join(ref, "MPLayers", "TRWP", "TRWP.cpp")),
                    ("ref_ISGMR", os.path.join(ref, "MPLayers", "ISGMR", "ISGMR.cpp"))):
    cmd = ["g++", "-O2", "-std=c++17", "-fopenmp", "-shared", "-fPIC", "-w",
           "-DTORCH_VERSION_MAJOR=2", "-DMAX_DISPARITY=256", "-DTORCH_EXTENSION_NAME=" + name,
           "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
    cmd += ["-I" + p for p in inc] + [src] + common
    cmd += ["-L" + libdir, "-Wl,-rpath," + libdir, "-lc10", "-ltorch", "-ltorch_cpu", "-ltorch_python",
            "-o", os.path.join(out, name + ".so")]
    print(" ".join(cmd))
    subprocess.check_call(cmd)
  return 0


if __name__ == "__main__":
  sys.exit(main())
