"""Compiles the HIP sources under csrc/ into libmplayers_hip.so (gfx950 only) with hipcc.

The scan kernels are instantiated once per R (labels per lane, 1..4); each instantiation is its
own translation unit so that they compile in parallel.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libmplayers_hip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-munsafe-fp-atomics", "-fno-honor-nans",
    # packed fp32 instructions are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fPIC",
]


def _units():
  units = [("mp_api", "mp_api.hip", []), ("mp_edge", "mp_edge.hip", []),
           ("mp_soft", "mp_soft.hip", []), ("mp_pack", "mp_pack.hip", []),
           ("mp_terms", "mp_terms.hip", []), ("mp_probe", "mp_probe.hip", []),
           ("mp_layout", "mp_layout.hip", [])]
  for r in (1, 2, 3, 4):
    units.append(("mp_fwd_r%d" % r, "mp_fwd.hip", ["-DMPL_INST_R=%d" % r]))
    units.append(("mp_bwd_r%d" % r, "mp_bwd.hip", ["-DMPL_INST_R=%d" % r]))
  return units


def _run(cmd):
  proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
  out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
  if proc.returncode != 0:
    raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
  return out


def build(verbose=False, extra_flags=(), lib_path=LIB, jobs=None):
  """Always recompiles; returns the path of the shared library."""
  hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
  obj_dir = OBJ if lib_path == LIB else lib_path + ".build"
  os.makedirs(obj_dir, exist_ok=True)
  jobs = jobs or min(8, os.cpu_count() or 1)
  cmds, objs = [], []
  for name, src, defs in _units():
    obj = os.path.join(obj_dir, name + ".o")
    objs.append(obj)
    cmds.append([hipcc] + HIPCC_FLAGS + list(extra_flags) + defs +
                ["-c", os.path.join(CSRC, src), "-o", obj])
  with ThreadPoolExecutor(max_workers=jobs) as pool:
    for cmd, out in zip(cmds, pool.map(_run, cmds)):
      if verbose:
        print(" ".join(cmd))
        if out.strip():
          print(out)
  link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", lib_path]
  out = _run(link)
  if verbose:
    print(" ".join(link))
    if out.strip():
      print(out)
  return lib_path


if __name__ == "__main__":
  print(build(verbose="-q" not in sys.argv))
