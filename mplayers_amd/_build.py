"""Compiles the HIP sources under csrc/ into libmplayers_hip.so (gfx950 only) with hipcc, and the
measurement probes (csrc/mp_probe.hip) into libmplayers_probe.so, which only the benchmark and the
tests load.

The scan kernels are instantiated once per R (labels per lane, 1..4), the forward scans also once
with and once without argmin labels; each instantiation is its own translation unit so that they
compile in parallel.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libmplayers_hip.so")
PROBE_LIB = os.path.join(HERE, "libmplayers_probe.so")
PROBE_UNITS = ("mp_probe",)  # objects of the probe library; every other unit is the product's

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-munsafe-fp-atomics", "-fno-honor-nans",
    # packed fp32 instructions are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fPIC",
    # "#pragma unroll" on loops whose trip count is a run-time value in some instantiations
    "-Wno-pass-failed",
]


def _units():
  units = [("mp_api", "mp_api.hip", []), ("mp_edge", "mp_edge.hip", []),
           ("mp_soft", "mp_soft.hip", []), ("mp_pack", "mp_pack.hip", []),
           ("mp_terms", "mp_terms.hip", []), ("mp_probe", "mp_probe.hip", []),
           ("mp_layout", "mp_layout.hip", [])]
  for r in (4, 3, 2, 1):  # (the largest units first)
    for t in (1, 0):
      units.append(("mp_fwd_r%d_t%d" % (r, t), "mp_fwd.hip",
                    ["-DMPL_INST_R=%d" % r, "-DMPL_INST_TRAIN=%d" % t]))
    units.append(("mp_bwd_r%d" % r, "mp_bwd.hip", ["-DMPL_INST_R=%d" % r]))
  return units


# host-only sources (the CPU forward path), compiled with the host compiler; no fused multiply-adds,
# so that the arithmetic is the reference's own (g++ -O2 on x86-64 contracts nothing)
HOST_UNITS = [("mp_cpu", os.path.join("cpu", "mp_cpu.cpp"))]
HOST_FLAGS = ["-O3", "-ffp-contract=off", "-std=c++17", "-fPIC", "-pthread", "-Wall", "-Wextra"]


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
  cxx = os.environ.get("CXX", "g++")
  for name, src in HOST_UNITS:
    cmds.append([cxx] + HOST_FLAGS + ["-c", os.path.join(CSRC, src), "-o",
                                      os.path.join(obj_dir, name + ".o")])
  with ThreadPoolExecutor(max_workers=jobs) as pool:
    for cmd, out in zip(cmds, pool.map(_run, cmds)):
      if verbose:
        print(" ".join(cmd))
        if out.strip():
          print(out)
  link(lib_path=lib_path, verbose=verbose)
  return lib_path


def link(lib_path=LIB, verbose=False):
  """Links the objects that are there into the product library and the probe library."""
  hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
  obj_dir = OBJ if lib_path == LIB else lib_path + ".build"
  probe_path = PROBE_LIB if lib_path == LIB else lib_path.replace(".so", "_probe.so")
  names = [name for name, _, _ in _units()]
  host = [name for name, _ in HOST_UNITS]
  groups = ((lib_path, [n for n in names if n not in PROBE_UNITS] + host, ["-lpthread"]),
            (probe_path, [n for n in names if n in PROBE_UNITS], []))
  for path, members, libs in groups:
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + \
        [os.path.join(obj_dir, n + ".o") for n in members] + libs + ["-o", path]
    out = _run(cmd)
    if verbose:
      print(" ".join(cmd))
      if out.strip():
        print(out)


if __name__ == "__main__":
  print(build(verbose="-q" not in sys.argv))
