"""Compiles csrc/mp_kernels.hip into libmplayers_hip.so (gfx950 only) with hipcc."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "csrc", "mp_kernels.hip")
LIB = os.path.join(HERE, "libmplayers_hip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-munsafe-fp-atomics",
    # packed fp32 instructions are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-shared", "-fPIC",
]


def build(verbose=False):
  """Always recompiles; returns the path of the shared library."""
  hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
  cmd = [hipcc] + HIPCC_FLAGS + [SRC, "-o", LIB]
  if verbose:
    print(" ".join(cmd))
  proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
  out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
  if proc.returncode != 0:
    raise RuntimeError("hipcc failed:\n" + out)
  if verbose and out.strip():
    print(out)
  return LIB


if __name__ == "__main__":
  print(build(verbose=True))
