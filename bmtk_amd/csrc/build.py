"""Compile the HIP sources into ``bmtk_amd/libbmtk_amd.so`` for gfx950.

Run as ``python -m bmtk_amd.csrc.build``.  hipcc cross-compiles without a GPU.
Flags that matter for results:
  -ffp-contract=off      no fused multiply-add, so the fp32 update rounds like a
                         scalar evaluation of the same expressions;
  -munsafe-fp-atomics    fp32 atomicAdd becomes the hardware global atomic
                         instead of a compare-and-swap loop (device memory only);
  -packed-fp32-ops off   no packed fp32 instructions are generated.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
LIB = os.path.join(PKG, "libbmtk_amd.so")
SOURCES = ["kernels.hip", "propagate_pull.hip", "simulate.hip", "simulate_fused.hip", "resident.hip", "resident_solo.hip", "backward.hip", "poisson.hip", "microbench.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
         "-munsafe-fp-atomics", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wall", "-Wno-unused-function"]


def build(verbose=False, extra=()):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + FLAGS + list(extra) + ["-o", LIB] + [os.path.join(HERE, s) for s in SOURCES]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, extra=sys.argv[1:]))
