"""Builds the gfx950 device library (libfnx_mi355x.so) in-tree with hipcc. No GPU is needed to build."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libfnx_mi355x.so")
SOURCES = ["fnx_verify.hip"]
FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off",                       # fused multiply-adds only where the code says fmaf: part of the results' definition
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-amdgpu-mfma-vgpr-form",       # matrix-core results in the ordinary registers: the kernels here take them up with vector instructions right away
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]


def build(verbose=False, extra=()):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *FLAGS, *extra, "-o", LIB] + [os.path.join(CSRC, s) for s in SOURCES]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(l for l in (r.stdout + r.stderr).splitlines() if "packed-fp32-ops" not in l and l.strip())
    if r.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out:
        print(out)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, extra=sys.argv[1:]))
