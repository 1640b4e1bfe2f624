"""Builds libarboretum.so (host C++ + HIP kernels for gfx950) in-tree with hipcc."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libarboretum.so")
SOURCES = ["device_builder.hip", "quantiser.hip", "predictor.hip", "booster.cpp", "config.cpp", "wrapper.cpp"]
# -ffp-contract=off: the gain arithmetic must round exactly like the host
# restatement (no fused multiply-add).  packed-fp32-ops is switched off
# because some packed forms have produced wrong results on this hardware.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function",
         "-Wno-unknown-warning-option", "-pthread"]


def hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    raise RuntimeError("hipcc not found")


def build(verbose=False):
    cmd = [hipcc()] + FLAGS + os.environ.get("ARB_EXTRA_FLAGS", "").split() + ["-x", "hip"] + [os.path.join(CSRC, s) for s in SOURCES] + ["-o", LIB]
    if verbose:
        print(" ".join(cmd))
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout)
        raise RuntimeError("hipcc failed building libarboretum.so")
    if verbose and res.stdout:
        print(res.stdout)
    return LIB


if __name__ == "__main__":
    build(verbose=True)
