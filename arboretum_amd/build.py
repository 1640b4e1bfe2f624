"""Builds libarboretum.so (host C++ + HIP kernels for gfx950) in-tree with hipcc."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libarboretum.so")
SOURCES = ["device_builder.hip", "exact_builder.hip", "hist_sum.hip", "quantiser.hip", "predictor.hip", "booster.cpp", "config.cpp",
           "wrapper.cpp"]
# -ffp-contract=off: the gain arithmetic must round exactly like the host
# restatement (no fused multiply-add).  packed-fp32-ops is switched off
# because some packed forms have produced wrong results on this hardware.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function",
         "-Wno-unknown-warning-option", "-pthread"]


def hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    raise RuntimeError("hipcc not found")


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd))
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout)
        raise RuntimeError("hipcc failed building libarboretum.so")
    if verbose and res.stdout:
        print(res.stdout)


def build(verbose=False, changed_only=False):
    """Compiles every source to an object file (in parallel) and links them.
    changed_only: keep the objects that are newer than their source and every header."""
    os.makedirs(OBJ, exist_ok=True)
    extra = os.environ.get("ARB_EXTRA_FLAGS", "").split()
    objs = [os.path.join(OBJ, os.path.splitext(s)[0] + ".o") for s in SOURCES]
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    headers += [os.path.join(HERE, "..", "include", f) for f in os.listdir(os.path.join(HERE, "..", "include"))]
    newest_header = max(os.path.getmtime(h) for h in headers)
    jobs = []
    for s, o in zip(SOURCES, objs):
        if changed_only and os.path.exists(o) and \
                os.path.getmtime(o) > max(newest_header, os.path.getmtime(os.path.join(CSRC, s))):
            continue
        jobs.append([hipcc()] + FLAGS + extra + ["-x", "hip", "-c", os.path.join(CSRC, s), "-o", o])
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        list(ex.map(lambda c: _run(c, verbose), jobs))
    _run([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-pthread"] + objs + ["-o", LIB], verbose)
    return LIB


if __name__ == "__main__":
    build(verbose=True, changed_only="--changed" in sys.argv[1:])
