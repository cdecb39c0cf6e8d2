"""Build libaddernet_hip.so for gfx950 with plain hipcc (no hipify, no torch extension).

The library has a C ABI (include/addernet_hip.h) and links only the HIP
runtime, so the Python side can load it with ctypes.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libaddernet_hip.so")
SOURCES = ["api.hip", "fwd.hip", "grad_x.hip", "grad_w.hip", "grad_w_mfma.hip", "conv1x1.hip", "col.hip", "bn_act.hip", "head.hip", "sgd.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    # keep hipcc from forming packed fp32 instructions out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _compile(src, verbose):
    obj = os.path.join(CSRC, src.replace(".hip", ".o"))
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode:
        raise RuntimeError(f"hipcc failed on {src}:\n{out}")
    if out.strip() and verbose:
        print(out)
    return obj


def build(verbose=False, jobs=4):
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, verbose), SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    build(verbose="-q" not in sys.argv)
    print("built", LIB)
