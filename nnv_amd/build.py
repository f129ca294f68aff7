"""Build recipe for libnnvhip.so (gfx950 only): hipcc on the sources in csrc/, in-tree output.

    python -m nnv_amd.build
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "libnnvhip.so")
SOURCES = ["ctx.hip", "sets.hip", "weights.hip", "fc_layer.hip", "layers.hip", "gemm.hip", "gemm_seg.hip", "conv.hip", "ranges.hip", "relu.hip", "chain.hip", "spec.hip", "elementwise.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-Wno-unknown-warning-option",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), p.stdout))
    return p.stdout


def build(verbose: bool = False, jobs: int = 8) -> str:
    """Compile every HIP source for gfx950 and link nnv_amd/libnnvhip.so.  Always recompiles."""
    os.makedirs(OBJ, exist_ok=True)
    objs = [os.path.join(OBJ, s.replace(".hip", ".o")) for s in SOURCES]

    def one(pair):
        src, obj = pair
        out = _run([HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])
        if verbose and out.strip():
            print(out)

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(one, zip(SOURCES, objs)))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
