"""Compile the HIP sources under csrc/ into vectorlink_gpu/libvlgpu.so for gfx950.

    python vectorlink-gpu_amd/build.py

hipcc cross-compiles without a GPU present.  The library is built in-tree so
that it travels with the source tree to the machine that runs it.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
OUT = os.path.join(HERE, "vectorlink_gpu", "libvlgpu.so")

SOURCES = ["error.cpp", "dist.hip", "queue.hip", "prune.hip", "beam.hip", "knn.hip", "graphopt.hip", "sketch.hip"]

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-ffp-contract=off",  # every fused multiply-add in the kernels is written explicitly
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = ["hipcc", "-x", "hip", *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        print(err, file=sys.stderr)
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    sources = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    with ThreadPoolExecutor(max_workers=min(8, len(sources))) as ex:
        objs = list(ex.map(_compile, sources))
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT, *objs]
    subprocess.run(cmd, check=True)
    if verbose:
        print(OUT)
    return OUT


if __name__ == "__main__":
    build()
