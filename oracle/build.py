"""Build the CPU oracle shared library (test infrastructure, not product code).

    python oracle/build.py

compiles oracle/vl_oracle.c with gcc into oracle/libvloracle.so.  The reference
is pure Python/Numba with no compilable sources, so there is no oracle/_ref
build: the oracle is pinned by known-answer vectors and closed forms instead.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "vl_oracle.c")
OUT = os.path.join(HERE, "libvloracle.so")


def build(force: bool = True) -> str:
    if not force and os.path.exists(OUT) and os.path.getmtime(OUT) >= os.path.getmtime(SRC):
        return OUT
    cmd = ["gcc", "-O2", "-ffp-contract=off", "-fopenmp", "-fvisibility=hidden",
           "-shared", "-fPIC", "-Wall", "-Wextra", "-o", OUT, SRC, "-lm"]
    subprocess.run(cmd, check=True)
    return OUT


if __name__ == "__main__":
    print(build(force=True))
    sys.exit(0)
