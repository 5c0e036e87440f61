"""Build the C oracle (test infrastructure) into oracle/_build/libaq_oracle.so.

The reference is pure Python and holds no compilable sources for this path, so
there is no oracle/_ref build: the C file here is the only CPU restatement.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "aq_oracle.c")
OUT_DIR = os.path.join(HERE, "_build")
OUT = os.path.join(OUT_DIR, "libaq_oracle.so")


def build(force: bool = True) -> str:
    os.makedirs(OUT_DIR, exist_ok=True)
    if not force and os.path.exists(OUT) and os.path.getmtime(OUT) >= os.path.getmtime(SRC):
        return OUT
    # -march=x86-64-v3 rather than native: the library is built in one container
    # and run on another host; AVX2 is present on both.
    cmd = [
        "gcc", "-O3", "-march=x86-64-v3", "-fopenmp", "-ffp-contract=off", "-fno-fast-math",
        "-shared", "-fPIC", "-o", OUT, SRC, "-lm",
    ]
    subprocess.run(cmd, check=True)
    return OUT


if __name__ == "__main__":
    print(build(force="--if-stale" not in sys.argv))
