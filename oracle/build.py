"""Build the C oracle into oracle/_build/liboracle.so (gcc, -O2, OpenMP).

TEST INFRASTRUCTURE ONLY.  The reference's own implementation of this path is CUDA
behind an import-time nvcc build, so it cannot be compiled in this image; there is
therefore no oracle/_ref build and the restatement is pinned by the checks listed in
the headers of lfw_ref.py / lfw_oracle.c.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
OUT_DIR = os.path.join(HERE, "_build")
LIB = os.path.join(OUT_DIR, "liboracle.so")
SOURCES = ["lfw_oracle.c"]


def build(verbose: bool = False) -> str:
    os.makedirs(OUT_DIR, exist_ok=True)
    srcs = [os.path.join(HERE, s) for s in SOURCES]
    cmd = ["gcc", "-O2", "-fopenmp", "-shared", "-fPIC", "-std=c11", "-Wall", "-Wextra",
           "-o", LIB] + srcs + ["-lm"]
    if verbose:
        print(" ".join(cmd))
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
