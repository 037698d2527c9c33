"""Builds t2fw_amd/lib/libt2fw_hip.so from t2fw_amd/csrc/*.hip with hipcc for gfx950.

    python -m t2fw_amd.build            # build (always recompiles)
    python -m t2fw_amd.build --if-missing

hipcc cross-compiles without a GPU, so the library is built ahead of time and shipped
in-tree; nothing is compiled at import time (the reference JIT-builds at import,
t2fw/functional_lfw.py:12-21).
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libt2fw_hip.so")
OBJ_DIR = os.path.join(LIB_DIR, "obj")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed-FP32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unused-command-line-argument",
]


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    return obj, err


def build(verbose=False):
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        results = list(ex.map(_compile, srcs))
    for obj, err in results:
        if verbose and err.strip():
            print(err, file=sys.stderr)
    objs = [o for o, _ in results]
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    return LIB_PATH


if __name__ == "__main__":
    if "--if-missing" in sys.argv and os.path.exists(LIB_PATH):
        print(LIB_PATH, "(exists)")
    else:
        print(build(verbose=True))
