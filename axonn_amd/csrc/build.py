"""Builds libaxn_gfx950.so (the product library) and libaxn_probe_gfx950.so (streaming
yardsticks for benchmarks, include/axn_probe.h) from the HIP sources in this directory.

    python -m axonn_amd.csrc.build

hipcc cross-compiles for gfx950 without a GPU.  The library links against the
HIP runtime by soname only, so inside a PyTorch process it binds to the HIP
runtime PyTorch has already loaded.
"""

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB_DIR = os.path.join(os.path.dirname(HERE), "lib")
LIB_PATH = os.path.join(LIB_DIR, "libaxn_gfx950.so")
PROBE_LIB_PATH = os.path.join(LIB_DIR, "libaxn_probe_gfx950.so")
OBJ_DIR = os.path.join(HERE, "build")

SOURCES = ["axn_api.hip", "gemm_bf16.hip", "gemm_f32.hip", "elementwise.hip", "embedding.hip", "optim.hip"]
PROBE_SOURCES = ["stream_probe.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Wall",
    "-Wno-unused-function",
    # packed fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + os.path.join(ROOT, "include"),
    "-I" + HERE,
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass does not know the packed-fp32 feature name; that warning is noise.
    out = "\n".join(
        line for line in proc.stdout.splitlines()
        if "packed-fp32-ops" not in line
    )
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_library(verbose=False, extra_flags=()):
    """Compiles every source and links the shared library; returns its path."""
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)

    def compile_one(src):
        obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
        out = _run([HIPCC, *FLAGS, *extra_flags, "-c", os.path.join(HERE, src), "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    every = SOURCES + PROBE_SOURCES
    with ThreadPoolExecutor(max_workers=min(len(every), os.cpu_count() or 1)) as pool:
        objs = list(pool.map(compile_one, every))
    for path, part in ((LIB_PATH, objs[:len(SOURCES)]), (PROBE_LIB_PATH, objs[len(SOURCES):])):
        out = _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *part, "-o", path])
        if verbose and out.strip():
            print(out)
    return LIB_PATH


if __name__ == "__main__":
    path = build_library(verbose=True)
    print("built", path)
    sys.exit(0)
