"""Compiles the HIP library of this package for gfx950 with hipcc.

The result, lib/libpl_sparse_conv.so, is kept in the tree (ignored by git) so
that it travels with the sources; nothing is built at import time.
"""
import os
import shutil
import subprocess

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
LIB_DIR = os.path.join(PKG, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libpl_sparse_conv.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-fno-gpu-rdc",
    # no packed fp32 VALU instructions in device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]

SOURCES = ["sparse_layout.cc", "sparse_conv_kernels.hip", "sparse_conv_capi.cc"]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def build_library(verbose=False):
    """Compile every source and link the shared library. Always recompiles."""
    os.makedirs(LIB_DIR, exist_ok=True)
    objs = []
    for src in SOURCES:
        obj = os.path.join(LIB_DIR, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc()] + HIPCC_FLAGS + ["-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
        if res.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
        if verbose and out.strip():
            print(out, flush=True)
        objs.append(obj)
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n%s" % res.stdout)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
