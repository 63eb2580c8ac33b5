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


LITE_DIR = os.path.join(PKG, "lite")
LITE_LIB_PATH = os.path.join(LIB_DIR, "libpl_lite_hip.so")
ROOT = os.path.dirname(PKG)
HOST_TEST_SRC = os.path.join(ROOT, "tests", "cpp", "sparse_conv_hip_test.cc")
HOST_TEST_BIN = os.path.join(ROOT, "tests", "cpp", "sparse_conv_hip_test")

LITE_SOURCES = [
    "core/tensor.cc",
    "core/op_lite.cc",
    "core/optimizer/mir/sparse_conv_detect_pass.cc",
    "operators/sparse_conv_op.cc",
    "operators/io_copy_op.cc",
    "kernels/hip/sparse_conv_compute.cc",
    "kernels/hip/io_copy_compute.cc",
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), res.stdout))
    return res.stdout


def build_host_mirror(verbose=False):
    """The C++ host side (the slice of the Lite operator / kernel surface with
    the TARGET(kHIP) sparse_conv2d kernels) and its test program. Host code
    only: compiled by hipcc for the HIP runtime headers, no device code."""
    inc = ["-I" + PKG, "-I" + os.path.join(ROOT, "include")]
    flags = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include"]
    srcs = [os.path.join(LITE_DIR, s) for s in LITE_SOURCES]
    _run(["g++"] + flags + inc + ["-shared", "-o", LITE_LIB_PATH] + srcs + ["-L" + LIB_DIR, "-lpl_sparse_conv", "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,$ORIGIN"], verbose)
    oracle_dir = os.path.join(ROOT, "oracle")
    _run(["make", "-C", oracle_dir, "-s", "libsparse_conv_oracle.so"], verbose)
    _run(["g++"] + flags + inc + ["-I" + oracle_dir, "-o", HOST_TEST_BIN, HOST_TEST_SRC, "-L" + LIB_DIR, "-lpl_lite_hip", "-lpl_sparse_conv", "-L" + oracle_dir, "-lsparse_conv_oracle",
                                  "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,$ORIGIN/../../paddle-lite_amd/lib:$ORIGIN/../../oracle:/opt/rocm/lib"], verbose)
    return LITE_LIB_PATH, HOST_TEST_BIN


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_host_mirror(verbose=True))
