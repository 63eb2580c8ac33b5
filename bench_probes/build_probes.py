"""Builds bench_probes/libpl_probe.so from floor_probes.hip and rate_probes.hip (hipcc, gfx950): the probes measure
launch, memory and store-pattern floors and instruction rates for bench.py; nothing of the operator links them.  build_programs() builds
bench_probes/lite_program_bench, the host-cost and graph-replay measurement of the C++ operator surface
(it links the package's two libraries, so they are built first)."""
import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libpl_probe.so")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-gpu-rdc", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build(verbose=False):
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    cmd = [exe] + FLAGS + ["-x", "hip", "-shared", os.path.join(HERE, "floor_probes.hip"), os.path.join(HERE, "rate_probes.hip"), "-o", LIB_PATH]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose:
        print(" ".join(cmd), flush=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd), res.stdout))
    return LIB_PATH


ROOT = os.path.dirname(HERE)
PKG = os.path.join(ROOT, "paddle-lite_amd")
PROGRAM_PATH = os.path.join(HERE, "lite_program_bench")


def build_programs(verbose=False):
    cmd = ["g++", "-O2", "-std=c++17", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", "-I" + PKG, "-I" + os.path.join(ROOT, "include"), "-o", PROGRAM_PATH,
           os.path.join(HERE, "lite_program_bench.cc"), "-L" + os.path.join(PKG, "lib"), "-lpl_lite_hip", "-lpl_sparse_conv", "-L/opt/rocm/lib", "-lamdhip64",
           "-Wl,-rpath,$ORIGIN/../paddle-lite_amd/lib:/opt/rocm/lib"]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose:
        print(" ".join(cmd), flush=True)
    if res.returncode != 0:
        raise RuntimeError("g++ failed: %s\n%s" % (" ".join(cmd), res.stdout))
    return PROGRAM_PATH


if __name__ == "__main__":
    print(build(verbose=True))
    print(build_programs(verbose=True))
