"""Builds bench_probes/libpl_probe.so from floor_probes.hip (hipcc, gfx950).  The probes measure launch,
memory and store-pattern floors for bench.py; nothing of the operator links them."""
import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libpl_probe.so")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-gpu-rdc", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build(verbose=False):
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    cmd = [exe] + FLAGS + ["-x", "hip", "-shared", os.path.join(HERE, "floor_probes.hip"), "-o", LIB_PATH]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose:
        print(" ".join(cmd), flush=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd), res.stdout))
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
