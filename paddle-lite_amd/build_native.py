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
    # leading scalar kernel arguments reach the wavefronts in registers instead of being loaded from the
    # kernel-argument segment (as many as the user SGPRs hold; csrc/kernarg_head.h)
    "-mllvm", "-amdgpu-kernarg-preload-count=14",
    "-Wall",
    "-Wno-unused-function",
]

# (source, object name, extra flags); the kernel file is built as four
# translation units so that they compile in parallel
SOURCES = [
    ("sparse_layout.cc", "sparse_layout.o", []),
    ("sparse_conv_capi.cc", "sparse_conv_capi.o", []),
    ("calib_kernels.hip", "calib_kernels.o", []),
    ("chunk_walk_kernels.hip", "chunk_walk_kernels.o", []),
    ("tile_walk_kernels.hip", "tile_walk_kernels.o", []),
    ("fp16_walk_kernels.hip", "fp16_walk_kernels.o", []),
    ("dwconv_kernels.hip", "dwconv_kernels.o", []),
    ("image_mfma_kernels.hip", "image_mfma_kernels.o", []),
    ("image_tr_kernels.hip", "image_tr_kernels.o", []),
    ("image_rows_kernels.hip", "image_rows_kernels.o", []),
    ("sparse_conv_kernels.hip", "sparse_conv_kernels_walk.o", ["-DPL_KERNEL_PART=0"]),
    ("sparse_conv_kernels.hip", "sparse_conv_kernels_mfma_f32.o", ["-DPL_KERNEL_PART=1"]),
    ("sparse_conv_kernels.hip", "sparse_conv_kernels_mfma_i8.o", ["-DPL_KERNEL_PART=2"]),
    ("sparse_conv_kernels.hip", "sparse_conv_kernels_mfma_acc32.o", ["-DPL_KERNEL_PART=3"]),
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def _compile_one(job):
    src, obj_name, extra = job
    obj = os.path.join(LIB_DIR, obj_name)
    cmd = [hipcc()] + HIPCC_FLAGS + extra + ["-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    return obj, res.returncode, out, " ".join(cmd)


def build_library(verbose=False):
    """Compile every source and link the shared library. Always recompiles."""
    from concurrent.futures import ThreadPoolExecutor

    os.makedirs(LIB_DIR, exist_ok=True)
    for stale in os.listdir(LIB_DIR):
        if stale.endswith(".o"):
            os.remove(os.path.join(LIB_DIR, stale))
    with ThreadPoolExecutor(max_workers=min(6, os.cpu_count() or 1)) as pool:
        results = list(pool.map(_compile_one, SOURCES))
    objs = []
    for obj, rc, out, cmd in results:
        if verbose:
            print(cmd, flush=True)
            if out.strip():
                print(out, flush=True)
        if rc != 0:
            raise RuntimeError("hipcc failed: %s\n%s" % (cmd, out))
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
MODEL_TOOL_SRC = os.path.join(ROOT, "tests", "cpp", "model_file_tool.cc")
MODEL_TOOL_BIN = os.path.join(ROOT, "tests", "cpp", "model_file_tool")

LITE_SOURCES = [
    "core/tensor.cc",
    "core/op_lite.cc",
    "core/optimizer/mir/graph.cc",
    "core/optimizer/mir/sparse_conv_detect_pass.cc",
    "core/optimizer/mir/int8_chain_pass.cc",
    "model_parser/model_parser.cc",
    "operators/sparse_conv_op.cc",
    "operators/io_copy_op.cc",
    "operators/calib_op.cc",
    "operators/conv_op.cc",
    "kernels/hip/sparse_conv_compute.cc",
    "kernels/hip/io_copy_compute.cc",
    "kernels/hip/calib_compute.cc",
    "kernels/hip/conv_depthwise.cc",
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
    _run(["g++"] + flags + inc + ["-o", MODEL_TOOL_BIN, MODEL_TOOL_SRC, "-L" + LIB_DIR, "-lpl_lite_hip", "-lpl_sparse_conv", "-L/opt/rocm/lib", "-lamdhip64",
                                  "-Wl,-rpath,$ORIGIN/../../paddle-lite_amd/lib:/opt/rocm/lib"], verbose)
    return LITE_LIB_PATH, HOST_TEST_BIN


SANITIZE_FLAGS = ["-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-static-libasan", "-static-libubsan", "-fno-omit-frame-pointer", "-O1", "-g"]


def _compile_host_object(job):
    cmd, obj = job
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    return obj, res.returncode, res.stdout, " ".join(cmd)


def build_sanitized(out_dir):
    """The host side once more with AddressSanitizer and UndefinedBehaviorSanitizer (host code only): every
    file of the C++ mirror, the layout decoder of the library and the CPU oracle compiled into
    out_dir/sparse_conv_hip_test and out_dir/model_file_tool.  The device library stays as it is: the test
    program's --cpu mode and the model-file tool never call into it.  Returns the two paths; raises
    RuntimeError when the compiler has no sanitizer runtime."""
    from concurrent.futures import ThreadPoolExecutor

    os.makedirs(out_dir, exist_ok=True)
    oracle_dir = os.path.join(ROOT, "oracle")
    inc = ["-I" + PKG, "-I" + os.path.join(ROOT, "include"), "-I" + oracle_dir, "-I/opt/rocm/include"]
    cxx = ["g++", "-std=c++17", "-Wall", "-D__HIP_PLATFORM_AMD__"] + SANITIZE_FLAGS + inc
    cc = ["gcc", "-std=c11"] + SANITIZE_FLAGS + inc
    shared = [os.path.join(LITE_DIR, s) for s in LITE_SOURCES] + [os.path.join(CSRC, "sparse_layout.cc")]
    jobs, objs = [], {}
    for src in shared + [HOST_TEST_SRC, MODEL_TOOL_SRC, os.path.join(oracle_dir, "sparse_conv_oracle.c")]:
        obj = os.path.join(out_dir, os.path.relpath(src, ROOT).replace(os.sep, "_") + ".o")
        objs[src] = obj
        jobs.append(((cc if src.endswith(".c") else cxx) + ["-c", src, "-o", obj], obj))
    with ThreadPoolExecutor(max_workers=min(6, os.cpu_count() or 1)) as pool:
        for obj, rc, out, cmd in pool.map(_compile_host_object, jobs):
            if rc != 0:
                raise RuntimeError("sanitizer build failed: %s\n%s" % (cmd, out))
    link = ["-L" + LIB_DIR, "-lpl_sparse_conv", "-L/opt/rocm/lib", "-lamdhip64", "-lm", "-Wl,-rpath," + LIB_DIR + ":/opt/rocm/lib"]
    test_bin, tool_bin = os.path.join(out_dir, "sparse_conv_hip_test"), os.path.join(out_dir, "model_file_tool")
    common = [objs[s] for s in shared]
    _run(["g++"] + SANITIZE_FLAGS + ["-o", test_bin, objs[HOST_TEST_SRC], objs[os.path.join(oracle_dir, "sparse_conv_oracle.c")]] + common + link, False)
    _run(["g++"] + SANITIZE_FLAGS + ["-o", tool_bin, objs[MODEL_TOOL_SRC]] + common + link, False)
    return test_bin, tool_bin


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_host_mirror(verbose=True))
