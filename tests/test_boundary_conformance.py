"""Conformance of the drop-in boundary with the reference's real headers.

tests/cpp/param_layout.cc prints the offset and size of every field of
SparseConvParam and ActivationParam, the struct sizes and the defaults of a
value-initialised parameter.  It is compiled once against the reference's
lite/operators/op_params.h (which is self-contained: plain g++, nothing
generated) and once against this repository's; the printouts must be
identical, i.e. a kernel compiled against either header reads the same bytes.

The kernel class itself (lite/kernels/hip/sparse_conv_compute.{h,cc}) cannot
be syntax-checked against the reference's kernel / registry headers here:
lite/core/type_system.h includes the cmake-generated lite/core/version.h, and
no stand-in for generated code is written."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference"
SRC = os.path.join(ROOT, "tests", "cpp", "param_layout.cc")

pytestmark = pytest.mark.skipif(not os.path.exists(os.path.join(REF, "lite", "operators", "op_params.h")), reason="needs the reference checkout")


def build_and_run(tmp_path, name, std, includes, extra_sources=()):
    exe = str(tmp_path / name)
    cmd = ["g++", "-std=" + std, "-O0", "-w"] + ["-I" + i for i in includes] + [SRC] + list(extra_sources) + ["-o", exe]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    assert res.returncode == 0, res.stdout[-3000:]
    return subprocess.run([exe], stdout=subprocess.PIPE, text=True, timeout=60, check=True).stdout


def test_param_structs_have_the_references_layout_and_defaults(tmp_path):
    # the reference header logs through its own logging.cc (no glog without LITE_WITH_LOG)
    ref = build_and_run(tmp_path, "layout_ref", "c++14", [REF], [os.path.join(REF, "lite", "utils", "log", "logging.cc")])
    own = build_and_run(tmp_path, "layout_own", "c++17", [os.path.join(ROOT, "paddle-lite_amd"), os.path.join(ROOT, "include")])
    assert "SparseConvParam.x offset 0 size 8" in ref  # no virtual table in front of the fields
    assert ref.count("\n") == 44  # 2 sizes, 21 + 19 fields, 2 lines of defaults
    assert own == ref
