"""CPU-side checks of the shipped library: it loads, exports every symbol the
header declares, its host packers agree with the oracle bit for bit, and it
refuses to compute without a device (no CPU fallback)."""
import ctypes as C
import json
import os
import re

import numpy as np
import pytest

from helpers import capi, pla, workloads
from oracle import oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "pl_sparse_conv.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pl_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) >= 11
    L = capi.lib()
    for n in names:
        assert hasattr(L, n), "libpl_sparse_conv.so does not export %s" % n
    assert sorted(capi.EXPORTS) == names
    assert L.pl_sparse_conv_abi_version() == capi.ABI_VERSION


def test_struct_layout_matches_header(tmp_path):
    """sizeof and offsetof of every field of the header's structs, printed by a
    C program compiled against the header, equal the ctypes mirror's."""
    import shutil
    import subprocess

    structs = {"pl_activation": capi.Activation, "pl_sparse_conv_tuning": capi.Tuning, "pl_sparse_conv_desc": capi.Desc, "pl_sparse_conv_info": capi.Info, "pl_dwconv_desc": capi.DwConvDesc}
    assert C.sizeof(capi.Activation) == 24
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler")
    lines = ["#include <stdio.h>", "#include <stddef.h>", '#include "pl_sparse_conv.h"', "int main(void) {"]
    for cname, cls in sorted(structs.items()):
        lines.append('  printf("%s %%zu\\n", sizeof(%s));' % (cname, cname))
        for fname, _ in cls._fields_:
            lines.append('  printf("%s.%s %%zu\\n", offsetof(%s, %s));' % (cname, fname, cname, fname))
    lines += ["  return 0;", "}"]
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.check_call([gcc, "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    want = dict(l.split() for l in subprocess.check_output([str(exe)], text=True).splitlines())
    for cname, cls in structs.items():
        assert C.sizeof(cls) == int(want[cname]), cname
        for fname, _ in cls._fields_:
            assert getattr(cls, fname).offset == int(want["%s.%s" % (cname, fname)]), (cname, fname)
    # every field of the header's structs is mirrored (declarators inside the typedef's braces)
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "pl_sparse_conv.h")).read(), flags=re.S)
    for cname, cls in structs.items():
        body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (cname, cname), text, flags=re.S).group(1)
        assert body.count(";") + body.count(",") == len(cls._fields_), cname


def _rand(rng, oc, ic, density, dtype, paired):
    if paired:
        m = np.repeat(rng.random_sample(((oc + 1) // 2, ic)) < density, 2, axis=0)[:oc]
    else:
        m = rng.random_sample((oc, ic)) < density
    v = rng.randint(1, 100, size=(oc, ic))
    return (v * m).astype(dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.int8])
def test_host_packers_equal_oracle_packers(dtype):
    rng = np.random.RandomState(17)
    for trial in range(120):
        oc, ic, n = int(rng.randint(1, 20)), int(rng.randint(1, 30)), int(rng.randint(1, 60))
        w = _rand(rng, oc, ic, rng.choice([0.0, 0.1, 0.4, 1.0]), dtype, paired=bool(trial % 2))
        if oc > 2:
            w[rng.randint(0, oc)] = 0
        for force in (None, True, False):
            got = pla.detect_and_pack(w, n, force_semi=force)
            if force is None:
                want = O.pack_like_pass(w, n)
            elif force:
                want = O.pack(w, n, O.LAYOUT_SEMI)
            else:
                want = O.pack(w, n, O.LAYOUT_PADDED if dtype == np.float32 else O.LAYOUT_UNPADDED)
            assert got.flag_semi == want.flag_semi and got.first_ic == want.first_ic
            assert np.array_equal(got.nonzero_weights, want.nonzero_weights)
            assert np.array_equal(got.oc_nonzeros, want.oc_nonzeros)
            assert np.array_equal(got.diffs, want.diffs)


def test_host_packers_known_answers():
    kat = json.load(open(os.path.join(ROOT, "tests", "golden", "packer_kat.json")))
    for case in kat["cases"]:
        w = np.array(case["dense"], dtype=case["dtype"]).reshape(case["rows"], case["cols"])
        got = pla.detect_and_pack(w, kat["im_size"])
        assert got.flag_semi == case["flag_semi"] and got.first_ic == case["first_ic"]
        assert got.nonzero_weights.tolist() == case["nonzero_weights"]
        assert got.diffs.tolist() == case["diffs"]
        used = case.get("oc_nonzeros", case.get("oc_nonzeros_used"))
        assert got.oc_nonzeros[:len(used)].tolist() == used


def test_sparse_threshold_gate():
    # the pass skips a conv whose zero fraction is below the threshold
    # (sparse_conv_detect_pass.cc:684-692); for the semi layout the stored
    # zero partners count as nonzeros
    w = np.zeros((4, 10), np.float32)
    w[:, :3] = 1.0  # 70 % zeros
    assert pla.detect_and_pack(w, 9, sparse_threshold=0.71) is None
    assert pla.detect_and_pack(w, 9, sparse_threshold=0.70) is not None
    with pytest.raises(ValueError):
        pla.detect_and_pack(w, 9, sparse_threshold=1.5)
    assert pla.detect_and_pack(np.ones((4, 10, 3, 3), np.float32), 9) is None  # not a 1x1 kernel


def test_unknown_activation_is_fatal():
    with pytest.raises(ValueError):
        pla.ActivationParam("sigmoid")


def test_weight_scale_size_is_checked():
    w = pla.detect_and_pack(_rand(np.random.RandomState(0), 6, 8, 0.5, np.int8, False), 4)
    p = pla.SparseConvParam(w, enable_int8=True, weight_scale=[0.1, 0.2])
    with pytest.raises(ValueError, match="weights scale size"):
        pla.SparseConvKernel(p, "int8", "float32").PrepareForRun()


def test_no_device_no_compute():
    """Without a gfx950 device the library must fail loudly, never compute on
    the CPU."""
    import torch

    if torch.cuda.is_available():
        pytest.skip("a device is present")
    assert capi.lib().pl_device_count() == 0
    case = workloads.make_int8("t", 1, 8, 4, 2, 2, 0.5, False, pla.ActivationParam(), False, seed=0)
    w = pla.detect_and_pack(case.dense, 4)
    p = pla.SparseConvParam(w, enable_int8=True, weight_scale=case.weight_scale, input_scale=0.01)
    with pytest.raises(capi.SparseConvError) as e:
        pla.SparseConvKernel(p, "int8", "float32").PrepareForRun()
    assert e.value.code == capi.PL_ERR_NO_DEVICE


def test_depthwise_host_checks_and_no_device():
    """The depthwise kernel class refuses what the reference's class refuses
    before any device work, and without a device prepare fails loudly."""
    import torch

    filt = np.ones((4, 1, 3, 3), dtype=np.int8)
    with pytest.raises(NotImplementedError):
        pla.DepthwiseConv(pla.ConvParam(np.ones((4, 1, 5, 5), dtype=np.int8))).PrepareForRun()  # "this type dw conv not impl"
    with pytest.raises(NotImplementedError):
        pla.DepthwiseConv(pla.ConvParam(filt, strides=(3, 3))).PrepareForRun()
    with pytest.raises(ValueError):
        pla.DepthwiseConv(pla.ConvParam(filt, weight_scale=[0.1, 0.2])).PrepareForRun()  # neither 1 nor one per channel
    with pytest.raises(ValueError):
        pla.ConvParam(np.ones((4, 2, 3, 3), dtype=np.int8))  # not a depthwise filter
    assert pla.ConvParam(filt, paddings=(1, 0)).paddings == [1, 1, 0, 0]  # two-element form, as ConvOp pads it
    k = pla.DepthwiseConv(pla.ConvParam(filt, strides=(2, 2)))
    assert k.out_shape((3, 4, 15, 13)) == (3, 4, 8, 7)
    if torch.cuda.is_available():
        pytest.skip("a device is present")
    with pytest.raises(capi.SparseConvError) as e:
        k.PrepareForRun()
    assert e.value.code == capi.PL_ERR_NO_DEVICE


def test_mobilenet_depthwise_workloads_chain_with_the_pointwise_ones():
    size = 112
    for i in range(13):
        dw = workloads.config5_depthwise_layer(i)
        ic, oc, hw = workloads.MOBILENET_V1_POINTWISE[i]
        assert dw.channels == ic and dw.in_size == size and dw.out_size == hw
        assert dw.filter.shape == (ic, 1, 3, 3) and dw.filter.dtype == np.int8
        size = hw
    a, b = workloads.config5_depthwise_layer(3), workloads.config5_depthwise_layer(3)
    assert np.array_equal(a.filter, b.filter) and a.output_scale == b.output_scale


def test_workloads_are_seeded_and_shaped():
    a, b = workloads.config3(batch=2), workloads.config3(batch=2)
    assert np.array_equal(a.x, b.x) and np.array_equal(a.dense, b.dense)
    assert a.dense.shape == (512, 512) and a.x.shape == (2, 512, 14, 14)
    assert abs(1 - a.nnz / (512 * 512.0) - 0.85) < 0.01
    c4 = workloads.config4(batch=1)
    assert O.count_semi(c4.dense)["flag_semi"] == 1 and O.count_semi(a.dense)["flag_semi"] == 0
    c2 = workloads.config2(batch=1)
    assert O.count_semi(c2.dense)["flag_semi"] == 1 and c2.dense.dtype == np.float32
    assert len(workloads.MOBILENET_V1_POINTWISE) == 13


def test_bench_refuses_more_than_one_gpu():
    """Every box has one GPU: bench.py --gpus N > 1 exits with a message
    instead of measuring anything."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert res.returncode != 0
    assert "one GPU" in res.stderr
    assert res.stdout.strip() == ""


def test_host_fp16_conversion_matches_the_oracle():
    import ctypes as C
    from oracle import oracle as O

    rng = np.random.default_rng(1)
    f = np.concatenate([rng.standard_normal(100000).astype(np.float32) * np.float32(10.0) ** rng.integers(-8, 5, 100000).astype(np.float32),
                        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 2.9802326e-8, np.inf, -np.inf], np.float32)])
    out = np.empty(f.size, np.uint16)
    assert capi.lib().pl_fp32_to_fp16(f.ctypes.data, out.ctypes.data, f.size) == capi.PL_OK
    assert np.array_equal(out, O.fp32_to_fp16(f).view(np.uint16))
