"""The host side under AddressSanitizer and UndefinedBehaviorSanitizer: the C++ mirror (ops, passes, model
file reader / writer), the library's layout decoder and the CPU oracle are compiled once more with
-fsanitize=address,undefined (build_native.build_sanitized) and run where no device is needed: the host test
program's --cpu mode, the model-file tool's self test (which loads every truncation of a file it wrote), and
the reference-written fixtures whole and cut short.  Any report of either sanitizer ends the process with a
non-zero status, which fails the test.  Skipped when the compiler has no sanitizer runtime."""
import importlib
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden", "model_file")
ENV = dict(os.environ, ASAN_OPTIONS="abort_on_error=0:detect_leaks=0", UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")


@pytest.fixture(scope="module")
def binaries(tmp_path_factory):
    probe_dir = tmp_path_factory.mktemp("san_probe")
    src = probe_dir / "probe.cc"
    src.write_text("#include <vector>\nint main() { std::vector<int> v(3); return v[2]; }\n")
    probe = subprocess.run(["g++", "-fsanitize=address,undefined", "-static-libasan", "-static-libubsan", "-o", str(probe_dir / "probe"), str(src)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    if probe.returncode != 0 or subprocess.run([str(probe_dir / "probe")], env=ENV).returncode != 0:
        pytest.skip("no sanitizer runtime for g++ here")
    build_native = importlib.import_module("paddle-lite_amd.build_native")
    if not os.path.exists(build_native.LIB_PATH):
        pytest.skip("the device library is not built (the sanitized programs link it): run __graft_entry__.build()")
    return build_native.build_sanitized(str(tmp_path_factory.mktemp("san_build")))


def run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300, env=ENV)
    return res.returncode, res.stdout


def assert_clean(out):
    assert "ERROR: AddressSanitizer" not in out and "runtime error:" not in out, out[-4000:]


def test_host_test_program_cpu_mode(binaries):
    rc, out = run([binaries[0], "--cpu"])
    assert_clean(out)
    assert rc == 0 and "cpu: 0 failure(s)" in out, out[-4000:]


def test_model_file_self_test_with_every_truncation(binaries):
    rc, out = run([binaries[1], "selftest"])
    assert_clean(out)
    assert rc == 0 and "selftest: ok" in out, out[-4000:]


@pytest.mark.parametrize("meta", [1, 2])
def test_reference_written_fixture_whole_and_cut_short(binaries, tmp_path, meta):
    nb = os.path.join(GOLDEN, "ref_example_v%d.nb" % meta)
    rc, out = run([binaries[1], "dump", nb])
    assert_clean(out)
    assert rc == 0
    with open(os.path.join(GOLDEN, "ref_example_v%d.dump.txt" % meta)) as f:
        want = f.read()
    assert out.endswith(want) or want in out  # a version notice may precede the dump
    with open(nb, "rb") as f:
        data = f.read()
    cut = str(tmp_path / "cut.nb")
    lengths = sorted(set(list(range(0, 64)) + list(range(64, len(data), max(1, len(data) // 60))) + [len(data) - 1]))
    for n in lengths:
        with open(cut, "wb") as f:
            f.write(data[:n])
        rc, out = run([binaries[1], "dump", cut])
        assert_clean(out)
        assert rc == 1 and "error:" in out, (n, out[-500:])
