"""The lane mapping of ds_read_b64_tr_b8 that both image kernels build their matrix-core operands on,
checked on the device against a plain numpy transposition: within each group of 16 lanes, byte b of lane j
is byte j % 8 of the eight bytes that lane 2 b + j / 8 addressed; and the low three bits of an address are
ignored (the read is 8-byte aligned)."""
import ctypes as C
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def probes():
    import importlib

    if ROOT not in sys.path:
        sys.path.insert(0, ROOT)
    bp = importlib.import_module("bench_probes.build_probes")
    if not os.path.exists(bp.LIB_PATH):
        pytest.skip("bench_probes/libpl_probe.so is not built")
    P = C.CDLL(bp.LIB_PATH)
    P.pl_probe_tr8_map.restype = C.c_int
    P.pl_probe_tr8_map.argtypes = [C.c_void_p, C.c_void_p]
    return P


def read_map(P, addr):
    addr = np.ascontiguousarray(addr, dtype=np.int32)
    src = np.zeros(64 * 8, dtype=np.uint16)
    rc = P.pl_probe_tr8_map(addr.ctypes.data, src.ctypes.data)
    assert rc == 0, "HIP error %d" % rc
    return src.reshape(64, 8).astype(np.int64)


def expected(addr):
    """numpy statement: per group of 16 lanes, the 16 x 8 byte matrix M[s][t] = addr[s] + t (what the lanes
    address) read as two 8 x 8 blocks (even and odd source lanes) and transposed."""
    addr = np.asarray(addr, dtype=np.int64) & ~7
    out = np.zeros((64, 8), dtype=np.int64)
    for g in range(4):
        m = addr[16 * g:16 * g + 16, None] + np.arange(8)[None, :]   # [source lane][byte]
        for half in range(2):
            block = m[half::2]                                         # source lanes 2 b + half, b = 0 .. 7
            out[16 * g + 8 * half:16 * g + 8 * half + 8] = block.T     # lane 8 half + t gets [b] = block[b][t]
    return out


@pytest.mark.parametrize("pattern", ["contiguous", "reversed", "rows_of_196", "random"])
def test_lane_mapping_equals_a_transposition(pattern):
    P = probes()
    rng = np.random.RandomState(3)
    if pattern == "contiguous":
        addr = 8 * np.arange(64)
    elif pattern == "reversed":
        addr = 1024 + 8 * (63 - np.arange(64))
    elif pattern == "rows_of_196":
        # the image kernels' case: 8 even channel rows 392 bytes apart (rows of 196 bytes), two runs of 8
        # positions per row and group of 16 lanes, each group 16 positions further along the rows
        lane = np.arange(64)
        addr = 392 * ((lane % 16) // 2) + 8 * (lane % 2) + 16 * (lane // 16)
    else:
        addr = 8 * rng.randint(0, 500, size=64)
    assert np.array_equal(read_map(P, addr), expected(addr))


def test_low_address_bits_are_ignored():
    P = probes()
    base = 8 * np.arange(64) + 64
    for off in (1, 4, 7):
        assert np.array_equal(read_map(P, base + off), expected(base))
