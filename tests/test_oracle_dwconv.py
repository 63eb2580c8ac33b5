"""Pins the depthwise 3x3 oracle (oracle/sparse_conv_oracle.c
plo_dwconv3x3_int8): its int32 sums against the reference header's own
conv_basic<int8, int32> with group == channels (oracle/_ref, where the
reference checkout is present) and against a numpy statement built from
shifted slices; its epilogue against closed forms."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from oracle import oracle as O  # noqa: E402

SHAPES = [(1, 1, 3, 3), (2, 3, 7, 7), (1, 4, 14, 14), (2, 2, 9, 6), (1, 2, 5, 12), (1, 1, 4, 4), (1, 3, 2, 2), (1, 2, 1, 5)]


def numpy_sums(x, w, stride, pad):
    n, c, h, ww = x.shape
    xp = np.zeros((n, c, h + 2 * pad, ww + 2 * pad), dtype=np.int64)
    xp[:, :, pad:pad + h, pad:pad + ww] = x
    oh, ow = O.dwconv_out_size(h, stride, pad), O.dwconv_out_size(ww, stride, pad)
    acc = np.zeros((n, c, oh, ow), dtype=np.int64)
    for ky in range(3):
        for kx in range(3):
            win = xp[:, :, ky:ky + stride * (oh - 1) + 1:stride, kx:kx + stride * (ow - 1) + 1:stride]
            acc += win * w[None, :, ky, kx, None, None].astype(np.int64)
    return acc.astype(np.int32)


def cases():
    for shape in SHAPES:
        for stride in (1, 2):
            for pad in (0, 1):
                if shape[2] + 2 * pad < 3 or shape[3] + 2 * pad < 3:
                    continue
                yield shape, stride, pad


@pytest.mark.parametrize("shape,stride,pad", list(cases()))
def test_sums_against_numpy(shape, stride, pad):
    rng = np.random.RandomState(hash((shape, stride, pad)) % (2 ** 31))
    x = rng.randint(-127, 128, size=shape).astype(np.int8)
    w = rng.randint(-127, 128, size=(shape[1], 3, 3)).astype(np.int8)
    got = O.dwconv3x3_int8(x, w, out="acc", stride=stride, pad=pad)
    assert np.array_equal(got, numpy_sums(x, w, stride, pad))


@pytest.mark.parametrize("shape,stride,pad", list(cases()))
def test_sums_against_reference_header(shape, stride, pad):
    if not O.have_ref():
        pytest.skip("oracle/_ref needs the reference checkout")
    rng = np.random.RandomState(7 + hash((shape, stride, pad)) % (2 ** 31))
    x = rng.randint(-127, 128, size=shape).astype(np.int8)
    w = rng.randint(-127, 128, size=(shape[1], 3, 3)).astype(np.int8)
    assert np.array_equal(O.dwconv3x3_int8(x, w, out="acc", stride=stride, pad=pad), O.ref_dwconv3x3_s8_s32(x, w, stride, pad))


def test_extreme_values_do_not_overflow():
    x = np.full((1, 2, 6, 6), -128, dtype=np.int8)
    w = np.full((2, 3, 3), -128, dtype=np.int8)
    acc = O.dwconv3x3_int8(x, w, out="acc", stride=1, pad=1)
    assert acc[0, 0, 2, 2] == 9 * 128 * 128 and acc[0, 0, 0, 0] == 4 * 128 * 128


def test_epilogue_closed_forms():
    rng = np.random.RandomState(3)
    x = rng.randint(-127, 128, size=(2, 3, 8, 8)).astype(np.int8)
    w = rng.randint(-127, 128, size=(3, 3, 3)).astype(np.int8)
    acc = numpy_sums(x, w, 1, 1)
    one = np.ones(3, dtype=np.float32)
    # scale 1, no bias, no activation: the sums themselves, saturated for int8
    assert np.array_equal(O.dwconv3x3_int8(x, w, one, out="fp32"), acc.astype(np.float32))
    assert np.array_equal(O.dwconv3x3_int8(x, w, one, out="int8"), np.clip(acc, -127, 127).astype(np.int8))
    # power-of-two scale and integer bias are exact in fp32; relu
    s = np.array([0.5, 0.25, 2.0], dtype=np.float32)
    b = np.array([1.0, -2.0, 3.0], dtype=np.float32)
    want = np.maximum(acc * s[None, :, None, None].astype(np.float64) + b[None, :, None, None], 0.0)
    got = O.dwconv3x3_int8(x, w, s, b, O.Act(O.ACT_RELU if hasattr(O, "ACT_RELU") else 1), out="fp32")
    assert np.array_equal(got, want.astype(np.float32))
    # rounding: halves go away from zero, -127 is the floor
    xs = np.zeros((1, 1, 3, 3), dtype=np.int8)
    ws = np.zeros((1, 3, 3), dtype=np.int8)
    ws[0, 1, 1] = 1
    for v, q in [(1, 1), (3, 2), (5, 3), (-1, -1), (-3, -2), (-5, -3), (127, 64), (-127, -64)]:
        xs[0, 0, 1, 1] = v
        out = O.dwconv3x3_int8(xs, ws, np.array([0.5], dtype=np.float32), out="int8", stride=1, pad=0)
        assert out.shape == (1, 1, 1, 1) and out[0, 0, 0, 0] == q, (v, q, out)
    xs[0, 0, 1, 1] = -128
    assert O.dwconv3x3_int8(xs, ws, np.array([2.0], dtype=np.float32), out="int8", stride=1, pad=0)[0, 0, 0, 0] == -127


def test_hard_swish_multiplies_by_the_scale():
    xs = np.zeros((1, 1, 3, 3), dtype=np.int8)
    ws = np.zeros((1, 3, 3), dtype=np.int8)
    ws[0, 1, 1] = 1
    xs[0, 0, 1, 1] = 4
    act = O.Act()
    act.type = 10
    act.hs_scale, act.hs_offset, act.hs_threshold = 0.25, 3.0, 6.0
    # v = 4: (4 * 0.25) * min(max(4 + 3, 0), 6) = 6
    assert O.dwconv3x3_int8(xs, ws, np.ones(1, dtype=np.float32), None, act, out="fp32", stride=1, pad=0)[0, 0, 0, 0] == 6.0
