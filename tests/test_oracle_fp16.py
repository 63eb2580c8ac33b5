"""fp16 arithmetic of the oracle (bit patterns, one rounding per operation)
pinned by what the mathematics fixes: conversions against numpy's float16 on
every binary16 value and on float32 inputs around every rounding boundary,
the fused multiply-add against exact rational arithmetic, and the walker
against a plain numpy restatement on small cases."""
import fractions

import numpy as np
import pytest

from oracle import oracle as O


def test_conversion_matches_numpy_everywhere():
    h = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(np.float16)
    f = h.astype(np.float32)
    back = O.fp32_to_fp16(f)
    ok = (back.view(np.uint16) == h.view(np.uint16)) | (np.isnan(h) & np.isnan(back))
    assert ok.all()
    # float32 values between halves: midpoints (ties to even) and their neighbours
    finite = h[np.isfinite(h)].astype(np.float64)
    finite.sort()
    mid = ((finite[:-1] + finite[1:]) / 2).astype(np.float32)  # exact in float32
    for cand in (mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf))):
        with np.errstate(over="ignore"):
            want = cand.astype(np.float16)
        assert np.array_equal(O.fp32_to_fp16(cand).view(np.uint16), want.view(np.uint16))
    big = np.array([65504.0, 65519.99, 65520.0, 70000.0, -65520.0, 1e-8, 2.0 ** -25, np.nextafter(np.float32(2.0 ** -25), np.float32(1))], np.float32)
    with np.errstate(over="ignore"):
        assert np.array_equal(O.fp32_to_fp16(big).view(np.uint16), big.astype(np.float16).view(np.uint16))


def _round_fraction_to_half(q):
    """Correctly rounded (nearest even) binary16 of an exact rational."""
    if q == 0:
        return np.float16(0.0)
    sign = -1 if q < 0 else 1
    a = abs(q)
    # candidates: the two neighbouring halves around a
    f = np.float16(float(a))  # float(a) is correctly rounded to double; may double-round, so repair below
    cands = [f, np.nextafter(f, np.float16(np.inf)), np.nextafter(f, np.float16(0))]
    best = None
    for c in cands:
        if not np.isfinite(c):
            continue
        d = abs(fractions.Fraction(float(c)) - a)
        key = (d, int(c.view(np.uint16)) & 1)
        if best is None or key < best[0]:
            best = (key, c)
    r = best[1]
    if a >= fractions.Fraction(65520):
        r = np.float16(np.inf)
    return np.float16(-r) if sign < 0 else r


def test_fused_multiply_add_against_exact_arithmetic():
    import ctypes as C

    lib = O.lib()
    rng = np.random.default_rng(5)
    # drive plo_sparse_conv_fp16 with K=1, one weight: out = fma(x, w, bias)
    n = 4000
    xs = rng.standard_normal(n).astype(np.float16)
    ws = (rng.standard_normal(n) * 4).astype(np.float16)
    bs = (rng.standard_normal(n) * 8).astype(np.float16)
    # include cancellation and tie-prone cases
    xs[:8] = np.array([1.0, 3.0, 0.1, 255.0, 1e-3, 2.0 ** -12, 1023.0, 0.333], np.float16)
    ws[:8] = np.array([1.0, 1.0 / 3.0, 10.0, 257.0, 1e-3, 2.0 ** -12, 1.0 + 2.0 ** -10, 3.0], np.float16)
    bs[:8] = np.array([-1.0, -1.0, -1.0, -65504.0, 1.0, 1.0, -1023.0, -1.0], np.float16)
    for x, w, b in zip(xs, ws, bs):
        dense = np.array([[np.float32(w)]], np.float32)
        pk = O.pack(dense, 1, O.LAYOUT_PADDED)
        got = O.sparse_conv_fp16(pk, np.array([[[[x]]]], np.float16), np.array([np.float32(b)], np.float32))
        exact = fractions.Fraction(float(x)) * fractions.Fraction(float(w)) + fractions.Fraction(float(b))
        want = _round_fraction_to_half(exact)
        assert got.ravel()[0].view(np.uint16) == want.view(np.uint16) or (got.ravel()[0] == 0 and want == 0), (x, w, b, got.ravel()[0], want)


def _numpy_walk(dense16, x16, bias16, act):
    """acc = bias; acc = round16(x*w + acc) in increasing channel order, via
    float64 (the product of two halves and a third half add exactly there
    except in far-apart magnitudes, which the inputs below avoid)."""
    oc, ic = dense16.shape
    b, _, h, w = x16.shape
    out = np.zeros((b, oc, h, w), np.float16)
    for r in range(oc):
        acc = np.full((b, h, w), bias16[r] if bias16 is not None else np.float16(0), np.float16)
        for k in range(ic):
            if dense16[r, k] != 0:
                acc = (x16[:, k].astype(np.float64) * np.float64(dense16[r, k]) + acc.astype(np.float64)).astype(np.float16)
        out[:, r] = acc
    if act == "relu":
        out = np.maximum(out, np.float16(0))
    return out


@pytest.mark.parametrize("paired", [False, True])
def test_walker_against_numpy(paired):
    rng = np.random.default_rng(9 + paired)
    oc, ic, hw = 7, 21, 10
    dense = (rng.standard_normal((oc, ic)) * (rng.random((oc, ic)) > 0.6)).astype(np.float32)
    if paired:
        dense[1] = np.where(dense[0] != 0, dense[1] + 0.5, 0)
        dense[3] = np.where(dense[2] != 0, 1.0, 0)
    x = rng.standard_normal((2, ic, 2, 5)).astype(np.float16)
    bias = rng.standard_normal(oc).astype(np.float32)
    pk = O.pack(dense, hw, O.LAYOUT_SEMI if paired else O.LAYOUT_PADDED)
    got = O.sparse_conv_fp16(pk, x, bias, O.Act(O.ACT_RELU))
    want = _numpy_walk(dense.astype(np.float16), x, bias.astype(np.float16), "relu")
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
