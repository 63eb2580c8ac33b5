"""The kernels round half away from zero as trunc(v + copysign(0.49999997, v))
after clamping to [-127, 127] (sparse_conv_kernels.hip, QuantizeI8).  Checked
here against the definition, max(v, -127) -> roundf -> min(., 127), on every
float32 whose magnitude lies in [2^-3, 256) plus the values around it; below
2^-3 both sides are zero by inspection (|v| + 0.5 < 1)."""
import numpy as np

HALF_BELOW = np.float32(np.nextafter(np.float32(0.5), np.float32(0.0)))


def kernel_formula(v):
    v = np.clip(v, np.float32(-127.0), np.float32(127.0))
    s = (v + np.copysign(HALF_BELOW, v)).astype(np.float32)
    return np.trunc(s).astype(np.int32)


def definition(v):
    v = np.maximum(v, np.float32(-127.0))
    t = np.trunc(v)
    frac = np.abs(v - t)  # exact in float32
    r = t + np.where(frac >= np.float32(0.5), np.copysign(np.float32(1.0), v), np.float32(0.0)).astype(np.float32)
    return np.minimum(r, np.float32(127.0)).astype(np.int32)


def test_round_half_away_identity_exhaustive():
    lo = np.float32(2.0 ** -3).view(np.uint32)
    hi = np.float32(256.0).view(np.uint32)
    step = 1 << 24
    for start in range(int(lo), int(hi), step):
        bits = np.arange(start, min(start + step, int(hi)), dtype=np.uint32)
        for sign in (np.uint32(0), np.uint32(0x80000000)):
            v = (bits | sign).view(np.float32)
            np.testing.assert_array_equal(kernel_formula(v), definition(v))


def test_round_half_away_special_values():
    v = np.array([0.0, -0.0, 0.49999997, -0.49999997, 0.5, -0.5, 1.5, -1.5, 2.5, 126.5, 126.49999, 127.0, 127.5, 1e9, -1e9, -127.5, -126.5, 1e-30, -1e-30], dtype=np.float32)
    want = np.array([0, 0, 0, 0, 1, -1, 2, -2, 3, 127, 126, 127, 127, 127, -127, -127, -127, 0, 0], dtype=np.int32)
    np.testing.assert_array_equal(kernel_formula(v), want)
    np.testing.assert_array_equal(definition(v), want)


def relu6_kernel_formula(v, coef):
    """ActQuantI8<relu6> of epilogue.h: one median over the intersected bounds,
    then the truncated sum with a half whose sign is the coefficient's."""
    coef = np.float32(coef)
    lo = np.maximum(np.minimum(np.float32(0.0), coef), np.float32(-127.0))
    hi = np.maximum(np.minimum(coef, np.float32(127.0)), lo)
    half = HALF_BELOW if coef >= 0 else -HALF_BELOW
    return np.trunc((np.clip(v, lo, hi) + half).astype(np.float32)).astype(np.int32)


def relu6_definition(v, coef):
    """min(max(v, 0), coef) as the reference computes relu6, then the
    quantisation by its definition."""
    r = np.minimum(np.maximum(v, np.float32(0.0)), np.float32(coef)).astype(np.float32)
    return definition(r)


def test_relu6_shortcut_identity():
    lo = np.float32(2.0 ** -3).view(np.uint32)
    hi = np.float32(256.0).view(np.uint32)
    step = 1 << 24
    for coef, stride in ((6.0, 1), (0.3, 5), (1.5, 7), (126.7, 5), (127.0, 7), (200.0, 5), (0.0, 11), (-3.0, 7), (-126.5, 11), (-200.0, 11)):
        for start in range(int(lo), int(hi), step):
            bits = np.arange(start, min(start + step, int(hi)), stride, dtype=np.uint32)
            for sign in (np.uint32(0), np.uint32(0x80000000)):
                v = (bits | sign).view(np.float32)
                np.testing.assert_array_equal(relu6_kernel_formula(v, coef), relu6_definition(v, coef))
        small = np.array([0.0, -0.0, 1e-30, -1e-30, 0.1, -0.1, 1e9, -1e9], dtype=np.float32)
        np.testing.assert_array_equal(relu6_kernel_formula(small, coef), relu6_definition(small, coef))
