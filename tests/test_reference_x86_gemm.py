"""The reference's x86 int8 GEMM (oracle/_ref/libref_x86_gemm.so, built from
lite/backends/x86/math/gemm_s8u8_*.cc where the checkout is present) driven
like its dense conv2d kernel drives a 1x1 convolution.  It is the "x86 dense
conv2d 1x1" leg of the benchmark's CPU baseline, a timing comparator: here it
is only shown to be called correctly.  With inputs in [-5, 5], the range of
the reference's own test (lite/tests/math/x86_conv_int8_compute_test.cc:96-97),
it equals exact integer arithmetic; over the full int8 range its saturating
16-bit pair sums make it deviate, which is why it is never used as a checker."""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.skipif(not O.have_ref_x86_gemm(), reason="oracle/_ref/libref_x86_gemm.so needs the reference checkout")


def exact(x, w, ws, in_scale, bias, relu_type, alpha):
    b, k = x.shape[0], x.shape[1]
    acc = np.einsum("mk,bkp->bmp", w.astype(np.int64), x.reshape(b, k, -1).astype(np.int64))
    v = acc * (ws.astype(np.float64) * in_scale)[None, :, None] + bias.astype(np.float64)[None, :, None]
    if relu_type == 1:
        v = np.maximum(v, 0)
    elif relu_type == 2:
        v = np.minimum(np.maximum(v, 0), alpha)
    elif relu_type == 3:
        v = np.where(v >= 0, v, v * alpha)
    return v.reshape(x.shape[0], w.shape[0], x.shape[2], x.shape[3])


@pytest.mark.parametrize("relu_type,alpha", [(0, 1.0), (1, 1.0), (2, 6.0), (3, 0.1)])
@pytest.mark.parametrize("threads", [1, 3])
def test_small_range_inputs_equal_exact_arithmetic(relu_type, alpha, threads):
    rng = np.random.RandomState(3 + relu_type)
    for (b, k, m, h, w_) in ((2, 64, 32, 14, 14), (3, 96, 48, 7, 7), (1, 512, 64, 14, 14)):
        x = rng.randint(-5, 6, size=(b, k, h, w_)).astype(np.int8)
        w = (rng.randint(-5, 6, size=(m, k)) * (rng.random_sample((m, k)) < 0.2)).astype(np.int8)
        ws = rng.uniform(0.001, 0.02, m).astype(np.float32)
        bias = (rng.standard_normal(m) * 0.1).astype(np.float32)
        out, secs = O.ref_x86_conv1x1_s8_f32(x, w, ws, 0.01, bias, relu_type, alpha, reps=1, threads=threads)
        assert secs > 0
        np.testing.assert_allclose(out, exact(x, w, ws, np.float32(0.01), bias, relu_type, alpha), rtol=1e-5, atol=1e-6)


def test_full_range_inputs_deviate():
    rng = np.random.RandomState(0)
    x = rng.randint(-127, 128, size=(1, 512, 14, 14)).astype(np.int8)
    w = rng.randint(-127, 128, size=(64, 512)).astype(np.int8)
    ws = np.full(64, 2e-4, dtype=np.float32)
    out, _ = O.ref_x86_conv1x1_s8_f32(x, w, ws, 1.0, np.zeros(64, np.float32), 0, 1.0)
    err = np.abs(out - exact(x, w, ws, np.float32(1.0), np.zeros(64, np.float32), 0, 1.0))
    assert err.max() > 0.5  # saturation in the 16-bit pair sums: a timing comparator only
