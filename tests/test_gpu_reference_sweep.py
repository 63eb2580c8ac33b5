"""The reference's own unit-test sweep, run on the GPU path.

lite/tests/math/sparse_conv_f32_compute_test.cc:391-403 and
sparse_conv_int8_compute_test.cc:498-507 loop over
m (output channels) in {1,16,64,128}, n (H*W, one image) in {1,32,128,256},
k (input channels) in {1,109,512}, bias in {0,1}, semi in {0,1}, sparsity in
{.5,.7,.8}, and activations {0,1,2,4,10} (fp32) / {0,1} (int8), with the
activation constants of the sweep's call (relu6 six = 6, leaky slope = 1,
hard_swish scale 1 / offset 1 / threshold 6; f32 test :136-156).  Inputs follow
the reference generators (uniform draws, value-thresholded masks: only the
largest positive weights survive; a "semi" mask that zeroes whole row pairs),
with a seeded numpy generator instead of random_device.  Expectations come
from the naive dense path the reference tests use (basic_gemm over every k,
zeros included) and are compared with the reference's own criteria:
fp32 results max_ratio <= 1e-4 or max_diff <= 5e-5 (tensor_cmp_host,
tensor_utils.h:267-330; test :336-361), int8 results |diff| <= 1 (:437-474).
The sparse layout comes from the detect-pass logic, as in the tests.
"""
import numpy as np
import pytest

from helpers import capi, workloads, pla, run_hip
from oracle import oracle as O

pytestmark = pytest.mark.gpu

MS, NS, KS = (1, 16, 64, 128), (1, 32, 128, 256), (1, 109, 512)
ACT_CODES = {0: pla.ActivationParam(), 1: pla.ActivationParam("relu"), 2: pla.ActivationParam("relu6", Relu_clipped_coef=6.0),
             4: pla.ActivationParam("leaky_relu", Leaky_relu_alpha=1.0), 10: pla.ActivationParam("hard_swish", hard_swish_threshold=6.0, hard_swish_scale=1.0, hard_swish_offset=1.0)}


def reference_weights_fp32(rng, m, k, sparsity, semi):
    w = rng.uniform(-1.0, 1.0, size=(m, k)).astype(np.float32)
    if not semi:
        keep = (w + 1.0) / 2.0 >= sparsity  # test :128-132
        return np.where(keep, w, 0).astype(np.float32)
    out = w.copy()
    flat = w.ravel()
    for i in range(m // 2):  # the test looks at flat element i for pair i (:112-118)
        if (flat[i] + 1.0) / 2.0 < sparsity:
            out[2 * i:2 * i + 2, :] = 0
    return out


def reference_weights_int8(rng, m, k, sparsity, semi):
    w = (-127 + 254 * rng.random(size=(m, k), dtype=np.float32)).astype(np.int32).astype(np.int8)  # truncation toward zero
    if not semi:
        keep = (w.astype(np.float32) + 128.0) / 255.0 >= sparsity  # test :110-114
        return np.where(keep, w, 0).astype(np.int8)
    out = w.copy()
    flat = w.ravel()
    for i in range(m // 2):
        if (float(flat[i]) + 128.0) / 255.0 < sparsity:
            out[2 * i:2 * i + 2, :] = 0
    return out


def cmp_host(truth, got):
    """tensor_cmp_host: the largest relative difference and the absolute
    difference at that element."""
    d = np.abs(truth.astype(np.float64) - got.astype(np.float64))
    r = d / (np.abs(truth.astype(np.float64)) + 1e-6)
    i = int(np.argmax(r))
    return float(r.ravel()[i]), float(d.ravel()[i])


@pytest.mark.parametrize("sparsity", [0.5, 0.7, 0.8])
@pytest.mark.parametrize("semi", [0, 1])
def test_fp32_sweep(semi, sparsity):
    rng = np.random.default_rng(1000 + 10 * semi + int(sparsity * 10))
    ran = 0
    for m in MS:
        for n in NS:
            for k in KS:
                w = reference_weights_fp32(rng, m, k, sparsity, semi)
                if not w.any():
                    continue  # nonzero_num <= 0 -> return true (:210-213)
                x = rng.uniform(-1.0, 1.0, size=(1, k, 1, n)).astype(np.float32)
                for has_bias in (0, 1):
                    bias = rng.uniform(-1.0, 1.0, size=m).astype(np.float32) if has_bias else None
                    for code, act in ACT_CODES.items():
                        case = workloads.Case("sweep", capi.KIND_FP32, x, w, bias, act)
                        got = run_hip(case).reshape(m, n)
                        oact = O.Act(code, 6.0, 1.0, 1.0, 1.0, 6.0)
                        truth = O.basic_gemm_f32(w, x.reshape(k, n), bias, oact)
                        ratio, diff = cmp_host(truth, got)
                        assert not (ratio > 1e-4 and diff > 5e-5), (m, n, k, has_bias, code, ratio, diff)
                        ran += 1
    assert ran > 200


@pytest.mark.parametrize("sparsity", [0.5, 0.7, 0.8])
@pytest.mark.parametrize("semi", [0, 1])
def test_int8_sweep(semi, sparsity):
    rng = np.random.default_rng(2000 + 10 * semi + int(sparsity * 10))
    ran = 0
    for m in MS:
        for n in NS:
            for k in KS:
                w = reference_weights_int8(rng, m, k, sparsity, semi)
                if not w.any():
                    continue
                x = (-127 + 254 * rng.random(size=(1, k, 1, n), dtype=np.float32)).astype(np.int32).astype(np.int8)
                # scales as the test sets them (:171-208): 1/127 each, output k/127
                sa = np.full(m, 1.0 / 127.0, np.float32)
                sb, sc = np.float32(1.0 / 127.0), np.float32(k / 127.0)
                for has_bias in (0, 1):
                    bias = rng.uniform(-1.0, 1.0, size=m).astype(np.float32) if has_bias else None
                    for code in (0, 1):
                        oact = O.Act(code, 6.0, 1.0, 1.0, 1.0, 6.0)
                        truth = O.basic_gemm_f32(O.int8_to_fp32(w, sa[0]), O.int8_to_fp32(x.reshape(k, n), sb), bias, oact)
                        case = workloads.Case("sweep", capi.KIND_INT8_FP32, x, w, bias, ACT_CODES[code], weight_scale=sa, input_scale=float(sb), output_scale=1.0)
                        got = run_hip(case).reshape(m, n)
                        ratio, diff = cmp_host(truth, got)
                        assert not (ratio > 1e-4 and diff > 5e-5), ("fp32 out", m, n, k, has_bias, code, ratio, diff)
                        case8 = workloads.Case("sweep", capi.KIND_INT8_INT8, x, w, bias, ACT_CODES[code], weight_scale=sa, input_scale=float(sb), output_scale=float(sc))
                        got8 = run_hip(case8).reshape(m, n)
                        want8 = O.fp32_to_int8(truth, sc)
                        assert np.abs(got8.astype(int) - want8.astype(int)).max() <= 1, ("int8 out", m, n, k, has_bias, code)
                        ran += 2
    assert ran > 100
