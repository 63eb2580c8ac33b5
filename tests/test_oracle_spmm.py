"""Pins the oracle's SpMM walkers and epilogue: exact integer matmul, the
reference's own naive math (oracle/_ref, when built), closed forms of the
epilogue and rounding known answers."""
import numpy as np
import pytest

from oracle import oracle as O

needs_ref = pytest.mark.skipif(not O.have_ref(), reason="oracle/_ref not built (reference checkout absent)")

ACTS = [O.Act(O.ACT_NONE), O.Act(O.ACT_RELU), O.Act(O.ACT_RELU6, relu6_coef=6.0),
        O.Act(O.ACT_LEAKY_RELU, leaky_alpha=0.1), O.Act(O.ACT_HARD_SWISH)]


def _mask(rng, M, K, sparsity, paired):
    if paired:
        half = rng.random(((M + 1) // 2, K)) >= sparsity
        return np.repeat(half, 2, axis=0)[:M]
    return rng.random((M, K)) >= sparsity


def make_int8(rng, M, K, batch, H, W, sparsity, paired):
    w = rng.integers(-127, 128, size=(M, K)).astype(np.int8)
    w[w == 0] = 1
    w = (w * _mask(rng, M, K, sparsity, paired)).astype(np.int8)
    x = rng.integers(-127, 128, size=(batch, K, H, W)).astype(np.int8)
    return w, x


def make_fp32(rng, M, K, batch, H, W, sparsity, paired):
    w = (rng.standard_normal((M, K)) * 0.1).astype(np.float32)
    w[w == 0] = 0.1
    w = (w * _mask(rng, M, K, sparsity, paired)).astype(np.float32)
    x = rng.uniform(-1, 1, size=(batch, K, H, W)).astype(np.float32)
    return w, x


def exact_acc(w, x):
    b, K, H, W = x.shape
    return np.einsum("mk,bkp->bmp", w.astype(np.int64), x.reshape(b, K, -1).astype(np.int64)).reshape(b, w.shape[0], H, W)


@pytest.mark.parametrize("paired", [False, True])
@pytest.mark.parametrize("shape", [(1, 1, 1, 1, 1), (5, 9, 2, 3, 5), (16, 109, 1, 4, 8), (64, 40, 3, 7, 7), (33, 128, 2, 14, 14)])
def test_int8_accumulators_equal_integer_matmul(shape, paired):
    M, K, batch, H, W = shape
    rng = np.random.default_rng(M * 1000 + K)
    w, x = make_int8(rng, M, K, batch, H, W, 0.7, paired)
    layout = O.LAYOUT_SEMI if paired else O.LAYOUT_UNPADDED
    pk = O.pack(w, H * W, layout)
    acc = O.sparse_conv_int8_acc(pk, x)
    assert np.array_equal(acc.astype(np.int64), exact_acc(w, x))
    # a semi layout of an unpaired matrix keeps the zero partner weights and
    # must give the same sums
    pk2 = O.pack(w, H * W, O.LAYOUT_SEMI)
    assert np.array_equal(O.sparse_conv_int8_acc(pk2, x), acc)


@needs_ref
def test_int8_accumulators_equal_reference_conv_basic():
    rng = np.random.default_rng(5)
    w, x = make_int8(rng, 24, 50, 3, 6, 5, 0.8, False)
    pk = O.pack(w, 30, O.LAYOUT_UNPADDED)
    assert np.array_equal(O.sparse_conv_int8_acc(pk, x), O.ref_conv1x1_s8_s32(x, w))


def test_int8_epilogue_reduces_to_accumulator():
    rng = np.random.default_rng(11)
    w, x = make_int8(rng, 8, 30, 2, 3, 3, 0.5, False)
    pk = O.pack(w, 9, O.LAYOUT_UNPADDED)
    out = O.sparse_conv_int8(pk, x, np.ones(8, np.float32))
    assert np.array_equal(out, exact_acc(w, x).astype(np.float32))
    # scale 2^-k and integer bias stay exact in fp32: closed form
    s = np.full(8, 2.0 ** -10, np.float32)
    b = np.arange(8, dtype=np.float32)
    out = O.sparse_conv_int8(pk, x, s, b, O.Act(O.ACT_RELU))
    expect = np.maximum(exact_acc(w, x) * 2.0 ** -10 + b[None, :, None, None], 0)
    assert np.array_equal(out, expect.astype(np.float32))


@pytest.mark.parametrize("act", ACTS, ids=lambda a: "act%d" % a.type)
def test_int8_outputs_follow_fma_then_activation(act):
    rng = np.random.default_rng(act.type + 3)
    M, K = 12, 64
    w, x = make_int8(rng, M, K, 2, 5, 4, 0.75, False)
    pk = O.pack(w, 20, O.LAYOUT_UNPADDED)
    scale = rng.uniform(0.001, 0.02, M).astype(np.float32) * np.float32(0.01)
    bias = (rng.standard_normal(M) * 0.1).astype(np.float32)
    acc = exact_acc(w, x)
    # independent numpy statement: one correctly rounded fma, then the act
    v = (acc.astype(np.float64) * scale.astype(np.float64)[None, :, None, None]
         + bias.astype(np.float64)[None, :, None, None]).astype(np.float32)
    # (float64 product of a <2^24 integer and a float32 is exact, the sum is
    # rounded once when cast: the same value as fmaf up to double rounding,
    # which cannot occur here because the exact sum fits 53 bits)
    if act.type == O.ACT_RELU:
        e = np.maximum(v, 0)
    elif act.type == O.ACT_RELU6:
        e = np.minimum(np.maximum(v, 0), np.float32(act.relu6_coef))
    elif act.type == O.ACT_LEAKY_RELU:
        e = np.where(v >= 0, v, v * np.float32(act.leaky_alpha))
    elif act.type == O.ACT_HARD_SWISH:
        inv = np.float32(1.0 / act.hs_scale)
        gate = np.minimum(np.maximum(v + np.float32(act.hs_offset), 0), np.float32(act.hs_threshold))
        e = (v * inv) * gate
    else:
        e = v
    out = O.sparse_conv_int8(pk, x, scale, bias, act)
    assert np.array_equal(out, e.astype(np.float32))
    # int8 output = the oracle's own rounding rule applied to the same values
    # with scales that map the range onto int8
    s8 = (scale / np.float32(0.05)).astype(np.float32)
    out8 = O.sparse_conv_int8(pk, x, s8, None, None, out_int8=True)
    v8 = (acc.astype(np.float64) * s8.astype(np.float64)[None, :, None, None]).astype(np.float32)
    r = np.sign(v8) * np.floor(np.abs(v8.astype(np.float64)) + 0.5)
    assert np.array_equal(out8, np.clip(r, -127, 127).astype(np.int8))


def test_rounding_known_answers():
    xs = np.array([0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 126.5, -126.5, 127.5, -127.5, -128.0, -200.0, 300.0, 0.49999997, -0.49999997, 0.0], np.float32)
    want = np.array([1, -1, 2, -2, 3, -3, 127, -127, 127, -127, -127, -127, 127, 0, 0, 0], np.int8)
    assert np.array_equal(O.fp32_to_int8(xs, 1.0), want)
    # through the kernel epilogue: acc = 2x as integer, scale 0.5
    w = np.array([[1]], np.int8)
    pk = O.pack(w, 1, O.LAYOUT_UNPADDED)
    for acc, q in [(1, 1), (-1, -1), (3, 2), (-3, -2), (253, 127), (-253, -127), (-127, -64), (127, 64)]:
        # acc = 1 * x needs |x| <= 127: use bias to reach the larger values
        x = np.array([[[[np.sign(acc) * min(abs(acc), 127)]]]], np.int8)
        rest = acc - int(x.ravel()[0])
        out = O.sparse_conv_int8(pk, x, np.array([0.5], np.float32), np.array([rest * 0.5], np.float32), None, out_int8=True)
        assert out.ravel()[0] == q, (acc, out)


@pytest.mark.parametrize("paired", [False, True])
@pytest.mark.parametrize("act", ACTS, ids=lambda a: "act%d" % a.type)
def test_fp32_walker_against_naive_dense(act, paired):
    rng = np.random.default_rng(17 + act.type)
    M, K, batch, H, W = 19, 57, 2, 6, 5
    w, x = make_fp32(rng, M, K, batch, H, W, 0.8, paired)
    bias = (rng.standard_normal(M) * 0.1).astype(np.float32)
    pk = O.pack(w, H * W, O.LAYOUT_SEMI if paired else O.LAYOUT_PADDED)
    out = O.sparse_conv_fp32(pk, x, bias, act)
    for b in range(batch):
        naive = O.basic_gemm_f32(w, x[b].reshape(K, -1), bias, act)
        np.testing.assert_allclose(out[b].reshape(M, -1), naive, rtol=1e-5, atol=1e-6)
    # float64 ground truth
    v = np.einsum("mk,bkp->bmp", w.astype(np.float64), x.reshape(batch, K, -1).astype(np.float64)) + bias[None, :, None]
    if act.type == O.ACT_NONE:
        np.testing.assert_allclose(out.reshape(batch, M, -1), v, rtol=1e-5, atol=1e-6)


@needs_ref
@pytest.mark.parametrize("act", ACTS, ids=lambda a: "act%d" % a.type)
def test_naive_restatement_equals_reference_header(act):
    rng = np.random.default_rng(23)
    a = rng.standard_normal((13, 31)).astype(np.float32)
    b = rng.standard_normal((31, 22)).astype(np.float32)
    bias = rng.standard_normal(13).astype(np.float32)
    for bb in (None, bias):
        assert np.array_equal(O.basic_gemm_f32(a, b, bb, act), O.ref_basic_gemm_f32(a, b, bb, act))
    x = b.reshape(1, 31, 2, 11)
    if act.type != O.ACT_LEAKY_RELU:  # conv_basic's leaky slope argument is its own
        np.testing.assert_allclose(O.ref_conv1x1_f32(x, a, bias, act).reshape(13, 22), O.basic_gemm_f32(a, b, bias, act), rtol=1e-5, atol=1e-6)


def test_unit_test_int8_reference_flow_agrees_within_one():
    """The reference int8 test compares kernels with dequantise -> basic_gemm ->
    fp32_to_int8 and tolerates |diff| <= 1
    (lite/tests/math/sparse_conv_int8_compute_test.cc:171-208, 414-474)."""
    rng = np.random.default_rng(31)
    M, K, N = 16, 109, 32
    w, x = make_int8(rng, M, K, 1, 1, N, 0.7, False)
    bias = rng.uniform(-1, 1, M).astype(np.float32)
    sa, sb, sc = np.float32(1 / 127.0), np.float32(1 / 127.0), np.float32(K / 127.0)
    c = O.basic_gemm_f32(O.int8_to_fp32(w, sa), O.int8_to_fp32(x.reshape(K, N), sb), bias, O.Act(O.ACT_RELU))
    want8 = O.fp32_to_int8(c, sc)
    pk = O.pack(w, N, O.LAYOUT_UNPADDED)
    ms, mb, act = O.merge_params(2, M, np.float32(sa), sb, sc, bias, O.Act(O.ACT_RELU))
    got8 = O.sparse_conv_int8(pk, x, ms, mb, act, out_int8=True).reshape(M, N)
    assert np.abs(got8.astype(int) - want8.astype(int)).max() <= 1
    gotf = O.sparse_conv_int8(pk, x, *O.merge_params(1, M, np.float32(sa), sb, 1.0, bias, O.Act(O.ACT_RELU))[:2], O.Act(O.ACT_RELU)).reshape(M, N)
    np.testing.assert_allclose(gotf, c, rtol=1e-4, atol=5e-5)


def test_merge_params_closed_forms():
    ws = np.array([0.5, 0.25, 2.0], np.float32)
    b = np.array([1.0, -2.0, 4.0], np.float32)
    ms, mb, a = O.merge_params(1, 3, ws, 0.5, 0.25, b, O.Act(O.ACT_RELU6, relu6_coef=6.0))
    assert ms.tolist() == [0.25, 0.125, 1.0] and mb.tolist() == b.tolist() and a.relu6_coef == 6.0
    ms, mb, a = O.merge_params(2, 3, ws, 0.5, 0.25, b, O.Act(O.ACT_RELU6, relu6_coef=6.0))
    assert ms.tolist() == [1.0, 0.5, 4.0] and mb.tolist() == [4.0, -8.0, 16.0] and a.relu6_coef == 24.0
    ms, _, a = O.merge_params(2, 3, np.float32(0.5), 0.5, 0.25, None, O.Act(O.ACT_HARD_SWISH))
    assert ms.tolist() == [1.0, 1.0, 1.0]
    assert (a.hs_scale, a.hs_offset, a.hs_threshold) == (24.0, 12.0, 24.0)
    _, _, a = O.merge_params(2, 3, ws, 0.5, 0.25, None, O.Act(O.ACT_LEAKY_RELU, leaky_alpha=0.5))
    assert a.leaky_alpha == 2.0  # the kernel class rescales the slope as well
    with pytest.raises(ValueError):
        O.merge_params(1, 3, ws[:2], 1.0, 1.0, None, None)


@pytest.mark.parametrize("kind", [0, 1, 2])
def test_dense_comparator_matches_walker(kind):
    rng = np.random.default_rng(41 + kind)
    M, K, batch, H, W = 70, 45, 3, 9, 7
    act = O.Act(O.ACT_LEAKY_RELU, leaky_alpha=0.1)
    if kind == 0:
        w, x = make_fp32(rng, M, K, batch, H, W, 0.8, False)
        bias = rng.standard_normal(M).astype(np.float32)
        pk = O.pack(w, H * W, O.LAYOUT_PADDED)
        got, used = O.dense_conv1x1(0, w, x, None, bias, act, threads=3)
        np.testing.assert_allclose(got, O.sparse_conv_fp32(pk, x, bias, act), rtol=1e-5, atol=1e-6)
    else:
        w, x = make_int8(rng, M, K, batch, H, W, 0.8, False)
        scale = rng.uniform(1e-5, 2e-4, M).astype(np.float32) * (20 if kind == 2 else 1)
        bias = rng.standard_normal(M).astype(np.float32)
        pk = O.pack(w, H * W, O.LAYOUT_UNPADDED)
        got, used = O.dense_conv1x1(kind, w, x, scale, bias, act, threads=3)
        assert np.array_equal(got, O.sparse_conv_int8(pk, x, scale, bias, act, out_int8=(kind == 2)))
    assert used == 3
