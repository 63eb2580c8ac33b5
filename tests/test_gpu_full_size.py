"""The benchmark configurations at their full sizes: direct comparison with
the oracle (it finishes in seconds on these), plus size-independent
properties (linearity of the int32 accumulators, agreement of the two
algorithms, batch independence)."""
import sys

import numpy as np
import pytest

from helpers import capi, workloads, pla, make_kernel, run_hip, run_oracle, assert_same

pytestmark = pytest.mark.gpu


def announce(*what):
    print("CASE", *what, file=sys.stderr, flush=True)


@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c4"])
def test_config_matches_oracle_at_full_size(name):
    announce("full", name)
    case = workloads.CONFIGS[name]()
    got = run_hip(case)
    want = run_oracle(case)
    assert_same(case, got, want, name)
    if case.kind == capi.KIND_INT8_INT8:
        # the workload is meant to exercise requantisation, not saturation
        sat = np.mean(np.abs(got.astype(np.int32)) == 127)
        assert sat < 0.5, "c4 output is mostly saturated (%.2f)" % sat


@pytest.mark.parametrize("name", ["c3", "c4"])
def test_int8_algorithms_agree_and_accumulators_are_linear(name):
    announce("props", name)
    case = workloads.CONFIGS[name]()
    case.kind = capi.KIND_INT8_ACC32
    walk = run_hip(case, capi.ALGO_ROW_WALK)
    mfma = run_hip(case, capi.ALGO_BLOCK_MFMA)
    assert np.array_equal(walk, mfma)
    # linearity: acc(x) = acc(x_even_bits) + acc(x_rest), with both parts valid int8
    lo = (case.x.astype(np.int16) // 2).astype(np.int8)
    hi = (case.x.astype(np.int16) - lo.astype(np.int16)).astype(np.int8)
    kernel, _ = make_kernel(case, capi.ALGO_BLOCK_MFMA)
    a = run_hip(case, kernel=kernel, x=lo)
    b = run_hip(case, kernel=kernel, x=hi)
    assert np.array_equal(a.astype(np.int64) + b.astype(np.int64), mfma.astype(np.int64))
    # checksum of checksums: sum over positions of acc = W @ (sum over positions of x)
    colsum = case.x.reshape(case.batch, case.x.shape[1], -1).astype(np.int64).sum(axis=2)  # [N, IC]
    want = colsum @ case.dense.astype(np.int64).T  # [N, OC]
    assert np.array_equal(mfma.reshape(case.batch, case.dense.shape[0], -1).astype(np.int64).sum(axis=2), want)


def test_batch_independence_and_image_permutation():
    announce("batch")
    case = workloads.config3(batch=8)
    full = run_hip(case)
    perm = np.array([3, 0, 7, 1, 6, 2, 5, 4])
    again = run_hip(case, x=np.ascontiguousarray(case.x[perm]))
    assert np.array_equal(again, full[perm])
    single = run_hip(case, x=np.ascontiguousarray(case.x[5:6]))
    assert np.array_equal(single[0], full[5])


@pytest.mark.parametrize("layer", [0, 5, 6, 11, 12])
def test_mobilenet_pointwise_layers_at_batch_8(layer):
    """Five of the thirteen config-5 layer shapes (first, the 14x14 and 7x7
    ones) with int8 requantisation and relu."""
    announce("c5 layer", layer)
    case = workloads.config5_layer(layer, batch=8)
    for algo in (capi.ALGO_BLOCK_MFMA, capi.ALGO_ROW_WALK):
        got = run_hip(case, algo)
        want = run_oracle(case)
        assert_same(case, got, want, "layer %d algo %d" % (layer, algo))
    sat = np.mean(got == 127)
    assert sat < 0.2


def test_mobilenet_pointwise_stack_chained_at_batch_64():
    """All thirteen config-5 layers at batch 64, run as the chained sequence
    the benchmark times: layer i+1 consumes layer i's int8 output on the
    device where the shapes chain, a fresh uniform int8 tensor is fed at the
    four spatial breaks.  Every layer is compared with the oracle on the
    first two and the last image of its actual input."""
    import torch

    prev = None
    chained_count = 0
    for i in range(13):
        announce("c5 chained layer", i)
        case = workloads.config5_layer(i)
        assert case.batch == 64
        ic, oc, hw = workloads.MOBILENET_V1_POINTWISE[i]
        kernel, _ = make_kernel(case, capi.ALGO_AUTO)
        chained = prev is not None and tuple(prev.shape[1:]) == (ic, hw, hw)
        chained_count += chained
        x = prev if chained else torch.from_numpy(case.x).cuda()
        out = kernel.Run(x)
        torch.cuda.synchronize()
        assert tuple(out.shape) == (64, oc, hw, hw) and out.dtype == torch.int8
        pick = [0, 1, 63]
        want = run_oracle(case, x=np.ascontiguousarray(x[pick].cpu().numpy()))
        got = out[pick].cpu().numpy()
        assert_same(case, got, want, "c5 chained layer %d" % i)
        assert np.mean(got == 127) < 0.2 and np.mean(got != 0) > 0.1, "layer %d output is degenerate" % i
        prev = out
    assert chained_count == 8  # 2->3, 4->5, 6->7 .. 10->11, 12->13


def test_mobilenet_body_26_launches_at_batch_64():
    """Depthwise 3x3 + pointwise, thirteen times, every layer consuming the
    previous layer's int8 output on the device (the `--config mobilenet`
    sequence of the benchmark), each layer compared with the oracle on the
    first two images of its actual input."""
    import torch

    from oracle import oracle as O

    rng = np.random.RandomState(5)
    x = torch.from_numpy(rng.randint(-127, 128, size=(64, 32, 112, 112)).astype(np.int8)).cuda()
    for i in range(13):
        announce("mobilenet block", i)
        dwc = workloads.config5_depthwise_layer(i)
        param = pla.ConvParam(dwc.filter, dwc.bias, strides=(dwc.stride, dwc.stride), paddings=(1, 1, 1, 1), activation_param=dwc.act, input_scale=dwc.input_scale,
                              weight_scale=dwc.weight_scale, output_scale=dwc.output_scale)
        dw = pla.DepthwiseConv(param, out_precision="int8")
        dw.PrepareForRun()
        t = dw.Run(x)
        torch.cuda.synchronize()
        a = O.Act()
        a.type = 1
        want = O.dwconv3x3_int8(x[:2].cpu().numpy(), dwc.filter[:, 0], dw.w_scale_, dw.bias_, a, out="int8", stride=dwc.stride, pad=1)
        assert np.array_equal(t[:2].cpu().numpy(), want), "depthwise layer %d differs from the oracle" % i
        case = workloads.config5_layer(i)
        kernel, _ = make_kernel(case)
        out = kernel.Run(t)
        torch.cuda.synchronize()
        want = run_oracle(case, x=np.ascontiguousarray(t[:2].cpu().numpy()))
        assert_same(case, out[:2].cpu().numpy(), want, "pointwise layer %d" % i)
        x = out
    assert tuple(x.shape) == (64, 1024, 7, 7)
