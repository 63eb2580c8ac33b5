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
