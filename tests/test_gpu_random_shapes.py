"""Seeded random shapes through the C ABI against the CPU oracle: the
hand-picked shapes of the other parity tests name the edges that were thought
of; these draw batch, channel counts, spatial sizes, sparsity, pairing,
activation and output kind at random (fixed seeds, so a failure names its
case).  int8 paths bit-exact, fp32 within 1e-5 relative (assert_same)."""
import sys

import numpy as np
import pytest

from helpers import capi, workloads, pla, run_hip, run_oracle, oracle_pack, assert_same
from test_gpu_dwconv import run_case as run_depthwise_case, ACTS as DW_ACTS

pytestmark = pytest.mark.gpu

AP = pla.ActivationParam
ACT_MAKERS = [
    lambda r: AP(),
    lambda r: AP("relu"),
    lambda r: AP("relu6", Relu_clipped_coef=float(r.choice([1.5, 6.0]))),
    lambda r: AP("leaky_relu", Leaky_relu_alpha=float(r.choice([0.01, 0.3]))),
    lambda r: AP("hard_swish"),
]
KINDS = [capi.KIND_FP32, capi.KIND_INT8_FP32, capi.KIND_INT8_INT8, capi.KIND_INT8_ACC32]


def draw_sparse_case(seed):
    r = np.random.RandomState(seed)
    kind = KINDS[seed % 4]
    # channel counts: mostly small, sometimes past the 64 / 512 / 1024 switches of the kernels
    ic = int(r.choice([r.randint(1, 40), r.randint(40, 300), r.randint(300, 1200)], p=[0.5, 0.35, 0.15]))
    oc = int(r.choice([r.randint(1, 40), r.randint(40, 200)], p=[0.6, 0.4]))
    h, w = int(r.randint(1, 24)), int(r.randint(1, 24))
    batch = int(r.randint(1, 5))
    sparsity = float(r.choice([0.0, 0.5, 0.8, 0.95, 1.0], p=[0.05, 0.25, 0.4, 0.25, 0.05]))
    paired = bool(r.randint(2)) and oc >= 2
    act = AP() if kind == capi.KIND_INT8_ACC32 else ACT_MAKERS[r.randint(len(ACT_MAKERS))](r)
    if kind == capi.KIND_FP32:
        case = workloads.make_fp32("r%d" % seed, batch, ic, oc, h, w, sparsity, paired, act, seed=seed)
    else:
        case = workloads.make_int8("r%d" % seed, batch, ic, oc, h, w, sparsity, paired, act, out_int8=(kind == capi.KIND_INT8_INT8), seed=seed,
                                   output_scale=0.07 if kind == capi.KIND_INT8_INT8 else 1.0)
        case.kind = kind
    return case, (kind, batch, ic, oc, h, w, sparsity, paired, act.active_type if act.has_active else 0)


@pytest.mark.parametrize("seed", range(96))
def test_sparse_conv_random_case(seed):
    case, what = draw_sparse_case(1000 + seed)
    print("CASE sparse_conv random", seed, what, file=sys.stderr, flush=True)
    algos = [capi.ALGO_AUTO] if case.kind == capi.KIND_FP32 else [capi.ALGO_ROW_WALK, capi.ALGO_BLOCK_MFMA]
    want = run_oracle(case, oracle_pack(case))
    for algo in algos:
        got = run_hip(case, algo)
        assert_same(case, got, want, "random case %d %s algo %d" % (seed, what, algo))


@pytest.mark.parametrize("seed", range(64))
def test_depthwise_random_case(seed):
    r = np.random.RandomState(5000 + seed)
    n, c = int(r.randint(1, 4)), int(r.choice([r.randint(1, 9), r.randint(9, 80)]))
    h, w = int(r.randint(1, 70)), int(r.randint(1, 70))
    stride, pad = int(r.randint(1, 3)), int(r.randint(0, 2))
    if h + 2 * pad < 3 or w + 2 * pad < 3:
        h, w = h + 2, w + 2
    out = ["int8", "fp32"][seed % 2]
    act = sorted(DW_ACTS)[r.randint(len(DW_ACTS))]
    print("CASE depthwise random", seed, (n, c, h, w, stride, pad, out, act), file=sys.stderr, flush=True)
    run_depthwise_case(n, c, h, w, stride, pad, out, DW_ACTS[act](), bool(r.randint(2)), seed=seed)
