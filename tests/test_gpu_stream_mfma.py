"""The streaming block MFMA kernel (workgroups that walk over tiles, the next
tile's activations in flight during the epilogue) against the CPU oracle and
against the one-tile-per-workgroup kernel, through the C ABI: bit-exact.
Shapes: 128 and 256 input channels, one to three row groups, images of
exactly one tile, of several whole tiles, with a short last tile (4, 16 or 20
quads), fewer tiles than resident workgroups, and weight blocks that are
absent."""
import sys

import numpy as np
import pytest

from helpers import capi, workloads, pla, make_kernel, run_hip, run_oracle, oracle_pack, assert_same

pytestmark = pytest.mark.gpu

STREAM_ALWAYS = capi.tuning(mfma_stream=capi.TUNE_ALWAYS)
STREAM_NEVER = capi.tuning(mfma_stream=capi.TUNE_NEVER)

AP = pla.ActivationParam
ACTS = {
    "none": AP(),
    "relu": AP("relu"),
    "relu6": AP("relu6", Relu_clipped_coef=6.0),
    "leaky": AP("leaky_relu", Leaky_relu_alpha=0.1),
    "hswish": AP("hard_swish"),
}


def announce(*what):
    print("CASE", *what, file=sys.stderr, flush=True)


def case_for(out_int8, batch, ic, oc, h, w, sparsity, paired, act, seed):
    c = workloads.make_int8("stream", batch, ic, oc, h, w, sparsity, paired, act, out_int8=out_int8, seed=seed, output_scale=0.05 if out_int8 else 1.0)
    return c


# (batch, ic, oc, h, w): H*W / 4 = 16, 64 (two tiles), 100 (short tile of 4 quads), 144 (16), 256, 36 (one tile of 4 + ...), 784 (short tile of 16)
SHAPES = [
    (3, 128, 128, 8, 8), (2, 128, 256, 16, 16), (2, 256, 128, 20, 20), (1, 128, 384, 24, 24), (1, 256, 256, 32, 32), (5, 128, 128, 12, 12), (2, 128, 256, 56, 56), (70, 256, 128, 4, 4),
]


@pytest.mark.parametrize("out_int8", [False, True], ids=["fp32out", "int8out"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_stream_mfma_bit_exact(shape, out_int8):
    announce("stream", shape, out_int8)
    batch, ic, oc, h, w = shape
    for act in ("leaky", "hswish"):
        case = case_for(out_int8, batch, ic, oc, h, w, 0.8, False, ACTS[act], seed=ic + oc + h)
        want = run_oracle(case, oracle_pack(case))
        got = run_hip(case, capi.ALGO_BLOCK_MFMA, tuning=STREAM_ALWAYS)
        assert_same(case, got, want, "stream %s %s" % (act, shape))
        assert np.array_equal(got, run_hip(case, capi.ALGO_BLOCK_MFMA, tuning=STREAM_NEVER))


@pytest.mark.parametrize("act", sorted(ACTS))
@pytest.mark.parametrize("paired", [False, True], ids=["unstructured", "semi"])
def test_stream_mfma_activations_and_structures(paired, act):
    announce("stream acts", paired, act)
    for out_int8 in (False, True):
        case = case_for(out_int8, 2, 128, 128, 16, 12, 0.75, paired, ACTS[act], seed=11)
        got = run_hip(case, capi.ALGO_BLOCK_MFMA, force_semi=paired, tuning=STREAM_ALWAYS)
        assert_same(case, got, run_oracle(case, oracle_pack(case, force_semi=paired)), "stream %s" % act)


def test_stream_mfma_absent_blocks_and_no_bias():
    announce("stream blocks")
    case = case_for(True, 3, 256, 256, 16, 16, 0.5, False, ACTS["relu6"], seed=3)
    case.dense[32:64, :] = 0        # a row block without weights
    case.dense[:, 64:128] = 0       # two k-steps no row uses
    case.dense[128:160, 0:224] = 0  # a row block with one k-step
    case.bias = None
    got = run_hip(case, capi.ALGO_BLOCK_MFMA, tuning=STREAM_ALWAYS)
    assert_same(case, got, run_oracle(case, oracle_pack(case)), "absent blocks")
    kernel, _ = make_kernel(case, capi.ALGO_BLOCK_MFMA)
    info = kernel.info()
    assert info["mfma_blocks"] < info["mfma_blocks_total"]


def test_auto_takes_the_streaming_kernel_on_the_large_semi_structured_config_and_matches():
    """128 x 128 -> 256 @56x56 at a reduced batch: what AUTO runs equals the
    kernel with streaming switched off (the full-size parity run is in
    test_gpu_full_size.py)."""
    announce("stream c4-like")
    case = workloads.config4(batch=16)
    got = run_hip(case, capi.ALGO_AUTO)
    ref = run_hip(case, capi.ALGO_AUTO, tuning=STREAM_NEVER)
    assert np.array_equal(got, ref)
    assert_same(case, got[:2], run_oracle(case, oracle_pack(case), x=case.x[:2]), "c4-like")
