"""Parity of the HIP kernels (called through the C ABI) with the CPU oracle on
identical seeded inputs: int8 paths bit-exact, fp32 within 1e-5 relative."""
import sys

import numpy as np
import pytest

from helpers import capi, workloads, pla, make_kernel, run_hip, run_oracle, oracle_pack, assert_same, merged_for_oracle
from oracle import oracle as O

pytestmark = pytest.mark.gpu

AP = pla.ActivationParam
ACTS = {
    "none": AP(),
    "relu": AP("relu"),
    "relu6": AP("relu6", Relu_clipped_coef=6.0),
    "leaky": AP("leaky_relu", Leaky_relu_alpha=0.1),
    "hswish": AP("hard_swish"),
}
ALGOS = {"walk": capi.ALGO_ROW_WALK, "mfma": capi.ALGO_BLOCK_MFMA}


def announce(*what):
    print("CASE", *what, file=sys.stderr, flush=True)


def small_case(kind, batch, ic, oc, h, w, sparsity, paired, act, seed, output_scale=1.0):
    if kind == capi.KIND_FP32:
        return workloads.make_fp32("t", batch, ic, oc, h, w, sparsity, paired, act, seed=seed)
    c = workloads.make_int8("t", batch, ic, oc, h, w, sparsity, paired, act, out_int8=(kind == capi.KIND_INT8_INT8), seed=seed, output_scale=output_scale)
    c.kind = kind
    return c


def test_library_sees_the_device():
    assert capi.lib().pl_device_count() >= 1


# (batch, ic, oc, h, w): aligned and ragged spatial sizes, channel counts off
# the 4 / 32 grids, odd output channels, single pixel, single channel
SHAPES = [(2, 64, 64, 4, 4), (3, 37, 29, 7, 7), (1, 96, 48, 8, 6), (2, 130, 67, 5, 3), (1, 1, 1, 1, 1), (5, 8, 33, 1, 1), (1, 512, 40, 14, 14)]


@pytest.mark.parametrize("algo", ["walk", "mfma"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("paired", [False, True], ids=["unstructured", "semi"])
def test_int32_accumulators_bit_exact(shape, paired, algo):
    announce("acc", shape, paired, algo)
    batch, ic, oc, h, w = shape
    case = small_case(capi.KIND_INT8_ACC32, batch, ic, oc, h, w, 0.7, paired, AP(), seed=ic * 7 + oc)
    got = run_hip(case, ALGOS[algo], force_semi=paired)
    want = run_oracle(case, oracle_pack(case, force_semi=paired))
    assert_same(case, got, want, "int32 accumulators")
    # independent of both: plain integer matmul
    ref = np.einsum("mk,bkp->bmp", case.dense.astype(np.int64), case.x.reshape(batch, ic, -1).astype(np.int64)).reshape(got.shape)
    assert np.array_equal(got.astype(np.int64), ref)


@pytest.mark.parametrize("algo", ["walk", "mfma"])
@pytest.mark.parametrize("act", sorted(ACTS))
@pytest.mark.parametrize("out_int8", [False, True], ids=["fp32out", "int8out"])
@pytest.mark.parametrize("paired", [False, True], ids=["unstructured", "semi"])
def test_int8_outputs_bit_exact(paired, out_int8, act, algo):
    announce("int8", paired, out_int8, act, algo)
    kind = capi.KIND_INT8_INT8 if out_int8 else capi.KIND_INT8_FP32
    for shape in [(2, 72, 45, 6, 6), (2, 50, 31, 5, 5)]:
        batch, ic, oc, h, w = shape
        case = small_case(kind, batch, ic, oc, h, w, 0.8, paired, ACTS[act], seed=11 + ic, output_scale=0.05 if out_int8 else 1.0)
        got = run_hip(case, ALGOS[algo], force_semi=paired)
        want = run_oracle(case, oracle_pack(case, force_semi=paired))
        assert_same(case, got, want, "int8 %s %s" % (act, shape))
        if out_int8:
            assert np.abs(got.astype(int)).max() <= 127


# at most 64 input channels: a workgroup of the block MFMA kernel takes two
# or four tiles at once; forced here, the library only does so by itself on
# problems that keep more than 1024 workgroups.  (batch, ic, oc, h, w): full and
# ragged channel groups, 1 / 2 / 4 / 8 row blocks, aligned and odd images,
# a tile count that is not a multiple of the tiles per workgroup.
FEW_CHANNEL_SHAPES = [(3, 32, 64, 16, 16), (2, 64, 128, 12, 12), (2, 20, 32, 16, 8), (3, 50, 256, 10, 10), (2, 32, 48, 7, 7), (5, 64, 64, 8, 8), (1, 32, 96, 16, 16)]


@pytest.mark.parametrize("kind", ["acc32", "fp32out", "int8out"])
@pytest.mark.parametrize("shape", FEW_CHANNEL_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_few_channel_tiles_bit_exact(shape, kind):
    announce("few-channel", shape, kind)
    k = {"acc32": capi.KIND_INT8_ACC32, "fp32out": capi.KIND_INT8_FP32, "int8out": capi.KIND_INT8_INT8}[kind]
    batch, ic, oc, h, w = shape
    for act in ("relu", "hswish"):
        case = small_case(k, batch, ic, oc, h, w, 0.6, False, AP() if kind == "acc32" else ACTS[act], seed=3 * ic + oc, output_scale=0.05 if kind == "int8out" else 1.0)
        got = run_hip(case, capi.ALGO_BLOCK_MFMA, tuning=capi.tuning(mfma_sub_tiles=capi.TUNE_ALWAYS))
        want = run_oracle(case, oracle_pack(case))
        assert_same(case, got, want, "few-channel %s %s %s" % (kind, act, shape))


# 512 input channels with the tile width forced (the library picks narrower
# tiles when full ones would leave CUs idle): widths that do and do not divide
# the quads of an image, on shapes whose last tile is partial.
@pytest.mark.parametrize("kind", ["acc32", "fp32out", "int8out"])
@pytest.mark.parametrize("tq", [32, 25, 13, 8])
@pytest.mark.parametrize("shape", [(3, 512, 96, 14, 14), (2, 512, 160, 16, 16), (5, 512, 33, 7, 7)], ids=lambda s: "x".join(map(str, s)))
def test_tile_widths_bit_exact(shape, tq, kind):
    announce("tile-width", shape, tq, kind)
    k = {"acc32": capi.KIND_INT8_ACC32, "fp32out": capi.KIND_INT8_FP32, "int8out": capi.KIND_INT8_INT8}[kind]
    batch, ic, oc, h, w = shape
    case = small_case(k, batch, ic, oc, h, w, 0.85, False, AP() if kind == "acc32" else ACTS["relu"], seed=oc + tq, output_scale=0.1 if kind == "int8out" else 1.0)
    got = run_hip(case, capi.ALGO_BLOCK_MFMA, tuning=capi.tuning(mfma_tile_quads=tq))
    want = run_oracle(case, oracle_pack(case))
    assert_same(case, got, want, "tile-width %s %s tq=%d" % (kind, shape, tq))


# more than 1024 input channels: the block MFMA kernel takes the k-steps a
# chunk at a time through one LDS tile.  Aligned and odd images, a channel
# count off the 32 grid, images smaller than a quad, a chunk count of one
# plus a remainder.
MANY_CHANNEL_SHAPES = [(2, 2048, 64, 4, 4), (1, 1100, 40, 6, 6), (1, 1030, 33, 7, 7), (3, 1500, 20, 1, 2), (1, 1056, 128, 8, 8)]


@pytest.mark.parametrize("kind", ["acc32", "fp32out", "int8out"])
@pytest.mark.parametrize("shape", MANY_CHANNEL_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_many_channels_bit_exact(shape, kind):
    announce("many-channel", shape, kind)
    k = {"acc32": capi.KIND_INT8_ACC32, "fp32out": capi.KIND_INT8_FP32, "int8out": capi.KIND_INT8_INT8}[kind]
    batch, ic, oc, h, w = shape
    case = small_case(k, batch, ic, oc, h, w, 0.9, False, AP() if kind == "acc32" else ACTS["leaky"], seed=ic + oc, output_scale=0.2 if kind == "int8out" else 1.0)
    got = run_hip(case, capi.ALGO_BLOCK_MFMA)
    want = run_oracle(case, oracle_pack(case))
    assert_same(case, got, want, "many-channel %s %s" % (kind, shape))
    # the default choice for int8 is the same kernel now
    got_auto = run_hip(case, capi.ALGO_AUTO)
    assert np.array_equal(got_auto, got)


@pytest.mark.parametrize("act", sorted(ACTS))
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("paired", [False, True], ids=["unstructured", "semi"])
def test_fp32_within_tolerance(shape, paired, act):
    announce("fp32", shape, paired, act)
    batch, ic, oc, h, w = shape
    case = small_case(capi.KIND_FP32, batch, ic, oc, h, w, 0.8, paired, ACTS[act], seed=ic + 3 * oc)
    got = run_hip(case, capi.ALGO_ROW_WALK, force_semi=paired)
    want = run_oracle(case, oracle_pack(case, force_semi=paired))
    assert_same(case, got, want, "fp32 %s" % act)
    # and against the dense naive reference formula in float64
    if act == "none":
        ref = np.einsum("mk,bkp->bmp", case.dense.astype(np.float64), case.x.reshape(batch, ic, -1).astype(np.float64)) + case.bias[None, :, None]
        np.testing.assert_allclose(got.reshape(batch, oc, -1), ref, rtol=1e-4, atol=1e-5)


# fp32 walk over channel chunks (256 positions per workgroup, 64 channels
# staged at a time); forced here, the library picks it by itself only for
# large problems.  Needs H*W % 4 == 0.  (batch, ic, oc, h, w): one chunk and
# several, a channel count off the chunk grid, more row groups than one slice
# holds (32 or 64), an odd row count, a tile that spans images.
CHUNKED_SHAPES = [(2, 64, 64, 4, 4), (1, 96, 48, 8, 6), (3, 130, 67, 4, 5), (1, 300, 150, 16, 16), (5, 70, 33, 2, 2), (2, 257, 20, 12, 12)]


@pytest.mark.parametrize("act", ["none", "relu6", "hswish"])
@pytest.mark.parametrize("shape", CHUNKED_SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("paired", [False, True], ids=["unstructured", "semi"])
def test_fp32_chunked_walk(shape, paired, act):
    announce("fp32 chunked", shape, paired, act)
    batch, ic, oc, h, w = shape
    case = small_case(capi.KIND_FP32, batch, ic, oc, h, w, 0.75, paired, ACTS[act], seed=ic + 3 * oc)
    want = run_oracle(case, oracle_pack(case, force_semi=paired))
    got = run_hip(case, capi.ALGO_ROW_WALK, force_semi=paired, tuning=capi.tuning(walk_chunked=capi.TUNE_ALWAYS))
    assert_same(case, got, want, "fp32 chunked %s %s" % (act, shape))
    # four row groups per wavefront instead of eight: the same bits
    assert np.array_equal(got, run_hip(case, capi.ALGO_ROW_WALK, force_semi=paired, tuning=capi.tuning(walk_chunked=capi.TUNE_ALWAYS, chunk_walk_groups=4)))
    # and the plain walk gives the same bits (same order of fused multiply-adds)
    plain = run_hip(case, capi.ALGO_ROW_WALK, force_semi=paired, tuning=capi.tuning(walk_chunked=capi.TUNE_NEVER, walk_tiled=capi.TUNE_NEVER))
    assert np.array_equal(got, plain)


# fp32 walk with the whole tile and the index lists in LDS (128 positions and
# sixteen list streams per workgroup); forced here, the library picks it by
# itself for large problems.  At most 271 channels; with 272 - 543 channels
# the tiles have 64 positions and a wavefront instruction walks four row groups.
# (batch, ic, oc, h, w): fewer row groups than streams, more, an odd row
# count, a tile that spans images, a last tile that is not full, the largest
# channel count, lists longer than one LDS piece; then tiles of 64: the
# smallest and the largest channel count, tiles that span and end inside images.
TILED_SHAPES = [(2, 64, 8, 4, 4), (1, 96, 48, 8, 6), (3, 130, 67, 4, 5), (1, 271, 150, 16, 16), (5, 70, 33, 2, 2), (2, 257, 20, 12, 12), (3, 256, 96, 10, 10),
                (3, 272, 33, 2, 2), (1, 300, 150, 16, 16), (2, 512, 40, 6, 6), (1, 543, 20, 4, 4)]
# map sizes that are not a multiple of 4 (the tile is staged and stored element by element): 7 x 7, single
# pixels (four neighbouring positions in four images), 3 x 5 and 13 x 13, on tiles of 128 and of 64 positions
TILED_SHAPES += [(3, 64, 48, 7, 7), (9, 96, 33, 1, 1), (2, 130, 67, 3, 5), (4, 256, 96, 9, 9), (2, 300, 40, 7, 7), (1, 512, 64, 13, 13)]
# 544 - 1087 channels: tiles of 32 positions, eight row groups per wavefront instruction; 1088 - 2175: tiles of 16,
# sixteen row groups; aligned maps and 7 x 7 / 3 x 3 ones, fewer row groups than a step holds
TILED_SHAPES += [(2, 544, 20, 4, 4), (1, 1024, 48, 6, 6), (2, 1087, 9, 2, 2), (3, 800, 33, 7, 7), (1, 2048, 40, 4, 4), (2, 2175, 9, 2, 2), (2, 1500, 70, 3, 3)]


@pytest.mark.parametrize("act", ["none", "relu6", "hswish"])
@pytest.mark.parametrize("shape", TILED_SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("paired", [False, True], ids=["unstructured", "semi"])
def test_fp32_tiled_walk(shape, paired, act):
    announce("fp32 tiled", shape, paired, act)
    batch, ic, oc, h, w = shape
    sparsity = 0.3 if ic == 256 else 0.75  # the dense case: lists of ~180 entries, several LDS pieces per stream
    case = small_case(capi.KIND_FP32, batch, ic, oc, h, w, sparsity, paired, ACTS[act], seed=ic + 3 * oc)
    want = run_oracle(case, oracle_pack(case, force_semi=paired))
    got = run_hip(case, capi.ALGO_ROW_WALK, force_semi=paired, tuning=capi.tuning(walk_tiled=capi.TUNE_ALWAYS))
    assert_same(case, got, want, "fp32 tiled %s %s" % (act, shape))
    # the row groups dealt differently between the tile's own workgroup and the
    # workgroups of the CUs without a tile (none, 3/16, half of the work; the
    # run above took the share the library computes): the same bits
    for split in (0, 3, 8):  # the field holds 1 + sixteenths
        assert np.array_equal(got, run_hip(case, capi.ALGO_ROW_WALK, force_semi=paired, tuning=capi.tuning(walk_tiled=capi.TUNE_ALWAYS, walk_split=1 + split))), "split %s" % split
    # one row group per wavefront instruction (two positions per lane) instead of a pair of them (four): the same bits
    assert np.array_equal(got, run_hip(case, capi.ALGO_ROW_WALK, force_semi=paired, tuning=capi.tuning(walk_tiled=capi.TUNE_ALWAYS, walk_pairs=capi.TUNE_NEVER))), "single row groups"
    assert np.array_equal(got, run_hip(case, capi.ALGO_ROW_WALK, force_semi=paired, tuning=capi.tuning(walk_tiled=capi.TUNE_ALWAYS, walk_pairs=capi.TUNE_NEVER, walk_split=4))), "single row groups, split"
    # and the plain walk gives the same bits (same order of fused multiply-adds)
    plain = run_hip(case, capi.ALGO_ROW_WALK, force_semi=paired, tuning=capi.tuning(walk_tiled=capi.TUNE_NEVER, walk_chunked=capi.TUNE_NEVER))
    assert np.array_equal(got, plain)


@pytest.mark.parametrize("ic", [96, 300], ids=["tiles_of_128", "tiles_of_64"])
def test_fp32_tiled_walk_with_tensors_off_the_16_byte_grid(ic):
    """Tensors that start 4 bytes behind a 16-byte boundary take the element-wise form of the tile walk: the same
    bits as the aligned call, nothing written outside the output."""
    import torch

    announce("fp32 tiled, unaligned", ic)
    case = small_case(capi.KIND_FP32, 3, ic, 40, 6, 6, 0.75, False, ACTS["relu6"], seed=ic)
    kernel, _ = make_kernel(case, capi.ALGO_ROW_WALK, tuning=capi.tuning(walk_tiled=capi.TUNE_ALWAYS))
    want = run_hip(case, kernel=kernel)
    assert_same(case, want, run_oracle(case), "aligned")
    flat_x = torch.zeros(case.x.size + 8, dtype=torch.float32, device="cuda")
    x = flat_x[1:1 + case.x.size].view(case.x.shape)
    x.copy_(torch.from_numpy(case.x))
    flat_o = torch.full((want.size + 8,), 77.0, dtype=torch.float32, device="cuda")
    out = flat_o[1:1 + want.size].view(want.shape)
    assert x.data_ptr() % 16 == 4 and out.data_ptr() % 16 == 4
    kernel.Run(x, out)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), want)
    host = flat_o.cpu().numpy()
    assert host[0] == 77.0 and (host[1 + want.size:] == 77.0).all()


def test_no_bias_and_single_scale():
    announce("nobias")
    for kind in (capi.KIND_FP32, capi.KIND_INT8_FP32, capi.KIND_INT8_INT8):
        case = small_case(kind, 2, 40, 24, 4, 4, 0.6, False, ACTS["relu"], seed=5, output_scale=0.04 if kind == capi.KIND_INT8_INT8 else 1.0)
        case.bias = None
        if kind != capi.KIND_FP32:
            case.weight_scale = np.array([0.01], np.float32)
        for algo in ([capi.ALGO_ROW_WALK] if kind == capi.KIND_FP32 else [capi.ALGO_ROW_WALK, capi.ALGO_BLOCK_MFMA]):
            assert_same(case, run_hip(case, algo), run_oracle(case), "kind %d algo %d" % (kind, algo))


def test_empty_rows_all_zero_and_dense():
    announce("empty/dense")
    rng = np.random.RandomState(3)
    for kind in (capi.KIND_FP32, capi.KIND_INT8_FP32):
        case = small_case(kind, 2, 36, 20, 4, 4, 0.7, False, ACTS["leaky"], seed=9)
        case.dense[[0, 3, 19]] = 0  # empty first, middle and last rows
        for algo in ([capi.ALGO_ROW_WALK] if kind == capi.KIND_FP32 else [capi.ALGO_ROW_WALK, capi.ALGO_BLOCK_MFMA]):
            assert_same(case, run_hip(case, algo), run_oracle(case), "empty rows")
        zero = small_case(kind, 1, 12, 6, 4, 4, 0.5, False, ACTS["none"], seed=1)
        zero.dense[:] = 0
        for algo in ([capi.ALGO_ROW_WALK] if kind == capi.KIND_FP32 else [capi.ALGO_ROW_WALK, capi.ALGO_BLOCK_MFMA]):
            got = run_hip(zero, algo)
            assert_same(zero, got, run_oracle(zero), "all-zero weights")
        full = small_case(kind, 1, 16, 8, 4, 4, 0.0, False, ACTS["none"], seed=2)
        assert np.count_nonzero(full.dense) == full.dense.size
        assert_same(full, run_hip(full, capi.ALGO_ROW_WALK), run_oracle(full), "fully dense weights")
    del rng


def test_runtime_spatial_size_may_differ_from_baked_one():
    """Diffs are byte offsets baked for one H*W; the library converts them to
    channel indices once, so a handle serves any spatial size and batch."""
    announce("respatial")
    case = small_case(capi.KIND_INT8_FP32, 1, 48, 32, 4, 4, 0.75, False, ACTS["relu"], seed=21)
    kernel, _ = make_kernel(case)
    for (b, h, w) in [(1, 4, 4), (3, 7, 5), (2, 8, 8), (4, 1, 3)]:
        x = np.random.RandomState(b * 100 + h).randint(-127, 128, size=(b, 48, h, w)).astype(np.int8)
        got = run_hip(case, kernel=kernel, x=x)
        pk = O.pack_like_pass(case.dense, h * w)  # the oracle needs Diffs for this size
        want = run_oracle(case, pk, x=x)
        assert_same(case, got, want, "spatial %dx%d batch %d" % (h, w, b))


def test_set_epilogue_replaces_scales():
    import ctypes as C

    announce("set_epilogue")
    case = small_case(capi.KIND_INT8_FP32, 2, 32, 16, 4, 4, 0.7, False, ACTS["relu"], seed=4)
    kernel, _ = make_kernel(case)
    new_ws = np.linspace(0.002, 0.01, 16).astype(np.float32)
    merged = (new_ws * np.float32(case.input_scale)).astype(np.float32)
    capi.check(capi.lib().pl_sparse_conv_set_epilogue(kernel._handle, merged.ctypes.data, None, None))
    case.weight_scale = new_ws
    assert_same(case, run_hip(case, kernel=kernel), run_oracle(case), "after set_epilogue")
    del C


@pytest.mark.parametrize("paired", [False, True], ids=["unstructured", "semi"])
@pytest.mark.parametrize("ic", [130, 600, 1500], ids=["pairs", "eight_groups_per_step", "sixteen_groups_per_step"])
def test_set_epilogue_replaces_the_bias_of_every_fp32_walk(paired, ic):
    """The walk with the tile and the lists in LDS starts its accumulators from
    the bias carried in its list headers: a new bias must reach those too, and
    a handle prepared without a bias must take one."""
    announce("set_epilogue bias", paired, ic)
    for had_bias in (True, False):
        case = small_case(capi.KIND_FP32, 3, ic, 67, 4, 5, 0.75, paired, ACTS["relu6"], seed=31)
        new_bias = np.linspace(-0.7, 0.9, 67).astype(np.float32)
        if not had_bias:
            case.bias = None
        outs = []
        for tune in (capi.tuning(walk_tiled=capi.TUNE_ALWAYS), capi.tuning(walk_tiled=capi.TUNE_NEVER, walk_chunked=capi.TUNE_NEVER), capi.tuning(walk_tiled=capi.TUNE_NEVER, walk_chunked=capi.TUNE_ALWAYS)):
            kernel, _ = make_kernel(case, capi.ALGO_ROW_WALK, force_semi=paired, tuning=tune)
            capi.check(capi.lib().pl_sparse_conv_set_epilogue(kernel._handle, None, new_bias.ctypes.data, None))
            outs.append(run_hip(case, kernel=kernel))
        case.bias = new_bias
        want = run_oracle(case, oracle_pack(case, force_semi=paired))
        assert_same(case, outs[0], want, "tile walk after set_epilogue(bias)")
        assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])


@pytest.mark.parametrize("quirks", [True, False], ids=["reference_quirks", "scaled_once"])
@pytest.mark.parametrize("act", ["relu6", "leaky", "hswish"])
def test_kernel_class_parameter_merging(act, quirks):
    """SparseConvKernel.PrepareForRun against the merging written out with
    numpy in helpers.merged_for_oracle (int8 -> int8, where it matters)."""
    announce("merge", act, quirks)
    case = small_case(capi.KIND_INT8_INT8, 2, 64, 32, 4, 4, 0.7, False, ACTS[act], seed=31, output_scale=0.05)
    got = run_hip(case, quirks=quirks)
    want = run_oracle(case, quirks=quirks)
    assert_same(case, got, want, "merged %s" % act)
    # the oracle's own restatement of PrepareForRun agrees on scale and bias
    ms, mb, _ = O.merge_params(2, 32, case.weight_scale, case.input_scale, case.output_scale, case.bias, None)
    s, b, _ = merged_for_oracle(case, quirks)
    assert np.array_equal(ms, s) and np.array_equal(mb, b)


def test_error_paths_return_codes():
    import ctypes as C

    announce("errors")
    L = capi.lib()
    case = small_case(capi.KIND_INT8_FP32, 1, 16, 8, 2, 2, 0.5, False, ACTS["none"], seed=1)
    w = pla.detect_and_pack(case.dense, 4)
    d = capi.Desc()
    d.struct_size = C.sizeof(capi.Desc)
    d.kind, d.flag_semi, d.first_ic, d.oc, d.ic, d.im_size = capi.KIND_INT8_FP32, 0, w.first_ic, 8, 16, 4
    d.nonzero_weights, d.n_weights = w.nonzero_weights.ctypes.data, w.nonzero_weights.size
    d.oc_nonzeros, d.diffs, d.n_diffs = w.oc_nonzeros.ctypes.data, w.diffs.ctypes.data, w.diffs.size
    scale = np.ones(8, np.float32)
    d.scale = scale.ctypes.data
    h = C.c_void_p()
    # corrupt index: walk leaves the channels
    bad = w.diffs.copy()
    bad[0] = 4 * 1000
    d.diffs = bad.ctypes.data
    assert L.pl_sparse_conv_prepare(C.byref(d), C.byref(h)) == capi.PL_ERR_BAD_LAYOUT and not h.value
    assert "channels" in capi.last_error()
    bad[0] = 3  # not a multiple of im_size
    assert L.pl_sparse_conv_prepare(C.byref(d), C.byref(h)) == capi.PL_ERR_BAD_LAYOUT
    d.diffs = w.diffs.ctypes.data
    d.scale = None
    assert L.pl_sparse_conv_prepare(C.byref(d), C.byref(h)) == capi.PL_ERR_BAD_ARG
    d.scale = scale.ctypes.data
    d.struct_size = 8
    assert L.pl_sparse_conv_prepare(C.byref(d), C.byref(h)) == capi.PL_ERR_BAD_ARG
    d.struct_size = C.sizeof(capi.Desc)
    d.kind, d.algo = capi.KIND_FP32, capi.ALGO_BLOCK_MFMA
    assert L.pl_sparse_conv_prepare(C.byref(d), C.byref(h)) == capi.PL_ERR_UNSUPPORTED
    d.kind, d.algo = capi.KIND_INT8_FP32, capi.ALGO_AUTO
    assert L.pl_sparse_conv_prepare(C.byref(d), C.byref(h)) == capi.PL_OK and h.value
    assert L.pl_sparse_conv_run(h, None, None, 1, 4, None) == capi.PL_ERR_BAD_ARG
    assert L.pl_sparse_conv_run(h, None, None, 0, 4, None) == capi.PL_OK  # empty batch
    L.pl_sparse_conv_destroy(h)


def test_fp32_more_channels_than_the_plain_walks_lds_tile():
    """The plain fp32 walk keeps all channels of 16 positions (plus a zero row)
    in LDS: 2559 channels fit, 2560 do not.  Beyond that the walk over channel
    chunks serves the shapes it supports (H*W a multiple of 4, aligned
    tensors); other shapes are refused at the call, not at prepare."""
    import torch

    announce("fp32 large K")
    for ic, h, w, ok in ((2559, 3, 3, True), (2560, 3, 3, False), (2560, 4, 4, True), (3000, 2, 6, True), (3000, 5, 5, False)):
        case = small_case(capi.KIND_FP32, 2, ic, 24, h, w, 0.9, False, ACTS["relu"], seed=ic + h)
        kernel, _ = make_kernel(case, capi.ALGO_ROW_WALK)  # prepare succeeds in every case
        if ok:
            got = run_hip(case, kernel=kernel)
            assert_same(case, got, run_oracle(case, oracle_pack(case)), "fp32 ic=%d %dx%d" % (ic, h, w))
        else:
            with pytest.raises(capi.SparseConvError) as e:
                kernel.Run(torch.from_numpy(case.x).cuda())
            assert e.value.code == capi.PL_ERR_UNSUPPORTED
