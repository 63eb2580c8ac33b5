"""Half-precision sparse_conv2d on the GPU (through the C ABI) against the
oracle's binary16 restatement: same values for every output (the kernel
issues the same sequence of half-precision operations)."""
import numpy as np
import pytest

from helpers import capi, workloads, pla, run_hip, run_oracle, oracle_pack, assert_same

pytestmark = pytest.mark.gpu

AP = pla.ActivationParam
ACTS = {
    "none": AP(),
    "relu": AP("relu"),
    "relu6": AP("relu6", Relu_clipped_coef=6.0),
    "leaky": AP("leaky_relu", Leaky_relu_alpha=0.1),
    "hswish": AP("hard_swish"),
}
# (batch, ic, oc, h, w): even and odd images, a single pixel, channel counts
# off the batch-of-eight grid, more channels than one 128-position tile
# holds, odd row counts for the semi layout's tail row
SHAPES = [(2, 64, 64, 4, 4), (3, 37, 29, 7, 7), (1, 96, 48, 8, 6), (2, 130, 67, 5, 3), (1, 1, 1, 1, 1), (5, 8, 33, 1, 1), (1, 700, 40, 14, 14), (2, 256, 96, 28, 28)]


def half_case(batch, ic, oc, h, w, sparsity, paired, act, seed):
    c = workloads.make_fp32("t", batch, ic, oc, h, w, sparsity, paired, act, seed=seed)
    c.kind = capi.KIND_FP16
    c.x = c.x.astype(np.float16)
    return c


@pytest.mark.parametrize("act", sorted(ACTS))
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("paired", [False, True], ids=["unstructured", "semi"])
def test_fp16_same_values(shape, paired, act):
    batch, ic, oc, h, w = shape
    case = half_case(batch, ic, oc, h, w, 0.7, paired, ACTS[act], seed=ic + 5 * oc)
    got = run_hip(case, capi.ALGO_AUTO, force_semi=paired)
    want = run_oracle(case, oracle_pack(case, force_semi=paired))
    assert got.dtype == np.float16
    assert_same(case, got, want, "fp16 %s %s" % (act, shape))


def test_fp16_no_bias_and_new_epilogue():
    case = half_case(2, 48, 20, 6, 6, 0.6, False, ACTS["relu"], seed=3)
    case.bias = None
    got = run_hip(case)
    assert_same(case, got, run_oracle(case), "fp16 without bias")


# Half-precision walk over channel chunks (256 positions per workgroup, 64
# channels staged at a time); forced here, the library picks it by itself only
# for large problems.  Needs H*W % 4 == 0.  (batch, ic, oc, h, w): one chunk
# and several, a channel count off the chunk grid, more row groups than one
# slice holds, an odd row count, a tile that spans images.
CHUNKED_SHAPES = [(2, 64, 64, 4, 4), (1, 96, 48, 8, 6), (3, 130, 67, 4, 5), (1, 300, 150, 16, 16), (5, 70, 33, 2, 2), (2, 257, 20, 12, 12)]


@pytest.mark.parametrize("act", ["none", "relu6", "hswish"])
@pytest.mark.parametrize("shape", CHUNKED_SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("paired", [False, True], ids=["unstructured", "semi"])
def test_fp16_chunked_walk(shape, paired, act):
    batch, ic, oc, h, w = shape
    case = half_case(batch, ic, oc, h, w, 0.75, paired, ACTS[act], seed=ic + 3 * oc)
    want = run_oracle(case, oracle_pack(case, force_semi=paired))
    got = run_hip(case, capi.ALGO_AUTO, force_semi=paired, tuning=capi.tuning(walk_chunked=capi.TUNE_ALWAYS))
    assert_same(case, got, want, "fp16 chunked %s %s" % (act, shape))
    # the plain half-precision walk gives the same bits (same order of operations)
    plain = run_hip(case, capi.ALGO_AUTO, force_semi=paired, tuning=capi.tuning(walk_chunked=capi.TUNE_NEVER))
    assert np.array_equal(got.view(np.uint16), plain.view(np.uint16))


# Half-precision walk with the whole tile (256 positions, all channels) and the list streams in LDS, two row
# groups per wavefront instruction; forced here, the library picks it by itself from 7 tiles on.  Needs
# H*W % 8 == 0 and at most 271 channels.  (batch, ic, oc, h, w): one tile shared by ten workgroups, a channel
# count off the staging pass of 128, an odd number of row groups (a pair without partner), a tile that spans
# images and ends inside one, a single row group.
TILED_SHAPES = [(2, 64, 64, 4, 4), (1, 96, 48, 8, 6), (3, 130, 67, 4, 6), (5, 70, 33, 2, 4), (2, 257, 20, 12, 12), (3, 200, 1, 8, 8), (1, 271, 96, 16, 24)]
# Tiles of 128 positions (four per lane) serve maps whose size is a multiple of 4 only and up to 543 channels:
# 14 x 14 and 2 x 2 maps, a tile that ends inside an image, channel counts above the wide tile's limit on maps of
# both kinds, the largest channel count.
TILED_SHAPES += [(3, 64, 48, 14, 14), (7, 40, 33, 2, 2), (2, 257, 20, 6, 6), (1, 300, 150, 16, 16), (2, 512, 64, 14, 14), (1, 543, 40, 4, 4)]
# Any other map size goes in and out of the tile value by value: 7 x 7, single pixels (neighbouring positions in
# different images), 3 x 5, 9 x 9, 13 x 13, a map of 2 x 3, on tiles of 256 and of 128 positions.
TILED_SHAPES += [(3, 64, 48, 7, 7), (9, 96, 33, 1, 1), (2, 130, 67, 3, 5), (4, 256, 96, 9, 9), (2, 300, 40, 7, 7), (1, 512, 64, 13, 13), (5, 48, 20, 2, 3)]
# More channels on maps of a multiple of 8 positions: 4 / 8 / 16 row groups per wavefront instruction on tiles of
# 128 / 64 / 32 positions (up to 543 / 1087 / 2175 channels); the same with odd maps and with a map of 36 positions
# whose channels do not fit the narrow form; fewer row groups than a step holds.
TILED_SHAPES += [(1, 300, 150, 8, 8), (2, 543, 20, 4, 4), (1, 1024, 48, 8, 8), (2, 1087, 9, 2, 4), (1, 2048, 40, 4, 4), (2, 2175, 9, 2, 4), (3, 800, 33, 7, 7), (2, 1500, 70, 3, 3), (2, 600, 20, 6, 6)]


@pytest.mark.parametrize("act", ["none", "relu", "relu6", "leaky", "hswish"])
@pytest.mark.parametrize("shape", TILED_SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("paired", [False, True], ids=["unstructured", "semi"])
def test_fp16_tile_walk(shape, paired, act):
    batch, ic, oc, h, w = shape
    case = half_case(batch, ic, oc, h, w, 0.75, paired, ACTS[act], seed=ic + 3 * oc)
    want = run_oracle(case, oracle_pack(case, force_semi=paired))
    got = run_hip(case, capi.ALGO_AUTO, force_semi=paired, tuning=capi.tuning(walk_tiled=capi.TUNE_ALWAYS))
    assert_same(case, got, want, "fp16 tile walk %s %s" % (act, shape))


@pytest.mark.parametrize("batch", [3, 24, 40, 64, 65])
@pytest.mark.parametrize("ic,size", [(256, 28), (512, 14)], ids=["wide_tiles", "narrow_tiles"])
@pytest.mark.parametrize("paired", [False, True], ids=["unstructured", "semi"])
def test_fp16_tile_walk_divisions(batch, paired, ic, size):
    """Tiles shared by several workgroups in equal parts, main and spare parts, one tile per workgroup and more
    tiles than CUs: the bits of the plain half-precision walk (the oracle's, by the tests above) every time."""
    batch = batch if size == 28 else 4 * batch
    case = half_case(batch, ic, 512, size, size, 0.85, paired, ACTS["relu"], seed=batch)
    tiled = run_hip(case, capi.ALGO_AUTO, force_semi=paired, tuning=capi.tuning(walk_tiled=capi.TUNE_ALWAYS))
    plain = run_hip(case, capi.ALGO_AUTO, force_semi=paired, tuning=capi.tuning(walk_tiled=capi.TUNE_NEVER, walk_chunked=capi.TUNE_NEVER))
    assert np.array_equal(tiled.view(np.uint16), plain.view(np.uint16))


@pytest.mark.parametrize("ic", [128, 600], ids=["pairs", "eight_groups_per_step"])
@pytest.mark.parametrize("size", [16, 14], ids=["wide_tiles", "narrow_tiles"])
@pytest.mark.parametrize("had_bias", [True, False], ids=["bias", "no_bias"])
def test_fp16_tile_walk_takes_a_new_bias(had_bias, size, ic):
    """set_epilogue rewrites the biases in the list streams (the accumulators start from them), also in a handle
    that was prepared without one."""
    from helpers import make_kernel

    case = half_case(12 if ic == 128 else 3, ic, 96, size, size, 0.8, False, ACTS["relu"], seed=9)
    if not had_bias:
        case.bias = None
    kernel, _ = make_kernel(case, tuning=capi.tuning(walk_tiled=capi.TUNE_ALWAYS))
    assert_same(case, run_hip(case, kernel=kernel), run_oracle(case), "fp16 tile walk, first bias")
    new_bias = np.linspace(-0.7, 0.9, 96).astype(np.float32)
    capi.check(capi.lib().pl_sparse_conv_set_epilogue(kernel._handle, None, new_bias.ctypes.data, None))
    case.bias = new_bias
    assert_same(case, run_hip(case, kernel=kernel), run_oracle(case), "fp16 tile walk, second bias")


def test_fp16_tile_walk_with_tensors_off_the_16_byte_grid():
    """Tensors that start 2 bytes behind a 16-byte boundary take the value-by-value form of the tile walk: the same
    bits as the aligned call, nothing written outside the output."""
    import torch

    from helpers import make_kernel

    case = half_case(3, 96, 40, 8, 8, 0.75, False, ACTS["relu6"], seed=4)
    kernel, _ = make_kernel(case, tuning=capi.tuning(walk_tiled=capi.TUNE_ALWAYS))
    want = run_hip(case, kernel=kernel)
    assert_same(case, want, run_oracle(case), "aligned")
    flat_x = torch.zeros(case.x.size + 16, dtype=torch.float16, device="cuda")
    x = flat_x[1:1 + case.x.size].view(case.x.shape)
    x.copy_(torch.from_numpy(case.x))
    flat_o = torch.full((want.size + 16,), 77.0, dtype=torch.float16, device="cuda")
    out = flat_o[1:1 + want.size].view(want.shape)
    assert x.data_ptr() % 16 == 2 and out.data_ptr() % 16 == 2
    kernel.Run(x, out)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint16), want.view(np.uint16))
    host = flat_o.cpu().numpy()
    assert host[0] == 77.0 and (host[1 + want.size:] == 77.0).all()
