"""The image MFMA kernel (one workgroup per image and 128 output rows, whole
image in LDS) against the CPU oracle through the C ABI: bit-exact for every
int8 kind.  Shapes cover every class of row alignment (H*W / 4 mod 4 = 0..3),
one to sixteen window quads left over at the end of a row, images smaller
than one window, every supported channel count and several row groups; and
the kernel for 7 x 7 maps (two images per workgroup)."""
import copy
import sys

import numpy as np
import pytest

from helpers import capi, workloads, pla, make_kernel, run_hip, run_oracle, oracle_pack, assert_same

pytestmark = pytest.mark.gpu

AP = pla.ActivationParam
ACTS = {
    "none": AP(),
    "relu": AP("relu"),
    "relu6": AP("relu6", Relu_clipped_coef=6.0),
    "leaky": AP("leaky_relu", Leaky_relu_alpha=0.1),
    "hswish": AP("hard_swish"),
}
KINDS = {"acc32": capi.KIND_INT8_ACC32, "fp32out": capi.KIND_INT8_FP32, "int8out": capi.KIND_INT8_INT8}


def announce(*what):
    print("CASE", *what, file=sys.stderr, flush=True)


def case_for(kind, batch, ic, oc, h, w, sparsity, paired, act, seed):
    c = workloads.make_int8("img", batch, ic, oc, h, w, sparsity, paired, act, out_int8=(kind == capi.KIND_INT8_INT8), seed=seed, output_scale=0.05 if kind == capi.KIND_INT8_INT8 else 1.0)
    c.kind = kind
    return c


# (batch, ic, oc, h, w).  H*W/4 mod 4: 14x14 -> 1, 6x10 -> 3, 8x8 -> 0, 6x9 -> ... (54 is not a multiple of 4, excluded),
# 10x10 -> 1, 12x14 -> 2, 16x16 -> 0 (largest image), 4x4 -> 0 (smaller than a window), 5x8 -> 2, 4x7 -> 3
# Maps with H*W = 4 (mod 8) can also be taken by the kernel with transposing LDS reads when it is
# asked for; both run here on every such shape (4x59 is the largest with 512 channels, 12x21 the largest at all,
# 2x10 the smallest, 6x6 / 4x11 / 4x13 have two to four windows per row).
SHAPES = [
    (3, 512, 128, 14, 14), (2, 256, 256, 6, 10), (2, 128, 128, 8, 8), (1, 512, 384, 10, 10), (2, 256, 128, 12, 14),
    (1, 512, 128, 16, 16), (3, 128, 256, 4, 4), (2, 256, 128, 5, 8), (2, 128, 128, 4, 7), (1, 512, 128, 9, 12), (9, 256, 128, 2, 10),
    (2, 512, 128, 4, 59), (1, 256, 128, 12, 21), (1, 128, 256, 6, 6), (2, 256, 128, 4, 11), (3, 128, 128, 4, 13),
]
IMAGE_KERNELS = {"regroup": capi.IMAGE_KERNEL_REGROUP, "transpose": capi.IMAGE_KERNEL_TRANSPOSE, "rows": capi.IMAGE_KERNEL_ROWS}
REGROUP = capi.tuning(image_kernel=capi.IMAGE_KERNEL_REGROUP)
# the regrouping kernel regroups 512-channel 14 x 14 images by transposing LDS reads unless told otherwise
VALU_REGROUP = capi.tuning(image_kernel=capi.IMAGE_KERNEL_REGROUP, image_tr_regroup=capi.TUNE_NEVER)


@pytest.mark.parametrize("image_kernel", sorted(IMAGE_KERNELS))
@pytest.mark.parametrize("kind", sorted(KINDS))
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_image_mfma_bit_exact(shape, kind, image_kernel):
    announce("image", shape, kind, image_kernel)
    batch, ic, oc, h, w = shape
    k = KINDS[kind]
    if image_kernel == "transpose" and (h * w) % 8 != 4:
        # refused, not rerouted
        case = case_for(k, batch, ic, oc, h, w, 0.85, False, ACTS["none"], seed=1)
        with pytest.raises(capi.SparseConvError) as e:
            run_hip(case, capi.ALGO_IMAGE_MFMA, tuning=capi.tuning(image_kernel=capi.IMAGE_KERNEL_TRANSPOSE))
        assert e.value.code == capi.PL_ERR_UNSUPPORTED
        return
    for act in (("none",) if kind == "acc32" else ("leaky", "hswish")):
        case = case_for(k, batch, ic, oc, h, w, 0.85, False, ACTS[act], seed=ic + 3 * oc + h * w)
        got = run_hip(case, capi.ALGO_IMAGE_MFMA, tuning=capi.tuning(image_kernel=IMAGE_KERNELS[image_kernel]))
        want = run_oracle(case, oracle_pack(case))
        assert_same(case, got, want, "image %s %s %s" % (kind, act, shape))
        if image_kernel == "regroup" and (ic, h * w) == (512, 196):
            assert np.array_equal(got, run_hip(case, capi.ALGO_IMAGE_MFMA, tuning=VALU_REGROUP)), "regrouping by the vector ALU"
    if kind == "acc32":
        ref = np.einsum("mk,bkp->bmp", case.dense.astype(np.int64), case.x.reshape(batch, ic, -1).astype(np.int64)).reshape(got.shape)
        assert np.array_equal(got.astype(np.int64), ref)


@pytest.mark.parametrize("act", sorted(ACTS))
@pytest.mark.parametrize("kind", sorted(KINDS))
def test_image_mfma_regroup_by_transposing_reads(kind, act):
    """512 channels, 14 x 14: the regrouping image kernel lets the LDS transpose (its own order of the
    channels inside a k-step); several row groups, an odd batch, every activation, channels of one parity
    only in some rows, and the same bits as with the vector-ALU regrouping."""
    announce("image tr regroup", kind, act)
    k = KINDS[kind]
    if kind == "acc32" and act != "none":
        pytest.skip("accumulators have no activation")
    case = case_for(k, 5, 512, 256, 14, 14, 0.85, False, ACTS[act], seed=len(act) + 31)
    case.dense[3, 0::2] = 0
    case.dense[4, 1::2] = 0
    case.dense[9] = 0
    got = run_hip(case, capi.ALGO_IMAGE_MFMA, tuning=REGROUP)
    assert_same(case, got, run_oracle(case, oracle_pack(case)), "tr regroup %s %s" % (kind, act))
    assert np.array_equal(got, run_hip(case, capi.ALGO_IMAGE_MFMA, tuning=VALU_REGROUP))


# 7 x 7 maps (49-byte channel rows, two images per workgroup): every supported
# channel count, one and several row groups, odd batches (a last pair with one
# image) and a single image.
SMALL_MAP_SHAPES = [(2, 256, 128, 7, 7), (5, 512, 256, 7, 7), (1, 1024, 128, 7, 7), (4, 1024, 256, 7, 7), (3, 512, 128, 7, 7)]


@pytest.mark.parametrize("kind", sorted(KINDS))
@pytest.mark.parametrize("shape", SMALL_MAP_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_small_map_mfma_bit_exact(shape, kind):
    announce("small map", shape, kind)
    batch, ic, oc, h, w = shape
    k = KINDS[kind]
    for act in (("none",) if kind == "acc32" else ("relu", "hswish")):
        case = case_for(k, batch, ic, oc, h, w, 0.9, False, ACTS[act], seed=ic + 5 * oc + batch)
        got = run_hip(case, capi.ALGO_IMAGE_MFMA)
        want = run_oracle(case, oracle_pack(case))
        assert_same(case, got, want, "small map %s %s %s" % (kind, act, shape))
        assert np.array_equal(got, run_hip(case, capi.ALGO_BLOCK_MFMA))
    if kind == "acc32":
        ref = np.einsum("mk,bkp->bmp", case.dense.astype(np.int64), case.x.reshape(batch, ic, -1).astype(np.int64)).reshape(got.shape)
        assert np.array_equal(got.astype(np.int64), ref)


@pytest.mark.parametrize("act", sorted(ACTS))
@pytest.mark.parametrize("out_int8", [False, True], ids=["fp32out", "int8out"])
@pytest.mark.parametrize("paired", [False, True], ids=["unstructured", "semi"])
def test_small_map_mfma_activations_and_structures(paired, out_int8, act):
    announce("small map acts", paired, out_int8, act)
    kind = capi.KIND_INT8_INT8 if out_int8 else capi.KIND_INT8_FP32
    case = case_for(kind, 3, 256, 128, 7, 7, 0.8, paired, ACTS[act], seed=78)
    if act == "none":
        case.bias = None
    got = run_hip(case, capi.ALGO_IMAGE_MFMA, force_semi=paired)
    want = run_oracle(case, oracle_pack(case, force_semi=paired))
    assert_same(case, got, want, "small map %s" % act)


def test_small_map_mfma_extremes_and_surroundings():
    """Largest magnitudes (accumulators of 1024 x 127 x 127), an empty output
    row, and the bytes around the output tensor stay untouched (rows of 49
    outputs are stored as dwords and single bytes at odd addresses)."""
    import torch

    announce("small map extremes")
    case = case_for(capi.KIND_INT8_ACC32, 3, 1024, 128, 7, 7, 0.5, False, AP(), seed=11)
    case.dense[7] = 0
    case.dense[64:66] = 127
    case.x[1] = -127
    got = run_hip(case, capi.ALGO_IMAGE_MFMA)
    ref = np.einsum("mk,bkp->bmp", case.dense.astype(np.int64), case.x.reshape(3, 1024, -1).astype(np.int64)).reshape(got.shape)
    assert np.array_equal(got.astype(np.int64), ref)
    assert np.all(got[:, 7] == 0)
    case8 = case_for(capi.KIND_INT8_INT8, 3, 512, 128, 7, 7, 0.9, False, ACTS["relu"], seed=12)
    kernel, _ = make_kernel(case8, capi.ALGO_IMAGE_MFMA)
    numel = 3 * 128 * 49
    guard = 64
    buf = torch.full((numel + 2 * guard,), 77, dtype=torch.int8, device="cuda")
    x = torch.from_numpy(case8.x).cuda()
    L = capi.lib()
    import ctypes as C

    capi.check(L.pl_sparse_conv_run(kernel._handle, x.data_ptr(), buf.data_ptr() + guard, 3, 49, C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    host = buf.cpu().numpy()
    assert (host[:guard] == 77).all() and (host[guard + numel:] == 77).all()
    assert np.array_equal(host[guard:guard + numel].reshape(3, 128, 7, 7), run_oracle(case8, oracle_pack(case8)))


@pytest.mark.parametrize("act", sorted(ACTS))
@pytest.mark.parametrize("out_int8", [False, True], ids=["fp32out", "int8out"])
@pytest.mark.parametrize("paired", [False, True], ids=["unstructured", "semi"])
def test_image_mfma_activations_and_structures(paired, out_int8, act):
    announce("image acts", paired, out_int8, act)
    kind = capi.KIND_INT8_INT8 if out_int8 else capi.KIND_INT8_FP32
    case = case_for(kind, 2, 128, 128, 14, 14, 0.8, paired, ACTS[act], seed=77)
    want = run_oracle(case, oracle_pack(case, force_semi=paired))
    for name, which in sorted(IMAGE_KERNELS.items()):
        got = run_hip(case, capi.ALGO_IMAGE_MFMA, force_semi=paired, tuning=capi.tuning(image_kernel=which))
        assert_same(case, got, want, "image %s %s" % (name, act))


@pytest.mark.parametrize("image_kernel", ["transpose", "rows"])
def test_image_mfma_shifted_window_kernels_extremes_and_surroundings(image_kernel):
    """Largest magnitudes (accumulators of 512 x 127 x 127 of either sign), an
    empty output row, channels of one parity only, and the bytes around the
    output tensor stay untouched (the windows of a row class reach in front of
    and behind the row; those lanes must not store)."""
    import ctypes as C

    import torch

    announce("image extremes", image_kernel)
    tr = capi.tuning(image_kernel=IMAGE_KERNELS[image_kernel])
    case = case_for(capi.KIND_INT8_ACC32, 3, 512, 128, 14, 14, 0.5, False, AP(), seed=21)
    case.dense[7] = 0
    case.dense[64:66] = 127
    case.dense[66:68] = -127
    case.dense[80, 0::2] = 0   # odd channels only
    case.dense[81, 1::2] = 0   # even channels only
    case.x[1] = -127
    got = run_hip(case, capi.ALGO_IMAGE_MFMA, tuning=tr)
    ref = np.einsum("mk,bkp->bmp", case.dense.astype(np.int64), case.x.reshape(3, 512, -1).astype(np.int64)).reshape(got.shape)
    assert np.array_equal(got.astype(np.int64), ref)
    assert np.all(got[:, 7] == 0)
    for kind, dt in ((capi.KIND_INT8_FP32, torch.float32), (capi.KIND_INT8_INT8, torch.int8)):
        c2 = case_for(kind, 3, 256, 256, 10, 10, 0.9, False, ACTS["relu"], seed=12)
        kernel, _ = make_kernel(c2, capi.ALGO_IMAGE_MFMA, tuning=tr)
        numel = 3 * 256 * 100
        guard = 64
        fill = 77
        buf = torch.full((numel + 2 * guard,), fill, dtype=dt, device="cuda")
        x = torch.from_numpy(c2.x).cuda()
        esz = buf.element_size()
        capi.check(capi.lib().pl_sparse_conv_run(kernel._handle, x.data_ptr(), buf.data_ptr() + guard * esz, 3, 100, C.c_void_p(torch.cuda.current_stream().cuda_stream)))
        torch.cuda.synchronize()
        host = buf.cpu().numpy()
        assert (host[:guard] == fill).all() and (host[guard + numel:] == fill).all()
        assert np.array_equal(host[guard:guard + numel].reshape(3, 256, 10, 10), run_oracle(c2, oracle_pack(c2)))


def test_image_mfma_agrees_with_the_other_algorithms_and_no_bias():
    announce("image vs others")
    case = case_for(capi.KIND_INT8_FP32, 4, 256, 256, 14, 14, 0.9, False, ACTS["relu"], seed=5)
    case.bias = None
    a = run_hip(case, capi.ALGO_IMAGE_MFMA)
    b = run_hip(case, capi.ALGO_BLOCK_MFMA)
    c = run_hip(case, capi.ALGO_ROW_WALK)
    assert np.array_equal(a, b) and np.array_equal(a, c)
    assert_same(case, a, run_oracle(case, oracle_pack(case)), "no bias")


def test_image_mfma_empty_and_dense_rows():
    announce("image extremes")
    case = case_for(capi.KIND_INT8_ACC32, 2, 128, 128, 6, 6, 0.5, False, AP(), seed=9)
    case.dense[5] = 0          # an output row without nonzeros
    case.dense[64:68] = 127    # fully dense rows of the largest magnitude
    case.x[0] = -127
    got = run_hip(case, capi.ALGO_IMAGE_MFMA)
    ref = np.einsum("mk,bkp->bmp", case.dense.astype(np.int64), case.x.reshape(2, 128, -1).astype(np.int64)).reshape(got.shape)
    assert np.array_equal(got.astype(np.int64), ref)
    assert np.all(got[:, 5] == 0)


def test_auto_picks_the_image_kernel_only_where_it_applies():
    announce("image auto")
    L = capi.lib()
    case = case_for(capi.KIND_INT8_FP32, 64, 512, 512, 14, 14, 0.85, False, ACTS["leaky"], seed=0)
    kernel, _ = make_kernel(case, capi.ALGO_AUTO)
    assert L.pl_sparse_conv_algo_for(kernel._handle, 64, 196) == capi.ALGO_IMAGE_MFMA
    assert L.pl_sparse_conv_algo_for(kernel._handle, 2, 196) == capi.ALGO_IMAGE_MFMA      # from two images on
    assert L.pl_sparse_conv_algo_for(kernel._handle, 1, 196) == capi.ALGO_IMAGE_MFMA      # and for a single one
    assert L.pl_sparse_conv_algo_for(kernel._handle, 64, 49) == capi.ALGO_IMAGE_MFMA      # 7x7 maps: pairs of images
    assert L.pl_sparse_conv_algo_for(kernel._handle, 1, 49) == capi.ALGO_IMAGE_MFMA       # at any batch
    assert L.pl_sparse_conv_algo_for(kernel._handle, 64, 50) == capi.ALGO_BLOCK_MFMA      # not a multiple of 4
    assert L.pl_sparse_conv_algo_for(kernel._handle, 4, 50) == capi.ALGO_ROW_WALK         # 200 positions
    assert L.pl_sparse_conv_algo_for(kernel._handle, 64, 28 * 28) == capi.ALGO_BLOCK_MFMA  # does not fit LDS
    # tuning.image_min_items asks for more (image, 128-row group) work items before the image kernel is taken
    picky, _ = make_kernel(case, capi.ALGO_AUTO, tuning=capi.tuning(image_min_items=128))
    assert L.pl_sparse_conv_algo_for(picky._handle, 64, 196) == capi.ALGO_IMAGE_MFMA
    assert L.pl_sparse_conv_algo_for(picky._handle, 2, 196) == capi.ALGO_BLOCK_MFMA
    assert L.pl_sparse_conv_algo_for(picky._handle, 1, 196) == capi.ALGO_ROW_WALK         # 196 positions in all
    assert L.pl_sparse_conv_algo_for(picky._handle, 32, 49) == capi.ALGO_BLOCK_MFMA
    # the same handle serves all of them
    import torch

    for batch, h, w in ((2, 14, 14), (1, 14, 14), (3, 7, 7), (1, 7, 7)):
        sub = copy.copy(case)  # same weights, another input size (the oracle's offsets are baked per H*W)
        sub.x = np.ascontiguousarray(case.x[:batch, :, :h, :w])
        got = kernel.Run(torch.from_numpy(sub.x).cuda()).cpu().numpy()
        assert np.array_equal(got, run_oracle(sub))
    # explicit requests outside the kernel's shapes are refused, not rerouted
    odd = case_for(capi.KIND_INT8_FP32, 1, 96, 128, 4, 4, 0.5, False, AP(), seed=1)
    with pytest.raises(capi.SparseConvError) as e:
        make_kernel(odd, capi.ALGO_IMAGE_MFMA)
    assert e.value.code == capi.PL_ERR_UNSUPPORTED
    k2, _ = make_kernel(case_for(capi.KIND_INT8_FP32, 1, 128, 128, 7, 7, 0.5, False, AP(), seed=1), capi.ALGO_IMAGE_MFMA)
    with pytest.raises(capi.SparseConvError) as e:
        k2.Run(torch.zeros((1, 128, 7, 7), dtype=torch.int8, device="cuda"))
    assert e.value.code == capi.PL_ERR_UNSUPPORTED


@pytest.mark.parametrize("kind", ["acc32", "fp32out", "int8out"])
def test_mixed_empty_sparse_and_dense_blocks_all_algorithms(kind):
    """A weight matrix whose 32x32 blocks are empty, 5 % filled or fully dense
    in equal parts (plus one all-zero row block and one all-zero k-step):
    every int8 algorithm against the oracle, and against each other."""
    announce("mixed blocks", kind)
    k = KINDS[kind]
    case = case_for(k, 3, 256, 256, 14, 14, 0.0, False, ACTS["none" if kind == "acc32" else "relu6"], seed=21)
    rng = np.random.RandomState(4)
    kinds = rng.randint(0, 3, size=(8, 8))  # 0 empty, 1 sparse, 2 dense
    kinds[3, :] = 0  # an empty row block
    kinds[:, 5] = 0  # a channel block no row uses
    mask = np.zeros((256, 256), dtype=bool)
    for bi in range(8):
        for bj in range(8):
            blk = {0: np.zeros((32, 32), bool), 1: rng.random_sample((32, 32)) < 0.05, 2: np.ones((32, 32), bool)}[int(kinds[bi, bj])]
            mask[32 * bi:32 * bi + 32, 32 * bj:32 * bj + 32] = blk
    case.dense = (case.dense * mask).astype(np.int8)
    want = run_oracle(case, oracle_pack(case))
    results = {}
    for name, algo in (("walk", capi.ALGO_ROW_WALK), ("block", capi.ALGO_BLOCK_MFMA), ("image", capi.ALGO_IMAGE_MFMA), ("auto", capi.ALGO_AUTO)):
        results[name] = run_hip(case, algo)
        assert_same(case, results[name], want, "mixed blocks %s %s" % (kind, name))
    kernel, _ = make_kernel(case, capi.ALGO_BLOCK_MFMA)
    info = kernel.info()
    assert info["mfma_blocks"] == int(np.count_nonzero([[mask[32 * i:32 * i + 32, 32 * j:32 * j + 32].any() for j in range(8)] for i in range(8)])) < info["mfma_blocks_total"] == 64


# Larger maps of a multiple of 196 positions, taken in slabs of 196 by the kernel with one row tile per wavefront:
# (batch, ic, oc, h, w); 28 x 28 = 4 slabs, 56 x 56 = 16, 14 x 42 = 3, 112 x 7 = 4 (rows of any shape: only H*W counts)
SLAB_SHAPES = [(2, 128, 256, 28, 28), (3, 256, 256, 28, 28), (1, 128, 128, 56, 56), (2, 512, 128, 14, 42), (5, 256, 384, 112, 7)]


@pytest.mark.parametrize("kind", sorted(KINDS))
@pytest.mark.parametrize("shape", SLAB_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_image_rows_slabs_bit_exact(shape, kind):
    announce("image slabs", shape, kind)
    batch, ic, oc, h, w = shape
    k = KINDS[kind]
    for act, paired in ((("none", False),) if kind == "acc32" else (("leaky", False), ("hswish", True), ("relu6", False))):
        case = case_for(k, batch, ic, oc, h, w, 0.85, paired, ACTS[act], seed=ic + 3 * oc + h * w)
        want = run_oracle(case, oracle_pack(case))
        got = run_hip(case, capi.ALGO_IMAGE_MFMA)
        assert_same(case, got, want, "image slabs %s %s %s" % (kind, act, shape))
        # the automatic choice takes the slabs for these few work items and gives the same bits
        kernel, _ = make_kernel(case, capi.ALGO_AUTO)
        assert capi.lib().pl_sparse_conv_algo_for(kernel._handle, batch, h * w) == capi.ALGO_IMAGE_MFMA
        assert np.array_equal(run_hip(case, kernel=kernel), got)
        # and the block kernel agrees
        assert np.array_equal(run_hip(case, capi.ALGO_BLOCK_MFMA), got)


def test_image_rows_slabs_rule_and_surroundings():
    """Slabs are taken while batch * slabs * oc / 128 is at most half the CU count; the kernel writes nothing
    outside its output and reads nothing it must not (the tensor sits inside a larger buffer)."""
    import torch

    L = capi.lib()
    case = case_for(capi.KIND_INT8_INT8, 4, 128, 256, 28, 28, 0.85, False, ACTS["relu"], seed=5)
    kernel, _ = make_kernel(case, capi.ALGO_AUTO)
    assert L.pl_sparse_conv_algo_for(kernel._handle, 16, 784) == capi.ALGO_IMAGE_MFMA   # 16 * 4 * 2 = 128 work items
    assert L.pl_sparse_conv_algo_for(kernel._handle, 17, 784) == capi.ALGO_BLOCK_MFMA
    assert L.pl_sparse_conv_algo_for(kernel._handle, 64, 784) == capi.ALGO_BLOCK_MFMA
    assert L.pl_sparse_conv_algo_for(kernel._handle, 4, 3136) == capi.ALGO_IMAGE_MFMA   # 4 * 16 * 2 = 128
    assert L.pl_sparse_conv_algo_for(kernel._handle, 5, 3136) == capi.ALGO_BLOCK_MFMA
    assert L.pl_sparse_conv_algo_for(kernel._handle, 1, 4 * 197) == capi.ALGO_BLOCK_MFMA  # not a multiple of 196
    regroup, _ = make_kernel(case, capi.ALGO_AUTO, tuning=REGROUP)                      # the other image kernels take no slabs
    assert L.pl_sparse_conv_algo_for(regroup._handle, 4, 784) == capi.ALGO_BLOCK_MFMA
    guard = 4096
    x = torch.from_numpy(case.x).cuda()
    xin = torch.randint(-127, 128, (x.numel() + 2 * guard,), dtype=torch.int8, device="cuda")
    xin[guard:guard + x.numel()] = x.reshape(-1)
    numel = 4 * 256 * 784
    buf = torch.full((numel + 2 * guard,), 77, dtype=torch.int8, device="cuda")
    kernel.Run(xin[guard:guard + x.numel()].view(x.shape), buf[guard:guard + numel].view(4, 256, 28, 28))
    torch.cuda.synchronize()
    host = buf.cpu().numpy()
    assert (host[:guard] == 77).all() and (host[guard + numel:] == 77).all()
    assert np.array_equal(host[guard:guard + numel].reshape(4, 256, 28, 28), run_oracle(case))
    with pytest.raises(capi.SparseConvError) as e:  # asked for explicitly on a map that has no slabs of 196
        forced, _ = make_kernel(case, capi.ALGO_IMAGE_MFMA)
        forced.Run(torch.zeros((1, 128, 20, 20), dtype=torch.int8, device="cuda"))
    assert e.value.code == capi.PL_ERR_UNSUPPORTED
