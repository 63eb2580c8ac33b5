"""int8 depthwise 3x3 convolution on the GPU, through the C ABI (the Python
kernel class calls pl_dwconv3x3_*), against the oracle: int8 and fp32 outputs
bit for bit (the kernel's fmaf order is the oracle's).  Shapes follow the
reference's conv_int8_compute_test.cc sweep in spirit (strides 1 / 2,
paddings 0 / 1, with and without bias, relu / relu6 / leaky_relu, odd sizes)
plus the MobileNetV1 depthwise shapes."""
import importlib

import numpy as np
import pytest

from helpers import capi
from oracle import oracle as O

pytestmark = pytest.mark.gpu
pla = importlib.import_module("paddle-lite_amd")


def oracle_act(ap):
    a = O.Act()
    a.type = ap.active_type if ap.has_active else 0
    a.relu6_coef = ap.Relu_clipped_coef
    a.leaky_alpha = ap.Leaky_relu_alpha
    a.hs_scale = ap.hard_swish_scale
    a.hs_offset = ap.hard_swish_offset
    a.hs_threshold = ap.hard_swish_threshold
    return a


def run_case(n, c, h, w, stride, pad, out, act, bias, seed, guard=64, **tuning):
    import torch

    rng = np.random.RandomState(seed)
    x = rng.randint(-127, 128, size=(n, c, h, w)).astype(np.int8)
    filt = rng.randint(-127, 128, size=(c, 1, 3, 3)).astype(np.int8)
    ws = rng.uniform(0.002, 0.02, size=c).astype(np.float32)
    b = (rng.standard_normal(c) * 0.5).astype(np.float32) if bias else None
    param = pla.ConvParam(filt, b, strides=(stride, stride), paddings=(pad, pad, pad, pad), activation_param=act, input_scale=0.02, weight_scale=ws,
                          output_scale=0.11 if out == "int8" else 1.0)
    k = pla.DepthwiseConv(param, out_precision="int8" if out == "int8" else "float32", **tuning)
    k.PrepareForRun()
    # the tensor sits inside a larger buffer whose surroundings must stay
    # untouched (output) and must not matter (input)
    xin = torch.from_numpy(rng.randint(-127, 128, size=x.size + 2 * guard).astype(np.int8)).cuda()
    xin[guard:guard + x.size] = torch.from_numpy(x.reshape(-1)).cuda()
    shape = k.out_shape(x.shape)
    numel = int(np.prod(shape))
    odt = torch.int8 if out == "int8" else torch.float32
    buf = torch.full((numel + 2 * guard,), 77, dtype=odt, device="cuda")
    k.Run(xin[guard:guard + x.size].view(n, c, h, w), buf[guard:guard + numel].view(shape))
    torch.cuda.synchronize()
    host = buf.cpu().numpy()
    assert (host[:guard] == 77).all() and (host[guard + numel:] == 77).all()
    got = host[guard:guard + numel].reshape(shape)
    want = O.dwconv3x3_int8(x, filt[:, 0], k.w_scale_, k.bias_, oracle_act(k.merged_act), out=out, stride=stride, pad=pad)
    if out == "int8":
        assert np.array_equal(got, want)
    else:
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


ACTS = {
    "none": lambda: pla.ActivationParam(),
    "relu": lambda: pla.ActivationParam("relu"),
    "relu6": lambda: pla.ActivationParam("relu6", Relu_clipped_coef=6.0),
    "leaky": lambda: pla.ActivationParam("leaky_relu", Leaky_relu_alpha=0.12),
    "hswish": lambda: pla.ActivationParam("hard_swish", hard_swish_scale=1.0 / 6.0, hard_swish_offset=3.0, hard_swish_threshold=6.0),
}

SMALL = [(1, 1, 3, 3), (2, 3, 7, 7), (1, 5, 14, 14), (2, 2, 9, 6), (1, 2, 5, 12), (3, 4, 4, 4), (1, 3, 2, 2), (1, 2, 1, 5), (1, 2, 33, 17), (2, 8, 28, 28), (1, 300, 7, 7)]


@pytest.mark.parametrize("shape", SMALL)
@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("pad", [0, 1])
@pytest.mark.parametrize("out", ["int8", "fp32"])
def test_shapes(shape, stride, pad, out):
    n, c, h, w = shape
    if h + 2 * pad < 3 or w + 2 * pad < 3:
        pytest.skip("input smaller than the filter")
    run_case(n, c, h, w, stride, pad, out, ACTS["relu"](), True, seed=h * 131 + w * 7 + stride + 2 * pad)


@pytest.mark.parametrize("act", sorted(ACTS))
@pytest.mark.parametrize("out", ["int8", "fp32"])
@pytest.mark.parametrize("bias", [False, True])
def test_activations(act, out, bias):
    run_case(2, 6, 14, 14, 1, 1, out, ACTS[act](), bias, seed=len(act) * 17 + bias)
    run_case(2, 6, 15, 13, 2, 1, out, ACTS[act](), bias, seed=len(act) * 19 + bias)


# (channels, input size, stride) of the thirteen depthwise layers of MobileNetV1-1.0
MOBILENET_V1_DEPTHWISE = [(32, 112, 1), (64, 112, 2), (128, 56, 1), (128, 56, 2), (256, 28, 1), (256, 28, 2), (512, 14, 1), (512, 14, 2), (1024, 7, 1)]


@pytest.mark.parametrize("layer", MOBILENET_V1_DEPTHWISE)
def test_mobilenet_shapes(layer):
    c, size, stride = layer
    run_case(2, c, size, size, stride, 1, "int8", ACTS["relu"](), True, seed=c + size + stride)


# every item shape the launcher can pick (output rows x groups of four output
# columns per thread), forced through the tuning knobs the library reads when
# a layer is prepared, on planes that are ragged against each of them
ITEM_SHAPES = {1: [(2, 1), (4, 1), (1, 2), (2, 2), (4, 2), (1, 4), (2, 4)], 2: [(2, 1), (1, 2), (2, 2), (1, 4)]}


@pytest.mark.parametrize("stride,rows,cols", [(s, r, c) for s in (1, 2) for (r, c) in ITEM_SHAPES[s]])
@pytest.mark.parametrize("out", ["int8", "fp32"])
def test_item_shapes(stride, rows, cols, out):
    for i, (n, c, h, w) in enumerate([(2, 3, 7, 7), (1, 5, 14, 14), (2, 2, 33, 17), (1, 4, 30, 61), (2, 40, 28, 28), (1, 2, 3, 70)]):
        for pad in (0, 1):
            run_case(n, c, h, w, stride, pad, out, ACTS["relu6"](), True, seed=1000 * rows + 100 * cols + 10 * i + pad + stride, item_rows=rows, item_cols=cols)


# narrow planes (w + 2 * pad <= 16) take one whole output row per thread by
# default; both that kernel and the general one, on every width it covers
@pytest.mark.parametrize("row_items", [capi.TUNE_NEVER, capi.TUNE_ALWAYS], ids=["general", "row-items"])
@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("out", ["int8", "fp32"])
def test_narrow_planes(row_items, stride, out):
    for pad in (0, 1):
        for w in range(3 - 2 * pad if 3 - 2 * pad > 0 else 1, 17 - 2 * pad):
            h = 1 + (5 * w) % 9 if pad else 3 + (5 * w) % 7
            run_case(2, 3, h, w, stride, pad, out, ACTS["hswish"](), True, seed=100 * w + 10 * pad + stride, row_items=row_items)
    run_case(3, 70, 14, 14, stride, 1, out, ACTS["relu"](), False, seed=5 + stride, row_items=row_items)  # several workgroups, the first and the last at the tensor's ends
    run_case(5, 33, 7, 7, stride, 1, out, ACTS["relu6"](), True, seed=6 + stride, row_items=row_items)


@pytest.mark.parametrize("stride", [1, 2])
def test_large_planes(stride):
    # more than 2^16 items per plane, and a plane whose item count is odd
    run_case(1, 2, 1100, 900, stride, 1, "int8", ACTS["relu"](), True, seed=77 + stride)
    run_case(1, 1, 515, 1030, stride, 0, "fp32", ACTS["leaky"](), True, seed=78 + stride)


def test_bad_arguments_are_refused():
    import torch

    filt = np.ones((4, 1, 3, 3), dtype=np.int8)
    with pytest.raises(NotImplementedError):
        pla.DepthwiseConv(pla.ConvParam(filt, strides=(3, 3))).PrepareForRun()
    with pytest.raises(NotImplementedError):
        pla.DepthwiseConv(pla.ConvParam(filt, paddings=(2, 2, 2, 2))).PrepareForRun()
    with pytest.raises(NotImplementedError):
        pla.DepthwiseConv(pla.ConvParam(np.ones((4, 1, 5, 5), dtype=np.int8))).PrepareForRun()
    k = pla.DepthwiseConv(pla.ConvParam(filt, paddings=(0, 0, 0, 0)))
    k.PrepareForRun()
    with pytest.raises(ValueError):
        k.Run(torch.zeros((1, 3, 8, 8), dtype=torch.int8, device="cuda"))  # channel count
    with pytest.raises(capi.SparseConvError):
        k.Run(torch.zeros((1, 4, 2, 2), dtype=torch.int8, device="cuda"))  # smaller than the filter
