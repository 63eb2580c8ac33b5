"""Seeded synthetic workloads of the sparse_conv2d benchmark configurations.

All draws come from numpy's MT19937 RandomState seeded per case, so a case
is the same on every machine.  Masks are Bernoulli per weight (unstructured)
or per (output-channel pair, input channel) block (semi-structured, both
weights of a kept block nonzero).
"""
import numpy as np

from . import capi
from .sparse_conv import ActivationParam


class Case(object):
    """One sparse 1x1 convolution problem (host arrays)."""

    def __init__(self, name, kind, x, dense, bias, act, weight_scale=None, input_scale=1.0, output_scale=1.0, paired=False):
        self.name = name
        self.kind = kind  # capi.KIND_*
        self.x = x
        self.dense = dense
        self.bias = bias
        self.act = act
        self.weight_scale = weight_scale
        self.input_scale = input_scale
        self.output_scale = output_scale
        self.paired = paired

    @property
    def batch(self):
        return self.x.shape[0]

    @property
    def im_size(self):
        return self.x.shape[2] * self.x.shape[3]

    @property
    def nnz(self):
        return int(np.count_nonzero(self.dense))

    def algorithmic_ops(self):
        """2 * nnz * batch * H * W (nonzero-counted operations)."""
        return 2.0 * self.nnz * self.batch * self.im_size

    def algorithmic_bytes(self, weights):
        """Input + output + compressed weights, each once."""
        oc, ic = self.dense.shape
        out_item = {capi.KIND_FP32: 4, capi.KIND_INT8_FP32: 4, capi.KIND_INT8_INT8: 1, capi.KIND_INT8_ACC32: 4, capi.KIND_FP16: 2}[self.kind]
        p = self.batch * self.im_size
        wbytes = weights.nonzero_weights.nbytes + weights.diffs.nbytes + 12 * oc
        return float(self.x.nbytes + p * oc * out_item + wbytes)


def _mask(rng, oc, ic, sparsity, paired):
    if paired:
        half = rng.random_sample(((oc + 1) // 2, ic)) >= sparsity
        return np.repeat(half, 2, axis=0)[:oc]
    return rng.random_sample((oc, ic)) >= sparsity


def _int8_nonzero(rng, shape):
    v = rng.randint(1, 128, size=shape).astype(np.int16)
    sign = rng.randint(0, 2, size=shape).astype(np.int16) * 2 - 1
    return (v * sign).astype(np.int8)


def make_fp32(name, batch, ic, oc, h, w, sparsity, paired, act, seed=0, w_sigma=0.1):
    rng = np.random.RandomState(seed)
    x = rng.uniform(-1.0, 1.0, size=(batch, ic, h, w)).astype(np.float32)
    vals = (rng.standard_normal((oc, ic)) * w_sigma).astype(np.float32)
    vals[vals == 0] = np.float32(w_sigma)
    dense = (vals * _mask(rng, oc, ic, sparsity, paired)).astype(np.float32)
    bias = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    return Case(name, capi.KIND_FP32, x, dense, bias, act, paired=paired)


def make_int8(name, batch, ic, oc, h, w, sparsity, paired, act, out_int8, seed=0, output_scale=1.0, input_scale=0.01):
    rng = np.random.RandomState(seed)
    x = rng.randint(-127, 128, size=(batch, ic, h, w)).astype(np.int8)
    dense = (_int8_nonzero(rng, (oc, ic)) * _mask(rng, oc, ic, sparsity, paired)).astype(np.int8)
    ws = rng.uniform(0.001, 0.02, size=oc).astype(np.float32)
    bias = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    kind = capi.KIND_INT8_INT8 if out_int8 else capi.KIND_INT8_FP32
    return Case(name, kind, x, dense, bias, act, weight_scale=ws, input_scale=input_scale, output_scale=output_scale, paired=paired)


DENSITY_SHAPES = {"metric": (64, 512, 512, 14), "wide": (16, 2048, 2048, 14)}


def config_density(shape, sparsity, blocked, seed=0):
    """int8 -> fp32 with leaky_relu at a chosen sparsity on one of
    DENSITY_SHAPES (batch, ic, oc, h = w): "metric" is the metric shape, "wide"
    a layer with sixteen times its dense work for the same input and output
    bytes.  blocked: zeros come as whole 32x32 blocks of the weight matrix (a
    Bernoulli mask over the grid of blocks, kept blocks fully dense) instead
    of single weights."""
    batch, ic, oc, hw = DENSITY_SHAPES[shape]
    c = make_int8("density_%s_%02d_%s" % (shape, round(sparsity * 100), "blocked" if blocked else "random"), batch, ic, oc, hw, hw, 0.0 if blocked else sparsity, False,
                  ActivationParam("leaky_relu", Leaky_relu_alpha=0.1), out_int8=False, seed=seed)
    if blocked:
        rng = np.random.RandomState(seed + 1000)
        keep = rng.random_sample((oc // 32, ic // 32)) >= sparsity
        c.dense = (c.dense * np.kron(keep, np.ones((32, 32), dtype=bool))).astype(np.int8)
    return c


def config1(batch=1):
    """fp32 unstructured, 1x96x56x56 -> 192, 80 % zeros, relu."""
    return make_fp32("c1_fp32_unstructured", batch, 96, 192, 56, 56, 0.80, False, ActivationParam("relu"), seed=0, w_sigma=0.1)


def config2(batch=32):
    """fp32 semi-structured, 32x256x28x28 -> 512, 90 % zeros, relu6."""
    return make_fp32("c2_fp32_semi", batch, 256, 512, 28, 28, 0.90, True, ActivationParam("relu6", Relu_clipped_coef=6.0), seed=0, w_sigma=0.05)


def config3(batch=64):
    """The metric configuration: int8 -> fp32, 64x512x14x14 -> 512, 85 %
    unstructured zeros, per-channel scales, leaky_relu(0.1)."""
    return make_int8("c3_int8_fp32_unstructured", batch, 512, 512, 14, 14, 0.85, False, ActivationParam("leaky_relu", Leaky_relu_alpha=0.1), out_int8=False, seed=0)


def config4(batch=128):
    """int8 -> int8 semi-structured, 128x128x56x56 -> 256, 75 % zeros,
    output scale 0.05, hard_swish."""
    return make_int8("c4_int8_int8_semi", batch, 128, 256, 56, 56, 0.75, True, ActivationParam("hard_swish"), out_int8=True, seed=0, output_scale=0.05)


MOBILENET_V1_POINTWISE = [
    (32, 64, 112), (64, 128, 56), (128, 128, 56), (128, 256, 28), (256, 256, 28), (256, 512, 14),
    (512, 512, 14), (512, 512, 14), (512, 512, 14), (512, 512, 14), (512, 512, 14), (512, 1024, 7), (1024, 1024, 7),
]


def config5_layer(index, batch=64, sparsity=0.90):
    """Layer `index` (0..12) of the MobileNetV1-1.0 pointwise stack, int8 ->
    int8 with relu.  The output scale is chosen from the weights so that the
    requantised output of uniform int8 inputs is not saturated:
    output_scale = 3 * sigma(acc * scale) / 127 with
    sigma(acc) = sqrt(nnz_per_row) * E|w| * E|x| estimated as
    sqrt(ic * (1 - sparsity)) * 73.3 * 73.3."""
    ic, oc, hw = MOBILENET_V1_POINTWISE[index]
    c = make_int8("c5_L%02d_%dx%d_%d" % (index + 1, ic, oc, hw), batch, ic, oc, hw, hw, sparsity, False, ActivationParam("relu"), out_int8=True, seed=100 + index)
    sigma_acc = np.sqrt(ic * (1.0 - sparsity)) * 73.3 * 73.3
    c.output_scale = float(3.0 * sigma_acc * float(np.mean(c.weight_scale)) * c.input_scale / 127.0)
    return c


# stride of the depthwise 3x3 layer in front of each pointwise layer above
MOBILENET_V1_DEPTHWISE_STRIDES = [1, 2, 1, 2, 1, 2, 1, 1, 1, 1, 1, 2, 1]


class DepthwiseCase(object):
    """One int8 depthwise 3x3 layer (padding 1, relu): filter [C, 1, 3, 3],
    per-channel weight scales, bias, input / output scales."""

    def __init__(self, name, channels, in_size, stride, filt, bias, weight_scale, input_scale, output_scale):
        self.name = name
        self.channels, self.in_size, self.stride = channels, in_size, stride
        self.out_size = (in_size + 2 - 3) // stride + 1
        self.filter = filt
        self.bias = bias
        self.weight_scale = weight_scale
        self.input_scale = input_scale
        self.output_scale = output_scale
        self.act = ActivationParam("relu")

    def algorithmic_bytes(self, batch):
        """Input + output + filters, scales and biases, each once."""
        c = self.channels
        return float(batch * c * (self.in_size ** 2 + self.out_size ** 2) + 9 * c + 8 * c)


def config5_depthwise_layer(index, sparsity=0.0):
    """The depthwise layer in front of pointwise layer `index` (0..12) of
    MobileNetV1-1.0: channels = that layer's input channels, int8 -> int8,
    relu.  Filters U{-127..127}, weight scales U[0.001, 0.02], input scale
    0.01; the output scale keeps the requantised output of typical inputs
    below saturation: 3 * sigma(acc * scale) / 127 with sigma(acc) =
    sqrt(9) * 73.3 * 40 (mean |w| of the uniform filters times a mean |x| of 40
    for inputs that went through a relu)."""
    ic, _, hw = MOBILENET_V1_POINTWISE[index]
    stride = MOBILENET_V1_DEPTHWISE_STRIDES[index]
    rng = np.random.RandomState(300 + index)
    filt = rng.randint(-127, 128, size=(ic, 1, 3, 3)).astype(np.int8)
    ws = rng.uniform(0.001, 0.02, size=ic).astype(np.float32)
    bias = (rng.standard_normal(ic) * 0.1).astype(np.float32)
    input_scale = 0.01
    output_scale = float(3.0 * 3.0 * 73.3 * 40.0 * float(np.mean(ws)) * input_scale / 127.0)
    return DepthwiseCase("c5_dw%02d_%d_%d_s%d" % (index + 1, ic, hw * stride, stride), ic, hw * stride, stride, filt, bias, ws, input_scale, output_scale)


CONFIGS = {"c1": config1, "c2": config2, "c3": config3, "c4": config4}
