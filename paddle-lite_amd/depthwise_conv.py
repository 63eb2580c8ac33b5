"""Host mirror of the reference's int8 depthwise 3x3 convolution kernel class
(lite/kernels/arm/conv_depthwise.{h,cc}: DepthwiseConv<kInt8, kFloat> and
DepthwiseConv<kInt8, kInt8>, picked by ConvCompute::PrepareForRun for
groups == input channels == output channels, lite/kernels/arm/conv_compute.cc)
with the HIP library behind it.  It is the layer between two pointwise
convolutions of a MobileNet, which is why it sits beside sparse_conv2d here.
"""
import ctypes as C

import numpy as np

from . import capi
from .sparse_conv import ActivationParam


class ConvParam(object):
    """The fields of operators::ConvParam the depthwise int8 kernels read
    (lite/operators/op_params.h ConvParam): filter [C, 1, 3, 3] int8, bias [C]
    fp32 or None, strides, paddings (up, down, left, right), dilations, groups,
    activation_param, input / weight / output scales."""

    def __init__(self, filter, bias=None, strides=(1, 1), paddings=(1, 1, 1, 1), dilations=(1, 1), groups=None, activation_param=None, input_scale=1.0,
                 weight_scale=(1.0,), output_scale=1.0):
        self.filter = np.ascontiguousarray(filter, dtype=np.int8)
        if self.filter.ndim != 4 or self.filter.shape[1] != 1:
            raise ValueError("a depthwise filter has the shape [channels, 1, kh, kw]")
        self.bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
        self.strides = [int(v) for v in strides]
        paddings = [int(v) for v in paddings]
        if len(paddings) == 2:  # ConvOp pads the two-element form to four (conv_op.h)
            paddings = [paddings[0], paddings[0], paddings[1], paddings[1]]
        self.paddings = paddings
        self.dilations = [int(v) for v in dilations]
        self.groups = int(self.filter.shape[0] if groups is None else groups)
        self.activation_param = activation_param.copy() if activation_param else ActivationParam()
        self.enable_int8 = True
        self.input_scale = float(input_scale)
        self.weight_scale = [float(v) for v in np.atleast_1d(weight_scale)]
        self.output_scale = float(output_scale)


class DepthwiseConv(object):
    """DepthwiseConv<kInt8, out_precision>.  PrepareForRun merges the scales
    as conv_depthwise.cc:158-200 (fp32 output: weight_scale * input_scale) and
    :257-322 (int8 output: / output_scale, bias / output_scale, relu6
    coefficient and hard_swish offset and threshold / output_scale)."""

    def __init__(self, param, out_precision="int8", item_rows=0, item_cols=0, share_lanes=capi.TUNE_RULE, row_items=capi.TUNE_RULE):
        # the four tuning arguments are the fields of pl_dwconv_desc of the same names (0 = by rule)
        self.tuning = (int(item_rows), int(item_cols), int(share_lanes), int(row_items))
        out = str(np.dtype(out_precision))
        if out not in ("int8", "float32"):
            raise ValueError("no depthwise kernel with %s output" % out)
        self.kind = capi.KIND_INT8_INT8 if out == "int8" else capi.KIND_INT8_FP32
        self.param = param
        self._handle = None
        self._first_epoch = True
        self.w_scale_ = None
        self.bias_ = None
        self.merged_act = None

    def PrepareForRun(self):
        p = self.param
        oc, _, kh, kw = p.filter.shape
        if kh != 3 or kw != 3:
            raise NotImplementedError("this type dw conv not impl")  # conv_depthwise.cc:319
        if p.groups != oc:
            raise ValueError("depthwise: groups must equal the channel count")
        if p.dilations != [1, 1]:
            raise NotImplementedError("depthwise 3x3: dilation 1 only")
        if p.strides[0] != p.strides[1] or p.strides[0] not in (1, 2):
            raise NotImplementedError("depthwise 3x3: stride 1 or 2 in both directions")
        if len(set(p.paddings)) != 1 or p.paddings[0] not in (0, 1):
            raise NotImplementedError("depthwise 3x3: padding 0 or 1 on all sides")
        ws = list(p.weight_scale)
        if len(ws) != 1 and len(ws) != oc:
            raise ValueError("weights scale size must = filter size or = 1")
        if len(ws) == 1:
            ws = ws * oc
        ws = np.asarray(ws, dtype=np.float32)
        isc, osc = np.float32(p.input_scale), np.float32(p.output_scale)
        act = p.activation_param.copy()
        bias = p.bias
        if self.kind == capi.KIND_INT8_INT8:
            scale = ws * isc / osc
            if bias is not None:
                bias = (bias / osc).astype(np.float32)
            f32 = lambda v: float(np.float32(np.float32(v) / osc))  # noqa: E731
            if act.active_type == capi.ACT_RELU6:
                act.Relu_clipped_coef = f32(act.Relu_clipped_coef)
            if act.active_type == capi.ACT_HARD_SWISH:
                act.hard_swish_offset = f32(act.hard_swish_offset)
                act.hard_swish_threshold = f32(act.hard_swish_threshold)
        else:
            scale = ws * isc
        self.w_scale_ = np.ascontiguousarray(scale, dtype=np.float32)
        self.bias_ = bias
        self.merged_act = act
        a = capi.Activation()
        a.type = act.active_type if act.has_active else capi.ACT_NONE
        a.relu6_coef = act.Relu_clipped_coef
        a.leaky_alpha = act.Leaky_relu_alpha
        a.hs_scale = act.hard_swish_scale  # multiplies (conv_block_utils.h cvt_kernel)
        a.hs_offset = act.hard_swish_offset
        a.hs_threshold = act.hard_swish_threshold
        self._capi_act = a
        d = capi.DwConvDesc()
        d.struct_size = C.sizeof(capi.DwConvDesc)
        d.kind = self.kind
        d.channels = oc
        d.stride = p.strides[0]
        d.pad = p.paddings[0]
        d.weights = p.filter.ctypes.data
        d.scale = self.w_scale_.ctypes.data
        d.bias = bias.ctypes.data if bias is not None else None
        d.act = a
        d.item_rows, d.item_cols, d.share_lanes, d.row_items = self.tuning
        h = C.c_void_p()
        capi.check(capi.lib().pl_dwconv3x3_prepare(C.byref(d), C.byref(h)))
        self._release()
        self._handle = h
        self._first_epoch = False

    def out_shape(self, x_shape):
        n, c, h, w = x_shape
        s, pad = self.param.strides[0], self.param.paddings[0]
        return (n, c, (h + 2 * pad - 3) // s + 1, (w + 2 * pad - 3) // s + 1)

    def Launch(self, x, out=None, stream=None):
        if self._first_epoch:
            self.PrepareForRun()
        return self.Run(x, out, stream)

    def Run(self, x, out=None, stream=None):
        import torch

        if self._handle is None:
            raise RuntimeError("PrepareForRun has not been called")
        c = self.param.filter.shape[0]
        if not x.is_cuda or not x.is_contiguous() or x.dtype != torch.int8 or x.dim() != 4 or x.shape[1] != c:
            raise ValueError("x must be a contiguous int8 NCHW device tensor with %d channels" % c)
        shape = self.out_shape(tuple(x.shape))
        odt = torch.int8 if self.kind == capi.KIND_INT8_INT8 else torch.float32
        if out is None:
            out = torch.empty(shape, dtype=odt, device=x.device)
        elif tuple(out.shape) != shape or out.dtype != odt or not out.is_contiguous() or out.device != x.device:
            raise ValueError("out must be a contiguous %s tensor of shape %s on the device of x" % (odt, shape))
        s = torch.cuda.current_stream(x.device).cuda_stream if stream is None else stream
        with torch.cuda.device(x.device):
            capi.check(capi.lib().pl_dwconv3x3_run(self._handle, C.c_void_p(x.data_ptr()), C.c_void_p(out.data_ptr()), x.shape[0], x.shape[2], x.shape[3], C.c_void_p(s)))
        return out

    def _release(self):
        if self._handle is not None:
            capi.lib().pl_dwconv3x3_destroy(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self._release()
        except Exception:
            pass


def conv_dw_fits(conv, dw, h, w):
    """True when `conv` (a prepared SparseConvKernel, int8 -> int8) followed by `dw` (a prepared DepthwiseConv,
    int8 -> int8) can run as one launch on h x w maps (pl_sparse_conv_dwconv3x3_fits)."""
    if conv._handle is None or dw._handle is None:
        raise RuntimeError("PrepareForRun has not been called")
    return bool(capi.lib().pl_sparse_conv_dwconv3x3_fits(conv._handle, dw._handle, int(h), int(w)))


def run_conv_dw(conv, dw, x, out=None, stream=None):
    """sparse_conv2d followed by depthwise_conv2d in one launch (pl_sparse_conv_dwconv3x3_run): the result of
    dw.Run(conv.Run(x)), bit for bit, without the tensor between them.  Raises where conv_dw_fits is False."""
    import torch

    if conv._handle is None or dw._handle is None:
        raise RuntimeError("PrepareForRun has not been called")
    if not x.is_cuda or not x.is_contiguous() or x.dtype != torch.int8 or x.dim() != 4 or x.shape[1] != conv.param.weights.ic:
        raise ValueError("x must be a contiguous int8 NCHW device tensor with %d channels" % conv.param.weights.ic)
    n, _, h, w = x.shape
    shape = dw.out_shape((n, conv.param.weights.oc, h, w))
    if out is None:
        out = torch.empty(shape, dtype=torch.int8, device=x.device)
    elif tuple(out.shape) != shape or out.dtype != torch.int8 or not out.is_contiguous() or out.device != x.device:
        raise ValueError("out must be a contiguous int8 tensor of shape %s on the device of x" % (shape,))
    s = torch.cuda.current_stream(x.device).cuda_stream if stream is None else stream
    with torch.cuda.device(x.device):
        capi.check(capi.lib().pl_sparse_conv_dwconv3x3_run(conv._handle, dw._handle, C.c_void_p(x.data_ptr()), C.c_void_p(out.data_ptr()), n, h, w, C.c_void_p(s)))
    return out
