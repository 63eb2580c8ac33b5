"""Host-side mirror of the sparse_conv2d operator surface.

Names follow the reference: SparseConvParam / ActivationParam are the
parameter bags of lite/operators/op_params.h:331-400, SparseConvKernel plays
the role of SparseConvCompute<Ptype, OutType>
(lite/kernels/arm/sparse_conv_compute.cc:31-267) with the HIP library behind
it, detect_and_pack is the weight part of sparse_conv_detect_pass
(lite/core/optimizer/mir/sparse_conv_detect_pass.cc:606-860).
"""
import ctypes as C

import numpy as np

from . import capi

_ACT_NAMES = {"": capi.ACT_NONE, "relu": capi.ACT_RELU, "relu6": capi.ACT_RELU6, "leaky_relu": capi.ACT_LEAKY_RELU, "hard_swish": capi.ACT_HARD_SWISH}


class ActivationParam(object):
    """Fields and defaults of ActivationParam the sparse kernels read
    (reference: lite/operators/op_params.h:331-362)."""

    def __init__(self, active_type=capi.ACT_NONE, has_active=None, Leaky_relu_alpha=0.0, Relu_clipped_coef=6.0, hard_swish_threshold=6.0, hard_swish_scale=6.0, hard_swish_offset=3.0):
        if isinstance(active_type, str):
            if active_type not in _ACT_NAMES:
                # same outcome as the op: unknown fused activation is fatal
                # (reference: lite/operators/sparse_conv_op.h:138-142)
                raise ValueError("The fused conv only supports fuse with relu, leaky relu, hard_swish, while the given activation type is " + active_type)
            active_type = _ACT_NAMES[active_type]
        self.active_type = int(active_type)
        self.has_active = bool(active_type) if has_active is None else bool(has_active)
        self.Leaky_relu_alpha = float(Leaky_relu_alpha)
        self.Relu_clipped_coef = float(Relu_clipped_coef)
        self.hard_swish_threshold = float(hard_swish_threshold)
        self.hard_swish_scale = float(hard_swish_scale)
        self.hard_swish_offset = float(hard_swish_offset)

    def copy(self):
        return ActivationParam(self.active_type, self.has_active, self.Leaky_relu_alpha, self.Relu_clipped_coef, self.hard_swish_threshold, self.hard_swish_scale, self.hard_swish_offset)


class SparseWeights(object):
    """The three persistable tensors the detect pass creates plus the two
    attributes it sets (first_ic, flag_semi)."""

    def __init__(self, nonzero_weights, oc_nonzeros, diffs, first_ic, flag_semi, oc, ic, im_size):
        self.nonzero_weights = np.ascontiguousarray(nonzero_weights)
        self.oc_nonzeros = np.ascontiguousarray(oc_nonzeros, dtype=np.uint32)
        self.diffs = np.ascontiguousarray(diffs, dtype=np.int32)
        self.first_ic = int(first_ic)
        self.flag_semi = int(flag_semi)
        self.oc, self.ic, self.im_size = int(oc), int(ic), int(im_size)


def _dtype_code(w):
    if w.dtype == np.float32:
        return 0
    if w.dtype == np.int8:
        return 1
    raise TypeError("sparse conv weights are float32 or int8")


def detect_and_pack(dense, im_size, sparse_threshold=None, force_semi=None):
    """Weight side of SparseConvDetectPass::Apply: analyse a dense [oc, ic]
    1x1 filter, decide flag_semi, pack.  Returns None when the zero fraction
    is below `sparse_threshold` (the pass then leaves the conv2d alone,
    sparse_conv_detect_pass.cc:684-692)."""
    dense = np.ascontiguousarray(dense)
    if dense.ndim == 4:
        if dense.shape[2:] != (1, 1):
            return None  # the pass only rewrites 1x1 kernels (:639-645)
        dense = dense.reshape(dense.shape[0], dense.shape[1])
    oc, ic = dense.shape
    dt = _dtype_code(dense)
    L = capi.lib()
    cn, cc, cb, fs = C.c_int32(), C.c_int32(), C.c_int32(), C.c_int32()
    zeros = capi.check(L.pl_sparse_count_semi(dt, dense.ctypes.data, oc, ic, C.byref(cn), C.byref(cc), C.byref(cb), C.byref(fs)))
    semi = fs.value if force_semi is None else int(bool(force_semi))
    if semi and not fs.value:
        paired = (oc // 2) * 2
        nz = dense != 0
        blocks = int(np.count_nonzero(nz[0:paired:2] | nz[1:paired:2]))
        tail = int(np.count_nonzero(nz[paired:]))
        n_w, n_d = 2 * blocks + tail, blocks + tail
        zeros = oc * ic - n_w
    elif semi:
        n_w, n_d = cn.value, cb.value
    elif dt == 0:
        nb = C.c_int32()
        zeros = capi.check(L.pl_sparse_count_zeros(dt, dense.ctypes.data, oc, ic, C.byref(nb)))
        n_w = n_d = nb.value
    else:
        n_w = n_d = int(np.count_nonzero(dense))
        zeros = oc * ic - n_w
    if sparse_threshold is not None:
        if not 0.0 <= sparse_threshold <= 1.0:
            raise ValueError("sparse_threshold must be in [0, 1]")  # opt_base.cc:78-81
        if zeros / float(oc * ic) < sparse_threshold:
            return None
    nzw = np.zeros(max(n_w, 1), dtype=dense.dtype)[:n_w]
    ocn = np.zeros(oc, dtype=np.uint32)
    dif = np.zeros(max(n_d, 1), dtype=np.int32)[:n_d]
    first_ic = capi.check(L.pl_sparse_pack(dt, semi, dense.ctypes.data, oc, ic, int(im_size), nzw.ctypes.data, n_w, ocn.ctypes.data, dif.ctypes.data, n_d))
    return SparseWeights(nzw, ocn, dif, first_ic, semi, oc, ic, im_size)


class SparseConvParam(object):
    """reference: lite/operators/op_params.h:373-400 (same field names)."""

    def __init__(self, weights, bias=None, activation_param=None, enable_int8=False, input_scale=1.0, weight_scale=(), output_scale=1.0):
        self.nonzero_weights = weights.nonzero_weights
        self.oc_nonzeros = weights.oc_nonzeros
        self.diffs = weights.diffs
        self.first_ic = weights.first_ic
        self.flag_semi = weights.flag_semi
        self.weights = weights
        self.bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
        self.strides = [1, 1]
        self.paddings = [0, 0, 0, 0]
        self.groups = 1
        self.dilations = [1, 1]
        self.fuse_relu = False
        self.activation_param = activation_param.copy() if activation_param else ActivationParam()
        self.enable_int8 = bool(enable_int8)
        self.input_scale = float(input_scale)
        self.weight_scale = [float(v) for v in np.atleast_1d(weight_scale)]
        self.output_scale = float(output_scale)
        self.bit_length = 8


_KINDS = {("float32", "float32"): capi.KIND_FP32, ("int8", "float32"): capi.KIND_INT8_FP32, ("int8", "int8"): capi.KIND_INT8_INT8, ("int8", "int32"): capi.KIND_INT8_ACC32,
          ("float16", "float16"): capi.KIND_FP16}


class SparseConvKernel(object):
    """SparseConvCompute<Ptype, OutType> with the HIP library behind it.

    precision/out_precision select the registration: ("float32","float32") =
    def, ("int8","float32") = int8_fp32_out, ("int8","int8") = int8_int8_out
    (reference: lite/kernels/arm/sparse_conv_compute.cc:369-430).
    ("int8","int32") exposes the raw accumulators for verification;
    ("float16","float16") is the half-precision kernel
    (sparse_conv_compute.cc:270-356): fp32 sparse tensors and bias in the
    parameter, converted to fp16 at PrepareForRun, fp16 activations.

    reference_quirks=True reproduces what the reference computes through its
    kernel class for int8 output: the leaky slope is divided by output_scale
    and the hard_swish offset / threshold are divided by output_scale twice
    (once in PrepareForRun, sparse_conv_compute.cc:86-100, once more inside
    the math function, sparse_conv_impl.cc:3713-3720).  False applies the
    output scale once and leaves the slope alone.
    """

    def __init__(self, param, precision="float32", out_precision="float32", algo=capi.ALGO_AUTO, reference_quirks=True, tuning=None):
        key = (str(np.dtype(precision)), str(np.dtype(out_precision)))
        if key not in _KINDS:
            raise ValueError("no sparse_conv2d kernel for %s -> %s" % key)
        self.kind = _KINDS[key]
        self.param = param
        self.algo = algo
        self.tuning = tuning  # capi.Tuning or None (every rule of the library applies)
        self.reference_quirks = reference_quirks
        self._handle = None
        self._first_epoch = True
        self.w_scale_ = []
        self.bias_ = None
        self.merged_act = None

    # -- SparseConvCompute::PrepareForRun
    def PrepareForRun(self):
        p = self.param
        oc = p.weights.oc
        act = p.activation_param.copy()
        bias = p.bias
        scale = None
        if self.kind not in (capi.KIND_FP32, capi.KIND_FP16):
            ws = list(p.weight_scale)
            if len(ws) != 1 and len(ws) != oc:
                raise ValueError("weights scale size must equal to filter size")
            if len(ws) == 1:
                ws = ws * oc
            ws = np.asarray(ws, dtype=np.float32)
            isc, osc = np.float32(p.input_scale), np.float32(p.output_scale)
            if self.kind == capi.KIND_INT8_INT8:
                scale = ws * isc / osc
                if bias is not None:
                    bias = (bias / osc).astype(np.float32)
                f32 = lambda v: float(np.float32(np.float32(v) / osc))  # noqa: E731
                if act.active_type == capi.ACT_RELU6:
                    act.Relu_clipped_coef = f32(act.Relu_clipped_coef)
                if act.active_type == capi.ACT_LEAKY_RELU and self.reference_quirks:
                    act.Leaky_relu_alpha = f32(act.Leaky_relu_alpha)
                if act.active_type == capi.ACT_HARD_SWISH:
                    act.hard_swish_scale = f32(act.hard_swish_scale)
                    act.hard_swish_offset = f32(act.hard_swish_offset)
                    act.hard_swish_threshold = f32(act.hard_swish_threshold)
            else:
                scale = ws * isc
            scale = np.ascontiguousarray(scale, dtype=np.float32)
            self.w_scale_ = scale
        self.bias_ = bias
        self.merged_act = act
        a = capi.Activation()
        a.type = act.active_type if act.has_active else capi.ACT_NONE
        a.relu6_coef = act.Relu_clipped_coef
        a.leaky_alpha = act.Leaky_relu_alpha
        a.hs_scale = act.hard_swish_scale
        a.hs_offset = act.hard_swish_offset
        a.hs_threshold = act.hard_swish_threshold
        if self.kind == capi.KIND_INT8_INT8 and a.type == capi.ACT_HARD_SWISH and self.reference_quirks:
            osc = np.float32(p.output_scale)
            a.hs_offset = float(np.float32(np.float32(a.hs_offset) / osc))
            a.hs_threshold = float(np.float32(np.float32(a.hs_threshold) / osc))
        self._capi_act = a
        w = p.weights
        d = capi.Desc()
        d.struct_size = C.sizeof(capi.Desc)
        d.kind = self.kind
        d.flag_semi = p.flag_semi
        d.first_ic = p.first_ic
        d.oc, d.ic, d.im_size = w.oc, w.ic, w.im_size
        d.algo = self.algo
        d.nonzero_weights = w.nonzero_weights.ctypes.data if w.nonzero_weights.size else None
        d.n_weights = w.nonzero_weights.size
        d.oc_nonzeros = w.oc_nonzeros.ctypes.data
        d.diffs = w.diffs.ctypes.data if w.diffs.size else None
        d.n_diffs = w.diffs.size
        d.scale = scale.ctypes.data if scale is not None else None
        d.bias = bias.ctypes.data if bias is not None else None
        d.act = a
        if self.tuning is not None:
            d.tuning = self.tuning
        h = C.c_void_p()
        capi.check(capi.lib().pl_sparse_conv_prepare(C.byref(d), C.byref(h)))
        self._release()
        self._handle = h
        self._first_epoch = False

    # -- KernelBase::Launch
    def Launch(self, x, out=None, stream=None):
        if self._first_epoch:
            self.PrepareForRun()
        return self.Run(x, out, stream)

    # -- SparseConvCompute::Run; x and out are CUDA-device torch tensors
    def Run(self, x, out=None, stream=None):
        import torch

        if self._handle is None:
            raise RuntimeError("PrepareForRun has not been called")
        if not x.is_cuda or not x.is_contiguous():
            raise ValueError("x must be a contiguous device tensor")
        want_in = {capi.KIND_FP32: torch.float32, capi.KIND_FP16: torch.float16}.get(self.kind, torch.int8)
        if x.dtype != want_in or x.dim() != 4 or x.shape[1] != self.param.weights.ic:
            raise ValueError("x must be %s NCHW with %d channels" % (want_in, self.param.weights.ic))
        n, _, hh, ww = x.shape
        odt = {capi.KIND_FP32: torch.float32, capi.KIND_INT8_FP32: torch.float32, capi.KIND_INT8_INT8: torch.int8, capi.KIND_INT8_ACC32: torch.int32, capi.KIND_FP16: torch.float16}[self.kind]
        # output shape as SparseConvOp::InferShapeImpl for 1x1 / stride 1 / pad 0
        # (reference: lite/operators/sparse_conv_op.cc:46-65)
        shape = (n, self.param.weights.oc, hh, ww)
        if out is None:
            out = torch.empty(shape, dtype=odt, device=x.device)
        elif tuple(out.shape) != shape or out.dtype != odt or not out.is_contiguous() or out.device != x.device:
            raise ValueError("out must be a contiguous %s tensor of shape %s on %s" % (odt, shape, x.device))
        if stream is None:
            stream = torch.cuda.current_stream(x.device).cuda_stream
        capi.check(capi.lib().pl_sparse_conv_run(self._handle, x.data_ptr(), out.data_ptr(), n, hh * ww, C.c_void_p(stream)))
        return out

    def info(self):
        i = capi.Info()
        capi.check(capi.lib().pl_sparse_conv_get_info(self._handle, C.byref(i)))
        return {f: getattr(i, f) for f, _ in capi.Info._fields_}

    def _release(self):
        if self._handle is not None:
            capi.lib().pl_sparse_conv_destroy(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self._release()
        except Exception:
            pass
