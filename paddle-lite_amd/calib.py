"""Host mirror of the reference's `calib` op for the two precision changes
that sit either side of an int8 sparse convolution.

Same names and meaning as lite/operators/op_params.h:74-78 (CalibParam) and
lite/kernels/arm/calib_compute.{h,cc} (CalibComputeFp32ToInt8,
CalibComputeInt8ToFp32; registered as `calib` with aliases `fp32_to_int8` and
`int8_to_fp32`, calib_compute.cc:186-330).  Tensors are device buffers given
as (pointer, element count); the work is done by the HIP kernels behind
pl_calib_fp32_to_int8 / pl_calib_int8_to_fp32.
"""
import ctypes as C

from . import capi


class CalibParam(object):
    """input / output: objects with data_ptr() and numel() (torch tensors on
    the device); scale: the per-tensor quantisation scale."""

    def __init__(self, input=None, output=None, scale=1.0):
        self.input = input
        self.output = output
        self.scale = float(scale)


class _CalibCompute(object):
    alias = None
    _entry = None

    def __init__(self, param):
        self.param = param

    def PrepareForRun(self):
        if self.param.input is None or self.param.output is None:
            raise ValueError("calib: Input and Out must be set")

    def Run(self, stream=0):
        p = self.param
        n = int(p.input.numel())
        if int(p.output.numel()) != n:
            raise ValueError("calib: Out must have the shape of Input")
        fn = getattr(capi.lib(), self._entry)
        capi.check(fn(C.c_void_p(p.input.data_ptr()), C.c_void_p(p.output.data_ptr()), n, C.c_float(p.scale), C.c_void_p(stream)))

    Launch = Run


class CalibComputeFp32ToInt8(_CalibCompute):
    """out = saturate(round_half_away(x * (1 / scale))), never below -127
    (calib_compute.cc:31-38 -> type_trans.cc:35-160)."""
    alias = "fp32_to_int8"
    _entry = "pl_calib_fp32_to_int8"


class CalibComputeInt8ToFp32(_CalibCompute):
    """out = x * scale (calib_compute.cc:60-68)."""
    alias = "int8_to_fp32"
    _entry = "pl_calib_int8_to_fp32"
