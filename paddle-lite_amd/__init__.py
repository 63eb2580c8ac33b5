"""MI355X-native sparse_conv2d (the 1x1 sparse convolution of Paddle-Lite).

The arithmetic lives in lib/libpl_sparse_conv.so (hand-written HIP for
gfx950 behind the C ABI of include/pl_sparse_conv.h).  This package is the
Python host side: a ctypes binding of that ABI, a mirror of the operator's
parameter handling, and the seeded synthetic workloads of the benchmark.
There is no CPU fallback: without the built library or without a gfx950
device every compute call raises.
"""
from . import capi  # noqa: F401
from .sparse_conv import (  # noqa: F401
    ActivationParam,
    SparseConvParam,
    SparseConvKernel,
    SparseWeights,
    detect_and_pack,
)

from .calib import CalibParam, CalibComputeFp32ToInt8, CalibComputeInt8ToFp32  # noqa: F401

__all__ = ["capi", "ActivationParam", "SparseConvParam", "SparseConvKernel", "SparseWeights", "detect_and_pack", "CalibParam", "CalibComputeFp32ToInt8", "CalibComputeInt8ToFp32"]
from .depthwise_conv import ConvParam, DepthwiseConv  # noqa: F401
