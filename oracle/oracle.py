"""numpy front end of the CPU oracle (oracle/libsparse_conv_oracle.so) and of the
reference's own naive math when oracle/_ref was built.

TEST INFRASTRUCTURE ONLY.  Importable from tests/, the smoke check and the
benchmark's cpu_baseline leg; never from the shipped package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libsparse_conv_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libref_naive.so")
_REF_OMP_PATH = os.path.join(_HERE, "_ref", "libref_naive_omp.so")

ACT_NONE, ACT_RELU, ACT_RELU6, ACT_LEAKY_RELU, ACT_HARD_SWISH = 0, 1, 2, 4, 10
LAYOUT_UNPADDED, LAYOUT_PADDED, LAYOUT_SEMI = 0, 1, 2


class Act(C.Structure):
    """Activation constants as the math functions consume them."""

    _fields_ = [
        ("type", C.c_int32),
        ("relu6_coef", C.c_float),
        ("leaky_alpha", C.c_float),
        ("hs_scale", C.c_float),
        ("hs_offset", C.c_float),
        ("hs_threshold", C.c_float),
    ]

    def __init__(self, type=ACT_NONE, relu6_coef=6.0, leaky_alpha=0.0,
                 hs_scale=6.0, hs_offset=3.0, hs_threshold=6.0):
        super().__init__(int(type), relu6_coef, leaky_alpha, hs_scale,
                         hs_offset, hs_threshold)

    def copy(self):
        return Act(self.type, self.relu6_coef, self.leaky_alpha, self.hs_scale,
                   self.hs_offset, self.hs_threshold)


def build(force=False):
    """Compile the oracle (and oracle/_ref where the reference is present)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-s", "all"])


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.plo_dense_conv1x1.restype = C.c_int
    return _lib


def have_ref():
    return os.path.exists(_REF_PATH)


_ref = {}


def ref(omp=False):
    path = _REF_OMP_PATH if omp else _REF_PATH
    if path not in _ref:
        _ref[path] = C.CDLL(path)
    return _ref[path]


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _dtype_code(w):
    if w.dtype == np.float32:
        return 0
    if w.dtype == np.int8:
        return 1
    raise TypeError("weights must be float32 or int8")


def _c(a, dt=None):
    if a is None:
        return None
    return np.ascontiguousarray(a, dtype=dt)


# ----------------------------------------------------------------- packers
def count_zeros_pad4(w):
    w = _c(w)
    nb = C.c_int(0)
    z = lib().plo_count_zeros_pad4(_dtype_code(w), _p(w), w.shape[0],
                                   w.shape[1], C.byref(nb))
    return z, nb.value


def count_semi(w, need_rows_gt1=False):
    w = _c(w)
    cn, cc, cb, fs = C.c_int(0), C.c_int(0), C.c_int(0), C.c_int(0)
    z = lib().plo_count_semi(_dtype_code(w), _p(w), w.shape[0], w.shape[1],
                             int(need_rows_gt1), C.byref(cn), C.byref(cc),
                             C.byref(cb), C.byref(fs))
    return dict(zeros=z, count_nonzeroes=cn.value, count_channels=cc.value,
                count_blocks=cb.value, flag_semi=fs.value)


class Packed(object):
    """The three weight tensors of a sparse_conv2d op plus its attributes."""

    def __init__(self, layout, nonzero_weights, oc_nonzeros, diffs, first_ic,
                 flag_semi, M, K, N):
        self.layout = layout
        self.nonzero_weights = nonzero_weights
        self.oc_nonzeros = oc_nonzeros
        self.diffs = diffs
        self.first_ic = first_ic
        self.flag_semi = flag_semi
        self.M, self.K, self.N = M, K, N


def pack(w, im_size, layout):
    """Run one of the three packers on a dense [M, K] matrix."""
    w = _c(w)
    M, K = w.shape
    dt = _dtype_code(w)
    if layout == LAYOUT_PADDED:
        _, n_w = count_zeros_pad4(w)
        n_d = n_w
        fn = lib().plo_pack_padded
    elif layout == LAYOUT_UNPADDED:
        n_w = int(np.count_nonzero(w))
        n_d = n_w
        fn = lib().plo_pack_unpadded
    else:
        c = count_semi(w)
        paired = (M // 2) * 2
        blocks2 = int(np.count_nonzero((w[0:paired:2] != 0) | (w[1:paired:2] != 0)))
        tail = int(np.count_nonzero(w[paired:]))
        n_w, n_d = 2 * blocks2 + tail, blocks2 + tail
        del c
        fn = lib().plo_pack_semi
    nz = np.zeros(max(n_w, 1), dtype=w.dtype)[:n_w]
    oc = np.zeros(M, dtype=np.uint32)
    df = np.zeros(max(n_d, 1), dtype=np.int32)[:n_d]
    first_ic = fn(dt, _p(w), M, K, int(im_size), _p(nz), _p(oc), _p(df))
    return Packed(layout, nz, oc, df, first_ic, int(layout == LAYOUT_SEMI), M,
                  K, int(im_size))


def pack_like_pass(w, im_size, need_rows_gt1=False):
    """Layout choice of sparse_conv_detect_pass: semi when the block rule
    fires, else padded for fp32 and unpadded for int8
    (reference: lite/core/optimizer/mir/sparse_conv_detect_pass.cc:732-780)."""
    w = _c(w)
    c = count_semi(w, need_rows_gt1)
    if c["flag_semi"]:
        return pack(w, im_size, LAYOUT_SEMI)
    return pack(w, im_size,
                LAYOUT_PADDED if w.dtype == np.float32 else LAYOUT_UNPADDED)


def decode(pk, dtype=None):
    dtype = dtype or pk.nonzero_weights.dtype
    out = np.zeros((pk.M, pk.K), dtype=dtype)
    nz = _c(pk.nonzero_weights)
    rc = lib().plo_decode(0 if dtype == np.float32 else 1, pk.layout, _p(nz),
                          _p(_c(pk.oc_nonzeros)), _p(_c(pk.diffs)),
                          pk.first_ic, pk.M, pk.K, pk.N, _p(out))
    if rc != 0:
        raise ValueError("layout does not decode")
    return out


# ------------------------------------------------------------------- SpMM
def sparse_conv_fp32(pk, x, bias=None, act=None):
    x = _c(x, np.float32)
    batch, K, N = x.shape[0], x.shape[1], int(np.prod(x.shape[2:]))
    out = np.empty((batch, pk.M) + x.shape[2:], dtype=np.float32)
    bias = _c(bias, np.float32)
    lib().plo_sparse_conv_fp32(_p(_c(pk.nonzero_weights)), _p(x),
                               _p(_c(pk.diffs)), _p(_c(pk.oc_nonzeros)),
                               _p(bias), _p(out), batch, pk.M, K, N,
                               pk.first_ic, pk.flag_semi,
                               C.byref(act) if act else None)
    return out


def fp32_to_fp16(x):
    """Element-wise conversion (round to nearest even); returns float16."""
    x = _c(x, np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().plo_fp32_to_fp16(_p(x), _p(out), C.c_int64(x.size))
    return out.view(np.float16)


def sparse_conv_fp16(pk, x, bias=None, act=None):
    """pk: the fp32 packing of the pass; x: float16 activations; bias: fp32
    (converted like the kernel class does).  Returns float16."""
    x = _c(x, np.float16)
    batch, K, N = x.shape[0], x.shape[1], int(np.prod(x.shape[2:]))
    out = np.empty((batch, pk.M) + x.shape[2:], dtype=np.uint16)
    w16 = _c(fp32_to_fp16(pk.nonzero_weights).view(np.uint16))
    b16 = _c(fp32_to_fp16(bias).view(np.uint16)) if bias is not None else None
    lib().plo_sparse_conv_fp16(_p(w16), _p(_c(x.view(np.uint16))), _p(_c(pk.diffs)), _p(_c(pk.oc_nonzeros)), _p(b16), _p(out), batch, pk.M, K, N,
                               pk.first_ic, pk.flag_semi, C.byref(act) if act else None)
    return out.view(np.float16)


def sparse_conv_int8(pk, x, scale, bias=None, act=None, out_int8=False):
    x = _c(x, np.int8)
    batch, K, N = x.shape[0], x.shape[1], int(np.prod(x.shape[2:]))
    out = np.empty((batch, pk.M) + x.shape[2:],
                   dtype=np.int8 if out_int8 else np.float32)
    scale = _c(scale, np.float32)
    bias = _c(bias, np.float32)
    fn = (lib().plo_sparse_conv_int8_int8 if out_int8 else
          lib().plo_sparse_conv_int8_fp32)
    fn(_p(_c(pk.nonzero_weights)), _p(x), _p(_c(pk.diffs)),
       _p(_c(pk.oc_nonzeros)), _p(bias), _p(scale), _p(out), batch, pk.M, K, N,
       pk.first_ic, pk.flag_semi, C.byref(act) if act else None)
    return out


def sparse_conv_int8_acc(pk, x):
    x = _c(x, np.int8)
    batch, K, N = x.shape[0], x.shape[1], int(np.prod(x.shape[2:]))
    out = np.empty((batch, pk.M) + x.shape[2:], dtype=np.int32)
    lib().plo_sparse_conv_int8_acc(_p(_c(pk.nonzero_weights)), _p(x),
                                   _p(_c(pk.diffs)), _p(_c(pk.oc_nonzeros)),
                                   _p(out), batch, pk.M, K, N, pk.first_ic,
                                   pk.flag_semi)
    return out


# ------------------------------------------------- naive dense reference
def _gemm_args(a, b, bias, act):
    act = act or Act()
    m, k = a.shape
    n = b.shape[1]
    c = np.zeros((m, n), dtype=np.float32)
    return (m, n, k, _p(a), _p(b), _p(c), _p(bias), int(bias is not None),
            int(act.type), C.c_float(act.relu6_coef),
            C.c_float(act.leaky_alpha), C.c_float(act.hs_scale),
            C.c_float(act.hs_offset), C.c_float(act.hs_threshold)), c


def basic_gemm_f32(a, b, bias=None, act=None):
    a, b, bias = _c(a, np.float32), _c(b, np.float32), _c(bias, np.float32)
    args, c = _gemm_args(a, b, bias, act)
    lib().plo_basic_gemm_f32(*args)
    return c


def ref_basic_gemm_f32(a, b, bias=None, act=None, omp=False):
    a, b, bias = _c(a, np.float32), _c(b, np.float32), _c(bias, np.float32)
    args, c = _gemm_args(a, b, bias, act)
    ref(omp).ref_basic_gemm_f32(*args)
    return c


def ref_conv1x1_f32(x, w, bias=None, act=None, omp=False):
    x, w, bias = _c(x, np.float32), _c(w, np.float32), _c(bias, np.float32)
    act = act or Act()
    n, cin, h, ww = x.shape
    out = np.zeros((n, w.shape[0], h, ww), dtype=np.float32)
    ref(omp).ref_conv1x1_f32(_p(x), _p(out), n, w.shape[0], h, ww, cin, _p(w),
                             _p(bias), int(bias is not None), int(act.type),
                             C.c_float(act.relu6_coef),
                             C.c_float(act.leaky_alpha),
                             C.c_float(act.hs_scale), C.c_float(act.hs_offset),
                             C.c_float(act.hs_threshold))
    return out


def ref_conv1x1_s8_s32(x, w, omp=False):
    x, w = _c(x, np.int8), _c(w, np.int8)
    n, cin, h, ww = x.shape
    out = np.zeros((n, w.shape[0], h, ww), dtype=np.int32)
    ref(omp).ref_conv1x1_s8_s32(_p(x), _p(out), n, w.shape[0], h, ww, cin,
                                _p(w))
    return out


def dwconv_out_size(size, stride, pad):
    return (size + 2 * pad - 3) // stride + 1


def dwconv3x3_int8(x, w, scale=None, bias=None, act=None, out="int8", stride=1,
                   pad=1):
    """int8 depthwise 3x3; out: "fp32", "int8" or "acc" (raw int32 sums)."""
    x, w = _c(x, np.int8), _c(w, np.int8)
    n, ch, h, ww = x.shape
    assert w.shape == (ch, 3, 3)
    kind = {"fp32": 1, "int8": 2, "acc": 3}[out]
    oh, ow = dwconv_out_size(h, stride, pad), dwconv_out_size(ww, stride, pad)
    res = np.zeros((n, ch, oh, ow),
                   dtype={1: np.float32, 2: np.int8, 3: np.int32}[kind])
    scale = None if scale is None else _c(scale, np.float32)
    bias = None if bias is None else _c(bias, np.float32)
    act = act or Act()
    rc = lib().plo_dwconv3x3_int8(_p(x), _p(w), _p(scale), _p(bias),
                                  C.byref(act), kind, n, ch, h, ww, stride,
                                  pad, _p(res))
    if rc != 0:
        raise ValueError("plo_dwconv3x3_int8: bad argument")
    return res


def ref_dwconv3x3_s8_s32(x, w, stride=1, pad=1):
    """The reference header's conv_basic<int8, int32> with group == channels."""
    x, w = _c(x, np.int8), _c(w, np.int8)
    n, ch, h, ww = x.shape
    oh, ow = dwconv_out_size(h, stride, pad), dwconv_out_size(ww, stride, pad)
    out = np.zeros((n, ch, oh, ow), dtype=np.int32)
    ref().ref_dwconv3x3_s8_s32(_p(x), _p(out), n, ch, oh, ow, h, ww, _p(w),
                               stride, pad)
    return out


def fp32_to_int8(x, scale):
    x = _c(x, np.float32)
    out = np.empty(x.shape, dtype=np.int8)
    lib().plo_fp32_to_int8(_p(x), _p(out), C.c_float(scale),
                           C.c_int64(x.size))
    return out


def int8_to_fp32(x, scale):
    x = _c(x, np.int8)
    out = np.empty(x.shape, dtype=np.float32)
    lib().plo_int8_to_fp32(_p(x), _p(out), C.c_float(scale), C.c_int64(x.size))
    return out


def merge_params(out_kind, M, weight_scale, input_scale, output_scale, bias,
                 act):
    """Returns (merged_scale, merged_bias, merged_act)."""
    ws = _c(np.atleast_1d(weight_scale), np.float32)
    bias = _c(bias, np.float32)
    ms = np.zeros(M, dtype=np.float32)
    mb = np.zeros(M, dtype=np.float32) if bias is not None else None
    a = act.copy() if act else Act()
    rc = lib().plo_merge_params(int(out_kind), M, _p(ws), ws.size,
                                C.c_float(input_scale),
                                C.c_float(output_scale), _p(bias), _p(ms),
                                _p(mb), C.byref(a))
    if rc != 0:
        raise ValueError("weights scale size must equal to filter size")
    return ms, mb, a


def dense_conv1x1(out_kind, w_dense, x, scale=None, bias=None, act=None,
                  threads=0):
    """Dense per-image GEMM comparator; returns (out, threads_used)."""
    if out_kind == 0:
        w_dense, x = _c(w_dense, np.float32), _c(x, np.float32)
        odt = np.float32
    else:
        w_dense, x = _c(w_dense, np.int8), _c(x, np.int8)
        odt = np.int8 if out_kind == 2 else np.float32
    batch, K, N = x.shape[0], x.shape[1], int(np.prod(x.shape[2:]))
    M = w_dense.shape[0]
    out = np.empty((batch, M) + x.shape[2:], dtype=odt)
    scale, bias = _c(scale, np.float32), _c(bias, np.float32)
    used = lib().plo_dense_conv1x1(int(out_kind), _p(w_dense), _p(x), _p(bias),
                                   _p(scale), _p(out), batch, M, K, N,
                                   C.byref(act) if act else None, int(threads))
    return out, used


# ------------------------------------------------- reference packers / x86 GEMM
_REF_PACKERS_PATH = os.path.join(_HERE, "_ref", "libref_packers.so")
_REF_X86_GEMM_PATH = os.path.join(_HERE, "_ref", "libref_x86_gemm.so")


def have_ref_packers():
    return os.path.exists(_REF_PACKERS_PATH)


def have_ref_x86_gemm():
    return os.path.exists(_REF_X86_GEMM_PATH)


def _ref_lib(path):
    if path not in _ref:
        _ref[path] = C.CDLL(path)
    return _ref[path]


def ref_count_zeros_pad4(w):
    """The reference's ComputeSparseZeros (lite/tests/math/conv_ut.h:183-207)."""
    w = _c(w)
    nb = C.c_int(0)
    z = _ref_lib(_REF_PACKERS_PATH).ref_count_zeros_pad4(_dtype_code(w), _p(w), w.shape[0], w.shape[1], C.byref(nb))
    return z, nb.value


def ref_count_semi(w):
    """The reference's ComputeSemiSparseZeros (conv_ut.h:209-274)."""
    w = _c(w)
    cn, cc, cb, fs = C.c_int(0), C.c_int(0), C.c_int(0), C.c_int(0)
    z = _ref_lib(_REF_PACKERS_PATH).ref_count_semi(_dtype_code(w), _p(w), w.shape[0], w.shape[1], C.byref(cn), C.byref(cc), C.byref(cb), C.byref(fs))
    return dict(zeros=z, count_nonzeroes=cn.value, count_channels=cc.value, count_blocks=cb.value, flag_semi=fs.value)


def ref_pack(w, im_size, layout):
    """The reference's ComputeSparseWeight (both overloads) /
    ComputeSemiSparseWeight (conv_ut.h:276-538) on a dense [M, K] matrix; the
    output sizes are what its tests allocate (conv_ut.h counting passes)."""
    w = _c(w)
    M, K = w.shape
    if layout == LAYOUT_PADDED:
        _, n_w = ref_count_zeros_pad4(w)
        n_d = n_w
    elif layout == LAYOUT_UNPADDED:
        n_w = n_d = int(np.count_nonzero(w))
    else:
        c = ref_count_semi(w)
        if not c["flag_semi"]:
            raise ValueError("the reference packs semi-structured only where its block rule fires")
        n_w, n_d = c["count_nonzeroes"], c["count_blocks"]
    nz = np.zeros(max(n_w, 1), dtype=w.dtype)[:n_w]
    oc = np.zeros(M, dtype=np.uint32)
    df = np.zeros(max(n_d, 1), dtype=np.int32)[:n_d]
    code = {LAYOUT_UNPADDED: 0, LAYOUT_PADDED: 1, LAYOUT_SEMI: 2}[layout]
    fn = _ref_lib(_REF_PACKERS_PATH).ref_pack
    fn.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int64]
    first_ic = fn(_dtype_code(w), code, _p(w), M, K, int(im_size), _p(nz), n_w, _p(oc), _p(df), n_d)
    if first_ic < 0:
        raise ValueError("the reference packer refused the matrix")
    return Packed(layout, nz, oc, df, first_ic, int(layout == LAYOUT_SEMI), M, K, int(im_size))


def ref_x86_conv1x1_s8_f32(x, w_dense, weight_scale, input_scale, bias=None, relu_type=0, relu_alpha=1.0, reps=1, threads=1):
    """The reference's x86 int8 GEMM run like its dense conv2d kernel runs a
    1x1 convolution (lite/kernels/x86/conv_compute.cc:215-340).  Returns
    (out, seconds spent in the compute calls)."""
    x, w_dense = _c(x, np.int8), _c(w_dense, np.int8)
    ws, bias = _c(weight_scale, np.float32), _c(bias, np.float32)
    batch, K, N = x.shape[0], x.shape[1], int(np.prod(x.shape[2:]))
    M = w_dense.shape[0]
    out = np.zeros((batch, M) + x.shape[2:], dtype=np.float32)
    fn = _ref_lib(_REF_X86_GEMM_PATH).ref_x86_conv1x1_s8_f32
    fn.restype = C.c_double
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_float, C.c_void_p, C.c_int, C.c_float, C.c_int, C.c_int]
    secs = fn(_p(x), _p(out), batch, M, N, K, _p(w_dense), _p(ws), float(input_scale), _p(bias), int(relu_type), float(relu_alpha), int(reps), int(threads))
    return out, secs
