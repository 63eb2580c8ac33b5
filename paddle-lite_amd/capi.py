"""ctypes binding of include/pl_sparse_conv.h (one function per entry point)."""
import ctypes as C
import os

PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG, "lib", "libpl_sparse_conv.so")

ABI_VERSION = 1

PL_OK, PL_ERR_BAD_ARG, PL_ERR_BAD_LAYOUT, PL_ERR_UNSUPPORTED, PL_ERR_HIP, PL_ERR_NO_DEVICE = 0, -1, -2, -3, -4, -5
KIND_FP32, KIND_INT8_FP32, KIND_INT8_INT8, KIND_INT8_ACC32, KIND_FP16 = 0, 1, 2, 3, 4
ACT_NONE, ACT_RELU, ACT_RELU6, ACT_LEAKY_RELU, ACT_HARD_SWISH = 0, 1, 2, 4, 10
ALGO_AUTO, ALGO_ROW_WALK, ALGO_BLOCK_MFMA, ALGO_IMAGE_MFMA = 0, 1, 2, 3
TUNE_RULE, TUNE_NEVER, TUNE_ALWAYS = 0, 1, 2
IMAGE_KERNEL_REGROUP, IMAGE_KERNEL_TRANSPOSE, IMAGE_KERNEL_ROWS = 1, 2, 3

EXPORTS = [
    "pl_sparse_conv_abi_version",
    "pl_last_error",
    "pl_device_count",
    "pl_sparse_conv_prepare",
    "pl_sparse_conv_run",
    "pl_sparse_conv_run_sequence",
    "pl_sparse_conv_get_info",
    "pl_sparse_conv_algo_for",
    "pl_sparse_conv_set_epilogue",
    "pl_sparse_conv_destroy",
    "pl_sparse_count_semi",
    "pl_sparse_count_zeros",
    "pl_sparse_pack",
    "pl_fp32_to_fp16",
    "pl_calib_fp32_to_int8",
    "pl_calib_int8_to_fp32",
    "pl_dwconv3x3_prepare",
    "pl_dwconv3x3_run",
    "pl_dwconv3x3_destroy",
    "pl_sparse_conv_dwconv3x3_fits",
    "pl_sparse_conv_dwconv3x3_pays",
    "pl_sparse_conv_dwconv3x3_run",
]


class Activation(C.Structure):
    _fields_ = [
        ("type", C.c_int32),
        ("relu6_coef", C.c_float),
        ("leaky_alpha", C.c_float),
        ("hs_scale", C.c_float),
        ("hs_offset", C.c_float),
        ("hs_threshold", C.c_float),
    ]


class Tuning(C.Structure):
    """pl_sparse_conv_tuning: every field 0 = the library's rule."""
    _fields_ = [
        ("image_kernel", C.c_int32),
        ("image_min_items", C.c_int32),
        ("mfma_stream", C.c_int32),
        ("mfma_sub_tiles", C.c_int32),
        ("mfma_tile_quads", C.c_int32),
        ("mfma_narrow_i8_stores", C.c_int32),
        ("wg_slots", C.c_int32),
        ("walk_tiled", C.c_int32),
        ("walk_split", C.c_int32),
        ("walk_chunked", C.c_int32),
        ("chunk_walk_groups", C.c_int32),
        ("walk_tile", C.c_int32),
        ("walk_threads", C.c_int32),
        ("walk_slices", C.c_int32),
        ("image_tr_regroup", C.c_int32),
        ("walk_pairs", C.c_int32),
    ]


def tuning(**fields):
    """A Tuning with the named fields set (the rest stay 0 = by rule)."""
    t = Tuning()
    for name, value in fields.items():
        if name not in dict(Tuning._fields_):
            raise ValueError("no tuning field %r" % name)
        setattr(t, name, int(value))
    return t


class DwConvDesc(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("kind", C.c_int32),
        ("channels", C.c_int32),
        ("stride", C.c_int32),
        ("pad", C.c_int32),
        ("weights", C.c_void_p),
        ("scale", C.c_void_p),
        ("bias", C.c_void_p),
        ("act", Activation),
        ("item_rows", C.c_int32),
        ("item_cols", C.c_int32),
        ("share_lanes", C.c_int32),
        ("row_items", C.c_int32),
    ]


class Desc(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("kind", C.c_int32),
        ("flag_semi", C.c_int32),
        ("first_ic", C.c_int32),
        ("oc", C.c_int32),
        ("ic", C.c_int32),
        ("im_size", C.c_int32),
        ("algo", C.c_int32),
        ("nonzero_weights", C.c_void_p),
        ("n_weights", C.c_int64),
        ("oc_nonzeros", C.c_void_p),
        ("diffs", C.c_void_p),
        ("n_diffs", C.c_int64),
        ("scale", C.c_void_p),
        ("bias", C.c_void_p),
        ("act", Activation),
        ("tuning", Tuning),
    ]


class Info(C.Structure):
    _fields_ = [
        ("algo", C.c_int32),
        ("oc", C.c_int32),
        ("ic", C.c_int32),
        ("nnz", C.c_int64),
        ("stored_weights", C.c_int64),
        ("index_entries", C.c_int64),
        ("device_bytes", C.c_int64),
        ("mfma_blocks", C.c_int64),
        ("mfma_blocks_total", C.c_int64),
    ]


class LibraryMissing(RuntimeError):
    pass


class SparseConvError(RuntimeError):
    def __init__(self, code, text):
        RuntimeError.__init__(self, "pl_sparse_conv error %d: %s" % (code, text))
        self.code = code


_lib = None


def lib():
    """Loads the built library; raises LibraryMissing if it was never built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise LibraryMissing(
            "%s is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
            "(or paddle-lite_amd/build_native.py). There is no fallback path." % LIB_PATH)
    L = C.CDLL(LIB_PATH)
    L.pl_sparse_conv_abi_version.restype = C.c_int
    L.pl_last_error.restype = C.c_char_p
    L.pl_device_count.restype = C.c_int
    L.pl_sparse_conv_prepare.argtypes = [C.POINTER(Desc), C.POINTER(C.c_void_p)]
    L.pl_sparse_conv_prepare.restype = C.c_int
    L.pl_sparse_conv_run.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p]
    L.pl_sparse_conv_run.restype = C.c_int
    L.pl_sparse_conv_run_sequence.argtypes = [C.c_void_p, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.POINTER(C.c_float)]
    L.pl_sparse_conv_run_sequence.restype = C.c_int
    L.pl_sparse_conv_get_info.argtypes = [C.c_void_p, C.POINTER(Info)]
    L.pl_sparse_conv_get_info.restype = C.c_int
    L.pl_sparse_conv_algo_for.argtypes = [C.c_void_p, C.c_int32, C.c_int32]
    L.pl_sparse_conv_algo_for.restype = C.c_int
    L.pl_sparse_conv_set_epilogue.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(Activation)]
    L.pl_sparse_conv_set_epilogue.restype = C.c_int
    L.pl_sparse_conv_destroy.argtypes = [C.c_void_p]
    L.pl_sparse_conv_destroy.restype = None
    L.pl_sparse_count_semi.argtypes = [C.c_int32, C.c_void_p, C.c_int32, C.c_int32] + [C.POINTER(C.c_int32)] * 4
    L.pl_sparse_count_semi.restype = C.c_int
    L.pl_sparse_count_zeros.argtypes = [C.c_int32, C.c_void_p, C.c_int32, C.c_int32, C.POINTER(C.c_int32)]
    L.pl_sparse_count_zeros.restype = C.c_int
    L.pl_sparse_pack.argtypes = [C.c_int32, C.c_int32, C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int64]
    L.pl_sparse_pack.restype = C.c_int
    L.pl_fp32_to_fp16.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
    L.pl_fp32_to_fp16.restype = C.c_int
    L.pl_calib_fp32_to_int8.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_float, C.c_void_p]
    L.pl_calib_fp32_to_int8.restype = C.c_int
    L.pl_calib_int8_to_fp32.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_float, C.c_void_p]
    L.pl_calib_int8_to_fp32.restype = C.c_int
    L.pl_dwconv3x3_prepare.argtypes = [C.POINTER(DwConvDesc), C.POINTER(C.c_void_p)]
    L.pl_dwconv3x3_prepare.restype = C.c_int
    L.pl_dwconv3x3_run.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_void_p]
    L.pl_dwconv3x3_run.restype = C.c_int
    L.pl_dwconv3x3_destroy.argtypes = [C.c_void_p]
    L.pl_dwconv3x3_destroy.restype = None
    L.pl_sparse_conv_dwconv3x3_fits.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32]
    L.pl_sparse_conv_dwconv3x3_fits.restype = C.c_int
    L.pl_sparse_conv_dwconv3x3_pays.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32]
    L.pl_sparse_conv_dwconv3x3_pays.restype = C.c_int
    L.pl_sparse_conv_dwconv3x3_run.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_void_p]
    L.pl_sparse_conv_dwconv3x3_run.restype = C.c_int
    if L.pl_sparse_conv_abi_version() != ABI_VERSION:
        raise LibraryMissing("libpl_sparse_conv.so has ABI %d, binding expects %d" % (L.pl_sparse_conv_abi_version(), ABI_VERSION))
    _lib = L
    return L


def last_error():
    return lib().pl_last_error().decode("utf-8", "replace")


def check(code):
    if code < 0:
        raise SparseConvError(code, last_error())
    return code
