"""The reference's own packers (lite/tests/math/conv_ut.h:183-538, compiled
from the reference checkout into oracle/_ref by oracle/Makefile) against the
oracle's restatement and the library's packers (the C ABI's host-side
pl_sparse_count_* / pl_sparse_pack) on several hundred random matrices:
every output tensor and first_ic bit for bit.  Skipped where oracle/_ref was
not built (no reference checkout)."""
import ctypes as C

import numpy as np
import pytest

from helpers import capi, pla
from oracle import oracle as O

pytestmark = pytest.mark.skipif(not O.have_ref_packers(), reason="oracle/_ref/libref_packers.so needs the reference checkout")


def random_matrix(rng, dtype, paired):
    m = int(rng.randint(1, 41))
    k = int(rng.randint(1, 70))
    sparsity = rng.choice([0.0, 0.3, 0.5, 0.8, 0.95, 1.0])
    if paired:
        m = max(m, 2)
        half = rng.random_sample(((m + 1) // 2, k)) >= sparsity
        mask = np.repeat(half, 2, axis=0)[:m]
    else:
        mask = rng.random_sample((m, k)) >= sparsity
    if dtype == np.float32:
        v = rng.standard_normal((m, k)).astype(np.float32)
        v[v == 0] = 1.0
    else:
        v = rng.randint(1, 128, size=(m, k)).astype(np.int8) * (rng.randint(0, 2, size=(m, k)) * 2 - 1).astype(np.int8)
    return (v * mask).astype(dtype)


def same(a, b, what):
    assert a.first_ic == b.first_ic, what
    assert np.array_equal(a.nonzero_weights.view(np.uint8), b.nonzero_weights.view(np.uint8)), what
    assert np.array_equal(a.oc_nonzeros, b.oc_nonzeros), what
    assert np.array_equal(a.diffs, b.diffs), what


def product_pack(w, im_size, semi):
    """The library's packers through the C ABI (host only, no device needed)."""
    weights = pla.detect_and_pack(w, im_size, force_semi=semi)
    return O.Packed(O.LAYOUT_SEMI if semi else (O.LAYOUT_PADDED if w.dtype == np.float32 else O.LAYOUT_UNPADDED), weights.nonzero_weights, weights.oc_nonzeros, weights.diffs, weights.first_ic, int(semi),
                    w.shape[0], w.shape[1], im_size)


@pytest.mark.parametrize("dtype", [np.float32, np.int8], ids=["fp32", "int8"])
def test_counting_passes_equal_the_references(dtype):
    rng = np.random.RandomState(11)
    for i in range(300):
        w = random_matrix(rng, dtype, paired=bool(i % 2))
        assert O.count_zeros_pad4(w) == O.ref_count_zeros_pad4(w), w.shape
        ref = O.ref_count_semi(w)
        # the test's copy of the rule adds "height > 1" to the pass's (conv_ut.h:263 against
        # sparse_conv_detect_pass.cc:356); the oracle states both, the library follows the pass
        assert O.count_semi(w, need_rows_gt1=True) == ref, w.shape
        if w.shape[0] == 1:
            continue
        assert O.count_semi(w) == ref, w.shape
        L = capi.lib()
        cn, cc, cb, fs = C.c_int32(), C.c_int32(), C.c_int32(), C.c_int32()
        z = L.pl_sparse_count_semi(0 if dtype == np.float32 else 1, w.ctypes.data_as(C.c_void_p), w.shape[0], w.shape[1], C.byref(cn), C.byref(cc), C.byref(cb), C.byref(fs))
        assert dict(zeros=z, count_nonzeroes=cn.value, count_channels=cc.value, count_blocks=cb.value, flag_semi=fs.value) == ref, w.shape
        nb = C.c_int32()
        z = L.pl_sparse_count_zeros(0 if dtype == np.float32 else 1, w.ctypes.data_as(C.c_void_p), w.shape[0], w.shape[1], C.byref(nb))
        assert (z, nb.value) == O.ref_count_zeros_pad4(w), w.shape


@pytest.mark.parametrize("dtype", [np.float32, np.int8], ids=["fp32", "int8"])
def test_packers_equal_the_references(dtype):
    rng = np.random.RandomState(12)
    n_semi = 0
    for i in range(300):
        w = random_matrix(rng, dtype, paired=bool(i % 2))
        im_size = int(rng.choice([1, 9, 49, 196, 3136]))
        for layout in (O.LAYOUT_UNPADDED, O.LAYOUT_PADDED):
            same(O.pack(w, im_size, layout), O.ref_pack(w, im_size, layout), (w.shape, layout))
        # the pass's own choice, as the library makes it
        if w.shape[0] == 1:
            continue  # the pass and the test's copy of its rule differ for a single row (see above)
        semi = bool(O.ref_count_semi(w)["flag_semi"])
        if semi:
            n_semi += 1
            ref = O.ref_pack(w, im_size, O.LAYOUT_SEMI)
            same(O.pack(w, im_size, O.LAYOUT_SEMI), ref, (w.shape, "semi"))
            same(product_pack(w, im_size, True), ref, (w.shape, "product semi"))
        else:
            layout = O.LAYOUT_PADDED if dtype == np.float32 else O.LAYOUT_UNPADDED
            same(product_pack(w, im_size, False), O.ref_pack(w, im_size, layout), (w.shape, "product"))
    assert n_semi > 50
