"""Pins the oracle's packers: reference known-answer vectors, decode round
trips on every small shape, and the layout's closed-form invariants."""
import json
import os

import numpy as np
import pytest

from oracle import oracle as O

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "packer_kat.json")
LAYOUTS = {"unpadded": O.LAYOUT_UNPADDED, "padded": O.LAYOUT_PADDED,
           "semi": O.LAYOUT_SEMI}


def _cases():
    with open(GOLDEN) as f:
        return json.load(f)


@pytest.mark.parametrize("case", _cases()["cases"], ids=lambda c: c["name"])
def test_known_answer_vectors(case):
    N = _cases()["im_size"]
    w = np.array(case["dense"], dtype=case["dtype"]).reshape(case["rows"], case["cols"])
    semi = O.count_semi(w)
    assert semi["flag_semi"] == case["flag_semi"]
    if case["layout"] == "semi":
        assert semi["count_nonzeroes"] == case["count_nonzeroes"]
        assert semi["count_channels"] == case["count_channels"]
        assert semi["count_blocks"] == case["count_blocks"]
    if "num_build_nonzeroes" in case:
        zeros, nb = O.count_zeros_pad4(w)
        assert nb == case["num_build_nonzeroes"]
        assert zeros == w.size - np.count_nonzero(w)
    pk = O.pack(w, N, LAYOUTS[case["layout"]])
    assert pk.first_ic == case["first_ic"]
    assert pk.nonzero_weights.tolist() == case["nonzero_weights"]
    assert pk.diffs.tolist() == case["diffs"]
    if "oc_nonzeros" in case:
        assert pk.oc_nonzeros.tolist() == case["oc_nonzeros"]
    else:
        used = case["oc_nonzeros_used"]
        assert pk.oc_nonzeros[:len(used)].tolist() == used
    # the layout chosen by the pass is the one the vector was made with
    auto = O.pack_like_pass(w, N)
    assert auto.layout == LAYOUTS[case["layout"]]
    assert np.array_equal(O.decode(pk), w)


def _random_matrix(rng, M, K, density, dtype, paired):
    if paired:
        half = rng.random(((M + 1) // 2, K)) < density
        mask = np.repeat(half, 2, axis=0)[:M]
    else:
        mask = rng.random((M, K)) < density
    if dtype == np.int8:
        vals = rng.integers(1, 128, size=(M, K)) * rng.choice([-1, 1], size=(M, K))
    else:
        vals = rng.standard_normal((M, K)).astype(np.float32) + 3.0
    return (vals * mask).astype(dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.int8])
@pytest.mark.parametrize("layout", [O.LAYOUT_UNPADDED, O.LAYOUT_PADDED, O.LAYOUT_SEMI])
def test_decode_round_trip_all_small_shapes(dtype, layout):
    rng = np.random.default_rng(1234)
    for M in range(1, 10):
        for K in range(1, 10):
            for density in (0.0, 0.15, 0.5, 1.0):
                for N in (1, 7, 12):
                    w = _random_matrix(rng, M, K, density, dtype, paired=(layout == O.LAYOUT_SEMI))
                    if M > 2 and density > 0:
                        w[rng.integers(0, M)] = 0  # force an empty row
                    pk = O.pack(w, N, layout)
                    assert np.array_equal(O.decode(pk), w), (M, K, density, N)


@pytest.mark.parametrize("dtype", [np.float32, np.int8])
def test_layout_invariants(dtype):
    rng = np.random.default_rng(7)
    s = np.dtype(dtype).itemsize
    for trial in range(40):
        M, K, N = rng.integers(1, 40), rng.integers(1, 60), int(rng.integers(1, 50))
        w = _random_matrix(rng, M, K, 0.25, dtype, paired=False)
        nnz_rows = np.count_nonzero(w, axis=1)
        # unpadded: cumulative counts, monotone; total of all raw diffs is 0
        pk = O.pack(w, N, O.LAYOUT_UNPADDED)
        assert np.array_equal(pk.oc_nonzeros, np.cumsum(nnz_rows))
        assert np.array_equal(pk.nonzero_weights, w[w != 0])
        # row-end entries hold the absolute byte offset of the next row's
        # first nonzero: (ic_next_first - first_ic) * s * N
        rows_with = np.nonzero(nnz_rows)[0]
        for a, b in zip(rows_with[:-1], rows_with[1:]):
            ic_next = np.nonzero(w[b])[0][0]
            assert pk.diffs[pk.oc_nonzeros[a] - 1] == (ic_next - pk.first_ic) * s * N
        if len(rows_with):
            r_last = rows_with[-1]
            ic_last = np.nonzero(w[r_last])[0][-1]
            assert pk.diffs[-1] == (pk.first_ic - ic_last) * s * N  # wrap
            assert pk.first_ic == np.nonzero(w[rows_with[0]])[0][0]
        # padded: each row starts at a multiple of four, padding is zero
        pp = O.pack(w, N, O.LAYOUT_PADDED)
        start = 0
        for r in range(M):
            assert start % 4 == 0
            assert pp.oc_nonzeros[r] == start + nnz_rows[r]
            assert np.array_equal(pp.nonzero_weights[start:start + nnz_rows[r]], w[r][w[r] != 0])
            end = start + (nnz_rows[r] + 3) // 4 * 4
            assert not pp.nonzero_weights[start + nnz_rows[r]:end].any()
            start = end
        assert pp.nonzero_weights.size == O.count_zeros_pad4(w)[1]
        assert np.all(np.diff(pp.oc_nonzeros.astype(np.int64)) >= 0)


@pytest.mark.parametrize("dtype", [np.float32, np.int8])
def test_semi_rule_matches_counting_formula(dtype):
    rng = np.random.default_rng(99)
    for trial in range(60):
        M, K = int(rng.integers(1, 24)), int(rng.integers(1, 40))
        paired = bool(trial % 2)
        w = _random_matrix(rng, M, K, rng.choice([0.1, 0.3, 0.6]), dtype, paired)
        m2 = (M // 2) * 2
        nz = w != 0
        nnz2 = int(nz[:m2].sum())
        blocks2 = int((nz[0:m2:2] | nz[1:m2:2]).sum())
        tail = int(nz[m2:].sum())
        for gt1 in (False, True):
            c = O.count_semi(w, gt1)
            expect = nnz2 * 5 >= blocks2 * 9 and (M > 1 or not gt1)
            assert c["flag_semi"] == int(expect)
            if expect:
                assert c["count_nonzeroes"] == 2 * blocks2 + tail
                assert c["count_blocks"] == blocks2 + tail
                assert c["count_channels"] == M // 2 + M % 2
            else:
                assert c["count_nonzeroes"] == nnz2 + tail == c["count_blocks"]
                assert c["count_channels"] == M
            assert c["zeros"] == M * K - c["count_nonzeroes"]


def test_semi_threshold_edge():
    # 5 blocks holding 9 nonzeros is exactly the 1.8 nonzeros-per-block limit
    w = np.zeros((2, 6), dtype=np.int8)
    w[0, :5] = 1
    w[1, :4] = 1
    assert O.count_semi(w)["flag_semi"] == 1
    w[1, 3] = 0  # 8 nonzeros in 5 blocks: below the limit
    assert O.count_semi(w)["flag_semi"] == 0
    # a single row is semi for the pass (no pairs: 0 >= 0) but not for the
    # unit test's copy of the rule
    one = np.ones((1, 3), dtype=np.float32)
    assert O.count_semi(one, False)["flag_semi"] == 1
    assert O.count_semi(one, True)["flag_semi"] == 0


def test_all_zero_matrix():
    for dtype in (np.float32, np.int8):
        w = np.zeros((4, 5), dtype=dtype)
        for layout in (O.LAYOUT_UNPADDED, O.LAYOUT_PADDED, O.LAYOUT_SEMI):
            pk = O.pack(w, 9, layout)
            assert pk.first_ic == 0
            assert pk.nonzero_weights.size == 0 and pk.diffs.size == 0
            assert not pk.oc_nonzeros.any()
            assert np.array_equal(O.decode(pk), w)
