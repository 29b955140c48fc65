"""Pins the CPU oracle's generators against fixtures that do not come from this repository:
the reference's own dump file, a build of the reference's own mask generator, and libstdc++'s
shuffle (tests/golden/make_golden.py says how golden.json was made)."""
import hashlib
import json
import os

import numpy as np
import pytest

from oracle import oracle as O

G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "golden.json")))


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def test_mask_reproduces_reference_dump():
    d = G["dump"]
    nrow, ncol, nnzb, brow, bcol, rp = d["header"]
    n, indptr, indices = O.random_mask(nrow, ncol, brow, bcol, 0.2, 2021)
    assert (n, rp) == (nnzb, 0) and n == d["indices_len"]
    assert indptr.tolist() == d["indptr"]
    assert indices[:32].tolist() == d["indices_head"]
    assert sha(indices) == d["indices_sha256"]


def test_value_stream_reproduces_reference_dump():
    d = G["dump"]
    v = O.reference_values(d["values_len"])
    assert v[:32].tolist() == d["values_head"]
    assert sha(v) == d["values_sha256"]
    assert set(np.unique(v)) <= set(range(-4, 5))
    # a second array filled by the same process continues the stream
    assert np.array_equal(O.reference_values(100, skip=50), O.reference_values(150)[50:])


@pytest.mark.parametrize("case", G["ref_masks"], ids=lambda c: "x".join(str(a) for a in c["args"]))
def test_mask_matches_reference_build(case):
    nrow, ncol, brow, bcol, dens, seed, div, pad = case["args"]
    nnzb, indptr, indices = O.random_mask(nrow, ncol, brow, bcol, dens, seed, div, pad)
    assert nnzb == case["nnzb"] and indices.size == case["indices_len"]
    assert sha(indptr) == case["indptr_sha256"] and sha(indices) == case["indices_sha256"]
    assert indices[:16].tolist() == case["indices_head"]
    # invariants of the format: sorted, unique, in range, prefix sums
    X = nrow // brow
    assert indptr[0] == 0 and indptr[X] == indices.size
    if pad == 1:
        for i in range(X):
            seg = indices[indptr[i]:indptr[i + 1]]
            assert np.all(np.diff(seg) > 0) and (seg.size == 0 or (seg[0] >= 0 and seg[-1] < ncol // bcol))


def test_mask_against_live_reference_build_if_present():
    if O.ref_lib() is None:
        pytest.skip("oracle/_ref not built here (reference tree absent); committed vectors cover it")
    for args in [(768, 640, 32, 1, 0.37, 99), (4096, 4096, 64, 1, 0.1, 2021), (96, 64, 16, 1, 0.5, 1)]:
        a = O.random_mask(*args)
        b = O.ref_random_mask(*args)
        assert a[0] == b[0] and np.array_equal(a[1], b[1]) and np.array_equal(a[2], b[2])


@pytest.mark.parametrize("case", G["permutations"], ids=lambda c: "n%d_s%d" % (c["n"], c["seed"]))
def test_permutation_matches_libstdcxx(case):
    p = O.row_permutation(case["n"], case["seed"])
    assert p[:16].tolist() == case["head"] and sha(p) == case["sha256"]
    assert np.array_equal(np.sort(p), np.arange(case["n"]))


def test_nnzb_is_float_arithmetic():
    # random_mask.cc:17 rounds block_density * X * Y evaluated in float
    for (nrow, ncol, brow, d, want) in [(1024, 1024, 64, 0.25, 4096), (4096, 4096, 64, 0.1, 26214),
                                         (4096, 1024, 32, 0.2, 26214), (2048, 4608, 64, 0.1, 14746),
                                         (512, 2304, 32, 0.3, 11059)]:
        assert O.mask_nnzb(nrow, ncol, brow, 1, d) == want
