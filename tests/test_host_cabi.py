"""CPU checks of the shipped library's host side through the C ABI: the shared library loads and
exports every symbol include/shflbw.h declares, and the host-side format code (mask, init_random,
dump/load, meta image, private image) matches the oracle and the golden fixtures.  No compute
entry point is called here (no GPU)."""
import ctypes as C
import hashlib
import json
import os
import re
import subprocess
import sys

import numpy as np
import pytest

import shflbw_sparse_nn_amd as S
from oracle import oracle as O
from shflbw_sparse_nn_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
G = json.load(open(os.path.join(ROOT, "tests", "golden", "golden.json")))


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def test_library_exports_every_declared_symbol():
    hdr = open(os.path.join(ROOT, "include", "shflbw.h")).read()
    declared = set(re.findall(r"^(?:int|void|const char\*)\s+(shflbw_[a-z_]+)\(", hdr, flags=re.M))
    assert declared == set(capi.EXPORTS), declared ^ set(capi.EXPORTS)
    lib = C.CDLL(capi.LIB_PATH)
    for name in sorted(declared):
        assert hasattr(lib, name), name
    # the static archive the reference's users link carries the same entry points
    syms = subprocess.check_output(["nm", "-g", "--defined-only", capi.ARCHIVE_PATH]).decode()
    for name in sorted(declared):
        assert re.search(r"\bT %s\b" % name, syms), name


def test_status_strings():
    lib = capi.load()
    assert lib.shflbw_status_string(0) == b"ok"
    assert len({lib.shflbw_status_string(i) for i in range(8)}) == 8


@pytest.mark.parametrize("case", G["ref_masks"], ids=lambda c: "x".join(str(a) for a in c["args"]))
def test_random_mask_matches_reference_vectors(case):
    nrow, ncol, brow, bcol, dens, seed, div, pad = case["args"]
    nnzb, indptr, indices = S.random_mask(nrow, ncol, brow, bcol, dens, seed, div, pad)
    assert nnzb == case["nnzb"] and sha(indptr) == case["indptr_sha256"] and sha(indices) == case["indices_sha256"]


def test_init_random_dump_equals_reference_dump():
    # fresh process: the value stream is the never-seeded rand(), exactly as in the reference's example
    code = ("import hashlib, shflbw_sparse_nn_amd as S\n"
            "m = S.BlockwiseSpMatrix(); m.init_random(1024, 1024, 32, 1, 0.2, False, 2021)\n"
            "t = m.dump().encode(); print(len(t), hashlib.sha256(t).hexdigest(), m.config_str)\n")
    out = subprocess.check_output([sys.executable, "-c", code], cwd=ROOT).decode().split(None, 2)
    assert int(out[0]) == G["dump"]["text_len"] and out[1] == G["dump"]["text_sha256"]
    assert out[2].strip() == "1024 1024 32 1 0.200012 2021 non-row-permute"


def test_init_random_permutation_and_filter():
    m = S.BlockwiseSpMatrix()
    m.init_random(4096, 4096, 64, 1, 0.1, True, 2021)
    p = [c for c in G["permutations"] if c["n"] == 4096 and c["seed"] == 2021][0]
    assert sha(m.row_permute_ids) == p["sha256"]
    assert m.nnzb == 26214 and abs(m.density - 26214 / 64 / 4096) < 1e-9 and m.row_permute and m.initialized
    nnzb, indptr, indices = O.random_mask(4096, 4096, 64, 1, 0.1, 2021)
    assert np.array_equal(m.indptr, indptr) and np.array_equal(m.indices, indices)
    assert set(np.unique(m.values.astype(np.float32))) <= set(range(-4, 5))
    f = S.BlockwiseSpFilter()
    f.init_random(64, 3, 3, 16, 32, 1, 0.25, True, 7)
    assert (f.nrow, f.ncol, f.F, f.R, f.S, f.C) == (64, 144, 64, 3, 3, 16)
    assert f.config_str == "64 3 3 16 32 1 %g 7 filter-permute " % f.density


def test_dump_load_round_trip_and_document_examples():
    from tests.test_oracle_numeric import DOC_PERMUTED, DOC_PLAIN
    m = S.BlockwiseSpMatrix()
    m.load("\n".join(l.split("#")[0] for l in DOC_PERMUTED.splitlines()))
    assert (m.nrow, m.ncol, m.nnzb, m.brow, m.bcol, m.row_permute) == (4, 4, 2, 2, 2, True)
    assert m.row_permute_ids.tolist() == [0, 3, 1, 2] and m.values.astype(np.float32).tolist() == [1, 2, 1, 2, 3, 1, 1, 2]
    assert m.dump() == "4\n4\n2\n2\n2\n1\n0 1 2 \n0 1 \n1 2 1 2 3 1 1 2 \n0 3 1 2 \n"
    m.load(DOC_PLAIN)
    assert m.row_permute_ids is None and m.dump() == "4\n4\n2\n2\n2\n0\n0 1 2 \n0 1 \n1 2 1 2 3 1 1 2 \n"
    a = S.BlockwiseSpMatrix()
    a.init_random(256, 192, 32, 1, 0.3, True, 5)
    b = S.BlockwiseSpMatrix()
    b.load(a.dump())
    for x, y in zip(a._arrays(), b._arrays()):
        assert np.array_equal(x, y)
    assert b.dump() == a.dump()
    assert O.parse_dump(a.dump())["indices"].tolist() == a.indices.tolist()


def test_error_statuses():
    m = S.BlockwiseSpMatrix()
    with pytest.raises(capi.ShflbwError) as e:
        m.init_random(100, 64, 32, 1, 0.5, False, 1)  # nrow % brow != 0 (assert in the reference)
    assert e.value.status == capi.ERR_SHAPE
    with pytest.raises(capi.ShflbwError) as e:
        m.dump()
    assert e.value.status == capi.ERR_STATE
    with pytest.raises(capi.ShflbwError) as e:
        m.transform_and_sync_device()
    assert e.value.status == capi.ERR_STATE
    with pytest.raises(capi.ShflbwError) as e:
        m.load("4 4 2 2 2 0 0 1")  # truncated
    assert e.value.status == capi.ERR_FORMAT
    ip = np.array([0, 1, 2], dtype=np.int32)
    with pytest.raises(capi.ShflbwError) as e:  # column index out of range
        m.set(32, 8, 16, 1, ip, np.array([0, 9], dtype=np.int32), np.zeros(32, dtype=np.float16))
    assert e.value.status == capi.ERR_FORMAT
    with pytest.raises(capi.ShflbwError) as e:  # not a permutation
        m.set(32, 8, 16, 1, ip, np.array([0, 7], dtype=np.int32), np.zeros(32, dtype=np.float16),
              np.zeros(32, dtype=np.int32))
    assert e.value.status == capi.ERR_FORMAT
    # spmm_init on a weight that was never synced: the reference asserts device_synced
    m.set(32, 8, 16, 1, ip, np.array([0, 7], dtype=np.int32), np.zeros(32, dtype=np.float16))
    op = S.SpmmBlockwiseOp()
    with pytest.raises(capi.ShflbwError) as e:
        op.initialize(m, 64, 4096, 8192)
    assert e.value.status == capi.ERR_STATE
    lib = capi.load()
    assert lib.shflbw_spmm_exec(C.byref(capi.SpmmState()), None) == capi.ERR_STATE
    assert lib.shflbw_spconv_exec(C.byref(capi.SpconvState()), None) == capi.ERR_STATE


def test_variant_table():
    for V in (32, 64, 128):
        names = S.spmm_variants(V)
        assert len(names) >= 1 and len(set(names)) == len(names)
    assert S.spmm_variants(48) == []


def test_static_archive_holds_the_operator_tables():
    """libblock_sparse.a must define, as unmangled data symbols, the Init/Exec function-pointer variable of
    every tile configuration named in the table file (the names a user of the reference links against,
    block_sparse/common/library_util.h:3-9), for SpMM and SpConv alike."""
    import re
    import subprocess
    pkg = os.path.join(ROOT, "shflbw_sparse_nn_amd")
    archive = os.path.join(pkg, "libblock_sparse.a")
    assert os.path.exists(archive), "build the library first (__graft_entry__.build())"
    tuples = []
    for line in open(os.path.join(pkg, "block_sparse", "common", "library_table.def")):
        m = re.match(r"SHFLBW_TILE\(([^)]*)\)", line.strip())
        if m:
            tuples.append([int(x) for x in m.group(1).split(",")])
    assert len(tuples) == 83
    syms = set()
    for line in subprocess.run(["nm", "--defined-only", archive], stdout=subprocess.PIPE, text=True,
                               check=True).stdout.splitlines():
        parts = line.split()
        if len(parts) == 3 and parts[1] in "DBd":
            syms.add(parts[2])
    for t in tuples:
        tag = "%dx%dx%d_%dx%dx%d_%dx%dx%d_%d" % tuple(t)
        for kind in ("SpmmBlockwise", "SpconvBlockwise"):
            for fn in ("Init", "Exec"):
                assert "%s_%s_%sFn" % (kind, tag, fn) in syms, (kind, tag, fn)


def test_state_struct_layout_matches_the_library():
    lib = capi.load()  # load() itself raises on a mismatch; spell the figures out here
    a, b = C.c_size_t(0), C.c_size_t(0)
    lib.shflbw_abi_sizes(C.byref(a), C.byref(b))
    assert (a.value, b.value) == (C.sizeof(capi.SpmmState), C.sizeof(capi.SpconvState))
    assert capi.SpmmState.ldb_bytes.offset == capi.SpmmState.brow.offset + 4


def test_spconv_forms_are_named():
    names = S.spconv_variants()
    assert len(names) >= 3 and len(set(names)) == len(names) and all(names)
    assert S.spconv_variant_name(len(names)) == ""


def test_set_with_equal_arrays_is_a_no_op():
    """dump() of the C++ veneer hands its public vectors back to the library first; when nothing changed
    the weight must keep its seed and config string (a changed one would mean the set went through
    and, on a synced weight, dropped the device image)."""
    m = S.BlockwiseSpMatrix()
    m.init_random(256, 128, 32, 1, 0.25, True, 99)
    cfg, seed = m.config_str, m.seed
    m.set(256, 128, 32, 1, m.indptr, m.indices, m.values, m.row_permute_ids)
    assert (m.config_str, m.seed) == (cfg, seed) and seed == 99
    v = m.values.copy()
    v[0] = v[0] + 1
    m.set(256, 128, 32, 1, m.indptr, m.indices, v, m.row_permute_ids)
    assert m.seed == 0  # a real change goes through


@pytest.mark.parametrize("V,permute", [(16, True), (32, False), (64, True)])
def test_library_spmm_host_reference_equals_the_oracle(V, permute):
    import workloads as P
    w = P.make_weight(128, 96, V, 0.3, permute, 5, dist=("normal", 1.0))
    B = P.make_dense(96, 40, 5, dist=("uniform", 1.0))
    Cm = P.make_dense(128, 40, 6, dist=("uniform", 1.0))
    m = S.BlockwiseSpMatrix()
    m.set(w["nrow"], w["ncol"], V, 1, w["indptr"], w["indices"], w["values"], w["row_permute_ids"])
    np.testing.assert_array_equal(m.host_reference(40, B), P.spmm_oracle(w, B))
    np.testing.assert_array_equal(m.host_reference(40, B, 0.5, Cm, -2.0), P.spmm_oracle(w, B, Cm, 0.5, -2.0))


@pytest.mark.parametrize("stride,R,Sx", [(1, 3, 3), (2, 3, 3), (2, 5, 1), (1, 1, 1)])
def test_library_spconv_host_reference_equals_the_oracle(stride, R, Sx):
    import workloads as P
    Cc, F, V = 16, 64, 32
    w = P.make_weight(F, R * Sx * Cc, V, 0.3, True, 11, dist=("normal", 1.0))
    x = np.random.default_rng(3).standard_normal((2, 9, 7, Cc)).astype(np.float16)
    f = S.BlockwiseSpFilter()
    f.set(F, R * Sx * Cc, V, 1, w["indptr"], w["indices"], w["values"], w["row_permute_ids"], R, Sx, Cc)
    np.testing.assert_array_equal(f.host_reference(x, stride), P.conv_oracle(w, R, Sx, Cc, x, stride))


@pytest.mark.parametrize("stride,R,Sx,permute", [(1, 3, 3, True), (2, 3, 3, True), (1, 5, 1, False)])
def test_library_reference_layout_host_reference_equals_the_oracle(stride, R, Sx, permute):
    import workloads as P
    Cc, F, V, Bn, H, W = 12, 64, 32, 8, 7, 6
    w = P.make_weight(F, R * Sx * Cc, V, 0.3, permute, 11, dist=("normal", 1.0))
    x = np.random.default_rng(4).standard_normal((Cc, H, W, Bn)).astype(np.float16)
    f = S.BlockwiseSpFilter()
    f.set(F, R * Sx * Cc, V, 1, w["indptr"], w["indices"], w["values"], w["row_permute_ids"], R, Sx, Cc)
    ref = O.spconv_reference_chwb(F, R, Sx, Cc, V, 1, w["indptr"], w["indices"], w["values"], w["row_permute_ids"],
                                  Bn, H, W, stride, x)
    np.testing.assert_array_equal(f.host_reference_chwb(x, stride), ref)
