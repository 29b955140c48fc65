"""GPU parity of the HIP SpMM against the CPU oracle, through the C ABI.

Integer-valued inputs (the reference's own test distribution, test/test.spmm.blockwise.cu and
cuda_array.h:62-66) must match the oracle bit for bit after one fp16 rounding: this is the
check of index, padding and permutation handling.  Float inputs are held to the stated
tolerances.
"""
import numpy as np
import pytest

import shflbw_sparse_nn_amd as S
from oracle import oracle as O
import workloads as P
from workloads import float_error_report, run_spmm

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2        # max relative error on elements that are not near-cancelled (north star)
SCALED_TOL = 2.0 ** -9  # |err| / sum|a b|: one fp16 rounding (2^-11) plus fp32 summation order


def _exact_case(torch, M, N, K, V, d, permute, variant=-1, seed=2021):
    w = P.make_weight(M, K, V, d, permute, seed, integer=True)
    B = P.make_dense(K, N, seed, integer=True)
    ref = O.float_to_half(P.spmm_oracle(w, B))
    got = run_spmm(torch, w, B, variant=variant)
    assert not np.isnan(got.astype(np.float32)).any(), "kernel left output elements unwritten"
    np.testing.assert_array_equal(got.view(np.uint16), ref.view(np.uint16))


# the reference's own test case: N = 960 exercises the column-residue path
@pytest.mark.parametrize("V", [16, 32, 64, 128])
@pytest.mark.parametrize("permute", [False, True])
def test_reference_case_all_variants(torch_gpu, V, permute):
    for variant in range(len(S.spmm_variants(V))):
        print("variant", variant, S.spmm_variants(V)[variant], flush=True)
        _exact_case(torch_gpu, 1024, 960, 1024, V, 0.1, permute, variant)


@pytest.mark.parametrize("M,N,K,V,d", [
    (64, 8, 16, 64, 1.0),       # one panel, one partial k-step, tiny N
    (128, 264, 96, 32, 0.5),    # N residue of 8
    (256, 512, 200, 64, 0.03),  # panels with very few (possibly zero) vectors
    (256, 128, 1024, 128, 0.3),
    (512, 1032, 777, 32, 0.2),  # K not a multiple of anything
    (1024, 1024, 1024, 64, 0.25),  # cfg0 shape
    (48, 72, 40, 16, 0.7),      # block height 16: three panels, ragged N and K
    (512, 1000, 513, 16, 0.15),
    (33728, 1056, 128, 64, 0.05),  # tall weight of the reference's sweep list (527 panels, three column tiles)
    (4096, 128, 512, 32, 0.1),     # N smaller than a column tile
    (2048, 6400, 64, 64, 0.5),     # short panels (2 stages), many column tiles: tile switches dominate
    # more than 2.5 MB of B under a column tile and several tiles per workgroup: every second tile is
    # walked from its last stage to its first (odd stage counts, partial last groups)
    (8192, 1536, 4096, 32, 0.05),
    (4096, 1024, 4096, 16, 0.03),
    (8192, 2048, 3000, 64, 0.06),
    (4096, 2048, 4096, 128, 0.07),
    (4096, 4096, 8192, 128, 0.05),  # 128 x 256 tiles, two per workgroup, the second walked backwards
])
def test_exact_shapes(torch_gpu, M, N, K, V, d):
    _exact_case(torch_gpu, M, N, K, V, d, True)


@pytest.mark.parametrize("V", [32, 64])
def test_narrow_tiles_on_a_large_problem(torch_gpu, V):
    # the 256-column role-split variant is the library's choice for small problems only; forced here on a
    # problem with two to four tiles per workgroup and 3 MB of B under a column tile (backwards walk on)
    names = S.spmm_variants(V)
    narrow = [i for i, n in enumerate(names) if n.startswith("ws%dx64x4c4p" % V)]
    assert narrow, names
    for variant in narrow:
        print("variant", variant, names[variant], flush=True)
        _exact_case(torch_gpu, 4096, 2048, 6144, V, 0.06, True, variant)


def test_dense_density_is_permuted_gemm(torch_gpu):
    # d = 1.0: a plain dense GEMM with permuted output rows
    M, N, K, V = 128, 256, 128, 64
    w = P.make_weight(M, K, V, 1.0, True, 7, integer=True)
    B = P.make_dense(K, N, 7, integer=True)
    got = run_spmm(torch_gpu, w, B).astype(np.float32)
    A = O.densify(w)
    np.testing.assert_array_equal(got, (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32))


def test_empty_panels_write_zeros(torch_gpu):
    M, N, K, V = 256, 128, 64, 64
    X = M // V
    indptr = np.array([0, 0, 3, 3, 3], dtype=np.int32)  # only panel 1 keeps vectors
    indices = np.array([1, 5, 63], dtype=np.int32)
    rng = np.random.default_rng(3)
    w = dict(nrow=M, ncol=K, brow=V, bcol=1, nnzb=3, indptr=indptr, indices=indices,
             values=rng.integers(-4, 5, size=3 * V).astype(np.float16), row_permute_ids=O.row_permutation(M, 5))
    B = P.make_dense(K, N, 3, integer=True)
    got = run_spmm(torch_gpu, w, B)
    ref = O.float_to_half(P.spmm_oracle(w, B))
    np.testing.assert_array_equal(got.view(np.uint16), ref.view(np.uint16))
    assert X == 4 and (got[np.sort(w["row_permute_ids"][:V])] == 0).all()


@pytest.mark.parametrize("V", [16, 32, 64, 128])
@pytest.mark.parametrize("permute", [False, True])
def test_beta_c_epilogue(torch_gpu, permute, V):
    # D = A*B + C, the overload the reference's example uses (example/spmm.blockwise.cu:50)
    M, N, K = 256, 256, 256
    w = P.make_weight(M, K, V, 0.2, permute, 11, integer=True)
    B = P.make_dense(K, N, 11, integer=True)
    Cm = P.make_dense(M, N, 11, integer=True, stream=3)
    got = run_spmm(torch_gpu, w, B, Cmat=Cm)
    ref = O.float_to_half(P.spmm_oracle(w, B, Cm, 1.0, 1.0))
    np.testing.assert_array_equal(got.view(np.uint16), ref.view(np.uint16))
    got2 = run_spmm(torch_gpu, w, B, Cmat=Cm, alpha=2.0, beta=-0.5)
    ref2 = O.float_to_half(P.spmm_oracle(w, B, Cm, 2.0, -0.5))
    np.testing.assert_array_equal(got2.view(np.uint16), ref2.view(np.uint16))


@pytest.mark.parametrize("V,M,K,N", [(16, 256, 256, 256), (32, 1024, 520, 2048), (64, 512, 384, 512), (128, 256, 256, 256)])
def test_beta_c_epilogue_float_values(torch_gpu, V, M, K, N):
    """With beta != 0 the library rounds twice: h = fp16(alpha * acc) goes through the staging area, then
    D = fp16(float(h) + beta * C).  (The reference rounds the accumulator to fp16 as well, common/mma.h:336-339, and
    then forms alpha * h + beta * C in half arithmetic, common/epilogue.h:58-62.)  The oracle rounds
    alpha * acc + beta * C once; the two differ by at most the first rounding, half an fp16 ulp of alpha * acc
    (2^-11 relative), plus one fp16 ulp of the result (2^-10 relative) where that moves the last rounding."""
    w = P.make_weight(M, K, V, 0.2, True, 12, dist=("uniform", 1.0))
    B = P.make_dense(K, N, 12, dist=("uniform", 1.0))
    Cm = P.make_dense(M, N, 12, dist=("normal", 4.0), stream=3)
    alpha, beta = 1.5, -0.75
    ref = P.spmm_oracle(w, B, Cm, alpha, beta)      # fp32, one rounding to come
    prod = P.spmm_oracle(w, B, None, alpha, 0.0)    # alpha * A * B alone
    for variant in range(len(S.spmm_variants(V))):
        name = S.spmm_variants(V)[variant]
        if name.startswith("slab") and K > 1128:
            continue
        got = run_spmm(torch_gpu, w, B, Cmat=Cm, alpha=alpha, beta=beta, variant=variant).astype(np.float32)
        tol = 2.0 ** -11 * np.abs(prod) + 2.0 ** -10 * np.abs(ref) + 2.0 ** -24
        # summation order of the variant against the oracle's: a few fp32 ulps of sum |a b|, far below the above
        tol += 2.0 ** -20 * P.abs_products_bound(w, B) * abs(alpha)
        bad = np.abs(got - ref) > tol
        assert not bad.any(), "%s: %d elements off by more than the two roundings allow" % (name, int(bad.sum()))


@pytest.mark.parametrize("name", ["cfg0", "cfg1", "cfg2"])
def test_graded_configs(torch_gpu, name):
    c = P.SPMM_CONFIGS[name]
    # integer twin: bit exact
    _exact_case(torch_gpu, c["M"], c["N"], c["K"], c["V"], c["d"], True)
    # float inputs as specified
    w = P.make_weight(c["M"], c["K"], c["V"], c["d"], True, 2021, dist=c["a_dist"])
    B = P.make_dense(c["K"], c["N"], 2021, dist=c["b_dist"])
    ref = P.spmm_oracle(w, B)
    got = run_spmm(torch_gpu, w, B)
    rel, scaled = float_error_report(got, ref, P.abs_products_bound(w, B))
    print(name, "max rel err (|ref| >= 1e-2 rms):", rel, " max err / sum|ab|:", scaled, flush=True)
    assert rel <= REL_TOL
    assert scaled <= SCALED_TOL


def test_linearity_full_size(torch_gpu):
    # size-independent property at the headline size: A*(B1 + B2) == A*B1 + A*B2, exactly.
    # B1 and B2 have disjoint supports and entries in {-1, 0, 1}, A has integers in [-4, 4]:
    # every sum stays below 2048 in magnitude, so all three results are exact in fp16.
    c = P.SPMM_CONFIGS["cfg1"]
    w = P.make_weight(c["M"], c["K"], c["V"], c["d"], True, 2021, integer=True)
    assert 4 * int(np.max(np.diff(w["indptr"]))) < 2048
    rng = np.random.default_rng(99)
    X = rng.integers(-1, 2, size=(c["K"], c["N"]))
    sel = rng.integers(0, 2, size=(c["K"], c["N"]))
    B1 = (X * sel).astype(np.float16)
    B2 = (X * (1 - sel)).astype(np.float16)
    d1 = run_spmm(torch_gpu, w, B1).astype(np.float32)
    d2 = run_spmm(torch_gpu, w, B2).astype(np.float32)
    d12 = run_spmm(torch_gpu, w, (B1 + B2).astype(np.float16)).astype(np.float32)
    np.testing.assert_array_equal(d12, d1 + d2)


@pytest.mark.parametrize("V", [16, 32, 64, 128])
def test_non_finite_activations_do_not_leak_through_padding(torch_gpu, V):
    """A panel's kept vectors are padded to whole groups of 64 slots with zero weights.  The padding gathers a row
    of zeros, not a row of B, so an Inf or NaN in B reaches exactly the outputs it reaches in the reference: rows
    of panels that keep that column.  Every tile variant; panel sizes that leave 1 .. 63 padding slots."""
    M, K, N = 4 * V, 192, 520
    w = P.make_weight(M, K, V, 0.3, True, 77, integer=True)
    w["values"] = np.where(w["values"] == 0, np.float16(1), w["values"]).astype(np.float16)  # 0 * inf is NaN in the reference too
    B = P.make_dense(K, N, 78, integer=True).astype(np.float16)
    B[5, :] = np.inf
    B[77, 3::7] = -np.inf
    B[130, 1::5] = np.nan
    B[K - 1, :] = np.inf  # the largest column id: what a repeated last id would have hit
    with np.errstate(invalid="ignore", over="ignore"):
        ref = O.float_to_half(P.spmm_oracle(w, B))
    for variant in range(len(S.spmm_variants(V))):
        got = run_spmm(torch_gpu, w, B, variant=variant)
        assert np.array_equal(np.isnan(got), np.isnan(ref)), "variant %d: NaN pattern differs" % variant
        ok = ~np.isnan(ref)
        np.testing.assert_array_equal(got[ok], ref[ok], err_msg="variant %d" % variant)


def _slab_variant(V):
    names = S.spmm_variants(V)
    hits = [i for i, n in enumerate(names) if n.startswith("slab")]
    assert len(hits) == 1, names
    return hits[0]


@pytest.mark.parametrize("M,N,K,V,d,permute", [
    (4096, 4096, 1024, 32, 0.2, True),    # cfg2 shape: four workgroups per column tile, four panels per wave
    (1024, 960, 1024, 32, 0.1, True),     # ragged N: the last column tile is half empty
    (2048, 1024, 777, 32, 0.15, False),   # K not a multiple of 8: filler rows between the last row and the zeros
    (64, 64, 8, 32, 1.0, True),           # one column tile, two panels, one step each
    (256, 24000, 96, 32, 0.5, True),      # more column tiles than compute units: workgroups refill the slab
    (8192, 128, 1128, 32, 0.05, True),    # the largest K the LDS takes; 256 panels over two column tiles
    (4096, 512, 512, 32, 0.02, True),     # about ten kept vectors a panel: groups with one to three steps, empty panels
    (96, 8, 40, 32, 0.6, True),           # N smaller than a piece of the second 32-column block
])
def test_slab_variant_exact(torch_gpu, M, N, K, V, d, permute):
    """The variant that keeps all rows of a 64-column slab of B in LDS (weights of few columns), forced here on
    shapes that exercise its job loop, its group stream across panels and its row of zeros."""
    _exact_case(torch_gpu, M, N, K, V, d, permute, _slab_variant(V))


def test_slab_variant_empty_panels_and_c(torch_gpu):
    V = 32
    M, N, K = 8 * V, 200, 128
    X = M // V
    counts = np.array([0, 0, 5, 0, 70, 1, 0, 0])  # leading, inner and trailing panels without a kept vector
    indptr = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    rng = np.random.default_rng(5)
    indices = np.concatenate([np.sort(rng.choice(K, c, replace=False)) for c in counts]).astype(np.int32)
    w = dict(nrow=M, ncol=K, brow=V, bcol=1, nnzb=int(counts.sum()), indptr=indptr, indices=indices,
             values=rng.integers(-4, 5, size=int(counts.sum()) * V).astype(np.float16),
             row_permute_ids=O.row_permutation(M, 5))
    assert X == len(counts)
    B = P.make_dense(K, N, 3, integer=True)
    Cm = P.make_dense(M, N, 3, integer=True, stream=3)
    v = _slab_variant(V)
    got = run_spmm(torch_gpu, w, B, variant=v)
    np.testing.assert_array_equal(got.view(np.uint16), O.float_to_half(P.spmm_oracle(w, B)).view(np.uint16))
    got = run_spmm(torch_gpu, w, B, Cmat=Cm, alpha=2.0, beta=-0.5, variant=v)
    np.testing.assert_array_equal(got.view(np.uint16), O.float_to_half(P.spmm_oracle(w, B, Cm, 2.0, -0.5)).view(np.uint16))


def test_slab_variant_refuses_wide_weights(torch_gpu):
    from shflbw_sparse_nn_amd import capi
    w = P.make_weight(64, 2048, 32, 0.1, True, 1, integer=True)
    B = P.make_dense(2048, 64, 1, integer=True)
    with pytest.raises(capi.ShflbwError) as e:
        run_spmm(torch_gpu, w, B, variant=_slab_variant(32))
    assert e.value.status == capi.ERR_UNSUPPORTED


def test_slab_variant_seeded_random_shapes(torch_gpu):
    """Thirty small seeded shapes (ragged N, K not a multiple of 8, densities from nearly empty to full, permuted or
    not, with and without C): every one bit-exact against the oracle."""
    rng = np.random.default_rng(20211)
    v = _slab_variant(32)
    for case in range(30):
        M = 32 * int(rng.integers(1, 20))
        K = int(rng.integers(1, 400))
        N = 8 * int(rng.integers(1, 60))
        d = float(rng.choice([0.02, 0.1, 0.3, 0.6, 1.0]))
        permute = bool(rng.integers(0, 2))
        with_c = bool(rng.integers(0, 2))
        print("case", case, (M, N, K, d, permute, with_c), flush=True)
        w = P.make_weight(M, K, 32, d, permute, 100 + case, integer=True)
        B = P.make_dense(K, N, 100 + case, integer=True)
        Cm = P.make_dense(M, N, 100 + case, integer=True, stream=3) if with_c else None
        got = run_spmm(torch_gpu, w, B, Cmat=Cm, variant=v)
        ref = O.float_to_half(P.spmm_oracle(w, B, Cm, 1.0, 1.0) if with_c else P.spmm_oracle(w, B))
        np.testing.assert_array_equal(got.view(np.uint16), ref.view(np.uint16), err_msg="case %d" % case)


def test_library_choice_seeded_random_shapes(torch_gpu):
    """Forty seeded shapes over every block height with the variant the library picks (tiles of 128, 256 or 512 columns
    by the size of the problem, the slab kernel where it applies): ragged N, K not a multiple of anything, densities
    from nearly empty to full, permuted or not, with and without C and a scale: bit-exact against the oracle."""
    import shflbw_sparse_nn_amd as S
    rng = np.random.default_rng(31415)
    seen = set()
    for case in range(40):
        V = int(rng.choice([16, 32, 64, 128]))
        M = V * int(rng.integers(1, 24))
        K = int(rng.integers(1, 700))
        N = 8 * int(rng.integers(1, 400))
        d = float(rng.choice([0.02, 0.1, 0.3, 0.6, 1.0]))
        permute = bool(rng.integers(0, 2))
        with_c = bool(rng.integers(0, 2))
        alpha = float(rng.choice([1.0, 2.0, -0.5]))
        w = P.make_weight(M, K, V, d, permute, 500 + case, integer=True)
        B = P.make_dense(K, N, 500 + case, integer=True)
        Cm = P.make_dense(M, N, 500 + case, integer=True, stream=3) if with_c else None
        m = P.upload_weight(w)
        dB = P.to_dev(torch_gpu, B)
        dC = None if Cm is None else P.to_dev(torch_gpu, Cm)
        dD = torch_gpu.full((M, N), float("nan"), dtype=torch_gpu.float16, device="cuda")
        op = S.SpmmBlockwiseOp()
        st = op.initialize(m, N, dB.data_ptr(), dD.data_ptr(), None if dC is None else dC.data_ptr(), alpha, 1.0 if with_c else 0.0)
        name = S.spmm_variants(V)[st.variant]
        seen.add(name)
        print("case", case, (M, N, K, V, d, permute, with_c, alpha), name, flush=True)
        op(torch_gpu.cuda.current_stream().cuda_stream)
        torch_gpu.cuda.synchronize()
        ref = O.float_to_half(P.spmm_oracle(w, B, Cm, alpha, 1.0) if with_c else P.spmm_oracle(w, B, None, alpha, 0.0))
        np.testing.assert_array_equal(dD.cpu().numpy().view(np.uint16), ref.view(np.uint16), err_msg="case %d" % case)
    print("variants met:", sorted(seen), flush=True)
    assert len(seen) >= 6

