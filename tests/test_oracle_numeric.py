"""Pins the oracle's SpMM / SpConv host references with checks the mathematics fixes: the
hand-worked examples of the reference's format document, dense GEMM on the densified matrix,
brute force on tiny inputs, special cases, and torch's dense convolution."""
import numpy as np
import pytest

from oracle import oracle as O
import workloads as P

# example/spmatrix_dump_load.md:22-41 (plain) and :66-91 (with row permutation 0 3 1 2)
DOC_PLAIN = """4\n4\n2\n2\n2\n0\n0 1 2\n0 1\n1 2 1 2 3 1 1 2\n"""
DOC_PERMUTED = """4 # rows\n4\n2\n2\n2\n1\n0 1 2 # offsets\n0 1\n1 2 1 2 3 1 1 2\n0 3 1 2 # permutation\n"""


def test_format_document_examples():
    m = O.parse_dump(DOC_PLAIN)
    assert np.array_equal(O.densify(m), [[1, 1, 0, 0], [2, 2, 0, 0], [0, 0, 3, 1], [0, 0, 1, 2]])
    mp = O.parse_dump(DOC_PERMUTED)
    # "row_permute_id[i] = j: the i-th row of the block-wise matrix is the j-th row of the matrix we save"
    assert np.array_equal(O.densify(mp), [[1, 1, 0, 0], [0, 0, 3, 1], [0, 0, 1, 2], [2, 2, 0, 0]])
    B = np.arange(1, 13, dtype=np.float16).reshape(4, 3)
    for m_ in (m, mp):
        D = O.spmm_reference(4, 4, 2, 2, m_["indptr"], m_["indices"], m_["values"], m_["row_permute_ids"], 3, B)
        assert np.array_equal(D, O.densify(m_) @ B.astype(np.float32))


def _brute(w, B):
    M, N, V = w["nrow"], B.shape[1], w["brow"]
    D = np.zeros((M, N), dtype=np.float64)
    vals = w["values"].astype(np.float64)
    for i in range(M // V):
        for p in range(w["indptr"][i], w["indptr"][i + 1]):
            k = w["indices"][p]
            for r in range(V):
                row = i * V + r
                if w["row_permute_ids"] is not None:
                    row = w["row_permute_ids"][row]
                D[row] += vals[p * V + r] * B[k].astype(np.float64)
    return D


@pytest.mark.parametrize("V,M,K,N,d,perm", [(16, 32, 32, 8, 0.5, True), (32, 64, 48, 24, 0.3, False),
                                            (64, 128, 40, 16, 1.0, True), (16, 48, 16, 8, 0.0, True)])
def test_spmm_brute_force_and_dense(V, M, K, N, d, perm):
    w = P.make_weight(M, K, V, d, perm, 5, integer=True)
    B = P.make_dense(K, N, 5, integer=True)
    D = P.spmm_oracle(w, B)
    assert np.array_equal(D, _brute(w, B))                       # exact on integers
    assert np.array_equal(D, O.densify(w).astype(np.float64) @ B.astype(np.float64))
    # identity permutation equals the non-permuted path
    w_id = dict(w, row_permute_ids=np.arange(M, dtype=np.int32))
    w_no = dict(w, row_permute_ids=None)
    assert np.array_equal(P.spmm_oracle(w_id, B), P.spmm_oracle(w_no, B))


def test_spmm_alpha_beta_and_threads():
    w = P.make_weight(128, 96, 32, 0.4, True, 9)
    B = P.make_dense(96, 40, 9)
    Cm = P.make_dense(128, 40, 9, stream=3)
    base = P.spmm_oracle(w, B)
    got = P.spmm_oracle(w, B, Cm, 0.5, -2.0)
    assert np.array_equal(got, base * np.float32(0.5) + Cm.astype(np.float32) * np.float32(-2.0))
    # threads only split independent rows: bit-identical for any thread count
    assert np.array_equal(P.spmm_oracle(w, B, nthreads=1), P.spmm_oracle(w, B, nthreads=5))
    # fp32 accumulation in ascending kept-k order, checked against an explicit fp32 loop on one row
    A = O.densify(w)
    r = int(w["row_permute_ids"][7])
    acc = np.zeros(40, dtype=np.float32)
    for k in w["indices"][w["indptr"][0]:w["indptr"][1]]:
        acc = acc + np.float32(A[r, k]) * B[k].astype(np.float32)
    assert np.array_equal(base[r], acc)


def test_half_conversion_exhaustive():
    h = np.arange(65536, dtype=np.uint16)
    f = O.half_to_float(h)
    ref = h.view(np.float16).astype(np.float32)
    assert np.array_equal(f.view(np.uint32)[~np.isnan(ref)], ref.view(np.uint32)[~np.isnan(ref)])
    back = O.float_to_half(f).view(np.uint16)
    ok = ~np.isnan(ref)
    assert np.array_equal(back[ok], h[ok])
    # round to nearest even on fp32 inputs between representable halves
    x = np.array([1.0 + 2 ** -11, 1.0 + 3 * 2 ** -11, 65519.9, 65520.0, 2 ** -25, 2 ** -25 * 1.0001, -2049.0, 2051.0],
                 dtype=np.float32)
    assert np.array_equal(O.float_to_half(x).view(np.uint16), x.astype(np.float16).view(np.uint16))


def test_meta_packing_closed_form():
    # sections rounded up to 8 ints: X=8 panels, nnzb=128, M=128 -> (16 + 128 + 128) ints = 1088 bytes
    nnzb, indptr, indices = O.random_mask(128, 64, 16, 1, 0.25, 7)
    perm = O.row_permutation(128, 7)
    meta, o1, o2 = O.pack_meta(128, 16, 1, indptr, indices, perm)
    assert nnzb == 128 and meta.size * 4 == 1088 and (o1, o2) == (16, 144)
    assert np.array_equal(meta[:9], indptr) and np.all(meta[9:16] == 0)
    assert np.array_equal(meta[o1:o1 + 128], indices) and np.array_equal(meta[o2:], perm)
    meta2, _, _ = O.pack_meta(128, 16, 1, indptr, indices, None)
    assert meta2.size == 16 + 128


def _conv_brute(w, R, S, C, x, stride):
    Bn, H, W, _ = x.shape
    F, V = w["nrow"], w["brow"]
    A = O.densify(w).reshape(F, R, S, C).astype(np.float64)
    Ho, Wo = (H + 2 * (R // 2) - R) // stride + 1, (W + 2 * (S // 2) - S) // stride + 1
    y = np.zeros((Bn, Ho, Wo, F))
    xp = np.zeros((Bn, H + 2 * (R // 2), W + 2 * (S // 2), C))
    xp[:, R // 2:R // 2 + H, S // 2:S // 2 + W] = x
    for ho in range(Ho):
        for wo in range(Wo):
            patch = xp[:, ho * stride:ho * stride + R, wo * stride:wo * stride + S, :]
            y[:, ho, wo, :] = np.einsum("brsc,frsc->bf", patch, A)
    return y


@pytest.mark.parametrize("stride,H,W,R,S", [(1, 6, 5, 3, 3), (2, 8, 7, 3, 3), (1, 4, 4, 1, 1), (2, 9, 9, 5, 3)])
def test_conv_nhwc_brute_force(stride, H, W, R, S):
    C, F, V, Bn = 8, 32, 16, 2
    w = P.make_weight(F, R * S * C, V, 0.4, True, 3, integer=True)
    x = np.random.default_rng(4).integers(-4, 5, size=(Bn, H, W, C)).astype(np.float16)
    got = P.conv_oracle(w, R, S, C, x, stride)
    assert np.array_equal(got, _conv_brute(w, R, S, C, x, stride))


def test_conv_nhwc_against_torch_conv2d():
    import torch
    C, F, V, Bn, H, W, R, S = 16, 64, 32, 3, 10, 9, 3, 3
    w = P.make_weight(F, R * S * C, V, 0.3, True, 8, integer=True)
    x = np.random.default_rng(5).integers(-4, 5, size=(Bn, H, W, C)).astype(np.float16)
    Wd = torch.from_numpy(O.densify(w).reshape(F, R, S, C)).permute(0, 3, 1, 2).double()  # F C R S
    xin = torch.from_numpy(x.astype(np.float64)).permute(0, 3, 1, 2)
    for stride in (1, 2):
        ref = torch.nn.functional.conv2d(xin, Wd, stride=stride, padding=(R // 2, S // 2)).permute(0, 2, 3, 1).numpy()
        assert np.array_equal(P.conv_oracle(w, R, S, C, x, stride), ref)


def test_conv_reference_layout_equals_nhwc_at_stride_1():
    # the reference's own C-H-W-B / F-H-W-B host reference and the NHWC restatement agree where both
    # are defined (stride 1, "same" padding): they differ only in tensor layout
    C, F, V, Bn, H, W, R, S = 8, 32, 16, 4, 5, 6, 3, 3
    w = P.make_weight(F, R * S * C, V, 0.5, True, 2, integer=True)
    x = np.random.default_rng(6).integers(-4, 5, size=(Bn, H, W, C)).astype(np.float16)
    nhwc = P.conv_oracle(w, R, S, C, x, 1)
    chwb = O.spconv_reference_chwb(F, R, S, C, V, 1, w["indptr"], w["indices"], w["values"], w["row_permute_ids"],
                                   Bn, H, W, 1, np.ascontiguousarray(x.transpose(3, 1, 2, 0)))
    assert np.array_equal(chwb.transpose(3, 1, 2, 0), nhwc)


@pytest.mark.parametrize("stride", [2, 3])
@pytest.mark.parametrize("permute", [False, True])
def test_conv_reference_layout_brute_force_at_larger_strides(stride, permute):
    """The reference's bounds rule at stride > 1 (spconv/blockwise_format.h:97-128): the OUTPUT grid is H x W too, and
    out[f, ho, wo, b] = sum w[f, r, t, c] * in[c, ho*stride - R/2 + r, wo*stride - S/2 + t, b] with every tap outside
    H x W reading zero.  A restatement that used H / stride outputs, dropped the stride or swapped the filter extents
    fails here (5 x 3 filter, H != W)."""
    C, F, V, Bn, H, W, R, S = 6, 32, 16, 8, 7, 9, 5, 3
    w = P.make_weight(F, R * S * C, V, 0.5, permute, 21, integer=True)
    x = np.random.default_rng(22).integers(-4, 5, size=(C, H, W, Bn)).astype(np.float16)
    A = O.densify(w).reshape(F, R, S, C).astype(np.float64)
    y = np.zeros((F, H, W, Bn))
    xd = x.astype(np.float64)
    for ho in range(H):
        for wo in range(W):
            for r in range(R):
                for t in range(S):
                    hi, wi = ho * stride - R // 2 + r, wo * stride - S // 2 + t
                    if 0 <= hi < H and 0 <= wi < W:
                        y[:, ho, wo, :] += A[:, r, t, :] @ xd[:, hi, wi, :]
    got = O.spconv_reference_chwb(F, R, S, C, V, 1, w["indptr"], w["indices"], w["values"], w["row_permute_ids"],
                                  Bn, H, W, stride, x)
    assert got.shape == (F, H, W, Bn)
    assert np.array_equal(got, y)
