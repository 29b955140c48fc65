"""Seeded Shfl-BW problems shared by the tests, the smoke check and the benchmark.

Mask and permutation come from the oracle's restatement of the reference generators
(seed 2021 is the reference's default, benchmark/argparse_util.h:31); value streams come
from numpy's PCG64 with fixed seeds.  `integer=True` gives the reference's own test
distribution, integers in [-4, 4] (spmm/blockwise_format.h:101, cuda_array.h:64), for which
every partial sum is exact in fp32 and the comparison is bit-exact.
"""
import numpy as np

from oracle import oracle as O


def _values(rng, n, dist, integer):
    if integer:
        return rng.integers(-4, 5, size=n).astype(np.float16)
    kind, scale = dist
    if kind == "uniform":
        return rng.uniform(-scale, scale, size=n).astype(np.float16)
    return (rng.standard_normal(n) * scale).astype(np.float16)


def make_weight(M, K, V, density, permute=True, seed=2021, integer=False, dist=("uniform", 1.0)):
    nnzb, indptr, indices = O.random_mask(M, K, V, 1, density, seed)
    perm = O.row_permutation(M, seed) if permute else None
    rng = np.random.default_rng(seed * 1000 + 1)
    values = _values(rng, nnzb * V, dist, integer)
    return dict(nrow=M, ncol=K, brow=V, bcol=1, nnzb=nnzb, indptr=indptr, indices=indices, values=values,
                row_permute_ids=perm)


def make_dense(rows, cols, seed=2021, integer=False, dist=("uniform", 1.0), stream=2):
    rng = np.random.default_rng(seed * 1000 + stream)
    return _values(rng, rows * cols, dist, integer).reshape(rows, cols)


def spmm_oracle(w, B, Cmat=None, alpha=1.0, beta=0.0, nthreads=0):
    return O.spmm_reference(w["nrow"], w["ncol"], w["brow"], w["bcol"], w["indptr"], w["indices"], w["values"],
                            w["row_permute_ids"], B.shape[1], B, alpha, Cmat, beta, nthreads)


def conv_oracle(w, R, S, Cc, x_nhwc, stride, nthreads=0):
    Bn, H, W, _ = x_nhwc.shape
    return O.spconv_reference_nhwc(w["nrow"], R, S, Cc, w["brow"], w["indptr"], w["indices"], w["values"],
                                   w["row_permute_ids"], Bn, H, W, stride, R // 2, S // 2, x_nhwc, nthreads)


def abs_products_bound(w, B):
    """sum_k |a_k * b_k| per output element (fp32): the scale against which fp32 summation
    order differences are measured."""
    wa = dict(w)
    wa["values"] = np.abs(w["values"])
    return spmm_oracle(wa, np.abs(B))


# the graded configurations (shape, block size, density, value distributions)
SPMM_CONFIGS = {
    "cfg0": dict(M=1024, K=1024, N=1024, V=64, d=0.25, a_dist=("uniform", 1.0), b_dist=("uniform", 1.0)),
    "cfg1": dict(M=4096, K=4096, N=4096, V=64, d=0.1, a_dist=("uniform", 1.0), b_dist=("uniform", 1.0)),
    "cfg2": dict(M=4096, K=1024, N=4096, V=32, d=0.2, a_dist=("normal", 0.02), b_dist=("normal", 1.0)),
}
CONV_CONFIGS = {
    "cfg3": dict(B=16, H=14, W=14, C=512, F=2048, R=3, S=3, stride=1, V=64, d=0.1, w_dist=("normal", 0.05),
                 x_dist=("normal", 1.0)),
    "cfg4": dict(B=32, H=28, W=28, C=256, F=512, R=3, S=3, stride=2, V=32, d=0.3, w_dist=("normal", 0.05),
                 x_dist=("normal", 1.0)),
}
