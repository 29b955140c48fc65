"""Seeded Shfl-BW problems and the device-side helpers shared by the benchmark, the smoke check and the tests.

Mask and permutation come from the oracle's restatement of the reference generators
(seed 2021 is the reference's default, benchmark/argparse_util.h:31); value streams come
from numpy's PCG64 with fixed seeds.  `integer=True` gives the reference's own test
distribution, integers in [-4, 4] (spmm/blockwise_format.h:101, cuda_array.h:64), for which
every partial sum is exact in fp32 and the comparison is bit-exact.
"""
import numpy as np

from oracle import oracle as O  # checker and CPU baseline only; never on the measured path


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


def conv_oracle_batch_first(w, R, S, Cc, x_chwb, stride):
    """The reference's loop nest on its own tensors: C-H-W-B in, F-H-W-B out, H and W bounding both."""
    _, H, W, Bn = x_chwb.shape
    return O.spconv_reference_chwb(w["nrow"], R, S, Cc, w["brow"], 1, w["indptr"], w["indices"], w["values"],
                                   w["row_permute_ids"], Bn, H, W, stride, x_chwb)


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
    # the reference's own test case on its own tensors (test/test.spconv.blockwise.cu:10-14: 128 x 14 x 14 x 256 -> 256,
    # 3 x 3, density 0.1): C-H-W-B input, F-H-W-B output, not one of the graded configurations
    "refconv": dict(B=128, H=14, W=14, C=256, F=256, R=3, S=3, stride=1, V=64, d=0.1, w_dist=("normal", 0.05),
                    x_dist=("normal", 1.0), layout="chwb"),
}


# ---------------------------------------------------------------------------------------
# device side: buffers through torch, calls through the C ABI (ctypes mirror in the package)
# ---------------------------------------------------------------------------------------
def _S():
    import shflbw_sparse_nn_amd as S  # raises when the HIP library has not been built
    return S


def to_dev(torch, a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.float16)
    return torch.from_numpy(a).cuda()


def to_host_f16(t):
    return t.cpu().view(t.dtype).numpy().astype(np.float16, copy=False)


def upload_weight(w, R=0, Sx=0, Cc=0, cls=None):
    m = (cls or _S().BlockwiseSpMatrix)()
    m.set(w["nrow"], w["ncol"], w["brow"], w["bcol"], w["indptr"], w["indices"], w["values"], w["row_permute_ids"],
          R, Sx, Cc)
    m.transform_and_sync_device()
    return m


def run_spmm(torch, w, B, Cmat=None, alpha=1.0, beta=None, variant=-1, poison=True):
    """D (numpy fp16, M x N) computed by the HIP library through the C ABI."""
    m = upload_weight(w)
    N = B.shape[1]
    dB = to_dev(torch, B)
    dC = None if Cmat is None else to_dev(torch, Cmat)
    # NaN-filled output: every element must be written by the kernel
    dD = torch.full((w["nrow"], N), float("nan"), dtype=torch.float16, device="cuda") if poison else \
        torch.zeros((w["nrow"], N), dtype=torch.float16, device="cuda")
    op = _S().SpmmBlockwiseOp(variant)
    op.initialize(m, N, dB.data_ptr(), dD.data_ptr(), None if dC is None else dC.data_ptr(), alpha, beta)
    op(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return dD.cpu().numpy()


def run_spconv(torch, w, R, Sx, Cc, x_nhwc, stride, variant=-1):
    f = upload_weight(w, R, Sx, Cc, cls=_S().BlockwiseSpFilter)
    Bn, H, W, _ = x_nhwc.shape
    dX = to_dev(torch, x_nhwc)
    op = _S().SpconvBlockwiseOp(variant)
    Ho = (H + 2 * (R // 2) - R) // stride + 1
    Wo = (W + 2 * (Sx // 2) - Sx) // stride + 1
    dY = torch.full((Bn, Ho, Wo, w["nrow"]), float("nan"), dtype=torch.float16, device="cuda")
    op.initialize(f, Bn, H, W, stride, dX.data_ptr(), dY.data_ptr())
    assert op.output_hw == (Ho, Wo)
    op(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    op.check()
    return dY.cpu().numpy()


def float_error_report(got_f16, ref_f32, bound_f32):
    """Two figures for float-valued inputs:
    rel: max |got - ref| / |ref| over elements with |ref| >= 1e-2 * rms(ref)  (north-star bar 1e-2)
    scaled: max |got - ref| / sum_k |a_k b_k|  (summation-order + one fp16 rounding; ~2^-10)"""
    got = got_f16.astype(np.float32)
    err = np.abs(got - ref_f32)
    rms = float(np.sqrt(np.mean(ref_f32.astype(np.float64) ** 2)))
    big = np.abs(ref_f32) >= 1e-2 * rms
    rel = float(np.max(err[big] / np.abs(ref_f32[big]))) if big.any() else 0.0
    scaled = float(np.max(err / np.maximum(bound_f32, 1e-30)))
    return rel, scaled
