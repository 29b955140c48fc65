"""Helpers for the GPU tests: device buffers through torch, calls through the C ABI."""
import numpy as np

import shflbw_sparse_nn_amd as S


def to_dev(torch, a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.float16)
    return torch.from_numpy(a).cuda()


def to_host_f16(t):
    return t.cpu().view(t.dtype).numpy().astype(np.float16, copy=False)


def upload_weight(w, R=0, Sx=0, Cc=0, cls=None):
    m = (cls or S.BlockwiseSpMatrix)()
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
    op = S.SpmmBlockwiseOp(variant)
    op.initialize(m, N, dB.data_ptr(), dD.data_ptr(), None if dC is None else dC.data_ptr(), alpha, beta)
    op(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return dD.cpu().numpy()


def run_spconv(torch, w, R, Sx, Cc, x_nhwc, stride, variant=0):
    f = upload_weight(w, R, Sx, Cc, cls=S.BlockwiseSpFilter)
    Bn, H, W, _ = x_nhwc.shape
    dX = to_dev(torch, x_nhwc)
    op = S.SpconvBlockwiseOp(variant)
    Ho = (H + 2 * (R // 2) - R) // stride + 1
    Wo = (W + 2 * (Sx // 2) - Sx) // stride + 1
    dY = torch.full((Bn, Ho, Wo, w["nrow"]), float("nan"), dtype=torch.float16, device="cuda")
    op.initialize(f, Bn, H, W, stride, dX.data_ptr(), dY.data_ptr())
    assert op.output_hw == (Ho, Wo)
    op(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
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
