"""The entry point that allocates nothing (shflbw_spconv_exec_static: scratch in a fixed device array) against
the existing pair shflbw_spconv_init + shflbw_spconv_exec: same kernels, so the outputs must be equal bit for
bit, also on float data.  Two calls in a row, the second on a smaller input (stale contents of the array from
the first call must not matter), then a third on the first input again; a problem whose scratch exceeds the
array is refused."""
import ctypes as C

import numpy as np
import pytest

import shflbw_sparse_nn_amd as S
import workloads as P
from shflbw_sparse_nn_amd import capi

pytestmark = pytest.mark.gpu


def _both(torch, f, w, x, stride, R, Sx):
    lib = capi.load()
    Bn, H, W, Cc = x.shape
    Ho, Wo = (H + 2 * (R // 2) - R) // stride + 1, (W + 2 * (Sx // 2) - Sx) // stride + 1
    dX = P.to_dev(torch, x)
    stream = torch.cuda.current_stream().cuda_stream
    # existing entry points
    dY0 = torch.full((Bn, Ho, Wo, w["nrow"]), float("nan"), dtype=torch.float16, device="cuda")
    op = S.SpconvBlockwiseOp(0)
    op.initialize(f, Bn, H, W, stride, dX.data_ptr(), dY0.data_ptr())
    op(stream)
    # the static one
    dY1 = torch.full((Bn, Ho, Wo, w["nrow"]), float("nan"), dtype=torch.float16, device="cuda")
    capi.check(lib.shflbw_spconv_exec_static(f._h, Bn, H, W, stride, dX.data_ptr(), dY1.data_ptr(), stream))
    torch.cuda.synchronize()
    return dY0.cpu().numpy(), dY1.cpu().numpy()


@pytest.mark.parametrize("V,stride", [(64, 1), (32, 2), (16, 1)])
def test_static_scratch_entry_equals_init_exec(torch_gpu, V, stride):
    torch = torch_gpu
    R = Sx = 3
    Cc, F = 64, 128
    w = P.make_weight(F, R * Sx * Cc, V, 0.25, True, 2021, dist=("normal", 0.05))
    f = P.upload_weight(w, R, Sx, Cc, cls=S.BlockwiseSpFilter)
    rng = np.random.default_rng(17)
    big = rng.standard_normal((6, 14 * stride, 14 * stride, Cc)).astype(np.float16)
    small = rng.standard_normal((2, 7 * stride, 9 * stride, Cc)).astype(np.float16)
    for x in (big, small, big):
        print("static conv", V, stride, x.shape, flush=True)
        y0, y1 = _both(torch, f, w, x, stride, R, Sx)
        assert not np.isnan(y1.astype(np.float32)).any()
        np.testing.assert_array_equal(y0.view(np.uint16), y1.view(np.uint16))
    # and against the oracle on integer data, so that "equal" cannot mean "equally wrong"
    wi = P.make_weight(F, R * Sx * Cc, V, 0.25, True, 2021, integer=True)
    fi = P.upload_weight(wi, R, Sx, Cc, cls=S.BlockwiseSpFilter)
    xi = rng.integers(-4, 5, size=(3, 8 * stride, 8 * stride, Cc)).astype(np.float16)
    from oracle import oracle as O
    _, y1 = _both(torch, fi, wi, xi, stride, R, Sx)
    ref = O.float_to_half(P.conv_oracle(wi, R, Sx, Cc, xi, stride))
    np.testing.assert_array_equal(y1.view(np.uint16), ref.view(np.uint16))


def test_static_scratch_entry_block_32_mid_sized_filter(torch_gpu):
    """Block height 32 with 384 <= R*S*C <= 1128 and many column tiles: the SpMM in the middle must be a gather variant
    (the variant that holds the rows of B in LDS cannot walk the planes), in the static entry and in init + exec."""
    from oracle import oracle as O
    R = Sx = 3
    Cc, F, V = 64, 512, 32
    w = P.make_weight(F, R * Sx * Cc, V, 0.25, True, 2021, integer=True)
    f = P.upload_weight(w, R, Sx, Cc, cls=S.BlockwiseSpFilter)
    x = np.random.default_rng(19).integers(-4, 5, size=(12, 28, 28, Cc)).astype(np.float16)
    y0, y1 = _both(torch_gpu, f, w, x, 1, R, Sx)
    ref = O.float_to_half(P.conv_oracle(w, R, Sx, Cc, x, 1))
    np.testing.assert_array_equal(y0.view(np.uint16), ref.view(np.uint16))
    np.testing.assert_array_equal(y1.view(np.uint16), ref.view(np.uint16))


def test_static_scratch_entry_refuses_what_does_not_fit(torch_gpu):
    torch = torch_gpu
    lib = capi.load()
    R = Sx = 3
    Cc, F, V = 256, 512, 32
    w = P.make_weight(F, R * Sx * Cc, V, 0.1, True, 2021, integer=True)
    f = P.upload_weight(w, R, Sx, Cc, cls=S.BlockwiseSpFilter)
    Bn, H, W = 64, 56, 56  # planes alone: 2 x 256 rows x ~215 000 positions x 2 bytes, far above the array
    dX = torch.zeros((Bn, H, W, Cc), dtype=torch.float16, device="cuda")
    dY = torch.zeros((Bn, H, W, F), dtype=torch.float16, device="cuda")
    rc = lib.shflbw_spconv_exec_static(f._h, Bn, H, W, 1, dX.data_ptr(), dY.data_ptr(), None)
    assert rc == capi.ERR_CAPACITY
    msg = lib.shflbw_last_error().decode()
    assert str(capi.STATIC_SCRATCH_BYTES) in msg
