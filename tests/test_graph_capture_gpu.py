"""`exec` is a pure launch (no allocation, no synchronisation, no memset): the reference calls it 111 times back to
back (benchmark/benchmark.spmm.cu:29-42), and a caller may record it into a HIP graph.  The SpMM launch and the
three launches of the convolution are captured once and replayed with new operand contents; every replay must
equal the eager result bit for bit, with eager work and synchronisation between the replays."""
import numpy as np
import pytest

import shflbw_sparse_nn_amd as S
from oracle import oracle as O
import workloads as P
from workloads import to_dev, upload_weight

pytestmark = pytest.mark.gpu


def _replays(torch, op, inputs, d_in, d_out, refs):
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    d_in.copy_(inputs[0])
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        op(side.cuda_stream)  # warm-up on the capture stream (module load, function attributes)
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        op(torch.cuda.current_stream().cuda_stream)
    for rnd in range(3):
        for i, x in enumerate(inputs):
            d_in.copy_(x)
            d_out.fill_(float("nan"))  # eager work between the replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            got = d_out.cpu().numpy()
            np.testing.assert_array_equal(got.view(np.uint16), refs[i].view(np.uint16), err_msg="replay %d/%d" % (rnd, i))


def test_spmm_exec_in_a_graph(torch_gpu):
    torch = torch_gpu
    M, K, N, V = 512, 512, 1024, 64
    w = P.make_weight(M, K, V, 0.2, True, 2021, integer=True)
    Bs = [P.make_dense(K, N, 2021 + i, integer=True) for i in range(2)]
    refs = [O.float_to_half(P.spmm_oracle(w, B)) for B in Bs]
    m = upload_weight(w)
    dB = torch.empty((K, N), dtype=torch.float16, device="cuda")
    dD = torch.empty((M, N), dtype=torch.float16, device="cuda")
    op = S.SpmmBlockwiseOp(-1)
    op.initialize(m, N, dB.data_ptr(), dD.data_ptr())
    _replays(torch, op, [to_dev(torch, B) for B in Bs], dB, dD, refs)


@pytest.mark.parametrize("variant", [0, 2, 3])  # three launches, batch-innermost three launches, one fused launch
def test_spconv_exec_in_a_graph(torch_gpu, variant):
    torch = torch_gpu
    Bn, H, W, C, F, R, Sx, stride, V = 8, 14, 14, 64, 128, 3, 3, 2, 64
    w = P.make_weight(F, R * Sx * C, V, 0.2, True, 2021, integer=True)
    xs = [np.random.default_rng(5 + i).integers(-4, 5, size=(Bn, H, W, C)).astype(np.float16) for i in range(2)]
    refs = [O.float_to_half(P.conv_oracle(w, R, Sx, C, x, stride)) for x in xs]
    f = upload_weight(w, R, Sx, C, cls=S.BlockwiseSpFilter)
    dX = torch.empty((Bn, H, W, C), dtype=torch.float16, device="cuda")
    dY = torch.empty(refs[0].shape, dtype=torch.float16, device="cuda")
    op = S.SpconvBlockwiseOp(variant)
    op.initialize(f, Bn, H, W, stride, dX.data_ptr(), dY.data_ptr())
    _replays(torch, op, [to_dev(torch, x) for x in xs], dX, dY, refs)


def test_slab_spmm_exec_in_a_graph(torch_gpu):
    torch = torch_gpu
    M, K, N, V = 1024, 520, 264, 32  # block height 32, few columns: the variant that keeps a slab of B in LDS
    w = P.make_weight(M, K, V, 0.2, True, 2021, integer=True)
    Bs = [P.make_dense(K, N, 2021 + i, integer=True) for i in range(2)]
    refs = [O.float_to_half(P.spmm_oracle(w, B)) for B in Bs]
    m = upload_weight(w)
    dB = torch.empty((K, N), dtype=torch.float16, device="cuda")
    dD = torch.empty((M, N), dtype=torch.float16, device="cuda")
    slab = [i for i, n in enumerate(S.spmm_variants(V)) if n.startswith("slab")][0]
    op = S.SpmmBlockwiseOp(slab)
    op.initialize(m, N, dB.data_ptr(), dD.data_ptr())
    _replays(torch, op, [to_dev(torch, B) for B in Bs], dB, dD, refs)


def test_reference_layout_spconv_exec_in_a_graph(torch_gpu):
    torch = torch_gpu
    Bn, H, W, C, F, R, Sx, stride, V = 8, 7, 7, 32, 64, 3, 3, 1, 32
    w = P.make_weight(F, R * Sx * C, V, 0.3, True, 2021, integer=True)
    xs = [np.random.default_rng(5 + i).integers(-4, 5, size=(C, H, W, Bn)).astype(np.float16) for i in range(2)]
    refs = [O.float_to_half(P.conv_oracle_batch_first(w, R, Sx, C, x, stride)) for x in xs]
    f = upload_weight(w, R, Sx, C, cls=S.BlockwiseSpFilter)
    dX = torch.empty((C, H, W, Bn), dtype=torch.float16, device="cuda")
    dY = torch.empty(refs[0].shape, dtype=torch.float16, device="cuda")
    op = S.SpconvBlockwiseOp()
    op.initialize(f, Bn, H, W, stride, dX.data_ptr(), dY.data_ptr(), batch_innermost=True)
    _replays(torch, op, [to_dev(torch, x) for x in xs], dX, dY, refs)
