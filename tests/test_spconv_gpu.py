"""GPU parity of the HIP sparse Conv2D (implicit GEMM over NHWC) against the CPU oracle, through the
C ABI.  Integer-valued inputs must match bit for bit after one fp16 rounding (index decode, padding,
stride and permutation handling); float inputs are held to the stated tolerances.  The reference's own
conv test never permutes the filter (test/test.spconv.blockwise.cu:21-33); every case here does."""
import numpy as np
import pytest

from oracle import oracle as O
import workloads as P
from workloads import float_error_report, run_spconv

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2
SCALED_TOL = 2.0 ** -9


def _exact(torch, Bn, H, W, C, F, R, S, stride, V, d, permute=True, seed=2021):
    w = P.make_weight(F, R * S * C, V, d, permute, seed, integer=True)
    x = np.random.default_rng(seed + 1).integers(-4, 5, size=(Bn, H, W, C)).astype(np.float16)
    ref = O.float_to_half(P.conv_oracle(w, R, S, C, x, stride))
    # 0: plane layout + SpMM + transpose, 1: one direct kernel; batches that are multiples of 8
    # also 2: planes and result with the batch innermost, 3: the steps of 2 in one launch, every XCD on its own columns
    forms = (0, 1)
    if Bn % 8 == 0:
        forms += (2, 3)
    for variant in forms:
        print("conv", (Bn, H, W, C, F, R, S, stride, V, d, permute), "form", variant, flush=True)
        got = run_spconv(torch, w, R, S, C, x, stride, variant)
        assert got.shape == ref.shape
        assert not np.isnan(got.astype(np.float32)).any(), "variant %d left output elements unwritten" % variant
        np.testing.assert_array_equal(got.view(np.uint16), ref.view(np.uint16), err_msg="variant %d" % variant)


@pytest.mark.parametrize("Bn,H,W,C,F,R,S,stride,V,d,permute", [
    (1, 5, 5, 8, 32, 3, 3, 1, 32, 0.5, True),     # tiny, pixel count not a multiple of anything
    (2, 7, 6, 16, 64, 3, 3, 2, 64, 0.3, True),    # stride 2, odd extents
    (3, 9, 9, 8, 128, 1, 1, 1, 128, 0.6, False),  # 1x1 filter, no permutation
    (2, 8, 8, 24, 64, 5, 3, 1, 32, 0.2, True),    # rectangular filter
    (4, 14, 14, 64, 128, 3, 3, 2, 64, 0.05, True),
    (2, 9, 7, 16, 48, 3, 3, 1, 16, 0.4, True),    # block height 16
    (2, 12, 10, 8, 64, 5, 5, 2, 32, 0.3, True),   # 5x5 stride 2: tap offsets 0..2 inside a phase plane
    (1, 11, 9, 16, 64, 3, 3, 3, 64, 0.5, True),   # stride 3: nine phase planes, one tap each
    (2, 6, 20, 8, 32, 1, 7, 1, 32, 0.4, True),    # 1x7 filter: seven tap offsets in one row
    # batches that are multiples of 8: the batch-innermost form runs too
    (8, 7, 6, 16, 64, 3, 3, 2, 64, 0.3, True),    # stride 2, odd extents
    (8, 5, 9, 8, 32, 5, 3, 1, 32, 0.4, False),    # rectangular filter, no permutation
    (24, 6, 5, 24, 48, 3, 3, 3, 16, 0.5, True),   # stride 3, block height 16, batch of 24
    (16, 4, 4, 8, 128, 1, 1, 1, 128, 0.6, True),  # 1x1 filter: no padding at all
    (8, 9, 8, 16, 64, 4, 2, 2, 32, 0.3, True),    # even filter extents: the output is larger than input / stride
    (8, 14, 14, 24, 48, 3, 3, 1, 16, 0.3, True),  # F and C no multiples of 64: ragged tiles in the layout phases
    (40, 9, 11, 8, 256, 3, 3, 1, 128, 0.2, True), # block height 128 (256-column tiles), batch of 40
    (12, 28, 28, 64, 512, 3, 3, 1, 32, 0.25, True), # block height 32 with 384 <= K <= 1128 and many column tiles: the middle must stay a gather
])
def test_exact_shapes(torch_gpu, Bn, H, W, C, F, R, S, stride, V, d, permute):
    _exact(torch_gpu, Bn, H, W, C, F, R, S, stride, V, d, permute)


@pytest.mark.parametrize("stride", [1, 2])
def test_reference_case(torch_gpu, stride):
    # shape of the reference's own conv test (test/test.spconv.blockwise.cu:10-15) with a smaller batch,
    # in NHWC and with a true strided convolution
    _exact(torch_gpu, 16, 14, 14, 256, 256, 3, 3, stride, 64, 0.1, True)


@pytest.mark.parametrize("name", ["cfg3", "cfg4"])
def test_graded_configs(torch_gpu, name):
    c = P.CONV_CONFIGS[name]
    _exact(torch_gpu, c["B"], c["H"], c["W"], c["C"], c["F"], c["R"], c["S"], c["stride"], c["V"], c["d"])
    w = P.make_weight(c["F"], c["R"] * c["S"] * c["C"], c["V"], c["d"], True, 2021, dist=c["w_dist"])
    x = P.make_dense(c["B"] * c["H"] * c["W"], c["C"], 2021, dist=c["x_dist"]).reshape(c["B"], c["H"], c["W"], c["C"])
    ref = P.conv_oracle(w, c["R"], c["S"], c["C"], x, c["stride"])
    bound = P.conv_oracle(dict(w, values=np.abs(w["values"])), c["R"], c["S"], c["C"], np.abs(x), c["stride"])
    got = run_spconv(torch_gpu, w, c["R"], c["S"], c["C"], x, c["stride"])
    rel, scaled = float_error_report(got.reshape(-1, c["F"]), ref.reshape(-1, c["F"]), bound.reshape(-1, c["F"]))
    print(name, "max rel err (|ref| >= 1e-2 rms):", rel, " max err / sum|ab|:", scaled, flush=True)
    assert rel <= REL_TOL and scaled <= SCALED_TOL


def test_shift_equivariance(torch_gpu):
    # size-independent property: for stride 1 a filter with one kept tap per row only shifts and scales the
    # input channel; checked through the dense formula on a full-size cfg3 input with integer values
    c = P.CONV_CONFIGS["cfg3"]
    F, V, C, R, S = 64, 64, c["C"], 3, 3
    indptr = np.array([0, 1], dtype=np.int32)
    k = (2 * S + 0) * C + 37  # tap (r=2, s=0), channel 37
    w = dict(nrow=F, ncol=R * S * C, brow=V, bcol=1, nnzb=1, indptr=indptr, indices=np.array([k], dtype=np.int32),
             values=(np.arange(F) % 5 - 2).astype(np.float16), row_permute_ids=O.row_permutation(F, 3))
    x = np.random.default_rng(8).integers(-4, 5, size=(c["B"], c["H"], c["W"], C)).astype(np.float16)
    got = run_spconv(torch_gpu, w, R, S, C, x, 1).astype(np.float32)
    shifted = np.zeros((c["B"], c["H"], c["W"]), dtype=np.float32)
    shifted[:, :-1, 1:] = x[:, 1:, :-1, 37]  # hi = ho + 1, wi = wo - 1
    for r in range(F):
        np.testing.assert_array_equal(got[..., w["row_permute_ids"][r]], shifted * float(w["values"][r]))


@pytest.mark.parametrize("patience", [0, -3000])
def test_fused_form_repeated_launches_and_two_streams(torch_gpu, patience):
    """The fused form keeps queues and counts in its scratch and clears them when a launch ends: many
    launches of one state in a row, with a new input each time, must all be right.  Two states over different
    tensors own different scratch, so their launches may overlap on two streams; no wait inside depends on a
    workgroup that is not running, so neither launch can block the other for good.  A negative patience makes
    every second workgroup join 30 us late and the others take its work over after one tick of waiting: the late ones
    find their numbers taken and leave, and the results must not change (the scratch counts the take-overs)."""
    import shflbw_sparse_nn_amd as S
    from shflbw_sparse_nn_amd import capi
    torch = torch_gpu
    Bn, H, W, C, F, R, Sx, stride, V = 8, 14, 14, 64, 256, 3, 3, 1, 64
    w = P.make_weight(F, R * Sx * C, V, 0.2, True, 2021, integer=True)
    f = P.upload_weight(w, R, Sx, C, cls=S.BlockwiseSpFilter)
    rng = np.random.default_rng(31)
    xs = [rng.integers(-4, 5, size=(Bn, H, W, C)).astype(np.float16) for _ in range(3)]
    refs = [O.float_to_half(P.conv_oracle(w, R, Sx, C, x, stride)) for x in xs]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    dX = [torch.empty((Bn, H, W, C), dtype=torch.float16, device="cuda") for _ in range(2)]
    dY = [torch.empty(refs[0].shape, dtype=torch.float16, device="cuda") for _ in range(2)]
    ops = []
    for i in range(2):
        op = S.SpconvBlockwiseOp(3)
        op.initialize(f, Bn, H, W, stride, dX[i].data_ptr(), dY[i].data_ptr())
        assert op._state.patience_ticks == 5000
        if patience:
            op._state.patience_ticks = patience
        ops.append(op)
    assert ops[0]._state.planes != ops[1]._state.planes  # scratch is per (geometry, tensors)
    assert ops[0]._state.spmm.packed_indices == ops[1]._state.spmm.packed_indices  # the ids per geometry only
    for rnd in range(6):
        print("fused conv round", rnd, flush=True)
        for i in range(2):
            dX[i].copy_(P.to_dev(torch, xs[(rnd + i) % 3]))
            dY[i].fill_(float("nan"))
        torch.cuda.synchronize()
        for i in range(2):
            for _ in range(3):  # back to back on its stream, overlapping the other stream's launches
                ops[i](streams[i].cuda_stream)
        torch.cuda.synchronize()
        for i in range(2):
            capi.check(capi.load().shflbw_spconv_check(ops[i]._state))
            np.testing.assert_array_equal(dY[i].cpu().numpy().view(np.uint16), refs[(rnd + i) % 3].view(np.uint16),
                                          err_msg="round %d stream %d" % (rnd, i))
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    for op in ops:  # the int at byte 60 of the synchronisation words counts the take-overs
        words = (ctypes.c_int * 16)()
        assert hip.hipMemcpy(words, ctypes.c_void_p(op._state.sync), 64, 2) == 0  # device to host
        if patience < 0:  # (with the default patience a take-over is rare but legal: nothing is asserted about it)
            assert words[15] > 0, words[15]


def test_fused_form_with_empty_row_panels(torch_gpu):
    """Row panels that keep no vector at all (legal through shflbw_weight_set and load) have no stage: their tiles
    are claimed, counted and written as zeros like any other."""
    Bn, H, W, C, F, R, Sx, stride, V = 8, 6, 7, 16, 256, 3, 3, 1, 32
    w = P.make_weight(F, R * Sx * C, V, 0.3, True, 77, integer=True)
    X = F // V
    keep = np.ones(X, dtype=bool)
    keep[[0, 3, 4, X - 1]] = False  # empty panels at the start, in a row, at the end
    counts = np.diff(w["indptr"]) * keep
    indptr = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    sel = np.concatenate([np.arange(w["indptr"][p], w["indptr"][p + 1]) for p in range(X) if keep[p]])
    w2 = dict(w, nnzb=int(indptr[-1]), indptr=indptr, indices=w["indices"][sel],
              values=w["values"].reshape(-1, V)[sel].reshape(-1))
    x = np.random.default_rng(78).integers(-4, 5, size=(Bn, H, W, C)).astype(np.float16)
    ref = O.float_to_half(P.conv_oracle(w2, R, Sx, C, x, stride))
    for variant in (0, 2, 3):
        got = run_spconv(torch_gpu, w2, R, Sx, C, x, stride, variant)
        np.testing.assert_array_equal(got.view(np.uint16), ref.view(np.uint16), err_msg="form %d" % variant)


def test_scratch_stays_bounded_over_fresh_tensor_pairs(torch_gpu):
    """A serving loop whose allocator hands out new addresses initialises a state per step: the gather ids are kept
    per geometry, the buffers the launches write are recycled, so the filter's scratch stops growing after
    SHFLBW_CONV_SCRATCH_DEPTH tensor pairs - and every result is still right."""
    import ctypes as C_
    import shflbw_sparse_nn_amd as S
    from shflbw_sparse_nn_amd import capi
    torch = torch_gpu
    lib = capi.load()
    Bn, H, W, C, F, R, Sx, stride, V = 8, 10, 10, 16, 64, 3, 3, 1, 32
    w = P.make_weight(F, R * Sx * C, V, 0.3, True, 5, integer=True)
    f = P.upload_weight(w, R, Sx, C, cls=S.BlockwiseSpFilter)
    x = np.random.default_rng(6).integers(-4, 5, size=(Bn, H, W, C)).astype(np.float16)
    ref = O.float_to_half(P.conv_oracle(w, R, Sx, C, x, stride))
    hx = P.to_dev(torch, x)
    keep, sizes = [], []
    for variant in (0, 2, 3):
        for i in range(40):
            dX, dY = hx.clone(), torch.full(ref.shape, float("nan"), dtype=torch.float16, device="cuda")
            keep.append((dX, dY))  # held, so that every pair has a fresh address
            op = S.SpconvBlockwiseOp(variant)
            op.initialize(f, Bn, H, W, stride, dX.data_ptr(), dY.data_ptr())
            op(torch.cuda.current_stream().cuda_stream)
            torch.cuda.synchronize()
            np.testing.assert_array_equal(dY.cpu().numpy().view(np.uint16), ref.view(np.uint16))
            b, n = C_.c_size_t(0), C_.c_int(0)
            capi.check(lib.shflbw_weight_scratch_bytes(f._h, C_.byref(b), C_.byref(n)))
            sizes.append((b.value, n.value))
        # flat from the depth of the pool on (this form's buffers have replaced the previous form's by then)
        assert len(set(sizes[-30:])) == 1, sizes[-30:]
    assert sizes[-1][1] <= 3 + 4  # one set of ids per form, at most SHFLBW_CONV_SCRATCH_DEPTH bulk buffers
    capi.check(lib.shflbw_weight_release_scratch(f._h))
    b, n = C_.c_size_t(1), C_.c_int(1)
    capi.check(lib.shflbw_weight_scratch_bytes(f._h, C_.byref(b), C_.byref(n)))
    assert (b.value, n.value) == (0, 0)


def test_non_finite_input_does_not_leak_through_padding(torch_gpu):
    """Padding slots of the filter's panels gather zeros (a row of zeros behind the planes, a row of zeros in the
    library for the im2col form, nothing in the direct kernel): an Inf in the input reaches only the outputs
    whose kept taps read it."""
    Bn, H, W, C, F, R, Sx, stride, V = 2, 9, 10, 16, 64, 3, 3, 1, 32
    w = P.make_weight(F, R * Sx * C, V, 0.3, True, 5, integer=True)
    w["values"] = np.where(w["values"] == 0, np.float16(1), w["values"]).astype(np.float16)
    x = np.random.default_rng(6).integers(-4, 5, size=(Bn, H, W, C)).astype(np.float16)
    x[0, 4, 5, 3] = np.inf
    x[1, 0, 0, C - 1] = -np.inf
    x[1, 8, 9, 7] = np.nan
    with np.errstate(invalid="ignore", over="ignore"):
        ref = O.float_to_half(P.conv_oracle(w, R, Sx, C, x, stride))
    assert np.isfinite(ref.astype(np.float32)).any() and not np.isfinite(ref.astype(np.float32)).all()
    for variant in (0, 1):
        got = run_spconv(torch_gpu, w, R, Sx, C, x, stride, variant)
        assert np.array_equal(np.isnan(got), np.isnan(ref)), "form %d: NaN pattern differs" % variant
        ok = ~np.isnan(ref)
        np.testing.assert_array_equal(got[ok], ref[ok], err_msg="form %d" % variant)
    # the batch-innermost forms need a batch of eights: the same two images four times over
    x8 = np.concatenate([x] * 4)
    with np.errstate(invalid="ignore", over="ignore"):
        ref8 = O.float_to_half(P.conv_oracle(w, R, Sx, C, x8, stride))
    for variant in (2, 3):
        got = run_spconv(torch_gpu, w, R, Sx, C, x8, stride, variant)
        assert np.array_equal(np.isnan(got), np.isnan(ref8)), "form %d: NaN pattern differs" % variant
        np.testing.assert_array_equal(got[~np.isnan(ref8)], ref8[~np.isnan(ref8)], err_msg="form %d" % variant)


@pytest.mark.parametrize("Bn,H,W,C,F,R,S,stride,V,d,permute", [
    (16, 14, 14, 64, 128, 3, 3, 1, 64, 0.2, True),
    (16, 14, 14, 64, 128, 3, 3, 2, 64, 0.2, True),    # the reference's "strided" case: taps beyond H x W read zero
    (8, 7, 9, 20, 64, 3, 3, 1, 32, 0.3, False),       # ragged extents, C not a multiple of 8
    (8, 6, 10, 16, 32, 5, 3, 2, 16, 0.4, True),       # block height 16, 5 x 3 filter
    (24, 5, 5, 8, 128, 1, 1, 1, 128, 0.5, True),      # 1 x 1 filter: no padding columns at all
    (8, 12, 12, 16, 64, 3, 3, 3, 32, 0.3, True),      # stride 3
])
def test_reference_layout_exact(torch_gpu, Bn, H, W, C, F, R, S, stride, V, d, permute):
    """The operator over the reference's own tensors (C-H-W-B in, F-H-W-B out, H and W bounding both) against the
    oracle's literal restatement of spconv/blockwise_format.h:55-132, bit for bit on integer data."""
    import shflbw_sparse_nn_amd as Sx
    torch = torch_gpu
    w = P.make_weight(F, R * S * C, V, d, permute, 2021, integer=True)
    x = np.random.default_rng(9).integers(-4, 5, size=(C, H, W, Bn)).astype(np.float16)
    ref = O.float_to_half(O.spconv_reference_chwb(F, R, S, C, V, 1, w["indptr"], w["indices"], w["values"],
                                                  w["row_permute_ids"], Bn, H, W, stride, x))
    f = P.upload_weight(w, R, S, C, cls=Sx.BlockwiseSpFilter)
    dX = P.to_dev(torch, x)
    dY = torch.full((F, H, W, Bn), float("nan"), dtype=torch.float16, device="cuda")
    op = Sx.SpconvBlockwiseOp()
    op.initialize(f, Bn, H, W, stride, dX.data_ptr(), dY.data_ptr(), batch_innermost=True)
    for _ in range(2):  # a second launch over the same scratch
        op(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    got = dY.cpu().numpy()
    assert not np.isnan(got.astype(np.float32)).any(), "output elements left unwritten"
    np.testing.assert_array_equal(got.view(np.uint16), ref.view(np.uint16))


def test_reference_layout_needs_a_batch_of_eights(torch_gpu):
    import shflbw_sparse_nn_amd as Sx
    from shflbw_sparse_nn_amd import capi
    w = P.make_weight(64, 9 * 8, 32, 0.3, True, 3, integer=True)
    f = P.upload_weight(w, 3, 3, 8, cls=Sx.BlockwiseSpFilter)
    t = torch_gpu.zeros(4096, dtype=torch_gpu.float16, device="cuda")
    with pytest.raises(capi.ShflbwError) as e:
        Sx.SpconvBlockwiseOp().initialize(f, 4, 5, 5, 1, t.data_ptr(), t.data_ptr(), batch_innermost=True)
    assert e.value.status == capi.ERR_SHAPE


def test_reference_layout_seeded_random_shapes(torch_gpu):
    """Twenty small seeded problems on the reference's tensors: filter extents 1..5, strides 1..3, batches of 8..32."""
    import shflbw_sparse_nn_amd as Sx
    torch = torch_gpu
    rng = np.random.default_rng(777)
    for case in range(20):
        V = int(rng.choice([16, 32, 64, 128]))
        F = V * int(rng.integers(1, 4))
        C = int(rng.integers(1, 24))
        R, S_ = int(rng.choice([1, 3, 5])), int(rng.choice([1, 2, 3, 5]))
        H, W = int(rng.integers(1, 12)), int(rng.integers(1, 12))
        Bn = 8 * int(rng.integers(1, 5))
        stride = int(rng.integers(1, 4))
        d = float(rng.choice([0.1, 0.4, 1.0]))
        print("case", case, (Bn, H, W, C, F, R, S_, stride, V, d), flush=True)
        w = P.make_weight(F, R * S_ * C, V, d, bool(rng.integers(0, 2)), 300 + case, integer=True)
        x = rng.integers(-4, 5, size=(C, H, W, Bn)).astype(np.float16)
        ref = O.float_to_half(P.conv_oracle_batch_first(w, R, S_, C, x, stride))
        f = P.upload_weight(w, R, S_, C, cls=Sx.BlockwiseSpFilter)
        dX = P.to_dev(torch, x)
        dY = torch.full((F, H, W, Bn), float("nan"), dtype=torch.float16, device="cuda")
        op = Sx.SpconvBlockwiseOp()
        op.initialize(f, Bn, H, W, stride, dX.data_ptr(), dY.data_ptr(), batch_innermost=True)
        op(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(dY.cpu().numpy().view(np.uint16), ref.view(np.uint16), err_msg="case %d" % case)


@pytest.mark.parametrize("variant", [2, 3])
def test_batch_innermost_forms_need_a_batch_of_eights(torch_gpu, variant):
    from shflbw_sparse_nn_amd import capi
    w = P.make_weight(64, 9 * 8, 32, 0.3, True, 3, integer=True)
    x = np.zeros((4, 5, 5, 8), dtype=np.float16)
    with pytest.raises(capi.ShflbwError) as e:
        run_spconv(torch_gpu, w, 3, 3, 8, x, 1, variant)
    assert e.value.status == capi.ERR_SHAPE


def test_direct_kernel_refuses_inputs_it_cannot_index(torch_gpu):
    """The direct kernel (every block height has one) indexes the input with 32 bits and says so in init."""
    import shflbw_sparse_nn_amd as S
    from shflbw_sparse_nn_amd import capi
    w = P.make_weight(64, 9 * 8, 16, 0.3, True, 3, integer=True)
    f = P.upload_weight(w, 3, 3, 8, cls=S.BlockwiseSpFilter)
    op = S.SpconvBlockwiseOp(1)
    t = torch_gpu.zeros(8, dtype=torch_gpu.float16, device="cuda")
    with pytest.raises(capi.ShflbwError) as e:
        op.initialize(f, 1 << 12, 1 << 8, 1 << 8, 1, t.data_ptr(), t.data_ptr())  # 2^31 input values; init reads no tensor
    assert e.value.status == capi.ERR_UNSUPPORTED and "2^31" in str(e.value)


@pytest.mark.parametrize("Bn,H,expected", [(8, 8, 2), (8, 16, 2), (12, 16, 0), (32, 8, 2), (20, 8, 0)])
def test_the_library_picks_the_batch_innermost_form_for_batches_of_eights(torch_gpu, Bn, H, expected):
    """shflbw_spconv_init: form 2 needs a batch that is a multiple of 8; other batches get form 0."""
    import shflbw_sparse_nn_amd as S
    torch = torch_gpu
    C, F = 8, 32
    w = P.make_weight(F, 9 * C, 32, 0.5, True, 3, integer=True)
    f = P.upload_weight(w, 3, 3, C, cls=S.BlockwiseSpFilter)
    dX = torch.zeros((Bn, H, H, C), dtype=torch.float16, device="cuda")
    dY = torch.zeros((Bn, H, H, F), dtype=torch.float16, device="cuda")
    op = S.SpconvBlockwiseOp()
    st = op.initialize(f, Bn, H, H, 1, dX.data_ptr(), dY.data_ptr())
    assert st.variant == expected, (Bn * H * H, st.variant)


@pytest.mark.parametrize("Bn,H,C,F,V,tile_cols", [
    (8, 6, 8, 64, 64, 128),       # 1 row panel, 4 tiles of 128 columns
    (8, 6, 16, 96, 32, 128),
    (16, 5, 8, 256, 128, 128),
    (16, 14, 8, 768, 64, 256),    # 12 row panels over 4096 columns: 384 tiles of 128, 96 of 512
    (16, 14, 8, 384, 32, 256),
    (16, 14, 8, 640, 32, 512),    # 20 row panels: 160 tiles of 512 columns
    (16, 14, 8, 1536, 128, 256),  # block height 128 has no wider tile than 256 columns
    (16, 14, 8, 96, 16, 512),     # block height 16 has the one width
])
def test_batch_innermost_form_tile_widths(torch_gpu, Bn, H, C, F, V, tile_cols):
    """The SpMM in the middle of form 2 takes its tile width from the size of the GEMM (128, 256 or 512 columns, as the
    SpMM proper does); every width gives the oracle's bits."""
    import shflbw_sparse_nn_amd as S
    torch = torch_gpu
    w = P.make_weight(F, 9 * C, V, 0.4, True, 77, integer=True)
    x = np.random.default_rng(78).integers(-4, 5, size=(Bn, H, H, C)).astype(np.float16)
    ref = O.float_to_half(P.conv_oracle(w, 3, 3, C, x, 1))
    f = P.upload_weight(w, 3, 3, C, cls=S.BlockwiseSpFilter)
    dX = P.to_dev(torch, x)
    dY = torch.full((Bn, H, H, F), float("nan"), dtype=torch.float16, device="cuda")
    op = S.SpconvBlockwiseOp(2)
    st = op.initialize(f, Bn, H, H, 1, dX.data_ptr(), dY.data_ptr())
    assert st.middle_tile_cols == tile_cols
    print("conv form 2", (Bn, H, C, F, V), "tiles of", st.middle_tile_cols, "columns, grid", st.grid_dim[0], flush=True)
    op(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    op.check()
    np.testing.assert_array_equal(dY.cpu().numpy().view(np.uint16), ref.view(np.uint16))


def test_library_choice_seeded_random_shapes(torch_gpu):
    """Twenty-four seeded NHWC problems with the form the library picks (form 2 for batches of eights, form 0 otherwise;
    the SpMM in the middle with tiles of 128, 256 or 512 columns): filter extents 1..5, strides 1..3, all block heights."""
    import shflbw_sparse_nn_amd as S
    torch = torch_gpu
    rng = np.random.default_rng(2718)
    forms = set()
    for case in range(24):
        V = int(rng.choice([16, 32, 64, 128]))
        F = V * int(rng.integers(1, 6))
        C = 8 * int(rng.integers(1, 6))  # the NHWC forms move channels in eights
        R, S_ = int(rng.choice([1, 3, 5])), int(rng.choice([1, 2, 3, 5]))
        H, W = int(rng.integers(3, 20)), int(rng.integers(3, 20))
        Bn = int(rng.choice([1, 2, 3, 8, 16, 24, 40]))
        stride = int(rng.integers(1, 4))
        d = float(rng.choice([0.1, 0.4, 1.0]))
        w = P.make_weight(F, R * S_ * C, V, d, bool(rng.integers(0, 2)), 900 + case, integer=True)
        x = rng.integers(-4, 5, size=(Bn, H, W, C)).astype(np.float16)
        ref = O.float_to_half(P.conv_oracle(w, R, S_, C, x, stride))
        f = P.upload_weight(w, R, S_, C, cls=S.BlockwiseSpFilter)
        dX = P.to_dev(torch, x)
        dY = torch.full(ref.shape, float("nan"), dtype=torch.float16, device="cuda")
        op = S.SpconvBlockwiseOp()
        st = op.initialize(f, Bn, H, W, stride, dX.data_ptr(), dY.data_ptr())
        forms.add(st.variant)
        print("case", case, (Bn, H, W, C, F, R, S_, stride, V, d), "form", st.variant, "tiles of", st.middle_tile_cols, flush=True)
        assert op.output_hw == ref.shape[1:3]
        op(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        op.check()
        np.testing.assert_array_equal(dY.cpu().numpy().view(np.uint16), ref.view(np.uint16), err_msg="case %d" % case)
    assert forms == {0, 2}

