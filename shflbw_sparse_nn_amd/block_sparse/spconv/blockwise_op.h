// Sparse Conv2D operator of the C++ veneer: SpconvBlockwiseOpState, SpconvBlockwiseOp<...>,
// SpconvBlockwiseInitFn / ExecFn and their pointer types (block_sparse/spconv/blockwise_op.h:6-17,
// 19-149, 161-193), forwarding to shflbw_spconv_init / shflbw_spconv_exec.
//
// Tensor layout differs from the reference by default: feature maps are NHWC
// (IFMap[b][hi][wi][c], OFMap[b][ho][wo][f]), H and W are the input extents, and stride is a
// true stride (output extent (H + 2*(R/2) - R)/stride + 1); the reference's maps are
// C-H-W-B / F-H-W-B with H, W doubling as input and output extent
// (spconv/blockwise_format.h:111-128).  The implicit-GEMM view (M = F, K ordered (r, s, c),
// zero for out-of-bounds taps, row permutation on F) is the reference's.  A filter whose fmap_layout is
// fmap_batch_first gets the reference's own tensors and bounds rule instead.
#pragma once
#include "blockwise_format.h"

struct SpconvBlockwiseOpState {
    size_t shared_mem_size = 0;
    dim3 gridDim;
    dim3 blockDim;
    bool initSuccess = false;
    struct Argument_t {
        int B, H, W, C, F, R, S, stride;
        half *A_values, *IFMap, *OFMap;
        int *A_bsr_indptr, *A_bsr_indices, *A_row_indices;
        float alpha, beta;
    } args{};
    int Ho = 0, Wo = 0;
    shflbw_spconv_state native{};
};

namespace shflbw_veneer {
inline SpconvBlockwiseOpState spconv_make_state(BlockwiseSpFilter<half>& spfilter, int block_height, int B, int H,
                                                int W, int stride, half* IFMap, half* OFMap)
{
    SpconvBlockwiseOpState st;
    assert(spfilter.brow == block_height && "operator block height must equal the filter block height");
    assert(spfilter.bcol == 1);
    assert(spfilter.device_synced);
    int rc = spfilter.fmap_layout == fmap_batch_first
                 ? shflbw_spconv_init_chwb(&st.native, spfilter.handle(), B, H, W, stride, IFMap, OFMap)
                 : shflbw_spconv_init(&st.native, spfilter.handle(), B, H, W, stride, IFMap, OFMap);
    if (rc != SHFLBW_OK) {
        std::cerr << "SpconvBlockwiseOp::initialize: " << shflbw_status_string(rc) << ": " << shflbw_last_error()
                  << std::endl;
        return st;
    }
    const shflbw_spconv_state& n = st.native;
    st.shared_mem_size = n.shared_mem_size;
    st.gridDim = dim3(n.grid_dim[0], n.grid_dim[1], n.grid_dim[2]);
    st.blockDim = dim3(n.block_dim[0], n.block_dim[1], n.block_dim[2]);
    st.args.B = B, st.args.H = H, st.args.W = W, st.args.C = n.args.C, st.args.F = n.args.F;
    st.args.R = n.args.R, st.args.S = n.args.S, st.args.stride = stride;
    st.args.A_values = static_cast<half*>(const_cast<void*>(n.args.A_values));
    st.args.IFMap = IFMap, st.args.OFMap = OFMap;
    st.args.A_bsr_indptr = const_cast<int*>(n.args.A_bsr_indptr);
    st.args.A_bsr_indices = const_cast<int*>(n.args.A_bsr_indices);
    st.args.A_row_indices = const_cast<int*>(n.args.A_row_indices);
    st.args.alpha = 1.0f, st.args.beta = 0.0f; // fixed, as in blockwise_op.h:89-94
    st.Ho = n.Ho, st.Wo = n.Wo;
    st.initSuccess = n.init_success != 0;
    return st;
}
} // namespace shflbw_veneer

template <typename ThreadBlockShape, typename WarpShape, typename MmaShape, int NStage, bool strided = true>
struct SpconvBlockwiseOp {
    static constexpr int BM = ThreadBlockShape::M;
    SpconvBlockwiseOpState _state;

    void initialize(BlockwiseSpFilter<half>& spfilter, int B, int H, int W, int stride, half* IFMap, half* OFMap)
    {
        _state = shflbw_veneer::spconv_make_state(spfilter, BM, B, H, W, stride, IFMap, OFMap);
    }
    void operator()(hipStream_t stream = nullptr)
    {
        if (!_state.initSuccess) {
            std::cerr << "SpconvBlockwiseOp: launch of an operator that failed to initialise" << std::endl;
            return;
        }
        SHFLBW_CHECK(shflbw_spconv_exec(&_state.native, stream));
    }
};

template <typename ThreadBlockShape, typename WarpShape, typename MmaShape, int NStage>
SpconvBlockwiseOpState SpconvBlockwiseInitFn(BlockwiseSpFilter<half>& spfilter, int B, int H, int W, int stride,
                                             half* IFMap, half* OFMap)
{
    return shflbw_veneer::spconv_make_state(spfilter, ThreadBlockShape::M, B, H, W, stride, IFMap, OFMap);
}

template <typename ThreadBlockShape, typename WarpShape, typename MmaShape, int NStage>
void SpconvBlockwiseExecFn(SpconvBlockwiseOpState& state, hipStream_t stream = nullptr)
{
    SHFLBW_CHECK(shflbw_spconv_exec(&state.native, stream));
}

typedef SpconvBlockwiseOpState (*SpconvBlockwiseInitFn_t)(BlockwiseSpFilter<half>&, int, int, int, int, half*,
                                                          half*);
typedef void (*SpconvBlockwiseExecFn_t)(SpconvBlockwiseOpState&, hipStream_t);
