// SpMM operator of the C++ veneer: SpmmBlockwiseOpState, SpmmBlockwiseOp<...>,
// SpmmBlockwiseInitFn / ExecFn and their pointer types (block_sparse/spmm/blockwise_op.h:6-17,
// 19-174, 188-215), forwarding to shflbw_spmm_init / shflbw_spmm_exec.
//
// The tiling template arguments are accepted for source compatibility; on gfx950 only the
// block height ThreadBlockShape::M selects anything (it must equal the weight's brow, as in
// blockwise_op.h:85).  The native tile variant is chosen by the library.
#pragma once
#include "blockwise_format.h"

struct SpmmBlockwiseOpState {
    size_t shared_mem_size = 0;
    dim3 gridDim;
    dim3 blockDim;
    bool initSuccess = false;
    struct Argument_t {
        int M, N, K;
        half *A_values, *B, *C, *D;
        int *A_bsr_indptr, *A_bsr_indices, *A_row_indices;
        float alpha, beta;
    } args{};
    shflbw_spmm_state native{}; // what the launch actually consumes
};

namespace shflbw_veneer {
inline SpmmBlockwiseOpState spmm_make_state(BlockwiseSpMatrix<half>& spmat, int block_height, int N, half* B,
                                            half* C, half* D, float alpha, float beta)
{
    SpmmBlockwiseOpState st;
    assert(spmat.brow == block_height && "operator block height must equal the matrix block height");
    assert(spmat.bcol == 1);
    assert(spmat.device_synced);
    int rc = shflbw_spmm_init(&st.native, spmat.handle(), N, B, C, D, alpha, beta);
    if (rc != SHFLBW_OK) {
        std::cerr << "SpmmBlockwiseOp::initialize: " << shflbw_status_string(rc) << ": " << shflbw_last_error()
                  << std::endl;
        return st; // initSuccess stays false (blockwise_op.h:10,131)
    }
    const shflbw_spmm_state& n = st.native;
    st.shared_mem_size = n.shared_mem_size;
    st.gridDim = dim3(n.grid_dim[0], n.grid_dim[1], n.grid_dim[2]);
    st.blockDim = dim3(n.block_dim[0], n.block_dim[1], n.block_dim[2]);
    st.args.M = n.args.M, st.args.N = n.args.N, st.args.K = n.args.K;
    st.args.A_values = static_cast<half*>(const_cast<void*>(n.args.A_values));
    st.args.B = B, st.args.C = C, st.args.D = D;
    st.args.A_bsr_indptr = const_cast<int*>(n.args.A_bsr_indptr);
    st.args.A_bsr_indices = const_cast<int*>(n.args.A_bsr_indices);
    st.args.A_row_indices = const_cast<int*>(n.args.A_row_indices);
    st.args.alpha = alpha, st.args.beta = beta;
    st.initSuccess = n.init_success != 0;
    return st;
}
} // namespace shflbw_veneer

template <typename ThreadBlockShape, typename WarpShape, typename MmaShape, int NStage>
struct SpmmBlockwiseOp {
    static constexpr int BM = ThreadBlockShape::M;
    SpmmBlockwiseOpState _state;

    // D = A * B (blockwise_op.h:143-146 sets alpha = 1, beta = 0, C = nullptr)
    void initialize(BlockwiseSpMatrix<half>& spmat, int N, half* B, half* D)
    {
        _state = shflbw_veneer::spmm_make_state(spmat, BM, N, B, nullptr, D, 1.0f, 0.0f);
    }
    // D = A * B + C (blockwise_op.h:153-159)
    void initialize(BlockwiseSpMatrix<half>& spmat, int N, half* B, half* C, half* D)
    {
        _state = shflbw_veneer::spmm_make_state(spmat, BM, N, B, C, D, 1.0f, 1.0f);
    }
    // general form.  The reference accepts alpha here but then multiplies by 1 (blockwise_op.h:95);
    // this veneer honours the value passed.
    void initialize(BlockwiseSpMatrix<half>& spmat, int N, half* B, half* C, half* D, float alpha, float beta)
    {
        _state = shflbw_veneer::spmm_make_state(spmat, BM, N, B, C, D, alpha, beta);
    }
    void operator()(hipStream_t stream = nullptr)
    {
        if (!_state.initSuccess) {
            std::cerr << "SpmmBlockwiseOp: launch of an operator that failed to initialise" << std::endl;
            return;
        }
        SHFLBW_CHECK(shflbw_spmm_exec(&_state.native, stream));
    }
};

template <typename ThreadBlockShape, typename WarpShape, typename MmaShape, int NStage>
SpmmBlockwiseOpState SpmmBlockwiseInitFn(BlockwiseSpMatrix<half>& spmat, int N, half* B, half* D)
{
    return shflbw_veneer::spmm_make_state(spmat, ThreadBlockShape::M, N, B, nullptr, D, 1.0f, 0.0f);
}

template <typename ThreadBlockShape, typename WarpShape, typename MmaShape, int NStage>
void SpmmBlockwiseExecFn(SpmmBlockwiseOpState& state, hipStream_t stream = nullptr)
{
    SHFLBW_CHECK(shflbw_spmm_exec(&state.native, stream));
}

typedef SpmmBlockwiseOpState (*SpmmBlockwiseInitFn_t)(BlockwiseSpMatrix<half>&, int, half*, half*);
typedef void (*SpmmBlockwiseExecFn_t)(SpmmBlockwiseOpState&, hipStream_t);
