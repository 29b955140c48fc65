// Sparse convolution filter of the C++ veneer: BlockwiseSpFilter<T>
// (block_sparse/spconv/blockwise_format.h:17-52).  The filter is the F x (R*S*C) Shfl-BW matrix
// whose column k is the tap (r, s, c) with k = (r*S + s)*C + c (spconv/conv_format.h:4-7,19-23).
#pragma once
#include "block_sparse/spmm/blockwise_format.h"

enum LayoutFilter {
    filter_channel_first, // F-R-S-C, the only layout the operators take
    filter_planar_first   // F-C-R-S
};

template <typename T>
struct BlockwiseSpFilter : public BlockwiseSpMatrix<T> {
    int F = 0; // filters (output channels)
    int C = 0; // input channels
    int R = 0; // filter rows
    int S = 0; // filter columns

    void init_random(int F_, int R_, int S_, int C_, int brow_, int bcol_, float expected_density,
                     bool filter_permute, unsigned seed_)
    {
        SHFLBW_CHECK(shflbw_filter_init_random(this->handle_, F_, R_, S_, C_, brow_, bcol_, expected_density,
                                               filter_permute ? 1 : 0, seed_));
        F = F_, R = R_, S = S_, C = C_;
        this->filter_R_ = R_, this->filter_S_ = S_, this->filter_C_ = C_;
        this->pull_host_arrays();
    }
};
