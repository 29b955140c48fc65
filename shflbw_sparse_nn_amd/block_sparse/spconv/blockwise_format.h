// Sparse convolution filter of the C++ veneer: BlockwiseSpFilter<T>
// (block_sparse/spconv/blockwise_format.h:17-52).  The filter is the F x (R*S*C) Shfl-BW matrix
// whose column k is the tap (r, s, c) with k = (r*S + s)*C + c (spconv/conv_format.h:4-7,19-23).
#pragma once
#include "block_sparse/spmm/blockwise_format.h"

enum LayoutFilter {
    filter_channel_first, // F-R-S-C, the only layout the operators take
    filter_planar_first   // F-C-R-S
};

// Layout of the feature maps the operators of a filter work on.  fmap_nhwc (the default here): IFMap[b][hi][wi][c],
// OFMap[b][ho][wo][f], H and W the input extents, true stride.  fmap_batch_first: the reference's own tensors,
// IFMap[c][h][w][b] and OFMap[f][h][w][b] with H, W bounding input and output alike
// (spconv/blockwise_format.h:111-128); set `spfilter.fmap_layout = fmap_batch_first;` before initialize().
enum LayoutFmap {
    fmap_nhwc,
    fmap_batch_first
};

template <typename T>
struct BlockwiseSpFilter : public BlockwiseSpMatrix<T> {
    LayoutFmap fmap_layout = fmap_nhwc;
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

    template <typename U>
    friend void get_host_reference(BlockwiseSpFilter<U>& spfilter, const int B, const int H, const int W,
                                   const int stride, const std::vector<U>& IFMap, std::vector<float>& OFMap_ref,
                                   LayoutFilter layout_filter);
};

// The convolution on the CPU, fp32 (spconv/blockwise_format.h:55-132), over the tensors `spfilter.fmap_layout`
// names: NHWC with H and W the input extents, padding R/2 and S/2, output [B][Ho][Wo][F] with
// Ho = (H + 2*(R/2) - R)/stride + 1; or, for fmap_batch_first, the reference's C-H-W-B input and F-H-W-B output of
// B*H*W*F values.  Only filter_channel_first filters exist here.
template <typename T>
void get_host_reference(BlockwiseSpFilter<T>& spfilter, const int B, const int H, const int W, const int stride,
                        const std::vector<T>& IFMap, std::vector<float>& OFMap_ref,
                        LayoutFilter layout_filter = filter_channel_first)
{
    assert(layout_filter == filter_channel_first);
    (void)layout_filter;
    spfilter.push_host_arrays();
    if (spfilter.fmap_layout == fmap_batch_first) {
        OFMap_ref.resize(static_cast<size_t>(B) * H * W * spfilter.F);
        SHFLBW_CHECK(shflbw_spconv_host_reference_chwb(spfilter.handle(), B, H, W, stride,
                                                       reinterpret_cast<const uint16_t*>(IFMap.data()), OFMap_ref.data()));
        return;
    }
    const int Ho = (H + 2 * (spfilter.R / 2) - spfilter.R) / stride + 1;
    const int Wo = (W + 2 * (spfilter.S / 2) - spfilter.S) / stride + 1;
    OFMap_ref.resize(static_cast<size_t>(B) * Ho * Wo * spfilter.F);
    SHFLBW_CHECK(shflbw_spconv_host_reference(spfilter.handle(), B, H, W, stride,
                                              reinterpret_cast<const uint16_t*>(IFMap.data()), OFMap_ref.data()));
}
