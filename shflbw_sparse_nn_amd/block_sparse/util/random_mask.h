// Block mask generator, C++ overloads of block_sparse/util/random_mask.h:4-10 on top of the C ABI.
#pragma once
#include <vector>
#include "shflbw.h"
#include "block_sparse/hip_error.h"

inline void random_mask(int nrow, int ncol, int brow, int bcol, float block_density, int& nnzb, int& padded_nnzb,
                        std::vector<int>& indptr, std::vector<int>& indices, int block_divisor, int block_padding,
                        unsigned seed)
{
    const int X = nrow / brow, Y = ncol / bcol;
    indptr.assign(X + 1, 0);
    // upper bound of the padded count: every panel may be rounded up to the padding unit
    indices.assign(static_cast<size_t>(X) * Y + static_cast<size_t>(X) * (block_padding > 0 ? block_padding : 1), 0);
    SHFLBW_CHECK(shflbw_random_mask_ex(nrow, ncol, brow, bcol, block_density, block_divisor, block_padding, seed, &nnzb,
                                       &padded_nnzb, indptr.data(), indices.data(), indices.size()));
    indices.resize(padded_nnzb);
}

inline void random_mask(int nrow, int ncol, int brow, int bcol, float block_density, int& nnzb,
                        std::vector<int>& indptr, std::vector<int>& indices, unsigned seed)
{
    int padded = 0;
    random_mask(nrow, ncol, brow, bcol, block_density, nnzb, padded, indptr, indices, 1, 1, seed);
}
