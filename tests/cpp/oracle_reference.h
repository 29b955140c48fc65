// CPU oracle entry points (oracle/shflbw_oracle.c) as used by the C++ tests: the counterpart of
// the reference's get_host_reference (spmm/blockwise_format.h:268-311 and
// spconv/blockwise_format.h:55-132).  Test infrastructure only: linked by the programs in this
// directory, never by the library.
#pragma once
#include <cstdint>
#include <cstdlib>
#include <iostream>
#include <vector>
#include "block_sparse/spconv/blockwise_format.h"
#include "block_sparse/spmm/blockwise_format.h"

extern "C" {
int oracle_spmm_reference(int nrow, int ncol, int brow, int bcol, const int* indptr, const int* indices,
                          const uint16_t* values, const int* row_permute_ids, int N, const uint16_t* B, float alpha,
                          const uint16_t* C, float beta, float* D_ref, int nthreads);
int oracle_spconv_reference_nhwc(int F, int R, int S, int C, int brow, const int* indptr, const int* indices,
                                 const uint16_t* values, const int* row_permute_ids, int B, int H, int W, int stride,
                                 int pad_h, int pad_w, const uint16_t* IFMap, float* OFMap_ref, int nthreads);
int oracle_spconv_reference_chwb(int F, int R, int S, int C, int brow, int bcol, const int* indptr, const int* indices,
                                 const uint16_t* values, const int* row_permute_ids, int B, int H, int W, int stride,
                                 const uint16_t* IFMap, float* OFMap_ref);
}

template <typename T>
void oracle_reference(BlockwiseSpMatrix<T>& spmat, int N, const std::vector<T>& B, float alpha,
                        const std::vector<T>& C, float beta, std::vector<float>& D_ref)
{
    D_ref.assign(static_cast<size_t>(spmat.nrow) * N, 0.f);
    int rc = oracle_spmm_reference(spmat.nrow, spmat.ncol, spmat.brow, spmat.bcol, spmat.indptr.data(),
                                   spmat.indices.data(), reinterpret_cast<const uint16_t*>(spmat.values.data()),
                                   spmat.row_permute ? spmat.row_permute_ids.data() : nullptr, N,
                                   reinterpret_cast<const uint16_t*>(B.data()), alpha,
                                   C.empty() ? nullptr : reinterpret_cast<const uint16_t*>(C.data()), beta,
                                   D_ref.data(), 0);
    if (rc != 0) {
        std::cerr << "oracle_spmm_reference failed: " << rc << std::endl;
        std::exit(EXIT_FAILURE);
    }
}

// NHWC feature maps, H and W are the input extents, padding R/2 and S/2
template <typename T>
void oracle_reference(BlockwiseSpFilter<T>& f, int B, int H, int W, int stride, const std::vector<T>& IFMap,
                        std::vector<float>& OFMap_ref)
{
    const int Ho = (H + 2 * (f.R / 2) - f.R) / stride + 1, Wo = (W + 2 * (f.S / 2) - f.S) / stride + 1;
    OFMap_ref.assign(static_cast<size_t>(B) * Ho * Wo * f.F, 0.f);
    int rc = oracle_spconv_reference_nhwc(f.F, f.R, f.S, f.C, f.brow, f.indptr.data(), f.indices.data(),
                                          reinterpret_cast<const uint16_t*>(f.values.data()),
                                          f.row_permute ? f.row_permute_ids.data() : nullptr, B, H, W, stride, f.R / 2,
                                          f.S / 2, reinterpret_cast<const uint16_t*>(IFMap.data()), OFMap_ref.data(), 0);
    if (rc != 0) {
        std::cerr << "oracle_spconv_reference_nhwc failed: " << rc << std::endl;
        std::exit(EXIT_FAILURE);
    }
}

// the reference's own tensors: C-H-W-B in, F-H-W-B out, H and W bounding both (spconv/blockwise_format.h:111-128)
template <typename T>
void oracle_reference_batch_first(BlockwiseSpFilter<T>& f, int B, int H, int W, int stride, const std::vector<T>& IFMap,
                                  std::vector<float>& OFMap_ref)
{
    OFMap_ref.assign(static_cast<size_t>(B) * H * W * f.F, 0.f);
    int rc = oracle_spconv_reference_chwb(f.F, f.R, f.S, f.C, f.brow, f.bcol, f.indptr.data(), f.indices.data(),
                                          reinterpret_cast<const uint16_t*>(f.values.data()),
                                          f.row_permute ? f.row_permute_ids.data() : nullptr, B, H, W, stride,
                                          reinterpret_cast<const uint16_t*>(IFMap.data()), OFMap_ref.data());
    if (rc != 0) {
        std::cerr << "oracle_spconv_reference_chwb failed: " << rc << std::endl;
        std::exit(EXIT_FAILURE);
    }
}

// The reference's acceptance rule (test/test_util.spmm.h:9-30): |ref - d| <= 1e-3 |ref| for every element.
template <typename T>
bool checkEqual(size_t count, const std::vector<T>& res, const std::vector<float>& ref, bool verbose = false)
{
    for (size_t i = 0; i < count; i++) {
        const float d = static_cast<float>(res[i]), r = ref[i];
        if (!(fabsf(r - d) <= 1e-3f * fabsf(r))) {
            if (verbose) printf("element %zu: result %f != %f\n", i, d, r);
            return false;
        }
    }
    return true;
}
