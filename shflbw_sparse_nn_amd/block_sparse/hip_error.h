// Error handling of the C++ veneer.  The reference's host API reports a failed runtime call by
// printing and exiting (block_sparse/cuda_error.h:7-26); the veneer keeps that contract on top
// of the C ABI, which itself only returns status codes.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <iostream>
#include "shflbw.h"

#define HIP_CHECK(expr)                                                                         \
    do {                                                                                        \
        hipError_t hip_check_err_ = (expr);                                                     \
        if (hip_check_err_ != hipSuccess) {                                                     \
            std::cerr << "Got bad hip status: " << hipGetErrorString(hip_check_err_)            \
                      << " at line: " << __LINE__ << " of file " << __FILE__ << std::endl;      \
            std::exit(EXIT_FAILURE);                                                            \
        }                                                                                       \
    } while (0)

inline bool isHipSuccess(hipError_t status)
{
    if (status == hipSuccess) return true;
    std::cerr << "Got bad hip status: " << hipGetErrorString(status) << std::endl;
    return false;
}

// A failed C-ABI call in a place where the reference would have asserted or exited.
#define SHFLBW_CHECK(expr)                                                                      \
    do {                                                                                        \
        int shflbw_check_rc_ = (expr);                                                          \
        if (shflbw_check_rc_ != SHFLBW_OK) {                                                    \
            std::cerr << "shflbw: " << shflbw_status_string(shflbw_check_rc_) << ": "           \
                      << shflbw_last_error() << " at line: " << __LINE__ << " of file "         \
                      << __FILE__ << std::endl;                                                 \
            std::exit(EXIT_FAILURE);                                                            \
        }                                                                                       \
    } while (0)
