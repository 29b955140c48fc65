// Include-path and type-name aliases so call sites written against the reference
// (block_sparse/cuda_array.h) compile unchanged; the implementation is hip_array.h.
#pragma once
#include "hip_array.h"
template <typename T> using CudaArray = HipArray<T>;
template <typename T> using CudaRandomArray = HipRandomArray<T>;
template <typename T> using CudaZerosArray = HipZerosArray<T>;
template <typename T> using CudaOnesArray = HipOnesArray<T>;
