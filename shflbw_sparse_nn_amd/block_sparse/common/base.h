// Small shared definitions of the veneer (block_sparse/common/base.h:15-24).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <cassert>
#include <cstdio>
#include <iostream>
#include <string>

#define CEIL(x, y) (((x) + (y)-1) / (y))
#define ROUND_UP(x, y) ((CEIL((x), (y))) * (y))

// Compile-time 3-D shape.  Of all the tiling template arguments the reference's operators
// take, only the block height ThreadBlockShape::M has a meaning on gfx950: the native kernels
// choose their own tiling per block height.
template <int M_, int N_, int K_>
struct ShapeBase {
    static constexpr int M = M_, N = N_, K = K_;
};
