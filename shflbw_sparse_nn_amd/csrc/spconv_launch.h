// Launch-side description of the native SpConv kernels (host + device shared).
#pragma once
#include <hip/hip_runtime.h>
#include "kernel_common.h"

namespace shflbw {

struct SpconvLaunchArgs {
    int B, H, W, C, F, R, S, stride, pad_h, pad_w, Ho, Wo;
    int X;       // filter row panels = F / V
    int n_tiles; // pixel tiles, filled by the launcher
    const half8_t* packedA;
    const int* kidx;      // kept k = (r*S + s)*C + c, 64-slot padded per panel
    const int* panel_desc; // per panel {k16 steps, first 64-slot group}
    const int* row_ids;   // F, or null
    const half_t* in;     // NHWC
    half_t* out;          // NHWC
};

struct SpconvVariant {
    int V;
    int BN; // output pixels per workgroup
    int threads;
    int lds_bytes;
    const char* name;
    hipError_t (*launch)(const SpconvLaunchArgs&, hipStream_t);
    hipError_t (*prepare)();
};

const SpconvVariant* spconv_variants(int* count);

} // namespace shflbw
