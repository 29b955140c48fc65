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

// Stages 1 and 3 of the plane form of the convolution: NHWC input -> channel-major padded planes (one per
// stride phase, `copies` = 1 or 2 with a copy moved by one value, rows of `pitch` values), and the
// filter-major result over plane positions (rows of NP values) -> NHWC output.
hipError_t launch_nhwc_to_planes(const SpconvLaunchArgs& a, half_t* planes, int PH, int PW, int pitch, int copies,
                                 hipStream_t stream);
hipError_t launch_planes_to_nhwc(const half_t* dm, half_t* out, int F, int NP, int B, int PH, int PW, int Ho, int Wo,
                                 hipStream_t stream);

// Plane-form ids computed on the device (for callers that may not copy from the host): slot-ordered and
// producer-major element offsets from the packed kept-column ids.
hipError_t launch_plane_ids(const int* kidx, int* ids, int* ids_pm, int slots, int C, int S, int stride, int PW,
                            int pitch, int copies, hipStream_t stream);

// Stages 1 and 3 of the im2col form of the convolution: NHWC input -> im2col matrix with rows of NP
// halves (NP a multiple of 64), and filter-major result -> NHWC output.
hipError_t launch_im2col_nhwc(const SpconvLaunchArgs& a, half_t* bm, int NP, hipStream_t stream);
hipError_t launch_transpose_to_nhwc(const half_t* dm, half_t* out, int F, int npix, int NP, hipStream_t stream);

} // namespace shflbw
