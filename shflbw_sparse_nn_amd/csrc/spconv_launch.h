// Launch-side description of the native SpConv kernels (host + device shared).
#pragma once
#include <hip/hip_runtime.h>
#include "kernel_common.h"
#include "spmm_launch.h"

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

// Geometry of the channel-major padded planes the plane forms of the convolution gather from.
struct PlaneGeom {
    int B, H, W, C, stride, pad_h, pad_w;
    int PH, PW;   // rows and (padded) columns of a phase plane
    int pitch;    // values per channel row of the plane tensor
    int copies;   // 1, or 2 with the copy moved by one value
    int nwanted;  // (copy, phase) planes some tap reads; the others are never written
    unsigned char wanted[32]; // copy * stride * stride + phase of each
    int batch_inner; // position n of a plane is (i * PW + j) * B + img instead of (img * PH + i) * PW + j
};

bool fill_wanted_planes(PlaneGeom& g, int R, int S);

// Arguments of the fused (single launch) form beside those of the SpMM in its middle.
struct ConvFuseArgs {
    PlaneGeom g;          // input side (phase 0)
    const half_t* in;     // NHWC input
    half_t* planes;
    int np64;             // plane positions written per channel row (rounded up to 64)
    int ct, pt;           // phase-0 chunk: ct channel tiles x pt position tiles of 64 (ct * pt = 8, 4 or 2)
    int ch_chunks, pos_chunks, n0chunks; // chunks per plane along channels / positions, and in total
    const half_t* fm;     // [F][ncols] filter-major result (phase 1 output, phase 2 input)
    half_t* out;          // NHWC output
    int F, ncols, Ho, Wo;
    int ft, mt;           // phase-2 chunk: ft filter tiles x mt column tiles of 64 (ft * mt = 8, 4 or 2)
    int f_chunks;         // chunks per column tile along F
    int slabs;            // column tiles of the GEMM
    int arrivals_per_slab; // finished tiles that complete a column tile (one per row panel)
    int* sync;            // synchronisation words, conv_sync_lines(slabs) cache lines of SYNC_LINE ints, all zero between launches
    unsigned magic_ps, magic_pw, magic_imgcols; // udiv_magic of PH*PW, PW and Ho*PW
    int help_ticks;       // 100 MHz ticks a workgroup without obligation keeps waiting for column tiles in phase 2
    int phases;           // bit 0: run phase 0, bit 1: run phase 2 (cleared: the layout kernels are launched around it)
};

struct ConvFusedKernel {
    int V;
    int BN;      // columns of the GEMM per tile
    int ncons;   // consumer waves per workgroup (arrivals per tile)
    int threads;
    int lds_bytes;
    hipError_t (*launch)(const SpmmLaunchArgs&, const ConvFuseArgs&, hipStream_t);
    hipError_t (*prepare)();
};
const ConvFusedKernel* conv_fused_kernel(int V);
// cache lines of synchronisation words the fused form needs for a problem with `slabs` column tiles
constexpr int CONV_LINE_SLAB0 = 27; // first of the two lines per column tile
inline int conv_sync_lines(int slabs) { return CONV_LINE_SLAB0 + 2 * slabs; }

// Batch-innermost (C-H-W-B in, F-H-W-B out) form of the convolution: the copy into padded phase planes and the
// role-split kernel whose epilogue writes compact output rows.
hipError_t launch_chwb_to_planes(const half_t* in, half_t* planes, int B, int H, int W, int C, int R, int S, int stride,
                                 int PHX, int PW, int pitch, hipStream_t stream);
struct ConvChwbKernel {
    int V;
    int BN;
    int threads;
    int lds_bytes;
    hipError_t (*launch)(const SpmmLaunchArgs&, hipStream_t);
    hipError_t (*prepare)();
};
const ConvChwbKernel* conv_chwb_kernel(int V);

// Stages 1 and 3 of the plane form of the convolution: NHWC input -> channel-major padded planes (one per
// stride phase, `copies` = 1 or 2 with a copy moved by one value, rows of `pitch` values), and the
// filter-major result over plane positions (rows of NP values) -> NHWC output.
// batch_inner: the positions of a plane (and of the result) run (row, column, image) instead of (image, row, column)
hipError_t launch_nhwc_to_planes(const SpconvLaunchArgs& a, half_t* planes, int PH, int PW, int pitch, int copies,
                                 hipStream_t stream, int batch_inner = 0);
hipError_t launch_planes_to_nhwc(const half_t* dm, half_t* out, int F, int NP, int B, int PH, int PW, int Ho, int Wo,
                                 hipStream_t stream, int batch_inner = 0);

// Plane-form ids computed on the device (for callers that may not copy from the host): slot-ordered and
// producer-major element offsets from the packed kept-column ids; padding slots get `zero_id`, the offset of a
// row of `pitch` zeros in `planes`, which the same launch clears.
hipError_t launch_plane_ids(const int* kidx, int* ids, int* ids_pm, int slots, int C, int S, int stride, int PW,
                            int pitch, int copies, int zero_id, half_t* planes, hipStream_t stream);

// Stages 1 and 3 of the im2col form of the convolution: NHWC input -> im2col matrix with rows of NP
// halves (NP a multiple of 64), and filter-major result -> NHWC output.
hipError_t launch_im2col_nhwc(const SpconvLaunchArgs& a, half_t* bm, int NP, hipStream_t stream);
hipError_t launch_transpose_to_nhwc(const half_t* dm, half_t* out, int F, int npix, int NP, hipStream_t stream);

} // namespace shflbw
