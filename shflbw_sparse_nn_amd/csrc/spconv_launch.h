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

// Arguments of the fused (single launch, XCD-local) form beside those of the SpMM in its middle.  The columns of
// the GEMM are those of the batch-innermost plane form (the padded output grid, ncols = Ho * PW * B); XCD x owns
// columns [x * cx, (x + 1) * cx) and, for them, a slab of planes, a filter-major result and a set of counters.
struct ConvXcdArgs {
    PlaneGeom g;          // input side: PH = Ho + (R-1)/stride rows, PW columns, pitch = values per channel row of a slab
    const half_t* in;     // NHWC input
    half_t* out;          // NHWC output
    half_t* slabs;        // nx slabs of slab_elems values: [stride^2 * C + 1][pitch], the last row stays zero
    size_t slab_elems;
    half_t* fm;           // nx results of fm_elems values: [F][cx]
    size_t fm_elems;
    int* sync;            // conv_xcd_sync_lines(nx) cache lines of SYNC_LINE ints, all zero between launches
    int nx, cx, ncols;    // XCDs, columns per XCD (a multiple of 64), columns in all
    int max_shift;        // largest tap offset: columns [n, n + max_shift] of a slab row feed column n
    int F, Ho, Wo;
    int ct, pt, ch_chunks; // phase-0 chunk: ct channel tiles x pt position tiles of 64 (ct * pt = 8, 4 or 2); chunks along C
    int ft, mt, f_chunks;  // phase-2 chunk: ft filter tiles x mt column tiles of 64; chunks along F
    unsigned magic_b, magic_pw; // udiv_magic of B and PW
    int spin_ticks;       // 100 MHz ticks a workgroup waits for a phase of its XCD to complete before it gives up
    int patience;         // ... and before it looks for work of workgroups that have not started
    int late_ticks;       // > 0 (tests only): the workgroups with odd numbers join this many ticks late
    int debug;            // diagnostic builds only: bits that switch parts of the kernel off (0 otherwise)
};

struct ConvXcdKernel {
    int V;
    int BN;      // columns of the GEMM per tile
    int threads;
    int lds_bytes;
    hipError_t (*launch)(const SpmmLaunchArgs&, const ConvXcdArgs&, hipStream_t);
    hipError_t (*prepare)();
};
const ConvXcdKernel* conv_xcd_kernel(int V);
constexpr int XCD_LINES = 4;      // cache lines of counters per XCD
constexpr int XCD_TAKEOVERS = 15; // int of the first line (the one with the flag) that counts the take-overs
inline int conv_xcd_sync_lines(int nx) { return 1 + nx * XCD_LINES; }
// writes the XCD every workgroup of a launch of `blocks` workgroups runs on to out[blocks] (device memory)
hipError_t launch_xcd_probe(int* out, int blocks, hipStream_t stream);

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
const ConvChwbKernel* conv_chwb_kernel(int V, int tile_cols, long X, long ncols, int cus);

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

} // namespace shflbw
