// Launch-side description of the native SpMM tile variants (host + device shared).
#pragma once
#include <hip/hip_runtime.h>
#include "kernel_common.h"

namespace shflbw {

struct SpmmLaunchArgs {
    int M, N, K;
    int X;       // row panels = M / V
    int n_tiles; // column tiles, filled by the launcher
    const half8_t* packedA; // private image: A fragments in register order
    const int* kidx;        // private image: kept column ids, 64-slot padded per panel
    const int* kidx_pm;     // same ids, each 64-slot group reordered producer-major: [16p + 4j + r] = [16j + 4p + r]
    const int* slab_ids;    // slab kernel only: the ids as LDS offsets of slab rows, [group][pair of slots][step][2]
    int slab_chunks;        // slab kernel only: the panels are dealt to this many workgroups per column tile (launcher)
    const int* panel_desc;  // private image: per panel {MFMA k16 steps = ceil(nnz/16), first 64-slot group}
    const int* row_ids;     // M, or null when rows are not permuted
    const half_t* B;
    const void* zero_row;   // 1 KiB of zeros on the device: what the padding slots (id -1) of a panel's last group gather
    int ldb_bytes;          // bytes between rows of B one id apart (N * 2 for a dense row-major B)
    const half_t* C;
    half_t* D;
    int ldd;                // values between two rows of C and D (N for the SpMM)
    int dmap_row, dmap_valid; // batch-innermost convolution only: see output_column()
    unsigned dmap_magic;      // udiv magic of dmap_row
    float alpha, beta;
    int num_cus; // compute units of the device (persistent kernels size their grid with it)
    int alternate; // role-split kernels: walk every second tile of a workgroup from its last stage to its first
                   // (pays when the rows of B under one column tile do not fit the XCD's L2)
};

struct SpmmVariant {
    int V;           // block size (rows per panel)
    int BN;          // output columns per workgroup
    int threads;     // workgroup size
    int lds_bytes;   // dynamic LDS
    const char* name;
    hipError_t (*launch)(const SpmmLaunchArgs&, hipStream_t);
    hipError_t (*prepare)(); // raises the dynamic-LDS limit of the kernel
    int max_k;               // 0, or the most columns of A the variant takes (it holds all rows of B in LDS)
};

const SpmmVariant* spmm_variants(int* count);

// device address of the library's row of zeros on the current device (looked up once per device); null on failure
const void* spmm_zero_row();

} // namespace shflbw
