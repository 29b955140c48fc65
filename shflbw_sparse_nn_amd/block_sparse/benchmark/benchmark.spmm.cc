// Benchmark of the block-sparse SpMM through the operator table.  Same command line, same shape
// padding, same timing loop (1 checked launch, 10 warm-up + 100 timed launches between two events) and
// the same output line per table entry as the reference's program (block_sparse/benchmark/
// benchmark.spmm.cu:10-52 timing, :54-124 main):
//   <arch> <matrix config> <n> <BM> <BN> <BK> <WM> <WN> <WK> <MM> <MN> <MK> <NSTAGE> <t> (us) <x> (effective tflop/s)
// "effective" is the dense-equivalent 2*m*n*k / t of the reference (benchmark.spmm.cu:107,117).  On gfx950
// every tile name of a block size runs the same native operator, so the lines of one block size
// differ only by run-to-run noise; --one-tile prints the first of them only.
#include <cstdio>
#include <fstream>
#include "argparse_util.h"
#include "block_sparse/cuda_array.h"
#include "block_sparse/spmm/spmm_library_decl.h"
#include "block_sparse/spmm/spmm_op.h"
#include "launch_timing.h"

#define GPU_ARCH 950 // gfx950; the reference prints its compute capability in this column

// one table entry on one problem: mean milliseconds per launch on `stream`, negative when the entry could not run
static float run_entry(SpmmBlockwiseInitFn_t init_fn, SpmmBlockwiseExecFn_t exec_fn, BlockwiseSpMatrix<half>& spmat, int N,
                       half* B, half* D, hipStream_t stream = nullptr)
{
    if (!launch_timing::device_clean("before the operator was set up")) return -1.f;
    SpmmBlockwiseOpState state = (*init_fn)(spmat, N, B, D);
    if (!state.initSuccess) {
        std::cerr << "operator set-up failed for this tile name" << std::endl;
        return -1.f;
    }
    // which native kernel stands behind the tile name on this problem (stderr: the result line on stdout stays the reference's)
    std::cerr << "native kernel: " << shflbw_spmm_variant_name(state.native.brow, state.native.variant) << std::endl;
    return launch_timing::mean_launch_ms([&] { (*exec_fn)(state, stream); }, stream, /* warmup */ 10, /* repeat */ 100);
}

struct TableEntry {
    int t[10]; // BM BN BK WM WN WK MM MN MK NSTAGE
    SpmmBlockwiseInitFn_t* init;
    SpmmBlockwiseExecFn_t* exec;
};
#define SHFLBW_TILE(BM, BN, BK, WM, WN, WK, MM, MN, MK, NS)                                              \
    {{BM, BN, BK, WM, WN, WK, MM, MN, MK, NS}, &NAME_FUN(SpmmBlockwise, Init, BM, BN, BK, WM, WN, WK, MM, MN, MK, NS), \
     &NAME_FUN(SpmmBlockwise, Exec, BM, BN, BK, WM, WN, WK, MM, MN, MK, NS)},
static const TableEntry table[] = {
#include "block_sparse/common/library_table.def"
};
#undef SHFLBW_TILE

int main(int argc, const char** argv)
{
    SpmmArgs a = parseSpmmArgs(argc, argv, /* verbose */ true);
    int m = a.m, n = a.n;
    const int k = a.k;
    // pad shapes (benchmark.spmm.cu:66-81)
    const int n_pad_to = 32;
    if (m % a.block_sz != 0) {
        m += a.block_sz - (m % a.block_sz);
        std::cerr << "m padded to : " << m << "\n";
    }
    if (n % n_pad_to != 0) {
        n += n_pad_to - (n % n_pad_to);
        std::cerr << "n padded to : " << n << " for better alignment.\n";
    }
    CudaRandomArray<half> B;
    CudaZerosArray<half> D;
    B.initialize(k * n);
    D.initialize(m * n);
    B.sync_device();
    D.sync_device();
    if (a.pattern_code != 0) return 0; // the reference has no operator behind the other pattern either

    BlockwiseSpMatrix<half> spmat;
    spmat.init_random(m, k, a.block_sz, 1, a.density, a.row_permute, a.seed);
    if (a.store_pattern) { // the text format of dump() (spmm/blockwise_format.h:125-149)
        std::ofstream out(a.store_path);
        spmat.dump(out);
    }
    spmat.transform_and_sync_device();

    const float gflop_count = (float)m / 1e9 * n * k * 2;
    int lines = 0;
    for (const TableEntry& e : table) {
        if (e.t[0] != a.block_sz) continue;
        std::cout << GPU_ARCH << " " << spmat.config_str << " ";
        printf("%d %d %d %d %d %d %d %d %d %d %d ", n, e.t[0], e.t[1], e.t[2], e.t[3], e.t[4], e.t[5], e.t[6], e.t[7],
               e.t[8], e.t[9]);
        const float dur = run_entry(*e.init, *e.exec, spmat, n, B.device_ptr, D.device_ptr);
        printf("%f (us) %f (effective tflop/s)\n", dur * 1e3, gflop_count / dur);
        fflush(stdout);
        lines++;
        if (a.one_tile) break;
    }
    if (lines == 0) std::cerr << "no operator for block size " << a.block_sz << "\n";
    return 0;
}
