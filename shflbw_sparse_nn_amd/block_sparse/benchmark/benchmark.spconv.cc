// Benchmark of the block-sparse convolution through the operator table.  Same command line, timing
// loop and output line per table entry as the reference's program (block_sparse/benchmark/
// benchmark.spconv.cu:10-52 timing, :54-130 main):
//   <arch> <filter config> <B> <H> <W> <stride> <BM> ... <NSTAGE> <t> (us) <x> (effective tflop/s)
// As there, --H and --W are the extents of the OUTPUT; the input tensor is (H*stride) x (W*stride)
// (benchmark.spconv.cu:90).  Tensors are NHWC here and the strided case is a true strided convolution
// with padding R/2, S/2, whose output is exactly H x W for odd filters.  "effective" is the
// dense-equivalent 2*B*H*W*C*R*S*F / t (benchmark.spconv.cu:103).
#include <cstdio>
#include <fstream>
#include "argparse_util.h"
#include "block_sparse/cuda_array.h"
#include "block_sparse/spconv/spconv_library_decl.h"
#include "block_sparse/spconv/spconv_op.h"
#include "launch_timing.h"

#define GPU_ARCH 950

// one table entry on one problem: mean milliseconds per launch on `stream`, negative when the entry could not run
static float run_entry(SpconvBlockwiseInitFn_t init_fn, SpconvBlockwiseExecFn_t exec_fn, BlockwiseSpFilter<half>& spfilter,
                       int B, int Hin, int Win, int stride, half* IFMap, half* OFMap, hipStream_t stream = nullptr)
{
    if (!launch_timing::device_clean("before the operator was set up")) return -1.f;
    SpconvBlockwiseOpState state = (*init_fn)(spfilter, B, Hin, Win, stride, IFMap, OFMap);
    if (!state.initSuccess) {
        std::cerr << "operator set-up failed for this tile name" << std::endl;
        return -1.f;
    }
    // which form of the convolution stands behind the tile name on this problem (stderr: the result line on stdout stays the reference's)
    std::cerr << "native kernel: " << shflbw_spconv_variant_name(state.native.variant) << std::endl;
    return launch_timing::mean_launch_ms([&] { (*exec_fn)(state, stream); }, stream, /* warmup */ 10, /* repeat */ 100);
}

struct TableEntry {
    int t[10];
    SpconvBlockwiseInitFn_t* init;
    SpconvBlockwiseExecFn_t* exec;
};
#define SHFLBW_TILE(BM, BN, BK, WM, WN, WK, MM, MN, MK, NS)                                                \
    {{BM, BN, BK, WM, WN, WK, MM, MN, MK, NS}, &NAME_FUN(SpconvBlockwise, Init, BM, BN, BK, WM, WN, WK, MM, MN, MK, NS), \
     &NAME_FUN(SpconvBlockwise, Exec, BM, BN, BK, WM, WN, WK, MM, MN, MK, NS)},
static const TableEntry table[] = {
#include "block_sparse/common/library_table.def"
};
#undef SHFLBW_TILE

int main(int argc, const char** argv)
{
    SpconvArgs a = parseSpconvArgs(argc, argv, /* verbose */ true);
    int F = a.F;
    if (F % a.block_sz != 0) { // benchmark.spconv.cu:69-78
        F += a.block_sz - (F % a.block_sz);
        std::cerr << "F padded to : " << F << "\n";
    }
    const int Hin = a.H * a.stride, Win = a.W * a.stride;
    CudaRandomArray<half> IFMap;
    CudaZerosArray<half> OFMap;
    IFMap.initialize(a.B * Hin * Win * a.C);
    // the library writes B x Ho x Wo x F; for odd filters that is exactly the H x W of the command line, for an
    // even R or S the padding R/2 makes it one larger (the reference always writes H x W)
    const int Ho = (Hin + 2 * (a.R / 2) - a.R) / a.stride + 1, Wo = (Win + 2 * (a.S / 2) - a.S) / a.stride + 1;
    OFMap.initialize(a.B * Ho * Wo * F);
    IFMap.sync_device();
    OFMap.sync_device();
    if (a.pattern_code != 0) return 0;

    BlockwiseSpFilter<half> spfilter;
    spfilter.init_random(F, a.R, a.S, a.C, a.block_sz, 1, a.density, a.row_permute, a.seed);
    if (a.store_pattern) { // the text format of dump() (spmm/blockwise_format.h:125-149)
        std::ofstream out(a.store_path);
        spfilter.dump(out);
    }
    spfilter.transform_and_sync_device();

    const float gflop_count = (float)a.B / 1e9 * a.H * a.W * a.C * a.R * a.S * F * 2;
    int lines = 0;
    for (const TableEntry& e : table) {
        if (e.t[0] != a.block_sz) continue;
        std::cout << GPU_ARCH << " " << spfilter.config_str << " ";
        printf("%d %d %d %d %d %d %d %d %d %d %d %d %d %d ", a.B, a.H, a.W, a.stride, e.t[0], e.t[1], e.t[2], e.t[3],
               e.t[4], e.t[5], e.t[6], e.t[7], e.t[8], e.t[9]);
        const float dur = run_entry(*e.init, *e.exec, spfilter, a.B, Hin, Win, a.stride, IFMap.device_ptr, OFMap.device_ptr);
        printf("%f (us) %f (effective tflop/s)\n", dur * 1e3, gflop_count / dur);
        fflush(stdout);
        lines++;
        if (a.one_tile) break;
    }
    if (lines == 0) std::cerr << "no operator for block size " << a.block_sz << "\n";
    return 0;
}
