// Every entry of the SpConv operator table against the CPU oracle, after the reference's
// test/test.spconv.blockwise.cu:10-14 (cases 128 x 14 x 14 x 256 -> 256, 3 x 3, stride 1 and 2,
// density 0.1, seed 2021), with NHWC feature maps and a true stride: the input is
// (h*stride) x (w*stride), the output h x w.  Plain and filter-permuted weights.  The batch is
// cut to 16 images to keep the CPU oracle quick; N = 16*14*14 = 3136 still leaves a ragged tile.
// Then the same filters over the reference's own batch-innermost tensors.
#include <cmath>
#include <tuple>
#include "block_sparse/cuda_array.h"
#include "block_sparse/spconv/spconv_library_decl.h"
#include "block_sparse/spconv/spconv_op.h"
#include "oracle_reference.h"

struct TableEntry {
    const char* name;
    int block_sz;
    SpconvBlockwiseInitFn_t* init;
    SpconvBlockwiseExecFn_t* exec;
};
#define STR2(x) #x
#define STR(x) STR2(x)
#define SHFLBW_TILE(BM, ...)                                                               \
    {STR(NAME_FUN(SpconvBlockwise, Init, BM, __VA_ARGS__)), BM, &NAME_FUN(SpconvBlockwise, Init, BM, __VA_ARGS__), \
     &NAME_FUN(SpconvBlockwise, Exec, BM, __VA_ARGS__)},
static const TableEntry table[] = {
#include "block_sparse/common/library_table.def"
};
#undef SHFLBW_TILE

static bool verify(SpconvBlockwiseInitFn_t init_fn, SpconvBlockwiseExecFn_t exec_fn, BlockwiseSpFilter<half>& f, int n,
                   int h_in, int w_in, int stride, CudaRandomArray<half>& IFMap, CudaZerosArray<half>& OFMap,
                   const std::vector<float>& ref)
{
    HIP_CHECK(hipDeviceSynchronize());
    HIP_CHECK(hipMemset(OFMap.device_ptr, 0xff, sizeof(half) * OFMap.size));
    SpconvBlockwiseOpState state = (*init_fn)(f, n, h_in, w_in, stride, IFMap.device_ptr, OFMap.device_ptr);
    if (!state.initSuccess) {
        std::cerr << "return due to unsuccessful initialization. " << std::endl;
        return false;
    }
    (*exec_fn)(state, nullptr);
    if (!isHipSuccess(hipDeviceSynchronize()) || !isHipSuccess(hipGetLastError())) {
        std::cerr << "kernel failed." << std::endl;
        return false;
    }
    OFMap.sync_host();
    return checkEqual<half>(ref.size(), OFMap.host_array, ref, true);
}

static int test_block_size(int block_sz, int n, int h, int w, int c, int f, int r, int s, int stride, float density,
                           unsigned seed)
{
    int failures = 0;
    BlockwiseSpFilter<half> plain, permuted;
    plain.init_random(f, r, s, c, block_sz, 1, density, false, seed);
    plain.transform_and_sync_device();
    permuted.init_random(f, r, s, c, block_sz, 1, density, true, seed);
    permuted.transform_and_sync_device();

    const int h_in = h * stride, w_in = w * stride;
    CudaRandomArray<half> IFMap;
    CudaZerosArray<half> OFMap;
    IFMap.initialize(n * h_in * w_in * c);
    OFMap.initialize(n * h * w * f);

    std::vector<float> ref_plain, ref_permuted;
    oracle_reference<half>(plain, n, h_in, w_in, stride, IFMap.host_array, ref_plain);
    oracle_reference<half>(permuted, n, h_in, w_in, stride, IFMap.host_array, ref_permuted);
    if (ref_plain.size() != static_cast<size_t>(OFMap.size)) {
        std::cerr << "output extent mismatch\n";
        return 1;
    }
    for (const TableEntry& e : table) {
        if (e.block_sz != block_sz) continue;
        bool ok0 = verify(*e.init, *e.exec, plain, n, h_in, w_in, stride, IFMap, OFMap, ref_plain);
        bool ok1 = verify(*e.init, *e.exec, permuted, n, h_in, w_in, stride, IFMap, OFMap, ref_permuted);
        std::cout << e.name << " " << plain.config_str << " n=" << n << " h=" << h << " w=" << w << " stride=" << stride
                  << (ok0 ? " Passed" : " Failed") << " | permuted" << (ok1 ? " Passed" : " Failed") << "\n";
        failures += !ok0 + !ok1;
    }

    // the same filters over the reference's own tensors (C-H-W-B in, F-H-W-B out, h x w bounding both)
    plain.fmap_layout = permuted.fmap_layout = fmap_batch_first;
    CudaRandomArray<half> IFMap_bf;
    IFMap_bf.initialize(n * h * w * c);
    oracle_reference_batch_first<half>(plain, n, h, w, stride, IFMap_bf.host_array, ref_plain);
    oracle_reference_batch_first<half>(permuted, n, h, w, stride, IFMap_bf.host_array, ref_permuted);
    for (const TableEntry& e : table) {
        if (e.block_sz != block_sz) continue;
        bool ok0 = verify(*e.init, *e.exec, plain, n, h, w, stride, IFMap_bf, OFMap, ref_plain);
        bool ok1 = verify(*e.init, *e.exec, permuted, n, h, w, stride, IFMap_bf, OFMap, ref_permuted);
        std::cout << e.name << " batch-first " << plain.config_str << " n=" << n << " h=" << h << " w=" << w
                  << " stride=" << stride << (ok0 ? " Passed" : " Failed") << " | permuted" << (ok1 ? " Passed" : " Failed")
                  << "\n";
        failures += !ok0 + !ok1;
    }
    return failures;
}

int main()
{
    const std::tuple<int, int, int, int, int, int, int, int, float, unsigned> cases[] = {
        std::make_tuple(16, 14, 14, 256, 256, 3, 3, 1, 0.1f, 2021u),
        std::make_tuple(16, 14, 14, 256, 256, 3, 3, 2, 0.1f, 2021u),
    };
    int failures = 0;
    for (auto& t : cases)
        for (int block_sz : {16, 32, 64, 128}) {
            if (shflbw_spmm_variant_count(block_sz) == 0) {
                std::cout << "block " << block_sz << ": no native kernel, skipped\n";
                continue;
            }
            failures += test_block_size(block_sz, std::get<0>(t), std::get<1>(t), std::get<2>(t), std::get<3>(t),
                                        std::get<4>(t), std::get<5>(t), std::get<6>(t), std::get<7>(t), std::get<8>(t),
                                        std::get<9>(t));
        }
    std::cout << (failures ? "FAILED " : "ALL PASSED ") << failures << " failure(s)\n";
    return failures ? EXIT_FAILURE : EXIT_SUCCESS;
}
