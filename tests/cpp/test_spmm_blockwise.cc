// Every entry of the SpMM operator table against the CPU oracle, the way the reference's own
// test drives its table (test/test.spmm.blockwise.cu:9-13 for the case, test/test_util.spmm.h:32-63
// for the verify step): plain and row-permuted weight, N = 960 (not a multiple of any tile
// width), inputs are small integers so a correct kernel is exact.  Also the header-form
// operator with D = A*B + C (example/spmm.blockwise.cu:36-50) and the text dump/load round trip.
#include <cmath>
#include <sstream>
#include <tuple>
#include "block_sparse/cuda_array.h"
#include "block_sparse/spmm/spmm_library_decl.h"
#include "block_sparse/spmm/spmm_op.h"
#include "oracle_reference.h"

struct TableEntry {
    const char* name;
    int block_sz;
    SpmmBlockwiseInitFn_t* init;
    SpmmBlockwiseExecFn_t* exec;
};
#define STR2(x) #x
#define STR(x) STR2(x)
#define SHFLBW_TILE(BM, ...)                                                           \
    {STR(NAME_FUN(SpmmBlockwise, Init, BM, __VA_ARGS__)), BM, &NAME_FUN(SpmmBlockwise, Init, BM, __VA_ARGS__), \
     &NAME_FUN(SpmmBlockwise, Exec, BM, __VA_ARGS__)},
static const TableEntry table[] = {
#include "block_sparse/common/library_table.def"
};
#undef SHFLBW_TILE

static bool verify(SpmmBlockwiseInitFn_t init_fn, SpmmBlockwiseExecFn_t exec_fn, BlockwiseSpMatrix<half>& spmat, int N,
                   CudaRandomArray<half>& B, CudaZerosArray<half>& D, const std::vector<float>& D_ref)
{
    HIP_CHECK(hipDeviceSynchronize());
    HIP_CHECK(hipMemset(D.device_ptr, 0xff, sizeof(half) * spmat.nrow * N)); // NaN pattern: every element must be written
    SpmmBlockwiseOpState state = (*init_fn)(spmat, N, B.device_ptr, D.device_ptr);
    if (!state.initSuccess) {
        std::cerr << "return due to unsuccessful initialization. " << std::endl;
        return false;
    }
    (*exec_fn)(state, nullptr);
    if (!isHipSuccess(hipDeviceSynchronize()) || !isHipSuccess(hipGetLastError())) {
        std::cerr << "kernel failed." << std::endl;
        return false;
    }
    D.sync_host();
    return checkEqual<half>(static_cast<size_t>(spmat.nrow) * N, D.host_array, D_ref, true);
}

static int test_block_size(int block_sz, int m, int n, int k, float density, unsigned seed)
{
    int failures = 0;
    BlockwiseSpMatrix<half> plain, permuted;
    plain.init_random(m, k, block_sz, 1, density, false, seed);
    plain.transform_and_sync_device();
    permuted.init_random(m, k, block_sz, 1, density, true, seed);
    permuted.transform_and_sync_device();

    CudaRandomArray<half> B;
    CudaZerosArray<half> C, D;
    B.initialize(k * n);
    C.initialize(m * n);
    D.initialize(m * n);

    std::vector<float> ref_plain, ref_permuted;
    oracle_reference<half>(plain, n, B.host_array, 1.0f, C.host_array, 0.0f, ref_plain);
    oracle_reference<half>(permuted, n, B.host_array, 1.0f, C.host_array, 0.0f, ref_permuted);

    for (const TableEntry& e : table) {
        if (e.block_sz != block_sz) continue;
        bool ok0 = verify(*e.init, *e.exec, plain, n, B, D, ref_plain);
        bool ok1 = verify(*e.init, *e.exec, permuted, n, B, D, ref_permuted);
        std::cout << e.name << " " << plain.config_str << " n=" << n << (ok0 ? " Passed" : " Failed") << " | "
                  << permuted.config_str << (ok1 ? " Passed" : " Failed") << "\n";
        failures += !ok0 + !ok1;
    }

    // header form, D = A*B + C with C = 1 (example/spmm.blockwise.cu)
    {
        CudaOnesArray<half> ones;
        ones.initialize(m * n);
        std::vector<float> ref;
        oracle_reference<half>(permuted, n, B.host_array, 1.0f, ones.host_array, 1.0f, ref);
        bool ok = false;
        auto run = [&](auto& op) {
            op.initialize(permuted, n, B.device_ptr, ones.device_ptr, D.device_ptr);
            op();
            HIP_CHECK(hipDeviceSynchronize());
            D.sync_host();
            ok = checkEqual<half>(static_cast<size_t>(m) * n, D.host_array, ref, true);
        };
        if (block_sz == 32) { SpmmBlockwiseOp<ShapeBase<32, 128, 32>, ShapeBase<32, 32, 32>, ShapeBase<16, 16, 16>, 3> op; run(op); }
        if (block_sz == 64) { SpmmBlockwiseOp<ShapeBase<64, 128, 32>, ShapeBase<32, 32, 32>, ShapeBase<16, 16, 16>, 3> op; run(op); }
        if (block_sz == 128) { SpmmBlockwiseOp<ShapeBase<128, 128, 32>, ShapeBase<32, 32, 32>, ShapeBase<16, 16, 16>, 3> op; run(op); }
        if (block_sz == 16) { SpmmBlockwiseOp<ShapeBase<16, 128, 32>, ShapeBase<16, 32, 32>, ShapeBase<16, 16, 16>, 3> op; run(op); }
        std::cout << "SpmmBlockwiseOp<" << block_sz << "> D=A*B+C " << (ok ? "Passed" : "Failed") << "\n";
        failures += !ok;
    }

    // dump -> load -> dump is the identity on the text, and the reloaded weight computes the same D
    {
        std::stringstream s0, s1;
        permuted.dump(s0);
        BlockwiseSpMatrix<half> again;
        std::stringstream in(s0.str());
        again.load(in);
        again.dump(s1);
        bool ok = s0.str() == s1.str();
        again.transform_and_sync_device();
        for (const TableEntry& e : table)
            if (e.block_sz == block_sz) {
                ok = ok && verify(*e.init, *e.exec, again, n, B, D, ref_permuted);
                break;
            }
        std::cout << "dump/load round trip block " << block_sz << (ok ? " Passed" : " Failed") << "\n";
        failures += !ok;
    }
    return failures;
}

int main(int argc, char** argv)
{
    const std::tuple<int, int, int, float, unsigned> cases[] = {
        std::make_tuple(1024, 960, 1024, 0.1f, 2021u), // N boundary handling
    };
    int failures = 0;
    for (auto& c : cases)
        for (int block_sz : {16, 32, 64, 128}) {
            if (shflbw_spmm_variant_count(block_sz) == 0) {
                std::cout << "block " << block_sz << ": no native kernel, skipped\n";
                continue;
            }
            failures += test_block_size(block_sz, std::get<0>(c), std::get<1>(c), std::get<2>(c), std::get<3>(c),
                                        std::get<4>(c));
        }
    std::cout << (failures ? "FAILED " : "ALL PASSED ") << failures << " failure(s)\n";
    return failures ? EXIT_FAILURE : EXIT_SUCCESS;
}
