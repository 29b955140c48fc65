// The three usage flows the reference ships as examples, written against this library's headers and
// linked against libblock_sparse.a only (no test oracle): header-form SpMM with D = A*B + C and the
// library's own get_host_reference as the check (example/spmm.blockwise.cu:17-52), a weight loaded from
// its text dump (example/load_bsr.spmm.blockwise.cu:10-28), and the header-form convolution
// (example/spconv.blockwise.cu:17-52, once over NHWC feature maps and once over the reference's own C-H-W-B / F-H-W-B).
// A fourth flow checks that dump() of a synced weight is read-only: sync, initialize, dump, launch.
#include <cmath>
#include <sstream>
#include "block_sparse/cuda_array.h"
#include "block_sparse/spconv/spconv_op.h"
#include "block_sparse/spmm/spmm_op.h"

// the acceptance rule of the reference's examples: |ref - d| <= 1e-3 |ref| for every element
static bool close_enough(const std::vector<half>& got, const std::vector<float>& ref, const char* what)
{
    if (got.size() != ref.size()) {
        printf("%s: %zu results for %zu reference values\n", what, got.size(), ref.size());
        return false;
    }
    size_t bad = 0;
    for (size_t i = 0; i < ref.size(); i++) {
        const float d = static_cast<float>(got[i]);
        if (!(std::fabs(ref[i] - d) <= 1e-3f * std::fabs(ref[i]))) {
            if (bad++ < 5) printf("%s: element %zu, result %f != %f\n", what, i, d, ref[i]);
        }
    }
    return bad == 0;
}

static bool spmm_flow(BlockwiseSpMatrix<half>& spmat, int n, const char* what, bool dump_before_launch = false)
{
    const int m = spmat.nrow, k = spmat.ncol;
    spmat.transform_and_sync_device();

    CudaRandomArray<half> B;
    CudaOnesArray<half> C;
    CudaZerosArray<half> D;
    B.initialize(k * n);
    C.initialize(m * n);
    D.initialize(m * n);
    B.sync_device();
    C.sync_device();
    D.sync_device();

    SpmmBlockwiseOp<ShapeBase<32, 128, 32>, ShapeBase<32, 32, 32>, ShapeBase<16, 16, 16>, 3> op;
    op.initialize(spmat, n, B.device_ptr, C.device_ptr, D.device_ptr);
    if (dump_before_launch) {
        std::ostringstream sink;
        spmat.dump(sink); // must leave the device image and the operator state alone
        if (!spmat.device_synced) {
            printf("%s: dump() dropped the device image\n", what);
            return false;
        }
    }
    op();
    HIP_CHECK(hipDeviceSynchronize());
    D.sync_host();

    std::vector<float> D_ref(static_cast<size_t>(m) * n);
    get_host_reference<half>(spmat, n, B.host_array, 1.0f, C.host_array, 1.0f, D_ref);
    const bool ok = close_enough(D.host_array, D_ref, what);
    std::cout << what << " (" << spmat.config_str << ")" << (ok ? " Passed" : " Failed") << "\n";
    return ok;
}

static bool spconv_flow(int stride, bool filter_permute)
{
    const int B = 32, H = 14, W = 14, C = 256, F = 256, R = 3, S = 3, block_sz = 32;
    BlockwiseSpFilter<half> spfilter;
    spfilter.init_random(F, R, S, C, block_sz, 1, 0.2f, filter_permute, 2021u);
    spfilter.transform_and_sync_device();

    // H, W are the output extents of the example; the input is (H*stride) x (W*stride)
    const int Hin = H * stride, Win = W * stride;
    CudaRandomArray<half> IFMap;
    CudaZerosArray<half> OFMap;
    IFMap.initialize(B * Hin * Win * C);
    OFMap.initialize(B * H * W * F);
    IFMap.sync_device();
    OFMap.sync_device();

    SpconvBlockwiseOp<ShapeBase<block_sz, 128, 32>, ShapeBase<32, 32, 32>, ShapeBase<16, 16, 16>, 3> op;
    op.initialize(spfilter, B, Hin, Win, stride, IFMap.device_ptr, OFMap.device_ptr);
    op();
    HIP_CHECK(hipDeviceSynchronize());
    OFMap.sync_host();

    std::vector<float> OFMap_ref;
    get_host_reference<half>(spfilter, B, Hin, Win, stride, IFMap.host_array, OFMap_ref, filter_channel_first);
    const bool ok = close_enough(OFMap.host_array, OFMap_ref, "spconv example");
    std::cout << "spconv example stride " << stride << " (" << spfilter.config_str << ")" << (ok ? " Passed" : " Failed")
              << "\n";
    return ok;
}

// example/spconv.blockwise.cu as it stands: C-H-W-B input allocated for (H*stride) x (W*stride), F-H-W-B output, the
// comparison indexed nn + (ww + (hh + ff*H)*W)*B
static bool spconv_flow_reference_layout(int stride)
{
    const int B = 32, H = 14, W = 14, C = 256, F = 256, R = 3, S = 3, block_sz = 32;
    BlockwiseSpFilter<half> spfilter;
    spfilter.init_random(F, R, S, C, block_sz, 1, 0.2f, false, 2021u);
    spfilter.fmap_layout = fmap_batch_first;
    spfilter.transform_and_sync_device();

    CudaRandomArray<half> IFMap;
    CudaZerosArray<half> OFMap;
    IFMap.initialize(B * (H * stride) * (W * stride) * C);
    OFMap.initialize(B * H * W * F);
    IFMap.sync_device();
    OFMap.sync_device();

    SpconvBlockwiseOp<ShapeBase<block_sz, 128, 32>, ShapeBase<32, 32, 32>, ShapeBase<16, 16, 16>, 3> op;
    op.initialize(spfilter, B, H, W, stride, IFMap.device_ptr, OFMap.device_ptr);
    op();
    HIP_CHECK(hipDeviceSynchronize());
    OFMap.sync_host();

    std::vector<float> OFMap_ref(B * H * W * F);
    get_host_reference<half>(spfilter, B, H, W, stride, IFMap.host_array, OFMap_ref, filter_channel_first);
    bool passed = true;
    for (int nn = 0; nn < B; nn++)
        for (int hh = 0; hh < H; hh++)
            for (int ww = 0; ww < W; ww++)
                for (int ff = 0; ff < F; ff++) {
                    const int idx = nn + (ww + (hh + ff * H) * W) * B;
                    const float o = static_cast<float>(OFMap.host_array[idx]), o_ref = OFMap_ref[idx];
                    if (!(std::fabs(o_ref - o) <= 1e-3f * std::fabs(o_ref))) {
                        if (passed) printf("n = %d, h = %d, w = %d, f = %d, result %f != %f\n", nn, hh, ww, ff, o, o_ref);
                        passed = false;
                    }
                }
    std::cout << "spconv example, reference layout, stride " << stride << " (" << spfilter.config_str << ")"
              << (passed ? " Passed" : " Failed") << "\n";
    return passed;
}

int main()
{
    int failures = 0;
    {
        BlockwiseSpMatrix<half> spmat; // example/spmm.blockwise.cu: 1024^3, block 32, density 0.2, seed 2021
        spmat.init_random(1024, 1024, 32, 1, 0.2f, false, 2021u);
        failures += !spmm_flow(spmat, 1024, "spmm example");
    }
    {
        // example/load_bsr.spmm.blockwise.cu reads the dump of such a weight from its standard input
        BlockwiseSpMatrix<half> source, spmat;
        source.init_random(1024, 1024, 32, 1, 0.2f, true, 2021u);
        std::stringstream text;
        source.dump(text);
        spmat.load(text);
        std::cout << "Finish matrix loading. Summary:\n" << spmat.config_str << std::endl;
        failures += !(spmat.brow == 32);
        failures += !spmm_flow(spmat, 1024, "load_bsr example");
    }
    {
        BlockwiseSpMatrix<half> spmat;
        spmat.init_random(512, 512, 32, 1, 0.2f, true, 7u);
        failures += !spmm_flow(spmat, 256, "dump between initialize and launch", true);
    }
    failures += !spconv_flow(1, false);
    failures += !spconv_flow(2, true);
    failures += !spconv_flow_reference_layout(1);
    failures += !spconv_flow_reference_layout(2);
    std::cout << (failures ? "FAILED " : "ALL PASSED ") << failures << " failure(s)\n";
    return failures ? EXIT_FAILURE : EXIT_SUCCESS;
}
