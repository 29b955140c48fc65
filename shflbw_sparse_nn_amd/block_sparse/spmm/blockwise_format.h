// Shfl-BW weight container of the C++ veneer: the public members and methods of
// BlockwiseSpMatrix<T> (block_sparse/spmm/blockwise_format.h:13-68) over the C ABI.
//
// The host-visible arrays (indptr, indices, values, row_permute_ids) are plain std::vectors
// the caller may read or fill, exactly as with the reference; transform_and_sync_device()
// hands them to the library, which uploads the reference's meta/data image and builds the
// private matrix-core ordered image the gfx950 kernels read.
#pragma once
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <istream>
#include <iterator>
#include <ostream>
#include <string>
#include <vector>
#include "block_sparse/common/base.h"
#include "block_sparse/hip_error.h"
#include "block_sparse/util/random_mask.h"
#include "shflbw.h"

template <typename T>
struct BlockwiseSpMatrix {
    static_assert(sizeof(T) == 2, "weights are IEEE binary16");

    // shape and pattern (blockwise_format.h:15-22)
    int nrow = 0, ncol = 0, nnzb = 0, brow = 0, bcol = 0;
    float density = 0.f;
    unsigned seed = 0;
    bool row_permute = false;

    // host format (blockwise_format.h:25-27)
    const int alignment = 8;
    std::vector<int> indptr, indices, row_permute_ids;
    std::vector<T> values;

    // packed host image (blockwise_format.h:30-31)
    std::vector<char> meta_h;
    std::vector<T> data_h;

    // device pointers, owned by the library handle (blockwise_format.h:35-42)
    struct DeviceRef {
        void* _meta = nullptr;
        T* _data = nullptr;
        int* csb_indptr = nullptr;
        int* csb_indices = nullptr;
        int* row_permute_ids = nullptr;
        T* csb_values = nullptr;
    } device_ref;

    bool initialized = false;
    bool device_synced = false;
    std::string config_str;

    BlockwiseSpMatrix() { SHFLBW_CHECK(shflbw_weight_create(&handle_)); }
    BlockwiseSpMatrix(const BlockwiseSpMatrix&) = delete;
    BlockwiseSpMatrix& operator=(const BlockwiseSpMatrix&) = delete;
    virtual ~BlockwiseSpMatrix() { shflbw_weight_destroy(handle_); } // frees the device image too (:48-58)

    void init_random(int nrow_, int ncol_, int brow_, int bcol_, float expected_density, bool row_permute_,
                     unsigned seed_)
    {
        SHFLBW_CHECK(shflbw_weight_init_random(handle_, nrow_, ncol_, brow_, bcol_, expected_density,
                                               row_permute_ ? 1 : 0, seed_));
        pull_host_arrays();
    }

    void load(std::istream& in)
    {
        std::string text((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
        SHFLBW_CHECK(shflbw_weight_load_text(handle_, text.data(), text.size()));
        pull_host_arrays();
    }

    // read-only as in the reference (blockwise_format.h:125-149): handing over vectors the library already
    // holds changes nothing, so a synced weight stays synced and its operator states stay valid
    void dump(std::ostream& out)
    {
        push_host_arrays();
        size_t need = 0;
        SHFLBW_CHECK(shflbw_weight_dump_text(handle_, nullptr, 0, &need));
        std::string text(need, '\0');
        SHFLBW_CHECK(shflbw_weight_dump_text(handle_, &text[0], text.size(), &need));
        out.write(text.data(), static_cast<std::streamsize>(need));
    }

    void transform_and_sync_device()
    {
        assert(initialized && "must call initialize() before sync to device.\n");
        push_host_arrays();
        SHFLBW_CHECK(shflbw_weight_sync_device(handle_));
        const int* meta = nullptr;
        size_t n_ints = 0;
        SHFLBW_CHECK(shflbw_weight_meta_host(handle_, &meta, &n_ints));
        meta_h.assign(reinterpret_cast<const char*>(meta), reinterpret_cast<const char*>(meta + n_ints));
        data_h = values;
        shflbw_device_ref r;
        SHFLBW_CHECK(shflbw_weight_device_ref(handle_, &r));
        device_ref._meta = r.meta;
        device_ref._data = static_cast<T*>(r.data);
        device_ref.csb_indptr = const_cast<int*>(r.csb_indptr);
        device_ref.csb_indices = const_cast<int*>(r.csb_indices);
        device_ref.row_permute_ids = const_cast<int*>(r.row_permute_ids);
        device_ref.csb_values = static_cast<T*>(const_cast<void*>(r.csb_values));
        device_synced = true;
    }

    // the C-ABI handle (for the operators of this veneer)
    shflbw_weight* handle() const { return handle_; }

protected:
    shflbw_weight* handle_ = nullptr;
    int filter_R_ = 0, filter_S_ = 0, filter_C_ = 0; // set by the filter subclass

    // library -> public members, after the library generated or parsed a weight
    void pull_host_arrays()
    {
        shflbw_weight_info info;
        SHFLBW_CHECK(shflbw_weight_get_info(handle_, &info));
        nrow = info.nrow, ncol = info.ncol, nnzb = info.nnzb, brow = info.brow, bcol = info.bcol;
        density = info.density, seed = info.seed, row_permute = info.row_permute != 0;
        const int *ip = nullptr, *ix = nullptr, *perm = nullptr;
        const uint16_t* v = nullptr;
        SHFLBW_CHECK(shflbw_weight_host_arrays(handle_, &ip, &ix, &v, &perm));
        indptr.assign(ip, ip + nrow / brow + 1);
        indices.assign(ix, ix + nnzb);
        values.resize(static_cast<size_t>(nnzb) * brow * bcol);
        std::memcpy(static_cast<void*>(values.data()), v, values.size() * sizeof(T));
        if (row_permute) row_permute_ids.assign(perm, perm + nrow);
        else row_permute_ids.clear();
        config_str = shflbw_weight_config_str(handle_);
        initialized = true;
        device_synced = false;
    }

    // public members -> library, so edits made by the caller (the reference lets users fill the
    // vectors by hand, example/spmatrix_dump_load.md) are what gets dumped or uploaded
    void push_host_arrays()
    {
        if (!initialized) return;
        SHFLBW_CHECK(shflbw_weight_set(handle_, nrow, ncol, brow, bcol, nnzb, indptr.data(), indices.data(),
                                       reinterpret_cast<const uint16_t*>(values.data()),
                                       row_permute ? row_permute_ids.data() : nullptr, filter_R_, filter_S_,
                                       filter_C_));
        // edited vectors drop the device image, as a new init_random does in the reference (:118-122)
        shflbw_weight_info info;
        SHFLBW_CHECK(shflbw_weight_get_info(handle_, &info));
        device_synced = info.device_synced != 0;
    }

    template <typename U>
    friend void get_host_reference(BlockwiseSpMatrix<U>& spmat, const int N, const std::vector<U>& B, float alpha,
                                   const std::vector<U>& C, float beta, std::vector<float>& D_ref);

};

// D_ref = alpha * A*B + beta * C on the CPU, fp32, M x N row-major (blockwise_format.h:268-311): the check
// the reference's examples run after the GPU launch.  Computed by the library's host code from the public
// vectors of `spmat`.
template <typename T>
void get_host_reference(BlockwiseSpMatrix<T>& spmat, const int N, const std::vector<T>& B, float alpha,
                        const std::vector<T>& C, float beta, std::vector<float>& D_ref)
{
    spmat.push_host_arrays();
    D_ref.resize(static_cast<size_t>(spmat.nrow) * N);
    SHFLBW_CHECK(shflbw_spmm_host_reference(spmat.handle(), N, reinterpret_cast<const uint16_t*>(B.data()), alpha,
                                            C.empty() ? nullptr : reinterpret_cast<const uint16_t*>(C.data()),
                                            C.empty() ? 0.f : beta, D_ref.data()));
}
