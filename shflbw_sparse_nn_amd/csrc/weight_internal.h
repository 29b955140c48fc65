// Internal definition of the weight container behind the C ABI (shflbw_weight).
// Host side of the Shfl-BW format: reference block_sparse/spmm/blockwise_format.h:13-68.
#pragma once
#include <cstdint>
#include <mutex>
#include <string>
#include <vector>

#include "shflbw.h"

struct shflbw_weight {
    // shape and pattern (blockwise_format.h:15-22)
    int nrow = 0, ncol = 0, nnzb = 0, brow = 0, bcol = 0;
    float density = 0.f;
    unsigned seed = 0;
    bool row_permute = false;
    int F = 0, R = 0, S = 0, C = 0; // filter view, spconv/blockwise_format.h:19-23

    // original format on host (:25-27)
    std::vector<int> indptr, indices, row_permute_ids;
    std::vector<uint16_t> values; // fp16 bits, column-major inside each block

    // reference-format image (:29-31): indptr | indices*bcol | row_permute_ids
    std::vector<int> meta_h;

    // private image for the gfx950 kernels, built by sync_device
    std::vector<int> group_ptr;      // X+1: cumulative count of 64-slot groups per panel
    std::vector<int> panel_desc;     // 2X: per panel {MFMA k16 steps = ceil(nnz/16), first 64-slot group}
    std::vector<int> packed_indices; // 64 * group_ptr[X]; tail slots hold -1 (a row of zeros)
    std::vector<int> packed_indices_pm; // each 64-slot group reordered: [16p + 4j + r] = packed_indices[16j + 4p + r]
    std::vector<uint16_t> packed_values; // 64 * brow * group_ptr[X]; MFMA fragment order, tail zero
    // slab form of the SpMM (block sizes 32 and 64, ncol <= SLAB_MAX_K; empty otherwise): the ids of every 64-slot
    // group as LDS byte offsets of slab rows, in the order the lanes of a wave load them (see build_packed_image)
    std::vector<int> packed_slab;

    bool initialized = false, device_synced = false;
    std::string config_str;

    // device buffers (owned)
    void* d_meta = nullptr;
    void* d_values = nullptr;
    void* d_group_ptr = nullptr; // holds panel_desc
    void* d_packed_indices = nullptr;
    void* d_packed_indices_pm = nullptr;
    void* d_packed_values = nullptr;
    void* d_packed_slab = nullptr;

    // Device scratch of the convolution, handed out by shflbw_spconv_init under `scratch_lock` and kept until the
    // weight is re-initialised or destroyed (or shflbw_weight_release_scratch).  Two kinds:
    //  * ConvIds: the kept-column ids rewritten as offsets into the layout-transformed input (slot order, then
    //    producer-major order).  They depend on the form and the geometry only, so one copy per (form, B, H, W,
    //    stride) serves every state; never recycled (a few hundred KB per geometry).
    //  * ConvBulk: the layout-transformed input, the filter-major result and the synchronisation words of one
    //    state, keyed by (form, geometry, input tensor, output tensor), so states over different tensors never
    //    share them and may run on different streams.  At most CONV_BULK_DEPTH of them exist per weight: one more
    //    distinct key recycles the least recently initialised one (same size: no allocation, no memset).
    struct ConvIds {
        int key[5]; // form, B, H, W, stride
        void* ptr;
        size_t bytes;
    };
    struct ConvBulk {
        int key[5];
        const void* in;
        const void* out;
        void* ptr;
        size_t bytes;
        unsigned long long stamp; // value of bulk_clock when it was last handed out
    };
    static constexpr int CONV_BULK_DEPTH = SHFLBW_CONV_SCRATCH_DEPTH;
    std::vector<ConvIds> conv_ids;
    std::vector<ConvBulk> conv_bulk;
    unsigned long long bulk_clock = 0;
    std::mutex scratch_lock;
};

namespace shflbw {

void set_error(const char* fmt, ...);

// fp16 bit helpers (IEEE binary16, round to nearest even)
float half_to_float(uint16_t h);
uint16_t float_to_half(float f);

// k-extent of one MFMA step for a block size: 32x32x16 tiles for V >= 32, 16x16x32 for V == 16
inline int mfma_kstep(int brow) { return brow >= 32 ? 16 : 32; }

// Geometry of the slab form of the SpMM: a workgroup holds up to SLAB_MAX_K rows of SLAB_ROW_BYTES bytes (64 columns)
// of B in LDS, one more row of zeros behind them (rounded up to a multiple of 8 rows) for the padding slots.
constexpr int SLAB_ROW_BYTES = 128;
constexpr int SLAB_MAX_K = 1128;
// LDS byte offset of what slot id `k` of a weight with `ncol` columns reads: the start of slab row k with the XOR key
// of the row, (k / 2) % 4, in the position of the 32-byte unit; padding slots (k < 0) read the row of zeros.
inline int slab_row_offset(int k, int ncol)
{
    return k < 0 ? ((ncol + 7) & ~7) * SLAB_ROW_BYTES : k * SLAB_ROW_BYTES + (((k >> 1) & 3) << 5);
}

// Which quarter of the LDS banks the 64 bytes of slab row k that one transposing read touches fall into (the other
// 64 bytes of the row: the same quarter with the lowest bit flipped): rows of different class never collide.
inline int slab_bank_class(int k) { return (k & 1) * 2 + ((k >> 2) & 1); }

// builds group_ptr / packed_indices / packed_values from the host arrays
int build_packed_image(shflbw_weight* w);

// frees device buffers (blockwise_format.h:48-52)
void clear_device(shflbw_weight* w);

} // namespace shflbw
