// Device side of the C ABI: uploads of the weight images and the SpMM / SpConv
// init + exec entry points.  Reference: block_sparse/spmm/blockwise_format.h:230-266
// (upload), block_sparse/spmm/blockwise_op.h:81-215 and
// block_sparse/spconv/blockwise_op.h:79-193 (init / exec).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "shflbw.h"
#include "spconv_launch.h"
#include "spmm_launch.h"
#include "weight_internal.h"

namespace shflbw {

#define SHFLBW_HIP_TRY(expr)                                                                            \
    do {                                                                                                \
        hipError_t e_ = (expr);                                                                         \
        if (e_ != hipSuccess) {                                                                         \
            set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__);       \
            return SHFLBW_ERR_HIP;                                                                      \
        }                                                                                               \
    } while (0)

static void release_conv_scratch(shflbw_weight* w);

void clear_device(shflbw_weight* w)
{
    void** bufs[] = {&w->d_meta, &w->d_values, &w->d_group_ptr, &w->d_packed_indices, &w->d_packed_indices_pm,
                     &w->d_packed_values, &w->d_packed_slab};
    for (void** b : bufs) {
        if (*b) (void)hipFree(*b);
        *b = nullptr;
    }
    release_conv_scratch(w);
}

// frees every device buffer the convolution inits of this weight allocated (the caller holds scratch_lock or owns w)
void release_conv_scratch(shflbw_weight* w)
{
    for (auto& e : w->conv_ids)
        if (e.ptr) (void)hipFree(e.ptr);
    for (auto& e : w->conv_bulk)
        if (e.ptr) (void)hipFree(e.ptr);
    w->conv_ids.clear();
    w->conv_bulk.clear();
}

static int upload_one(void** dst, const void* src, size_t bytes)
{
    // zero-length arrays (an empty matrix) still get a valid pointer
    SHFLBW_HIP_TRY(hipMalloc(dst, bytes ? bytes : 16));
    if (bytes) SHFLBW_HIP_TRY(hipMemcpy(*dst, src, bytes, hipMemcpyHostToDevice));
    return SHFLBW_OK;
}

int upload(shflbw_weight* w)
{
    int rc;
    if ((rc = upload_one(&w->d_meta, w->meta_h.data(), w->meta_h.size() * sizeof(int))) ||
        (rc = upload_one(&w->d_values, w->values.data(), w->values.size() * sizeof(uint16_t))) ||
        (rc = upload_one(&w->d_group_ptr, w->panel_desc.data(), w->panel_desc.size() * sizeof(int))) ||
        (rc = upload_one(&w->d_packed_indices, w->packed_indices.data(), w->packed_indices.size() * sizeof(int))) ||
        (rc = upload_one(&w->d_packed_indices_pm, w->packed_indices_pm.data(),
                         w->packed_indices_pm.size() * sizeof(int))) ||
        (rc = upload_one(&w->d_packed_values, w->packed_values.data(), w->packed_values.size() * sizeof(uint16_t))) ||
        (rc = upload_one(&w->d_packed_slab, w->packed_slab.data(), w->packed_slab.size() * sizeof(int)))) {
        clear_device(w);
        return rc;
    }
    return SHFLBW_OK;
}

// compute units of the current device, looked up once per device
static int device_compute_units()
{
    static std::mutex lock;
    static int cached[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    std::lock_guard<std::mutex> guard(lock);
    if (cached[dev] == 0) {
        int n = 0;
        cached[dev] = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0 ? n : 256;
    }
    return cached[dev];
}

static const SpmmVariant* find_spmm_variant(int brow, int variant, int* n_for_brow)
{
    int count = 0;
    const SpmmVariant* all = spmm_variants(&count);
    const SpmmVariant* hit = nullptr;
    int seen = 0;
    for (int i = 0; i < count; i++) {
        if (all[i].V != brow) continue;
        if (seen == variant) hit = &all[i];
        seen++;
    }
    if (n_for_brow) *n_for_brow = seen;
    return hit;
}

static const SpconvVariant* find_spconv_variant(int brow, int variant, int* n_for_brow)
{
    int count = 0;
    const SpconvVariant* all = spconv_variants(&count);
    const SpconvVariant* hit = nullptr;
    int seen = 0;
    for (int i = 0; i < count; i++) {
        if (all[i].V != brow) continue;
        if (seen == variant) hit = &all[i];
        seen++;
    }
    if (n_for_brow) *n_for_brow = seen;
    return hit;
}

// the persistent role-split variants ("ws..." names) form gather addresses from 32-bit byte offsets
static bool spmm_variant_offsets32(const SpmmVariant* v) { return v && v->name[0] == 'w'; }

// Tile choice when the caller does not force one: the table lists the preferred (persistent, 512 columns
// wide) variant of every block size first.  When its tiles would occupy at most half of the compute units,
// the role-split variant with 256-column tiles is taken instead (twice the tiles; measured 15-25 % faster
// there, 5-20 % slower once the wide tiles fill the chip), and the one with 128-column tiles while even those
// are no more than the compute units.
// Block height 32 and at most SLAB_MAX_K columns: the slab variant moves less data between the L2 and the
// compute units once a workgroup runs enough kept vectors over the 128 KiB slab it has to load first.  Taken
// when (34 shapes measured with both kernels, each pair on one box)
//  * a workgroup's panels keep at least 3 vectors per column of A on average (3.2: 5 % faster, 2.4: 5-20 %
//    slower, 1.6: equal to 30 % slower: the slab load is not paid back),
//  * A has at least 384 columns (at 256 B fits the L2, the gathers of the role-split kernel all hit, and the
//    two kernels tie),
//  * there are at least 32 column tiles, so that four or more workgroups of an XCD stream the same chunk of A
//    at the same time and share it in their L2 (16 tiles: 15 % slower).
// Inside these bounds: equal to 28 % faster (M = 4096, K = 1024, N = 4096, density 0.2: 15.1 against 16.5 us;
// M = 8192, density 0.3: 31.3 against 38.7 us).
static int auto_spmm_variant(const shflbw_weight* w, int N, bool allow_slab)
{
    const int brow = w->brow, X = w->nrow / w->brow;
    int count = 0;
    const SpmmVariant* all = spmm_variants(&count);
    if (allow_slab && brow == 32 && !w->packed_slab.empty() && w->ncol >= 384 && X > 0) {
        int seen = 0;
        for (int i = 0; i < count; i++) {
            if (all[i].V != brow) continue;
            if (all[i].max_k >= w->ncol) {
                const int cus = (device_compute_units() / 8) * 8;
                const int n_tiles = (N + all[i].BN - 1) / all[i].BN;
                const int chunks = std::max(1, std::min(X, cus / n_tiles)); // as the launcher deals the panels
                const double panels_per_wg = (double)X / chunks;
                const double vectors_per_column = panels_per_wg * w->nnzb / ((double)X * w->ncol);
                if (vectors_per_column >= 3.0 && n_tiles >= 32) return seen;
            }
            seen++;
        }
    }
    // the role-split variant of this block size with tiles of `bn` columns, -1 when there is none
    auto role_split_with = [&](int bn) {
        int seen = 0;
        for (int i = 0; i < count; i++) {
            if (all[i].V != brow) continue;
            if (all[i].name[0] == 'w' && all[i].BN == bn) return seen; // "ws..." names
            seen++;
        }
        return -1;
    };
    // small problems: 128-column tiles while they do not outnumber the compute units (39 shapes of block heights 32, 64
    // and 128 measured against the wider tiles: 6-17 % faster up to one tile per compute unit, 10-25 % slower from two on)
    if ((long)X * ((N + 127) / 128) <= device_compute_units()) {
        const int narrow = role_split_with(128);
        if (narrow >= 0) return narrow;
    }
    const SpmmVariant* first = find_spmm_variant(brow, 0, nullptr);
    if (!first || first->BN != 512) return 0;
    const long wide_tiles = (long)X * ((N + 511) / 512);
    if (wide_tiles > device_compute_units() / 2) return 0;
    const int medium = role_split_with(256);
    return medium >= 0 ? medium : 0;
}

// Geometry of the plane form of a convolution and the layout of its device scratch.
struct PlaneForm {
    int PH, PW;     // rows and (padded to 8) columns of one phase plane
    int copies;     // 2 when some tap offset is odd (a second copy moved by one value keeps gathers aligned)
    long np;        // plane positions = columns of the SpMM in the middle
    long pitch;     // values per channel row of the plane tensor
    long rows;      // channel rows: copies * stride^2 * C
    size_t slots;   // padded kept-vector slots of the filter
    int Ho, Wo;
    size_t planes_bytes, dm_bytes, ids_bytes; // planes | result_fm, and (the entry point without allocation) | ids | ids_pm behind them
    size_t total_bytes() const { return planes_bytes + dm_bytes + 2 * ids_bytes; }
};

static int plane_form_geometry(const shflbw_weight* f, int B, int H, int W, int stride, PlaneForm* g)
{
    const int s = stride, ph = f->R / 2, pw = f->S / 2;
    g->PH = (H + 2 * ph + s - 1) / s;
    g->PW = ((W + 2 * pw + s - 1) / s + 7) / 8 * 8;
    g->np = (long)B * g->PH * g->PW;
    const long max_shift = (long)((f->R - 1) / s) * g->PW + (f->S - 1) / s; // largest tap offset
    g->pitch = (g->np + max_shift + 8 + 63) / 64 * 64;
    g->copies = (f->S - 1) / s >= 1 ? 2 : 1;
    if (g->copies * s * s > 32) {
        set_error("spconv: stride %d has too many phase planes for the plane form", s);
        return SHFLBW_ERR_UNSUPPORTED;
    }
    g->rows = (long)g->copies * s * s * f->C;
    if (g->np > 0x7fffffffL || (unsigned long long)(g->rows + 1) * (unsigned long long)g->pitch * 2ull > 0xffffffffull) {
        set_error("spconv: problem too large for the plane form (%ld rows of %ld positions)", g->rows, g->pitch);
        return SHFLBW_ERR_UNSUPPORTED;
    }
    auto up256 = [](size_t n) { return (n + 255) / 256 * 256; };
    g->slots = f->packed_indices.size();
    g->planes_bytes = up256((size_t)(g->rows + 1) * g->pitch * 2); // one more row: zeros, for the padding slots
    g->dm_bytes = up256((size_t)f->F * g->np * 2);
    g->ids_bytes = up256(g->slots * sizeof(int) + 64);
    g->Ho = (H + 2 * ph - f->R) / s + 1;
    g->Wo = (W + 2 * pw - f->S) / s + 1;
    return SHFLBW_OK;
}

// launch arguments of the SpMM kernels from a state; BN is the tile width of the kernel that will run
static void fill_spmm_launch_args(const shflbw_spmm_state* state, int BN, SpmmLaunchArgs* out)
{
    SpmmLaunchArgs& a = *out;
    a.M = state->args.M;
    a.N = state->args.N;
    a.K = state->args.K;
    a.X = a.M / state->brow;
    a.n_tiles = 0;
    a.packedA = (const half8_t*)state->packed_values;
    a.kidx = state->packed_indices;
    a.kidx_pm = state->packed_indices_pm;
    a.slab_ids = state->packed_slab;
    a.slab_chunks = 1;
    a.panel_desc = state->panel_ptr;
    a.row_ids = state->args.A_row_indices;
    a.B = (const half_t*)state->args.B;
    a.ldb_bytes = state->ldb_bytes;
    a.zero_row = state->zero_row;
    a.C = (const half_t*)state->args.C;
    a.D = (half_t*)state->args.D;
    a.alpha = state->args.alpha;
    a.beta = state->args.beta;
    a.num_cus = device_compute_units();
    a.ldd = a.N;
    a.dmap_row = a.dmap_valid = 0, a.dmap_magic = 0;
    // rows of B one column tile can touch: above about 2.5 MB they do not stay in the 4 MB L2 of an XCD
    // from one round of tiles to the next, and alternating the direction of the walk pays (measured:
    // +1 % at 2 MB, -4 % at 3 MB, -7 % at 4 MB, -13 % at 8 MB)
    a.alternate = (double)a.K * a.ldb_bytes * BN / (a.N > 0 ? a.N : 1) > 2.5 * 1024 * 1024;
}

} // namespace shflbw

using namespace shflbw;

extern "C" {

int shflbw_spmm_variant_count(int brow)
{
    int n = 0;
    find_spmm_variant(brow, 0, &n);
    return n;
}

const char* shflbw_spmm_variant_name(int brow, int variant)
{
    const SpmmVariant* v = find_spmm_variant(brow, variant, nullptr);
    return v ? v->name : "";
}

// `gather_only`: the caller will point the gather at something other than a K x N matrix (the planes of a
// convolution, ids rewritten as element offsets), which only the variants that gather rows by id can walk: the
// variants that hold all K rows of B in LDS are left out of the automatic choice and refused when forced.
static int spmm_init_impl(shflbw_spmm_state* state, const shflbw_weight* w, int N, const void* B, const void* C, void* D,
                          float alpha, float beta, int variant, bool gather_only)
{
    if (!state) return SHFLBW_ERR_INVALID;
    memset(state, 0, sizeof(*state));
    if (!w || !B || !D) {
        set_error("spmm_init: null weight, B or D");
        return SHFLBW_ERR_INVALID;
    }
    if (!w->device_synced) { // assert at blockwise_op.h:87
        set_error("spmm_init: sparse matrix is not synced to device");
        return SHFLBW_ERR_STATE;
    }
    if (w->bcol != 1) { // assert at blockwise_op.h:86 (BK = 1)
        set_error("spmm_init: bcol must be 1 (got %d)", w->bcol);
        return SHFLBW_ERR_UNSUPPORTED;
    }
    if (N <= 0 || (N % 8) != 0) {
        set_error("spmm_init: N must be a positive multiple of 8 (got %d)", N);
        return SHFLBW_ERR_SHAPE;
    }
    if (beta != 0.f && !C) {
        set_error("spmm_init: beta != 0 needs C");
        return SHFLBW_ERR_INVALID;
    }
    if (((uintptr_t)B | (uintptr_t)D | (uintptr_t)C) & 15) {
        set_error("spmm_init: B, C and D must be 16-byte aligned");
        return SHFLBW_ERR_INVALID;
    }
    const int X = w->nrow / w->brow;
    // the role-split kernels address the rows of B with 32-bit byte offsets
    const bool wide_b = (unsigned long long)w->ncol * (unsigned long long)N * 2ull + (unsigned long long)N * 2ull > 0xffffffffull;
    if (variant < 0) {
        variant = auto_spmm_variant(w, N, !gather_only);
        if (wide_b) { // first variant of this block size with 64-bit addressing
            int n = 0;
            find_spmm_variant(w->brow, 0, &n);
            for (int i = 0; i < n; i++)
                if (!spmm_variant_offsets32(find_spmm_variant(w->brow, i, nullptr))) {
                    variant = i;
                    break;
                }
        }
    }
    const SpmmVariant* v = find_spmm_variant(w->brow, variant, nullptr);
    if (!v) {
        set_error("spmm_init: no tile variant %d for block size %d", variant, w->brow);
        return SHFLBW_ERR_UNSUPPORTED;
    }
    if (v->max_k > 0 && gather_only) {
        set_error("spmm_init: tile variant %s holds the rows of B in LDS and cannot walk the planes of a convolution", v->name);
        return SHFLBW_ERR_UNSUPPORTED;
    }
    if (v->max_k > 0 && (w->ncol > v->max_k || w->packed_slab.empty())) {
        set_error("spmm_init: tile variant %s holds all rows of B in LDS: at most %d columns of A (got %d)", v->name,
                  v->max_k, w->ncol);
        return SHFLBW_ERR_UNSUPPORTED;
    }
    if (wide_b && spmm_variant_offsets32(v)) {
        set_error("spmm_init: B (%d x %d fp16) exceeds the 4 GiB the tile variant %s can address", w->ncol, N, v->name);
        return SHFLBW_ERR_UNSUPPORTED;
    }
    SHFLBW_HIP_TRY(v->prepare());

    shflbw_device_ref ref;
    shflbw_weight_device_ref(w, &ref);
    state->args.M = w->nrow;
    state->args.N = N;
    state->args.K = w->ncol;
    state->args.A_values = ref.csb_values;
    state->args.B = B;
    state->args.C = C;
    state->args.D = D;
    state->args.A_bsr_indptr = ref.csb_indptr;
    state->args.A_bsr_indices = ref.csb_indices;
    state->args.A_row_indices = ref.row_permute_ids;
    state->args.alpha = alpha;
    state->args.beta = beta;
    state->packed_values = w->d_packed_values;
    state->packed_indices = (const int*)w->d_packed_indices;
    state->packed_indices_pm = (const int*)w->d_packed_indices_pm;
    state->packed_slab = w->packed_slab.empty() ? nullptr : (const int*)w->d_packed_slab;
    state->panel_ptr = (const int*)w->d_group_ptr;
    state->brow = w->brow;
    state->ldb_bytes = N * 2;
    state->zero_row = spmm_zero_row();
    if (!state->zero_row) {
        set_error("spmm_init: cannot look up the library's row of zeros on this device");
        return SHFLBW_ERR_HIP;
    }
    state->variant = variant;
    state->shared_mem_size = (size_t)v->lds_bytes;
    state->grid_dim[0] = (unsigned)(X * ((N + v->BN - 1) / v->BN));
    state->grid_dim[1] = state->grid_dim[2] = 1;
    state->block_dim[0] = (unsigned)v->threads;
    state->block_dim[1] = state->block_dim[2] = 1;
    state->init_success = 1;
    return SHFLBW_OK;
}

int shflbw_spmm_init_variant(shflbw_spmm_state* state, const shflbw_weight* w, int N, const void* B, const void* C,
                             void* D, float alpha, float beta, int variant)
{
    return spmm_init_impl(state, w, N, B, C, D, alpha, beta, variant, false);
}

int shflbw_spmm_init(shflbw_spmm_state* state, const shflbw_weight* w, int N, const void* B, const void* C, void* D,
                     float alpha, float beta)
{
    return shflbw_spmm_init_variant(state, w, N, B, C, D, alpha, beta, -1);
}

int shflbw_spmm_exec(const shflbw_spmm_state* state, void* stream)
{
    if (!state || !state->init_success) {
        set_error("spmm_exec: state was not initialised successfully");
        return SHFLBW_ERR_STATE;
    }
    const SpmmVariant* v = find_spmm_variant(state->brow, state->variant, nullptr);
    if (!v) return SHFLBW_ERR_UNSUPPORTED;
    SpmmLaunchArgs a;
    fill_spmm_launch_args(state, v->BN, &a);
    if (a.X == 0) return SHFLBW_OK;
    hipError_t e = v->launch(a, (hipStream_t)stream);
    if (e != hipSuccess) {
        set_error("spmm_exec: launch failed: %s", hipGetErrorString(e));
        return SHFLBW_ERR_HIP;
    }
    return SHFLBW_OK;
}


int shflbw_spconv_init(shflbw_spconv_state* state, const shflbw_weight* f, int B, int H, int W, int stride,
                       const void* IFMap, void* OFMap)
{
    return shflbw_spconv_init_variant(state, f, B, H, W, stride, IFMap, OFMap, -1);
}

} // extern "C"

namespace {

// forms of the convolution (shflbw_spconv_variant_name)
enum ConvForm { FORM_PLANES = 0, FORM_DIRECT = 1, FORM_BPLANES = 2, FORM_FUSED = 3, FORM_CHWB = 4, FORM_COUNT = 5 };

// Argument checks of a convolution and every field of the state that does not depend on device scratch.
int spconv_fill_state(shflbw_spconv_state* state, const shflbw_weight* f, int B, int H, int W, int stride,
                      const void* IFMap, void* OFMap, int variant)
{
    if (!state) return SHFLBW_ERR_INVALID;
    memset(state, 0, sizeof(*state));
    if (!f || !IFMap || !OFMap) {
        set_error("spconv_init: null filter, IFMap or OFMap");
        return SHFLBW_ERR_INVALID;
    }
    if (!f->device_synced) { // assert at spconv/blockwise_op.h:83
        set_error("spconv_init: sparse filter is not synced to device");
        return SHFLBW_ERR_STATE;
    }
    if (f->R <= 0) {
        set_error("spconv_init: weight has no filter view (use shflbw_filter_init_random or pass R,S,C to shflbw_weight_set)");
        return SHFLBW_ERR_STATE;
    }
    if (f->bcol != 1) {
        set_error("spconv_init: bcol must be 1 (got %d)", f->bcol);
        return SHFLBW_ERR_UNSUPPORTED;
    }
    if (B <= 0 || H <= 0 || W <= 0 || stride <= 0) {
        set_error("spconv_init: non-positive B, H, W or stride");
        return SHFLBW_ERR_INVALID;
    }
    if (variant != FORM_CHWB && ((f->C % 8) != 0 || (f->F % 8) != 0)) { // NHWC forms move 8 channels / 8 filters at a time
        set_error("spconv_init: C and F must be multiples of 8 (got %d, %d)", f->C, f->F);
        return SHFLBW_ERR_SHAPE;
    }
    if (((uintptr_t)IFMap | (uintptr_t)OFMap) & 15) {
        set_error("spconv_init: IFMap and OFMap must be 16-byte aligned");
        return SHFLBW_ERR_INVALID;
    }
    const int Ho = (H + 2 * (f->R / 2) - f->R) / stride + 1;
    const int Wo = (W + 2 * (f->S / 2) - f->S) / stride + 1;
    if (Ho <= 0 || Wo <= 0) {
        set_error("spconv_init: empty output (%d x %d)", Ho, Wo);
        return SHFLBW_ERR_SHAPE;
    }
    if (variant < 0 || variant >= FORM_COUNT) {
        set_error("spconv_init: variant %d does not exist (0 = plane form, 1 = direct kernel, 2 = batch-innermost plane "
                  "form, 3 = batch-innermost plane form fused into one launch)", variant);
        return SHFLBW_ERR_INVALID;
    }
    if (variant == FORM_DIRECT) {
        const SpconvVariant* v = find_spconv_variant(f->brow, 0, nullptr);
        if (!v) {
            set_error("spconv_init: the direct kernel (variant 1) exists for block sizes 16, 32, 64 and 128, not %d; "
                      "the plane forms (0, 2, 3) serve every block size", f->brow);
            return SHFLBW_ERR_UNSUPPORTED;
        }
        if ((unsigned long long)B * H * W * f->C > 0x7fffffffull) {
            set_error("spconv_init: input of %d x %d x %d x %d values exceeds the 2^31 the direct kernel can index", B, H, W, f->C);
            return SHFLBW_ERR_UNSUPPORTED;
        }
        SHFLBW_HIP_TRY(v->prepare());
    }
    shflbw_device_ref ref;
    shflbw_weight_device_ref(f, &ref);
    state->args.B = B;
    state->args.H = H;
    state->args.W = W;
    state->args.C = f->C;
    state->args.F = f->F;
    state->args.R = f->R;
    state->args.S = f->S;
    state->args.stride = stride;
    state->args.A_values = ref.csb_values;
    state->args.IFMap = IFMap;
    state->args.OFMap = OFMap;
    state->args.A_bsr_indptr = ref.csb_indptr;
    state->args.A_bsr_indices = ref.csb_indices;
    state->args.A_row_indices = ref.row_permute_ids;
    state->args.alpha = 1.f; // spconv/blockwise_op.h:89-94
    state->args.beta = 0.f;
    state->Ho = Ho;
    state->Wo = Wo;
    state->packed_values = f->d_packed_values;
    state->packed_indices = (const int*)f->d_packed_indices;
    state->panel_ptr = (const int*)f->d_group_ptr;
    state->brow = f->brow;
    state->variant = variant;
    return SHFLBW_OK;
}

size_t up256(size_t n) { return (n + 255) / 256 * 256; }

// The gather ids of one (form, geometry) on the device: `ids_bytes` of slot-ordered ids, then the same ids in the
// producer-major order of every 64-slot group.  `offset_of(k)` maps a kept column k = (r*S + t)*C + c to its element
// offset in the layout-transformed input; padding slots (k < 0) get `zero_id`, the offset of a row of zeros.  Built
// and uploaded on the first call for a key, found afterwards.  The caller holds the weight's scratch_lock.
template <class OffsetOf>
int conv_ids_for(shflbw_weight* fw, const int (&key)[5], int zero_id, OffsetOf offset_of, const int** ids, const int** ids_pm)
{
    const size_t slots = fw->packed_indices.size();
    const size_t ids_bytes = up256(slots * sizeof(int) + 64);
    for (auto& e : fw->conv_ids)
        if (memcmp(e.key, key, sizeof(key)) == 0 && e.bytes == 2 * ids_bytes) {
            *ids = (const int*)e.ptr;
            *ids_pm = (const int*)((const char*)e.ptr + ids_bytes);
            return SHFLBW_OK;
        }
    std::vector<int> h(2 * ids_bytes / sizeof(int), 0);
    int* pm = h.data() + ids_bytes / sizeof(int);
    for (size_t q = 0; q < slots; q++) {
        const int k = fw->packed_indices[q];
        const int id = k < 0 ? zero_id : offset_of(k);
        h[q] = id;
        const size_t grp = q / 64; // producer-major order inside every 64-slot group
        const int j = (int)(q % 64) / 16, p = (int)(q % 16) / 4, r = (int)(q % 4);
        pm[grp * 64 + 16 * p + 4 * j + r] = id;
    }
    void* d = nullptr;
    SHFLBW_HIP_TRY(hipMalloc(&d, 2 * ids_bytes));
    if (hipMemcpy(d, h.data(), 2 * ids_bytes, hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipFree(d);
        set_error("spconv_init: cannot upload the gather ids");
        return SHFLBW_ERR_HIP;
    }
    fw->conv_ids.push_back(shflbw_weight::ConvIds{{key[0], key[1], key[2], key[3], key[4]}, d, 2 * ids_bytes});
    *ids = (const int*)d;
    *ids_pm = (const int*)((const char*)d + ids_bytes);
    return SHFLBW_OK;
}

// The bulk scratch (layout-transformed input, filter-major result, counters) of a state: the buffer of an equal
// (form, geometry, tensors) if there is one; else a new one, cleared, while fewer than CONV_BULK_DEPTH exist; else the
// least recently handed out one - as it is when it served the same geometry (what has to be zero in it still is: the
// parts of the planes no launch writes, the counters every launch leaves at zero), freed and allocated anew
// otherwise.  The caller holds the weight's scratch_lock.
int conv_bulk_for(shflbw_weight* fw, const int (&key)[5], const void* in, const void* out, size_t bytes, char** ptr)
{
    auto& pool = fw->conv_bulk;
    fw->bulk_clock++;
    for (auto& e : pool)
        if (e.bytes == bytes && memcmp(e.key, key, sizeof(key)) == 0 && e.in == in && e.out == out) {
            e.stamp = fw->bulk_clock;
            *ptr = (char*)e.ptr;
            return SHFLBW_OK;
        }
    if ((int)pool.size() >= shflbw_weight::CONV_BULK_DEPTH) {
        size_t lru = 0;
        for (size_t i = 1; i < pool.size(); i++)
            if (pool[i].stamp < pool[lru].stamp) lru = i;
        if (pool[lru].bytes == bytes && memcmp(pool[lru].key, key, sizeof(key)) == 0) {
            pool[lru].in = in, pool[lru].out = out, pool[lru].stamp = fw->bulk_clock;
            *ptr = (char*)pool[lru].ptr;
            return SHFLBW_OK;
        }
        (void)hipFree(pool[lru].ptr);
        pool.erase(pool.begin() + lru);
    }
    void* d = nullptr;
    if (hipMalloc(&d, bytes) != hipSuccess) {
        set_error("spconv_init: cannot allocate %zu bytes of device scratch", bytes);
        return SHFLBW_ERR_HIP;
    }
    // cleared before any stream can launch on it (the caller's stream need not be ordered behind the one the clear runs on)
    if (hipMemset(d, 0, bytes) != hipSuccess || hipStreamSynchronize(nullptr) != hipSuccess) {
        (void)hipFree(d);
        set_error("spconv_init: cannot clear %zu bytes of device scratch", bytes);
        return SHFLBW_ERR_HIP;
    }
    pool.push_back(shflbw_weight::ConvBulk{{key[0], key[1], key[2], key[3], key[4]}, in, out, d, bytes, fw->bulk_clock});
    *ptr = (char*)d;
    return SHFLBW_OK;
}

// Sets up the SpMM launch in the middle of a plane form: N columns, the planes as B, `result` as D, the rewritten ids
// (element offsets: one id apart is one value apart) and `id_space` as the extent the ids address.
int bind_middle(shflbw_spconv_state* state, const shflbw_weight* f, long N, const void* planes, void* result,
                const int* ids, const int* ids_pm, long id_space)
{
    // only the variants that gather rows by id can walk the planes; the first one of the block size (role-split)
    int rc = spmm_init_impl(&state->spmm, f, (int)N, planes, nullptr, result, 1.f, 0.f, -1, true);
    if (rc != SHFLBW_OK) return rc;
    state->spmm.packed_indices = ids;
    state->spmm.packed_indices_pm = ids_pm;
    state->spmm.ldb_bytes = 2;
    state->spmm.args.K = (int)id_space;
    return SHFLBW_OK;
}

void copy_middle_launch_figures(shflbw_spconv_state* state)
{
    state->shared_mem_size = state->spmm.shared_mem_size;
    state->grid_dim[0] = state->spmm.grid_dim[0];
    state->block_dim[0] = state->spmm.block_dim[0];
    state->grid_dim[1] = state->grid_dim[2] = 1;
    state->block_dim[1] = state->block_dim[2] = 1;
}

// Form 0.  Points a state at its scratch (laid out by `g`) and sets up the SpMM launch in the middle.
int bind_plane_form(shflbw_spconv_state* state, const shflbw_weight* f, const PlaneForm& g, char* planes, char* result,
                    const int* ids, const int* ids_pm)
{
    state->planes = planes;
    state->result_fm = result;
    state->np = (int)g.np;
    state->plane_rows = g.PH;
    state->plane_cols = g.PW;
    state->plane_pitch = (int)g.pitch;
    state->plane_copies = g.copies;
    state->ncols = (int)g.np;
    int rc = bind_middle(state, f, g.np, planes, result, ids, ids_pm, (g.rows + 1) * g.pitch);
    if (rc != SHFLBW_OK) return rc;
    copy_middle_launch_figures(state);
    state->init_success = 1;
    return SHFLBW_OK;
}

int init_planes(shflbw_spconv_state* state, const shflbw_weight* f, int B, int H, int W, int stride, const void* IFMap,
                void* OFMap)
{
    int rc = spconv_fill_state(state, f, B, H, W, stride, IFMap, OFMap, FORM_PLANES);
    if (rc != SHFLBW_OK) return rc;
    PlaneForm g;
    if ((rc = plane_form_geometry(f, B, H, W, stride, &g)) != SHFLBW_OK) return rc;
    // The scratch cache is bookkeeping of the handle, not part of the weight's value; it is the one member an
    // init call changes, under its lock.
    shflbw_weight* fw = const_cast<shflbw_weight*>(f);
    std::lock_guard<std::mutex> scratch_guard(fw->scratch_lock);
    const int key[5] = {FORM_PLANES, B, H, W, stride};
    const int s = stride, copies = g.copies, C = f->C, S = f->S;
    const long PW = g.PW, pitch = g.pitch;
    const int *ids = nullptr, *ids_pm = nullptr;
    // kept-column id k = (r*S + t)*C + c  ->  element offset of (copy, phase, channel) row + tap offset
    rc = conv_ids_for(fw, key, (int)(g.rows * pitch), [&](int k) {
        const int c = k % C, tap = k / C, r = tap / S, t = tap % S;
        const long shift = (long)(r / s) * PW + t / s;
        const int copy = copies == 2 ? (int)(shift & 1) : 0;
        const int phase = (r % s) * s + t % s;
        return (int)((((long)copy * s * s + phase) * C + c) * pitch + shift - copy);
    }, &ids, &ids_pm);
    if (rc != SHFLBW_OK) return rc;
    char* bulk = nullptr;
    if ((rc = conv_bulk_for(fw, key, IFMap, OFMap, g.planes_bytes + g.dm_bytes, &bulk)) != SHFLBW_OK) return rc;
    return bind_plane_form(state, f, g, bulk, bulk + g.planes_bytes, ids, ids_pm);
}

// XCDs of the current device when it deals the workgroups of a launch to them the way the fused form counts on:
// consecutive workgroup ids go to consecutive XCDs, round-robin from whichever XCD the launch starts on, so a launch of
// a multiple of n workgroups puts the same number on every XCD; and every XCD has the same number of compute units.
// Checked once per device with probe launches of two sizes; 0 when the device deals differently (the fused form is
// then not offered; `why` says what was seen).
int device_xcds(std::string* why)
{
    static std::mutex lock;
    static int cached[64] = {}; // 0 = unknown, -1 = not usable
    static std::string seen[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    std::lock_guard<std::mutex> guard(lock);
    if (cached[dev] == 0) {
        cached[dev] = -1;
        const int sizes[2] = {1024, 256};
        int* d = nullptr;
        int n_all = 0;
        bool ok = hipMalloc((void**)&d, 1024 * sizeof(int)) == hipSuccess;
        if (!ok) seen[dev] = "probe allocation failed";
        for (int round = 0; ok && round < 2; round++) {
            const int blocks = sizes[round];
            std::vector<int> h(blocks, -1);
            ok = hipMemset(d, 0xff, blocks * sizeof(int)) == hipSuccess && launch_xcd_probe(d, blocks, nullptr) == hipSuccess &&
                 hipMemcpy(h.data(), d, blocks * sizeof(int), hipMemcpyDeviceToHost) == hipSuccess;
            if (!ok) {
                seen[dev] = "probe launch failed";
                break;
            }
            int n = 0;
            for (int v : h) n = std::max(n, v + 1);
            ok = n >= 1 && n <= 8 && (round == 0 || n == n_all) && device_compute_units() % n == 0 && h[0] >= 0;
            for (int i = 0; ok && i < blocks; i++) ok = h[i] == (h[0] + i) % n;
            n_all = n;
            if (!ok) {
                char buf[256];
                int len = snprintf(buf, sizeof(buf), "launch of %d workgroups, %d XCD ids, workgroups 0.. ran on XCDs", blocks, n);
                for (int i = 0; i < 24 && len < (int)sizeof(buf) - 8; i++) len += snprintf(buf + len, sizeof(buf) - len, " %d", h[i]);
                seen[dev] = buf;
            }
        }
        if (d) (void)hipFree(d);
        if (ok) cached[dev] = n_all;
    }
    if (why) *why = seen[dev];
    return cached[dev] > 0 ? cached[dev] : 0;
}

// Geometry of the batch-innermost plane forms (2, 3, 4): phase planes planes[phase (a, b)][c][(i * PW + j) * B + img] =
// in(i * stride + a - R/2, j * stride + b - S/2) of image img and channel c, PHX = Ho + (R-1)/stride rows and
// PW = Wo + (S-1)/stride columns.  Every tap offset is a multiple of B values, 16 bytes or more: one copy of the planes
// serves all taps.  The GEMM runs over the Ho * PW * B columns (ho, j, img) of the padded output grid.
struct BatchPlanes {
    int Ho, Wo;
    long PHX, PW;
    long np;        // values of one channel plane
    long rows;      // channel rows: stride^2 * C
    long ncols;     // columns of the GEMM
    long max_shift; // largest tap offset in values
};

void batch_planes_geometry(const shflbw_weight* f, int B, int stride, int Ho, int Wo, BatchPlanes* g)
{
    const int s = stride;
    g->Ho = Ho, g->Wo = Wo;
    g->PHX = Ho + (f->R - 1) / s;
    g->PW = Wo + (f->S - 1) / s;
    g->np = g->PHX * g->PW * B;
    g->rows = (long)s * s * f->C;
    g->ncols = (long)Ho * g->PW * B;
    g->max_shift = ((long)((f->R - 1) / s) * g->PW + (f->S - 1) / s) * B;
}

//   form 4: the caller's tensors are C-H-W-B / F-H-W-B (the reference's), H and W bound input and output alike,
//           the SpMM writes OFMap itself (its epilogue drops the padding columns, output_column());
//   form 2: the caller's tensors are NHWC with true stride and padding; the SpMM writes result_fm[f][(ho, wo, img)],
//           a tile transpose writes OFMap.
int init_batch_planes(shflbw_spconv_state* state, const shflbw_weight* f, int B, int H, int W, int stride,
                      const void* IFMap, void* OFMap, int variant)
{
    int rc = spconv_fill_state(state, f, B, H, W, stride, IFMap, OFMap, variant);
    if (rc != SHFLBW_OK) return rc;
    if (B % 8 != 0) { // the reference's kernel moves 8 batch entries at a time too (spconv/blockwise_kernel.h:200-207)
        set_error("spconv_init: the batch must be a multiple of 8 for this form (got %d)", B);
        return SHFLBW_ERR_SHAPE;
    }
    if (variant == FORM_CHWB) { // H and W are the extents of the output grid and the bounds of the input (spconv/blockwise_format.h:111-115)
        state->Ho = H;
        state->Wo = W;
    }
    BatchPlanes g;
    batch_planes_geometry(f, B, stride, state->Ho, state->Wo, &g);
    // the SpMM in the middle: tile width by the size of the GEMM, as for the SpMM proper
    const ConvChwbKernel* k = conv_chwb_kernel(f->brow, 0, f->nrow / f->brow, g.ncols, device_compute_units());
    if (!k) {
        set_error("spconv_init: no kernel for block size %d", f->brow);
        return SHFLBW_ERR_UNSUPPORTED;
    }
    SHFLBW_HIP_TRY(k->prepare());
    state->middle_tile_cols = k->BN;
    const int s = stride, C = f->C, S = f->S;
    const long pitch = (g.np + g.max_shift + 8 + 63) / 64 * 64;
    if (g.ncols > 0x7fffffffL || (unsigned long long)(g.rows + 1) * (unsigned long long)pitch * 2ull > 0xffffffffull) {
        set_error("spconv_init: problem too large (%ld channel rows of %ld values)", g.rows, pitch);
        return SHFLBW_ERR_UNSUPPORTED;
    }
    const size_t planes_bytes = up256((size_t)(g.rows + 1) * pitch * 2); // one more row: zeros, for the padding slots
    const size_t dm_bytes = variant == FORM_BPLANES ? up256((size_t)f->F * g.Ho * g.Wo * B * 2) : 0;
    shflbw_weight* fw = const_cast<shflbw_weight*>(f); // the scratch cache is bookkeeping of the handle (see init_planes)
    std::lock_guard<std::mutex> scratch_guard(fw->scratch_lock);
    const int key[5] = {variant, B, H, W, stride};
    const long PW = g.PW;
    const int *ids = nullptr, *ids_pm = nullptr;
    // kept-column id k = (r*S + t)*C + c  ->  element offset of the (phase, channel) row + tap offset
    rc = conv_ids_for(fw, key, (int)(g.rows * pitch), [&](int kk) {
        const int c = kk % C, tap = kk / C, r = tap / S, t = tap % S;
        return (int)((((long)(r % s) * s + t % s) * C + c) * pitch + ((long)(r / s) * PW + t / s) * B);
    }, &ids, &ids_pm);
    if (rc != SHFLBW_OK) return rc;
    char* bulk = nullptr;
    if ((rc = conv_bulk_for(fw, key, IFMap, OFMap, planes_bytes + dm_bytes, &bulk)) != SHFLBW_OK) return rc;
    state->planes = bulk;
    state->result_fm = variant == FORM_BPLANES ? bulk + planes_bytes : nullptr;
    state->np = (int)g.np;
    state->plane_rows = (int)g.PHX;
    state->plane_cols = (int)g.PW;
    state->plane_pitch = (int)pitch;
    state->plane_copies = 1;
    state->ncols = (int)g.ncols;
    // the SpMM in the middle: row f of its result is the row of filter f, in OFMap itself (form 4) or in result_fm
    rc = bind_middle(state, f, g.ncols, state->planes, variant == FORM_BPLANES ? state->result_fm : OFMap, ids, ids_pm,
                     (g.rows + 1) * pitch);
    if (rc != SHFLBW_OK) return rc;
    state->shared_mem_size = (size_t)k->lds_bytes;
    state->grid_dim[0] = (unsigned)((f->nrow / f->brow) * ((g.ncols + k->BN - 1) / k->BN));
    state->block_dim[0] = (unsigned)k->threads;
    state->grid_dim[1] = state->grid_dim[2] = 1;
    state->block_dim[1] = state->block_dim[2] = 1;
    state->init_success = 1;
    return SHFLBW_OK;
}

// Layout of the fused form's bulk scratch: nx slabs of planes | nx filter-major results | counters.
struct FusedForm {
    BatchPlanes g;
    int nx;          // XCDs of the device
    long cx;         // columns of the GEMM per XCD (a multiple of 64)
    long pitch;      // values per channel row of a slab: cx + the largest tap offset, rounded up to 64
    size_t slab_bytes, fm_bytes, sync_bytes;
    size_t total_bytes() const { return (size_t)nx * (slab_bytes + fm_bytes) + sync_bytes; }
};

int fused_form_geometry(const shflbw_weight* f, int B, int stride, int Ho, int Wo, int nx, FusedForm* g)
{
    batch_planes_geometry(f, B, stride, Ho, Wo, &g->g);
    g->nx = nx;
    g->cx = ((g->g.ncols + nx - 1) / nx + 63) / 64 * 64;
    g->pitch = (g->cx + g->g.max_shift + 63) / 64 * 64;
    if (stride * stride > 32 || g->g.ncols > 0x7fffffffL ||
        (unsigned long long)(g->g.rows + 1) * (unsigned long long)g->pitch * 2ull > 0x7fffffffull ||
        (unsigned long long)f->F * (unsigned long long)g->cx > 0x7fffffffull) {
        set_error("spconv_init: problem too large for the fused form (%ld channel rows of %ld values per XCD)", g->g.rows, g->pitch);
        return SHFLBW_ERR_UNSUPPORTED;
    }
    g->slab_bytes = up256((size_t)(g->g.rows + 1) * g->pitch * 2); // one more row: zeros, for the padding slots
    g->fm_bytes = up256((size_t)f->F * g->cx * 2);
    g->sync_bytes = (size_t)conv_xcd_sync_lines(nx) * SYNC_LINE * sizeof(int);
    return SHFLBW_OK;
}

// form 3: NHWC tensors, the three steps of form 2 in one launch, every XCD on its own columns (spconv_xcd_kernel)
int init_fused(shflbw_spconv_state* state, const shflbw_weight* f, int B, int H, int W, int stride, const void* IFMap,
               void* OFMap)
{
    int rc = spconv_fill_state(state, f, B, H, W, stride, IFMap, OFMap, FORM_FUSED);
    if (rc != SHFLBW_OK) return rc;
    if (B % 8 != 0) {
        set_error("spconv_init: the batch must be a multiple of 8 for this form (got %d)", B);
        return SHFLBW_ERR_SHAPE;
    }
    const ConvXcdKernel* k = conv_xcd_kernel(f->brow);
    if (!k) {
        set_error("spconv_init: no fused kernel for block size %d", f->brow);
        return SHFLBW_ERR_UNSUPPORTED;
    }
    std::string why;
    const int nx = device_xcds(&why);
    if (nx <= 0) {
        set_error("spconv_init: this device does not deal workgroups to its XCDs in the way the fused form counts on (%s)", why.c_str());
        return SHFLBW_ERR_UNSUPPORTED;
    }
    if (device_compute_units() / nx > 32) {
        set_error("spconv_init: the fused form numbers at most 32 workgroups per XCD (this device: %d)", device_compute_units() / nx);
        return SHFLBW_ERR_UNSUPPORTED;
    }
    SHFLBW_HIP_TRY(k->prepare());
    FusedForm g;
    if ((rc = fused_form_geometry(f, B, stride, state->Ho, state->Wo, nx, &g)) != SHFLBW_OK) return rc;
    const int s = stride, C = f->C, S = f->S;
    const long PW = g.g.PW, pitch = g.pitch;
    shflbw_weight* fw = const_cast<shflbw_weight*>(f); // the scratch cache is bookkeeping of the handle (see init_planes)
    std::lock_guard<std::mutex> scratch_guard(fw->scratch_lock);
    const int key[5] = {FORM_FUSED, B, H, W, stride};
    const int *ids = nullptr, *ids_pm = nullptr;
    // kept-column id k = (r*S + t)*C + c  ->  element offset inside a slab: (phase, channel) row + tap offset
    rc = conv_ids_for(fw, key, (int)(g.g.rows * pitch), [&](int kk) {
        const int c = kk % C, tap = kk / C, r = tap / S, t = tap % S;
        return (int)((((long)(r % s) * s + t % s) * C + c) * pitch + ((long)(r / s) * PW + t / s) * B);
    }, &ids, &ids_pm);
    if (rc != SHFLBW_OK) return rc;
    char* bulk = nullptr;
    if ((rc = conv_bulk_for(fw, key, IFMap, OFMap, g.total_bytes(), &bulk)) != SHFLBW_OK) return rc;
    state->planes = bulk;
    state->result_fm = bulk + (size_t)nx * g.slab_bytes;
    state->sync = bulk + (size_t)nx * (g.slab_bytes + g.fm_bytes);
    state->np = (int)g.g.np;
    state->plane_rows = (int)g.g.PHX;
    state->plane_cols = (int)g.g.PW;
    state->plane_pitch = (int)pitch;
    state->plane_copies = 1;
    state->ncols = (int)g.g.ncols;
    state->xcds = nx;
    state->cols_per_xcd = (int)g.cx;
    state->patience_ticks = 5000; // 50 us
    // the SpMM in the middle, as one XCD sees it: cx columns, its slab as B, its result as D
    rc = bind_middle(state, f, g.cx, state->planes, state->result_fm, ids, ids_pm, (g.g.rows + 1) * pitch);
    if (rc != SHFLBW_OK) return rc;
    state->shared_mem_size = (size_t)k->lds_bytes;
    state->grid_dim[0] = (unsigned)(device_compute_units() / nx * nx);
    state->block_dim[0] = (unsigned)k->threads;
    state->grid_dim[1] = state->grid_dim[2] = 1;
    state->block_dim[1] = state->block_dim[2] = 1;
    state->init_success = 1;
    return SHFLBW_OK;
}

// launch arguments every form shares
void fill_conv_launch_args(const shflbw_spconv_state* state, SpconvLaunchArgs* out)
{
    SpconvLaunchArgs& a = *out;
    a.B = state->args.B;
    a.H = state->args.H;
    a.W = state->args.W;
    a.C = state->args.C;
    a.F = state->args.F;
    a.R = state->args.R;
    a.S = state->args.S;
    a.stride = state->args.stride;
    a.pad_h = a.R / 2;
    a.pad_w = a.S / 2;
    a.Ho = state->Ho;
    a.Wo = state->Wo;
    a.X = a.F / state->brow;
    a.n_tiles = 0;
    a.packedA = (const half8_t*)state->packed_values;
    a.kidx = state->packed_indices;
    a.panel_desc = state->panel_ptr;
    a.row_ids = state->args.A_row_indices;
    a.in = (const half_t*)state->args.IFMap;
    a.out = (half_t*)state->args.OFMap;
}

// Chunks of the layout phases of the fused form: `tiles` = 8, 4 or 2 tiles of 64 x 64 per chunk, as many of them
// along the contiguous axis of the source (`along` tiles there) as there are.  Picks the chunk size that needs the
// fewest rounds of the `workers` workgroups of an XCD, a round costing its tiles plus a fixed latency of about
// four tiles' worth.
void pick_chunk(int along_tiles, int across_tiles, int workers, int* t_along, int* t_across, int* chunks_along)
{
    auto pow2_le = [](int n, int cap) { int p = 1; while (p * 2 <= n && p * 2 <= cap) p *= 2; return p; };
    long best_cost = -1;
    for (int tiles = 8; tiles >= 2; tiles >>= 1) {
        const int ta = pow2_le(along_tiles, tiles), tb = tiles / ta;
        const long chunks = (long)((along_tiles + ta - 1) / ta) * ((across_tiles + tb - 1) / tb);
        const long rounds = (chunks + workers - 1) / workers;
        const long cost = rounds * (tiles + 4);
        if (best_cost < 0 || cost < best_cost) {
            best_cost = cost;
            *t_along = ta, *t_across = tb, *chunks_along = (along_tiles + ta - 1) / ta;
        }
    }
}

} // namespace

extern "C" {

int shflbw_spconv_init_variant(shflbw_spconv_state* state, const shflbw_weight* f, int B, int H, int W, int stride,
                               const void* IFMap, void* OFMap, int variant)
{
    if (variant == FORM_CHWB) {
        if (state) memset(state, 0, sizeof(*state));
        set_error("spconv_init: form 4 works on C-H-W-B / F-H-W-B tensors; call shflbw_spconv_init_chwb");
        return SHFLBW_ERR_INVALID;
    }
    // the library's choice: the batch-innermost form wherever the batch allows it (one copy of the planes instead of
    // two, no dead plane rows in the result; with the tile width of its SpMM chosen by the size of the GEMM it is level
    // with the plane form on the smallest layers and ahead from a few hundred output pixels on), else the plane form
    if (variant < 0) {
        variant = FORM_PLANES;
        if (f && f->R > 0 && B > 0 && B % 8 == 0 && H > 0 && W > 0 && stride > 0) {
            const long Ho = (H + 2 * (f->R / 2) - f->R) / stride + 1, Wo = (W + 2 * (f->S / 2) - f->S) / stride + 1;
            if (Ho > 0 && Wo > 0) variant = FORM_BPLANES;
        }
    }
    if (variant == FORM_BPLANES) return init_batch_planes(state, f, B, H, W, stride, IFMap, OFMap, FORM_BPLANES);
    if (variant == FORM_FUSED) return init_fused(state, f, B, H, W, stride, IFMap, OFMap);
    if (variant == FORM_PLANES) return init_planes(state, f, B, H, W, stride, IFMap, OFMap);
    int rc = spconv_fill_state(state, f, B, H, W, stride, IFMap, OFMap, variant);
    if (rc != SHFLBW_OK) return rc;
    // the direct kernel
    const SpconvVariant* v = find_spconv_variant(f->brow, 0, nullptr);
    const long npix = (long)B * state->Ho * state->Wo;
    state->shared_mem_size = (size_t)v->lds_bytes;
    state->grid_dim[0] = (unsigned)((f->F / f->brow) * ((npix + v->BN - 1) / v->BN));
    state->block_dim[0] = (unsigned)v->threads;
    state->grid_dim[1] = state->grid_dim[2] = 1;
    state->block_dim[1] = state->block_dim[2] = 1;
    state->init_success = 1;
    return SHFLBW_OK;
}

int shflbw_spconv_init_chwb(shflbw_spconv_state* state, const shflbw_weight* f, int B, int H, int W, int stride,
                            const void* IFMap, void* OFMap)
{
    return init_batch_planes(state, f, B, H, W, stride, IFMap, OFMap, FORM_CHWB);
}

int shflbw_spconv_exec(const shflbw_spconv_state* state, void* stream)
{
    if (!state || !state->init_success) {
        set_error("spconv_exec: state was not initialised successfully");
        return SHFLBW_ERR_STATE;
    }
    SpconvLaunchArgs a;
    fill_conv_launch_args(state, &a);
    hipError_t e = hipSuccess;
    if (state->variant == FORM_CHWB || state->variant == FORM_BPLANES) {
        const ConvChwbKernel* k = conv_chwb_kernel(state->brow, state->middle_tile_cols, 0, 0, 0);
        if (!k) return SHFLBW_ERR_UNSUPPORTED;
        const bool nhwc = state->variant == FORM_BPLANES;
        e = nhwc ? launch_nhwc_to_planes(a, (half_t*)state->planes, state->plane_rows, state->plane_cols,
                                         state->plane_pitch, 1, (hipStream_t)stream, 1)
                 : launch_chwb_to_planes(a.in, (half_t*)state->planes, a.B, a.H, a.W, a.C, a.R, a.S, a.stride,
                                         state->plane_rows, state->plane_cols, state->plane_pitch, (hipStream_t)stream);
        SpmmLaunchArgs m;
        fill_spmm_launch_args(&state->spmm, k->BN, &m);
        m.alternate = 0;
        m.ldd = a.Ho * a.Wo * a.B;                  // a row of the result: one filter, Ho x Wo x B values
        m.dmap_row = state->plane_cols * a.B;       // columns of the GEMM per row of the padded output grid
        m.dmap_valid = a.Wo * a.B;                  // ... of which the first Wo x B are output values
        m.dmap_magic = udiv_magic(m.dmap_row);
        if (e == hipSuccess && m.X > 0) e = k->launch(m, (hipStream_t)stream);
        if (e == hipSuccess && nhwc) // result_fm[f][(ho, wo, img)] -> OFMap[img][ho][wo][f]
            e = launch_planes_to_nhwc((const half_t*)state->result_fm, a.out, a.F, a.Ho * a.Wo * a.B, a.B, a.Ho, a.Wo,
                                      a.Ho, a.Wo, (hipStream_t)stream, 1);
    } else if (state->variant == FORM_FUSED) {
        const ConvXcdKernel* k = conv_xcd_kernel(state->brow);
        if (!k || state->xcds <= 0 || state->cols_per_xcd <= 0) return SHFLBW_ERR_UNSUPPORTED;
        SpmmLaunchArgs m;
        fill_spmm_launch_args(&state->spmm, k->BN, &m);
        if (m.X == 0) return SHFLBW_OK;
        m.alternate = 0; // a slab is far smaller than an L2
        m.ldd = state->cols_per_xcd;
        const int s = a.stride, nx = state->xcds, cx = state->cols_per_xcd;
        ConvXcdArgs c;
        c.g = PlaneGeom{a.B, a.H, a.W, a.C, s, a.pad_h, a.pad_w, state->plane_rows, state->plane_cols, state->plane_pitch, 1, 0, {}, 1};
        if (!fill_wanted_planes(c.g, a.R, a.S)) return SHFLBW_ERR_UNSUPPORTED;
        c.in = a.in;
        c.out = a.out;
        c.nx = nx, c.cx = cx, c.ncols = state->ncols;
        c.max_shift = (((a.R - 1) / s) * state->plane_cols + (a.S - 1) / s) * a.B;
        c.slabs = (half_t*)state->planes;
        c.slab_elems = up256((size_t)(s * s * a.C + 1) * state->plane_pitch * 2) / 2;
        c.fm = (half_t*)state->result_fm;
        c.fm_elems = up256((size_t)a.F * cx * 2) / 2;
        c.sync = (int*)state->sync;
        c.F = a.F, c.Ho = a.Ho, c.Wo = a.Wo;
        const int workers = std::max(1, m.num_cus / nx);
        const int n_x = std::min(cx, state->ncols); // the columns of a full XCD
        pick_chunk((a.C + 63) / 64, (n_x + c.max_shift + 63) / 64 * c.g.nwanted, workers, &c.ct, &c.pt, &c.ch_chunks);
        pick_chunk((a.F + 63) / 64, (n_x + 63) / 64, workers, &c.ft, &c.mt, &c.f_chunks);
        c.magic_b = udiv_magic(a.B);
        c.magic_pw = udiv_magic(state->plane_cols);
        c.spin_ticks = 20000000; // 0.2 s
        c.patience = state->patience_ticks > 0 ? state->patience_ticks : state->patience_ticks < 0 ? 1 : 5000;
        c.late_ticks = state->patience_ticks < 0 ? std::min(-state->patience_ticks, 10000) : 0;
        c.debug = 0;
#ifdef SHFLBW_CONV_STAMPS
        if (const char* dbg = getenv("SHFLBW_CONV_DEBUG")) c.debug = atoi(dbg);
#endif
        e = k->launch(m, c, (hipStream_t)stream);
    } else if (state->variant == FORM_PLANES) {
        e = launch_nhwc_to_planes(a, (half_t*)state->planes, state->plane_rows, state->plane_cols, state->plane_pitch,
                                  state->plane_copies, (hipStream_t)stream);
        if (e == hipSuccess) {
            int rc = shflbw_spmm_exec(&state->spmm, stream);
            if (rc != SHFLBW_OK) return rc;
            e = launch_planes_to_nhwc((const half_t*)state->result_fm, a.out, a.F, state->np, a.B, state->plane_rows,
                                      state->plane_cols, a.Ho, a.Wo, (hipStream_t)stream);
        }
    } else {
        const SpconvVariant* v = find_spconv_variant(state->brow, 0, nullptr); // the direct kernel of this block size
        if (!v) return SHFLBW_ERR_UNSUPPORTED;
        e = v->launch(a, (hipStream_t)stream);
    }
    if (e != hipSuccess) {
        set_error("spconv_exec: launch failed: %s", hipGetErrorString(e));
        return SHFLBW_ERR_HIP;
    }
    return SHFLBW_OK;
}

int shflbw_spconv_check(const shflbw_spconv_state* state)
{
    if (!state || !state->init_success) {
        set_error("spconv_check: state was not initialised successfully");
        return SHFLBW_ERR_STATE;
    }
    if (state->variant != FORM_FUSED) return SHFLBW_OK;
    int flag = 0;
    SHFLBW_HIP_TRY(hipMemcpy(&flag, state->sync, sizeof(int), hipMemcpyDeviceToHost)); // waits for the device
    if (flag != 0) {
        // leave the scratch as a fresh one: no counter may keep what the failed launch left in it
        SHFLBW_HIP_TRY(hipMemset(state->sync, 0, (size_t)conv_xcd_sync_lines(state->xcds) * SYNC_LINE * sizeof(int)));
        set_error(flag == 1 ? "spconv_check: the workgroups of a fused launch were not dealt to the XCDs the way init had checked; results are invalid"
                            : "spconv_check: a wait between the phases of the fused form ran out of time; results are invalid");
        return SHFLBW_ERR_HIP;
    }
    return SHFLBW_OK;
}

// ---------------------------------------------------------------------------------------------------
// The entry point that allocates nothing: the scratch of the plane form in a fixed device array.
// `scratch` below is only the host-side handle of the symbol; the device address of each GPU's copy
// comes from hipGetSymbolAddress, once per device, and only that address is handed to kernels.
// ---------------------------------------------------------------------------------------------------
} // extern "C"

static __device__ __align__(256) unsigned char scratch[SHFLBW_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_static_lock;
void* g_static_addr[kMaxDevices] = {};

// device address of this GPU's copy of `scratch` (looked up on the first call with that device current)
int static_scratch_address(char** out)
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        set_error("spconv_exec_static: cannot tell the current device");
        return SHFLBW_ERR_HIP;
    }
    std::lock_guard<std::mutex> guard(g_static_lock);
    if (!g_static_addr[dev]) {
        void* ptr = nullptr;
        hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            set_error("spconv_exec_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
            return SHFLBW_ERR_HIP;
        }
        g_static_addr[dev] = ptr;
    }
    *out = (char*)g_static_addr[dev];
    return SHFLBW_OK;
}
} // namespace

extern "C" {

int shflbw_spconv_exec_static(const shflbw_weight* f, int B, int H, int W, int stride, const void* IFMap, void* OFMap,
                              void* stream)
{
    shflbw_spconv_state st;
    int rc = spconv_fill_state(&st, f, B, H, W, stride, IFMap, OFMap, FORM_PLANES);
    if (rc != SHFLBW_OK) return rc;
    PlaneForm g;
    if ((rc = plane_form_geometry(f, B, H, W, stride, &g)) != SHFLBW_OK) return rc;
    if (g.total_bytes() > (size_t)SHFLBW_STATIC_SCRATCH_BYTES) {
        set_error("spconv_exec_static: this problem needs %zu bytes of scratch, the fixed array holds %zu", g.total_bytes(),
                  (size_t)SHFLBW_STATIC_SCRATCH_BYTES);
        return SHFLBW_ERR_CAPACITY;
    }
    char* base = nullptr;
    if ((rc = static_scratch_address(&base)) != SHFLBW_OK) return rc;
    // Nothing in the array has to start at zero: the layout pass writes every plane position a pixel's taps
    // read (zeros outside the image), the rest only feeds plane positions that are no output pixel.
    int* ids = (int*)(base + g.planes_bytes + g.dm_bytes);
    int* ids_pm = (int*)(base + g.planes_bytes + g.dm_bytes + g.ids_bytes);
    if ((rc = bind_plane_form(&st, f, g, base, base + g.planes_bytes, ids, ids_pm)) != SHFLBW_OK) return rc;
    hipError_t e = launch_plane_ids((const int*)f->d_packed_indices, ids, ids_pm, (int)g.slots, f->C, f->S, stride, g.PW,
                                    (int)g.pitch, g.copies, (int)(g.rows * g.pitch), (half_t*)base, (hipStream_t)stream);
    if (e != hipSuccess) {
        set_error("spconv_exec_static: id launch failed: %s", hipGetErrorString(e));
        return SHFLBW_ERR_HIP;
    }
    return shflbw_spconv_exec(&st, stream);
}

static const char* const g_spconv_forms[FORM_COUNT] = {
    "planes+spmm+transpose",  // 0: NHWC -> channel-major planes, SpMM gather with tap offsets, transpose to NHWC: three launches
    "direct",                 // 1: one kernel, im2col gather from NHWC in the tile loads
    "bplanes+spmm+transpose", // 2: NHWC tensors, planes and result with the batch innermost (batch a multiple of 8): three launches
    "bplanes-fused",          // 3: the steps of form 2 in one persistent launch, every XCD on its own columns
    "chwb-planes+spmm",       // 4: the reference's batch-innermost tensors (shflbw_spconv_init_chwb only): padded copy, SpMM
};

int shflbw_spconv_variant_count(void) { return FORM_COUNT; }

const char* shflbw_spconv_variant_name(int variant)
{
    return variant >= 0 && variant < FORM_COUNT ? g_spconv_forms[variant] : "";
}

int shflbw_weight_release_scratch(shflbw_weight* w)
{
    if (!w) return SHFLBW_ERR_INVALID;
    std::lock_guard<std::mutex> guard(w->scratch_lock);
    release_conv_scratch(w);
    return SHFLBW_OK;
}

int shflbw_weight_scratch_bytes(const shflbw_weight* w, size_t* bytes, int* buffers)
{
    if (!w) return SHFLBW_ERR_INVALID;
    shflbw_weight* fw = const_cast<shflbw_weight*>(w);
    std::lock_guard<std::mutex> guard(fw->scratch_lock);
    size_t total = 0;
    for (auto& e : w->conv_ids) total += e.bytes;
    for (auto& e : w->conv_bulk) total += e.bytes;
    if (bytes) *bytes = total;
    if (buffers) *buffers = (int)(w->conv_ids.size() + w->conv_bulk.size());
    return SHFLBW_OK;
}

void shflbw_abi_sizes(size_t* spmm_state_bytes, size_t* spconv_state_bytes)
{
    if (spmm_state_bytes) *spmm_state_bytes = sizeof(shflbw_spmm_state);
    if (spconv_state_bytes) *spconv_state_bytes = sizeof(shflbw_spconv_state);
}

int shflbw_device_info(int* compute_units, int* clock_khz, size_t* lds_bytes, char* arch, size_t arch_cap)
{
    int dev = 0;
    SHFLBW_HIP_TRY(hipGetDevice(&dev));
    hipDeviceProp_t p;
    SHFLBW_HIP_TRY(hipGetDeviceProperties(&p, dev));
    if (compute_units) *compute_units = p.multiProcessorCount;
    if (clock_khz) *clock_khz = p.clockRate;
    if (lds_bytes) *lds_bytes = p.sharedMemPerBlock;
    if (arch && arch_cap) {
        strncpy(arch, p.gcnArchName, arch_cap - 1);
        arch[arch_cap - 1] = 0;
    }
    return SHFLBW_OK;
}

} // extern "C"
