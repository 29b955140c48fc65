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

void clear_device(shflbw_weight* w)
{
    void** bufs[] = {&w->d_meta, &w->d_values, &w->d_group_ptr, &w->d_packed_indices, &w->d_packed_indices_pm,
                     &w->d_packed_values, &w->d_packed_slab};
    for (void** b : bufs) {
        if (*b) (void)hipFree(*b);
        *b = nullptr;
    }
    for (auto& sc : w->conv_scratch)
        if (sc.ptr) (void)hipFree(sc.ptr);
    w->conv_scratch.clear();
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

// compute units of the current device, looked up once per process
static int device_compute_units()
{
    static int cached = 0;
    if (cached == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            cached = n;
        else
            cached = 256;
    }
    return cached;
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
// there, 5-20 % slower once the wide tiles fill the chip).
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
static int auto_spmm_variant(const shflbw_weight* w, int N)
{
    const int brow = w->brow, X = w->nrow / w->brow;
    int count = 0;
    const SpmmVariant* all = spmm_variants(&count);
    if (brow == 32 && !w->packed_slab.empty() && w->ncol >= 384 && X > 0) {
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
    const SpmmVariant* first = find_spmm_variant(brow, 0, nullptr);
    if (!first || first->BN != 512) return 0;
    const long wide_tiles = (long)X * ((N + 511) / 512);
    if (wide_tiles > device_compute_units() / 2) return 0;
    int seen = 0;
    for (int i = 0; i < count; i++) {
        if (all[i].V != brow) continue;
        const bool role_split = all[i].name[0] == 'w'; // "ws..." names
        if (role_split && all[i].BN == 256) return seen;
        seen++;
    }
    return 0;
}

// Geometry of the plane form of a convolution and the layout of its device scratch.
struct PlaneForm {
    int PH, PW;     // rows and (padded to 8) columns of one phase plane
    int copies;     // 2 when some tap offset is odd (a second copy moved by one value keeps gathers aligned)
    long np;        // plane positions = columns of the SpMM in the middle
    long pitch;     // values per channel row of the plane tensor
    long rows;      // channel rows: copies * stride^2 * C
    size_t slots;   // padded kept-vector slots of the filter
    long ncols;     // columns of the fused form: plane positions of output rows only, B * Ho * PW
    int Ho, Wo;
    size_t planes_bytes, dm_bytes, ids_bytes, sync_bytes; // scratch = planes | result_fm | ids | ids_pm | sync words
    size_t total_bytes() const { return planes_bytes + dm_bytes + 2 * ids_bytes + sync_bytes; }
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
    g->ncols = (long)B * g->Ho * g->PW;
    g->sync_bytes = (size_t)conv_sync_lines((int)((g->ncols + 255) / 256)) * SYNC_LINE * sizeof(int); // column tiles are 256 wide at least
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
    a.img_cols = 1, a.img_skip = 0;
    a.ldd = a.N;
    a.dmap_row = a.dmap_valid = 0, a.dmap_magic = 0;
    a.tile_arrivals = nullptr;
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

int shflbw_spmm_init_variant(shflbw_spmm_state* state, const shflbw_weight* w, int N, const void* B, const void* C,
                             void* D, float alpha, float beta, int variant)
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
        variant = auto_spmm_variant(w, N);
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

// Argument checks of a convolution and every field of the state that does not depend on device scratch.
static int spconv_fill_state(shflbw_spconv_state* state, const shflbw_weight* f, int B, int H, int W, int stride,
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
    if (variant != 4 && ((f->C % 8) != 0 || (f->F % 8) != 0)) { // NHWC forms move 8 channels / 8 filters at a time
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
    if (variant < 0 || variant >= shflbw_spconv_variant_count()) {
        set_error("spconv_init: variant %d does not exist (0 = plane form, 1 = direct kernel, 2 = im2col form, 3 = plane form fused into one launch)", variant);
        return SHFLBW_ERR_INVALID;
    }
    const SpconvVariant* v = find_spconv_variant(f->brow, 0, nullptr); // the direct kernel, where one exists
    if (variant == 1) {
        if (!v) {
            set_error("spconv_init: no direct kernel for block size %d", f->brow);
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

// Points a state of the plane form at its scratch (planes | result_fm | ids | ids_pm, laid out by `g`) and sets
// up the SpMM launch in the middle.  The ids must be in the scratch when the state is executed.
static int bind_plane_form(shflbw_spconv_state* state, const shflbw_weight* f, const PlaneForm& g, char* scratch,
                           bool fused)
{
    state->planes = scratch;
    state->result_fm = scratch + g.planes_bytes;
    state->np = (int)g.np;
    state->plane_rows = g.PH;
    state->plane_cols = g.PW;
    state->plane_pitch = (int)g.pitch;
    state->plane_copies = g.copies;
    state->ncols = (int)g.ncols;
    state->sync = scratch + g.planes_bytes + g.dm_bytes + 2 * g.ids_bytes;
    // the three-launch form computes every plane position, the fused form only those of output rows
    int rc = fused ? shflbw_spmm_init_variant(&state->spmm, f, (int)g.ncols, state->planes, nullptr, state->result_fm, 1.f, 0.f, 0)
                   : shflbw_spmm_init(&state->spmm, f, (int)g.np, state->planes, nullptr, state->result_fm, 1.f, 0.f);
    if (rc != SHFLBW_OK) return rc;
    if (fused) {
        const ConvFusedKernel* k = conv_fused_kernel(f->brow);
        if (!k) {
            set_error("spconv_init: no fused kernel for block size %d", f->brow);
            return SHFLBW_ERR_UNSUPPORTED;
        }
        SHFLBW_HIP_TRY(k->prepare());
        state->spmm.shared_mem_size = (size_t)k->lds_bytes;
        state->spmm.grid_dim[0] = (unsigned)((f->nrow / f->brow) * ((g.ncols + k->BN - 1) / k->BN));
        state->spmm.block_dim[0] = (unsigned)k->threads;
    }
    // the gather walks the planes: ids are element offsets, one id apart is one value apart
    state->spmm.packed_indices = (const int*)(scratch + g.planes_bytes + g.dm_bytes);
    state->spmm.packed_indices_pm = (const int*)(scratch + g.planes_bytes + g.dm_bytes + g.ids_bytes);
    state->spmm.ldb_bytes = 2;
    state->spmm.args.K = (int)((g.rows + 1) * g.pitch); // extent of the id space
    state->shared_mem_size = state->spmm.shared_mem_size; // the figures of the middle (SpMM) launch
    state->grid_dim[0] = state->spmm.grid_dim[0];
    state->block_dim[0] = state->spmm.block_dim[0];
    state->grid_dim[1] = state->grid_dim[2] = 1;
    state->block_dim[1] = state->block_dim[2] = 1;
    state->init_success = 1;
    return SHFLBW_OK;
}

static int init_batch_planes(shflbw_spconv_state* state, const shflbw_weight* f, int B, int H, int W, int stride,
                             const void* IFMap, void* OFMap, int variant);

int shflbw_spconv_init_variant(shflbw_spconv_state* state, const shflbw_weight* f, int B, int H, int W, int stride,
                               const void* IFMap, void* OFMap, int variant)
{
    if (variant == 4) {
        if (state) memset(state, 0, sizeof(*state));
        set_error("spconv_init: form 4 works on C-H-W-B / F-H-W-B tensors; call shflbw_spconv_init_chwb");
        return SHFLBW_ERR_INVALID;
    }
    // the library's choice: the batch-innermost plane form where the batch allows it (one copy of the planes instead
    // of two, no dead plane rows in the result: cfg3 22.9 against 25.3 us, cfg4 24.0 against 25.9), else the plane form
    if (variant < 0) variant = B > 0 && B % 8 == 0 ? 5 : 0;
    if (variant == 5) return init_batch_planes(state, f, B, H, W, stride, IFMap, OFMap, 5);
    int frc = spconv_fill_state(state, f, B, H, W, stride, IFMap, OFMap, variant);
    if (frc != SHFLBW_OK) return frc;
    const int Ho = state->Ho, Wo = state->Wo;
    const SpconvVariant* v = find_spconv_variant(f->brow, 0, nullptr); // the direct kernel, where one exists
    const long npix = (long)B * Ho * Wo;
    // The scratch cache is bookkeeping of the handle, not part of the weight's value; it is the one member an
    // init call changes, under its lock.
    shflbw_weight* fw = const_cast<shflbw_weight*>(f);
    std::lock_guard<std::mutex> scratch_guard(fw->scratch_lock);
    const int key[5] = {variant, B, H, W, stride};
    auto cached_scratch = [&](size_t bytes, bool* fresh) -> void* {
        for (auto& sc : fw->conv_scratch)
            if (sc.bytes == bytes && memcmp(sc.key, key, sizeof(key)) == 0 && sc.in == IFMap && sc.out == OFMap) {
                *fresh = false;
                return sc.ptr;
            }
        void* ptr = nullptr;
        if (hipMalloc(&ptr, bytes) != hipSuccess) return nullptr;
        shflbw_weight::Scratch sc{bytes, ptr, {key[0], key[1], key[2], key[3], key[4]}, IFMap, OFMap};
        fw->conv_scratch.push_back(sc);
        *fresh = true;
        return ptr;
    };
    if (variant == 0 || variant == 3) {
        // plane forms: geometry of the phase planes (see spconv_gfx950.hip)
        PlaneForm g;
        int grc = plane_form_geometry(f, B, H, W, stride, &g);
        if (grc != SHFLBW_OK) return grc;
        const int s = stride;
        const long PW = g.PW, pitch = g.pitch;
        const int copies = g.copies;
        const size_t slots = g.slots, planes_bytes = g.planes_bytes, dm_bytes = g.dm_bytes, ids_bytes = g.ids_bytes;
        bool fresh = false;
        char* scratch = (char*)cached_scratch(g.total_bytes(), &fresh);
        if (!scratch) {
            set_error("spconv_init: cannot allocate %zu bytes of device scratch", g.total_bytes());
            return SHFLBW_ERR_HIP;
        }
        int* d_ids = (int*)(scratch + planes_bytes + dm_bytes);
        int* d_ids_pm = (int*)(scratch + planes_bytes + dm_bytes + ids_bytes);
        if (fresh) {
            // the tail of every channel row and the positions no image covers are read (for results
            // nobody uses) but never written
            SHFLBW_HIP_TRY(hipMemset(scratch, 0, planes_bytes));
            // the synchronisation words of the fused form start at zero (every launch leaves them so)
            SHFLBW_HIP_TRY(hipMemset(scratch + planes_bytes + dm_bytes + 2 * ids_bytes, 0, g.sync_bytes));
            // kept-column id k = (r*S + t)*C + c  ->  element offset of (copy, phase, channel) row + tap offset
            std::vector<int> ids(slots), ids_pm(slots);
            for (size_t q = 0; q < slots; q++) {
                const int k = f->packed_indices[q];
                if (k < 0) { // padding slot: the row of zeros behind the last channel row
                    ids[q] = (int)(g.rows * pitch);
                    continue;
                }
                const int c = k % f->C, tap = k / f->C, r = tap / f->S, t = tap % f->S;
                const long shift = (long)(r / s) * PW + t / s;
                const int copy = copies == 2 ? (int)(shift & 1) : 0;
                const int phase = (r % s) * s + t % s;
                ids[q] = (int)((((long)copy * s * s + phase) * f->C + c) * pitch + shift - copy);
            }
            for (size_t q = 0; q < slots; q++) { // producer-major order inside every 64-slot group
                const size_t grp = q / 64;
                const int j = (int)(q % 64) / 16, p = (int)(q % 16) / 4, r = (int)(q % 4);
                ids_pm[grp * 64 + 16 * p + 4 * j + r] = ids[q];
            }
            SHFLBW_HIP_TRY(hipMemcpy(d_ids, ids.data(), slots * sizeof(int), hipMemcpyHostToDevice));
            SHFLBW_HIP_TRY(hipMemcpy(d_ids_pm, ids_pm.data(), slots * sizeof(int), hipMemcpyHostToDevice));
        }
        return bind_plane_form(state, f, g, scratch, variant == 3);
    }
    if (variant == 2) {
        // im2col form: scratch for the im2col matrix [K][np] and the filter-major result [F][np]
        const long np = (npix + 63) / 64 * 64;
        const long K = (long)f->R * f->S * f->C;
        if (np > 0x7fffffffL || (unsigned long long)K * (unsigned long long)np * 2ull > 0xffffffffull) {
            set_error("spconv_init: problem too large for the im2col form (im2col matrix of %ld x %ld)", K, np);
            return SHFLBW_ERR_UNSUPPORTED;
        }
        const size_t bm_bytes = (size_t)K * np * 2, dm_bytes = (size_t)f->F * np * 2;
        bool fresh = false;
        void* scratch = cached_scratch(bm_bytes + dm_bytes, &fresh);
        if (!scratch) {
            set_error("spconv_init: cannot allocate %zu bytes of device scratch", bm_bytes + dm_bytes);
            return SHFLBW_ERR_HIP;
        }
        state->im2col = scratch;
        state->result_fm = (char*)scratch + bm_bytes;
        state->np = (int)np;
        int rc = shflbw_spmm_init(&state->spmm, f, (int)np, state->im2col, nullptr, state->result_fm, 1.f, 0.f);
        if (rc != SHFLBW_OK) return rc;
    }
    if (variant == 1) {
        state->shared_mem_size = (size_t)v->lds_bytes;
        state->grid_dim[0] = (unsigned)((f->F / f->brow) * ((npix + v->BN - 1) / v->BN));
        state->block_dim[0] = (unsigned)v->threads;
    } else { // the figures of the middle (SpMM) launch
        state->shared_mem_size = state->spmm.shared_mem_size;
        state->grid_dim[0] = state->spmm.grid_dim[0];
        state->block_dim[0] = state->spmm.block_dim[0];
    }
    state->grid_dim[1] = state->grid_dim[2] = 1;
    state->block_dim[1] = state->block_dim[2] = 1;
    state->init_success = 1;
    return SHFLBW_OK;
}

// Forms 4 and 5: phase planes with the batch innermost, planes[phase (a, b)][c][(i * PW + j) * B + img] =
// in(i * stride + a - R/2, j * stride + b - S/2) of image img and channel c, PHX = Ho + (R-1)/stride rows and
// PW = Wo + (S-1)/stride columns.  Every tap offset is a multiple of B values, 16 bytes or more: one copy of the
// planes serves all taps.  The SpMM runs over the Ho * PW * B columns (ho, j, img) of the padded output grid and
// drops the padding columns in its epilogue (output_column()).
//   form 4: the caller's tensors are C-H-W-B / F-H-W-B (the reference's), H and W bound input and output alike,
//           the SpMM writes OFMap itself;
//   form 5: the caller's tensors are NHWC with true stride and padding; the SpMM writes result_fm[f][(ho, wo, img)],
//           a tile transpose writes OFMap.
static int init_batch_planes(shflbw_spconv_state* state, const shflbw_weight* f, int B, int H, int W, int stride,
                             const void* IFMap, void* OFMap, int variant)
{
    int rc = spconv_fill_state(state, f, B, H, W, stride, IFMap, OFMap, variant);
    if (rc != SHFLBW_OK) return rc;
    if (B % 8 != 0) { // the reference's kernel moves 8 batch entries at a time too (spconv/blockwise_kernel.h:200-207)
        set_error("spconv_init: the batch must be a multiple of 8 for this form (got %d)", B);
        return SHFLBW_ERR_SHAPE;
    }
    const ConvChwbKernel* k = conv_chwb_kernel(f->brow);
    if (!k) {
        set_error("spconv_init: no kernel for block size %d", f->brow);
        return SHFLBW_ERR_UNSUPPORTED;
    }
    SHFLBW_HIP_TRY(k->prepare());
    if (variant == 4) { // H and W are the extents of the output grid and the bounds of the input (spconv/blockwise_format.h:111-115)
        state->Ho = H;
        state->Wo = W;
    }
    const int s = stride, Ho = state->Ho, Wo = state->Wo;
    const long PHX = Ho + (f->R - 1) / s, PW = Wo + (f->S - 1) / s;
    const long np = PHX * PW * B;                                  // values of one channel plane
    const long pitch = (np + (long)((f->S - 1) / s) * B + 8 + 63) / 64 * 64;
    const long rows = (long)s * s * f->C;
    const long ncols = (long)Ho * PW * B;                          // columns of the GEMM: the padded output grid
    if (ncols > 0x7fffffffL || (unsigned long long)(rows + 1) * (unsigned long long)pitch * 2ull > 0xffffffffull) {
        set_error("spconv_init: problem too large (%ld channel rows of %ld values)", rows, pitch);
        return SHFLBW_ERR_UNSUPPORTED;
    }
    auto up256 = [](size_t n) { return (n + 255) / 256 * 256; };
    const size_t slots = f->packed_indices.size();
    const size_t planes_bytes = up256((size_t)(rows + 1) * pitch * 2), ids_bytes = up256(slots * sizeof(int) + 64);
    const size_t dm_bytes = variant == 5 ? up256((size_t)f->F * Ho * Wo * B * 2) : 0;
    const size_t total = planes_bytes + dm_bytes + 2 * ids_bytes;
    shflbw_weight* fw = const_cast<shflbw_weight*>(f); // the scratch cache is bookkeeping of the handle (see shflbw_spconv_init_variant)
    std::lock_guard<std::mutex> scratch_guard(fw->scratch_lock);
    char* scratch = nullptr;
    const int key[5] = {variant, B, H, W, stride};
    for (auto& sc : fw->conv_scratch)
        if (sc.bytes == total && memcmp(sc.key, key, sizeof(key)) == 0 && sc.in == IFMap && sc.out == OFMap)
            scratch = (char*)sc.ptr;
    if (!scratch) {
        void* ptr = nullptr;
        if (hipMalloc(&ptr, total) != hipSuccess) {
            set_error("spconv_init: cannot allocate %zu bytes of device scratch", total);
            return SHFLBW_ERR_HIP;
        }
        fw->conv_scratch.push_back(shflbw_weight::Scratch{total, ptr, {variant, B, H, W, stride}, IFMap, OFMap});
        scratch = (char*)ptr;
        SHFLBW_HIP_TRY(hipMemset(scratch, 0, planes_bytes)); // includes the row of zeros behind the last channel row
        // kept-column id k = (r*S + t)*C + c  ->  element offset of the (phase, channel) row + tap offset
        std::vector<int> ids(slots), ids_pm(slots);
        for (size_t q = 0; q < slots; q++) {
            const int kk = f->packed_indices[q];
            if (kk < 0) {
                ids[q] = (int)(rows * pitch);
                continue;
            }
            const int c = kk % f->C, tap = kk / f->C, r = tap / f->S, t = tap % f->S;
            ids[q] = (int)((((long)(r % s) * s + t % s) * f->C + c) * pitch + ((long)(r / s) * PW + t / s) * B);
        }
        for (size_t q = 0; q < slots; q++) { // producer-major order inside every 64-slot group
            const size_t grp = q / 64;
            const int j = (int)(q % 64) / 16, p = (int)(q % 16) / 4, r = (int)(q % 4);
            ids_pm[grp * 64 + 16 * p + 4 * j + r] = ids[q];
        }
        char* ids_dev = scratch + planes_bytes + dm_bytes;
        SHFLBW_HIP_TRY(hipMemcpy(ids_dev, ids.data(), slots * sizeof(int), hipMemcpyHostToDevice));
        SHFLBW_HIP_TRY(hipMemcpy(ids_dev + ids_bytes, ids_pm.data(), slots * sizeof(int), hipMemcpyHostToDevice));
    }
    state->planes = scratch;
    state->result_fm = variant == 5 ? scratch + planes_bytes : nullptr;
    state->np = (int)np;
    state->plane_rows = (int)PHX;
    state->plane_cols = (int)PW;
    state->plane_pitch = (int)pitch;
    state->plane_copies = 1;
    state->ncols = (int)ncols;
    // the SpMM in the middle: row f of its result is the row of filter f, in OFMap itself (form 4) or in result_fm
    rc = shflbw_spmm_init_variant(&state->spmm, f, (int)ncols, state->planes, nullptr,
                                  variant == 5 ? state->result_fm : OFMap, 1.f, 0.f, 0);
    if (rc != SHFLBW_OK) return rc;
    state->spmm.packed_indices = (const int*)(scratch + planes_bytes + dm_bytes);
    state->spmm.packed_indices_pm = (const int*)(scratch + planes_bytes + dm_bytes + ids_bytes);
    state->spmm.ldb_bytes = 2;
    state->spmm.args.K = (int)((rows + 1) * pitch);
    state->shared_mem_size = (size_t)k->lds_bytes;
    state->grid_dim[0] = (unsigned)((f->nrow / f->brow) * ((ncols + k->BN - 1) / k->BN));
    state->block_dim[0] = (unsigned)k->threads;
    state->grid_dim[1] = state->grid_dim[2] = 1;
    state->block_dim[1] = state->block_dim[2] = 1;
    state->init_success = 1;
    return SHFLBW_OK;
}

int shflbw_spconv_init_chwb(shflbw_spconv_state* state, const shflbw_weight* f, int B, int H, int W, int stride,
                            const void* IFMap, void* OFMap)
{
    return init_batch_planes(state, f, B, H, W, stride, IFMap, OFMap, 4);
}

int shflbw_spconv_exec(const shflbw_spconv_state* state, void* stream)
{
    if (!state || !state->init_success) {
        set_error("spconv_exec: state was not initialised successfully");
        return SHFLBW_ERR_STATE;
    }
    const SpconvVariant* v = find_spconv_variant(state->brow, 0, nullptr); // the direct kernel of this block size
    if (!v && state->variant == 1) return SHFLBW_ERR_UNSUPPORTED;
    SpconvLaunchArgs a;
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
    if (state->variant == 4 || state->variant == 5) {
        const ConvChwbKernel* k = conv_chwb_kernel(state->brow);
        if (!k) return SHFLBW_ERR_UNSUPPORTED;
        const bool nhwc = state->variant == 5;
        hipError_t e = nhwc ? launch_nhwc_to_planes(a, (half_t*)state->planes, state->plane_rows, state->plane_cols,
                                                    state->plane_pitch, 1, (hipStream_t)stream, 1)
                            : launch_chwb_to_planes(a.in, (half_t*)state->planes, a.B, a.H, a.W, a.C, a.R, a.S, a.stride,
                                                    state->plane_rows, state->plane_cols, state->plane_pitch,
                                                    (hipStream_t)stream);
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
        if (e != hipSuccess) {
            set_error("spconv_exec: launch failed: %s", hipGetErrorString(e));
            return SHFLBW_ERR_HIP;
        }
        return SHFLBW_OK;
    }
    if (state->variant == 3) {
        const ConvFusedKernel* k = conv_fused_kernel(state->brow);
        if (!k) return SHFLBW_ERR_UNSUPPORTED;
        SpmmLaunchArgs m;
        fill_spmm_launch_args(&state->spmm, k->BN, &m);
        if (m.X == 0) return SHFLBW_OK;
        m.alternate = 0; // the planes under one column tile are far smaller than an L2
        m.img_cols = a.Ho * state->plane_cols;
        m.img_skip = (state->plane_rows - a.Ho) * state->plane_cols;
        m.tile_arrivals = (int*)state->sync + CONV_LINE_SLAB0 * SYNC_LINE;
        ConvFuseArgs c;
        c.g = PlaneGeom{a.B, a.H, a.W, a.C, a.stride, a.pad_h, a.pad_w, state->plane_rows, state->plane_cols,
                        state->plane_pitch, state->plane_copies, 0, {}};
        if (!fill_wanted_planes(c.g, a.R, a.S)) return SHFLBW_ERR_UNSUPPORTED;
        // chunks of the two layout phases: 8, 4 or 2 tiles of 64 x 64, the largest size that still gives every
        // workgroup a chunk; along the contiguous axis of the source (channels, filters) as many tiles as there are
        auto pow2_le = [](int n, int cap) { int p = 1; while (p * 2 <= n && p * 2 <= cap) p *= 2; return p; };
        const int grid = std::min((m.num_cus / 8) * 8, ((m.X * ((state->ncols + k->BN - 1) / k->BN) + 7) / 8) * 8);
        c.in = a.in;
        c.planes = (half_t*)state->planes;
        c.np64 = (state->np + 63) / 64 * 64;
        for (int tiles = 8; tiles >= 2; tiles >>= 1) {
            c.ct = pow2_le((a.C + 63) / 64, tiles);
            c.pt = tiles / c.ct;
            c.ch_chunks = (a.C + c.ct * 64 - 1) / (c.ct * 64);
            c.pos_chunks = (c.np64 + c.pt * 64 - 1) / (c.pt * 64);
            c.n0chunks = c.g.nwanted * c.ch_chunks * c.pos_chunks;
            if (c.n0chunks >= grid) break;
        }
        c.fm = (const half_t*)state->result_fm;
        c.out = a.out;
        c.F = a.F;
        c.ncols = state->ncols;
        c.Ho = a.Ho;
        c.Wo = a.Wo;
        for (int tiles = 8; tiles >= 2; tiles >>= 1) {
            c.ft = pow2_le((a.F + 63) / 64, tiles);
            c.mt = tiles / c.ft;
            c.f_chunks = (a.F + c.ft * 64 - 1) / (c.ft * 64);
            if (c.f_chunks * ((k->BN / 64 + c.mt - 1) / c.mt) >= m.X) break; // a chunk for every workgroup of a column tile
        }
        c.slabs = (state->ncols + k->BN - 1) / k->BN;
        c.arrivals_per_slab = m.X;
        c.sync = (int*)state->sync;
        c.magic_ps = udiv_magic(state->plane_rows * state->plane_cols);
        c.magic_pw = udiv_magic(state->plane_cols);
        c.magic_imgcols = udiv_magic(a.Ho * state->plane_cols);
        c.help_ticks = 3000; // 30 us
        // Measurement knob: SHFLBW_FUSED_PHASES (bit 0: input rewrite inside the launch, bit 1: NHWC output inside
        // the launch; default 3).  A cleared bit runs that step as its own launch around the fused kernel.
        static const int phases = [] {
            const char* e = getenv("SHFLBW_FUSED_PHASES");
            return e ? atoi(e) & 3 : 3;
        }();
        c.phases = phases;
        hipError_t e = hipSuccess;
        if (!(phases & 1))
            e = launch_nhwc_to_planes(a, (half_t*)state->planes, state->plane_rows, state->plane_cols, state->plane_pitch,
                                      state->plane_copies, (hipStream_t)stream);
        if (e == hipSuccess) e = k->launch(m, c, (hipStream_t)stream);
        if (e == hipSuccess && !(phases & 2)) // the compact result has Ho rows per image
            e = launch_planes_to_nhwc((const half_t*)state->result_fm, a.out, a.F, state->ncols, a.B, a.Ho,
                                      state->plane_cols, a.Ho, a.Wo, (hipStream_t)stream);
        if (e != hipSuccess) {
            set_error("spconv_exec: fused launch failed: %s", hipGetErrorString(e));
            return SHFLBW_ERR_HIP;
        }
        return SHFLBW_OK;
    }
    if (state->variant == 0) {
        hipError_t e = launch_nhwc_to_planes(a, (half_t*)state->planes, state->plane_rows, state->plane_cols,
                                             state->plane_pitch, state->plane_copies, (hipStream_t)stream);
        if (e != hipSuccess) {
            set_error("spconv_exec: plane layout launch failed: %s", hipGetErrorString(e));
            return SHFLBW_ERR_HIP;
        }
        int rc = shflbw_spmm_exec(&state->spmm, stream);
        if (rc != SHFLBW_OK) return rc;
        e = launch_planes_to_nhwc((const half_t*)state->result_fm, a.out, a.F, state->np, a.B, state->plane_rows,
                                  state->plane_cols, a.Ho, a.Wo, (hipStream_t)stream);
        if (e != hipSuccess) {
            set_error("spconv_exec: transpose launch failed: %s", hipGetErrorString(e));
            return SHFLBW_ERR_HIP;
        }
        return SHFLBW_OK;
    }
    if (state->variant == 2) {
        hipError_t e = launch_im2col_nhwc(a, (half_t*)state->im2col, state->np, (hipStream_t)stream);
        if (e != hipSuccess) {
            set_error("spconv_exec: im2col launch failed: %s", hipGetErrorString(e));
            return SHFLBW_ERR_HIP;
        }
        int rc = shflbw_spmm_exec(&state->spmm, stream);
        if (rc != SHFLBW_OK) return rc;
        e = launch_transpose_to_nhwc((const half_t*)state->result_fm, a.out, a.F, a.B * a.Ho * a.Wo, state->np,
                                     (hipStream_t)stream);
        if (e != hipSuccess) {
            set_error("spconv_exec: transpose launch failed: %s", hipGetErrorString(e));
            return SHFLBW_ERR_HIP;
        }
        return SHFLBW_OK;
    }
    hipError_t e = v->launch(a, (hipStream_t)stream);
    if (e != hipSuccess) {
        set_error("spconv_exec: launch failed: %s", hipGetErrorString(e));
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
    int rc = spconv_fill_state(&st, f, B, H, W, stride, IFMap, OFMap, 0);
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
    if ((rc = bind_plane_form(&st, f, g, base, false)) != SHFLBW_OK) return rc;
    hipError_t e = launch_plane_ids((const int*)f->d_packed_indices, (int*)(base + g.planes_bytes + g.dm_bytes),
                                    (int*)(base + g.planes_bytes + g.dm_bytes + g.ids_bytes), (int)g.slots, f->C, f->S,
                                    stride, g.PW, (int)g.pitch, g.copies, (int)(g.rows * g.pitch), (half_t*)base,
                                    (hipStream_t)stream);
    if (e != hipSuccess) {
        set_error("spconv_exec_static: id launch failed: %s", hipGetErrorString(e));
        return SHFLBW_ERR_HIP;
    }
    return shflbw_spconv_exec(&st, stream);
}

static const char* const g_spconv_forms[] = {
    "planes+spmm+transpose",  // 0: NHWC -> channel-major planes, SpMM gather with tap offsets, transpose to NHWC: three launches
    "direct",                 // 1: one kernel, im2col gather from NHWC in the tile loads
    "im2col+spmm+transpose",  // 2: explicit im2col matrix, three launches
    "fused-planes",           // 3: the steps of form 0 in one persistent launch
    "chwb-planes+spmm",       // 4: the reference's batch-innermost tensors (shflbw_spconv_init_chwb only): padded copy, SpMM
    "bplanes+spmm+transpose", // 5: NHWC tensors, planes and result with the batch innermost (batch a multiple of 8): three launches
};

int shflbw_spconv_variant_count(void) { return (int)(sizeof(g_spconv_forms) / sizeof(g_spconv_forms[0])); }

const char* shflbw_spconv_variant_name(int variant)
{
    return variant >= 0 && variant < shflbw_spconv_variant_count() ? g_spconv_forms[variant] : "";
}

int shflbw_weight_release_scratch(shflbw_weight* w)
{
    if (!w) return SHFLBW_ERR_INVALID;
    std::lock_guard<std::mutex> guard(w->scratch_lock);
    for (auto& sc : w->conv_scratch)
        if (sc.ptr) (void)hipFree(sc.ptr);
    w->conv_scratch.clear();
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
