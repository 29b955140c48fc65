// Host side of the Shfl-BW weight format behind the C ABI: mask generator, random
// initialisation, text dump/load, the reference-format meta image and the private
// MFMA-ordered image.  Reference: block_sparse/util/random_mask.cc,
// block_sparse/spmm/blockwise_format.h, block_sparse/spconv/blockwise_format.h.
#include "weight_internal.h"

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <random>
#include <sstream>

namespace shflbw {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

float half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h >> 15) << 31;
    int exp = (h >> 10) & 31;
    uint32_t man = h & 1023u;
    uint32_t out;
    if (exp == 31) {
        out = sign | 0x7f800000u | (man << 13);
    } else if (exp != 0) {
        out = sign | (uint32_t)(exp + 112) << 23 | (man << 13);
    } else if (man == 0) {
        out = sign;
    } else {
        // subnormal half = man * 2^-24: exact in float
        float f = (float)man * 5.9604644775390625e-8f;
        memcpy(&out, &f, 4);
        out |= sign;
    }
    float r;
    memcpy(&r, &out, 4);
    return r;
}

uint16_t float_to_half(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    u &= 0x7fffffffu;
    if (u > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((u >> 13) & 0x3ffu)); // NaN
    if (u >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);                       // overflow -> inf
    if (u < 0x33000001u) return sign;                                              // <= 2^-25 -> 0 (ties to even)
    int e = (int)(u >> 23);
    uint32_t m = (u & 0x7fffffu) | 0x800000u;
    int drop = (e >= 113) ? 13 : (126 - e); // bits discarded from the 24-bit significand
    uint32_t kept = m >> drop;
    uint32_t rest = m & ((1u << drop) - 1u);
    uint32_t half_ulp = 1u << (drop - 1);
    if (rest > half_ulp || (rest == half_ulp && (kept & 1u))) kept++;
    uint32_t bits = (e >= 113) ? (((uint32_t)(e - 113) << 10) + kept) // kept carries the hidden bit: adds 1 to the exponent field
                               : kept;
    return (uint16_t)(sign | bits);
}

void clear_device(shflbw_weight* w); // defined in device.hip

// ---------------------------------------------------------------------------------
// mask: util/random_mask.cc:10-57.  The bits of the result depend on libstdc++'s
// std::shuffle and std::default_random_engine, so exactly those calls are made.
// ---------------------------------------------------------------------------------
static int random_mask_impl(int nrow, int ncol, int brow, int bcol, float block_density,
                            int block_divisor, int block_padding, unsigned seed,
                            int& nnzb, int& padded_nnzb, std::vector<int>& indptr, std::vector<int>& indices)
{
    if (nrow <= 0 || ncol <= 0 || brow <= 0 || bcol <= 0 || block_divisor <= 0 || block_padding <= 0) {
        set_error("random_mask: non-positive size");
        return SHFLBW_ERR_INVALID;
    }
    const int X = nrow / brow;
    const int Y = ncol / bcol;
    const int groups_kept = (int)(std::round(block_density * X * Y / block_divisor));
    const long total_groups = (long)X * (Y / block_divisor);
    if (groups_kept < 0 || groups_kept > total_groups) {
        set_error("random_mask: density %g out of range", (double)block_density);
        return SHFLBW_ERR_INVALID;
    }
    nnzb = groups_kept * block_divisor;

    // which panel each kept group falls into: shuffle all candidate slots, keep a prefix
    std::vector<int> slot(total_groups);
    std::iota(slot.begin(), slot.end(), 0);
    std::shuffle(slot.begin(), slot.end(), std::default_random_engine(seed));
    std::vector<int> per_panel(X, 0);
    for (int g = 0; g < groups_kept; g++) per_panel[slot[g] % X] += block_divisor;

    indptr.assign(1, 0);
    indptr.reserve(X + 1);
    indices.clear();
    indices.reserve(nnzb + (size_t)X * (block_padding - 1));
    std::vector<int> cols(Y);
    int running = 0, kept_total = 0;
    for (int i = 0; i < X; i++) {
        std::iota(cols.begin(), cols.end(), 0);
        std::shuffle(cols.begin(), cols.end(), std::default_random_engine(seed + i + 1));
        const int cnt = per_panel[i];
        std::sort(cols.begin(), cols.begin() + cnt);
        indices.insert(indices.end(), cols.begin(), cols.begin() + cnt);
        kept_total += cnt;
        running += cnt;
        for (; running % block_padding != 0; running++) indices.push_back(cols[cnt - 1]);
        indptr.push_back(running);
    }
    if (kept_total != nnzb) {
        set_error("random_mask: internal count mismatch");
        return SHFLBW_ERR_INVALID;
    }
    padded_nnzb = running;
    return SHFLBW_OK;
}

static void make_config_str(shflbw_weight* w)
{
    std::stringstream s;
    if (w->R > 0) { // spconv/blockwise_format.h:42-51
        s << w->F << " " << w->R << " " << w->S << " " << w->C << " " << w->brow << " " << w->bcol << " "
          << w->density << " " << w->seed << " " << (w->row_permute ? "filter-permute " : "non-filter-permute ");
    } else { // spmm/blockwise_format.h:105-114
        s << w->nrow << " " << w->ncol << " " << w->brow << " " << w->bcol << " " << w->density << " " << w->seed
          << " " << (w->row_permute ? "row-permute " : "non-row-permute ");
    }
    w->config_str = s.str();
}

static void mark_initialized(shflbw_weight* w)
{
    w->initialized = true;
    if (w->device_synced) { // blockwise_format.h:118-122
        clear_device(w);
        w->device_synced = false;
    }
    w->meta_h.clear();
    w->group_ptr.clear();
    w->panel_desc.clear();
    w->packed_indices.clear();
    w->packed_indices_pm.clear();
    w->packed_values.clear();
    w->packed_slab.clear();
}

static int check_pattern(int nrow, int ncol, int brow, int bcol, int nnzb, const int* indptr, const int* indices,
                         const int* perm)
{
    if (nrow <= 0 || ncol <= 0 || brow <= 0 || bcol <= 0 || nnzb < 0) {
        set_error("weight: non-positive size");
        return SHFLBW_ERR_INVALID;
    }
    if (nrow % brow != 0 || ncol % bcol != 0) { // blockwise_format.h:74-75
        set_error("weight: nrow %% brow or ncol %% bcol != 0 (%d %% %d, %d %% %d)", nrow, brow, ncol, bcol);
        return SHFLBW_ERR_SHAPE;
    }
    const int X = nrow / brow, Y = ncol / bcol;
    if (indptr[0] != 0 || indptr[X] != nnzb) {
        set_error("weight: indptr[0] must be 0 and indptr[X] must equal nnzb");
        return SHFLBW_ERR_FORMAT;
    }
    for (int i = 0; i < X; i++)
        if (indptr[i + 1] < indptr[i]) {
            set_error("weight: indptr not monotone at panel %d", i);
            return SHFLBW_ERR_FORMAT;
        }
    for (int p = 0; p < nnzb; p++)
        if (indices[p] < 0 || indices[p] >= Y) {
            set_error("weight: column index %d out of range at %d", indices[p], p);
            return SHFLBW_ERR_FORMAT;
        }
    if (perm) {
        std::vector<char> seen(nrow, 0);
        for (int r = 0; r < nrow; r++) {
            if (perm[r] < 0 || perm[r] >= nrow || seen[perm[r]]) {
                set_error("weight: row_permute_ids is not a permutation (entry %d)", r);
                return SHFLBW_ERR_FORMAT;
            }
            seen[perm[r]] = 1;
        }
    }
    return SHFLBW_OK;
}

// ---------------------------------------------------------------------------------
// private image.  Panel i keeps nnz_i vectors; they are padded to a multiple of 64
// slots.  packed_indices: the column ids, tail slots hold -1 (their values are zero and
// the kernels gather a row of zeros for them, so that a non-finite B cannot leak through 0 * x).  packed_values: per MFMA k-step, the A operand in register
// order, so one wave reads a fragment as 64 consecutive 16-byte pieces:
//   V >= 32 (32x32x16 tiles): step s covers slots 16s..16s+15; block mb covers rows
//     32mb..32mb+31; lane l holds row 32mb + l%32, slots 16s + 8*(l/32) + 0..7.
//   V == 16 (16x16x32 tiles): step s covers slots 32s..32s+31; lane l holds row l%16,
//     slots 32s + 8*(l/16) + 0..7.
// ---------------------------------------------------------------------------------
int build_packed_image(shflbw_weight* w)
{
    if (w->bcol != 1) {
        set_error("private image needs bcol == 1 (got %d)", w->bcol);
        return SHFLBW_ERR_UNSUPPORTED;
    }
    const int V = w->brow;
    if (V != 16 && V != 32 && V != 64 && V != 128) {
        set_error("no gfx950 kernel for block size %d (16, 32, 64, 128 are built)", V);
        return SHFLBW_ERR_UNSUPPORTED;
    }
    const int X = w->nrow / V;
    w->group_ptr.assign(X + 1, 0);
    for (int i = 0; i < X; i++) {
        int nnz = w->indptr[i + 1] - w->indptr[i];
        w->group_ptr[i + 1] = w->group_ptr[i] + (nnz + 63) / 64;
    }
    w->panel_desc.assign(2 * (size_t)X, 0);
    for (int i = 0; i < X; i++) {
        w->panel_desc[2 * i] = (w->indptr[i + 1] - w->indptr[i] + 15) / 16;
        w->panel_desc[2 * i + 1] = w->group_ptr[i];
    }
    const size_t slots = (size_t)w->group_ptr[X] * 64;
    w->packed_indices.assign(slots, 0);
    w->packed_indices_pm.assign(slots, 0);
    w->packed_values.assign(slots * V, 0);
    const bool slab = V == 32 && w->ncol <= SLAB_MAX_K;
    w->packed_slab.assign(slab ? slots : 0, 0);
    for (int i = 0; i < X; i++) {
        const int begin = w->indptr[i], nnz = w->indptr[i + 1] - begin;
        const size_t slot0 = (size_t)w->group_ptr[i] * 64;
        const int padded = (w->group_ptr[i + 1] - w->group_ptr[i]) * 64;
        // Order of the panel's kept vectors in the image: ascending ids, except for the slab form.  There the four
        // slab rows of slots 4j .. 4j+3 are read by one LDS instruction and should lie in four different bank
        // groups (slab_bank_class): every quad takes the next id of each of the classes with the most ids left.
        std::vector<int> ord(nnz);
        for (int q = 0; q < nnz; q++) ord[q] = q;
        if (slab) {
            std::vector<int> of_class[4];
            for (int q = nnz - 1; q >= 0; q--) of_class[slab_bank_class(w->indices[begin + q])].push_back(q); // back() = smallest id
            for (int q = 0; q < nnz;) {
                int cls[4] = {0, 1, 2, 3};
                std::stable_sort(cls, cls + 4, [&](int x, int y) { return of_class[x].size() > of_class[y].size(); });
                const int quad_end = std::min(nnz, q + 4);
                for (int t = 0; q < quad_end; t++) {
                    std::vector<int>& from = of_class[cls[t % 4]];
                    if (from.empty()) continue; // fewer than four classes left: the fullest ones give a second id
                    ord[q++] = from.back();
                    from.pop_back();
                }
            }
        }
        for (int q = 0; q < padded; q++)
            w->packed_indices[slot0 + q] = q < nnz ? w->indices[begin + ord[q]] : -1; // padding: gathered from a row of zeros
        for (int q = 0; q < padded; q++) {
            const int grp = q / 64, j = (q % 64) / 16, p = (q % 16) / 4, r = q % 4;
            w->packed_indices_pm[slot0 + grp * 64 + 16 * p + 4 * j + r] = w->packed_indices[slot0 + q];
        }
        // slab form: a lane of the consumer addresses slots s and s + 4 of every 16-slot step, s = 8 (pair / 4) +
        // pair % 4 for its pair number 0..7; the eight offsets a lane needs for the four steps of a group are
        // stored together, [group][pair][step][s, s + 4]
        for (int q = 0; slab && q < padded; q++) {
            const int grp = q / 64, step = (q % 64) / 16, s = q % 16;
            const int pair = (s / 8) * 4 + s % 4, hi = (s % 8) / 4;
            w->packed_slab[slot0 + grp * 64 + pair * 8 + step * 2 + hi] = slab_row_offset(w->packed_indices[slot0 + q], w->ncol);
        }
        uint16_t* dst = w->packed_values.data() + slot0 * V;
        const uint16_t* src = w->values.data() + (size_t)begin * V;
        if (V >= 32) {
            const int MB = V / 32;
            for (int q = 0; q < nnz; q++) {
                const int s = q / 16, half_k = (q % 16) / 8, j = q % 8;
                for (int r = 0; r < V; r++) {
                    const int mb = r / 32, lane = half_k * 32 + r % 32;
                    dst[(((size_t)s * MB + mb) * 64 + lane) * 8 + j] = src[(size_t)ord[q] * V + r];
                }
            }
        } else {
            for (int q = 0; q < nnz; q++) {
                const int s = q / 32, quarter = (q % 32) / 8, j = q % 8;
                for (int r = 0; r < 16; r++) {
                    const int lane = quarter * 16 + r;
                    dst[((size_t)s * 64 + lane) * 8 + j] = src[(size_t)ord[q] * 16 + r];
                }
            }
        }
    }
    return SHFLBW_OK;
}

// reference-format meta image: blockwise_format.h:205-229
static void build_meta(shflbw_weight* w)
{
    auto up8 = [](size_t n) { return (n + 7) / 8 * 8; };
    const size_t o_idx = up8(w->indptr.size());
    const size_t o_perm = o_idx + up8(w->indices.size());
    w->meta_h.assign(o_perm + up8(w->row_permute_ids.size()), 0);
    std::copy(w->indptr.begin(), w->indptr.end(), w->meta_h.begin());
    for (size_t p = 0; p < w->indices.size(); p++) w->meta_h[o_idx + p] = w->indices[p] * w->bcol;
    std::copy(w->row_permute_ids.begin(), w->row_permute_ids.end(), w->meta_h.begin() + o_perm);
}

int upload(shflbw_weight* w); // device.hip

} // namespace shflbw

using namespace shflbw;

extern "C" {

const char* shflbw_status_string(int status)
{
    switch (status) {
    case SHFLBW_OK: return "ok";
    case SHFLBW_ERR_INVALID: return "invalid argument";
    case SHFLBW_ERR_SHAPE: return "shape precondition violated";
    case SHFLBW_ERR_STATE: return "object not initialised or not synced to the device";
    case SHFLBW_ERR_HIP: return "HIP runtime error";
    case SHFLBW_ERR_UNSUPPORTED: return "unsupported configuration";
    case SHFLBW_ERR_FORMAT: return "malformed input";
    case SHFLBW_ERR_CAPACITY: return "buffer too small";
    default: return "unknown status";
    }
}

const char* shflbw_last_error(void) { return g_err; }

int shflbw_random_mask_ex(int nrow, int ncol, int brow, int bcol, float block_density, int block_divisor,
                          int block_padding, unsigned seed, int* nnzb, int* padded_nnzb, int* indptr, int* indices,
                          size_t indices_cap)
{
    if (!nnzb || !padded_nnzb || !indptr || !indices) {
        set_error("random_mask: null output");
        return SHFLBW_ERR_INVALID;
    }
    std::vector<int> ip, ix;
    int rc = random_mask_impl(nrow, ncol, brow, bcol, block_density, block_divisor, block_padding, seed, *nnzb,
                              *padded_nnzb, ip, ix);
    if (rc) return rc;
    if (ix.size() > indices_cap) {
        set_error("random_mask: indices need %zu ints, capacity %zu", ix.size(), indices_cap);
        return SHFLBW_ERR_CAPACITY;
    }
    std::copy(ip.begin(), ip.end(), indptr);
    std::copy(ix.begin(), ix.end(), indices);
    return SHFLBW_OK;
}

int shflbw_random_mask(int nrow, int ncol, int brow, int bcol, float block_density, unsigned seed, int* nnzb,
                       int* indptr, int* indices, size_t indices_cap)
{
    int padded = 0; // random_mask.cc:59-67: divisor 1, padding 1
    return shflbw_random_mask_ex(nrow, ncol, brow, bcol, block_density, 1, 1, seed, nnzb, &padded, indptr, indices,
                                 indices_cap);
}

int shflbw_weight_create(shflbw_weight** out)
{
    if (!out) return SHFLBW_ERR_INVALID;
    *out = new (std::nothrow) shflbw_weight();
    return *out ? SHFLBW_OK : SHFLBW_ERR_INVALID;
}

void shflbw_weight_destroy(shflbw_weight* w)
{
    if (!w) return;
    if (w->device_synced) clear_device(w);
    delete w;
}

int shflbw_weight_init_random(shflbw_weight* w, int nrow, int ncol, int brow, int bcol, float expected_density,
                              int row_permute, unsigned seed)
{
    if (!w) return SHFLBW_ERR_INVALID;
    if (nrow <= 0 || ncol <= 0 || brow <= 0 || bcol <= 0) {
        set_error("init_random: non-positive size");
        return SHFLBW_ERR_INVALID;
    }
    if (nrow % brow != 0 || ncol % bcol != 0) { // asserts at blockwise_format.h:74-75
        set_error("init_random: nrow %% brow or ncol %% bcol != 0");
        return SHFLBW_ERR_SHAPE;
    }
    int nnzb = 0, padded = 0;
    std::vector<int> ip, ix;
    int rc = random_mask_impl(nrow, ncol, brow, bcol, expected_density, 1, 1, seed, nnzb, padded, ip, ix);
    if (rc) return rc;
    w->nrow = nrow;
    w->ncol = ncol;
    w->brow = brow;
    w->bcol = bcol;
    w->seed = seed;
    w->row_permute = row_permute != 0;
    w->nnzb = nnzb;
    w->indptr.swap(ip);
    w->indices.swap(ix);
    w->density = (float)nnzb / (nrow / brow) / (ncol / bcol);
    w->F = w->R = w->S = w->C = 0;
    if (w->row_permute) { // :89-95
        w->row_permute_ids.resize(nrow);
        std::iota(w->row_permute_ids.begin(), w->row_permute_ids.end(), 0);
        std::shuffle(w->row_permute_ids.begin(), w->row_permute_ids.end(), std::default_random_engine(seed));
    } else {
        w->row_permute_ids.clear();
    }
    w->values.resize((size_t)nnzb * brow * bcol); // :99-102
    for (auto& v : w->values) v = float_to_half((float)(std::rand() % 9 - 4));
    make_config_str(w);
    mark_initialized(w);
    return SHFLBW_OK;
}

int shflbw_filter_init_random(shflbw_weight* w, int F, int R, int S, int C, int brow, int bcol,
                              float expected_density, int filter_permute, unsigned seed)
{
    if (!w) return SHFLBW_ERR_INVALID;
    if (F <= 0 || R <= 0 || S <= 0 || C <= 0) {
        set_error("filter init_random: non-positive size");
        return SHFLBW_ERR_INVALID;
    }
    int rc = shflbw_weight_init_random(w, F, R * S * C, brow, bcol, expected_density, filter_permute, seed);
    if (rc) return rc;
    w->F = F;
    w->R = R;
    w->S = S;
    w->C = C;
    make_config_str(w);
    return SHFLBW_OK;
}

int shflbw_weight_set(shflbw_weight* w, int nrow, int ncol, int brow, int bcol, int nnzb, const int* indptr,
                      const int* indices, const uint16_t* values, const int* row_permute_ids, int R, int S, int C)
{
    if (!w || !indptr || (nnzb > 0 && (!indices || !values))) {
        set_error("weight_set: null array");
        return SHFLBW_ERR_INVALID;
    }
    int rc = check_pattern(nrow, ncol, brow, bcol, nnzb, indptr, indices, row_permute_ids);
    if (rc) return rc;
    if ((R | S | C) != 0 && (R <= 0 || S <= 0 || C <= 0 || (long)R * S * C != ncol)) {
        set_error("weight_set: filter view R*S*C (%d*%d*%d) != ncol %d", R, S, C, ncol);
        return SHFLBW_ERR_SHAPE;
    }
    const int X = nrow / brow;
    // Arrays equal to what the weight already holds change nothing: the device image, the states made from it,
    // the seed and the config string stay valid (the veneer hands its public vectors over before every dump
    // and sync, and the reference's dump is read-only, blockwise_format.h:125-149).
    if (w->initialized && w->nrow == nrow && w->ncol == ncol && w->brow == brow && w->bcol == bcol &&
        w->nnzb == nnzb && w->row_permute == (row_permute_ids != nullptr) && w->R == R && w->S == S && w->C == C &&
        std::equal(indptr, indptr + X + 1, w->indptr.begin()) && std::equal(indices, indices + nnzb, w->indices.begin()) &&
        std::equal(values, values + (size_t)nnzb * brow * bcol, w->values.begin()) &&
        (!row_permute_ids || std::equal(row_permute_ids, row_permute_ids + nrow, w->row_permute_ids.begin())))
        return SHFLBW_OK;
    w->nrow = nrow;
    w->ncol = ncol;
    w->brow = brow;
    w->bcol = bcol;
    w->nnzb = nnzb;
    w->seed = 0;
    w->row_permute = row_permute_ids != nullptr;
    w->indptr.assign(indptr, indptr + X + 1);
    w->indices.assign(indices, indices + nnzb);
    w->values.assign(values, values + (size_t)nnzb * brow * bcol);
    if (row_permute_ids)
        w->row_permute_ids.assign(row_permute_ids, row_permute_ids + nrow);
    else
        w->row_permute_ids.clear();
    w->density = (float)nnzb / X / (ncol / bcol);
    w->F = R > 0 ? nrow : 0;
    w->R = R;
    w->S = S;
    w->C = C;
    make_config_str(w);
    mark_initialized(w);
    return SHFLBW_OK;
}

int shflbw_weight_set_values(shflbw_weight* w, const uint16_t* values, size_t count)
{
    if (!w || !values) return SHFLBW_ERR_INVALID;
    if (!w->initialized) {
        set_error("set_values: weight not initialised");
        return SHFLBW_ERR_STATE;
    }
    if (count != w->values.size()) {
        set_error("set_values: expected %zu values, got %zu", w->values.size(), count);
        return SHFLBW_ERR_SHAPE;
    }
    w->values.assign(values, values + count);
    mark_initialized(w);
    return SHFLBW_OK;
}

int shflbw_weight_dump_text(const shflbw_weight* w, char* buf, size_t cap, size_t* needed)
{
    if (!w || !needed) return SHFLBW_ERR_INVALID;
    if (!w->initialized) {
        set_error("dump: weight not initialised");
        return SHFLBW_ERR_STATE;
    }
    // same stream formatting as blockwise_format.h:125-149 so the text is identical
    std::ostringstream out;
    out << w->nrow << std::endl << w->ncol << std::endl << w->nnzb << std::endl;
    out << w->brow << std::endl << w->bcol << std::endl << w->row_permute << std::endl;
    for (int x = 0; x < w->nrow / w->brow + 1; x++) out << w->indptr[x] << " ";
    out << std::endl;
    for (int x = 0; x < w->nnzb; x++) out << w->indices[x] << " ";
    out << std::endl;
    for (size_t x = 0; x < w->values.size(); x++) out << half_to_float(w->values[x]) << " ";
    out << std::endl;
    if (w->row_permute) {
        for (int x = 0; x < w->nrow; x++) out << w->row_permute_ids[x] << " ";
        out << std::endl;
    }
    const std::string s = out.str();
    *needed = s.size();
    if (buf && cap > 0) memcpy(buf, s.data(), std::min(cap, s.size()));
    if (buf && cap < s.size()) return SHFLBW_ERR_CAPACITY;
    return SHFLBW_OK;
}

int shflbw_weight_load_text(shflbw_weight* w, const char* text, size_t len)
{
    if (!w || !text) return SHFLBW_ERR_INVALID;
    std::istringstream in(std::string(text, len));
    int nrow, ncol, nnzb, brow, bcol, rp; // :154
    if (!(in >> nrow >> ncol >> nnzb >> brow >> bcol >> rp)) {
        set_error("load: cannot read the six header numbers");
        return SHFLBW_ERR_FORMAT;
    }
    if (nrow <= 0 || ncol <= 0 || brow <= 0 || bcol <= 0 || nnzb < 0 || nrow % brow || ncol % bcol) {
        set_error("load: bad header %d %d %d %d %d", nrow, ncol, nnzb, brow, bcol);
        return SHFLBW_ERR_FORMAT;
    }
    const int X = nrow / brow;
    std::vector<int> ip(X + 1), ix(nnzb), perm;
    std::vector<uint16_t> vals((size_t)nnzb * brow * bcol);
    for (auto& v : ip) in >> v;
    for (auto& v : ix) in >> v;
    for (auto& v : vals) {
        float y;
        in >> y;
        v = float_to_half(y);
    }
    if (rp) {
        perm.resize(nrow);
        for (auto& v : perm) in >> v;
    }
    if (!in) {
        set_error("load: text ended early or holds a non-number");
        return SHFLBW_ERR_FORMAT;
    }
    return shflbw_weight_set(w, nrow, ncol, brow, bcol, nnzb, ip.data(), ix.data(), vals.data(),
                             rp ? perm.data() : nullptr, 0, 0, 0);
}

int shflbw_weight_get_info(const shflbw_weight* w, shflbw_weight_info* info)
{
    if (!w || !info) return SHFLBW_ERR_INVALID;
    info->nrow = w->nrow;
    info->ncol = w->ncol;
    info->nnzb = w->nnzb;
    info->brow = w->brow;
    info->bcol = w->bcol;
    info->density = w->density;
    info->seed = w->seed;
    info->row_permute = w->row_permute;
    info->initialized = w->initialized;
    info->device_synced = w->device_synced;
    info->F = w->F;
    info->R = w->R;
    info->S = w->S;
    info->C = w->C;
    return SHFLBW_OK;
}

int shflbw_weight_host_arrays(const shflbw_weight* w, const int** indptr, const int** indices,
                              const uint16_t** values, const int** row_permute_ids)
{
    if (!w) return SHFLBW_ERR_INVALID;
    if (!w->initialized) {
        set_error("host_arrays: weight not initialised");
        return SHFLBW_ERR_STATE;
    }
    if (indptr) *indptr = w->indptr.data();
    if (indices) *indices = w->indices.data();
    if (values) *values = w->values.data();
    if (row_permute_ids) *row_permute_ids = w->row_permute ? w->row_permute_ids.data() : nullptr;
    return SHFLBW_OK;
}

const char* shflbw_weight_config_str(const shflbw_weight* w) { return w ? w->config_str.c_str() : ""; }

int shflbw_weight_sync_device(shflbw_weight* w)
{
    if (!w) return SHFLBW_ERR_INVALID;
    if (!w->initialized) { // assert at blockwise_format.h:203
        set_error("sync_device: weight not initialised");
        return SHFLBW_ERR_STATE;
    }
    if (w->device_synced) {
        clear_device(w);
        w->device_synced = false;
    }
    build_meta(w);
    int rc = build_packed_image(w);
    if (rc) return rc;
    rc = upload(w);
    if (rc) return rc;
    w->device_synced = true;
    return SHFLBW_OK;
}

int shflbw_weight_meta_host(const shflbw_weight* w, const int** meta, size_t* n_ints)
{
    if (!w || !meta || !n_ints) return SHFLBW_ERR_INVALID;
    if (w->meta_h.empty()) {
        set_error("meta_host: weight not synced");
        return SHFLBW_ERR_STATE;
    }
    *meta = w->meta_h.data();
    *n_ints = w->meta_h.size();
    return SHFLBW_OK;
}

int shflbw_weight_device_ref(const shflbw_weight* w, shflbw_device_ref* ref)
{
    if (!w || !ref) return SHFLBW_ERR_INVALID;
    if (!w->device_synced) {
        set_error("device_ref: weight not synced");
        return SHFLBW_ERR_STATE;
    }
    auto up8 = [](size_t n) { return (n + 7) / 8 * 8; };
    const int* meta = (const int*)w->d_meta;
    ref->meta = w->d_meta;
    ref->data = w->d_values;
    ref->csb_indptr = meta; // blockwise_format.h:245-262
    ref->csb_indices = meta + up8(w->indptr.size());
    ref->row_permute_ids =
        w->row_permute ? meta + up8(w->indptr.size()) + up8(w->indices.size()) : nullptr;
    ref->csb_values = w->d_values;
    return SHFLBW_OK;
}

} // extern "C"
