// CPU reference results of the two operators, computed from a weight's host arrays: what the
// reference library ships as get_host_reference for its users' own checks
// (block_sparse/spmm/blockwise_format.h:268-311 and block_sparse/spconv/blockwise_format.h:55-132).
// Every output element is the fp32 sum of its products in ascending order of the kept vectors of
// its panel, the order those functions use, so results do not depend on how the loops are nested
// here.  Host code only; nothing on the GPU path calls it.
#include <cstring>
#include <vector>

#include "weight_internal.h"

using namespace shflbw;

namespace {

// y[0..n) += a * x[0..n)
inline void axpy(float a, const float* x, float* y, int n)
{
    for (int i = 0; i < n; i++) y[i] += a * x[i];
}

std::vector<float> widen(const uint16_t* h, size_t n)
{
    std::vector<float> f(n);
    for (size_t i = 0; i < n; i++) f[i] = half_to_float(h[i]);
    return f;
}

int usable(const shflbw_weight* w, const char* who)
{
    if (!w || !w->initialized) {
        set_error("%s: weight not initialised", who);
        return SHFLBW_ERR_STATE;
    }
    if (w->bcol != 1) {
        set_error("%s: bcol must be 1 (got %d)", who, w->bcol);
        return SHFLBW_ERR_UNSUPPORTED;
    }
    return SHFLBW_OK;
}

} // namespace

extern "C" {

int shflbw_spmm_host_reference(const shflbw_weight* w, int N, const uint16_t* B, float alpha, const uint16_t* C,
                               float beta, float* D_ref)
{
    int rc = usable(w, "spmm_host_reference");
    if (rc) return rc;
    if (N <= 0 || !B || !D_ref || (beta != 0.f && !C)) {
        set_error("spmm_host_reference: null operand or non-positive N");
        return SHFLBW_ERR_INVALID;
    }
    const int V = w->brow, X = w->nrow / V;
    const std::vector<float> Bf = widen(B, (size_t)w->ncol * N);
    memset(D_ref, 0, sizeof(float) * (size_t)w->nrow * N);
    for (int panel = 0; panel < X; panel++)
        for (int r = 0; r < V; r++) {
            const int stored = panel * V + r;
            float* out = D_ref + (size_t)(w->row_permute ? w->row_permute_ids[stored] : stored) * N;
            for (int p = w->indptr[panel]; p < w->indptr[panel + 1]; p++)
                axpy(half_to_float(w->values[(size_t)p * V + r]), Bf.data() + (size_t)w->indices[p] * N, out, N);
        }
    for (size_t i = 0; i < (size_t)w->nrow * N; i++)
        D_ref[i] = D_ref[i] * alpha + (C ? half_to_float(C[i]) : 0.f) * beta;
    return SHFLBW_OK;
}

int shflbw_spconv_host_reference(const shflbw_weight* f, int B, int H, int W, int stride, const uint16_t* IFMap,
                                 float* OFMap_ref)
{
    int rc = usable(f, "spconv_host_reference");
    if (rc) return rc;
    if (f->R <= 0) {
        set_error("spconv_host_reference: weight has no filter view");
        return SHFLBW_ERR_STATE;
    }
    if (B <= 0 || H <= 0 || W <= 0 || stride <= 0 || !IFMap || !OFMap_ref) {
        set_error("spconv_host_reference: null tensor or non-positive extent");
        return SHFLBW_ERR_INVALID;
    }
    const int V = f->brow, X = f->F / V, Cc = f->C, R = f->R, S = f->S, F = f->F;
    const int ph = R / 2, pw = S / 2;
    const int Ho = (H + 2 * ph - R) / stride + 1, Wo = (W + 2 * pw - S) / stride + 1;
    if (Ho <= 0 || Wo <= 0) {
        set_error("spconv_host_reference: empty output");
        return SHFLBW_ERR_SHAPE;
    }
    const std::vector<float> in = widen(IFMap, (size_t)B * H * W * Cc);
    memset(OFMap_ref, 0, sizeof(float) * (size_t)B * Ho * Wo * F);
    std::vector<float> wcol(V);
    std::vector<int> orow(V);
    for (int panel = 0; panel < X; panel++) {
        for (int r = 0; r < V; r++) orow[r] = f->row_permute ? f->row_permute_ids[panel * V + r] : panel * V + r;
        for (int p = f->indptr[panel]; p < f->indptr[panel + 1]; p++) {
            const int k = f->indices[p], c = k % Cc, tap = k / Cc, t = tap % S, rr = tap / S; // k = (r*S + s)*C + c
            for (int r = 0; r < V; r++) wcol[r] = half_to_float(f->values[(size_t)p * V + r]);
            for (int b = 0; b < B; b++)
                for (int ho = 0; ho < Ho; ho++) {
                    const int hi = ho * stride - ph + rr;
                    if (hi < 0 || hi >= H) continue; // a tap outside the image adds zero
                    for (int wo = 0; wo < Wo; wo++) {
                        const int wi = wo * stride - pw + t;
                        if (wi < 0 || wi >= W) continue;
                        const float x = in[((size_t)(b * H + hi) * W + wi) * Cc + c];
                        float* out = OFMap_ref + ((size_t)(b * Ho + ho) * Wo + wo) * F;
                        for (int r = 0; r < V; r++) out[orow[r]] += wcol[r] * x;
                    }
                }
        }
    }
    return SHFLBW_OK;
}

int shflbw_spconv_host_reference_chwb(const shflbw_weight* f, int B, int H, int W, int stride, const uint16_t* IFMap,
                                      float* OFMap_ref)
{
    int rc = usable(f, "spconv_host_reference_chwb");
    if (rc) return rc;
    if (f->R <= 0) {
        set_error("spconv_host_reference_chwb: weight has no filter view");
        return SHFLBW_ERR_STATE;
    }
    if (B <= 0 || H <= 0 || W <= 0 || stride <= 0 || !IFMap || !OFMap_ref) {
        set_error("spconv_host_reference_chwb: null tensor or non-positive extent");
        return SHFLBW_ERR_INVALID;
    }
    // tensors C-H-W-B and F-H-W-B; H, W bound input and output alike (spconv/blockwise_format.h:111-128)
    const int V = f->brow, X = f->F / V, Cc = f->C, R = f->R, S = f->S;
    const size_t plane = (size_t)H * W * B;
    const std::vector<float> in = widen(IFMap, plane * Cc);
    memset(OFMap_ref, 0, sizeof(float) * plane * f->F);
    for (int panel = 0; panel < X; panel++)
        for (int p = f->indptr[panel]; p < f->indptr[panel + 1]; p++) {
            const int k = f->indices[p], c = k % Cc, tap = k / Cc, t = tap % S, rr = tap / S;
            for (int r = 0; r < V; r++) {
                const int stored = panel * V + r;
                const float wv = half_to_float(f->values[(size_t)p * V + r]);
                float* out = OFMap_ref + (size_t)(f->row_permute ? f->row_permute_ids[stored] : stored) * plane;
                for (int ho = 0; ho < H; ho++) {
                    const int hi = ho * stride - R / 2 + rr;
                    if (hi < 0 || hi >= H) continue;
                    for (int wo = 0; wo < W; wo++) {
                        const int wi = wo * stride - S / 2 + t;
                        if (wi < 0 || wi >= W) continue;
                        axpy(wv, in.data() + ((size_t)(c * H + hi) * W + wi) * B, out + ((size_t)ho * W + wo) * B, B);
                    }
                }
            }
        }
    return SHFLBW_OK;
}

} // extern "C"
