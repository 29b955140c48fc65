// Shfl-BW sparse Conv2D for gfx950 as an implicit GEMM over NHWC tensors:
//   OFMap[b][ho][wo][perm[f]] = sum over kept k=(r,s,c) of W_stored[f][k] * IFMap[b][ho*stride-pad+r][wo*stride-pad+s][c]
// GEMM view: M = F (sparse, permuted rows), K = R*S*C ordered (r,s,c), N = B*Ho*Wo pixels.
//
// Replaces the reference's block_sparse/spconv/blockwise_kernel.h:66-261 (main loop) and
// block_sparse/spconv/conv_format.h:14-82 (col2im address generation).  The im2col addresses
// are generated while the activation tile is loaded: a thread owns 8 neighbouring output
// pixels, keeps their input origin in registers, and for each kept k of the stage adds the
// tap offset, fetches the 8 activations (zero outside the image) and stores them as one
// 16-byte piece into the same swizzled [k][pixel] LDS layout the SpMM kernel uses, so the
// matrix-core part (transposing LDS loads, 32x32x16 fp16 MFMA, fp32 accumulate) is shared.
#include "kernel_common.h"
#include "spconv_launch.h"

namespace shflbw {

template <int V, int WN, int NWAVES, int KT>
struct SpconvCfg {
    static constexpr int BN = WN * NWAVES;
    static constexpr int MB = V / 32;
    static constexpr int NB = WN / 32;
    static constexpr int ROWB = BN * 2;
    static constexpr int CPR = BN / 8;
    static constexpr int SPT = KT / 16;
    static constexpr int THREADS = NWAVES * 64;
    static constexpr int PIECES = KT * CPR;          // 16-byte pieces per stage
    static constexpr int PPT = PIECES / THREADS;     // pieces per thread
    static constexpr int ROWS_PER_PASS = THREADS / CPR;
    static constexpr int LDS_BYTES = KT * ROWB;
    static_assert(V % 32 == 0 && WN % 32 == 0, "32x32x16 tiles");
    static_assert(BN >= 128 && BN <= 512 && (BN & (BN - 1)) == 0, "row swizzle range");
    static_assert(PIECES % THREADS == 0 && THREADS % CPR == 0 && ROWS_PER_PASS % 4 == 0,
                  "a thread keeps one column piece and a fixed row phase across passes");
};

template <int V, int WN, int NWAVES, int KT>
__global__ void __launch_bounds__(NWAVES * 64) spconv_shflbw_kernel(SpconvLaunchArgs a)
{
    using Cfg = SpconvCfg<V, WN, NWAVES, KT>;
    constexpr int BN = Cfg::BN, MB = Cfg::MB, NB = Cfg::NB, ROWB = Cfg::ROWB, CPR = Cfg::CPR, SPT = Cfg::SPT;
    constexpr int PPT = Cfg::PPT, RPP = Cfg::ROWS_PER_PASS;

    extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(SHFLBW_LDS char*)lds_raw;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lid = xcd_local_id(blockIdx.x, a.X * a.n_tiles);
    const int nt = lid / a.X;
    const int panel = lid - nt * a.X;
    const int n0 = nt * BN;
    const int npix = a.B * a.Ho * a.Wo;

    const int2_t pd = ((const SHFLBW_CONST int2_t*)(uintptr_t)a.panel_desc)[panel];
    const int g0 = pd.y;
    const int* __restrict__ kidx = a.kidx + (size_t)g0 * 64;
    const half8_t* __restrict__ pA = a.packedA + (size_t)g0 * (64 * V / 8);
    const int nsteps = pd.x;
    const int ntiles = (nsteps + SPT - 1) / SPT;

    // ---- the 8 output pixels this thread loads activations for (same for every pass)
    const int row0 = tid / CPR;      // row of the first pass; later passes add RPP (a multiple of 4)
    const int pc = tid % CPR;        // physical 16-byte piece inside the LDS row
    const int lc = ((((pc >> 1) ^ row_xor32(row0 & 3))) << 1) | (pc & 1); // logical piece = 8 pixels
    int pix_base[8]; // element offset of input pixel (b, ho*stride - pad_h, wo*stride - pad_w), channel 0
    int pix_hw[8];   // (hi0 + 0x4000) << 16 | (wi0 + 0x4000); a pixel past the end gets an always-invalid origin
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const int p = n0 + lc * 8 + e;
        if (p < npix) {
            const int wo = p % a.Wo, ho = (p / a.Wo) % a.Ho, b = p / (a.Wo * a.Ho);
            const int hi0 = ho * a.stride - a.pad_h, wi0 = wo * a.stride - a.pad_w;
            pix_base[e] = ((b * a.H + hi0) * a.W + wi0) * a.C;
            pix_hw[e] = ((hi0 + 0x4000) << 16) | (wi0 + 0x4000);
        } else {
            pix_base[e] = 0;
            pix_hw[e] = 0; // hi0 = wi0 = -16384: every tap is out of bounds -> zeros
        }
    }
    const uint32_t wr_off = (uint32_t)(row0 * ROWB + pc * 16);

    const int li = lane & 15;
    uint32_t boff[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const int unit = (wave * WN + nb * 32) / 16 + ((lane >> 4) & 1);
        boff[nb] = (uint32_t)((8 * (lane >> 5) + (li >> 2)) * ROWB + ((unit ^ row_xor32(li >> 2)) << 5) + ((li & 3) << 3));
    }

    float16_t acc[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[mb][nb][i] = 0.f;

    const int SC = a.S * a.C;
    for (int t = 0; t < ntiles; t++) {
        // ---- im2col gather of KT rows x BN pixels into LDS
        half8_t piece[PPT];
#pragma unroll
        for (int j = 0; j < PPT; j++) {
            const int k = kidx[t * Cfg::SPT * 16 + row0 + j * RPP];
            const int r = k / SC, rem = k - r * SC, s = rem / a.C, c = rem - s * a.C;
            const int tap = (r * a.W + s) * a.C + c;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int hi = (pix_hw[e] >> 16) - 0x4000 + r, wi = (pix_hw[e] & 0xffff) - 0x4000 + s;
                const bool ok = hi >= 0 && hi < a.H && wi >= 0 && wi < a.W;
                piece[j][e] = ok ? a.in[pix_base[e] + tap] : (half_t)0.f;
            }
        }
        __syncthreads(); // previous stage fully consumed
#pragma unroll
        for (int j = 0; j < PPT; j++)
            *(SHFLBW_LDS half8_t*)(uintptr_t)(lds0 + wr_off + j * RPP * ROWB) = piece[j];
        __syncthreads();

#pragma unroll
        for (int kk = 0; kk < SPT; kk++) {
            const int step = t * SPT + kk;
            if (step < nsteps) {
                half8_t afrag[MB], bfrag[NB];
#pragma unroll
                for (int mb = 0; mb < MB; mb++) afrag[mb] = pA[((size_t)step * MB + mb) * 64 + lane];
#pragma unroll
                for (int nb = 0; nb < NB; nb++) {
                    const half4_t lo = lds_read_tr16(lds0 + boff[nb] + (kk * 16) * ROWB);
                    const half4_t hi = lds_read_tr16(lds0 + boff[nb] + (kk * 16 + 4) * ROWB);
                    bfrag[nb] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                }
#pragma unroll
                for (int mb = 0; mb < MB; mb++)
#pragma unroll
                    for (int nb = 0; nb < NB; nb++)
                        acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bfrag[nb], afrag[mb], acc[mb][nb], 0, 0, 0);
            }
        }
    }

    // ---- epilogue: one fp32 -> fp16 rounding, NHWC store; a lane holds output channel
    // perm[panel*V + mb*32 + lane%32] of 16 pixels per 32x32 block
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        const int srow = panel * V + mb * 32 + (lane & 31);
        const int f = a.row_ids ? a.row_ids[srow] : srow;
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int p = n0 + wave * WN + nb * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3);
                if (p < npix) a.out[(size_t)p * a.F + f] = (half_t)acc[mb][nb][i];
            }
    }
}

template <int V, int WN, int NWAVES, int KT>
static hipError_t launch_conv(const SpconvLaunchArgs& a, hipStream_t stream)
{
    using Cfg = SpconvCfg<V, WN, NWAVES, KT>;
    const int npix = a.B * a.Ho * a.Wo;
    SpconvLaunchArgs b = a;
    b.n_tiles = (npix + Cfg::BN - 1) / Cfg::BN;
    hipLaunchKernelGGL((spconv_shflbw_kernel<V, WN, NWAVES, KT>), dim3(a.X * b.n_tiles), dim3(Cfg::THREADS),
                       Cfg::LDS_BYTES, stream, b);
    return hipGetLastError();
}

template <int V, int WN, int NWAVES, int KT>
static hipError_t prepare_conv()
{
    using Cfg = SpconvCfg<V, WN, NWAVES, KT>;
    return hipFuncSetAttribute((const void*)spconv_shflbw_kernel<V, WN, NWAVES, KT>,
                               hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES);
}

#define SHFLBW_CONV_VARIANT(V, WN, NW, KT)                                                          \
    {                                                                                               \
        V, WN* NW, NW * 64, SpconvCfg<V, WN, NW, KT>::LDS_BYTES, #V "x" #WN "x" #NW "w_k" #KT,      \
            &launch_conv<V, WN, NW, KT>, &prepare_conv<V, WN, NW, KT>                               \
    }

static const SpconvVariant g_conv_variants[] = {
    SHFLBW_CONV_VARIANT(64, 32, 4, 32),
    SHFLBW_CONV_VARIANT(32, 32, 4, 32),
    SHFLBW_CONV_VARIANT(128, 32, 4, 32),
};

const SpconvVariant* spconv_variants(int* count)
{
    *count = (int)(sizeof(g_conv_variants) / sizeof(g_conv_variants[0]));
    return g_conv_variants;
}

} // namespace shflbw
