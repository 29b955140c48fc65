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


// =======================================================================================
// im2col form of the convolution: three launches on the caller's stream
//   1. im2col_nhwc_kernel:   NHWC input -> im2col matrix Bm[k][p], k = (r,s,c), p = output pixel,
//                            rows of NP fp16 (NP = pixel count rounded up to 64), zero outside the image
//   2. the SpMM kernel:      Dm[f][p] = A_sparse * Bm (row permutation applied to f)
//   3. transpose_to_nhwc_kernel: Dm[f][p] -> OFMap[p][f]
// The gather that the sparse filter needs is a gather of whole rows of a [k][pixel] matrix; NHWC
// keeps channels, not pixels, contiguous, and a row-permuted filter scatters its output channels,
// so both ends are turned into plain 64 x 64 tile transposes and the middle is the tuned SpMM.
// =======================================================================================
constexpr int TT = 64; // transpose tile edge

// 256 threads move a 64 x 64 fp16 tile: `load(i, j)` returns the 16-byte piece j (8 halves) of source
// row i; `store(o, q, v)` receives the 8 halves at source rows 8q .. 8q+7 of source column o.
// Piece j of row i sits at piece position j ^ (i / 8) of its LDS row, so the eight row groups a
// wave reads in one instruction fall into eight different bank groups.
template <typename Load, typename Store>
__device__ __forceinline__ void transpose_tile_64(half_t (*tile)[TT], Load load, Store store)
{
    const int t = threadIdx.x;
#pragma unroll
    for (int pass = 0; pass < 2; pass++) {
        const int i = (t >> 3) + pass * 32, j = t & 7;
        *(half8_t*)&tile[i][(j ^ ((i >> 3) & 7)) * 8] = load(i, j);
    }
    __syncthreads();
#pragma unroll
    for (int pass = 0; pass < 2; pass++) {
        const int o = (t >> 3) + pass * 32, q = t & 7;
        const int c = (((o >> 3) ^ q) << 3) | (o & 7);
        half8_t v;
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = tile[q * 8 + e][c];
        store(o, q, v);
    }
}

// grid: (pixel tiles, channel tiles, filter rows r); block 256.  A workgroup walks the S taps of its
// filter row: the pixel decode is done once, and the loads of the next tap are in flight while the
// current one goes through LDS.
__global__ void __launch_bounds__(256) im2col_nhwc_kernel(const half_t* __restrict__ in, half_t* __restrict__ bm, int B,
                                                          int H, int W, int C, int S, int stride, int pad_h, int pad_w,
                                                          int Ho, int Wo, int NP)
{
    __shared__ __attribute__((aligned(16))) half_t tile[TT][TT];
    const int t = threadIdx.x;
    const int p0 = blockIdx.x * TT, c0 = blockIdx.y * TT, r = blockIdx.z;
    const int npix = B * Ho * Wo;
    // the two source pieces of this thread: pixels p0 + i, channels c0 + 8j ..
    const int j = t & 7, c = c0 + j * 8;
    long base[2]; // element offset of (b, hi, wi = wo*stride - pad_w, c)
    bool row_ok[2]; // the input row hi exists
    int wi0[2];
#pragma unroll
    for (int pass = 0; pass < 2; pass++) {
        const int p = p0 + (t >> 3) + pass * 32;
        const int wo = p % Wo, ho = (p / Wo) % Ho, b = p / (Wo * Ho);
        const int hi = ho * stride - pad_h + r;
        wi0[pass] = wo * stride - pad_w;
        row_ok[pass] = p < npix && c < C && hi >= 0 && hi < H;
        base[pass] = ((long)(b * H + hi) * W + wi0[pass]) * C + c;
    }
    auto fetch = [&](int s, int pass) {
        half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
        const int wi = wi0[pass] + s;
        if (row_ok[pass] && wi >= 0 && wi < W) v = *(const half8_t*)(in + base[pass] + (long)s * C);
        return v;
    };
    half8_t nxt[2] = {fetch(0, 0), fetch(0, 1)};
    for (int s = 0; s < S; s++) {
#pragma unroll
        for (int pass = 0; pass < 2; pass++) {
            const int i = (t >> 3) + pass * 32;
            *(half8_t*)&tile[i][(j ^ ((i >> 3) & 7)) * 8] = nxt[pass];
        }
        __syncthreads();
        if (s + 1 < S) {
            nxt[0] = fetch(s + 1, 0);
            nxt[1] = fetch(s + 1, 1);
        }
        const int tap = r * S + s;
#pragma unroll
        for (int pass = 0; pass < 2; pass++) {
            const int o = (t >> 3) + pass * 32, q = t & 7;
            const int col = (((o >> 3) ^ q) << 3) | (o & 7);
            half8_t v;
#pragma unroll
            for (int e = 0; e < 8; e++) v[e] = tile[q * 8 + e][col];
            if (c0 + o < C) *(half8_t*)(bm + ((size_t)tap * C + c0 + o) * NP + p0 + q * 8) = v;
        }
        __syncthreads();
    }
}

// grid: (pixel tiles, filter tiles); block 256
__global__ void __launch_bounds__(256) transpose_to_nhwc_kernel(const half_t* __restrict__ dm, half_t* __restrict__ out,
                                                                int F, int npix, int NP)
{
    __shared__ __attribute__((aligned(16))) half_t tile[TT][TT];
    const int p0 = blockIdx.x * TT, f0 = blockIdx.y * TT;
    transpose_tile_64(
        tile,
        [&](int i, int j) { // source row = filter f0 + i, piece = pixels p0 + 8j ..
            half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
            if (f0 + i < F) v = *(const half8_t*)(dm + (size_t)(f0 + i) * NP + p0 + j * 8);
            return v;
        },
        [&](int o, int q, half8_t v) { // destination row = pixel p0 + o, filters f0 + 8q ..
            const int pix = p0 + o, f = f0 + q * 8;
            if (pix < npix && f < F) *(half8_t*)(out + (size_t)pix * F + f) = v;
        });
}

// =======================================================================================
// Plane form of the convolution (the default): three launches on the caller's stream
//   1. nhwc_to_planes_kernel: NHWC input -> channel-major, zero-padded planes.  With stride s the
//      padded image is split into its s x s phases; phase (a, b) holds the padded positions
//      (s i + a, s j + b) as a grid of PH x PW values (PW a multiple of 8), images back to back:
//      position n' = img * PH * PW + i * PW + j.  One such row of `pitch` values per channel and
//      phase.  A second copy of everything, moved by one value (copy[x] = base[x + 1]), serves the
//      taps whose offset is odd, so that the gather below stays at least 4-byte aligned.
//   2. the SpMM kernel over the positions n' as columns: the output pixel (ho, wo) of an image is
//      the position (i, j) = (ho, wo), and tap (r, t) of channel c reads phase (r % s, t % s) of
//      that channel at the constant offset (r / s) * PW + t / s.  The kept-column id of a vector is
//      replaced by that element offset and the "row pitch" of B by one element: the im2col
//      address generation is the offset of the gather, no im2col matrix exists.  Positions that
//      are no output pixel (i >= Ho or j >= Wo) compute values nobody reads.
//   3. planes_to_nhwc_kernel: Dm[f][n'] -> OFMap[pixel][f] for the positions that are pixels.
// =======================================================================================
struct PlaneGeom {
    int B, H, W, C, stride, pad_h, pad_w;
    int PH, PW;   // rows and (padded) columns of a phase plane
    int pitch;    // values per channel row of the plane tensor
    int copies;   // 1, or 2 with the copy moved by one value
    int nwanted;  // (copy, phase) planes some tap reads; the others are never written
    unsigned char wanted[32]; // copy * stride * stride + phase of each
};

// grid: (position tiles, channel tiles, wanted planes); block 256
__global__ void __launch_bounds__(256) nhwc_to_planes_kernel(const half_t* __restrict__ in, half_t* __restrict__ planes,
                                                             PlaneGeom g)
{
    __shared__ __attribute__((aligned(16))) half_t tile[TT][TT];
    const int p0 = blockIdx.x * TT, c0 = blockIdx.y * TT;
    const int nphase = g.stride * g.stride;
    const int copy = g.wanted[blockIdx.z] / nphase, phase = g.wanted[blockIdx.z] % nphase;
    const int pa = phase / g.stride, pb = phase % g.stride;
    const int PS = g.PH * g.PW;
    half_t* dst = planes + ((size_t)(copy * nphase + phase) * g.C) * g.pitch;
    transpose_tile_64(
        tile,
        [&](int i, int j) { // source row = position p0 + i (+ copy), piece = channels c0 + 8j ..
            half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
            const int n = p0 + i + copy;
            const int img = n / PS, rem = n % PS;
            const int hi = (rem / g.PW) * g.stride + pa - g.pad_h, wi = (rem % g.PW) * g.stride + pb - g.pad_w;
            const int c = c0 + j * 8;
            if (img < g.B && hi >= 0 && hi < g.H && wi >= 0 && wi < g.W && c < g.C)
                v = *(const half8_t*)(in + ((size_t)(img * g.H + hi) * g.W + wi) * g.C + c);
            return v;
        },
        [&](int o, int q, half8_t v) { // destination row = channel c0 + o, positions p0 + 8q ..
            if (c0 + o < g.C) *(half8_t*)(dst + (size_t)(c0 + o) * g.pitch + p0 + q * 8) = v;
        });
}

// grid: (position tiles, filter tiles); block 256.  dm has rows of NP values.
__global__ void __launch_bounds__(256) planes_to_nhwc_kernel(const half_t* __restrict__ dm, half_t* __restrict__ out, int F,
                                                             int NP, int B, int PH, int PW, int Ho, int Wo)
{
    __shared__ __attribute__((aligned(16))) half_t tile[TT][TT];
    const int p0 = blockIdx.x * TT, f0 = blockIdx.y * TT;
    const int PS = PH * PW;
    transpose_tile_64(
        tile,
        [&](int i, int j) { // source row = filter f0 + i, piece = positions p0 + 8j ..
            half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
            if (f0 + i < F && p0 + j * 8 < NP) v = *(const half8_t*)(dm + (size_t)(f0 + i) * NP + p0 + j * 8);
            return v;
        },
        [&](int o, int q, half8_t v) { // destination row = the pixel at position p0 + o, filters f0 + 8q ..
            const int n = p0 + o, f = f0 + q * 8;
            const int img = n / PS, rem = n % PS, ho = rem / PW, wo = rem % PW;
            if (img < B && ho < Ho && wo < Wo && f < F) *(half8_t*)(out + ((size_t)(img * Ho + ho) * Wo + wo) * F + f) = v;
        });
}

// Kept-column ids of the packed image (k = (r*S + t)*C + c per slot) -> element offsets into the plane
// tensor, in slot order and in the producer-major order of every 64-slot group; the device-side twin of
// the rewrite shflbw_spconv_init does on the host.
__global__ void __launch_bounds__(256) plane_ids_kernel(const int* __restrict__ kidx, int* __restrict__ ids,
                                                        int* __restrict__ ids_pm, int slots, int C, int S, int stride,
                                                        int PW, int pitch, int copies)
{
    const int q = blockIdx.x * 256 + threadIdx.x;
    if (q >= slots) return;
    const int k = kidx[q];
    const int c = k % C, tap = k / C, r = tap / S, t = tap % S;
    const int shift = (r / stride) * PW + t / stride;
    const int copy = copies == 2 ? (shift & 1) : 0;
    const int phase = (r % stride) * stride + t % stride;
    const int id = ((copy * stride * stride + phase) * C + c) * pitch + shift - copy;
    ids[q] = id;
    const int grp = q / 64, j = (q % 64) / 16, p = (q % 16) / 4, rr = q % 4;
    ids_pm[grp * 64 + 16 * p + 4 * j + rr] = id;
}

hipError_t launch_plane_ids(const int* kidx, int* ids, int* ids_pm, int slots, int C, int S, int stride, int PW,
                            int pitch, int copies, hipStream_t stream)
{
    if (slots <= 0) return hipSuccess;
    hipLaunchKernelGGL(plane_ids_kernel, dim3((slots + 255) / 256), dim3(256), 0, stream, kidx, ids, ids_pm, slots, C, S,
                       stride, PW, pitch, copies);
    return hipGetLastError();
}

hipError_t launch_nhwc_to_planes(const SpconvLaunchArgs& a, half_t* planes, int PH, int PW, int pitch, int copies,
                                 hipStream_t stream)
{
    PlaneGeom g{a.B, a.H, a.W, a.C, a.stride, a.pad_h, a.pad_w, PH, PW, pitch, copies, 0, {}};
    // the planes the taps read: tap (r, t) -> phase (r % s, t % s), copy = parity of its offset when there are two
    const int s = a.stride, nphase = s * s;
    if (copies * nphase > (int)sizeof(g.wanted)) return hipErrorInvalidValue;
    bool want[32] = {};
    for (int r = 0; r < a.R; r++)
        for (int t = 0; t < a.S; t++) {
            const int shift = (r / s) * PW + t / s;
            want[(copies == 2 ? (shift & 1) : 0) * nphase + (r % s) * s + t % s] = true;
        }
    for (int i = 0; i < copies * nphase; i++)
        if (want[i]) g.wanted[g.nwanted++] = (unsigned char)i;
    const int np = a.B * PH * PW;
    const dim3 grid((np + TT - 1) / TT, (a.C + TT - 1) / TT, g.nwanted);
    hipLaunchKernelGGL(nhwc_to_planes_kernel, grid, dim3(256), 0, stream, a.in, planes, g);
    return hipGetLastError();
}

hipError_t launch_planes_to_nhwc(const half_t* dm, half_t* out, int F, int NP, int B, int PH, int PW, int Ho, int Wo,
                                 hipStream_t stream)
{
    const dim3 grid((NP + TT - 1) / TT, (F + TT - 1) / TT);
    hipLaunchKernelGGL(planes_to_nhwc_kernel, grid, dim3(256), 0, stream, dm, out, F, NP, B, PH, PW, Ho, Wo);
    return hipGetLastError();
}

hipError_t launch_im2col_nhwc(const SpconvLaunchArgs& a, half_t* bm, int NP, hipStream_t stream)
{
    const dim3 grid(NP / TT, (a.C + TT - 1) / TT, a.R);
    hipLaunchKernelGGL(im2col_nhwc_kernel, grid, dim3(256), 0, stream, a.in, bm, a.B, a.H, a.W, a.C, a.S, a.stride,
                       a.pad_h, a.pad_w, a.Ho, a.Wo, NP);
    return hipGetLastError();
}

hipError_t launch_transpose_to_nhwc(const half_t* dm, half_t* out, int F, int npix, int NP, hipStream_t stream)
{
    const dim3 grid(NP / TT, (F + TT - 1) / TT);
    hipLaunchKernelGGL(transpose_to_nhwc_kernel, grid, dim3(256), 0, stream, dm, out, F, npix, NP);
    return hipGetLastError();
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
