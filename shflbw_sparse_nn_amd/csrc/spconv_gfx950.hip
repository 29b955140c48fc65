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
#include "spmm_ws.h"

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
                const bool ok = k >= 0 && hi >= 0 && hi < a.H && wi >= 0 && wi < a.W; // k < 0: padding slot
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
            const int img = g.batch_inner ? n % g.B : n / PS, rem = g.batch_inner ? n / g.B : n % PS;
            const int hi = (rem / g.PW) * g.stride + pa - g.pad_h, wi = (rem % g.PW) * g.stride + pb - g.pad_w;
            const int c = c0 + j * 8;
            if (img < g.B && rem < PS && hi >= 0 && hi < g.H && wi >= 0 && wi < g.W && c < g.C)
                v = *(const half8_t*)(in + ((size_t)(img * g.H + hi) * g.W + wi) * g.C + c);
            return v;
        },
        [&](int o, int q, half8_t v) { // destination row = channel c0 + o, positions p0 + 8q ..
            if (c0 + o < g.C) *(half8_t*)(dst + (size_t)(c0 + o) * g.pitch + p0 + q * 8) = v;
        });
}

// grid: (position tiles, filter tiles); block 256.  dm has rows of NP values.
__global__ void __launch_bounds__(256) planes_to_nhwc_kernel(const half_t* __restrict__ dm, half_t* __restrict__ out, int F,
                                                             int NP, int B, int PH, int PW, int Ho, int Wo, int batch_inner)
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
            const int img = batch_inner ? n % B : n / PS, rem = batch_inner ? n / B : n % PS, ho = rem / PW, wo = rem % PW;
            // streaming store: the output is not read again here and should not push the next launch's input out of the caches
            if (img < B && ho < Ho && wo < Wo && f < F)
                __builtin_nontemporal_store(v, (half8_t*)(out + ((size_t)(img * Ho + ho) * Wo + wo) * F + f));
        });
}

// the (copy, phase) planes some tap reads: tap (r, t) -> phase (r % s, t % s), copy = parity of its offset when
// there are two copies
bool fill_wanted_planes(PlaneGeom& g, int R, int S)
{
    const int s = g.stride, nphase = s * s;
    if (g.copies * nphase > (int)sizeof(g.wanted)) return false;
    bool want[32] = {};
    for (int r = 0; r < R; r++)
        for (int t = 0; t < S; t++) {
            const int shift = (r / s) * g.PW + t / s;
            want[(g.copies == 2 ? (shift & 1) : 0) * nphase + (r % s) * s + t % s] = true;
        }
    g.nwanted = 0;
    for (int i = 0; i < g.copies * nphase; i++)
        if (want[i]) g.wanted[g.nwanted++] = (unsigned char)i;
    return true;
}

// =======================================================================================
// Fused form of the convolution: ONE persistent launch.
//   phase 0  every workgroup takes chunks of the NHWC -> planes rewrite from a queue (64 x 64 tile transposes,
//            eight tiles at a time) until the queue is empty, then waits until all chunks have been written;
//   phase 1  the role-split SpMM over its tiles (gather ids are plane offsets; the columns of the GEMM are the
//            plane positions of output rows only: m = (img * Ho + i) * PW + j), result rows of fp16 in the
//            filter-major scratch fm[f][m]; every consumer wave counts its finished tile in the arrival word of
//            the tile's column tile;
//   phase 2  when all tiles of a column tile have arrived, its fm[F][BN] slab is transposed to NHWC in chunks
//            taken from that column tile's queue.
// No wait depends on a workgroup that is not running: phase 0 waits only for chunks that running workgroups
// have claimed; in phase 2 the workgroup whose arrival completes a column tile finds it complete when it gets
// there and empties its queue (alone, if it must), every other wait is bounded by a time budget and only adds
// helpers.  The words in `sync` are all zero between launches: the last workgroup to leave clears them.
// Data written by one workgroup and read by another (planes, fm) is stored with device scope, followed by a
// wait for the acknowledgement and an arrival count; the reader passes an acquire fence after it has seen
// the count.
// =======================================================================================

// Layout of the synchronisation words, in cache lines of SYNC_LINE ints (conv_sync_lines() of them): line 0 the XCDs
// whose workgroups have all left, line 1 a flag (a wait that cannot time out did), lines 2.. the eight phase-0 queues,
// then per queue the chunks of it that are written, then per XCD the workgroups that have left, then the number of
// phase-0 queues whose chunks are all written, then two lines per column tile: finished tiles, phase-2 queue.
constexpr int LINE_LEFT_ALL = 0, LINE_GAVE_UP = 1, LINE_Q0 = 2, LINE_DONE0 = 10, LINE_LEFT = 18, LINE_ALLDONE0 = 26,
              LINE_SLAB0 = CONV_LINE_SLAB0;

// Diagnostic build (-DSHFLBW_CONV_STAMPS): workgroups 0 and 100 leave 100 MHz timestamps of their phase boundaries
// in the flag line of the synchronisation words (ints 16.. of line 1).
#ifdef SHFLBW_CONV_STAMPS
#define CONV_STAMP(i)                                                                                           \
    do {                                                                                                        \
        if (tid == 0 && (blockIdx.x == 0 || blockIdx.x == 100))                                                 \
            ((unsigned long long*)(c.sync + LINE_GAVE_UP * SYNC_LINE + 16))[(blockIdx.x == 0 ? 0 : 12) + (i)] = wall_clock64(); \
    } while (0)
#else
#define CONV_STAMP(i) do { } while (0)
#endif

__device__ __forceinline__ int sync_load(const int* p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// 512 threads transpose 2 * nk (nk = 1, 2 or 4) 64 x 64 fp16 tiles through LDS at `lds` (8 KiB per tile):
// `load(tile, i, j)` returns the 16-byte piece j (8 halves) of source row i of a tile; `store(tile, o, q, v)` receives
// the halves at source rows 8q .. 8q+7 of source column o.  Threads 0..255 own tiles 0..nk-1, threads 256..511 tiles
// nk..2nk-1; all loads of a thread are in flight before the first one is used.  Piece j of row i sits at piece
// position j ^ (i / 8) of its LDS row, so the eight row groups a wave reads in one instruction fall into eight
// different bank groups.
template <typename Load, typename Store>
__device__ __forceinline__ void transpose_tiles(uint32_t lds, int tid, int nk, Load load, Store store)
{
    const int half = tid >> 8, t = tid & 255;
    half8_t v[4][2];
#pragma unroll
    for (int k = 0; k < 4; k++)
        if (k < nk) {
#pragma unroll
            for (int pass = 0; pass < 2; pass++) v[k][pass] = load(half * nk + k, (t >> 3) + pass * 32, t & 7);
        }
#pragma unroll
    for (int k = 0; k < 4; k++)
        if (k < nk) {
#pragma unroll
            for (int pass = 0; pass < 2; pass++) {
                const int i = (t >> 3) + pass * 32, j = t & 7;
                *(SHFLBW_LDS half8_t*)(uintptr_t)(lds + (half * nk + k) * (TT * TT * 2) + i * (TT * 2) + ((j ^ ((i >> 3) & 7)) << 4)) =
                    v[k][pass];
            }
        }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 4; k++)
        if (k < nk) {
#pragma unroll
            for (int pass = 0; pass < 2; pass++) {
                const int o = (t >> 3) + pass * 32, q = t & 7;
                const int c = (((o >> 3) ^ q) << 3) | (o & 7);
                half8_t r;
#pragma unroll
                for (int e = 0; e < 8; e++)
                    r[e] = *(SHFLBW_LDS half_t*)(uintptr_t)(lds + (half * nk + k) * (TT * TT * 2) + (q * 8 + e) * (TT * 2) + c * 2);
                store(half * nk + k, o, q, r);
            }
        }
    __syncthreads();
}

template <int V, int WN, int NCONS, int NPROD, int KT, int NSTAGE>
__global__ void __launch_bounds__((NCONS + NPROD) * 64) spconv_fused_kernel(SpmmLaunchArgs a, ConvFuseArgs c)
{
    using Cfg = SpmmWsCfg<V, WN, NCONS, NPROD, KT, NSTAGE>;
    static_assert((NCONS + NPROD) * 64 == 512 && Cfg::RING_BYTES >= 8 * TT * TT * 2, "the layout phases use 512 threads and up to 64 KiB");
    extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
    __shared__ int mailbox[2];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(SHFLBW_LDS char*)lds_raw;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int X = a.X;
    if (tid == 0) *(SHFLBW_LDS unsigned*)(uintptr_t)(lds0 + Cfg::LDS_BYTES) = 0u; // consumer waves count finished tiles here
    __syncthreads();
    CONV_STAMP(0);

    // ================= phase 0: NHWC input -> channel-major padded planes =================
    if (c.phases & 1) {
        const PlaneGeom& g = c.g;
        const int nphase = g.stride * g.stride, PS = g.PH * g.PW;
        // The chunk list is cut into eight ranges with a queue each; a workgroup serves the queue of its XCD first and
        // then the others (a queue that a load shows to be exhausted is skipped without an atomic).  A chunk is written
        // once its stores are acknowledged; the workgroup that writes the last chunk of a queue counts the queue.
        const int per_q = (c.n0chunks + 7) >> 3;
        const int xcd = blockIdx.x & 7;
        const int nk = (c.ct * c.pt) >> 1;
        int tried = 0;
        while (true) {
            if (tid == 0) {
                int chunk = -1;
                while (tried < 8) {
                    const int qi = (xcd + tried) & 7;
                    const int lo = qi * per_q, size = min(c.n0chunks, lo + per_q) - lo;
                    int* q = c.sync + (LINE_Q0 + qi) * SYNC_LINE;
                    if (size > 0 && sync_load(q) < size) {
                        const int got = __hip_atomic_fetch_add(q, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        if (got < size) {
                            chunk = lo + got;
                            break;
                        }
                    }
                    tried++;
                }
                mailbox[0] = chunk;
            }
            __syncthreads();
            const int chunk = __builtin_amdgcn_readfirstlane(mailbox[0]);
            if (chunk < 0) break;
            const int plane = chunk / (c.ch_chunks * c.pos_chunks), rem = chunk % (c.ch_chunks * c.pos_chunks);
            const int p_base = (rem / c.ch_chunks) * (c.pt * TT), c_base = (rem % c.ch_chunks) * (c.ct * TT);
            const int copy = g.wanted[plane] / nphase, phase = g.wanted[plane] % nphase;
            const int pa = phase / g.stride, pb = phase % g.stride;
            half_t* dst = c.planes + ((size_t)(copy * nphase + phase) * g.C) * g.pitch;
            transpose_tiles(
                lds0, tid, nk,
                [&](int tile, int i, int j) { // source row = position (+ copy), piece = 8 channels
                    half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
                    const int n = p_base + (tile / c.ct) * TT + i + copy;
                    const int ch = c_base + (tile % c.ct) * TT + j * 8;
                    int img, r2, prow, pcol;
                    fast_divmod(n, PS, c.magic_ps, img, r2);
                    fast_divmod(r2, g.PW, c.magic_pw, prow, pcol);
                    const int hi = prow * g.stride + pa - g.pad_h, wi = pcol * g.stride + pb - g.pad_w;
                    if (img < g.B && hi >= 0 && hi < g.H && wi >= 0 && wi < g.W && ch < g.C)
                        v = *(const half8_t*)(c.in + ((size_t)(img * g.H + hi) * g.W + wi) * g.C + ch);
                    return v;
                },
                [&](int tile, int o, int q, half8_t v) { // destination row = channel, 8 positions
                    const int ch = c_base + (tile % c.ct) * TT + o;
                    const int p = p_base + (tile / c.ct) * TT + q * 8;
                    if (ch < g.C && p < c.np64) store_result_16B(dst + (size_t)ch * g.pitch + p, v);
                });
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (tid == 0) {
                const int qi = min(chunk / per_q, 7), size = min(c.n0chunks, (qi + 1) * per_q) - qi * per_q;
                if (__hip_atomic_fetch_add(c.sync + (LINE_DONE0 + qi) * SYNC_LINE, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == size - 1)
                    __hip_atomic_fetch_add(c.sync + LINE_ALLDONE0 * SYNC_LINE, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        CONV_STAMP(1);
        CONV_STAMP(2);
        // Wait until every queue is written.  The planes were not read by this launch so far, so no cache holds lines of
        // them except the up-to-date ones of their writers (caches start a launch invalidated, and the stores go through
        // to memory): the gathers that follow need no invalidation of their own.
        if (tid == 0) {
            const int queues = (c.n0chunks + per_q - 1) / max(per_q, 1);
            const unsigned long long t0 = wall_clock64();
            while (sync_load(c.sync + LINE_ALLDONE0 * SYNC_LINE) < queues) {
                if (wall_clock64() - t0 > 200000000ull) { // two seconds: cannot happen, chunks are only held by running workgroups
                    __hip_atomic_store(c.sync + LINE_GAVE_UP * SYNC_LINE, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
                __builtin_amdgcn_s_sleep(8);
            }
        }
        __syncthreads();
        CONV_STAMP(3);
        CONV_STAMP(4);
    }

    // ================= phase 1: the SpMM over this workgroup's tiles =================
    const int T = X * a.n_tiles;
    const int per = (T + 7) >> 3;
    const int S = gridDim.x >> 3;
    const int id_first = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
    const int id_end = min(T, ((blockIdx.x & 7) + 1) * per);
    {
        if (wave >= NCONS)
            ws_producer<Cfg, V, NCONS, NPROD, KT, NSTAGE, true>(a, lds0, lane, wave - NCONS, id_first, id_end, S);
        else if constexpr (V == 16)
            ws_consumer16<Cfg, WN, NCONS, true>(a, lds0, lane, wave, id_first, id_end, S);
        else
            ws_consumer<Cfg, V, WN, NCONS, true>(a, lds0, lane, wave, id_first, id_end, S);
    }
    __syncthreads(); // both roles are through: the ring is free
    CONV_STAMP(5);

    // ================= phase 2: fm[F][BN] slabs -> NHWC output =================
    if (c.phases & 2) {
        const int chunks_per_slab = c.f_chunks * ((Cfg::BN / TT + c.mt - 1) / c.mt);
        const int img_cols = c.Ho * c.g.PW;
        const unsigned long long t0 = wall_clock64();
        // One visit to every column tile this workgroup computed a tile of (in its tile order).  A column tile that is
        // complete is emptied; for one that is not, the workgroup waits while it has time left and moves on otherwise:
        // the workgroup whose arrival completes it comes by later and empties it.
        int prev = -1;
        for (int id = id_first; id < id_end; id += S) {
            const int s = id / X;
            if (s == prev) continue;
            prev = s;
            if (tid == 0) {
                int ok = 0;
                while (true) {
                    if (sync_load(c.sync + (LINE_SLAB0 + 2 * s) * SYNC_LINE) >= c.arrivals_per_slab) {
                        ok = 1;
                        break;
                    }
                    if (wall_clock64() - t0 > (unsigned long long)c.help_ticks) break;
                    __builtin_amdgcn_s_sleep(2);
                }
                mailbox[1] = ok;
            }
            __syncthreads();
            const int ok = __builtin_amdgcn_readfirstlane(mailbox[1]);
            __syncthreads();
            if (!ok) continue;
            // the result rows were not read by this launch so far (see the planes above): no invalidation needed
            CONV_STAMP(6);
            CONV_STAMP(7);
            while (true) {
                if (tid == 0)
                    mailbox[0] = __hip_atomic_fetch_add(c.sync + (LINE_SLAB0 + 2 * s + 1) * SYNC_LINE, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __syncthreads();
                const int chunk = __builtin_amdgcn_readfirstlane(mailbox[0]);
                if (chunk >= chunks_per_slab) break;
                const int f_base = (chunk % c.f_chunks) * (c.ft * TT);
                const int m_base = s * Cfg::BN + (chunk / c.f_chunks) * (c.mt * TT);
                const int m_end = min(c.ncols, (s + 1) * Cfg::BN);
                transpose_tiles(
                    lds0, tid, (c.ft * c.mt) >> 1,
                    [&](int tile, int i, int j) { // source row = filter, piece = 8 columns of the GEMM
                        half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
                        const int f = f_base + (tile % c.ft) * TT + i;
                        const int m = m_base + (tile / c.ft) * TT + j * 8;
                        if (f < c.F && m < m_end) v = *(const half8_t*)(c.fm + (size_t)f * c.ncols + m);
                        return v;
                    },
                    [&](int tile, int o, int q, half8_t v) { // destination row = the pixel of column m, 8 filters
                        const int m = m_base + (tile / c.ft) * TT + o;
                        const int f = f_base + (tile % c.ft) * TT + q * 8;
                        int img, r2, ho, wo;
                        fast_divmod(m, img_cols, c.magic_imgcols, img, r2);
                        fast_divmod(r2, c.g.PW, c.magic_pw, ho, wo);
                        if (m < m_end && wo < c.Wo && f < c.F)
                            *(half8_t*)(c.out + ((size_t)(img * c.Ho + ho) * c.Wo + wo) * c.F + f) = v;
                    });
            }
        }
    }

    // ================= leave: the last workgroup clears the words for the next launch =================
    // counted per XCD first (one line each), then the XCDs on one line
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    CONV_STAMP(8);
    if (tid == 0) {
        const int xcd = blockIdx.x & 7, per_xcd = (int)gridDim.x >> 3; // the grid is a multiple of 8
        if (__hip_atomic_fetch_add(c.sync + (LINE_LEFT + xcd) * SYNC_LINE, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == per_xcd - 1 &&
            __hip_atomic_fetch_add(c.sync + LINE_LEFT_ALL * SYNC_LINE, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 7) {
            for (int i = 0; i < LINE_SLAB0 + 2 * c.slabs; i++)
                if (i != LINE_GAVE_UP) __hip_atomic_store(c.sync + i * SYNC_LINE, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// Kept-column ids of the packed image (k = (r*S + t)*C + c per slot) -> element offsets into the plane
// tensor, in slot order and in the producer-major order of every 64-slot group; the device-side twin of
// the rewrite shflbw_spconv_init does on the host.
__global__ void __launch_bounds__(256) plane_ids_kernel(const int* __restrict__ kidx, int* __restrict__ ids,
                                                        int* __restrict__ ids_pm, int slots, int C, int S, int stride,
                                                        int PW, int pitch, int copies, int zero_id, half_t* planes)
{
    const int q = blockIdx.x * 256 + threadIdx.x;
    // the row of zeros behind the last channel row, which the padding slots gather
    for (int i = q * 8; i < pitch; i += gridDim.x * 256 * 8) *(half8_t*)(planes + (size_t)zero_id + i) = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    if (q >= slots) return;
    const int k = kidx[q];
    int id = zero_id; // padding slot
    if (k >= 0) {
        const int c = k % C, tap = k / C, r = tap / S, t = tap % S;
        const int shift = (r / stride) * PW + t / stride;
        const int copy = copies == 2 ? (shift & 1) : 0;
        const int phase = (r % stride) * stride + t % stride;
        id = ((copy * stride * stride + phase) * C + c) * pitch + shift - copy;
    }
    ids[q] = id;
    const int grp = q / 64, j = (q % 64) / 16, p = (q % 16) / 4, rr = q % 4;
    ids_pm[grp * 64 + 16 * p + 4 * j + rr] = id;
}

hipError_t launch_plane_ids(const int* kidx, int* ids, int* ids_pm, int slots, int C, int S, int stride, int PW,
                            int pitch, int copies, int zero_id, half_t* planes, hipStream_t stream)
{
    if (slots <= 0) return hipSuccess;
    hipLaunchKernelGGL(plane_ids_kernel, dim3((slots + 255) / 256), dim3(256), 0, stream, kidx, ids, ids_pm, slots, C, S,
                       stride, PW, pitch, copies, zero_id, planes);
    return hipGetLastError();
}

hipError_t launch_nhwc_to_planes(const SpconvLaunchArgs& a, half_t* planes, int PH, int PW, int pitch, int copies,
                                 hipStream_t stream, int batch_inner)
{
    PlaneGeom g{a.B, a.H, a.W, a.C, a.stride, a.pad_h, a.pad_w, PH, PW, pitch, copies, 0, {}, batch_inner};
    if (!fill_wanted_planes(g, a.R, a.S)) return hipErrorInvalidValue;
    const int np = a.B * PH * PW;
    const dim3 grid((np + TT - 1) / TT, (a.C + TT - 1) / TT, g.nwanted);
    hipLaunchKernelGGL(nhwc_to_planes_kernel, grid, dim3(256), 0, stream, a.in, planes, g);
    return hipGetLastError();
}

hipError_t launch_planes_to_nhwc(const half_t* dm, half_t* out, int F, int NP, int B, int PH, int PW, int Ho, int Wo,
                                 hipStream_t stream, int batch_inner)
{
    const dim3 grid((NP + TT - 1) / TT, (F + TT - 1) / TT);
    hipLaunchKernelGGL(planes_to_nhwc_kernel, grid, dim3(256), 0, stream, dm, out, F, NP, B, PH, PW, Ho, Wo, batch_inner);
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

// =======================================================================================
// Convolution over the reference's own tensors (spconv/blockwise_format.h:111-128): input C-H-W-B, output
// F-H-W-B, batch innermost, H and W the extents of the OUTPUT grid and at the same time the bounds of the input
// (out(ho, wo) reads in(ho*stride - R/2 + r, wo*stride - S/2 + t) where that lies inside H x W, zero elsewhere).
// With the batch innermost both ends of the GEMM are contiguous: a kept vector k = (r, t, c) is a run of channel
// c's plane at a constant offset, and a row of the result is a row of the output.  Two launches:
//   1. chwb_to_planes_kernel: pure copy with zero fill into padded phase planes
//        planes[phase (a, b)][c][(i * PW + j) * B + n] = in[c][i*stride + a - R/2][j*stride + b - S/2][n]
//      with PHX = H + (R-1)/stride rows and PW = W + (S-1)/stride columns per plane: tap (r, t) of output (ho, wo)
//      reads phase (r % stride, t % stride) at (ho + r / stride, wo + t / stride).  B is a multiple of 8, so
//      every tap offset is a multiple of 16 bytes and no shifted copy is needed.
//   2. the role-split SpMM over the H * PW * B columns (ho, j, n) of the padded output grid; its epilogue maps a
//      column to the compact output row and drops the (S-1)/stride padding columns per row (output_column()).
// =======================================================================================
struct ChwbGeom {
    int B, H, W, C, stride, pad_h, pad_w;
    int PHX, PW;  // rows and columns of a phase plane
    int pitch;    // values per channel row of the plane tensor
};

// one thread per 16-byte piece (8 batch entries): grid.x covers the pieces of one channel plane, grid.y the channels,
// grid.z the phases
__global__ void __launch_bounds__(256) chwb_to_planes_kernel(const half_t* __restrict__ in, half_t* __restrict__ planes,
                                                             ChwbGeom g, unsigned magic_row, unsigned magic_b8)
{
    const int b8 = g.B >> 3, row_pieces = g.PW * b8;
    const int piece = blockIdx.x * 256 + threadIdx.x;
    if (piece >= g.PHX * row_pieces) return;
    const int c = blockIdx.y, phase = blockIdx.z;
    const int pa = phase / g.stride, pb = phase % g.stride;
    int i, rem, j, n8;
    fast_divmod(piece, row_pieces, magic_row, i, rem);
    fast_divmod(rem, b8, magic_b8, j, n8);
    const int hi = i * g.stride + pa - g.pad_h, wi = j * g.stride + pb - g.pad_w;
    half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (hi >= 0 && hi < g.H && wi >= 0 && wi < g.W) v = *(const half8_t*)(in + ((size_t)(c * g.H + hi) * g.W + wi) * g.B + n8 * 8);
    *(half8_t*)(planes + ((size_t)phase * g.C + c) * g.pitch + (size_t)piece * 8) = v;
}

hipError_t launch_chwb_to_planes(const half_t* in, half_t* planes, int B, int H, int W, int C, int R, int S, int stride,
                                 int PHX, int PW, int pitch, hipStream_t stream)
{
    ChwbGeom g{B, H, W, C, stride, R / 2, S / 2, PHX, PW, pitch};
    const int pieces = PHX * PW * (B >> 3);
    const dim3 grid((pieces + 255) / 256, C, stride * stride);
    hipLaunchKernelGGL(chwb_to_planes_kernel, grid, dim3(256), 0, stream, in, planes, g, udiv_magic(PW * (B >> 3)),
                       udiv_magic(B >> 3));
    return hipGetLastError();
}

template <int V, int WN, int NCONS, int NPROD, int KT, int NSTAGE>
__global__ void __launch_bounds__((NCONS + NPROD) * 64) spconv_chwb_kernel(SpmmLaunchArgs a)
{
    using Cfg = SpmmWsCfg<V, WN, NCONS, NPROD, KT, NSTAGE>;
    extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(SHFLBW_LDS char*)lds_raw;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // tiles as in the SpMM kernel: XCD x owns a contiguous range of the column-tile-major ids
    const int T = a.X * a.n_tiles;
    const int per = (T + 7) >> 3;
    const int xcd = blockIdx.x & 7;
    const int S = gridDim.x >> 3;
    const int id_first = xcd * per + (blockIdx.x >> 3);
    const int id_end = min(T, (xcd + 1) * per);
    if (wave >= NCONS)
        ws_producer<Cfg, V, NCONS, NPROD, KT, NSTAGE, false>(a, lds0, lane, wave - NCONS, id_first, id_end, S);
    else if constexpr (V == 16)
        ws_consumer16<Cfg, WN, NCONS, false, true>(a, lds0, lane, wave, id_first, id_end, S);
    else
        ws_consumer<Cfg, V, WN, NCONS, false, true>(a, lds0, lane, wave, id_first, id_end, S);
}

template <int V, int WN, int NCONS, int NPROD, int KT, int NSTAGE>
static hipError_t launch_chwb(const SpmmLaunchArgs& a, hipStream_t stream)
{
    using Cfg = SpmmWsCfg<V, WN, NCONS, NPROD, KT, NSTAGE>;
    SpmmLaunchArgs b = a;
    b.n_tiles = (a.N + Cfg::BN - 1) / Cfg::BN;
    const int T = a.X * b.n_tiles;
    int grid = a.num_cus > 0 ? a.num_cus : 256;
    grid = (grid / 8) * 8;
    const int need = ((T + 7) / 8) * 8;
    if (grid > need) grid = need;
    hipLaunchKernelGGL((spconv_chwb_kernel<V, WN, NCONS, NPROD, KT, NSTAGE>), dim3(grid), dim3(Cfg::THREADS), Cfg::LDS_BYTES,
                       stream, b);
    return hipGetLastError();
}

template <int V, int WN, int NCONS, int NPROD, int KT, int NSTAGE>
static hipError_t prepare_chwb()
{
    using Cfg = SpmmWsCfg<V, WN, NCONS, NPROD, KT, NSTAGE>;
    return hipFuncSetAttribute((const void*)spconv_chwb_kernel<V, WN, NCONS, NPROD, KT, NSTAGE>,
                               hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES);
}

#define SHFLBW_CHWB(V, WN, NC, NP, KT, NS)                                                                             \
    {                                                                                                                  \
        V, WN* NC, (NC + NP) * 64, SpmmWsCfg<V, WN, NC, NP, KT, NS>::LDS_BYTES, &launch_chwb<V, WN, NC, NP, KT, NS>,  \
            &prepare_chwb<V, WN, NC, NP, KT, NS>                                                                       \
    }

static const ConvChwbKernel g_chwb[] = {
    SHFLBW_CHWB(64, 128, 4, 4, 32, 4),
    SHFLBW_CHWB(32, 128, 4, 4, 32, 4),
    SHFLBW_CHWB(16, 128, 4, 4, 32, 4),
    SHFLBW_CHWB(128, 64, 4, 4, 32, 6),
};

const ConvChwbKernel* conv_chwb_kernel(int V)
{
    for (const ConvChwbKernel& k : g_chwb)
        if (k.V == V) return &k;
    return nullptr;
}

template <int V, int WN, int NCONS, int NPROD, int KT, int NSTAGE>
static hipError_t launch_fused(const SpmmLaunchArgs& a, const ConvFuseArgs& c, hipStream_t stream)
{
    using Cfg = SpmmWsCfg<V, WN, NCONS, NPROD, KT, NSTAGE>;
    SpmmLaunchArgs b = a;
    b.n_tiles = (a.N + Cfg::BN - 1) / Cfg::BN;
    const int T = a.X * b.n_tiles;
    int grid = a.num_cus > 0 ? a.num_cus : 256;
    grid = (grid / 8) * 8;
    const int need = ((T + 7) / 8) * 8;
    if (grid > need) grid = need;
    hipLaunchKernelGGL((spconv_fused_kernel<V, WN, NCONS, NPROD, KT, NSTAGE>), dim3(grid), dim3(Cfg::THREADS),
                       Cfg::LDS_BYTES + 16, stream, b, c);
    return hipGetLastError();
}

template <int V, int WN, int NCONS, int NPROD, int KT, int NSTAGE>
static hipError_t prepare_fused()
{
    using Cfg = SpmmWsCfg<V, WN, NCONS, NPROD, KT, NSTAGE>;
    return hipFuncSetAttribute((const void*)spconv_fused_kernel<V, WN, NCONS, NPROD, KT, NSTAGE>,
                               hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES + 16);
}

#define SHFLBW_FUSED(V, WN, NC, NP, KT, NS)                                                                     \
    {                                                                                                           \
        V, WN* NC, NC, (NC + NP) * 64, SpmmWsCfg<V, WN, NC, NP, KT, NS>::LDS_BYTES + 16, &launch_fused<V, WN, NC, NP, KT, NS>, \
            &prepare_fused<V, WN, NC, NP, KT, NS>                                                               \
    }

// one fused kernel per block height: the tile shape of the SpMM default of that height
static const ConvFusedKernel g_fused[] = {
    SHFLBW_FUSED(64, 128, 4, 4, 32, 4),
    SHFLBW_FUSED(32, 128, 4, 4, 32, 4),
    SHFLBW_FUSED(16, 128, 4, 4, 32, 4),
    SHFLBW_FUSED(128, 64, 4, 4, 32, 6),
};

const ConvFusedKernel* conv_fused_kernel(int V)
{
    for (const ConvFusedKernel& k : g_fused)
        if (k.V == V) return &k;
    return nullptr;
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
