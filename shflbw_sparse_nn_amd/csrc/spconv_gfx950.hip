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
    static constexpr int MB = V / 32;   // 32-row blocks of a panel (block height 16: none, one 16x16x32 tile row)
    static constexpr int NB = WN / 32;
    static constexpr int NB16 = WN / 16; // 16-column blocks of a wave (block height 16)
    static constexpr int ROWB = BN * 2;
    static constexpr int CPR = BN / 8;
    static constexpr int SPT = KT / 16;
    static constexpr int THREADS = NWAVES * 64;
    static constexpr int PIECES = KT * CPR;          // 16-byte pieces per stage
    static constexpr int PPT = PIECES / THREADS;     // pieces per thread
    static constexpr int ROWS_PER_PASS = THREADS / CPR;
    static constexpr int LDS_BYTES = KT * ROWB;
    static_assert((V % 32 == 0 || (V == 16 && KT == 32)) && WN % 32 == 0, "32x32x16 tiles, or 16x16x32 for V = 16");
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
    constexpr bool V16 = V == 16;       // 16x16x32 tiles: one 32-slot step per A fragment, a lane holds 4 pixels of one filter
    constexpr int NB16 = Cfg::NB16;

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

    float16_t acc[V16 ? 1 : MB][NB];
#pragma unroll
    for (int mb = 0; mb < (V16 ? 1 : MB); mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[mb][nb][i] = 0.f;
    // block height 16: the fragment addresses and accumulators of the 16x16x32 tiles (as in the SpMM's consumer for
    // that block height: rows 8 (lane / 16) + (lane % 16) / 4 and four further down, 16-column units)
    uint32_t boff16[NB16];
    float4_t acc16[NB16];
#pragma unroll
    for (int nb = 0; nb < NB16; nb++) {
        const int unit = (wave * WN + nb * 16) / 16;
        boff16[nb] = (uint32_t)((8 * (lane >> 4) + (li >> 2)) * ROWB + ((unit ^ row_xor32(li >> 2)) << 5) + ((li & 3) << 3));
        acc16[nb] = float4_t{0.f, 0.f, 0.f, 0.f};
    }

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

        if constexpr (V16) { // one 32-slot step per stage; an odd last 16-slot step has zero weights behind it
            static_assert(!V16 || SPT == 2, "a stage is one 32-slot step");
            if (t * SPT < nsteps) {
                const half8_t afrag = pA[(size_t)t * 64 + lane];
#pragma unroll
                for (int nb = 0; nb < NB16; nb++) {
                    const half4_t lo = lds_read_tr16(lds0 + boff16[nb]);
                    const half4_t hi = lds_read_tr16(lds0 + boff16[nb] + 4 * ROWB);
                    const half8_t bfrag = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                    acc16[nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bfrag, afrag, acc16[nb], 0, 0, 0);
                }
            }
        } else
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
    // perm[panel*V + mb*32 + lane%32] of 16 pixels per 32x32 block (block height 16: channel perm[panel*16 + lane%16]
    // of 4 pixels per 16x16 block)
    if constexpr (V16) {
        const int srow = panel * V + (lane & 15);
        const int f = a.row_ids ? a.row_ids[srow] : srow;
#pragma unroll
        for (int nb = 0; nb < NB16; nb++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int p = n0 + wave * WN + nb * 16 + (lane >> 4) * 4 + i;
                if (p < npix) a.out[(size_t)p * a.F + f] = (half_t)acc16[nb][i];
            }
    }
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
            // written through (device scope): the planes do not wait dirty in the L2s for the end of the launch
            if (c0 + o < g.C) store_result_16B<true>(dst + (size_t)(c0 + o) * g.pitch + p0 + q * 8, v);
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
            // written through: the output is not read again here, and nothing waits dirty for the end of the launch (a
            // streaming store was 1 % slower, an ordinary one 5 %)
            if (img < B && ho < Ho && wo < Wo && f < F)
                store_result_16B<true>(out + ((size_t)(img * Ho + ho) * Wo + wo) * F + f, v);
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

// =======================================================================================
// Fused form of the convolution: ONE persistent launch in which every XCD works for itself.
//
// The columns of the GEMM (the padded output grid with the batch innermost, as in the batch-innermost plane form:
// column (ho, j, img) = (ho * PW + j) * B + img, which is also the plane position tap (0, 0) of that output reads)
// are cut into one contiguous range of `cx` columns per XCD.  The workgroups of an XCD then run three phases over
// that range, on buffers nobody else touches and that stay in the XCD's own L2:
//   phase 0  NHWC input -> the XCD's slab of channel-major padded planes, positions [x * cx, x * cx + cx + largest tap
//            offset): slab[(phase * C + c) * pitch + local position]; 64 x 64 tile transposes, a few per chunk;
//   phase 1  the role-split SpMM over the range, tiles of (row panel x column tile): the gather ids are offsets into
//            the slab, the result rows go to the XCD's filter-major scratch fm[f][local column];
//   phase 2  fm -> NHWC output, 64 x 64 tile transposes, padding columns (j >= Wo) dropped.
// A phase starts when the units of work (chunks, tiles) of the one before are counted complete.  The counting is
// between workgroups of one XCD, so it is done in that XCD's L2 (xcd_fetch_add / xcd_read, about 0.7 us a round trip
// instead of a trip to memory), and the data handed from one workgroup to another needs no device-scope
// write-through: it is stored normally, acknowledged by the L2 (s_waitcnt vmcnt(0)) before the writer counts it, and
// read by compute units that have not touched those cache lines before in this launch (every line of the slab and of
// fm has exactly one writing workgroup: tiles start at multiples of 64 values and the pitches are multiples of 64).
//
// Who does what is fixed, so that no unit has to be claimed (a claim is another round trip): the W = gridDim.x / nx
// workgroups of an XCD carry the numbers l = blockIdx.x / nx = 0 .. W-1 (consecutive workgroup ids go to consecutive
// XCDs; the host has checked that on this device), and number l does the units l, l + W, l + 2W, ... of every phase.
// A number is taken by setting its bit in the XCD's PRESENT word.  No wait may depend on a workgroup that is not
// running (two such launches can share the chip, each with a part of its workgroups resident): a workgroup that has
// waited `patience` ticks for a phase looks for numbers nobody has taken, takes them and does their units as
// well, in this and the following phases; the late owner of such a number finds its bit set and leaves at once
// (so does a workgroup that finds itself on an XCD where its number is taken: the work is then done once, by the
// first).  Waits are bounded all the same (`spin_ticks`): a wait that runs out raises the flag word and the
// workgroup leaves; shflbw_spconv_check reports it.  The words are all zero between launches: the last of the W
// workgroups of an XCD to leave clears them.
// =======================================================================================

// synchronisation words: line 0 holds the flag and, at int XCD_TAKEOVERS, the count of take-overs since the scratch
// was made; XCD x owns lines 1 + x * XCD_LINES ..
constexpr int XPRESENT = 0, XD0 = 1, XD1 = 2, XLEFT = 3;
static_assert(XLEFT < XCD_LINES, "counter lines per XCD");

// Diagnostic build (-DSHFLBW_CONV_STAMPS): workgroups 0 and 9 leave 100 MHz timestamps of their phase boundaries
// behind the flag word (ints 16.. of line 0), and bits of `debug` switch parts of the kernel off.
#ifdef SHFLBW_CONV_STAMPS
#define CONV_DEBUG(bit) ((c.debug & (bit)) != 0)
#define CONV_STAMP(i)                                                                                           \
    do {                                                                                                        \
        if (tid == 0 && (blockIdx.x == 0 || blockIdx.x == 9))                                                   \
            ((unsigned long long*)(c.sync + 16))[(blockIdx.x == 0 ? 0 : 12) + (i)] = wall_clock64();            \
    } while (0)
#else
#define CONV_DEBUG(bit) false
#define CONV_STAMP(i) do { } while (0)
#endif

template <int V, int WN, int NCONS, int NPROD, int KT, int NSTAGE>
__global__ void __launch_bounds__((NCONS + NPROD) * 64) spconv_xcd_kernel(SpmmLaunchArgs a, ConvXcdArgs c)
{
    using Cfg = SpmmWsCfg<V, WN, NCONS, NPROD, KT, NSTAGE>;
    static_assert((NCONS + NPROD) * 64 == 512 && Cfg::RING_BYTES >= 8 * TT * TT * 2, "the layout phases use 512 threads and up to 64 KiB");
    extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
    __shared__ int mailbox;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(SHFLBW_LDS char*)lds_raw;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    CONV_STAMP(0);

    const int x = xcd_id();
    if (x >= c.nx) { // an XCD the host did not see when it probed the device: nothing here can be trusted
        if (wave == 0) {
            if (lane == 0) __hip_atomic_store(c.sync, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        return;
    }
    int* const sx = c.sync + (1 + x * XCD_LINES) * SYNC_LINE;
    const int W = (int)gridDim.x / c.nx;                   // workgroups of this launch on every XCD (at most 32)
    const int me = (int)blockIdx.x / c.nx;                 // this one's number among them
    const unsigned all_numbers = W >= 32 ? 0xffffffffu : (1u << W) - 1u;
    const int col0 = x * c.cx;
    const int n_x = min(c.cx, c.ncols - col0); // columns of this XCD (<= 0: none)

    // Counting is done by lane 0 of wave 0.  `wave == 0` is uniform for a wave (a scalar branch: whole waves take it
    // or skip it), and every use below is ONE such block between two workgroup barriers, so every wave passes the
    // same barriers in the same order however the compiler arranges the lane-0 code.  (Two lane-0 blocks next to
    // each other across a loop's back edge were merged by the compiler into a path of their own, and the other lanes
    // of wave 0 went through the barriers of the next iteration ahead of lane 0.)
    auto publish = [&](auto&& lane0_value) __attribute__((always_inline)) {
        __syncthreads(); // everybody has read the previous value
        if (wave == 0) {
            if (lane == 0) mailbox = lane0_value();
        }
        __syncthreads();
        return __builtin_amdgcn_readfirstlane(mailbox);
    };

    const PlaneGeom& g = c.g;
    half_t* const slab = c.slabs + (size_t)x * c.slab_elems;
    half_t* const fm = c.fm + (size_t)x * c.fm_elems;
    SpmmLaunchArgs b = a; // the XCD's own GEMM: its slab as B, its scratch as D, local column numbers
    b.N = max(n_x, 0);
    b.n_tiles = (b.N + Cfg::BN - 1) / Cfg::BN;
    b.B = slab;
    b.D = fm;
    b.ldd = c.cx;

    // ---- units of the three phases
    const int npos = n_x + c.max_shift; // local positions some column of this XCD reads
    const int pos_chunks = (npos + c.pt * TT - 1) / (c.pt * TT);
    const int n0units = n_x > 0 ? g.nwanted * c.ch_chunks * pos_chunks : 0;
    const int n1units = n_x > 0 ? a.X * b.n_tiles : 0;
    const int col_chunks = (n_x + c.mt * TT - 1) / (c.mt * TT);
    const int n2units = n_x > 0 ? c.f_chunks * col_chunks : 0;

    // phase 0: the chunks number l owns
    auto phase0 = [&](int l) __attribute__((always_inline)) {
        const int nk = (c.ct * c.pt) >> 1;
        int done = 0;
        for (int chunk = l; chunk < n0units; chunk += W, done++) {
            const int plane = chunk / (c.ch_chunks * pos_chunks), rem = chunk % (c.ch_chunks * pos_chunks);
            const int p_base = (rem / c.ch_chunks) * (c.pt * TT), c_base = (rem % c.ch_chunks) * (c.ct * TT);
            const int phase = g.wanted[plane];
            const int pa = phase / g.stride, pb = phase % g.stride;
            half_t* dst = slab + (size_t)phase * g.C * g.pitch;
            if (CONV_DEBUG(1)) continue;
            transpose_tiles(
                lds0, tid, nk,
                [&](int tile, int i, int j) { // source row = plane position, piece = 8 channels
                    half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
                    const int gpos = col0 + p_base + (tile / c.ct) * TT + i;
                    const int ch = c_base + (tile % c.ct) * TT + j * 8;
                    int rem2, img, prow, pcol;
                    fast_divmod(gpos, g.B, c.magic_b, rem2, img);
                    fast_divmod(rem2, g.PW, c.magic_pw, prow, pcol);
                    const int hi = prow * g.stride + pa - g.pad_h, wi = pcol * g.stride + pb - g.pad_w;
                    if (prow < g.PH && hi >= 0 && hi < g.H && wi >= 0 && wi < g.W && ch < g.C)
                        v = *(const half8_t*)(c.in + ((size_t)(img * g.H + hi) * g.W + wi) * g.C + ch);
                    return v;
                },
                [&](int tile, int o, int q, half8_t v) { // destination row = channel, 8 positions
                    const int ch = c_base + (tile % c.ct) * TT + o;
                    const int p = p_base + (tile / c.ct) * TT + q * 8;
                    if (ch < g.C && p < g.pitch) *(half8_t*)(dst + (size_t)ch * g.pitch + p) = v;
                });
        }
        return done;
    };
    // phase 1: the tiles number l owns, as one stream (the producers run ahead across its tile boundaries)
    auto phase1 = [&](int l) __attribute__((always_inline)) {
        if (l >= n1units || CONV_DEBUG(2)) return l < n1units ? (n1units - l + W - 1) / W : 0;
        if (wave >= NCONS)
            ws_producer<Cfg, V, NCONS, NPROD, KT, NSTAGE>(b, lds0, lane, wave - NCONS, l, n1units, W);
        else if constexpr (V == 16)
            ws_consumer16<Cfg, WN, NCONS, true>(b, lds0, lane, wave, l, n1units, W);
        else
            ws_consumer<Cfg, V, WN, NCONS, true>(b, lds0, lane, wave, l, n1units, W);
        return (n1units - l + W - 1) / W;
    };
    // phase 2: the chunks number l owns
    auto phase2 = [&](int l) __attribute__((always_inline)) {
        for (int chunk = l; chunk < n2units; chunk += W) {
            const int f_base = (chunk % c.f_chunks) * (c.ft * TT);
            const int m_base = (chunk / c.f_chunks) * (c.mt * TT);
            if (CONV_DEBUG(4)) continue;
            transpose_tiles(
                lds0, tid, (c.ft * c.mt) >> 1,
                [&](int tile, int i, int j) { // source row = filter, piece = 8 columns of the GEMM
                    half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
                    const int f = f_base + (tile % c.ft) * TT + i;
                    const int m = m_base + (tile / c.ft) * TT + j * 8;
                    if (f < c.F && m < n_x) v = *(const half8_t*)(fm + (size_t)f * c.cx + m);
                    return v;
                },
                [&](int tile, int o, int q, half8_t v) { // destination row = the pixel of column m, 8 filters
                    const int m = m_base + (tile / c.ft) * TT + o;
                    const int f = f_base + (tile % c.ft) * TT + q * 8;
                    int rem2, img, ho, wo;
                    fast_divmod(col0 + m, g.B, c.magic_b, rem2, img);
                    fast_divmod(rem2, g.PW, c.magic_pw, ho, wo);
                    // streaming store: the output is not read again here
                    if (m < n_x && wo < c.Wo && f < c.F)
                        __builtin_nontemporal_store(v, (half8_t*)(c.out + ((size_t)(img * c.Ho + ho) * c.Wo + wo) * c.F + f));
                });
        }
    };
    // Ends a phase for this workgroup: its stores are acknowledged by the L2 (every wave waits for its own before the
    // barrier), then lane 0 counts `units` as done in `word` and waits until the word has reached `target`.  Returns
    // -1 then; -2 when the time ran out; -3 when `refused` (this workgroup's number turned out to be somebody else's:
    // nothing is counted); or, after `patience` ticks of waiting, a number nobody had taken and that this workgroup
    // has taken now (its units of this phase are to be done and the phase ended again).
    auto end_phase = [&](int* word, int units, int target, bool refused) __attribute__((always_inline)) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        return publish([&]() {
            if (refused) return -3;
            if (units > 0) (void)xcd_fetch_add(word, units);
            // the clock is looked at once in 64 polls: reading it takes longer than a poll (at every poll when the
            // caller has set a patience below 64 ticks, which is how the tests reach the take-over path)
            const unsigned sparse_clock = c.patience < 64 ? 0u : 63u;
            unsigned long long t0 = 0, asked = 0;
            for (unsigned polls = 1; xcd_read(word) < target; polls++) {
                if ((polls & sparse_clock) == 0) {
                    const unsigned long long now = wall_clock64();
                    if (t0 == 0) t0 = asked = now;
                    if (now - t0 > (unsigned long long)c.spin_ticks) {
                        __hip_atomic_store(c.sync, 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        return -2;
                    }
                    if (now - asked > (unsigned long long)c.patience) {
                        asked = now;
                        const unsigned missing = all_numbers & ~(unsigned)xcd_read(sx + XPRESENT * SYNC_LINE);
                        if (missing) {
                            const int l = __builtin_ctz(missing);
                            if (!((unsigned)xcd_fetch_or(sx + XPRESENT * SYNC_LINE, (int)(1u << l)) & (1u << l))) {
                                (void)__hip_atomic_fetch_add(c.sync + XCD_TAKEOVERS, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                return l;
                            }
                        }
                    }
                }
                __builtin_amdgcn_s_sleep(1);
            }
            return -1;
        });
    };

    // ---- take this workgroup's number; the answer is looked at after its first units (the atomic is under way
    // while they run: what a second holder of a number writes is what the first one writes)
    unsigned taken_before = 0;
    if (c.late_ticks > 0 && (me & 1)) { // tests of the take-over path: every second workgroup joins late
        const unsigned long long t = wall_clock64();
        while (wall_clock64() - t < (unsigned long long)c.late_ticks) __builtin_amdgcn_s_sleep(8);
    }
    if (wave == 0) {
        if (lane == 0) taken_before = (unsigned)xcd_fetch_or(sx + XPRESENT * SYNC_LINE, (int)(1u << me));
    }
    unsigned mine = 1u << me; // the numbers this workgroup does the units of
    bool alive = n_x > 0;

    // ================= phase 0: NHWC input -> this XCD's slab of planes =================
    // (each phase: the units of the numbers in `todo`, then the end of the phase - which may come back with one more
    // number, if one had to be taken over)
    unsigned todo = mine;
    for (bool first = true; alive; first = false) {
        int units = 0;
        for (unsigned m = todo; m; m &= m - 1) units += phase0(__builtin_ctz(m));
        if (first) CONV_STAMP(1);
        // While the workgroup waits for the phase: the first stages of its first tile of phase 1 (kept-column ids,
        // A fragments) are read once by two waves that have nothing to do, so that the producers find them in the
        // L2 instead of waiting for memory twice in a row.  The loads are issued here and looked at after the wait.
        int w0 = 0, w1 = 0, w2 = 0;
        if (first && me < n1units && (wave == 1 || wave == 2) && !CONV_DEBUG(32)) {
            const int2_t pd = ((const SHFLBW_CONST int2_t*)(uintptr_t)a.panel_desc)[me % a.X];
            const int groups = (pd.x + 3) / 4; // 64-slot groups of the panel
            const char* src = wave == 1 ? (const char*)(KT == 16 ? a.kidx_pm : a.kidx) + (size_t)pd.y * 256
                                        : (const char*)a.packedA + (size_t)pd.y * (64 * V * 2);
            const size_t bytes = wave == 1 ? (size_t)min(groups, 8) * 256 : (size_t)min(groups, 3) * (64 * V * 2);
            const size_t off = (size_t)lane * 128; // one value per 128-byte line, 8 KiB per round of the wave
            if (off < bytes) w0 = *(const int*)(src + off);
            if (off + 8192 < bytes) w1 = *(const int*)(src + off + 8192);
            if (off + 16384 < bytes) w2 = *(const int*)(src + off + 16384);
        }
        // (a number somebody else holds already: that workgroup does, or did, its units)
        const int r = end_phase(sx + XD0 * SYNC_LINE, units, n0units, first && ((taken_before >> me) & 1u));
        asm volatile("" : : "v"(w0), "v"(w1), "v"(w2));
        if (r == -1) break;
        if (r < -1) alive = false;
        else mine |= (todo = 1u << r);
    }
    CONV_STAMP(2);

    // ================= phase 1: the SpMM over this XCD's columns =================
    todo = mine;
    for (bool first = true; alive; first = false) {
        int units = 0;
        for (unsigned m = todo; m; m &= m - 1) units += phase1(__builtin_ctz(m));
        if (first) CONV_STAMP(3);
        const int r = end_phase(sx + XD1 * SYNC_LINE, units, n1units, false); // a number without units in phase 0 may still be free
        if (r == -1) break;
        if (r < -1) alive = false;
        else mine |= (todo = 1u << r);
    }
    CONV_STAMP(4);

    // ================= phase 2: this XCD's fm[F][n_x] -> NHWC output =================
    if (alive) {
        for (unsigned m = mine; m; m &= m - 1) phase2(__builtin_ctz(m));
        CONV_STAMP(5);
    }

    // ================= leave: the last workgroup of the XCD clears its words for the next launch =================
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    CONV_STAMP(6);
    if (wave == 0) {
        if (lane == 0) {
            const int before = xcd_fetch_add(sx + XLEFT * SYNC_LINE, 1);
            if (before == W - 1)
                for (int i = 0; i <= XLEFT; i++)
                    __hip_atomic_store(sx + i * SYNC_LINE, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            else if (before >= W) // more workgroups on this XCD than its share: the counting was wrong
                __hip_atomic_store(c.sync, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// One wave per workgroup reports the XCD it runs on: the host checks that workgroup i of a launch lands on XCD
// i % nx before it lets the fused form count on that.
__global__ void xcd_probe_kernel(int* out)
{
    if (threadIdx.x == 0) out[blockIdx.x] = xcd_id();
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
        ws_producer<Cfg, V, NCONS, NPROD, KT, NSTAGE>(a, lds0, lane, wave - NCONS, id_first, id_end, S);
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

// (the widest tile of a block size first)
static const ConvChwbKernel g_chwb[] = {
    SHFLBW_CHWB(64, 128, 4, 4, 32, 4), SHFLBW_CHWB(64, 64, 4, 4, 32, 6),  SHFLBW_CHWB(64, 32, 4, 4, 32, 6),
    SHFLBW_CHWB(32, 128, 4, 4, 32, 4), SHFLBW_CHWB(32, 64, 4, 4, 32, 6),  SHFLBW_CHWB(32, 32, 4, 4, 32, 6),
    SHFLBW_CHWB(16, 128, 4, 4, 32, 4),
    SHFLBW_CHWB(128, 64, 4, 4, 32, 6), SHFLBW_CHWB(128, 32, 4, 4, 32, 6),
};

// The kernel of block height V with tiles of `tile_cols` columns; tile_cols <= 0: the choice for a GEMM of X row panels
// by `ncols` columns on `cus` compute units, as for the SpMM - 128-column tiles while there are at most as many of them as
// compute units, 256-column tiles while the 512-column ones would fill at most half of the compute units, the widest
// otherwise.
const ConvChwbKernel* conv_chwb_kernel(int V, int tile_cols, long X, long ncols, int cus)
{
    const ConvChwbKernel* widest = nullptr;
    for (const ConvChwbKernel& k : g_chwb) {
        if (k.V != V) continue;
        if (!widest) widest = &k;
        if (k.BN == tile_cols) return &k;
    }
    if (tile_cols > 0 || !widest) return nullptr;
    auto with = [&](int bn) -> const ConvChwbKernel* {
        for (const ConvChwbKernel& k : g_chwb)
            if (k.V == V && k.BN == bn) return &k;
        return nullptr;
    };
    const ConvChwbKernel* k = nullptr;
    if (X * ((ncols + 127) / 128) <= cus && (k = with(128))) return k;
    if (widest->BN == 512 && X * ((ncols + 511) / 512) <= cus / 2 && (k = with(256))) return k;
    return widest;
}

template <int V, int WN, int NCONS, int NPROD, int KT, int NSTAGE>
static hipError_t launch_xcd(const SpmmLaunchArgs& a, const ConvXcdArgs& c, hipStream_t stream)
{
    using Cfg = SpmmWsCfg<V, WN, NCONS, NPROD, KT, NSTAGE>;
    // one persistent workgroup per compute unit, the same number on every XCD
    int grid = a.num_cus > 0 ? a.num_cus : 256;
    grid = (grid / c.nx) * c.nx;
    if (grid <= 0 || c.nx <= 0 || grid / c.nx > 32 || c.cx <= 0 || (c.cx % TT) != 0 || (c.g.pitch % TT) != 0 || c.g.pitch < c.cx + c.max_shift)
        return hipErrorInvalidValue;
    hipLaunchKernelGGL((spconv_xcd_kernel<V, WN, NCONS, NPROD, KT, NSTAGE>), dim3(grid), dim3(Cfg::THREADS), Cfg::LDS_BYTES,
                       stream, a, c);
    return hipGetLastError();
}

template <int V, int WN, int NCONS, int NPROD, int KT, int NSTAGE>
static hipError_t prepare_xcd()
{
    using Cfg = SpmmWsCfg<V, WN, NCONS, NPROD, KT, NSTAGE>;
    return hipFuncSetAttribute((const void*)spconv_xcd_kernel<V, WN, NCONS, NPROD, KT, NSTAGE>,
                               hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES);
}

#define SHFLBW_XCD(V, WN, NC, NP, KT, NS)                                                                            \
    {                                                                                                                \
        V, WN* NC, (NC + NP) * 64, SpmmWsCfg<V, WN, NC, NP, KT, NS>::LDS_BYTES, &launch_xcd<V, WN, NC, NP, KT, NS>,  \
            &prepare_xcd<V, WN, NC, NP, KT, NS>                                                                      \
    }

// one fused kernel per block height: the tile shape of the SpMM default of that height
static const ConvXcdKernel g_xcd[] = {
    SHFLBW_XCD(64, 128, 4, 4, 32, 4),
    SHFLBW_XCD(32, 128, 4, 4, 32, 4),
    SHFLBW_XCD(16, 128, 4, 4, 32, 4),
    SHFLBW_XCD(128, 64, 4, 4, 32, 6),
};

const ConvXcdKernel* conv_xcd_kernel(int V)
{
    for (const ConvXcdKernel& k : g_xcd)
        if (k.V == V) return &k;
    return nullptr;
}

hipError_t launch_xcd_probe(int* out, int blocks, hipStream_t stream)
{
    hipLaunchKernelGGL(xcd_probe_kernel, dim3(blocks), dim3(64), 0, stream, out);
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
    SHFLBW_CONV_VARIANT(16, 32, 4, 32),
};

const SpconvVariant* spconv_variants(int* count)
{
    *count = (int)(sizeof(g_conv_variants) / sizeof(g_conv_variants[0]));
    return g_conv_variants;
}

} // namespace shflbw
