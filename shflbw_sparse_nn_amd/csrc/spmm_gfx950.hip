// Shfl-BW SpMM for gfx950 (MI355X):  D[perm[r]] = alpha * (A_stored[r,:] * B) + beta * C[perm[r]].
//
// Replaces the reference's kernel and its device primitives
// (block_sparse/spmm/blockwise_kernel.h:108-294 main loop, :552-579 epilogue,
// block_sparse/common/{mma,memcpy,swizzle,epilogue}.h) with a design for 64-lane waves:
//
//  * one workgroup = one row panel (V stored rows) x BN output columns; its waves split BN;
//  * the kept activation rows B[k, n0:n0+BN] are gathered straight from global memory into a
//    ring of LDS stages (16 bytes per lane, no register round trip), KT rows per stage;
//  * a wave reads its B operand with transposing LDS loads (the rows are n-contiguous, the
//    matrix core wants 8 consecutive k per lane), the 32-byte pieces of each LDS row are
//    XOR-swizzled so these loads are bank-conflict free;
//  * the A operand comes from the weight's private image, already in register order: each
//    fragment is 1 KiB that one wave instruction copies into the stage next to the B rows;
//  * the kept-column ids are wave-uniform per gathered row and come through scalar loads, so
//    the vector-memory counter only ever counts the LDS copies and the waits are exact;
//  * fp32 accumulators are rounded once to fp16, staged through LDS and scattered as whole
//    row segments through the permutation.
#include <mutex>
#include <type_traits>

#include "kernel_common.h"
#include "spmm_launch.h"
#include <algorithm>
#include "spmm_slab.h"
#include "spmm_ws.h"

namespace shflbw {

template <int V, int WN, int NWAVES, int KT, int NSTAGE>
struct SpmmCfg {
    static constexpr int BN = WN * NWAVES;
    static constexpr int MB = V / 32;        // 32-row blocks of the panel
    static constexpr int NB = WN / 32;       // 32-column blocks of a wave's slice
    static constexpr int ROWB = BN * 2;      // bytes of one gathered row in LDS
    static constexpr int CPR = BN / 8;       // 16-byte pieces per row
    static constexpr int RPI = 64 / CPR > 0 ? 64 / CPR : 1; // rows covered by one gather instruction
    static constexpr int IPR = CPR / 64 > 0 ? CPR / 64 : 1; // gather instructions per row (BN > 512)
    static constexpr int SPT = KT / 16;         // MFMA k-steps per stage
    static constexpr int B_BYTES = KT * ROWB;   // gathered rows of one stage
    static constexpr int A_FRAGS = SPT * MB;    // 1 KiB A fragments of one stage
    static constexpr int STAGE_BYTES = B_BYTES + A_FRAGS * 1024;
    static constexpr int INSTR = KT * CPR / 64; // 1 KiB gather instructions per stage
    static constexpr int IPW = INSTR / NWAVES;  // ... issued by each wave
    static constexpr int RPW = KT / NWAVES;     // gathered rows owned by each wave
    static constexpr int AIPW = (A_FRAGS + NWAVES - 1) / NWAVES; // A fragment copies per wave
    static constexpr int DMA_PER_ITER = IPW + AIPW;              // per wave and stage
    static constexpr int EPI_ROWB = ROWB + 16;  // padded row of the output staging tile
    static constexpr int PIPE_BYTES = NSTAGE * STAGE_BYTES;
    static constexpr int EPI_BYTES = V * EPI_ROWB;
    static constexpr int LDS_BYTES = PIPE_BYTES > EPI_BYTES ? PIPE_BYTES : EPI_BYTES;
    static constexpr int THREADS = NWAVES * 64;
    static_assert(V % 32 == 0 && WN % 32 == 0, "32x32x16 tiles");
    static_assert(BN >= 128 && BN <= 512 && (BN & (BN - 1)) == 0, "row swizzle needs 8..32 32-byte pieces per row");
    static_assert(KT % 16 == 0 && 64 % KT == 0, "stage depth must divide the 64-slot padding");
    static_assert(KT % NWAVES == 0 && INSTR % NWAVES == 0, "gather must split evenly over the waves");
    static_assert(IPW * RPI == RPW, "a wave's gather instructions cover whole rows");
    static_assert((NSTAGE - 2) * DMA_PER_ITER < 64, "vmcnt is a 6-bit counter");
    static_assert(NSTAGE >= 2, "double buffering at least");
};

template <int V, int WN, int NWAVES, int KT, int NSTAGE>
__global__ void __launch_bounds__(NWAVES * 64) spmm_shflbw_kernel(SpmmLaunchArgs a)
{
    using Cfg = SpmmCfg<V, WN, NWAVES, KT, NSTAGE>;
    constexpr int BN = Cfg::BN, MB = Cfg::MB, NB = Cfg::NB, ROWB = Cfg::ROWB, CPR = Cfg::CPR;
    constexpr int IPW = Cfg::IPW, SPT = Cfg::SPT, EPI_ROWB = Cfg::EPI_ROWB, RPI = Cfg::RPI, RPW = Cfg::RPW;
    constexpr int AIPW = Cfg::AIPW, A_FRAGS = Cfg::A_FRAGS;

    extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(SHFLBW_LDS char*)lds_raw;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lid = xcd_local_id(blockIdx.x, a.X * a.n_tiles);
    const int nt = lid / a.X;
    const int panel = lid - nt * a.X;
    const int n0 = nt * BN;
    const int N = a.N;

    const int2_t pd = ((const SHFLBW_CONST int2_t*)(uintptr_t)a.panel_desc)[panel]; // {k16 steps, first 64-slot group}
    const int g0 = pd.y;
    const SHFLBW_CONST int* kidx =
        (const SHFLBW_CONST int*)(uintptr_t)(a.kidx + (size_t)g0 * 64 + wave * RPW); // this wave's rows of a stage
    const char* __restrict__ pA = (const char*)a.packedA + (size_t)g0 * (64 * V * 2) + lane * 16;
    const int nsteps = pd.x;
    const int ntiles = (nsteps + SPT - 1) / SPT;

    // ---- per-lane constants of the gather.  Instruction j of this wave fills LDS pieces
    // (wave*IPW + j)*64 + lane of the stage; `sub` says which of the RPI rows the lane is in.
    const int sub = lane / CPR;
    int gcol[IPW];
#pragma unroll
    for (int j = 0; j < IPW; j++) {
        const int piece = ((wave * IPW + j) << 6) + lane;
        const int row = piece / CPR, pc = piece % CPR;
        const int lc = ((((pc >> 1) ^ row_xor32(row & 3))) << 1) | (pc & 1);
        const int col = n0 + lc * 8;
        gcol[j] = col < N ? col : 0; // columns past N are never stored; keep the address valid
    }
    // ---- per-lane constants of the transposing loads
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

    // output row of every stored row of the panel: lane l of register q holds row 64q + l
    int rid[(V + 63) / 64];
#pragma unroll
    for (int q = 0; q < (V + 63) / 64; q++) {
        const int r = min(q * 64 + lane, V - 1);
        rid[q] = a.row_ids ? a.row_ids[panel * V + r] : panel * V + r;
    }

    // kept-column ids of this wave's rows for the tile that is gathered next (scalar loads)
    int ks[RPW];
    auto load_idx = [&](int tile) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < RPW; r++) ks[r] = kidx[tile * KT + r];
    };
    // all copies of one stage issued by this wave: its rows of B and its share of the A fragments
    auto fill_stage = [&](int tile, int stage) __attribute__((always_inline)) {
        const uint32_t sb = lds0 + stage * Cfg::STAGE_BYTES;
#pragma unroll
        for (int j = 0; j < AIPW; j++) {
            const int f = (wave * AIPW + j) % A_FRAGS; // surplus waves repeat a fragment (same bytes)
            global_to_lds_16B(pA + ((size_t)tile * A_FRAGS + f) * 1024, sb + Cfg::B_BYTES + f * 1024);
        }
#pragma unroll
        for (int j = 0; j < IPW; j++) {
            int k = ks[j * RPI];
#pragma unroll
            for (int q = 1; q < RPI; q++) k = (sub == q) ? ks[j * RPI + q] : k;
            // a padding slot (id -1) gathers 16 bytes per lane of the row of zeros
            const half_t* src = k < 0 ? (const half_t*)a.zero_row + lane * 8
                                      : (const half_t*)((const char*)a.B + (size_t)k * a.ldb_bytes) + gcol[j];
            global_to_lds_16B(src, sb + (wave * IPW + j) * 1024);
        }
    };

    // ---- prologue: fill NSTAGE-1 stages
#pragma unroll
    for (int s = 0; s < NSTAGE - 1; s++) {
        if (s < ntiles) {
            load_idx(s);
            fill_stage(s, s);
        }
    }
    if (NSTAGE - 1 < ntiles) load_idx(NSTAGE - 1);

    int stage = 0;         // stage holding tile t
    int fill = NSTAGE - 1; // stage that receives tile t + NSTAGE - 1
    for (int t = 0; t < ntiles; t++) {
        // this wave's copies of tile t must have landed; the (NSTAGE-2) stages issued after it
        // may stay in flight (they did get issued if tile t+NSTAGE-2 exists)
        if (t + NSTAGE - 2 < ntiles)
            __builtin_amdgcn_s_waitcnt(vmcnt_imm((NSTAGE - 2) * Cfg::DMA_PER_ITER));
        else
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        __syncthreads(); // every wave's share of tile t is in LDS; stage `fill` is no longer read

        if (t + NSTAGE - 1 < ntiles) {
            fill_stage(t + NSTAGE - 1, fill);
            if (t + NSTAGE < ntiles) load_idx(t + NSTAGE);
        }

        const uint32_t sb = lds0 + stage * Cfg::STAGE_BYTES;
#pragma unroll
        for (int kk = 0; kk < SPT; kk++) {
            if (t * SPT + kk < nsteps) {
                half8_t afrag[MB], bfrag[NB];
#pragma unroll
                for (int mb = 0; mb < MB; mb++)
                    afrag[mb] = *(SHFLBW_LDS half8_t*)(uintptr_t)(sb + Cfg::B_BYTES + (kk * MB + mb) * 1024 + lane * 16);
#pragma unroll
                for (int nb = 0; nb < NB; nb++) {
                    const half4_t lo = lds_read_tr16(sb + boff[nb] + (kk * 16) * ROWB);
                    const half4_t hi = lds_read_tr16(sb + boff[nb] + (kk * 16 + 4) * ROWB);
                    bfrag[nb] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                }
#pragma unroll
                for (int mb = 0; mb < MB; mb++)
#pragma unroll
                    for (int nb = 0; nb < NB; nb++)
                        acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bfrag[nb], afrag[mb], acc[mb][nb], 0, 0, 0);
            }
        }
        stage = (stage + 1 == NSTAGE) ? 0 : stage + 1;
        fill = (fill + 1 == NSTAGE) ? 0 : fill + 1;
    }

    // ---- epilogue: fp32 -> fp16 once, stage the V x BN tile in LDS, scatter row segments
    __syncthreads(); // all waves are done reading the pipeline stages
    const float alpha = a.alpha;
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
            for (int ig = 0; ig < 4; ig++) {
                half4_t h;
#pragma unroll
                for (int e = 0; e < 4; e++) h[e] = (half_t)scaled(acc[mb][nb][ig * 4 + e], alpha, a.beta != 0.f);
                const int m = mb * 32 + (lane & 31);
                const int n = wave * WN + nb * 32 + ig * 8 + (lane >> 5) * 4;
                *(SHFLBW_LDS half4_t*)(uintptr_t)(lds0 + m * EPI_ROWB + n * 2) = h;
            }
    __syncthreads();
    const float beta = a.beta;
    constexpr int PIECES = V * CPR;
    constexpr int NIT = PIECES / Cfg::THREADS;
    static_assert(PIECES % Cfg::THREADS == 0, "whole passes over the staged tile");
    // all loads (row ids were fetched before the main loop, C here) are issued before the first
    // store: the vector-memory counter is in-order, a load behind a store would wait for it
    half8_t v[NIT], c[NIT];
    size_t off[NIT];
    bool ok[NIT];
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int id = it * Cfg::THREADS + threadIdx.x;
        const int r = id / CPR, pc = id % CPR;
        const int col = n0 + pc * 8;
        ok[it] = col < N;
        v[it] = *(SHFLBW_LDS half8_t*)(uintptr_t)(lds0 + r * EPI_ROWB + pc * 16);
        const int orow = __shfl(rid[r >> 6], r & 63);
        off[it] = (size_t)orow * N + col;
        if (beta != 0.f && ok[it]) c[it] = *(const half8_t*)(a.C + off[it]);
    }
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        if (beta != 0.f) {
#pragma unroll
            for (int e = 0; e < 8; e++) v[it][e] = (half_t)((float)v[it][e] + beta * (float)c[it][e]);
        }
        if (ok[it]) *(half8_t*)(a.D + off[it]) = v[it];
    }
}

// kept-column id for a lane: one gather instruction covers `rpi` consecutive rows, `sub` says
// which of them the lane belongs to; the ids are wave-uniform, the select makes them per-lane
template <int N_>
__device__ __forceinline__ int ks_sel(const int (&ks)[N_], int base, int sub, int rpi)
{
    int k = ks[base];
#pragma unroll
    for (int q = 1; q < 4; q++)
        if (q < rpi) k = (sub == q) ? ks[base + q] : k;
    return k;
}

template <int V, int WN, int NCONS, int NPROD, int KT, int NSTAGE>
__global__ void
__launch_bounds__((NCONS + NPROD) * 64, (SpmmWsCfg<V, WN, NCONS, NPROD, KT, NSTAGE>::WGS_PER_CU * (NCONS + NPROD) + 3) / 4)
spmm_shflbw_ws_kernel(SpmmLaunchArgs a)
{
    using Cfg = SpmmWsCfg<V, WN, NCONS, NPROD, KT, NSTAGE>;

    extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(SHFLBW_LDS char*)lds_raw;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int X = a.X;

    // ---- this workgroup's tiles: XCD x owns the contiguous id range [x*per, (x+1)*per), ids are
    // n-tile major (id = nt*X + panel); the S workgroups of the XCD stride through that range.
    const int T = X * a.n_tiles;
    const int per = (T + 7) >> 3;
    const int xcd = blockIdx.x & 7;
    const int S = gridDim.x >> 3;
    const int id_first = xcd * per + (blockIdx.x >> 3);
    const int id_end = min(T, (xcd + 1) * per);

    if (wave >= NCONS) {
        ws_producer<Cfg, V, NCONS, NPROD, KT, NSTAGE>(a, lds0, lane, wave - NCONS, id_first, id_end, S);
        return;
    }

    if constexpr (V == 16)
        ws_consumer16<Cfg, WN, NCONS>(a, lds0, lane, wave, id_first, id_end, S);
    else
        ws_consumer<Cfg, V, WN, NCONS>(a, lds0, lane, wave, id_first, id_end, S);
}

template <int V, int WN, int NCONS, int NPROD, int KT, int NSTAGE>
static hipError_t launch_ws(const SpmmLaunchArgs& a, hipStream_t stream)
{
    using Cfg = SpmmWsCfg<V, WN, NCONS, NPROD, KT, NSTAGE>;
    SpmmLaunchArgs b = a;
    b.n_tiles = (a.N + Cfg::BN - 1) / Cfg::BN;
    const int T = a.X * b.n_tiles;
    // the gather addresses rows of B with 32-bit byte offsets
    if ((unsigned long long)a.K * (unsigned long long)a.ldb_bytes + (unsigned long long)a.N * 2ull > 0xffffffffull)
        return hipErrorInvalidValue;
    // one persistent workgroup per compute unit; fewer when there are fewer tiles (multiple of 8 XCDs)
    int grid = (a.num_cus > 0 ? a.num_cus : 256) * Cfg::WGS_PER_CU;
    grid = (grid / 8) * 8;
    const int need = ((T + 7) / 8) * 8;
    if (grid > need) grid = need;
    hipLaunchKernelGGL((spmm_shflbw_ws_kernel<V, WN, NCONS, NPROD, KT, NSTAGE>), dim3(grid),
                       dim3(Cfg::THREADS), Cfg::LDS_BYTES, stream, b);
    return hipGetLastError();
}

template <int V, int WN, int NCONS, int NPROD, int KT, int NSTAGE>
static hipError_t prepare_ws()
{
    using Cfg = SpmmWsCfg<V, WN, NCONS, NPROD, KT, NSTAGE>;
    return hipFuncSetAttribute((const void*)spmm_shflbw_ws_kernel<V, WN, NCONS, NPROD, KT, NSTAGE>,
                               hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES);
}

#define SHFLBW_WS_VARIANT(V, WN, NC, NP, KT, NS)                                                             \
    {                                                                                                        \
        V, WN* NC, (NC + NP) * 64, SpmmWsCfg<V, WN, NC, NP, KT, NS>::LDS_BYTES,                               \
            "ws" #V "x" #WN "x" #NC "c" #NP "p_k" #KT "_s" #NS, &launch_ws<V, WN, NC, NP, KT, NS>,           \
            &prepare_ws<V, WN, NC, NP, KT, NS>                                                                \
    }

// ---------------------------------------------------------------------------------------
// slab form (all rows of a 64-column slab of B in LDS): launcher
// ---------------------------------------------------------------------------------------
static hipError_t launch_slab(const SpmmLaunchArgs& a, hipStream_t stream)
{
    using Cfg = SpmmSlabCfg;
    if (a.K > Cfg::MAX_K || !a.slab_ids || a.K <= 0) return hipErrorInvalidValue;
    SpmmLaunchArgs b = a;
    b.n_tiles = (a.N + Cfg::BN - 1) / Cfg::BN;
    // the panels under one column tile are dealt to as many workgroups as it takes to give every compute unit a job
    // ... and so that the panels of one wave have at most RID_REGS * 64 rows
    const int cus = ((a.num_cus > 0 ? a.num_cus : 256) / 8) * 8;
    const int rows_per_wg = Cfg::NW * Cfg::RID_REGS * 64;
    b.slab_chunks = std::max(1, std::min(a.X, std::max(cus / b.n_tiles, (a.M + rows_per_wg - 1) / rows_per_wg)));
    const int T = b.n_tiles * b.slab_chunks;
    const int grid = std::min(cus, ((T + 7) / 8) * 8);
    hipLaunchKernelGGL(spmm_shflbw_slab_kernel, dim3(grid), dim3(Cfg::THREADS), Cfg::lds_bytes(a.K), stream, b);
    return hipGetLastError();
}

static hipError_t prepare_slab()
{
    return hipFuncSetAttribute((const void*)spmm_shflbw_slab_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                               SpmmSlabCfg::LDS_MAX);
}

#define SHFLBW_SLAB_VARIANT()                                                                                     \
    {                                                                                                             \
        SpmmSlabCfg::V, SpmmSlabCfg::BN, SpmmSlabCfg::THREADS, SpmmSlabCfg::LDS_MAX, "slab32x64", &launch_slab,    \
            &prepare_slab, SpmmSlabCfg::MAX_K                                                                     \
    }

// ---------------------------------------------------------------------------------------
// variant table
// ---------------------------------------------------------------------------------------
template <int V, int WN, int NWAVES, int KT, int NSTAGE>
static hipError_t launch_variant(const SpmmLaunchArgs& a, hipStream_t stream)
{
    using Cfg = SpmmCfg<V, WN, NWAVES, KT, NSTAGE>;
    const int n_tiles = (a.N + Cfg::BN - 1) / Cfg::BN;
    SpmmLaunchArgs b = a;
    b.n_tiles = n_tiles;
    hipLaunchKernelGGL((spmm_shflbw_kernel<V, WN, NWAVES, KT, NSTAGE>), dim3(a.X * n_tiles), dim3(Cfg::THREADS),
                       Cfg::LDS_BYTES, stream, b);
    return hipGetLastError();
}

template <int V, int WN, int NWAVES, int KT, int NSTAGE>
static hipError_t prepare_variant()
{
    using Cfg = SpmmCfg<V, WN, NWAVES, KT, NSTAGE>;
    return hipFuncSetAttribute((const void*)spmm_shflbw_kernel<V, WN, NWAVES, KT, NSTAGE>,
                               hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES);
}

#define SHFLBW_VARIANT(V, WN, NW, KT, NS)                                                                   \
    {                                                                                                       \
        V, WN* NW, NW * 64, SpmmCfg<V, WN, NW, KT, NS>::LDS_BYTES, #V "x" #WN "x" #NW "w_k" #KT "_s" #NS,       \
            &launch_variant<V, WN, NW, KT, NS>, &prepare_variant<V, WN, NW, KT, NS>                          \
    }

static const SpmmVariant g_variants[] = {
    // block 64 (the first entry of a block size is the library's choice; measured order)
    SHFLBW_WS_VARIANT(64, 128, 4, 4, 32, 4),
    SHFLBW_WS_VARIANT(64, 128, 4, 4, 16, 5),
    SHFLBW_WS_VARIANT(64, 64, 4, 4, 32, 6),
    SHFLBW_WS_VARIANT(64, 128, 4, 4, 16, 6),
    SHFLBW_WS_VARIANT(64, 64, 8, 8, 32, 4),
    SHFLBW_WS_VARIANT(64, 128, 4, 4, 32, 3),
    SHFLBW_WS_VARIANT(64, 128, 4, 4, 16, 4),
    SHFLBW_WS_VARIANT(64, 64, 4, 4, 32, 3), // two workgroups per compute unit
    SHFLBW_VARIANT(64, 64, 4, 32, 3),
    SHFLBW_VARIANT(64, 64, 4, 32, 2),
    SHFLBW_VARIANT(64, 64, 4, 16, 4),
    SHFLBW_VARIANT(64, 128, 2, 32, 3),
    SHFLBW_VARIANT(64, 128, 4, 16, 3),
    SHFLBW_VARIANT(64, 64, 2, 32, 3),
    SHFLBW_VARIANT(64, 32, 4, 32, 3),
    SHFLBW_WS_VARIANT(64, 32, 4, 4, 32, 6), // 128-column tiles: problems too small for the wider ones
    // block 32
    SHFLBW_WS_VARIANT(32, 128, 4, 4, 32, 4),
    SHFLBW_WS_VARIANT(32, 128, 4, 4, 16, 6),
    SHFLBW_WS_VARIANT(32, 64, 4, 4, 32, 6),
    SHFLBW_WS_VARIANT(32, 64, 4, 4, 32, 3), // two workgroups per compute unit
    SHFLBW_VARIANT(32, 64, 4, 32, 3),
    SHFLBW_VARIANT(32, 128, 2, 32, 3),
    SHFLBW_VARIANT(32, 128, 4, 16, 3),
    SHFLBW_VARIANT(32, 64, 2, 32, 3),
    SHFLBW_SLAB_VARIANT(), // weights of at most SLAB_MAX_K columns
    SHFLBW_WS_VARIANT(32, 32, 4, 4, 32, 6), // 128-column tiles: problems too small for the wider ones
    // block 16
    SHFLBW_WS_VARIANT(16, 128, 4, 4, 32, 4),
    // block 128
    SHFLBW_WS_VARIANT(128, 64, 4, 4, 32, 6),
    SHFLBW_WS_VARIANT(128, 64, 4, 4, 32, 5),
    SHFLBW_VARIANT(128, 64, 4, 32, 3),
    SHFLBW_VARIANT(128, 32, 4, 32, 3),
    SHFLBW_WS_VARIANT(128, 32, 4, 4, 32, 6), // 128-column tiles: problems too small for the wider ones
};

// The row of zeros the padding slots gather.  `g_zero_row` is the host-side handle of the symbol; kernels get
// the device address, looked up once per device.
static __device__ __align__(1024) unsigned char g_zero_row[1024];

const void* spmm_zero_row()
{
    static std::mutex lock;
    static void* addr[64] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
    std::lock_guard<std::mutex> guard(lock);
    if (!addr[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_zero_row)) != hipSuccess) return nullptr;
        addr[dev] = p;
    }
    return addr[dev];
}

const SpmmVariant* spmm_variants(int* count)
{
    *count = (int)(sizeof(g_variants) / sizeof(g_variants[0]));
    return g_variants;
}

} // namespace shflbw
