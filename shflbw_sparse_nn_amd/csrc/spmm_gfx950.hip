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
#include <type_traits>

#include "kernel_common.h"
#include "spmm_launch.h"

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
            global_to_lds_16B(a.B + ((size_t)k * N + gcol[j]), sb + (wave * IPW + j) * 1024);
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
                for (int e = 0; e < 4; e++) h[e] = (half_t)(acc[mb][nb][ig * 4 + e] * alpha);
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

// =======================================================================================
// Persistent, role-split kernel.
//
// One workgroup stays on a compute unit and walks a list of output tiles.  Its waves have
// two roles:
//   producers only issue the global->LDS copies (gathered B rows, A fragments) into a ring of
//     NSTAGE stages and run ahead of the math across tile boundaries;
//   consumers only read LDS and issue MFMA; each owns V x WN of the tile, reads the first
//     fragments of the next stage while the matrix cores work on the current one, and at the
//     end of a tile converts, stages its own sub-tile through a private LDS area and scatters
//     row segments - no workgroup barrier, so the stores overlap the next tile's main loop.
// One s_barrier per stage couples the roles: barrier g means "stage g+1 has landed and
// stage g-1 is no longer read".
// Scalar loads have a latency of several hundred cycles and return out of order (only a full
// wait is possible), so nothing on the stage cadence depends on a fresh one: per-panel
// descriptors are fetched one tile ahead, and the kept-column ids come from a producer-major
// copy of the index array, 16 ids (a producer's rows of four stages) per load, one such
// group ahead.  The consumer's stage loop is branch-free (two alternating
// fragment sets) so that its LDS reads really run one stage ahead of the MFMAs.
// Tiles are dealt so that the workgroups of one XCD work on the same B column slab.
// =======================================================================================
template <int V, int WN, int NCONS, int NPROD, int KT, int NSTAGE>
struct SpmmWsCfg {
    static constexpr int BN = WN * NCONS;
    static constexpr int MB = V / 32;
    static constexpr int NB = WN / 32;
    static constexpr int ROWB = BN * 2;
    static constexpr int B_BYTES = KT * ROWB;
    static constexpr int A_FRAGS = MB;                    // one MFMA k-step per stage
    static constexpr int STAGE_BYTES = B_BYTES + A_FRAGS * 1024;
    static constexpr int RPW = KT / NPROD;                // gathered rows (= copies) per producer and stage
    static constexpr int A_HI = A_FRAGS % NPROD;          // producers [0, A_HI) copy one more A fragment
    static constexpr int A_LO = A_FRAGS / NPROD;
    static constexpr int EPI_ROWB = WN * 2 + 16;
    static constexpr int EPI_WAVE_BYTES = 32 * EPI_ROWB;  // one 32-row block of a consumer's sub-tile
    static constexpr int RING_BYTES = NSTAGE * STAGE_BYTES;
    static constexpr int LDS_BYTES = RING_BYTES + NCONS * EPI_WAVE_BYTES;
    static constexpr int THREADS = (NCONS + NPROD) * 64;
    static_assert(V % 32 == 0 && WN % 32 == 0, "32x32x16 tiles");
    static_assert(BN == 512, "one gathered row is exactly one 1 KiB copy instruction");
    static_assert(KT == 16 && NPROD == 4, "the producer-major index copy is laid out for 4 producers x 4 rows x 4 stages");
    static_assert(NSTAGE >= 3, "one stage computed, one landed, one in flight");
    static_assert((NSTAGE - 3) * (RPW + A_LO + 1) < 64, "vmcnt is a 6-bit counter");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of a gfx950 compute unit");
};

__device__ __forceinline__ void wg_barrier()
{
    // bare barrier: no implied wait on outstanding global stores or copies
    asm volatile("s_barrier" ::: "memory");
}

// Walks the tile ids id, id+S, ... < end of one workgroup and keeps the descriptor of the
// current and of the following tile in scalar registers, so a tile switch never waits for memory.
struct TileWalker {
    int id, end, S, X;
    int2_t cur, nxt; // {k16 steps, first 64-slot group} of the panel of tile id / id+S
    const SHFLBW_CONST int2_t* desc;
    __device__ __forceinline__ int2_t fetch(int i) const
    {
        int2_t z = {0, 0};
        if (i < end) z = desc[i % X];
        return z;
    }
    __device__ __forceinline__ void init(const int* d, int first, int end_, int S_, int X_)
    {
        desc = (const SHFLBW_CONST int2_t*)(uintptr_t)d;
        id = first, end = end_, S = S_, X = X_;
        cur = fetch(id);
        nxt = fetch(id + S);
    }
    __device__ __forceinline__ void advance()
    {
        id += S;
        cur = nxt;
        nxt = fetch(id + S);
    }
    __device__ __forceinline__ bool valid() const { return id < end; }
    // skip tiles whose panel keeps no vector (they have no stage)
    __device__ __forceinline__ void skip_empty()
    {
        while (valid() && cur.x == 0) advance();
    }
};

template <int V, int WN, int NCONS, int NPROD, int KT, int NSTAGE>
__global__ void __launch_bounds__((NCONS + NPROD) * 64) spmm_shflbw_ws_kernel(SpmmLaunchArgs a)
{
    using Cfg = SpmmWsCfg<V, WN, NCONS, NPROD, KT, NSTAGE>;
    constexpr int BN = Cfg::BN, MB = Cfg::MB, NB = Cfg::NB, ROWB = Cfg::ROWB;
    constexpr int RPW = Cfg::RPW, A_FRAGS = Cfg::A_FRAGS;
    constexpr int STAGE_BYTES = Cfg::STAGE_BYTES, B_BYTES = Cfg::B_BYTES;

    extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(SHFLBW_LDS char*)lds_raw;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int N = a.N, X = a.X;

    // ---- this workgroup's tiles: XCD x owns the contiguous id range [x*per, (x+1)*per), ids are
    // n-tile major (id = nt*X + panel); the S workgroups of the XCD stride through that range.
    const int T = X * a.n_tiles;
    const int per = (T + 7) >> 3;
    const int xcd = blockIdx.x & 7;
    const int S = gridDim.x >> 3;
    const int id_first = xcd * per + (blockIdx.x >> 3);
    const int id_end = min(T, (xcd + 1) * per);

    if (wave >= NCONS) {
        // =========================== producer ===========================
        // A wave issues roughly one instruction every four to five cycles, and its vector-ALU
        // work would compete with the MFMAs of the consumer on the same SIMD; so the per-stage
        // path below is scalar bookkeeping plus the copies, nothing else, and the scalar state is
        // kept small enough to stay in registers.
        const int pw = wave - NCONS;
        const uint32_t rowbytes = (uint32_t)N * 2;
        const SHFLBW_CONST int2_t* desc = (const SHFLBW_CONST int2_t*)(uintptr_t)a.panel_desc;
        const SHFLBW_CONST int* kpm_all = (const SHFLBW_CONST int*)(uintptr_t)(a.kidx_pm + pw * 16);

        // -- cursor over the non-empty tiles of this workgroup: `cur` is the tile whose stages are
        // being issued, `nxt` the following non-empty one (descriptor {k16 steps, first group})
        int id = id_first, idn = id_first;
        int2_t cur = {0, 0}, nxt = {0, 0};
        auto find_next = [&]() __attribute__((always_inline)) { // idn, nxt <- next non-empty tile after idn
            nxt.x = 0;
            for (idn += S; idn < id_end; idn += S) {
                nxt = desc[idn % X];
                if (nxt.x > 0) break;
            }
        };
        idn = id_first - S;
        find_next();
        id = idn, cur = nxt; // first non-empty tile (cur.x == 0: none)
        if (cur.x > 0) find_next();

        int ti = 0;                // stage inside the tile
        const char* pA = nullptr;  // this wave's A fragment of the stage issued next
        uint32_t voff[RPW];        // per-lane byte offset inside a B row, one per copy of a stage
        const uint32_t aoff = lane * 16;
        auto open_tile = [&]() __attribute__((always_inline)) {
            ti = 0;
            const int n0 = (id / X) * BN;
            pA = (const char*)a.packedA + (size_t)cur.y * (64 * V * 2) + pw * 1024;
#pragma unroll
            for (int j = 0; j < RPW; j++) {
                // copy j fills row pw*RPW + j of the stage; the lane's 16-byte piece lands at
                // physical position `lane`, i.e. it must fetch logical piece lc of the row
                const int row = pw * RPW + j;
                const int lc = ((((lane >> 1) ^ row_xor32(row & 3))) << 1) | (lane & 1);
                const int col = n0 + lc * 8;
                voff[j] = (uint32_t)(col < N ? col : 0) * 2; // columns past N are never stored
            }
        };

        // -- kept-column ids: the producer-major copy holds, per 64-slot group, the 16 ids of this
        // producer contiguously (position 4*j + r: row r of stage j of the group).  `gc*` is the
        // group being issued, `gn*` the one after it in the stream (possibly the next tile's first),
        // loaded a whole group ahead.  Named vector values, never an indexable array: a
        // runtime-indexed array would be demoted to scratch memory, and a scratch load waits for
        // every copy in flight.
        int4_t gc0 = {0, 0, 0, 0}, gc1 = gc0, gc2 = gc0, gc3 = gc0;
        int4_t gn0 = gc0, gn1 = gc0, gn2 = gc0, gn3 = gc0;
        auto load_group = [&](int first_group, int q) __attribute__((always_inline)) {
            const SHFLBW_CONST int4_t* g = (const SHFLBW_CONST int4_t*)(kpm_all + ((size_t)first_group + q) * 64);
            gn0 = g[0], gn1 = g[1], gn2 = g[2], gn3 = g[3];
        };
        // called when group q of the current tile becomes the group being issued
        auto rotate_groups = [&](int q) __attribute__((always_inline)) {
            gc0 = gn0, gc1 = gn1, gc2 = gn2, gc3 = gn3;
            if ((q + 1) * 4 < cur.x)
                load_group(cur.y, q + 1);
            else if (nxt.x > 0)
                load_group(nxt.y, 0);
        };

        uint32_t sb = lds0; // ring slot (LDS byte address) of the next stage to issue
        uint32_t sbp_b = lds0 + pw * RPW * 1024; // ... where this wave's rows go
        uint32_t sbp_a = lds0 + pw * 1024;       // ... and its A fragment (plus the B area size)
        int issued = 0;
        auto issue_one = [&]() __attribute__((always_inline)) {
            if (cur.x == 0) return;
            // sbp = this wave's part of the stage: its B rows start at sbp, its A fragment slots at
            // sbp + A_BASE (both offsets are compile-time immediates of the copies)
            constexpr int A_BASE = B_BYTES; // plus pw*1024, folded into sbp_a
            if (Cfg::A_LO > 0 || pw < Cfg::A_HI) {
#pragma unroll
                for (int j = 0; j < Cfg::A_LO + 1; j++)
                    if (j < Cfg::A_LO || pw < Cfg::A_HI) {
                        if (j == 0) global_to_lds_16B_sbase<A_BASE>(pA, aoff, sbp_a);
                        if (j == 1) global_to_lds_16B_sbase<A_BASE + NPROD * 1024>(pA + NPROD * 1024, aoff, sbp_a);
                    }
            }
            const int js = ti & 3;
            int ks[RPW];
#pragma unroll
            for (int r = 0; r < RPW; r++) {
                int k = gc0[r];
                k = js == 1 ? gc1[r] : k;
                k = js == 2 ? gc2[r] : k;
                k = js == 3 ? gc3[r] : k;
                ks[r] = k;
            }
            static_assert(RPW == 4 && Cfg::A_LO + 1 <= 2, "copies are spelled out for 4 rows and up to 2 fragments");
            global_to_lds_16B_sbase<0 * 1024>((const char*)a.B + (uint64_t)(uint32_t)ks[0] * rowbytes, voff[0], sbp_b);
            global_to_lds_16B_sbase<1 * 1024>((const char*)a.B + (uint64_t)(uint32_t)ks[1] * rowbytes, voff[1], sbp_b);
            global_to_lds_16B_sbase<2 * 1024>((const char*)a.B + (uint64_t)(uint32_t)ks[2] * rowbytes, voff[2], sbp_b);
            global_to_lds_16B_sbase<3 * 1024>((const char*)a.B + (uint64_t)(uint32_t)ks[3] * rowbytes, voff[3], sbp_b);
            sbp_b = (sb + STAGE_BYTES == lds0 + Cfg::RING_BYTES) ? sbp_b - (NSTAGE - 1) * STAGE_BYTES : sbp_b + STAGE_BYTES;
            sbp_a = (sb + STAGE_BYTES == lds0 + Cfg::RING_BYTES) ? sbp_a - (NSTAGE - 1) * STAGE_BYTES : sbp_a + STAGE_BYTES;
            sb = (sb + STAGE_BYTES == lds0 + Cfg::RING_BYTES) ? lds0 : sb + STAGE_BYTES;
            pA += A_FRAGS * 1024;
            issued++;
            if (++ti == cur.x) { // next tile
                id = idn, cur = nxt;
                if (cur.x > 0) {
                    find_next();
                    open_tile();
                    rotate_groups(0);
                }
            } else if ((ti & 3) == 0) {
                rotate_groups(ti >> 2);
            }
        };

        if (cur.x > 0) {
            load_group(cur.y, 0);
            open_tile();
            rotate_groups(0);
        }
        for (int s = 0; s < NSTAGE - 2; s++) issue_one();
        // barrier g = -1, 0, 1, ..., issued-1: stage g+1 has landed; afterwards slot of stage g-1 is free
        for (int g = -1; g < issued; g++) {
            // copies of at most NSTAGE-3 later stages may stay in flight.  The count uses the
            // smaller per-stage number of copies (producers that also copy an A fragment issue one
            // more), which can only make the wait stricter; at the tail fewer stages follow and
            // everything is drained.
            if (NSTAGE > 3 && issued - (g + 2) >= NSTAGE - 3)
                __builtin_amdgcn_s_waitcnt(vmcnt_imm((NSTAGE - 3) * (RPW + Cfg::A_LO)));
            else
                __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
            wg_barrier();
            issue_one();
        }
        return;
    }

    // =========================== consumer ===========================
    const int cw = wave;
    const int li = lane & 15;
    uint32_t boff[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const int unit = (cw * WN + nb * 32) / 16 + ((lane >> 4) & 1);
        boff[nb] = (uint32_t)((8 * (lane >> 5) + (li >> 2)) * ROWB + ((unit ^ row_xor32(li >> 2)) << 5) + ((li & 3) << 3));
    }
    const uint32_t aoff = (uint32_t)(B_BYTES + lane * 16);
    const uint32_t epi = lds0 + Cfg::RING_BYTES + cw * Cfg::EPI_WAVE_BYTES;

    struct Frags {
        half8_t a[MB], b[NB];
    };
    Frags f0, f1;
    auto load_frags = [&](uint32_t sbase, Frags& f) __attribute__((always_inline)) {
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
            f.a[mb] = *(SHFLBW_LDS half8_t*)(uintptr_t)(sbase + aoff + mb * 1024);
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            const half4_t lo = lds_read_tr16(sbase + boff[nb]);
            const half4_t hi = lds_read_tr16(sbase + boff[nb] + 4 * ROWB);
            f.b[nb] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
    };

    TileWalker w;
    w.init(a.panel_desc, id_first, id_end, S, X);
    bool primed = false; // fragments of the upcoming stage are in f0
    uint32_t sb = lds0;  // ring slot of the stage computed next
    const float alpha = a.alpha, beta = a.beta;
    for (; w.valid(); w.advance()) {
        const int panel = w.id % X;
        const int n0 = (w.id / X) * BN;
        const int ntl = w.cur.x;

        float16_t acc[MB][NB];
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
#pragma unroll
                for (int i = 0; i < 16; i++) acc[mb][nb][i] = 0.f;

        // output row of every stored row of the panel (lane l of register q: row 64q + l); fetched
        // now so the loads are long done when the epilogue needs them
        int rid[(V + 63) / 64];
#pragma unroll
        for (int q = 0; q < (V + 63) / 64; q++) {
            const int r = min(q * 64 + lane, V - 1);
            rid[q] = a.row_ids ? a.row_ids[panel * V + r] : panel * V + r;
        }

        auto mma = [&](const Frags& f) __attribute__((always_inline)) {
#pragma unroll
            for (int mb = 0; mb < MB; mb++)
#pragma unroll
                for (int nb = 0; nb < NB; nb++)
                    acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.b[nb], f.a[mb], acc[mb][nb], 0, 0, 0);
        };
        // One stage: `cur` holds its fragments.  Reads the following stage's fragments into `nxt`
        // (that stage has landed once the barrier is passed; past the end of the stream the reads
        // hit a stale slot and are never used).  Padded k-steps have zero A values, so every step
        // is computed unconditionally and the loop body stays branch-free.
        auto stage = [&](Frags& cur, Frags& nxt) __attribute__((always_inline)) {
            sb = (sb + STAGE_BYTES == lds0 + Cfg::RING_BYTES) ? lds0 : sb + STAGE_BYTES;
            wg_barrier();
            // scheduling fences: the reads of the following fragments must be issued before the
            // MFMAs that overlap them, not sunk down to their first use
            load_frags(sb, nxt);
            __builtin_amdgcn_sched_barrier(0);
            mma(cur);
            __builtin_amdgcn_sched_barrier(0);
        };

        if (ntl > 0 && !primed) { // very first stage of the stream
            wg_barrier();
            load_frags(sb, f0);
            primed = true;
        }
        {
            int s = 0;
            for (; s + 1 < ntl; s += 2) {
                stage(f0, f1);
                stage(f1, f0);
            }
            if (s < ntl) {
                stage(f0, f1);
                f0 = f1;
            }
        }

        // ---- epilogue of this wave's V x WN sub-tile, one 32-row block at a time: accumulators
        // -> fp16 (one rounding) -> private LDS area (a lane holds 4 consecutive columns of one
        // row per 8-byte write) -> 16-byte pieces of whole row segments -> scattered rows of D
        constexpr int PR = WN / 8;       // 16-byte pieces per row of the sub-tile
        constexpr int RPS = 64 / PR;     // rows per store instruction
        constexpr int NIT = 32 / RPS;
        const int pc = lane % PR;
        const int col = n0 + cw * WN + pc * 8;
        const bool col_ok = col < N;
        const uint32_t wr = epi + (lane & 31) * Cfg::EPI_ROWB + (lane >> 5) * 8;
        const uint32_t rd = epi + (lane / PR) * Cfg::EPI_ROWB + pc * 16;
        // specialised on "alpha == 1" and "beta == 0" so that the common path has no branch (a
        // branch per piece would put a full wait at every join)
        auto epi_block = [&](int mb, auto scale, auto add_c) __attribute__((always_inline)) {
            constexpr bool SCALE = decltype(scale)::value, ADDC = decltype(add_c)::value;
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
#pragma unroll
                for (int ig = 0; ig < 4; ig++) {
                    half4_t h;
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        h[e] = (half_t)(SCALE ? acc[mb][nb][ig * 4 + e] * alpha : acc[mb][nb][ig * 4 + e]);
                    *(SHFLBW_LDS half4_t*)(uintptr_t)(wr + (nb * 32 + ig * 8) * 2) = h;
                }
            // all loads (LDS pieces, C when used), then all stores: the vector-memory counter is
            // in-order, a load issued behind a store would wait for the store to complete
            half8_t v[NIT], c[NIT];
            size_t off[NIT];
#pragma unroll
            for (int it = 0; it < NIT; it++) {
                v[it] = *(SHFLBW_LDS half8_t*)(uintptr_t)(rd + it * RPS * Cfg::EPI_ROWB);
                const int rr = mb * 32 + it * RPS + lane / PR;
                const int orow = __shfl(rid[rr >> 6], rr & 63);
                off[it] = (size_t)orow * N + col;
            }
            if (col_ok) {
                if (ADDC) {
#pragma unroll
                    for (int it = 0; it < NIT; it++) c[it] = *(const half8_t*)(a.C + off[it]);
#pragma unroll
                    for (int it = 0; it < NIT; it++)
#pragma unroll
                        for (int e = 0; e < 8; e++) v[it][e] = (half_t)((float)v[it][e] + beta * (float)c[it][e]);
                }
#pragma unroll
                for (int it = 0; it < NIT; it++) *(half8_t*)(a.D + off[it]) = v[it];
            }
        };
        // The row ids were loaded at the start of the tile.  Consume them here once: the wait the
        // compiler places is satisfied long ago, and afterwards the values are plain registers,
        // so no later use can make a block wait for the stores of the block before it.
#pragma unroll
        for (int q = 0; q < (V + 63) / 64; q++) asm volatile("" : "+v"(rid[q]));
        using T = std::true_type;
        using F = std::false_type;
        // one straight-line sequence over all 32-row blocks per specialisation
        if (beta == 0.f && alpha == 1.f) {
#pragma unroll
            for (int mb = 0; mb < MB; mb++) epi_block(mb, F{}, F{});
        } else if (beta == 0.f) {
#pragma unroll
            for (int mb = 0; mb < MB; mb++) epi_block(mb, T{}, F{});
        } else {
#pragma unroll
            for (int mb = 0; mb < MB; mb++) epi_block(mb, T{}, T{});
        }
    }
}

template <int V, int WN, int NCONS, int NPROD, int KT, int NSTAGE>
static hipError_t launch_ws(const SpmmLaunchArgs& a, hipStream_t stream)
{
    using Cfg = SpmmWsCfg<V, WN, NCONS, NPROD, KT, NSTAGE>;
    SpmmLaunchArgs b = a;
    b.n_tiles = (a.N + Cfg::BN - 1) / Cfg::BN;
    const int T = a.X * b.n_tiles;
    // one persistent workgroup per compute unit; fewer when there are fewer tiles (multiple of 8 XCDs)
    int grid = a.num_cus > 0 ? a.num_cus : 256;
    grid = (grid / 8) * 8;
    const int need = ((T + 7) / 8) * 8;
    if (grid > need) grid = need;
    hipLaunchKernelGGL((spmm_shflbw_ws_kernel<V, WN, NCONS, NPROD, KT, NSTAGE>), dim3(grid), dim3(Cfg::THREADS),
                       Cfg::LDS_BYTES, stream, b);
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
    // block 64
    SHFLBW_WS_VARIANT(64, 128, 4, 4, 16, 6),
    SHFLBW_WS_VARIANT(64, 128, 4, 4, 16, 5),
    SHFLBW_WS_VARIANT(64, 128, 4, 4, 16, 4),
    SHFLBW_VARIANT(64, 64, 4, 32, 3),
    SHFLBW_VARIANT(64, 64, 4, 32, 2),
    SHFLBW_VARIANT(64, 64, 4, 16, 4),
    SHFLBW_VARIANT(64, 128, 2, 32, 3),
    SHFLBW_VARIANT(64, 128, 4, 16, 3),
    SHFLBW_VARIANT(64, 64, 2, 32, 3),
    SHFLBW_VARIANT(64, 32, 4, 32, 3),
    // block 32
    SHFLBW_WS_VARIANT(32, 128, 4, 4, 16, 6),
    SHFLBW_VARIANT(32, 64, 4, 32, 3),
    SHFLBW_VARIANT(32, 128, 2, 32, 3),
    SHFLBW_VARIANT(32, 128, 4, 16, 3),
    SHFLBW_VARIANT(32, 64, 2, 32, 3),
    // block 128
    SHFLBW_VARIANT(128, 64, 4, 32, 3),
    SHFLBW_VARIANT(128, 32, 4, 32, 3),
};

const SpmmVariant* spmm_variants(int* count)
{
    *count = (int)(sizeof(g_variants) / sizeof(g_variants[0]));
    return g_variants;
}

} // namespace shflbw
