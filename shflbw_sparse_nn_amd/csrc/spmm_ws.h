// Role-split (producer / consumer) building blocks of the persistent gfx950 kernels, shared by the SpMM
// kernel and the fused convolution kernel: LDS ring configuration, barrier protocol, tile walker, the consumer
// (transposing LDS reads, MFMA, per-wave epilogue) and the producer (global->LDS gathers of kept rows and A
// fragments).  Replaces, together with the kernels built from it, the reference's main loop and device
// primitives (block_sparse/spmm/blockwise_kernel.h:108-294, block_sparse/common/{mma,memcpy,swizzle,epilogue}.h).
#pragma once
#ifndef SHFLBW_EPI_LINES
#define SHFLBW_EPI_LINES 1
#endif
#include <type_traits>

#include "kernel_common.h"
#include "spmm_launch.h"

namespace shflbw {

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
    static constexpr int KSPS = KT / 16;                  // 16-slot steps per stage
    // 1 KiB A fragments per stage, contiguous in memory and LDS: V >= 32 has V/32 per 16-slot step
    // (32x32x16 tiles), V == 16 has one per 32-slot step (16x16x32 tiles)
    static constexpr int A_FRAGS = V == 16 ? KT / 32 : KSPS * MB;
    static constexpr int STAGE_BYTES = B_BYTES + A_FRAGS * 1024;
    static constexpr int RPW = KT / NPROD;                // gathered rows per producer and stage
    static constexpr int RPI = 1024 / ROWB;               // rows one 1 KiB copy instruction covers (BN = 256: two, BN = 128: four)
    static constexpr int CPW = RPW / RPI;                 // copies of B rows per producer and stage
    static constexpr int A_HI = A_FRAGS % NPROD;          // producers [0, A_HI) copy one more A fragment
    static constexpr int A_LO = A_FRAGS / NPROD;
    static constexpr int OPS = CPW + A_LO;                // copies per stage every producer issues at least
    static constexpr int EPI_ROWB = 32 * 2 + 16;
    static constexpr int EPI_ROWS = NCONS > 4 ? 16 : 32;  // rows of a 32 x 32 accumulator block staged at a time
    static constexpr int EPI_WAVE_BYTES = EPI_ROWS * EPI_ROWB;
    static constexpr int RING_BYTES = NSTAGE * STAGE_BYTES;
    static constexpr int LDS_BYTES = RING_BYTES + NCONS * EPI_WAVE_BYTES;
    static constexpr int THREADS = (NCONS + NPROD) * 64;
    // Workgroups a compute unit holds at once.  Two of them (their rings together fill the LDS, their registers
    // the file: at most 128 per wave) let one workgroup's epilogue stores run beside the other's stage loop.
    static constexpr int WGS_PER_CU = LDS_BYTES <= 79 * 1024 && THREADS <= 512 ? 2 : 1;
    static_assert((V % 32 == 0 || (V == 16 && KT == 32)) && WN % 32 == 0, "32x32x16 tiles, or 16x16x32 for V = 16");
    static_assert(BN == 512 || ((BN == 256 || BN == 128) && RPW == 8), "a 1 KiB copy instruction covers one gathered row, two or four");
    static_assert((KT == 16 || KT == 32) && (RPW == 4 || RPW == 8), "a 64-slot group is 4 or 2 stages; rows go in fours");
    static_assert(A_LO <= 2 && (A_LO == 0 || A_HI == 0), "the same number of A fragments for all producers that copy any");
    // A producer passes one barrier before every stage it issues.  The barrier in front of stage j is the
    // one after which the consumers no longer read stage j - NSTAGE, i.e. their barrier number j - (NSTAGE-2):
    // the consumers therefore pass NSTAGE - 2 extra barriers before their first one.
    static constexpr int START_BARRIERS = NSTAGE - 2;
    static_assert(THREADS <= 1024, "workgroup size limit");
    static_assert(NSTAGE >= 3, "one stage computed, one landed, one in flight");
    static_assert((NSTAGE - 3) * (CPW + (A_LO > 0 ? A_LO : 1)) < 64, "vmcnt is a 6-bit counter");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of a gfx950 compute unit");
};

__device__ __forceinline__ void wg_barrier()
{
    // bare barrier: no implied wait on outstanding global stores or copies
    asm volatile("s_barrier" ::: "memory");
}

// The NSTAGE - 1 barriers a producer passes after its last stage: number U of them waits until at most
// NSTAGE - 3 - U stages of OPS copies each are outstanding.
template <int U, int NSTAGE, int OPS>
__device__ __forceinline__ void producer_tail()
{
    if constexpr (U < NSTAGE - 1) {
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((NSTAGE - 3 - U > 0 ? NSTAGE - 3 - U : 0) * OPS));
        wg_barrier();
        producer_tail<U + 1, NSTAGE, OPS>();
    }
}

// Convolution over batch-innermost feature maps: the columns of the GEMM are the positions (i, j, b) of a padded
// output grid, a.dmap_row of them per grid row, of which the first a.dmap_valid are output values.  Maps a column
// (a multiple of 8; dmap_row and dmap_valid are multiples of 8 too) to its column in the compact output row and
// says whether it is one.
__device__ __forceinline__ bool output_column(const SpmmLaunchArgs& a, int& col)
{
    int q, r;
    fast_divmod(col, a.dmap_row, a.dmap_magic, q, r);
    col = q * a.dmap_valid + r;
    return r < a.dmap_valid;
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

// Consumer role of the role-split kernels: wave `cw` of NCONS owns the V x WN sub-tile at column
// cw*WN of every tile of the workgroup.  `Cfg` describes the LDS ring (stage size and count) and the
// per-wave epilogue area; the barrier protocol is: after START_BARRIERS start-up barriers, barrier
// number t (counted from 0) is passed once stage t of the workgroup's stage stream is complete in
// LDS; a consumer executes one barrier before its first stage and one more per stage.
// XCD_LOCAL: the result is read back by workgroups of the same XCD in the same launch and is stored without device
// scope (it stays in that XCD's L2); DMAP: see output_column().
template <typename Cfg, int V, int WN, int NCONS, bool XCD_LOCAL = false, bool DMAP = false>
__device__ __forceinline__ void ws_consumer(const SpmmLaunchArgs& a, uint32_t lds0, int lane, int cw, int id_first,
                                            int id_end, int S)
{
    constexpr int BN = Cfg::BN, MB = Cfg::MB, NB = Cfg::NB, ROWB = Cfg::ROWB;
    constexpr int STAGE_BYTES = Cfg::STAGE_BYTES, B_BYTES = Cfg::B_BYTES;
    const int N = a.N, X = a.X;
    const int li = lane & 15;
    uint32_t boff[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const int unit = (cw * WN + nb * 32) / 16 + ((lane >> 4) & 1);
        boff[nb] = (uint32_t)((8 * (lane >> 5) + (li >> 2)) * ROWB + ((unit ^ row_xor32(li >> 2)) << 5) + ((li & 3) << 3));
    }
    const uint32_t aoff = (uint32_t)(B_BYTES + lane * 16);
    const uint32_t epi = lds0 + Cfg::RING_BYTES + cw * Cfg::EPI_WAVE_BYTES;
    constexpr int KSPS = Cfg::KSPS; // k16 steps per LDS stage: rows 16h.. of the B area and A block h belong to step h
    static_assert(KSPS == 1 || KSPS == 2, "one or two k16 steps per LDS stage");

    struct Frags {
        half8_t a[MB], b[NB];
    };
    Frags f0, f1;
    auto load_frags = [&](uint32_t stage_base, int h, Frags& f) __attribute__((always_inline)) {
        const uint32_t sbase = stage_base + h * (16 * ROWB);
        const uint32_t abase = stage_base + aoff + h * (MB * 1024);
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
            f.a[mb] = *(SHFLBW_LDS half8_t*)(uintptr_t)(abase + mb * 1024);
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
        // Scheduling pattern for "load_frags(next); mma(current)": the MFMAs only need registers that
        // were filled a stage ago, so they start right away and the LDS reads are spread behind them,
        // RPM reads per MFMA; the remaining MFMAs follow the last read.
        auto interleave_reads = [&]() __attribute__((always_inline)) {
            constexpr int NRD = MB + 2 * NB, NMM = MB * NB, RPM = (NRD + NMM - 1) / NMM, G = (NRD + RPM - 1) / RPM;
            static_assert(G <= NMM, "every group of reads sits behind an MFMA");
#pragma unroll
            for (int i = 0; i < G; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
                __builtin_amdgcn_sched_group_barrier(0x100, RPM, 0); // LDS reads
            }
            if (NMM - G > 0) __builtin_amdgcn_sched_group_barrier(0x008, NMM - G, 0);
            __builtin_amdgcn_sched_barrier(0);
        };
        auto stage = [&](Frags& cur, Frags& nxt) __attribute__((always_inline)) {
            sb = (sb + STAGE_BYTES == lds0 + Cfg::RING_BYTES) ? lds0 : sb + STAGE_BYTES;
            wg_barrier();
            load_frags(sb, 0, nxt);
            mma(cur);
            interleave_reads();
        };

        if (ntl > 0 && !primed) { // very first stage of the stream
#pragma unroll
            for (int i = 0; i < Cfg::START_BARRIERS; i++) wg_barrier();
            wg_barrier();
            load_frags(sb, 0, f0);
            primed = true;
        }
        if (KSPS == 1) {
            int s = 0;
            for (; s + 1 < ntl; s += 2) {
                stage(f0, f1);
                stage(f1, f0);
            }
            if (s < ntl) {
                stage(f0, f1);
                f0 = f1;
            }
        } else {
            // two k16 steps per LDS stage: the odd step's fragments come from the stage already
            // present, only the step into the next stage passes a barrier.  A tile with an odd
            // number of steps computes one padded step (zero A values).
            for (int p = 0; p < (ntl + 1) >> 1; p++) {
                load_frags(sb, 1, f1);
                mma(f0);
                interleave_reads();
                stage(f1, f0);
            }
        }

        // ---- epilogue of this wave's V x WN sub-tile, one 32 x 32 accumulator block at a time:
        // fp16 (one rounding) -> private LDS area (a lane holds 4 consecutive columns of one row
        // per 8-byte write) -> 16-byte pieces of 64-byte row segments -> scattered rows of D.  The
        // staging area is small on purpose: the LDS belongs to the stage ring.
        constexpr int PR = 4;                 // 16-byte pieces per 32-column row segment
        constexpr int RPS = 64 / PR;          // rows per store instruction
        constexpr int ER = Cfg::EPI_ROWS;     // rows staged at a time: 32 (whole block) or 16 (half, by lanes)
        constexpr int NIT = ER / RPS;
        const int pc = lane % PR;
        const int col0 = n0 + cw * WN + pc * 8;
        const uint32_t wr = epi + (lane & (ER - 1)) * Cfg::EPI_ROWB + (lane >> 5) * 8;
        const uint32_t rd = epi + (lane / PR) * Cfg::EPI_ROWB + pc * 16;
        // specialised on "alpha == 1" and "beta == 0" so that the common path has no branch (a
        // branch per piece would put a full wait at every join)
        // Whole lines: with an even number of 32-column blocks, 16 rows of two neighbouring blocks are staged at a time
        // (rows of 128 bytes + 16) and eight lanes store one 128-byte line of a row: half as many write requests to the
        // L2s as with 64-byte row segments (cfg1 -2 %, 11 % at N = 16384, where every epilogue runs beside other
        // workgroups' gathers).  Not where two workgroups share a compute unit (128 registers per wave: it spills).
        constexpr bool LINES = SHFLBW_EPI_LINES && NB % 2 == 0 && 16 * (128 + 16) <= Cfg::EPI_WAVE_BYTES && Cfg::WGS_PER_CU == 1;
        constexpr int LROWB = 128 + 16;
        const uint32_t wrl = epi + (lane & 15) * LROWB + (lane >> 5) * 8;
        const uint32_t rdl = epi + (lane >> 3) * LROWB + (lane & 7) * 16;
        auto epi_lines = [&](int mb, auto scale, auto add_c) __attribute__((always_inline)) {
            constexpr bool SCALE = decltype(scale)::value, ADDC = decltype(add_c)::value;
#pragma unroll
            for (int np = 0; np < NB / 2; np++)
#pragma unroll
                for (int hh = 0; hh < 2; hh++) { // rows 16 hh .. 16 hh + 15 of the block: the lanes with bit 4 equal to hh
                    size_t roff[2];
#pragma unroll
                    for (int it = 0; it < 2; it++) {
                        const int rr = mb * 32 + hh * 16 + it * 8 + (lane >> 3);
                        roff[it] = (size_t)__shfl(rid[rr >> 6], rr & 63) * a.ldd;
                    }
                    if (((lane >> 4) & 1) == hh) {
#pragma unroll
                        for (int nb2 = 0; nb2 < 2; nb2++)
#pragma unroll
                            for (int ig = 0; ig < 4; ig++) {
                                half4_t h;
#pragma unroll
                                for (int e = 0; e < 4; e++) {
                                    const float x = acc[mb][np * 2 + nb2][ig * 4 + e];
                                    h[e] = (half_t)(SCALE ? scaled(x, alpha, ADDC) : x);
                                }
                                *(SHFLBW_LDS half4_t*)(uintptr_t)(wrl + nb2 * 64 + ig * 16) = h;
                            }
                    }
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                    half8_t v[2], c[2];
#pragma unroll
                    for (int it = 0; it < 2; it++) v[it] = *(SHFLBW_LDS half8_t*)(uintptr_t)(rdl + it * 8 * LROWB);
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier(); // the next 16 rows overwrite what other lanes have just read
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                    int col = n0 + cw * WN + np * 64 + (lane & 7) * 8;
                    bool keep = col < N;
                    if (DMAP) keep = keep && output_column(a, col);
                    if (keep) {
                        if (ADDC) {
#pragma unroll
                            for (int it = 0; it < 2; it++) c[it] = *(const half8_t*)(a.C + roff[it] + col);
#pragma unroll
                            for (int it = 0; it < 2; it++)
#pragma unroll
                                for (int e = 0; e < 8; e++)
                                    v[it][e] = (half_t)((float)v[it][e] + beta * (float)c[it][e]);
                        }
#pragma unroll
                        for (int it = 0; it < 2; it++) store_result_16B<!XCD_LOCAL>(a.D + roff[it] + col, v[it]);
                    }
                }
        };
        auto epi_block = [&](int mb, auto scale, auto add_c) __attribute__((always_inline)) {
            constexpr bool SCALE = decltype(scale)::value, ADDC = decltype(add_c)::value;
            if constexpr (LINES) {
                epi_lines(mb, scale, add_c);
                return;
            }
#pragma unroll
            for (int hh = 0; hh < 32 / ER; hh++) {
                size_t roff[NIT]; // element offset of the lane's output row, without the column
#pragma unroll
                for (int it = 0; it < NIT; it++) {
                    const int rr = mb * 32 + hh * ER + it * RPS + lane / PR;
                    roff[it] = (size_t)__shfl(rid[rr >> 6], rr & 63) * a.ldd;
                }
#pragma unroll
                for (int nb = 0; nb < NB; nb++) {
                    if (ER == 32 || ((lane >> 4) & 1) == hh) { // a lane holds row lane % 32 of the block
#pragma unroll
                        for (int ig = 0; ig < 4; ig++) {
                            half4_t h;
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                h[e] = (half_t)(SCALE ? scaled(acc[mb][nb][ig * 4 + e], alpha, ADDC) : acc[mb][nb][ig * 4 + e]);
                            *(SHFLBW_LDS half4_t*)(uintptr_t)(wr + ig * 16) = h;
                        }
                    }
                    // all loads (LDS pieces, C when used), then all stores: the vector-memory
                    // counter is in-order, a load issued behind a store would wait for the store
                    if constexpr (ER != 32) { // only half of the lanes wrote: the wave meets before any lane reads
                        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                        __builtin_amdgcn_wave_barrier();
                        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                    }
                    half8_t v[NIT], c[NIT];
#pragma unroll
                    for (int it = 0; it < NIT; it++)
                        v[it] = *(SHFLBW_LDS half8_t*)(uintptr_t)(rd + it * RPS * Cfg::EPI_ROWB);
                    int col = col0 + nb * 32;
                    bool keep = col < N;
                    if (DMAP) keep = keep && output_column(a, col);
                    if (keep) {
                        if (ADDC) {
#pragma unroll
                            for (int it = 0; it < NIT; it++) c[it] = *(const half8_t*)(a.C + roff[it] + col);
#pragma unroll
                            for (int it = 0; it < NIT; it++)
#pragma unroll
                                for (int e = 0; e < 8; e++)
                                    v[it][e] = (half_t)((float)v[it][e] + beta * (float)c[it][e]);
                        }
#pragma unroll
                        for (int it = 0; it < NIT; it++) store_result_16B<!XCD_LOCAL>(a.D + roff[it] + col, v[it]);
                    }
                }
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

// Consumer role for block height 16: 16x16x32 tiles, one 32-slot step per LDS stage, same barrier
// protocol and ring as ws_consumer.  Wave `cw` owns the 16 x WN sub-tile at column cw*WN.  A lane of
// the result holds output row lane % 16 and, per 16-column block, the 4 columns 4*(lane/16) + 0..3.
template <typename Cfg, int WN, int NCONS, bool XCD_LOCAL = false, bool DMAP = false>
__device__ __forceinline__ void ws_consumer16(const SpmmLaunchArgs& a, uint32_t lds0, int lane, int cw, int id_first,
                                              int id_end, int S)
{
    constexpr int V = 16, BN = Cfg::BN, NB = WN / 16, ROWB = Cfg::ROWB;
    constexpr int STAGE_BYTES = Cfg::STAGE_BYTES, B_BYTES = Cfg::B_BYTES;
    static_assert(Cfg::KSPS == 2 && WN % 64 == 0, "one 32-slot step per stage");
    const int N = a.N, X = a.X;
    const int li = lane & 15;
    uint32_t boff[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const int unit = (cw * WN + nb * 16) / 16;
        boff[nb] = (uint32_t)((8 * (lane >> 4) + (li >> 2)) * ROWB + ((unit ^ row_xor32(li >> 2)) << 5) + ((li & 3) << 3));
    }
    const uint32_t aoff = (uint32_t)(B_BYTES + lane * 16);
    const uint32_t epi = lds0 + Cfg::RING_BYTES + cw * Cfg::EPI_WAVE_BYTES;

    struct Frags {
        half8_t a, b[NB];
    };
    Frags f0, f1;
    auto load_frags = [&](uint32_t sbase, Frags& f) __attribute__((always_inline)) {
        f.a = *(SHFLBW_LDS half8_t*)(uintptr_t)(sbase + aoff);
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            const half4_t lo = lds_read_tr16(sbase + boff[nb]);
            const half4_t hi = lds_read_tr16(sbase + boff[nb] + 4 * ROWB);
            f.b[nb] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
    };

    TileWalker w;
    w.init(a.panel_desc, id_first, id_end, S, X);
    bool primed = false;
    uint32_t sb = lds0;
    const float alpha = a.alpha, beta = a.beta;
    for (; w.valid(); w.advance()) {
        const int panel = w.id % X;
        const int n0 = (w.id / X) * BN;
        const int ntl = (w.cur.x + 1) >> 1; // 32-slot steps

        float4_t acc[NB];
#pragma unroll
        for (int nb = 0; nb < NB; nb++) acc[nb] = float4_t{0.f, 0.f, 0.f, 0.f};
        const int srow = panel * V + li;
        const int orow = a.row_ids ? a.row_ids[srow] : srow;

        auto mma = [&](const Frags& f) __attribute__((always_inline)) {
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
                acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f.b[nb], f.a, acc[nb], 0, 0, 0);
        };
        auto stage = [&](Frags& cur, Frags& nxt) __attribute__((always_inline)) {
            sb = (sb + STAGE_BYTES == lds0 + Cfg::RING_BYTES) ? lds0 : sb + STAGE_BYTES;
            wg_barrier();
            load_frags(sb, nxt);
            __builtin_amdgcn_sched_barrier(0);
            mma(cur);
            __builtin_amdgcn_sched_barrier(0);
        };
        if (ntl > 0 && !primed) {
#pragma unroll
            for (int i = 0; i < Cfg::START_BARRIERS; i++) wg_barrier();
            wg_barrier();
            load_frags(sb, f0);
            primed = true;
        }
        int s = 0;
        for (; s + 1 < ntl; s += 2) {
            stage(f0, f1);
            stage(f1, f0);
        }
        if (s < ntl) {
            stage(f0, f1);
            f0 = f1;
        }

        // ---- epilogue: 16 rows x 64 columns at a time through the private LDS area (row of 128
        // bytes + 16), read back as 16-byte pieces of 128-byte row segments, 8 rows per store
        constexpr int EROWB = 64 * 2 + 16;
        static_assert(16 * EROWB <= Cfg::EPI_WAVE_BYTES, "epilogue staging area");
        const uint32_t wr = epi + li * EROWB + (lane >> 4) * 8;
        const uint32_t rd = epi + (lane >> 3) * EROWB + (lane & 7) * 16;
        size_t roff[2];
#pragma unroll
        for (int it = 0; it < 2; it++) roff[it] = (size_t)__shfl(orow, it * 8 + (lane >> 3)) * a.ldd;
#pragma unroll
        for (int h = 0; h < WN / 64; h++) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                half4_t hv;
#pragma unroll
                for (int e = 0; e < 4; e++) hv[e] = (half_t)scaled(acc[h * 4 + q][e], alpha, beta != 0.f);
                *(SHFLBW_LDS half4_t*)(uintptr_t)(wr + q * 32) = hv;
            }
            half8_t v[2];
#pragma unroll
            for (int it = 0; it < 2; it++) v[it] = *(SHFLBW_LDS half8_t*)(uintptr_t)(rd + it * 8 * EROWB);
            int col = n0 + cw * WN + h * 64 + (lane & 7) * 8;
            bool keep = col < N;
            if (DMAP) keep = keep && output_column(a, col);
            if (keep) {
                if (beta != 0.f) {
                    half8_t c[2];
#pragma unroll
                    for (int it = 0; it < 2; it++) c[it] = *(const half8_t*)(a.C + roff[it] + col);
#pragma unroll
                    for (int it = 0; it < 2; it++)
#pragma unroll
                        for (int e = 0; e < 8; e++) v[it][e] = (half_t)((float)v[it][e] + beta * (float)c[it][e]);
                }
#pragma unroll
                for (int it = 0; it < 2; it++) store_result_16B<!XCD_LOCAL>(a.D + roff[it] + col, v[it]);
            }
        }
    }
}

// Four gathered rows of B (ids k, wave-uniform) into four consecutive 1 KiB LDS rows starting
// ROW0 rows after sbp: per row one scalar multiply (id * row bytes fits 32 bits), one vector add
// onto the lane's column offset, and the copy; the add doubles as the wait state the copy needs
// after the write of M0.
template <int ROW0>
__device__ __forceinline__ void gather_rows4(int4_t k, uint32_t rowbytes, const uint32_t (&voff)[4], const void* B,
                                             uint32_t sbp)
{
    constexpr int O = ROW0 * 1024;
    uint32_t t0, t1, t2, t3, v0, v1, v2, v3;
    asm volatile("s_mul_i32 %[t0], %[k0], %[rb]\n\t"
                 "s_mul_i32 %[t1], %[k1], %[rb]\n\t"
                 "s_mul_i32 %[t2], %[k2], %[rb]\n\t"
                 "s_mul_i32 %[t3], %[k3], %[rb]\n\t"
                 "s_add_i32 m0, %[sbp], %[o0]\n\t"
                 "v_add_u32 %[v0], %[t0], %[l0]\n\t"
                 "global_load_lds_dwordx4 %[v0], %[B]\n\t"
                 "s_add_i32 m0, %[sbp], %[o1]\n\t"
                 "v_add_u32 %[v1], %[t1], %[l1]\n\t"
                 "global_load_lds_dwordx4 %[v1], %[B]\n\t"
                 "s_add_i32 m0, %[sbp], %[o2]\n\t"
                 "v_add_u32 %[v2], %[t2], %[l2]\n\t"
                 "global_load_lds_dwordx4 %[v2], %[B]\n\t"
                 "s_add_i32 m0, %[sbp], %[o3]\n\t"
                 "v_add_u32 %[v3], %[t3], %[l3]\n\t"
                 "global_load_lds_dwordx4 %[v3], %[B]"
                 : [t0] "=&s"(t0), [t1] "=&s"(t1), [t2] "=&s"(t2), [t3] "=&s"(t3), [v0] "=&v"(v0), [v1] "=&v"(v1),
                   [v2] "=&v"(v2), [v3] "=&v"(v3)
                 : [k0] "s"(k.x), [k1] "s"(k.y), [k2] "s"(k.z), [k3] "s"(k.w), [rb] "s"(rowbytes), [l0] "v"(voff[0]),
                   [l1] "v"(voff[1]), [l2] "v"(voff[2]), [l3] "v"(voff[3]), [B] "s"(B), [sbp] "s"(sbp), [o0] "n"(O),
                   [o1] "n"(O + 0x400), [o2] "n"(O + 0x800), [o3] "n"(O + 0xc00)
                 : "m0", "scc");
}

// Producer role: wave `pw` of NPROD issues its share of every stage of the workgroup's tile list (ids
// id_first, id_first + S, ... < id_end; id = column tile * X + panel).
template <typename Cfg, int V, int NCONS, int NPROD, int KT, int NSTAGE>
__device__ __forceinline__ void ws_producer(const SpmmLaunchArgs& a, uint32_t lds0, int lane, int pw, int id_first,
                                            int id_end, int S)
{
    constexpr int BN = Cfg::BN, RPW = Cfg::RPW;
    constexpr int STAGE_BYTES = Cfg::STAGE_BYTES, B_BYTES = Cfg::B_BYTES;
    const int N = a.N, X = a.X;
    // =========================== producer ===========================
    // A wave issues roughly one instruction every five to six cycles, whatever the kind, and
    // the workgroup advances one stage per producer round: the round is kept to the copies,
    // one multiply and one add per gathered row, and a handful of scalar bookkeeping.
    //  * addresses are a 64-bit base in scalar registers plus a 32-bit per-lane offset; the
    //    row offset id * row bytes goes into the lane offset (B must be smaller than 4 GiB);
    //  * the stream is walked group by group (64 slots = up to four stages of one tile); the
    //    16 ids a producer needs for the next group are fetched by one scalar load at the
    //    start of the current group and first touched when that group is finished, several
    //    hundred cycles later, so the full wait a scalar load needs never stalls.
    const uint32_t rowbytes = (uint32_t)a.ldb_bytes;
    const SHFLBW_CONST int2_t* desc = (const SHFLBW_CONST int2_t*)(uintptr_t)a.panel_desc;
    constexpr int KSPS = Cfg::KSPS;
    constexpr int NSG = 64 / KT; // stages per group
    // ids of a group for this producer, as int4 number q.  Four rows per producer and stage:
    // stage j uses int4 j - with 16-row stages from the producer-major copy [16 pw + 4 j + r],
    // with 32-row stages (8 producers) from slots 32 j + 4 pw + r of the slot-ordered array.
    // Eight rows per producer and stage (32-row stages, 4 producers): stage j uses int4 2j and
    // 2j+1, slots 32 j + 8 pw + r.
    auto group_ptr = [&](int group, int q) __attribute__((always_inline)) {
        const int* base = KT == 16   ? a.kidx_pm + (size_t)group * 64 + pw * 16 + q * 4
                          : RPW == 8 ? a.kidx + (size_t)group * 64 + (q >> 1) * 32 + pw * 8 + (q & 1) * 4
                                     : a.kidx + (size_t)group * 64 + (q & 1) * 32 + pw * 4;
        return (const SHFLBW_CONST int4_t*)(uintptr_t)base;
    };

    // -- cursor over the non-empty tiles of this workgroup
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
    if (cur.x == 0) return; // no stage at all: the consumers pass no barrier either
    bool have_next = false;   // `nxt` describes the tile after `cur`

    // -- per-tile lane offsets: copy j of a stage fills row pw*RPW + j (swizzle key j % 4); the
    // lane's 16-byte piece lands at physical position `lane`, so it fetches logical piece lc
    // -- direction: the workgroups of an XCD walk their tiles in step, all over the same columns of B.
    // Every second tile of a workgroup is walked from its last stage to its first, so that a round of
    // tiles starts on the rows of B the round before touched last (what is left of them in the
    // XCD's L2) instead of on the ones it evicted first.  Only the order of the stages changes; inside
    // a stage rows and A fragments stay as packed, and the consumers take the stages as they come.
    bool rev = false;
    uint32_t voff[4];
    uint32_t va = 0;             // lane offset of this wave's A fragment of the next stage
    uint32_t dva = 0;            // ... and its step from stage to stage
    const char* tileA = nullptr; // A fragments of the current tile
    // Padding slots (id -1, only in the last group of a panel) gather from the row of zeros: its address less the
    // tile's column offset, so that the lane offsets voff[] of the tile apply to it as they do to a row of B.
    const char* zb = nullptr;
    bool pad_group = false;      // the group being issued may hold padding slots
    auto open_tile = [&]() __attribute__((always_inline)) {
        const int n0 = (id / X) * BN;
        tileA = (const char*)a.packedA + (size_t)cur.y * (64 * V * 2);
        zb = (const char*)a.zero_row - (size_t)n0 * 2;
        const int nst = (cur.x + KSPS - 1) / KSPS;
        va = pw * 1024 + lane * 16 + (rev ? (uint32_t)(nst - 1) * (Cfg::A_FRAGS * 1024) : 0u);
        dva = rev ? (uint32_t) - (Cfg::A_FRAGS * 1024) : (uint32_t)(Cfg::A_FRAGS * 1024);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            // one copy = one row of 64 pieces (swizzle key j % 4), or the rows 2j and 2j + 1 of this
            // producer, 32 pieces each, in the lower and the upper half of the wave, or the rows 4j .. 4j + 3,
            // 16 pieces each, in the four quarters of the wave
            const int key = Cfg::RPI == 1 ? j : Cfg::RPI == 2 ? (2 * j + (lane >> 5)) & 3 : lane >> 4;
            const int pc = Cfg::RPI == 1 ? lane : Cfg::RPI == 2 ? lane & 31 : lane & 15;
            const int lc = ((((pc >> 1) ^ row_xor32(key))) << 1) | (pc & 1);
            const int col = n0 + lc * 8;
            int c = col < N ? col : n0; // columns past N are never stored; any valid column of the tile will do
            voff[j] = (uint32_t)c * 2;
        }
    };

    // -- everything on the stage cadence, specialised on whether this producer also copies an A
    // fragment per stage: its copies per stage are then a compile-time number and the waits exact
    auto run = [&](auto has_a_tag) __attribute__((always_inline)) {
        constexpr bool HAS_A = decltype(has_a_tag)::value;
        constexpr int NA = HAS_A ? (Cfg::A_LO > 0 ? Cfg::A_LO : 1) : 0; // A fragments per stage of this producer
        constexpr int MYOPS = Cfg::CPW + NA;                            // its copies per stage
        // ring position of the next stage: LDS address of this wave's rows
        uint32_t sbp = lds0 + pw * RPW * Cfg::ROWB;
        // this wave's first A fragment slot relative to sbp (a second one lies NPROD fragments further)
        const int a_rel = B_BYTES + pw * 1024 - pw * RPW * Cfg::ROWB;
        // One stage, branch-free: the barrier in front of stage j tells that the consumers are done with
        // the ring slot it overwrites; before arriving there the stage the consumers read next (issued
        // NSTAGE - 2 stages ago) must have landed, NSTAGE - 3 younger stages stay in flight.  In front
        // of the first stages nothing is outstanding and the wait falls through.
        auto stage = [&](int4_t ka, int4_t kb) __attribute__((always_inline)) {
            __builtin_amdgcn_s_waitcnt(vmcnt_imm((NSTAGE - 3) * MYOPS));
            wg_barrier();
            if (pad_group) {
                // same copies, one at a time, each from B or from the row of zeros
                const int ks[8] = {ka.x, ka.y, ka.z, ka.w, kb.x, kb.y, kb.z, kb.w};
                if (Cfg::RPI == 1) {
                    auto row = [&](auto jj) __attribute__((always_inline)) {
                        constexpr int j = decltype(jj)::value;
                        const bool pad = ks[j] < 0;
                        global_to_lds_16B_sbase<j * 0x400>(pad ? (const void*)zb : (const void*)a.B,
                                                           (pad ? 0u : (uint32_t)ks[j] * rowbytes) + voff[j & 3], sbp);
                    };
                    row(std::integral_constant<int, 0>{});
                    row(std::integral_constant<int, 1>{});
                    row(std::integral_constant<int, 2>{});
                    row(std::integral_constant<int, 3>{});
                    if (RPW == 8) {
                        row(std::integral_constant<int, 4>{});
                        row(std::integral_constant<int, 5>{});
                        row(std::integral_constant<int, 6>{});
                        row(std::integral_constant<int, 7>{});
                    }
                } else if (Cfg::RPI == 2) {
                    const bool hi = lane >= 32;
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const int k = hi ? ks[2 * j + 1] : ks[2 * j];
                        const char* src = k < 0 ? zb : (const char*)a.B + (size_t)((uint32_t)k * rowbytes);
                        global_to_lds_16B(src + voff[j], sbp + j * 0x400);
                    }
                } else {
                    const int q = lane >> 4; // the quarter of the wave: row 4j + q of the producer
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        const int k = q == 0 ? ks[4 * j] : q == 1 ? ks[4 * j + 1] : q == 2 ? ks[4 * j + 2] : ks[4 * j + 3];
                        const char* src = k < 0 ? zb : (const char*)a.B + (size_t)((uint32_t)k * rowbytes);
                        global_to_lds_16B(src + voff[j], sbp + j * 0x400);
                    }
                }
            } else if (Cfg::RPI == 1) {
                gather_rows4<0>(ka, rowbytes, voff, a.B, sbp);
                if (RPW == 8) gather_rows4<4>(kb, rowbytes, voff, a.B, sbp);
            } else if (Cfg::RPI == 4) {
                // 256-byte rows: quarter q of the wave fetches row 4j + q
                const int q = lane >> 4;
                const int k0 = q == 0 ? ka.x : q == 1 ? ka.y : q == 2 ? ka.z : ka.w;
                const int k1 = q == 0 ? kb.x : q == 1 ? kb.y : q == 2 ? kb.z : kb.w;
                global_to_lds_16B_sbase<0x000>(a.B, (uint32_t)k0 * rowbytes + voff[0], sbp);
                global_to_lds_16B_sbase<0x400>(a.B, (uint32_t)k1 * rowbytes + voff[1], sbp);
            } else {
                // 512-byte rows: the lower half of the wave fetches row 2j, the upper half row 2j + 1
                const bool hi = lane >= 32;
                global_to_lds_16B_sbase<0x000>(a.B, (uint32_t)(hi ? ka.y : ka.x) * rowbytes + voff[0], sbp);
                global_to_lds_16B_sbase<0x400>(a.B, (uint32_t)(hi ? ka.w : ka.z) * rowbytes + voff[1], sbp);
                global_to_lds_16B_sbase<0x800>(a.B, (uint32_t)(hi ? kb.y : kb.x) * rowbytes + voff[2], sbp);
                global_to_lds_16B_sbase<0xc00>(a.B, (uint32_t)(hi ? kb.w : kb.z) * rowbytes + voff[3], sbp);
            }
            if (HAS_A)
                asm volatile("s_add_i32 m0, %[sbp], %[arel]\n\t"
                             "s_nop 0\n\t"
                             "global_load_lds_dwordx4 %[va], %[A]"
                             :
                             : [sbp] "s"(sbp), [arel] "s"(a_rel), [va] "v"(va), [A] "s"(tileA)
                             : "m0", "scc");
            if (NA == 2) // its second fragment, NPROD fragments further in memory and in the stage
                asm volatile("s_add_i32 m0, %[sbp], %[arel]\n\t"
                             "s_nop 0\n\t"
                             "global_load_lds_dwordx4 %[va], %[A]"
                             :
                             : [sbp] "s"(sbp), [arel] "s"(a_rel + NPROD * 1024), [va] "v"(va), [A] "s"(tileA + NPROD * 1024)
                             : "m0", "scc");
            va += dva;
            sbp = (sbp + STAGE_BYTES == lds0 + pw * RPW * Cfg::ROWB + Cfg::RING_BYTES) ? sbp - (NSTAGE - 1) * STAGE_BYTES
                                                                                        : sbp + STAGE_BYTES;
        };

        // -- groups: gc* = ids of the group being issued, gn* = ids of the group after it in the
        // stream, requested at the start of this group and first touched at its end
        int4_t gc0 = *group_ptr(cur.y, 0), gc1 = *group_ptr(cur.y, 1), gc2 = *group_ptr(cur.y, 2),
               gc3 = *group_ptr(cur.y, 3);
        open_tile();
        // the ids are consumed here once, so that the loop below starts without a pending scalar
        // load on them (it would otherwise wait, together with the loads of the following group,
        // at the top of every iteration)
        asm volatile("" : : "s"(gc0.x), "s"(gc1.x), "s"(gc2.x), "s"(gc3.x));
        // stages of one group, first to last or last to first; a whole group is straight-line code
        auto issue_group = [&](int n, bool back) __attribute__((always_inline)) {
            if (KT == 16) { // four stages per group, stage j uses int4 j
                if (n == NSG && !back) {
                    stage(gc0, gc0);
                    stage(gc1, gc1);
                    stage(gc2, gc2);
                    stage(gc3, gc3);
                } else if (n == NSG) {
                    stage(gc3, gc3);
                    stage(gc2, gc2);
                    stage(gc1, gc1);
                    stage(gc0, gc0);
                } else if (!back) {
                    stage(gc0, gc0);
                    if (n > 1) stage(gc1, gc1);
                    if (n > 2) stage(gc2, gc2);
                } else {
                    if (n > 2) stage(gc2, gc2);
                    if (n > 1) stage(gc1, gc1);
                    stage(gc0, gc0);
                }
            } else if (RPW == 8) { // two stages per group, stage j uses int4 2j and 2j + 1
                if (n == NSG && !back) {
                    stage(gc0, gc1);
                    stage(gc2, gc3);
                } else if (n == NSG) {
                    stage(gc2, gc3);
                    stage(gc0, gc1);
                } else {
                    stage(gc0, gc1);
                }
            } else { // two stages per group, stage j uses int4 j
                if (n == NSG && !back) {
                    stage(gc0, gc0);
                    stage(gc1, gc1);
                } else if (n == NSG) {
                    stage(gc1, gc1);
                    stage(gc0, gc0);
                } else {
                    stage(gc0, gc0);
                }
            }
        };
        auto groups_of = [&](int k16_steps) __attribute__((always_inline)) {
            return ((k16_steps + KSPS - 1) / KSPS + NSG - 1) / NSG;
        };
        while (true) {
            const int nst = (cur.x + KSPS - 1) / KSPS; // stages of this tile
            const int ngroups = (nst + NSG - 1) / NSG;
            if (!have_next && ngroups == 1) { // the first group already needs to know what follows
                find_next();
                have_next = true;
            }
            for (int q = 0; q < ngroups; q++) {
                const int g = rev ? ngroups - 1 - q : q;                              // group of the tile
                const int n = g + 1 == ngroups ? nst - NSG * (ngroups - 1) : NSG;     // its stages
                // the group that follows in the stream (the next tile may be walked the other way round); at
                // the very end simply this one again
                int gnext = cur.y + (rev ? g - 1 : g + 1);
                if (q + 1 == ngroups)
                    gnext = nxt.x > 0 ? nxt.y + ((rev != (a.alternate != 0)) ? groups_of(nxt.x) - 1 : 0) : cur.y + g;
                const int4_t gn0 = *group_ptr(gnext, 0), gn1 = *group_ptr(gnext, 1), gn2 = *group_ptr(gnext, 2),
                             gn3 = *group_ptr(gnext, 3);
                pad_group = g + 1 == ngroups;
                issue_group(n, rev);
                if (!have_next) { // deferred from the start: not needed before the first copies are out
                    find_next();
                    have_next = true;
                }
                gc0 = gn0, gc1 = gn1, gc2 = gn2, gc3 = gn3;
            }
            if (nxt.x == 0) break;
            id = idn, cur = nxt;
            if (a.alternate) rev = !rev;
            find_next();
            open_tile();
        }
        // -- tail: the consumers pass NSTAGE - 1 more barriers.  Barrier number u of them stands in front
        // of the stage issued NSTAGE - 2 - u stages ago (NSTAGE - 3 - u younger ones may be in flight);
        // the last one only releases the consumers' final stage.
        producer_tail<0, NSTAGE, MYOPS>();
    };
    if (Cfg::A_LO > 0 || pw < Cfg::A_HI)
        run(std::true_type{});
    else
        run(std::false_type{});
}

} // namespace shflbw
