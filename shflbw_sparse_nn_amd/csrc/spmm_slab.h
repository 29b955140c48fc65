// Slab form of the SpMM for block height 32 and weights with few columns (K <= SLAB_MAX_K): a workgroup copies
// all K rows of a 64-column slab of B into LDS once and then runs many row panels over it, so a row of B crosses
// the path from the L2 to the compute unit once per workgroup instead of once per panel that keeps it.  What
// streams instead are the A fragments (64 bytes per kept vector, straight into registers) and the kept-column
// ids, stored for this kernel as LDS byte offsets of the slab rows.  A fetched value of A feeds 64 MACs here, a
// gathered value of B in the role-split kernel feeds V = 32.  Replaces, for such shapes, the reference's main
// loop (block_sparse/spmm/blockwise_kernel.h:108-294) like the role-split kernel does for all others.
//
// All eight waves are alike and independent once the slab is filled: a wave owns a contiguous run of panels and
// walks their kept vectors in batches of two MFMA steps (32 slots), NBUF batches (A fragments and offsets) in
// flight in registers, across panel boundaries.  Per step a wave reads its two B fragments from the rows the
// offsets name (transposing reads; the 32-byte units of row r are XOR-ed with (r / 2) % 4, and the host orders a
// panel's vectors so that the four rows one read touches lie in different bank groups) and issues two MFMAs.
// A panel's 32 x 64 result goes through the wave's private staging area to D like in the role-split kernel.
#pragma once
#include "kernel_common.h"
#include "spmm_launch.h"
#include "weight_internal.h"

namespace shflbw {

struct SpmmSlabCfg {
    static constexpr int V = 32;
    static constexpr int BN = 64;            // columns of the slab
    static constexpr int ROWB = BN * 2;      // bytes of a slab row
    static constexpr int NW = 8;             // waves of a workgroup
    static constexpr int THREADS = NW * 64;
    static constexpr int NB = BN / 32;
    static constexpr int NBUF = 8;           // batches a wave keeps in flight (even: the fragment sets alternate)
    static constexpr int FETCH_OPS = 3;      // loads per batch: two A fragments and a quad of offsets
    static constexpr int RID_REGS = 8;       // a wave's panels have at most RID_REGS * 64 rows
    static constexpr int EPI_ROWB = BN * 2 + 16;          // a staged row: all 64 columns and 16 bytes of padding
    static constexpr int EPI_WAVE_BYTES = 16 * EPI_ROWB;  // 16 rows at a time
    static constexpr int LDS_MAX = 160 * 1024;
    // rows of B the LDS holds beside the row of zeros and the staging areas, rounded down to the 8 rows of a copy
    static constexpr int MAX_K = ((LDS_MAX - NW * EPI_WAVE_BYTES) / ROWB - 1) / 8 * 8;
    static_assert(ROWB == SLAB_ROW_BYTES && MAX_K == SLAB_MAX_K, "the host packs the offsets for this geometry");
    static_assert(NBUF % 2 == 0 && (NBUF - 2) * FETCH_OPS < 64, "fragment sets alternate; vmcnt is a 6-bit counter");
    static constexpr int lds_bytes(int K) { return (((K + 7) & ~7) + 1) * ROWB + NW * EPI_WAVE_BYTES; }
};

__global__ void __launch_bounds__(SpmmSlabCfg::THREADS) spmm_shflbw_slab_kernel(SpmmLaunchArgs a)
{
    using Cfg = SpmmSlabCfg;
    constexpr int V = Cfg::V, NB = Cfg::NB, NBUF = Cfg::NBUF, ROWB = Cfg::ROWB, NW = Cfg::NW, BN = Cfg::BN;
    extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(SHFLBW_LDS char*)lds_raw;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int X = a.X, N = a.N, K = a.K;
    const int Kp = (K + 7) & ~7; // slab rows [K, Kp) are filler, row Kp is the row of zeros
    const uint32_t epi = lds0 + (uint32_t)(Kp + 1) * ROWB + wave * Cfg::EPI_WAVE_BYTES;
    const SHFLBW_CONST int2_t* desc = (const SHFLBW_CONST int2_t*)(uintptr_t)a.panel_desc;

    // jobs = (column tile, chunk of panels), chunk-minor; XCD x owns a contiguous range of them, so the
    // workgroups of an XCD share a few slabs of B and, over all chunks, the whole of A in their L2
    const int chunks = a.slab_chunks, ppc = (X + chunks - 1) / chunks;
    const int T = a.n_tiles * chunks;
    const int per = (T + 7) >> 3, xcd = blockIdx.x & 7, S = gridDim.x >> 3;
    const int job_end = min(T, (xcd + 1) * per);

    // lane constants of the transposing reads: a 16-lane group reads 4 rows x 32 bytes; lanes 16..31 the next
    // 32 bytes, lanes 32..63 the rows of slots 8..15
    const int li = lane & 15;
    const uint32_t lc = (uint32_t)((((lane >> 4) & 1) << 5) | ((li & 3) << 3));
    // which two slots (s, s + 4) of a step this lane addresses: pair number (lane / 32) * 4 + (lane % 16) / 4, 32 bytes
    // of offsets per pair and 64-slot group, 16 per batch
    const uint32_t pair32 = (uint32_t)(((lane >> 5) * 4 + (li >> 2)) * 32);
    const uint32_t lane16 = (uint32_t)lane * 16;
    // epilogue: a lane writes 4 columns (per 32-column block) of row lane % 16, reads 16-byte piece lane % 8 of row lane / 8
    const uint32_t wr = epi + (lane & 15) * Cfg::EPI_ROWB + (lane >> 5) * 8;
    const uint32_t rd = epi + (lane >> 3) * Cfg::EPI_ROWB + (lane & 7) * 16;
    const float alpha = a.alpha, beta = a.beta;

    struct Batch {
        half8_t a[2]; // A fragments of the two steps
        int4_t i;     // slab offsets: {step 0: slot s, s + 4; step 1: slot s, s + 4}
    };
    struct Frags {
        half8_t b[2][NB]; // B fragments of the two steps
    };

    bool first = true;
    for (int job = xcd * per + (blockIdx.x >> 3); job < job_end; job += S) {
        const int nt = job / chunks, ch = job - nt * chunks;
        const int n0 = nt * BN;
        // ---- the slab first, so that everything below runs while it is on its way: rows 8q .. 8q+7 per copy
        // instruction (lane l: row l / 8, 16-byte position l % 8)
        if (!first) __syncthreads(); // every wave is done with the slab of the job before
        first = false;
        for (int q = wave; q < (Kp >> 3); q += NW) {
            const int row = q * 8 + (lane >> 3);
            const int pp = lane & 7;
            const int lp = (((pp >> 1) ^ ((row >> 1) & 3)) << 1) | (pp & 1); // the piece of the row that belongs here
            int col = n0 + lp * 8;
            col = col < N ? col : n0; // columns past N are never stored
            const char* src = (const char*)a.B + (size_t)min(row, K - 1) * (uint32_t)a.ldb_bytes + (size_t)col * 2;
            global_to_lds_16B(src, lds0 + q * 1024);
        }
        if (wave == 0 && lane < ROWB / 16) {
            const half8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
            *(SHFLBW_LDS half8_t*)(uintptr_t)(lds0 + Kp * ROWB + lane * 16) = z;
        }

        const int P0 = min(X, ch * ppc), P1 = min(X, P0 + ppc);
        const int pwv = (P1 - P0 + NW - 1) / NW;
        const int pa = min(P1, P0 + wave * pwv), pb = min(P1, pa + pwv); // this wave's panels
        // output rows of all panels of this wave, 64 per register (the launcher keeps a wave's share within
        // RID_REGS * 64 rows): fetched here, complete when the slab is, so no epilogue waits for memory
        int ridreg[Cfg::RID_REGS];
#pragma unroll
        for (int q = 0; q < Cfg::RID_REGS; q++) {
            const int r = pa * V + q * 64 + lane;
            ridreg[q] = r;
            if (a.row_ids && r < pb * V) ridreg[q] = a.row_ids[r];
        }

        // ---- consumer side of the stream: panel p, n_left batches of it still to compute
        float16_t acc[NB];
        int p = pa, n_left = 0;
        auto open_panel = [&]() __attribute__((always_inline)) {
            n_left = (desc[p].x + 1) >> 1; // batches of two steps; an odd last step has zero weights behind it
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
#pragma unroll
                for (int i = 0; i < 16; i++) acc[nb][i] = 0.f;
        };
        // fp32 -> fp16 (one rounding) -> staging area, 16 rows of all 64 columns at a time -> rows of D, eight lanes
        // to a row: every store instruction writes whole 128-byte lines (half lines, written at different times,
        // cost 1.4 x the bytes at the memory side with streaming stores)
        auto epilogue = [&]() __attribute__((always_inline)) {
            const int i0 = (p - pa) * V; // first row of the panel among the wave's rows
            int rid = ridreg[0];
#pragma unroll
            for (int q = 1; q < Cfg::RID_REGS; q++) rid = (i0 >> 6) == q ? ridreg[q] : rid;
            const int col = n0 + (lane & 7) * 8;
#pragma unroll
            for (int hh = 0; hh < 2; hh++) { // rows 16 hh .. 16 hh + 15: held by the lanes with bit 4 equal to hh
                size_t roff[2];
#pragma unroll
                for (int it = 0; it < 2; it++)
                    roff[it] = (size_t)__shfl(rid, (i0 & 63) + hh * 16 + it * 8 + (lane >> 3)) * a.ldd;
                if (((lane >> 4) & 1) == hh) {
#pragma unroll
                    for (int nb = 0; nb < NB; nb++)
#pragma unroll
                        for (int ig = 0; ig < 4; ig++) {
                            half4_t h;
#pragma unroll
                            for (int e = 0; e < 4; e++) h[e] = (half_t)scaled(acc[nb][ig * 4 + e], alpha, beta != 0.f);
                            *(SHFLBW_LDS half4_t*)(uintptr_t)(wr + nb * 64 + ig * 16) = h;
                        }
                }
                // Lanes exchange data through the staging area.  For the compiler every lane is a thread of its own: it
                // may run the lanes that do not write through their reads first unless the wave is told to meet here.
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                half8_t v[2];
#pragma unroll
                for (int it = 0; it < 2; it++) v[it] = *(SHFLBW_LDS half8_t*)(uintptr_t)(rd + it * 8 * Cfg::EPI_ROWB);
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier(); // the next 16 rows overwrite what other lanes have just read
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                if (col < N) {
                    if (beta != 0.f) {
#pragma unroll
                        for (int it = 0; it < 2; it++) {
                            const half8_t c = *(const half8_t*)(a.C + roff[it] + col);
#pragma unroll
                            for (int e = 0; e < 8; e++) v[it][e] = (half_t)((float)v[it][e] + beta * (float)c[e]);
                        }
                    }
#pragma unroll
                    for (int it = 0; it < 2; it++) // streaming stores: D must not push A and the slabs out of the L2
                        __builtin_nontemporal_store(v[it], (half8_t*)(a.D + roff[it] + col));
                }
            }
        };
        // stores panel p (its steps are all done) and moves to the next panel that has steps; panels without
        // a kept vector are stored on the way (zeros, or beta * C).  False when the wave has no panel left.
        auto close_panels = [&]() __attribute__((always_inline)) {
            do {
                epilogue();
                if (++p >= pb) return false;
                open_panel();
            } while (n_left == 0);
            return true;
        };
        bool more = false;
        if (pa < pb) {
            open_panel();
            more = n_left > 0 || close_panels();
        }

        // ---- fetching side: batch number lpos (in units of 32 slots of the packed image) of panel lp is next;
        // a panel's batches are contiguous, the next panel starts at its own first 64-slot group.  Past the last
        // batch of the wave the same batch is fetched again and never used.
        int lp = p, lpos = 0, lend = 0;
        bool lrun = more;
        if (more) {
            const int2_t d = desc[p];
            lpos = d.y * 2;
            lend = lpos + ((d.x + 1) >> 1);
        }
        // The fetches are inline assembly, FETCH_OPS loads per batch, and the wait in front of a batch's use is
        // written by hand: with the loads and the epilogue's stores on one counter the compiler would wait for
        // everything in flight.  Loads return in order among themselves, so "at most n * FETCH_OPS operations
        // outstanding" means that the batch n fetches before the latest is complete, whatever the stores do.
        auto fetch = [&](Batch& b) __attribute__((always_inline)) {
            const char* A = (const char*)a.packedA + (size_t)lpos * (32 * V * 2);
            const char* I = (const char*)a.slab_ids + (size_t)(lpos >> 1) * 256 + (lpos & 1) * 16;
            asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(b.a[0]) : "v"(lane16), "s"(A));
            asm volatile("global_load_dwordx4 %0, %1, %2 offset:1024" : "=v"(b.a[1]) : "v"(lane16), "s"(A));
            asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(b.i) : "v"(pair32), "s"(I));
            if (lrun && ++lpos == lend) {
                lrun = false;
                lpos--; // stay on the last batch unless another panel follows
                while (++lp < pb) {
                    const int2_t d = desc[lp];
                    if (d.x > 0) {
                        lpos = d.y * 2;
                        lend = lpos + ((d.x + 1) >> 1);
                        lrun = true;
                        break;
                    }
                }
            }
        };
        // waits until the batch fetched NBUF - 2 fetches before the latest has arrived; the registers pass through
        // the statement so that nothing that reads them can be scheduled in front of the wait
        auto arrived = [&](Batch& b) __attribute__((always_inline)) {
            asm volatile("s_waitcnt vmcnt(%3)" : "+v"(b.a[0]), "+v"(b.a[1]), "+v"(b.i) : "n"((NBUF - 2) * Cfg::FETCH_OPS));
        };
        Batch buf[NBUF];
        if (more) {
#pragma unroll
            for (int j = 0; j < NBUF; j++) fetch(buf[j]);
        }

        // a wait the compiler sees: it also covers the row ids above, and must not be repeated at their use
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        asm volatile("" ::: "memory");
        __syncthreads();
        if (!more) continue;

        // B fragments: two transposing reads per fragment, from the rows the offsets name
        auto read_frags = [&](const Batch& b, Frags& f) __attribute__((always_inline)) {
            const int ids[4] = {b.i.x, b.i.y, b.i.z, b.i.w};
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const uint32_t alo = lds0 + ((uint32_t)ids[2 * h] ^ lc), ahi = lds0 + ((uint32_t)ids[2 * h + 1] ^ lc);
#pragma unroll
                for (int nb = 0; nb < NB; nb++) {
                    const half4_t l = lds_read_tr16(alo ^ (nb << 6));
                    const half4_t u = lds_read_tr16(ahi ^ (nb << 6));
                    f.b[h][nb] = __builtin_shufflevector(l, u, 0, 1, 2, 3, 4, 5, 6, 7);
                }
            }
        };
        auto mma = [&](const Frags& f, const Batch& b) __attribute__((always_inline)) {
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int nb = 0; nb < NB; nb++)
                    acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.b[h][nb], b.a[h], acc[nb], 0, 0, 0);
        };
        // the reads of a batch's fragments are issued one batch ahead of its MFMAs, also across the end of a panel
        Frags fr[2];
        asm volatile("s_waitcnt vmcnt(0)" : "+v"(buf[0].a[0]), "+v"(buf[0].a[1]), "+v"(buf[0].i)); // nothing reads them earlier
        read_frags(buf[0], fr[0]);
        for (bool done = false; !done;) {
#pragma unroll
            for (int j = 0; j < NBUF; j++) {
                arrived(buf[(j + 1) % NBUF]);
                read_frags(buf[(j + 1) % NBUF], fr[(j + 1) & 1]);
                mma(fr[j & 1], buf[j]);
                fetch(buf[j]);
                if (--n_left == 0 && !close_panels()) {
                    done = true;
                    break;
                }
            }
        }
    }
}

} // namespace shflbw
