// Device-side building blocks shared by the gfx950 SpMM and SpConv kernels.
// Wave = 64 lanes.  Matrix cores are driven as D' = Bfrag x Afrag (activation rows,
// weight columns), so one lane ends up holding consecutive output columns of one
// output row, which makes the fp16 conversion and the LDS-staged row scatter cheap.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace shflbw {

typedef _Float16 half_t;
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef int int2_t __attribute__((ext_vector_type(2)));
typedef int int4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

#define SHFLBW_LDS __attribute__((address_space(3)))
#define SHFLBW_INLINE_LAMBDA __attribute__((always_inline))
// read-only data addressed uniformly by a wave: loads through this address space are scalar
#define SHFLBW_CONST __attribute__((address_space(4)))

// s_waitcnt immediate that waits only for the vector-memory counter to drop to n
// (gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt_hi[15:14]).
__device__ __forceinline__ constexpr int vmcnt_imm(int n)
{
    return (n & 0xf) | (0x7 << 4) | (0xf << 8) | ((n >> 4) << 14);
}

// XOR mask, in 32-byte units, applied to the position of a piece inside its LDS row.
// Rows r, r+1, r+2, r+3 (r % 4 == 0) read by one transposing load then touch eight
// distinct 32-byte bank groups for the two neighbouring column halves, both when the
// LDS serves 128 B and when it serves 256 B per clock.
__device__ __forceinline__ constexpr int row_xor32(int row_mod4)
{
    return 2 * row_mod4 + (row_mod4 >> 1); // 0, 2, 5, 7
}

// Transposing LDS load: inside each group of 16 lanes, lane i supplies the address of
// four consecutive halves of row i/4 (piece i%4 of a 4 x 16 block) and receives column
// i of that block (rows 0..3).
__device__ __forceinline__ half4_t lds_read_tr16(uint32_t byte_addr)
{
    short4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((SHFLBW_LDS short4_t*)(uintptr_t)byte_addr);
    return __builtin_bit_cast(half4_t, v);
}

// One wave instruction moves 64 x 16 bytes from per-lane global addresses to 1 KiB of
// consecutive LDS starting at the wave-uniform byte address `lds_base` (lane l lands at
// +16 l).  Issued as inline assembly on purpose: the compiler then neither counts it nor
// orders LDS reads after it, so the kernels place exact `s_waitcnt vmcnt(n)` themselves
// and keep several stages in flight.  M0 carries the LDS address; one wait state is
// required between the scalar write of M0 and the load.  No "memory" clobber: the
// statement is ordered against barriers and explicit waits because it is volatile, and
// a clobber would stop the compiler from using scalar loads for read-only metadata.
__device__ __forceinline__ void global_to_lds_16B(const void* gptr, uint32_t lds_base)
{
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gptr), "s"(lds_base)
                 : "m0");
}

// Same copy with the address split into a wave-uniform 64-bit base (scalar registers) and a
// per-lane 32-bit byte offset: no vector-ALU address arithmetic is needed per copy, which
// matters because vector-ALU work of one wave competes with the MFMAs of its SIMD neighbour.
template <int LDS_IMM>
__device__ __forceinline__ void global_to_lds_16B_sbase(const void* sbase, uint32_t lane_off, uint32_t lds_base)
{
    // LDS address = lds_base + LDS_IMM, formed directly in M0
    asm volatile("s_add_i32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(lane_off), "s"(sbase), "s"(lds_base), "n"(LDS_IMM)
                 : "m0", "scc");
}

// s_waitcnt on the vector-memory counter that the compiler also treats as a memory fence, for
// waits that publish LDS contents written by copies the compiler does not know about
template <int N>
__device__ __forceinline__ void wait_vmcnt_fence()
{
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// 16-byte store of result values.
// DEVICE_SCOPE (the SpMM proper): the line is written through to memory instead of staying dirty in the XCD's L2,
// where its later eviction would fall into the gathers of the next tile.  The compiler has no form of this store,
// so it is inline assembly, and the compiler's hazard pass does not look inside: a vector-ALU write to the data
// registers directly behind a store of more than 8 bytes needs wait states, which the s_nop supplies (the
// registers are free for reuse after the statement).
// Otherwise (results that workgroups of the same XCD read back in the same launch): an ordinary store, the line
// stays in the XCD's L2.
template <bool DEVICE_SCOPE = true>
__device__ __forceinline__ void store_result_16B(half_t* p, half8_t v)
{
    if constexpr (DEVICE_SCOPE)
        asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
    else
        asm volatile("global_store_dwordx4 %0, %1, off\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
}

// alpha * acc as the reference's `d * alpha + c * beta` leaves it (spmm/blockwise_format.h:307): without a C term the sum
// is `d * alpha + (+0)`, which turns a product of -0 (a zero accumulator under a negative alpha) into +0; with a C term
// the product goes on unchanged (x + (-0) == x for every x).  One fused multiply-add either way.
__device__ __forceinline__ float scaled(float acc, float alpha, bool c_term_follows)
{
    return __builtin_fmaf(acc, alpha, c_term_follows ? -0.f : 0.f);
}

// Words that workgroups of one launch count in (queues, arrival counts) are kept one cache line apart: atomics on
// one line are served one after the other (about 11 ns each with every compute unit taking part).
constexpr int SYNC_LINE = 64; // ints

// Counting between the workgroups of ONE XCD.  The compute units of an XCD share its L2, where every atomic is
// executed; these atomics carry no device scope, so they stay in that L2 instead of going to memory (about 220 ns a
// round trip on an idle chip; atomics on one cache line are served one after the other, about 11 ns each).  Only
// workgroups that run on the same XCD may use a given word.  The read is an atomic too (maximum with a value below
// every count): an atomic is never served by the compute unit's own cache, and a load that carries device scope,
// which is not either, turned out slower than the atomic once the line is being counted in (the waits of the
// fused convolution took 3.0 instead of 1.8 us with it).
__device__ __forceinline__ int xcd_fetch_add(int* p, int v)
{
    return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ int xcd_fetch_or(int* p, int v)
{
    return __hip_atomic_fetch_or(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ int xcd_read(int* p)
{
    return __hip_atomic_fetch_max(p, -1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// the XCD this wave runs on (0 .. 7 on an MI355X in its single-partition mode)
__device__ __forceinline__ int xcd_id()
{
    unsigned v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
    return (int)(v & 15u);
}

// n / d and n % d for n < 2^31 with magic = floor(2^32 / d) computed on the host (udiv_magic below): the product's high word
// is the quotient or one less, one correction step settles it; an integer division by a run-time value costs about
// forty instructions, and the layout phases do several per 16-byte piece
__device__ __forceinline__ void fast_divmod(int n, int d, unsigned magic, int& q, int& r)
{
    q = (int)__umulhi((unsigned)n, magic);
    r = n - q * d;
    if (r >= d) {
        q++;
        r -= d;
    }
}

// floor(2^32 / d) for fast_divmod
inline unsigned udiv_magic(int d) { return d <= 1 ? 0xffffffffu : (unsigned)(0x100000000ull / (unsigned)d); }

// Logical workgroup id for a 1-D grid: the hardware deals consecutive workgroup ids
// round-robin to the 8 XCDs; this makes consecutive *logical* ids share an XCD (and
// therefore its L2), so tiles that gather the same activation slab run side by side.
__device__ __forceinline__ int xcd_local_id(int wg, int total)
{
    const int per = total >> 3;
    return (wg < (per << 3)) ? (wg & 7) * per + (wg >> 3) : wg;
}

} // namespace shflbw
