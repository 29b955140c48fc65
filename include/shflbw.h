/*
 * shflbw.h -- C ABI of the MI355X (gfx950) Shfl-BW sparse inference library.
 *
 * Shfl-BW weights: an M x K fp16 matrix stored as row panels of `brow` (V) rows;
 * inside a panel only some V x 1 column vectors are kept; an optional row
 * permutation says which logical output row each stored row is.  Two
 * operators: SpMM  D = A_sparse * B_dense (+ C)  and SpConv2D (implicit GEMM).
 *
 * Every entry point below replaces one piece of the host API of the reference
 * library (hgyhungry/ShflBW_Sparse_NN, paths relative to its root); the
 * citation says which.  Plain pointers and sizes only; all functions return a
 * shflbw_status (0 = success) and never terminate the process.
 *
 * fp16 data crosses this boundary as raw IEEE binary16 bit patterns
 * (uint16_t on the host, 2-byte elements on the device).
 */
#ifndef SHFLBW_H
#define SHFLBW_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum shflbw_status {
    SHFLBW_OK = 0,
    SHFLBW_ERR_INVALID = 1,     /* null pointer / bad argument */
    SHFLBW_ERR_SHAPE = 2,       /* shape precondition violated (nrow % brow, N % 8, ...) */
    SHFLBW_ERR_STATE = 3,       /* object not initialised / not synced to the device */
    SHFLBW_ERR_HIP = 4,         /* a HIP runtime call failed; see shflbw_last_error() */
    SHFLBW_ERR_UNSUPPORTED = 5, /* block size / layout without a kernel */
    SHFLBW_ERR_FORMAT = 6,      /* malformed text dump or inconsistent arrays */
    SHFLBW_ERR_CAPACITY = 7     /* caller buffer too small */
} shflbw_status;

/* Human readable text for a status; and the detail of the last failure on this thread. */
const char* shflbw_status_string(int status);
const char* shflbw_last_error(void);

/* ------------------------------------------------------------------------- *
 * Mask generator.  Replaces block_sparse/util/random_mask.h:4-10
 * (random_mask, 12- and 9-argument forms; util/random_mask.cc:10-67).
 * indptr: X+1 ints (X = nrow/brow); indices: `indices_cap` ints.
 * ------------------------------------------------------------------------- */
int shflbw_random_mask_ex(int nrow, int ncol, int brow, int bcol, float block_density,
                          int block_divisor, int block_padding, unsigned seed,
                          int* nnzb, int* padded_nnzb, int* indptr, int* indices, size_t indices_cap);
int shflbw_random_mask(int nrow, int ncol, int brow, int bcol, float block_density, unsigned seed,
                       int* nnzb, int* indptr, int* indices, size_t indices_cap);

/* ------------------------------------------------------------------------- *
 * Weight container.  Replaces BlockwiseSpMatrix<half>
 * (block_sparse/spmm/blockwise_format.h:13-68) and BlockwiseSpFilter<half>
 * (block_sparse/spconv/blockwise_format.h:17-27).  The object owns its host
 * arrays and its device buffers; shflbw_weight_destroy frees both
 * (blockwise_format.h:48-58).
 * ------------------------------------------------------------------------- */
typedef struct shflbw_weight shflbw_weight;

typedef struct shflbw_weight_info {
    int nrow, ncol, nnzb, brow, bcol;
    float density;
    unsigned seed;
    int row_permute;
    int initialized, device_synced;
    int F, R, S, C; /* filter view (nrow = F, ncol = R*S*C); all 0 for a plain matrix */
} shflbw_weight_info;

/* Device pointers of a synced weight: DeviceRef, blockwise_format.h:35-42. */
typedef struct shflbw_device_ref {
    void* meta;                 /* indptr | indices*bcol | row_permute_ids, 8-int aligned sections */
    void* data;                 /* values, verbatim */
    const int* csb_indptr;      /* X+1 */
    const int* csb_indices;     /* nnzb, pre-multiplied by bcol */
    const int* row_permute_ids; /* nrow, or NULL when not permuted */
    const void* csb_values;     /* nnzb*brow*bcol fp16 */
} shflbw_device_ref;

int shflbw_weight_create(shflbw_weight** out);
void shflbw_weight_destroy(shflbw_weight* w);

/* BlockwiseSpMatrix::init_random, blockwise_format.h:70-123: mask, permutation
 * (iota + std::shuffle with default_random_engine(seed)), values rand()%9-4. */
int shflbw_weight_init_random(shflbw_weight* w, int nrow, int ncol, int brow, int bcol,
                              float expected_density, int row_permute, unsigned seed);
/* BlockwiseSpFilter::init_random, spconv/blockwise_format.h:30-52 (matrix is F x (R*S*C),
 * column k = (r*S + s)*C + c). */
int shflbw_filter_init_random(shflbw_weight* w, int F, int R, int S, int C, int brow, int bcol,
                              float expected_density, int filter_permute, unsigned seed);
/* Build from caller arrays (what `load` does from text).  values: nnzb*brow*bcol fp16 bit
 * patterns, column-major inside each block (blockwise_format.h:297).  row_permute_ids may be
 * NULL (not permuted).  For a filter pass R,S,C (> 0) with ncol == R*S*C; else 0,0,0. */
int shflbw_weight_set(shflbw_weight* w, int nrow, int ncol, int brow, int bcol, int nnzb,
                      const int* indptr, const int* indices, const uint16_t* values,
                      const int* row_permute_ids, int R, int S, int C);
/* Replace the values only (same pattern); drops a previous device image. */
int shflbw_weight_set_values(shflbw_weight* w, const uint16_t* values, size_t count);

/* BlockwiseSpMatrix::dump / load, blockwise_format.h:125-198 (text format of
 * example/spmatrix_dump_load.md).  dump: writes at most `cap` bytes (no terminator) and
 * always reports the size needed. */
int shflbw_weight_dump_text(const shflbw_weight* w, char* buf, size_t cap, size_t* needed);
int shflbw_weight_load_text(shflbw_weight* w, const char* text, size_t len);

/* CPU reference results for a caller's own checks.  Replaces get_host_reference of
 * blockwise_format.h:268-311 (SpMM: D_ref = alpha * A*B + beta * C, fp32, M x N row-major; C may be
 * NULL when beta == 0) and of spconv/blockwise_format.h:55-132 (convolution; here over NHWC tensors with
 * true stride: IFMap[b][hi][wi][c] fp16 bits, OFMap_ref[b][ho][wo][f] fp32, padding R/2, S/2).  Every
 * element is the fp32 sum in ascending order of the kept vectors, as in the reference.  Host arrays
 * in, host array out; works on any initialised weight, synced or not. */
int shflbw_spmm_host_reference(const shflbw_weight* w, int N, const uint16_t* B, float alpha,
                               const uint16_t* C, float beta, float* D_ref);
int shflbw_spconv_host_reference(const shflbw_weight* filter, int B, int H, int W, int stride,
                                 const uint16_t* IFMap, float* OFMap_ref);
/* ... and over the reference's C-H-W-B / F-H-W-B tensors with its own bounds rule (see shflbw_spconv_init_chwb):
 * spconv/blockwise_format.h:55-132 as it stands. */
int shflbw_spconv_host_reference_chwb(const shflbw_weight* filter, int B, int H, int W, int stride,
                                      const uint16_t* IFMap, float* OFMap_ref);

int shflbw_weight_get_info(const shflbw_weight* w, shflbw_weight_info* info);
/* Borrowed pointers to the host arrays (valid until the weight is re-initialised/destroyed). */
int shflbw_weight_host_arrays(const shflbw_weight* w, const int** indptr, const int** indices,
                              const uint16_t** values, const int** row_permute_ids);
/* config_str, blockwise_format.h:105-114 / spconv/blockwise_format.h:42-51. */
const char* shflbw_weight_config_str(const shflbw_weight* w);

/* transform_and_sync_device, blockwise_format.h:200-266: packs the meta image, uploads
 * meta + values, and additionally builds the private MFMA-ordered image the gfx950 kernels
 * read.  meta_host: the packed host image (meta_h), valid after a sync. */
int shflbw_weight_sync_device(shflbw_weight* w);
int shflbw_weight_meta_host(const shflbw_weight* w, const int** meta, size_t* n_ints);
int shflbw_weight_device_ref(const shflbw_weight* w, shflbw_device_ref* ref);

/* ------------------------------------------------------------------------- *
 * SpMM.  Replaces SpmmBlockwiseOpState (spmm/blockwise_op.h:6-17),
 * SpmmBlockwiseOp::initialize / operator() (:81-174) and
 * SpmmBlockwiseInitFn / SpmmBlockwiseExecFn (:188-215).
 *   D[row_permute_ids[r]][:] = alpha * (A_stored[r,:] * B) + beta * C[row_permute_ids[r]][:]
 * B: K x N row-major fp16, C/D: M x N row-major fp16, all device pointers, caller owned.
 * Preconditions: weight synced; bcol == 1; N % 8 == 0; B, C, D 16-byte aligned.
 * The state is a copyable POD holding raw pointers; it dangles if the weight is
 * re-initialised or destroyed (same as the reference).
 * Rounding: fp32 accumulation; with beta == 0 one rounding to fp16 (of alpha * acc).  With beta != 0 two: alpha * acc is
 * rounded to fp16 first, then fp16(float(that) + beta * C) - the reference rounds the accumulator to fp16 as well
 * (common/mma.h:336-339) and then combines in half arithmetic (common/epilogue.h:58-62); a host reference that rounds
 * alpha * acc + beta * C once differs by at most half an fp16 ulp of alpha * acc plus one ulp of the result.
 * ------------------------------------------------------------------------- */
typedef struct shflbw_spmm_state {
    size_t shared_mem_size;
    unsigned grid_dim[3];
    unsigned block_dim[3];
    int init_success;
    int variant; /* native tile variant chosen for this problem */
    struct {
        int M, N, K;
        const void* A_values;
        const void* B;
        const void* C;
        void* D;
        const int* A_bsr_indptr;
        const int* A_bsr_indices;
        const int* A_row_indices;
        float alpha, beta;
    } args;
    /* private device image (owned by the weight) */
    const void* packed_values;
    const int* packed_indices;
    const int* packed_indices_pm;
    const int* panel_ptr;
    int brow;
    int ldb_bytes; /* distance in bytes between two rows of B that are one kept-column id apart: N * 2 */
    const void* zero_row; /* 1 KiB of zeros inside the library (device memory): gathered for the padding slots */
    const int* packed_slab; /* the ids as LDS offsets for the tile variants that hold B in LDS; NULL when the weight has too many columns */
} shflbw_spmm_state;

/* C may be NULL when beta == 0.  variant < 0 selects automatically. */
int shflbw_spmm_init(shflbw_spmm_state* state, const shflbw_weight* w, int N,
                     const void* B, const void* C, void* D, float alpha, float beta);
int shflbw_spmm_init_variant(shflbw_spmm_state* state, const shflbw_weight* w, int N,
                             const void* B, const void* C, void* D, float alpha, float beta, int variant);
/* Asynchronous launch on `stream` (a hipStream_t, NULL = default stream); launch only:
 * no allocation, no synchronisation (benchmark loop, benchmark/benchmark.spmm.cu:29-42). */
int shflbw_spmm_exec(const shflbw_spmm_state* state, void* stream);
/* Number of native tile variants available for a block size, and a short name for each. */
int shflbw_spmm_variant_count(int brow);
const char* shflbw_spmm_variant_name(int brow, int variant);

/* ------------------------------------------------------------------------- *
 * SpConv2D as implicit GEMM.  Replaces SpconvBlockwiseOpState
 * (spconv/blockwise_op.h:6-17), SpconvBlockwiseOp::initialize / operator() (:79-149)
 * and SpconvBlockwiseInitFn / ExecFn (:161-193).
 *   GEMM view: M = F, K = R*S*C ordered (r, s, c), N = B*Ho*Wo; alpha = 1, beta = 0.
 *   Tensors are NHWC: IFMap[b][hi][wi][c], OFMap[b][ho][wo][f] (fp16, device, caller owned).
 *   H, W are the INPUT extents; padding is R/2, S/2 ("same" for stride 1, as the
 *   reference's col2im, spconv/conv_format.h:77-81); Ho = (H + 2*(R/2) - R)/stride + 1.
 * Preconditions: filter synced, bcol == 1, C % 8 == 0, F % 8 == 0.
 * init allocates device scratch inside the filter object (freed with it or by shflbw_weight_release_scratch):
 * the gather ids once per (form, B, H, W, stride), and per (form, geometry, IFMap, OFMap) the buffers the launches
 * write - states over different tensors never share those and may run on different streams.  At most
 * SHFLBW_CONV_SCRATCH_DEPTH such buffers exist per filter: initialising a state over one more tensor pair recycles
 * the buffers of the least recently initialised one (no allocation, no copy when the geometry is the same), whose
 * state must not be executed afterwards.  exec only launches, in order on `stream`.
 * shflbw_spconv_init_variant (variant < 0, and shflbw_spconv_init: the library's choice - variant 2 when B % 8 == 0,
 * else variant 0):
 *   variant 0 = plane form, three launches: the input is rewritten once per call as channel-major padded
 *     planes (one per stride phase); the SpMM kernel then gathers, for a kept k = (r, s, c), the
 *     plane of channel c at the constant offset of tap (r, s) - the im2col matrix is never built,
 *     its address generation is the per-id offset of the gather; a tile transpose writes NHWC;
 *   variant 1 = a single direct kernel (im2col gather from NHWC in the tile loads; every block size);
 *   variant 2 = plane form with the batch innermost in the planes and in the filter-major result (B % 8 == 0):
 *     every tap offset is then a multiple of 16 bytes, one copy of the planes serves all taps, and the result
 *     holds output pixels only; three launches;
 *   variant 3 = the steps of variant 2 in ONE persistent launch (B % 8 == 0): every XCD of the GPU rewrites the
 *     input, runs the SpMM and writes NHWC for its own range of output columns, in its own L2; the phases are
 *     counted between the workgroups of an XCD.  Needs a device that deals consecutive workgroups to consecutive
 *     XCDs (checked at init; SHFLBW_ERR_UNSUPPORTED otherwise).  Its waits are bounded: should one run out the launch still ends,
 *     and shflbw_spconv_check reports it.
 * ------------------------------------------------------------------------- */
#define SHFLBW_CONV_SCRATCH_DEPTH 4
typedef struct shflbw_spconv_state {
    size_t shared_mem_size;
    unsigned grid_dim[3];
    unsigned block_dim[3];
    int init_success;
    int variant;
    struct {
        int B, H, W, C, F, R, S, stride;
        const void* A_values;
        const void* IFMap;
        void* OFMap;
        const int* A_bsr_indptr;
        const int* A_bsr_indices;
        const int* A_row_indices;
        float alpha, beta;
    } args;
    int Ho, Wo;
    const void* packed_values;
    const int* packed_indices;
    const int* panel_ptr;
    int brow;
    /* Device scratch owned by the filter and the state of the SpMM launch in the middle.
     * Plane form (variant 0): `planes` holds the input as channel-major zero-padded planes
     * [plane_copies][stride*stride][C][plane_pitch]; a "pixel" of the GEMM is a position
     * b*plane_rows*plane_cols + i*plane_cols + j of that padded grid, np = ncols = B*plane_rows*plane_cols of
     * them, and result_fm is [F][np].  Batch-innermost forms (variants 2, 4): `planes` is
     * [stride*stride][C][plane_pitch] with position (i*plane_cols + j)*B + b, plane_rows = Ho + (R-1)/stride,
     * plane_cols = Wo + (S-1)/stride; ncols = Ho*plane_cols*B columns of the GEMM; result_fm (variant 2) is
     * [F][Ho*Wo*B].  Fused form (variant 3): the columns are those of variant 2, cols_per_xcd of them per XCD;
     * `planes` holds xcds slabs [stride*stride*C + 1][plane_pitch] (the positions one XCD's columns read),
     * result_fm xcds results [F][cols_per_xcd], `sync` the counters (all zero between launches). */
    void* result_fm;
    int np;
    void* planes;
    int plane_rows, plane_cols, plane_pitch, plane_copies;
    int ncols;
    int middle_tile_cols; /* variants 2 and 4: columns of a tile of the SpMM launch in the middle (512, 256 or 128, by the size of the GEMM) */
    int xcds, cols_per_xcd;
    int patience_ticks; /* fused form: 100 MHz ticks a workgroup waits for a phase before it takes over the work of workgroups
                         * of the launch that have not started yet (init sets 5000 = 50 us; a caller may change it).
                         * A negative value -t is for tests of that path: a patience of one tick, and every second
                         * workgroup joins min(t, 10000) ticks late.  The int at byte 60 of `sync` counts the take-overs. */
    void* sync;
    shflbw_spmm_state spmm;
} shflbw_spconv_state;

int shflbw_spconv_init(shflbw_spconv_state* state, const shflbw_weight* filter,
                       int B, int H, int W, int stride, const void* IFMap, void* OFMap);
int shflbw_spconv_init_variant(shflbw_spconv_state* state, const shflbw_weight* filter,
                               int B, int H, int W, int stride, const void* IFMap, void* OFMap, int variant);
int shflbw_spconv_exec(const shflbw_spconv_state* state, void* stream);
/* The same operator over the reference's own tensors (spconv/blockwise_format.h:111-128, spconv/conv_format.h:49-82):
 * IFMap[c][hi][wi][b] and OFMap[f][ho][wo][b], batch innermost; H and W are the extents of the output grid and at
 * the same time the bounds of the input: out(ho, wo) reads in(ho*stride - R/2 + r, wo*stride - S/2 + s) where that lies
 * inside H x W and zero elsewhere (so IFMap holds C*H*W*B values and OFMap F*H*W*B, whatever the stride).
 * Precondition as in the reference's kernel (spconv/blockwise_kernel.h:200-207): B % 8 == 0.  exec launches a padded
 * copy of the input and one SpMM launch that writes OFMap directly (form 4 of shflbw_spconv_variant_name). */
int shflbw_spconv_init_chwb(shflbw_spconv_state* state, const shflbw_weight* filter,
                            int B, int H, int W, int stride, const void* IFMap, void* OFMap);
/* No counterpart in the reference.  For callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  One complete convolution in the plane
 * form, the same launches as shflbw_spconv_init + shflbw_spconv_exec, with all scratch (the planes, the
 * filter-major result, the rewritten ids, which a small kernel computes on the device) in a fixed device
 * array inside the library: SHFLBW_STATIC_SCRATCH_BYTES on every GPU the library runs on, held until the
 * process ends.  Calls no hipMalloc / hipFree and copies nothing from the host; launches on `stream` only.
 * A problem whose scratch exceeds the array is refused with SHFLBW_ERR_CAPACITY (the message names both
 * sizes).  All calls on one GPU share the array: calls that overlap in time on one GPU race, also on
 * different streams; calls in stream order are safe, nothing of an earlier call is relied on. */
#define SHFLBW_STATIC_SCRATCH_BYTES (40u * 1024u * 1024u)
int shflbw_spconv_exec_static(const shflbw_weight* filter, int B, int H, int W, int stride,
                              const void* IFMap, void* OFMap, void* stream);

/* No counterpart in the reference.  Synchronous: waits for the device, then tells whether every launch of the
 * fused form (variant 3) on this state's scratch ran to completion: SHFLBW_ERR_HIP when the workgroups were not dealt to
 * the XCDs the way init had checked, or when a bounded wait between its phases ran out (the output of that launch
 * is then invalid; the scratch is reset for further launches).  SHFLBW_OK for every other form. */
int shflbw_spconv_check(const shflbw_spconv_state* state);

/* Forms of the convolution shflbw_spconv_init_variant accepts, and a short name for each. */
int shflbw_spconv_variant_count(void);
const char* shflbw_spconv_variant_name(int variant);
/* Frees the device scratch every shflbw_spconv_init on this filter allocated; states made before
 * dangle (the reference has no scratch; its states dangle the same way when the filter is
 * re-initialised, spmm/blockwise_op.h:118-122). */
int shflbw_weight_release_scratch(shflbw_weight* filter);
/* Device bytes and number of buffers of convolution scratch the filter holds at the moment. */
int shflbw_weight_scratch_bytes(const shflbw_weight* filter, size_t* bytes, int* buffers);

/* sizeof the two state structs as this library was compiled, for FFI mirrors to check their layout. */
void shflbw_abi_sizes(size_t* spmm_state_bytes, size_t* spconv_state_bytes);

/* Library / device facts (for logs): compute units, clock (kHz), LDS bytes per workgroup. */
int shflbw_device_info(int* compute_units, int* clock_khz, size_t* lds_bytes, char* arch, size_t arch_cap);

#ifdef __cplusplus
}
#endif
#endif /* SHFLBW_H */
