/*
 * qgemm.h -- C ABI of the MI355X (gfx950) scaled mixed-precision GEMM library.
 *
 * Plain pointers and sizes only.  Every data pointer is a DEVICE pointer owned
 * by the caller; calls enqueue work on a HIP stream and return without
 * synchronising, like the reference launchers (stream 0, no sync:
 * src/gemm/sm89_gemm_kernel_v3.cu:289-298).  Every entry returns a
 * qgemm_status_t; the C++ forwarders in gemm.h / mix_gemm.h turn that back
 * into the reference's print / throw behaviour.
 */
#ifndef QGEMM_H_
#define QGEMM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum qgemm_status {
    QGEMM_OK = 0,
    QGEMM_ERR_INVALID_ARG = 1,   /* null pointer, zero size, unknown enum value     */
    QGEMM_ERR_UNSUPPORTED = 2,   /* dtype / layout combination with no kernel        */
    QGEMM_ERR_NO_DEVICE = 3,     /* no HIP device visible                            */
    QGEMM_ERR_LAUNCH = 4,        /* hipLaunchKernel or another HIP call failed       */
    QGEMM_ERR_ALLOC = 5,         /* workspace allocation failed                      */
    QGEMM_ERR_NOT_DIVISIBLE_M = 6, /* reference dispatch contract: M % 32 != 0       */
    QGEMM_ERR_NOT_DIVISIBLE_N = 7, /*                              N % 32 != 0       */
    QGEMM_ERR_NOT_DIVISIBLE_K = 8, /*                              K % 32 != 0       */
    QGEMM_ERR_TOO_LARGE = 9,     /* a dimension or stride exceeds what kernels index */
    QGEMM_ERR_SCRATCH_TOO_SMALL = 10 /* qgemm_scaled_gemm_static: the call needs more than the static scratch */
} qgemm_status_t;

typedef enum qgemm_dtype {
    QGEMM_DT_F32 = 0,
    QGEMM_DT_BF16 = 1,
    QGEMM_DT_F16 = 2,
    QGEMM_DT_I8 = 3,
    QGEMM_DT_F8E4M3 = 4,        /* OCP e4m3 ("e4m3fn"): the encoding gfx950 MFMA decodes */
    QGEMM_DT_I32 = 5
} qgemm_dtype_t;

/* Where B's K index runs.  Replaces the two loader families of the reference:
 * src/include/gemm_utils.cuh:93,108 (B[k*N+n]) and :259,271 (B[n*K+k]). */
typedef enum qgemm_layout_b {
    QGEMM_B_KN = 0,             /* "NN": B is K x N row-major, B[k*ldB + n]  (GEMM_kernel_v1..v5)     */
    QGEMM_B_NK = 1              /* "NT": B is N x K row-major, B[n*ldB + k]  (GEMM_kernel_v3_1, v4_1) */
} qgemm_layout_b_t;

typedef enum qgemm_scale_mode {
    QGEMM_SCALE_PER_MATRIX = 1, /* a_scale, b_scale point at one float each                          */
    QGEMM_SCALE_BLOCK128 = 2    /* a_scale per (row, 128-wide K block), b_scale per 128x128 block     */
} qgemm_scale_mode_t;

typedef enum qgemm_layout {
    /* A[m*K + k], B[n*K + k]; a_scale[m*KB + kb], b_scale[nb*KB + kb]  (KB = ceil(K/128)) */
    QGEMM_LAYOUT_K_CONTIGUOUS = 0,
    /* The contract of fp8_mm (src/mix_gemm/hip_mix_gemm_kernel.cpp:425-439):
     * A[m + k*M], B[k*N + n]; a_scale[m + kb*M], b_scale[nb + kb*ceil(N/128)] */
    QGEMM_LAYOUT_REFERENCE = 1
} qgemm_layout_t;

/* Library set-up.  Replaces blas::blas_init / blas::blas_destroy
 * (include/blas.h:33-48): selects the current HIP device, loads the kernels.
 * Idempotent; the compute entries call it lazily.  qgemm_shutdown waits for
 * the device and frees every workspace block. */
int qgemm_init(void);
int qgemm_shutdown(void);

/* Number of visible HIP devices (0 when none): lets a host-only caller decide
 * without touching any compute entry. */
int qgemm_device_count(void);

const char *qgemm_status_string(int status);

/* Plain GEMM, C[M,N] = A[M,K] * B, fp32 accumulation (int32 for int8).
 * Replaces GEMM_kernel_v1 .. v5, v3_1, v4_1 (include/gemm.h:25-66).
 *   in_dtype   BF16 | F16 | I8 | F8E4M3        out_dtype  F32 | BF16 | F16 (I32 for I8 input)
 *   A          row-major M x K, leading dimension ldA (elements)
 *   B          per layout_b, leading dimension ldB (elements)
 *   C          row-major M x N, leading dimension ldC (elements)
 *   stream     hipStream_t, NULL = default stream
 * The reference accepts ldA/ldB and ignores them (its loaders index with K and
 * N); this entry honours them, which is the same thing for ldA = K, ldB = N|K. */
int qgemm_gemm(int in_dtype, int out_dtype, int layout_b, const void *A, size_t ldA, const void *B, size_t ldB,
               void *C, size_t ldC, size_t M, size_t N, size_t K, void *stream);

/* Scaled GEMM, C = (A o Q_A) x (B o Q_B).
 * Replaces select_BLOCK_TILE_SIZE_M / fp8_mm (src/mix_gemm/hip_mix_gemm_kernel.cpp:489-516)
 * and the int8_mm stub (src/gemm/sm80_gemm_kernel.cu:14-22).
 *   in_dtype   I8 (int32 accumulate, exact) | F8E4M3 (fp32 accumulate)
 *   out_dtype  F32 | BF16 | F16 ; I32 with I8 input and per-matrix scales returns the raw accumulators (scales ignored)
 *   scale_mode PER_MATRIX: C = acc * (a_scale[0] * b_scale[0])
 *              BLOCK128  : acc += (P_kb * a_scale[m,kb]) * b_scale[n/128,kb] per 128-wide K block (the last block may
 *                          be partial); P_kb is the fp32 partial of an fp8 block or the exact int32 partial of an int8
 *                          block, converted to fp32 once (the int8 twin of hip_mix_gemm_kernel.cpp:231-244, which the
 *                          reference only has for fp8)
 *   layout     see qgemm_layout_t;  C is row-major with leading dimension ldC
 *   split_k    0 = choose, 1 = never split, n > 1 = split K into n slices (deterministic
 *              two-pass reduction through the library workspace)
 * QGEMM_LAYOUT_REFERENCE enforces the reference's dispatch contract and
 * returns QGEMM_ERR_NOT_DIVISIBLE_{M,N,K} where the reference throws. */
int qgemm_scaled_gemm(int in_dtype, int out_dtype, int scale_mode, int layout, const void *A, const void *B,
                      const float *a_scale, const float *b_scale, void *C, size_t ldC, size_t M, size_t N,
                      size_t K, int split_k, void *stream);

/* qgemm_scaled_gemm for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, same kernels and
 * same results as qgemm_scaled_gemm; whatever that entry would take from the library workspace (split-K partial
 * planes, the transposed a_scale of QGEMM_LAYOUT_K_CONTIGUOUS block scales, the transposed operands of
 * QGEMM_LAYOUT_REFERENCE) comes from a static device array of QGEMM_STATIC_SCRATCH_BYTES that every GPU the
 * library runs on holds until the process ends.  The call allocates and frees nothing.  A problem that needs
 * more returns QGEMM_ERR_SCRATCH_TOO_SMALL and launches nothing.  All calls on one GPU share the array: two
 * calls whose kernels overlap in time on one GPU (different streams, or threads) race. */
#define QGEMM_STATIC_SCRATCH_BYTES ((size_t)32 << 20)
int qgemm_scaled_gemm_static(int in_dtype, int out_dtype, int scale_mode, int layout, const void *A, const void *B,
                             const float *a_scale, const float *b_scale, void *C, size_t ldC, size_t M, size_t N,
                             size_t K, int split_k, void *stream);

/* Library workspace (no reference counterpart: the reference's entries take none).  Calls that split K, that
 * take operands or scales in an arrangement the kernels do not read directly, and the per-matrix quantiser keep
 * their intermediate data in one device block owned by the library and grown on demand.  A block that is
 * outgrown is replaced but stays allocated until qgemm_shutdown, so launches already enqueued and graphs
 * already captured remain valid.  Calls on different streams share the block: each such call waits (on the
 * device, through an event) for the previous user on another stream.  While a stream is being captured into a
 * graph the library neither allocates nor touches that event: a call that would have to grow the block returns
 * QGEMM_ERR_ALLOC, and replays of graphs that use the workspace must not overlap other users of it.
 * qgemm_reserve_workspace makes the block at least `bytes` large ahead of time (it allocates: call it before a
 * capture begins, never during one; a block that has to grow at least doubles); qgemm_workspace_info reports
 * its address and size (NULL / 0 before first use). */
int qgemm_reserve_workspace(size_t bytes);
int qgemm_workspace_info(void **base, size_t *bytes);

/* out[n*M + m] = in[m*N + n] for 1-, 2- or 4-byte elements.
 * Replaces matrix_transpose<T> (src/transpose/transpose.cu:60-74), which
 * handles 2-byte elements with M % 64 == 0 and N % 32 == 0 only; any M, N here. */
int qgemm_transpose(int elem_bytes, const void *in, void *out, size_t M, size_t N, void *stream);

/* Quantiser for the operands of qgemm_scaled_gemm: the Q_A / Q_B of C = (A o Q_A) x (B o Q_B) that
 * README.md:1 of the reference describes ("input matrix will be quantized") and no file of it implements.
 *   x        rows x cols, F32 / BF16 / F16, row stride ld elements (device)
 *   q        rows x cols bytes (I8 or F8E4M3), row stride ldq
 *   scales   QGEMM_QUANT_PER_MATRIX: 1 float, s = max|x| / 127 (int8) or / 448 (fp8)
 *            QGEMM_QUANT_BLOCK_1x128 / _128x128: one float per block (max|x| of the block / 127 or / 448), written to
 *            scales[ib * scale_rs + jb * scale_cs] (ib: block row, jb: block column; strides in floats),
 *            so the a_scale / b_scale arrangement of either layout of qgemm_scaled_gemm can be produced
 *            directly (hip_mix_gemm_kernel.cpp:137,149)
 * q = round-to-nearest-even(x / s), saturated to +-127 / +-448; an all-zero block gets s = 1. */
typedef enum qgemm_quant_mode {
    QGEMM_QUANT_PER_MATRIX = 1,
    QGEMM_QUANT_BLOCK_1x128 = 2,
    QGEMM_QUANT_BLOCK_128x128 = 3
} qgemm_quant_mode_t;
int qgemm_quantize(int in_dtype, int out_dtype, int mode, const void *x, size_t ld, size_t rows, size_t cols, void *q,
                   size_t ldq, float *scales, size_t scale_rs, size_t scale_cs, void *stream);

/* Tile raster used by the GEMM kernels: linear workgroup id -> (tile_m, tile_n).
 * Replaces the GROUP_SIZE_M swizzle of src/gemm/sm89_gemm_kernel_v3.cu:169-183
 * (and fixes its clamp), composed with the 8-XCD remap the reference only names
 * (XCD_SWIZZLE, include/gpu_type.h:24).  Host-callable so tests can check it is
 * a bijection. */
int qgemm_tile_map(uint32_t wg, uint32_t tiles_m, uint32_t tiles_n, uint32_t group_m, uint32_t *tile_m,
                   uint32_t *tile_n);

/* Tuning / diagnostics (no reference counterpart: the reference picks its tile at compile time,
 * src/include/gemm_config.h:30-36).
 * qgemm_set_option(key, value): "force_split" (K slices, 0 = heuristic), "group_m", "kmajor", "stagger", "k_rot",
 *   "stagger_groups", "as_groups", "row_split" (0: one launch always; 1: the rows "a+b" or columns "a|b" of a partly
 *   empty last round of 256 x 256 tiles as a second launch where the estimate gains; 2 / 3: rows / columns wherever
 *   possible), "small_tiles" (0: 17 .. 256 rows against few columns keep a tall tile with a K split instead of several
 *   row tiles of the skinny-M kernel), "c_plain" (0 / 1: non-temporal / ordinary stores for C; -1: the library's
 *   choice), "b_stream" (0 / 1: copies of B without / with the streaming hint; -1: the library's choice); "force_config" accepts only -1 (back to the heuristic).
 *   "k_rot": with at most 256 rows the workgroups of column tile i start their K loops 3 i steps in and wrap round
 *   (memory channels), so the order of an fp32 sum depends on the column tile: results are the same from run to
 *   run, but equal rows of A against equal columns of B at different column positions may differ in the last bits.
 *   k_rot = 0 makes every workgroup start at K step 0 (position-independent sums); -1 restores the default.
 * qgemm_force_config(name) pins the row `name` of the variant tables for every following GEMM call (NULL or "":
 *   back to the heuristic).  Rows are addressed by name only; a call whose family has no row of that name returns
 *   QGEMM_ERR_UNSUPPORTED, a name no family has is QGEMM_ERR_INVALID_ARG here.
 * qgemm_variant_count / qgemm_variant_name enumerate the rows of the family that serves (in_dtype, scale_mode,
 *   k_major) -- arguments as for qgemm_plan -- so that callers never depend on the order of a table.
 * qgemm_last_config writes the name of the kernel variant the last GEMM call chose. */
int qgemm_set_option(const char *key, long value);
int qgemm_force_config(const char *name);
int qgemm_variant_count(int in_dtype, int scale_mode, int k_major);
int qgemm_variant_name(int in_dtype, int scale_mode, int k_major, int index, char *buf, size_t buflen);
int qgemm_last_config(char *buf, size_t buflen);

/* Which kernel configuration the library would run for a problem with dense, 16-byte aligned operands: the name
 * qgemm_last_config would report after the call ("256x256_w2x2_solo", "128x128_w2x2_dma_tn_splitk2", ...;
 * "transpose+<name>" when operands stored K-major go through the transpose kernels first).  Nothing is launched
 * and no device is needed (256 CUs are assumed before qgemm_init).  No reference counterpart: the reference picks
 * its tile at compile time (src/include/gemm_config.h:30-36).
 *   scale_mode 0 = plain GEMM (qgemm_gemm), else as for qgemm_scaled_gemm
 *   k_major    bit 0: A is stored K x M, bit 1: B is stored K x N (2 = QGEMM_B_KN, 3 = QGEMM_LAYOUT_REFERENCE) */
int qgemm_plan(int in_dtype, int scale_mode, int k_major, size_t M, size_t N, size_t K, char *buf, size_t buflen);

/* Self-check of the MFMA / LDS-DMA lane layouts the kernels assume, run on the
 * current device.  Writes a short report into buf; returns QGEMM_OK when every
 * assumption holds.  (Counterpart of the reference's playground/ layout probes.) */
int qgemm_selftest_layouts(char *buf, size_t buflen);

#ifdef __cplusplus
}
#endif
#endif /* QGEMM_H_ */
