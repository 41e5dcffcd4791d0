// MFMA GEMM kernel for gfx950.  Native operands are "NT": A is M x K, B is N x K, both with K
// contiguous; GemmCfg::KMAJ adds operands stored K x M / K x N (read through the transposing LDS
// loads).  One template covers int8, fp8-e4m3, bf16 and fp16 inputs.
//
// Replaces the device kernels of the reference:
//   GEMM_kernel_bf16_v1..v5      src/gemm/sm89_gemm_kernel_v{1,2,3,4,5}.cu
//   FP8_GEMM_kernel              src/mix_gemm/hip_mix_gemm_kernel.cpp:249-378
// It is not a translation of either: the tiling, the LDS layout and the load
// path are built around the CDNA4 matrix core.
//
// Data movement
//   * A K step is 128 bytes of every tile row (128 fp8/int8 or 64 bf16/fp16):
//     one full 128-byte cache line per row.
//   * Global -> LDS goes through buffer_load_dwordx4 ... lds (no VGPR staging, no
//     ds_write).  One such instruction moves 8 rows x 128 bytes = 1 KiB; lanes
//     8r .. 8r+7 fetch the eight 16-byte chunks of row r, so every quad of lanes
//     is one contiguous 64-byte request (the texture addresser only merges
//     neighbouring lanes; one lane per row costs 4x the cycles).  The hardware
//     stores lane l's 16 bytes at destination + 16*l.
//   * LDS layout ("row block" = 16 rows x 128 B = 2 KiB, two such instructions):
//     16-byte slot of (row r, chunk c) = 8*r + ((c + r) & 7).  The rotation is
//     applied on the global side (lane 8r+j fetches chunk (j - r) & 7), so the LDS
//     write stays linear in the lane id as the DMA requires.  The MFMA fragment
//     read (lane l: row l & 15, chunk 4*half + (l >> 4)) is then free of bank
//     conflicts without padding: measured 4.35 cycles per ds_read_b128 of a wave,
//     the same as a lane-linear read, where a rotation by r >> 1 costs 8.1 and no
//     rotation 16 (the LDS does not serve the 64 lanes of a 16-byte read sixteen
//     consecutive lanes at a time).  (The intent of the reference's
//     shared_memory_swizzle_coordinate, src/include/gemm_utils.cuh:15-20, which it
//     applies on the read side only.)
//   * Which K bytes a lane group holds does not matter as long as A and B agree:
//     the contraction index is summed away.
//   * LDS holds two stages in the simple pipeline (up to eight for the small tiles), three A and two
//     B buffers in the pipelined ones.
//
// Math
//   * The B fragment is fed as the first MFMA operand and the A fragment as the
//     second, so each lane ends up with 4 consecutive columns (n) of one row
//     (m) of C: row-major C is written with 8- or 16-byte stores.
//   * Per-matrix scales are applied once in the epilogue.  128-block scales are
//     applied in the K loop: one 16x16x128 MFMA on a zero accumulator gives the
//     partial product of exactly one scale block, which is folded in with one
//     FMA per element (hip_mix_gemm_kernel.cpp:231-244).
#pragma once
#include <type_traits>

#include "common.h"

namespace qgemm {

struct GemmArgs {
    const char *A;        // M x K, row stride lda bytes (KMAJ & 1: K x M, stride between k rows)
    const char *B;        // N x K, row stride ldb bytes (KMAJ & 2: K x N, stride between k rows)
    char *C;              // M x N row-major, ldc elements; split-K: plane z at C + z*split_stride elements
    const float *as;      // per-matrix: 1 float; block: as[m*as_ms + kb*as_ks]
    const float *bs;      // per-matrix: 1 float; block: bs[nb*bs_ns + kb*bs_ks]
    uint32_t M, N;
    uint32_t ksteps;      // K steps of 128 bytes in total, the last one possibly partial
    uint32_t k_tail;      // bytes of K in the last step when it is partial (a multiple of 16), 0 when it is whole
    uint32_t lda, ldb;    // bytes
    uint32_t ldc;         // elements
    uint32_t tiles_m, tiles_n, group_m;
    uint32_t nsplit, ksteps_per_split;
    uint64_t split_stride;
    uint32_t as_ms, as_ks, bs_ns, bs_ks;
    uint32_t nb_max;      // ceil(N/128) - 1
    uint32_t as_groups;   // rows with two K groups, block scales: a_scale is K-contiguous (as_ks == 1), 16-byte aligned rows,
                          // every K slice and k_rot a multiple of four steps: the scales travel four K blocks at a time
    int out_dtype;        // qgemm_dtype_t of C
    int per_matrix_scale; // multiply by as[0]*bs[0] in the epilogue
    int vec_store;        // 0: scalar stores; 1: C and ldc allow 4-element vector stores; 2: also 16-byte row pieces
    int c_plain;          // ordinary instead of non-temporal stores for C (run_nt: launches of at most one round of tiles)
    int b_stream;         // B is read once by the launch (one or two row tiles): its copies carry the streaming hint
    uint32_t k_rot;                  // simple pipeline and skinny-M kernel: the workgroups of column tile i start their K loops (i * k_rot) % nk steps in (0: at 0)
    uint32_t stagger, stagger_wgs;   // the first stagger_wgs workgroups start (id / 8 % stagger_groups) * stagger microseconds late (0: off)
    uint32_t stagger_groups;
    unsigned long long *dbg_cycles;   // measurement builds only (QGEMM_STAMP): time stamps per wave
};

// How the K loop is scheduled.
//   PIPE_SIMPLE    every wave: wait for tile k, barrier, start tile k+1, read fragments, MFMA.
//   PIPE_SOLO      4 waves = 1 per SIMD, each with a 128 x 128 wave tile (64 accumulator tiles).  A
//                  fragments are streamed two rows of MFMAs ahead, B fragments of step k+1 replace
//                  those of step k as they die in its last two rows, copies ride between the MFMAs:
//                  few LDS reads per MFMA and one barrier per K step.  A triple-buffered, B
//                  double-buffered in LDS (160 KiB for 256 x 256).
//                  With 8 waves (128 x 64 wave tiles) the same schedule runs two waves per SIMD and
//                  keeps the accumulators in vector registers, which the block-scale fold needs.
// Global -> LDS always goes through buffer_load_dwordx4 ... lds: no VGPR staging, the wave only waits on vmcnt.
enum Pipe : int { PIPE_SIMPLE = 0, PIPE_SOLO = 2 };

template <int ARITH_, bool BLOCK_SCALE_, int BM_, int BN_, int WAVES_M_, int WAVES_N_, int PIPE_ = PIPE_SIMPLE,
          int KMAJ_ = 0, int STAGES_ = 0, int KGROUPS_ = 1, bool ASK_ = false, bool COPYW_ = false>
struct GemmCfg {
    // COPYW (solo pipeline, four computing waves with 128 x 64 wave tiles on a 256 x 128 tile): four more waves issue
    // every copy of the K loop, at the places the schedule has them; the computing waves, one per SIMD, issue fragment
    // reads, MFMAs and (block scales) the fold, and nothing that queues at the memory pipe.  Their accumulators are
    // compiler-managed as in the 8-wave form, so block scales are possible, and since they have no copies in flight
    // the tile may be K-major (the compiler's wait in front of a transposing read then waits for nothing).
    static constexpr bool COPYW = COPYW_;
    // ASK (block scales, solo pipeline): a_scale is read with the K blocks contiguous, a_scale[m * as_ms + kb], the
    // arrangement of QGEMM_LAYOUT_K_CONTIGUOUS, instead of rows contiguous, a_scale[m + kb * as_ks].  A compile-time
    // choice: as a branch inside the K loop it cost the 8-wave kernel 758 spilled registers.
    static constexpr bool ASK = ASK_;
    // The simple pipeline loads one scale per lane and K step at a_scale[m * as_ms + kb * as_ks] with
    // whatever strides they are given: rows-contiguous scales are one 256-byte request per 64 rows, K-contiguous
    // ones 64 requests, which these tiles (a step of several hundred cycles per wave) can afford and which saves the
    // launch that would copy the scales into the other order.
    static constexpr bool AS_ANY_STRIDE = BLOCK_SCALE_ && PIPE_ != PIPE_SOLO;
    // STAGES (simple pipeline): number of LDS stages, 0 = chosen below.
    // KGROUPS = 2: the workgroup has two sets of WAVES_M x WAVES_N waves and two waves that copy; set 0 computes
    // the even K steps and set 1 the odd ones of the same tile, half a turn apart, and the two partial sums meet in
    // LDS before the epilogue.  A tile that is alone on its CU (a shape with no more tiles than CUs) otherwise
    // reads its fragments and runs its MFMAs in turn, with nothing to overlap either with: two waves per SIMD
    // working on different K steps do what a second workgroup on the CU would.
    static constexpr int KG = KGROUPS_;
    // KMAJ: which operands are stored K-major (bit 0: A is K x M with M contiguous, bit 1: B is K x N with N
    // contiguous) instead of K-contiguous.  A K-major tile keeps its rows of K in LDS and the MFMA fragments
    // are taken out of it with the transposing LDS reads (ds_read_b64_tr_b8 / _b16).
    static constexpr int KMAJ = KMAJ_;
    static constexpr bool KMA = (KMAJ_ & 1) != 0, KMB = (KMAJ_ & 2) != 0;
    static constexpr int ES = (ARITH_ == AR_BF16 || ARITH_ == AR_F16) ? 2 : 1;   // operand element bytes
    static constexpr int KE = 128 / ES;                                          // K elements per step
    static constexpr int PIPE = PIPE_;
    static constexpr bool A3 = PIPE_ == PIPE_SOLO;      // solo: three A buffers and two B buffers instead of whole stages
    static constexpr int ARITH = ARITH_;
    static constexpr bool BLOCK_SCALE = BLOCK_SCALE_;
    static constexpr int BM = BM_, BN = BN_, BKB = 128;         // BKB: bytes of K per step
    static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
    static constexpr int NW = WAVES_M * WAVES_N * KGROUPS_;
    // K groups: four more waves that only copy (waves NW .. NW+3, see the K loop)
    static constexpr int NPROD = (KGROUPS_ == 2 || COPYW_) ? 4 : 0;
    static constexpr int THREADS = (NW + NPROD) * kWave;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;  // wave tile
    static constexpr int TM = WM / 16, TN = WN / 16;            // 16x16 MFMA tiles per wave
    static constexpr int RBA = BM / 16, RBB = BN / 16;          // 2 KiB row blocks per stage
    static constexpr int NLOAD = (RBA + RBB) * 2;               // 1 KiB load instructions per stage
    static constexpr int LPT = NLOAD / NW;                      // ... per wave
    static constexpr int A_BYTES = RBA * 2048, B_BYTES = RBB * 2048;
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int LPT_A = RBA * 2 / NW;                  // A load instructions per wave
    // simple pipeline: as many stages in flight as LDS and the 6-bit vmcnt allow (at most
    // 8).  A workgroup that streams a narrow strip of B (skinny M) otherwise waits one full memory round trip
    // per K step.  The block-scale form keeps two (its scale loads share vmcnt with the copies), except with K
    // groups, where the scales travel to LDS like the operands.
    static constexpr int NSTAGE_FIT = (160 * 1024) / STAGE_BYTES, NSTAGE_CNT = 2 + 63 / LPT;
    // Only for the small tiles: a 128 x 128 tile with two stages leaves room for two workgroups per CU, which is
    // worth more to a compute-bound shape than deeper prefetch.
    static constexpr int NSTAGE = STAGES_ > 0 ? STAGES_
                                  : (PIPE != PIPE_SIMPLE || BLOCK_SCALE || BM * BN > 64 * 128 || KMAJ_ != 0) ? 2
                                  : (NSTAGE_FIT < NSTAGE_CNT ? (NSTAGE_FIT < 8 ? NSTAGE_FIT : 8)
                                                             : (NSTAGE_CNT < 8 ? NSTAGE_CNT : 8));
    // Block scales with K groups: the a_scale values of a stage (one float per tile row, at most 128) travel to LDS
    // like the operands, 512 bytes per stage behind the ring, so that every copy of the loop is of one kind and the
    // wave's own count of copies in flight stays exact (a register load among them makes the compiler wait for all).
    // (or, K-contiguous a_scale: four slots of BM rows x four K blocks, see the K loop)
    // (copying waves beside the solo schedule, the twin for K-contiguous a_scale: the same four slots, see SCALES_LDS)
    static constexpr int SCALE_LDS = (BLOCK_SCALE_ && KGROUPS_ == 2) ? (NSTAGE * 512 > 64 * BM_ ? NSTAGE * 512 : 64 * BM_)
                                     : (BLOCK_SCALE_ && COPYW_ && ASK_) ? 64 * BM_ : 0;
    static constexpr int LDS_BYTES = (A3 ? 3 * A_BYTES + 2 * B_BYTES : NSTAGE * STAGE_BYTES) + SCALE_LDS;
    static_assert(STAGES_ == 0 || (PIPE == PIPE_SIMPLE && (!BLOCK_SCALE || KGROUPS_ == 2) &&
                                   (KMAJ_ == 0 || KGROUPS_ == 2) && STAGES_ >= 2 && STAGES_ <= NSTAGE_FIT && STAGES_ <= NSTAGE_CNT),
                  "explicit stage count: simple pipeline, within LDS and the 6-bit counter");
    static_assert(KGROUPS_ == 1 || (KGROUPS_ == 2 && PIPE == PIPE_SIMPLE &&
                                    NSTAGE >= 4 && (!BLOCK_SCALE_ || (BM_ <= 128 && BN_ <= 128))),
                  "K groups: simple pipeline, at least four stages");
    static_assert(BM % (16 * WAVES_M) == 0 && BN % (16 * WAVES_N) == 0, "wave tile must be a multiple of 16");
    static_assert(NLOAD % NW == 0, "load instructions must divide evenly over the waves");
    static_assert(!BLOCK_SCALE || ARITH == AR_F8 || ARITH == AR_I8, "block scales: fp8 and int8 operands");
    static_assert(!BLOCK_SCALE || (128 % WN == 0 || WN % 128 == 0), "wave tile must align with 128-wide scale blocks");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS is 160 KiB per CU");
    static_assert(PIPE != PIPE_SOLO || ((NW == 4 || NW == 8) && TN >= 4 &&
                                        ((TM % 4 == 0 && TM >= 8) || (TM == 6 && NW == 8))),
                  "solo: 4 or 8 waves, at least 8 rows (8 waves: or 6) of at least 4 MFMAs per step");
    static_assert(!COPYW_ || (PIPE_ == PIPE_SOLO && WAVES_M_ * WAVES_N_ == 4 && KGROUPS_ == 1), "copying waves beside four computing waves: solo pipeline");
    static_assert(PIPE != PIPE_SOLO || !BLOCK_SCALE || NW == 8 || COPYW_,
                  "solo with block scales: the accumulators have to live in the 256 vector registers of a wave");
    static_assert(PIPE == PIPE_SIMPLE || (RBA * 2) % NW == 0, "A loads must divide evenly over the waves");
    static_assert(KMAJ == 0 || NW % 4 == 0, "K-major tiles: the swizzle of a copy must not depend on the instruction");
    static_assert((!KMA || (BM * ES) % 128 == 0) && (!KMB || (BN * ES) % 128 == 0),
                  "K-major tiles are made of whole 128-byte panels");
    // The compiler makes every transposing LDS read wait for all global->LDS copies in flight (vmcnt(0)): it cannot
    // tell that they target another buffer.  The simple pipeline issues the next stage's copies behind the reads
    // of a step, so nothing is in flight there; the pipelined schedules live on copies in flight and would stall.
    // (The rows with two K groups keep a deep ring all the same: their copies are issued by waves of their own, and
    // the waves that read have none in flight.)
    static_assert(KMAJ == 0 || PIPE == PIPE_SIMPLE || COPYW_, "K-major tiles: simple pipeline, or copying waves");
    static_assert(!ASK_ || (BLOCK_SCALE_ && PIPE_ == PIPE_SOLO), "K-contiguous a_scale: block scales, solo pipeline");
};

// Time stamps of a measurement build (-DQGEMM_DEBUG_BUILD=1; the library proper compiles them to nothing): up to N
// readings of the 100 MHz clock all CUs share, written per wave to GemmArgs::dbg_cycles when the kernel ends.
#if QGEMM_DEBUG_BUILD
#define QGEMM_STAMP_DECL(N) unsigned long long qgemm_stamp_[N] = {}
#define QGEMM_STAMP(I) (qgemm_stamp_[I] = __builtin_amdgcn_s_memrealtime())
#define QGEMM_STAMP_WRITE(PTR, SLOT, N, COND)                                              \
    do {                                                                                   \
        if ((PTR) && (COND))                                                               \
            for (int i_ = 0; i_ < (N); ++i_) (PTR)[(size_t)(SLOT) * (N) + i_] = qgemm_stamp_[i_]; \
    } while (0)
#else
#define QGEMM_STAMP_DECL(N) ((void)0)
#define QGEMM_STAMP(I) ((void)0)
#define QGEMM_STAMP_WRITE(PTR, SLOT, N, COND) ((void)0)
#endif

typedef __attribute__((address_space(3))) void lds_void;
typedef short v4s __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v2i lds_v2i;
typedef __attribute__((address_space(3))) v4s lds_v4s;

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void *base, uint32_t bytes) {
    // raw buffer, 32-bit data format word as used for untyped loads on gfx9
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes, 0x00020000);
}

// vmcnt(n) only (expcnt / lgkmcnt left at "no wait"), gfx9 encoding.
__device__ inline constexpr int waitcnt_vm(int n) { return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8); }
// lgkmcnt(0) only
__device__ inline constexpr int waitcnt_lgkm0() { return 0xF | (3 << 14) | (0x7 << 4) | (0 << 8); }

// s_barrier that nothing is scheduled across (MFMAs have no memory dependence the
// compiler could see, so it would otherwise be free to move them into the other phase)
__device__ inline void phase_barrier() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
}

// 16-byte slot of (row r in 0..15, chunk c in 0..7) inside a 2 KiB row block
__host__ __device__ inline constexpr int lds_slot(int r, int c) { return 8 * r + ((c + r) & 7); }

// K-major tiles (row = one k, 128 bytes of m or n; panels of KE rows): the 16-byte chunk c of row k sits in
// slot c ^ kmajor_swz(k).  A transposing read takes, per 16 lanes, 8 rows x 16 bytes (1-byte elements:
// rows k0 .. k0+7 with k0 a multiple of 8, groups of lanes 16 rows apart) or 4 rows x 32 bytes (2-byte
// elements: rows k0 .. k0+3, groups 8 rows apart).  Rows two apart share their banks (64 banks x 4 bytes
// = two 128-byte rows), so the XOR has to separate rows of equal parity inside a group and the two groups
// of a half wave: bits 1-2 and 4 of k for bytes, bits 1 and 3 for 16-bit elements.
template <int ES>
__host__ __device__ inline constexpr int kmajor_swz(int k) {
    return ES == 1 ? (((k >> 1) & 3) | (((k >> 4) & 1) << 2)) : ((((k >> 1) & 1) << 1) | (((k >> 3) & 1) << 2));
}

template <int ARITH>
struct AccT { typedef v4f type; };
template <>
struct AccT<AR_I8> { typedef v4i type; };

// one 16 x 16 x (128 bytes of K) update: x = B fragment (rows n), y = A fragment (rows m)
template <int ARITH>
__device__ inline typename AccT<ARITH>::type mma128(v4i x0, v4i x1, v4i y0, v4i y1, typename AccT<ARITH>::type c) {
    if constexpr (ARITH == AR_F8) {
        v8i x = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
        v8i y = {y0[0], y0[1], y0[2], y0[3], y1[0], y1[1], y1[2], y1[3]};
        // cbsz = blgp = 0 selects e4m3 for both operands; zero scale operands select the unscaled form
        return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(x, y, c, 0, 0, 0, 0, 0, 0);
    } else if constexpr (ARITH == AR_I8) {
        c = __builtin_amdgcn_mfma_i32_16x16x64_i8(x0, y0, c, 0, 0, 0);
        return __builtin_amdgcn_mfma_i32_16x16x64_i8(x1, y1, c, 0, 0, 0);
    } else if constexpr (ARITH == AR_BF16) {
        c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, x0), __builtin_bit_cast(v8bf, y0), c, 0, 0, 0);
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, x1), __builtin_bit_cast(v8bf, y1), c, 0, 0, 0);
    } else {
        c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, x0), __builtin_bit_cast(v8h, y0), c, 0, 0, 0);
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, x1), __builtin_bit_cast(v8h, y1), c, 0, 0, 0);
    }
}

// The same update with the accumulator pinned in place in the accumulation registers.  With all 256 of them
// holding accumulators (solo pipeline) the register allocator otherwise routes part of them through a
// temporary, with copies and the wait states those need between the MFMAs.  x0/y0 and x1/y1 halves of the
// 16-byte MFMAs are issued by the caller a row apart (`half`), so no dependent pair is back to back.
template <int ARITH>
__device__ inline void mma128_inplace(v4i x0, v4i x1, v4i y0, v4i y1, typename AccT<ARITH>::type &c, int half) {
    if constexpr (ARITH == AR_F8) {
        v8i x = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
        v8i y = {y0[0], y0[1], y0[2], y0[3], y1[0], y1[1], y1[2], y1[3]};
        if (half == 0) asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y));
    } else {
        const v4i x = half ? x1 : x0, y = half ? y1 : y0;
        if constexpr (ARITH == AR_I8) asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y));
        else if constexpr (ARITH == AR_BF16) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y));
        else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y));
    }
}

template <class C>
__global__ void __launch_bounds__(C::THREADS) gemm_nt_kernel(const GemmArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass only needs the launch stub
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    // part_t: what one MFMA step of 128 bytes of K delivers (int32 for int8 operands, else fp32); acc_t: the running
    // sums.  With block scales the sums are fp32 whatever the operands: an int8 partial product of one K block is an
    // exact int32, converted once and folded in like the fp8 kernel's fp32 partial.
    typedef typename AccT<C::ARITH>::type part_t;
    typedef std::conditional_t<C::BLOCK_SCALE, v4f, part_t> acc_t;
    QGEMM_STAMP_DECL(4);               // start, K loop start, K loop end, end
    QGEMM_STAMP(0);

    // Staggered start (the host asks for it where C is written in 4-byte elements over three or more rounds of
    // tiles).  Left alone, all CUs finish a round of 256 x 256 tiles together and write 64 MiB of C at once, which is
    // what the memory takes 10 us to absorb: the epilogue of such a tile takes 10 - 12 us against 4.6 us for the 2-byte
    // output, with the matrix cores of the whole part idle.  The workgroups of the first round therefore start in
    // groups a microsecond or two apart (s_sleep: 64 clocks per unit), the offsets carry through every later round,
    // and the bursts interleave with other CUs' K loops.  int8 8192^3 to f32, interleaved in one process, us: none
    // 381.0, four groups 2 us apart 374.2, eight groups 1 us apart 367.9 (what the host asks for), 8 x 2 371.7,
    // 16 x 1 383.6, 32 x 1 412.3; the same product with bf16 output 359.9.  8192 x 8192 x 4096: 226.4 / 216.2 / 213.2.
    if (p.stagger > 0 && blockIdx.x < p.stagger_wgs) {
        const int g = (blockIdx.x >> 3) % p.stagger_groups;            // (workgroup i runs on XCD i % 8: whole rows of XCDs per group)
        for (int i = 0; i < g * (int)p.stagger; ++i) __builtin_amdgcn_s_sleep(32);
    }
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kg = wave / (C::WAVES_M * C::WAVES_N);              // K group of this wave (0 unless GemmCfg::KG == 2)
    const int wave_q = wave % (C::WAVES_M * C::WAVES_N);          // its place in the group
    const int wm = wave_q / C::WAVES_N, wn = wave_q % C::WAVES_N;

    // ---- which tile, which K slice
    uint32_t wg = blockIdx.x, z = 0;
    if (p.nsplit > 1) {
        z = __builtin_amdgcn_readfirstlane(wg % p.nsplit);
        wg = __builtin_amdgcn_readfirstlane(wg / p.nsplit);
    }
    uint32_t tm, tn;
    tile_map(wg, p.tiles_m, p.tiles_n, p.group_m, tm, tn);
    // the divisions of tile_map run on the vector ALU: bring the (uniform) result back to scalar registers so
    // that everything derived from it (buffer descriptors, scalar offsets) stays there
    tm = __builtin_amdgcn_readfirstlane(tm);
    tn = __builtin_amdgcn_readfirstlane(tn);
    const uint32_t row0 = tm * C::BM, col0 = tn * C::BN;
    const uint32_t kbeg = z * p.ksteps_per_split;
    const uint32_t kend = kbeg + p.ksteps_per_split < p.ksteps ? kbeg + p.ksteps_per_split : p.ksteps;
    const int nk = (int)(kend - kbeg);

    // ---- buffer resources: base at this tile's first row and first K byte; the
    // range ends with the last valid row, so rows past M / N read as out of
    // range (never a fault; the DMA then writes zeros) and only ever feed outputs
    // that are not stored.
    const uint32_t a_rows = p.M - row0 < (uint32_t)C::BM ? p.M - row0 : C::BM;
    const uint32_t b_rows = p.N - col0 < (uint32_t)C::BN ? p.N - col0 : C::BN;
    // A partial last K step (K bytes not a multiple of 128; the slice that ends with the last step has it): the
    // ranges end with the last byte of K, and in that one step the lanes whose 16-byte chunk of a K-contiguous row
    // lies past the end of the row present an offset that is out of range (bit 31; the host keeps every valid
    // offset below 2^31 for such shapes), so the DMA writes zeros where the next row's bytes would have landed.
    // A K-major operand needs nothing: its k rows past the end of K lie past the end of the range.
    const bool has_tail = p.k_tail != 0 && kend == p.ksteps && nk > 0;
    const uint32_t kbytes = has_tail ? (uint32_t)(nk - 1) * C::BKB + p.k_tail : (uint32_t)nk * C::BKB;
    // K-major operand: rows are k (stride lda / ldb bytes), the tile starts at column row0 / col0; the range ends
    // with the last column of the last k row of this K slice.  Columns past M / N inside an earlier row read
    // the neighbouring row instead (valid memory) and, as above, only feed outputs that are not stored.
    const uint32_t krows = nk > 0 ? kbytes / C::ES : 1;
    const __amdgpu_buffer_rsrc_t ra =
        C::KMA ? make_rsrc(p.A + (size_t)kbeg * C::KE * p.lda + (size_t)row0 * C::ES,
                           (krows - 1) * p.lda + (p.M - row0) * C::ES)
               : make_rsrc(p.A + (size_t)row0 * p.lda + (size_t)kbeg * C::BKB, (a_rows - 1) * p.lda + kbytes);
    const __amdgpu_buffer_rsrc_t rb =
        C::KMB ? make_rsrc(p.B + (size_t)kbeg * C::KE * p.ldb + (size_t)col0 * C::ES,
                           (krows - 1) * p.ldb + (p.N - col0) * C::ES)
               : make_rsrc(p.B + (size_t)col0 * p.ldb + (size_t)kbeg * C::BKB, (b_rows - 1) * p.ldb + kbytes);

    // ---- the LPT load instructions of this wave.  Instruction q = wave + i*NW (0 .. NLOAD-1) covers
    // rows 8*(q & 1) .. +7 of row block q >> 1 and lands at stage + 1024*q.  With NW even, q & 1 =
    // wave & 1 for every i, so the per-lane part of the address (row inside the block, rotated
    // chunk) is the same for all of them: one VGPR per operand; the row block goes into the scalar
    // offset of the instruction, which the buffer range check includes.
    static_assert(C::NW % 2 == 0 && C::RBA % (C::NW / 2) == 0, "A / B split of the loads must not depend on the wave");
    constexpr int LPT_A0 = C::LPT_A;                                    // loads i < LPT_A0 fetch A, the rest B
    // (GemmCfg::COPYW: the copying waves NW .. NW+3 take the places of waves 0 .. 3 in everything that follows)
    const int lw = (C::COPYW && wave >= C::NW) ? wave - C::NW : wave;
    const int ld_r = 8 * (lw & 1) + (lane >> 3);                        // row inside the row block
    const int ld_chunk = ((lane & 7) - ld_r) & 7;                         // rotation: see lds_slot
    // K-major tile: row block blk holds k rows 16 * (blk % (KE/16)) .. +15 of panel blk / (KE/16) (a panel = 128
    // bytes of m or n).  Bit 4 of k is bit 0 of blk = bit 1 of the wave number for every instruction of the wave
    // (NW / 2 and KE / 16 are even), so the swizzled chunk is one VGPR here too.
    const int ld_chunk_km = (lane & 7) ^ kmajor_swz<C::ES>(ld_r + 16 * ((lw >> 1) & 1));
    const uint32_t voff_a = ld_r * p.lda + (C::KMA ? ld_chunk_km : ld_chunk) * 16;
    const uint32_t voff_b = ld_r * p.ldb + (C::KMB ? ld_chunk_km : ld_chunk) * 16;
    // (the chunk of a lane is the same in every copy instruction of every pipeline: (lane & 7) - (lane >> 3) mod 8)
    const uint32_t tail_or = (has_tail && (uint32_t)ld_chunk * 16 >= p.k_tail) ? 0x80000000u : 0u;
    const uint32_t voff_a_t = C::KMA ? voff_a : (voff_a | tail_or), voff_b_t = C::KMB ? voff_b : (voff_b | tail_or);
    const int kt_tail = has_tail ? nk - 1 : -1;              // the step (of this slice) that is partial
    // K step the loop's step kt stands for (rotated start, simple pipeline only: the pipelined kernels run
    // compute-bound shapes, whose workgroups share panels and should stay in step)
    constexpr bool K_ROT = C::PIPE == PIPE_SIMPLE;
    const int k_first = K_ROT && p.k_rot && nk > 0 ? (int)((tn * p.k_rot) % (uint32_t)nk) : 0;    // by column tile: the row tiles of a panel of B stay in step
    auto kpos = [&](int kt) -> int {
        if constexpr (K_ROT) {
            const int k = kt + k_first;
            return k >= nk ? k - nk : k;
        } else {
            return kt;
        }
    };
    auto load_soff = [&](int i, int kt_loop) -> uint32_t {              // scalar: row block + K step
        const int kt = kpos(kt_loop);
        const bool is_a = i < LPT_A0;
        const uint32_t blk = (lw >> 1) + (is_a ? i : i - LPT_A0) * (C::NW / 2);
        const uint32_t ld = is_a ? p.lda : p.ldb;
        if (is_a ? C::KMA : C::KMB) {
            constexpr uint32_t BPP = C::KE / 16;                        // row blocks per panel
            return ((uint32_t)kt * C::KE + (blk % BPP) * 16) * ld + (blk / BPP) * 128;
        }
        return blk * 16 * ld + (uint32_t)kt * C::BKB;
    };

    auto issue_stage = [&](int kt) {       // global -> LDS
        char *stage = smem + (kt % C::NSTAGE) * C::STAGE_BYTES;
        const bool tl = kpos(kt) == kt_tail;
        const uint32_t va = tl ? voff_a_t : voff_a, vb = tl ? voff_b_t : voff_b;
#pragma unroll
        for (int i = 0; i < C::LPT; ++i) {
            lds_void *dst = (lds_void *)(stage + (wave + i * C::NW) * 1024);
            // (B read once by the launch, i.e. streamed out of memory: its copies carry the streaming hint)
            if (i < LPT_A0)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, dst, 16, va, load_soff(i, kt), 0, 0);
            else if (p.b_stream)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, dst, 16, vb, load_soff(i, kt), 0, 2);
            else
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, dst, 16, vb, load_soff(i, kt), 0, 0);
        }
    };

    // ---- block scales (fp8 only): a_scale per row of each A fragment, b_scale per 128 columns.
    // a_scale is read with the rows contiguous (as_ms == 1: a_scale[m + kb*as_ks], the host guarantees it):
    // lane l fetches the scale of wave-tile row l (and l + 64), one 256-byte request per 64 rows, through a
    // buffer load (rows past M read as 0 or as some other finite scale; they only meet zero operands).  A
    // step later every lane picks the row of each of its A fragments (row l & 15 of row block a) out of
    // those registers: with ds_bpermute in the simple pipeline, with lane swaps on the vector
    // ALU in the solo pipeline.  One load per lane and fragment instead (16 distinct rows per instruction,
    // every row a request of its own) keeps the texture addresser busy for longer than the MFMAs of the
    // step take.
    constexpr int NBS = C::BLOCK_SCALE ? (C::WN + 127) / 128 : 1;
    constexpr int NLD = C::BLOCK_SCALE ? (C::WM + 63) / 64 : 1;
    float as_cur[C::TM], bs_cur[NBS], bs_raw[NBS];
    int as_raw[NLD];
    uint32_t as_voff = 0, bs_off[NBS];
    const int bp0 = (lane & 15) * 4;
    __amdgpu_buffer_rsrc_t ras = make_rsrc(p.as, 0);
    if constexpr (C::BLOCK_SCALE) {
        // rows contiguous (as_ms == 1), p.as_ks floats from one K block to the next (p.as_ks > p.M when the rows
        // are part of a taller matrix); or, solo pipeline only, K blocks contiguous (as_ks == 1), as_ms floats from
        // one row to the next
        ras = make_rsrc(p.as, ((p.ksteps - 1) * p.as_ks + (p.M - 1) * p.as_ms + 1) * 4);
        as_voff = (row0 + wm * C::WM + lane) * p.as_ms * 4;
#pragma unroll
        for (int j = 0; j < NBS; ++j) {
            uint32_t nb = (col0 + wn * C::WN) / 128 + j;
            nb = nb < p.nb_max ? nb : p.nb_max;
            bs_off[j] = nb * p.bs_ns;
        }
    }
    auto fetch_scales = [&](int kt) {          // start the loads for K step kt
        if constexpr (C::BLOCK_SCALE) {
            const uint32_t kb = kbeg + kpos(kt);
#pragma unroll
            for (int j = 0; j < NLD; ++j)
                as_raw[j] = __builtin_amdgcn_raw_buffer_load_b32(ras, as_voff, (64 * j * p.as_ms + kb * p.as_ks) * 4, 0);
            // (the solo pipeline fetches one step past the end of K: keep that read inside the array)
            const uint32_t kbc = kb < p.ksteps ? kb : p.ksteps - 1;
#pragma unroll
            for (int j = 0; j < NBS; ++j) bs_raw[j] = p.bs[bs_off[j] + kbc * p.bs_ks];
        }
    };
    auto expand_scales = [&]() {               // what fetch_scales brought becomes as_cur / bs_cur
        if constexpr (C::BLOCK_SCALE) {
#pragma unroll
            for (int a = 0; a < C::TM; ++a)
                as_cur[a] = __builtin_bit_cast(
                    float, __builtin_amdgcn_ds_bpermute(bp0 + ((16 * a) & 63) * 4, as_raw[(16 * a) / 64]));
#pragma unroll
            for (int j = 0; j < NBS; ++j) bs_cur[j] = bs_raw[j];
        }
    };

    acc_t acc[C::TM][C::TN];
#pragma unroll
    for (int a = 0; a < C::TM; ++a)
#pragma unroll
        for (int b = 0; b < C::TN; ++b) acc[a][b] = acc_t{0, 0, 0, 0};

    // ---- fragment addresses: lane l is row l & 15, K group l >> 4; its two 16-byte pieces
    // of a K step are chunks (l >> 4) and 4 + (l >> 4) of that row
    const int fr = lane & 15, fg = lane >> 4;
    const int off0 = lds_slot(fr, fg) * 16, off1 = lds_slot(fr, 4 + fg) * 16;
    const int a_blk0 = (wm * C::TM) * 2048;
    const int b_blk0 = (C::RBA + wn * C::TN) * 2048;
    // K-major tile: the 16 columns of fragment x16 (counted in 16-column units from the tile's first column)
    // are chunk c of panel pn; the lane's 16 bytes of a half step are k rows 64*half + 16*fg .. +15 (bytes) or
    // 32*half + 8*fg .. +7 (16-bit), fetched by two transposing reads.  Lane j of a group of 16 supplies the
    // address of 8 bytes of the group's row j >> 1 (bytes: 2 lanes per 16-byte row piece) or j >> 2 (16-bit: 4
    // lanes per 32-byte row piece) and receives column j of the block.  Everything lane-dependent is in km_lane;
    // the chunk of the fragment comes in by XOR (see kmajor_swz), the rest is an immediate offset.
    const int km_lane = C::ES == 1 ? ((16 * fg + (fr >> 1)) * 128 + 16 * kmajor_swz<1>(16 * fg + (fr >> 1)) + 8 * (fr & 1))
                                   : ((8 * fg + (fr >> 2)) * 128 +
                                      16 * (((fr >> 1) & 1) | kmajor_swz<2>(8 * fg + (fr >> 2))) + 8 * (fr & 1));
    auto frag_km = [&](const char *tile, int x16, int half) {
        constexpr int PER_PANEL = 8 / C::ES;                            // fragments per 128-byte panel
        const int pn = x16 / PER_PANEL, c = (x16 % PER_PANEL) * C::ES;
        const char *q = tile + (pn * C::KE + half * (C::KE / 2)) * 128 + (km_lane ^ (16 * c));
        if constexpr (C::ES == 1) {
            const v2i lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i *)q);
            const v2i hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i *)(q + 8 * 128));
            return v4i{lo[0], lo[1], hi[0], hi[1]};
        } else {
            const v2i lo = __builtin_bit_cast(v2i, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s *)q));
            const v2i hi = __builtin_bit_cast(v2i, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s *)(q + 4 * 128)));
            return v4i{lo[0], lo[1], hi[0], hi[1]};
        }
    };
    auto frag_a = [&](const char *stage, int a, int half) {
        if constexpr (C::KMA) return frag_km(stage, wm * C::TM + a, half);
        else return *(const v4i *)(stage + a_blk0 + a * 2048 + (half ? off1 : off0));
    };
    auto frag_b = [&](const char *stage, int b, int half) {
        if constexpr (C::KMB) return frag_km(stage + C::RBA * 2048, wn * C::TN + b, half);
        else return *(const v4i *)(stage + b_blk0 + b * 2048 + (half ? off1 : off0));
    };

    // ---- K loop
    QGEMM_STAMP(1);
    if constexpr (C::PIPE != PIPE_SIMPLE) {
        // A buffer is first read one barrier after the wait of its last copier, and is first
        // overwritten one barrier after the lgkmcnt(0) of its last reader.
        constexpr int NA_BUF = 3;
        constexpr int B_BASE = NA_BUF * C::A_BYTES;
        constexpr int LPT_A = C::LPT_A, LPT_B = C::LPT - C::LPT_A;
        // instruction i < LPT_A of this wave belongs to A, the rest to B (RBA*2 % NW == 0)
        // Solo pipelines: the row-block part of a copy's address sits in a vector register per copy (there are
        // registers to spare) and the scalar offset is the K step alone, one register for all copies of a step;
        // with one wave per SIMD every scalar add between two MFMAs is issue time the MFMAs do not get (with two
        // waves per SIMD it still pays: int8 -1.8 %, fp8 -1.4 %, bf16 -0.8 % on 8192^3; block scales unchanged).
        constexpr bool VOFF_PER_COPY = C::PIPE == PIPE_SOLO && C::KMAJ == 0 && LPT_A % 4 == 0 && LPT_B % 4 == 0;
        // ... and a wave's copies are neighbours in LDS (instruction q = wave * LPT_A + i of the A list, likewise
        // for B; elsewhere q = wave + i * NW), so that four of them share one LDS base in M0 and differ in the
        // instruction's immediate offset (0 .. 3072).  The hardware adds that immediate to the global address as
        // well: the descriptors of these kernels start GROUP_SPAN bytes below the tile and every vector offset
        // carries GROUP_SPAN minus its immediate, so no offset is negative and the range check sees the same sums.
        constexpr int GROUP_SPAN = 3072;
        uint32_t vo_copy[VOFF_PER_COPY ? C::LPT : 1];
        __amdgpu_buffer_rsrc_t ra_g = ra, rb_g = rb;
        if constexpr (VOFF_PER_COPY) {
            const uint32_t a_rows_ = p.M - row0 < (uint32_t)C::BM ? p.M - row0 : C::BM;
            const uint32_t b_rows_ = p.N - col0 < (uint32_t)C::BN ? p.N - col0 : C::BN;
            ra_g = make_rsrc(p.A + (size_t)row0 * p.lda + (size_t)kbeg * C::BKB - GROUP_SPAN, (a_rows_ - 1) * p.lda + kbytes + GROUP_SPAN);
            rb_g = make_rsrc(p.B + (size_t)col0 * p.ldb + (size_t)kbeg * C::BKB - GROUP_SPAN, (b_rows_ - 1) * p.ldb + kbytes + GROUP_SPAN);
            const uint32_t chunk = (((lane & 7) - (lane >> 3)) & 7) * 16;          // rotation: see lds_slot
#pragma unroll
            for (int i = 0; i < C::LPT; ++i) {
                const bool is_a = i < LPT_A;
                const int il = is_a ? i : i - LPT_A;
                const uint32_t q = lw * (is_a ? LPT_A : LPT_B) + il;
                const uint32_t row = (q >> 1) * 16 + (q & 1) * 8 + (lane >> 3);
                vo_copy[i] = row * (is_a ? p.lda : p.ldb) + chunk + GROUP_SPAN - (il & 3) * 1024;
            }
        }
        // one LDS-DMA instruction with the immediate offset 1024 * k (a literal: the builtin wants a constant)
        auto dma = [&](const __amdgpu_buffer_rsrc_t &rs, char *dst, uint32_t vo, uint32_t so, int k) {
            switch (k) {
                case 0: __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_void *)dst, 16, vo, so, 0, 0); break;
                case 1: __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_void *)dst, 16, vo, so, 1024, 0); break;
                case 2: __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_void *)dst, 16, vo, so, 2048, 0); break;
                default: __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_void *)dst, 16, vo, so, 3072, 0); break;
            }
        };
        // (tor: tail_or when the copy belongs to the partial last K step, else 0: the literal 0 in the unrolled groups
        // of the K loop, where the OR then costs nothing)
        auto issue_a1 = [&](int i, int kt, int buf, uint32_t tor) {
            if constexpr (VOFF_PER_COPY) {
                char *grp = smem + buf * C::A_BYTES + (lw * LPT_A + (i & ~3)) * 1024;
                dma(ra_g, grp, vo_copy[i] | tor, (uint32_t)kt * C::BKB, i & 3);
            } else {
                lds_void *dst = (lds_void *)(smem + buf * C::A_BYTES + (lw + i * C::NW) * 1024);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, dst, 16, C::KMA ? voff_a : (voff_a | tor), load_soff(i, kt), 0, 0);
            }
        };
        auto issue_b1 = [&](int i, int kt, uint32_t tor) {
            if constexpr (VOFF_PER_COPY) {
                const int il = i - LPT_A;
                char *grp = smem + B_BASE + (kt & 1) * C::B_BYTES + (lw * LPT_B + (il & ~3)) * 1024;
                dma(rb_g, grp, vo_copy[i] | tor, (uint32_t)kt * C::BKB, il & 3);
            } else {
                lds_void *dst = (lds_void *)(smem + B_BASE + (kt & 1) * C::B_BYTES + (lw + i * C::NW) * 1024 - C::A_BYTES);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, dst, 16, C::KMB ? voff_b : (voff_b | tor), load_soff(i, kt), 0, 0);
            }
        };
        auto next_buf = [&](int bufi) { return bufi + 1 == NA_BUF ? 0 : bufi + 1; };
        if constexpr (C::PIPE == PIPE_SOLO) {
            // K step kt of a wave (TM rows of TN MFMAs; all B fragments and up to four A fragments in registers):
            //   row a = 0 .. TM-1:   [copies]  read A(kt)[a+2] (last two rows: A(kt+1)[0], [1]);
            //                        TN MFMAs  acc[a][*] += B(kt)[*] x A(kt)[a]
            //   in the last row B(kt)[b] is dead after its MFMA and B(kt+1)[b] is read into its registers.
            // One barrier per step, in front of row TM-2, preceded by the wait for this wave's reads and for all
            // its copies but the A copies of this step.  Copies: A(kt+2) -> A buffer (kt+2) % 3 in rows 0 .. 3,
            // B(kt+2) -> B buffer kt & 1 in the two rows behind the barrier.  So A(kt+1) and B(kt+1), issued a whole
            // step earlier, are known to have landed exactly where they are first read (rows TM-2 .. TM-1), and the
            // buffers being overwritten (A(kt-1): read before the barrier of step kt-1; B(kt): read in the last row
            // of step kt-1, before this step's barrier) are free.  64 KiB per step at 64 B/clk per CU keeps the
            // load path busy for half of a step: every copy gets a full step to land.
            constexpr int TMs = C::TM;
            constexpr int COPY_ROWS_A = 4, CPR_A = (LPT_A + COPY_ROWS_A - 1) / COPY_ROWS_A;   // A copies per row
            // A fragment ring: row a lives in slot a % RING and is read AHEAD rows before it is used (one row
            // ahead is less than the LDS latency under load: the wave then waits in front of every row).
            // (wave tiles of six row blocks, the 192-row tile: three slots; a read then lands in the slot of the row
            // whose last MFMA has just been issued)
            constexpr int RING = TMs % 4 == 0 ? 4 : 3, AHEAD = 2;
            constexpr int BR = TMs - AHEAD;                  // row the barrier stands in front of
            constexpr int CPR_B = (LPT_B + AHEAD - 1) / AHEAD;                              // B copies per row
            constexpr int SLOTS = C::TN - 2;                 // MFMAs of a row a copy can ride behind
            constexpr int CPS_A = (CPR_A + SLOTS - 1) / SLOTS, CPS_B = (CPR_B + SLOTS - 1) / SLOTS;   // copies per slot
            static_assert(BR >= COPY_ROWS_A && TMs % RING == 0, "A copies ride in front of the barrier");
            v4i fbr[C::TN][2];         // B fragments
            v4i far[RING][2];          // A fragment ring
            int a_rd = 0, a_wr = 2;
            // block scales of the current step (as_raw / bs_raw hold what fetch_scales brought for the next).
            // as_b[a] = a_scale of row l & 15 of row block a for every lane l: lane l of as_raw[j] holds the scale of
            // wave-tile row 64 j + l, and each of its four 16-lane rows is spread over the whole wave with three
            // lane swaps on the vector ALU (v_permlane16_swap: odd rows of one register against even rows of
            // the other; v_permlane32_swap: upper half against lower half).  The same pick through ds_bpermute
            // shares the LDS queue, which answers in order, with the fragment reads issued two rows ahead: waiting
            // for a pick then means waiting for those reads as well (7 % of the K loop on config 4).
            // a_scale as the caller has it, K blocks contiguous (GemmCfg::ASK): lane l fetches the scales of
            // two K blocks of its row at once with an 8-byte load (4-byte alignment is enough; behind a row's last
            // block the second half is the next row's first scale or, past the end of the array, the zero of the
            // range check: nobody uses it), on every other step, so the 64 rows of a load, 64 requests of their
            // own, cost the texture addresser half of what one strided dword per step would.  Either way block kb
            // sits in component kb & 1 of as_pair.
            float as_b[TMs], bs_c[NBS], sc[2][NBS] = {};        // (sc: zero until the first row of the first step has set it)
            v2i as_pair[NLD];
            constexpr bool as_kcont = C::ASK;
            // Copying waves and K-contiguous a_scale (the twin `_ks` of the row with copying waves): the computing waves
            // fetch no scales themselves.  A copying wave brings the scales of four K blocks of 64 tile rows in one
            // 16-byte-per-lane copy, in front of the A copies of every fourth step, into slot (kt / 4) % 4 of four
            // behind the operand buffers ([row][4 K blocks]; the host picks this twin only where rows and K slices
            // start at multiples of four blocks), and a computing wave reads the eight values of its lane for the
            // next step where the other kernels distribute what they fetched.  That takes the last memory instruction
            // but the b_scale load out of the computing waves, the lane swaps with it, and a row of a_scale costs
            // the fill path one request per four steps instead of one per two from each of the waves that share it.
            constexpr bool SCALES_LDS = C::BLOCK_SCALE && C::COPYW && C::ASK;
            constexpr int SC_BASE = 3 * C::A_BYTES + 2 * C::B_BYTES;
            auto fetch_a_scales = [&](int kt, int comp) {      // for K step kt (of this slice; comp = kt & 1)
                if constexpr (C::BLOCK_SCALE && !SCALES_LDS) {
                    const uint32_t kb = kbeg + kt;
                    if (as_kcont) {
                        if (comp == 0) {
#pragma unroll
                            for (int j = 0; j < NLD; ++j)
                                as_pair[j] = __builtin_bit_cast(
                                    v2i, __builtin_amdgcn_raw_buffer_load_b64(ras, as_voff, (64 * j * p.as_ms + kb) * 4, 0));
                        }
                    } else {
#pragma unroll
                        for (int j = 0; j < NLD; ++j)
                            as_pair[j][comp] = __builtin_amdgcn_raw_buffer_load_b32(ras, as_voff, (64 * j + kb * p.as_ks) * 4, 0);
                    }
                }
            };
            auto fetch_b_scales = [&](int kt) {
                if constexpr (C::BLOCK_SCALE) {
                    // (one step past the end of K is fetched like the others: keep that read inside the array)
                    const uint32_t kb = kbeg + kt, kbc = kb < p.ksteps ? kb : p.ksteps - 1;
#pragma unroll
                    for (int j = 0; j < NBS; ++j) bs_raw[j] = p.bs[bs_off[j] + kbc * p.bs_ks];
                }
            };
            // With one b_scale per wave tile and K block (NBS == 1) the factor a_scale * b_scale is formed here, on
            // the two registers the loads brought, instead of once per row of MFMAs: the same product, the same bits.
            auto rotate_scales = [&](int comp, int kt_next) {  // (kt_next: the step the scales are for)
                if constexpr (SCALES_LDS) {
                    const char *sc_ = smem + SC_BASE + ((kt_next >> 2) & 3) * (16 * C::BM) + (kt_next & 3) * 4 +
                                      (wm * C::WM + (lane & 15)) * 16;
#pragma unroll
                    for (int a = 0; a < TMs; ++a) {
                        const float x = *(const float *)(sc_ + a * 256);
                        as_b[a] = NBS == 1 ? x * bs_raw[0] : x;
                    }
#pragma unroll
                    for (int j = 0; j < NBS; ++j) bs_c[j] = bs_raw[j];
                } else if constexpr (C::BLOCK_SCALE) {
#pragma unroll
                    for (int j = 0; j < NLD; ++j) {
                        unsigned x = (unsigned)as_pair[j][comp];
                        if constexpr (NBS == 1)
                            x = __builtin_bit_cast(unsigned, __builtin_bit_cast(float, x) * bs_raw[0]);
                        const auto r = __builtin_amdgcn_permlane16_swap(x, x, false, false);      // (R0 R0 R2 R2), (R1 R1 R3 R3)
                        const auto e = __builtin_amdgcn_permlane32_swap(r[0], r[0], false, false);  // all R0, all R2
                        const auto o = __builtin_amdgcn_permlane32_swap(r[1], r[1], false, false);  // all R1, all R3
                        const unsigned rows[4] = {e[0], o[0], e[1], o[1]};
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            if (4 * j + q < TMs) as_b[4 * j + q] = __builtin_bit_cast(float, rows[q]);
                    }
#pragma unroll
                    for (int j = 0; j < NBS; ++j) bs_c[j] = bs_raw[j];
                }
            };
            auto rd_a = [&](int buf, int a, int slot) {
                const char *sa_ = smem + buf * C::A_BYTES;
                far[slot][0] = frag_a(sa_, a, 0);
                far[slot][1] = frag_a(sa_, a, 1);
            };
            auto rd_b = [&](int kt, int b) {
                const char *sb_ = smem + B_BASE + (kt & 1) * C::B_BYTES - C::A_BYTES;   // frag_b adds RBA row blocks
                fbr[b][0] = frag_b(sb_, b, 0);
                fbr[b][1] = frag_b(sb_, b, 1);
            };
            // 4 waves: 256 accumulator registers per lane, pinned in place (see mma128_inplace); the two
            // halves of a 16-byte MFMA pair are then issued a row apart.  8 waves: compiler-managed.
            constexpr bool PINNED = C::NW == 4 && !C::COPYW;
            constexpr int HALVES = (PINNED && C::ARITH != AR_F8) ? 2 : 1;
            auto mma = [&](int a, int b, int half) {
                if constexpr (PINNED)
                    mma128_inplace<C::ARITH>(fbr[b][0], fbr[b][1], far[a % RING][0], far[a % RING][1], acc[a][b], half);
                else if constexpr (!C::BLOCK_SCALE)       // (block scales: the K loop below starts every MFMA from zero)
                    acc[a][b] = mma128<C::ARITH>(fbr[b][0], fbr[b][1], far[a % RING][0], far[a % RING][1], acc[a][b]);
            };
            // The last two steps issue their copies (and the last one its scale fetch) past the end of K like
            // every other step: the buffer range check turns what lies beyond the operand into zeros, the
            // rest is data nobody reads, and one straight-line loop body serves all steps (a second, guarded
            // copy of the body cost register spills of its own).
            // (generic_tag: the form of the step outside the unrolled groups.  Only there can the copies a step issues,
            // those of step kt + 2, be the ones of a partial last K step: they carry the OR that puts the lanes past
            // the end of K out of range, 0 for every other step.)
            // Block scales: the partial product of the last tile of a step is folded behind the first MFMA of the next
            // step instead of at the end of its own, where the wave would wait out that MFMA with nothing else to
            // issue (CARRY: the steps of the unrolled groups, all alike, so that they stay one instantiation; the
            // first of them folds a zero, and what the last leaves over is folded behind the group loop).
            constexpr int BEHIND = 2;          // MFMAs between a partial product and its fold
            part_t left_over = {0, 0, 0, 0};   // the partial product a step leaves to the next
            auto step = [&](int kt, int par, auto generic_tag, auto carry_tag) {             // par = kt & 1
                constexpr bool GENERIC = decltype(generic_tag)::value;
                constexpr bool CARRY = decltype(carry_tag)::value && C::BLOCK_SCALE;
                const uint32_t tor = GENERIC ? (kt + 2 == kt_tail ? tail_or : 0u) : 0u;
                const int a_nx = next_buf(a_rd);
                constexpr bool copies = !C::COPYW;            // (the copying waves' loop is below)
                // block scales of this step (fetched one step ahead) and the fetch for the next one, in front of
                // this step's copies: by the time they are used nothing older is still in flight
                // block scales: fetch_scales brings the a_scale rows of step kt+1 (in front of this step's
                // copies: by the time they are used nothing older is in flight).  The factor of row a,
                // a_scale[row] * b_scale, is made one row ahead: the cross-lane pick behind the first
                // MFMA of row a-1, the multiply behind the second MFMA of row a, so two factors are live at a time.
                part_t part[BEHIND + 1];
                fetch_a_scales(kt + 1, par ^ 1);
                fetch_b_scales(kt + 1);
                // Order of the MFMAs of a step: row by row.  With copying waves (one computing wave per SIMD, four MFMAs
                // to a row) and block scales the last two rows go column by column instead, (TM-2, b), (TM-1, b),
                // B(kt+1)[b]: read behind the last row's own four MFMAs, the first B fragment of the next step is
                // wanted three MFMAs after its read is issued; this way it is seven.  (1 - 2.4 % on four shapes with
                // block scales, whose wave has the fold to issue as well; nothing measurable without.)
                constexpr bool JOINT = C::COPYW && C::BLOCK_SCALE;
                constexpr int NT = TMs * C::TN, J0 = (TMs - 2) * C::TN;
                static_assert(!JOINT || BR == TMs - 2, "the joint rows start at the barrier");
                auto row_of_tile = [&](int i) { return (JOINT && i >= J0) ? TMs - 2 + ((i - J0) & 1) : i / C::TN; };
                auto col_of_tile = [&](int i) { return (JOINT && i >= J0) ? (i - J0) >> 1 : i % C::TN; };
                auto fold = [&](int i) {
                    if constexpr (C::BLOCK_SCALE) {
                        const int pa = row_of_tile(i), pb = col_of_tile(i);
                        const float f = sc[pa % 2][(pb * 16) / 128];
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[pa][pb][r] += (float)part[i % (BEHIND + 1)][r] * f;
                    }
                };
                // the last tile of the step before (its factor is still in sc: a row's factor is replaced behind the
                // second MFMA of the same row of the next step at the earliest)
                auto fold_left_over = [&]() {
                    if constexpr (C::BLOCK_SCALE) {
                        const float f = sc[(TMs - 1) % 2][((C::TN - 1) * 16) / 128];
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[TMs - 1][C::TN - 1][r] += (float)left_over[r] * f;
                    }
                };
                // the side instructions of a row go between its MFMAs, one at a time: a run of them in front
                // of the row would leave the matrix core idle once they take longer than one MFMA
                auto side = [&](int a, int slot) {   // slot 0 .. TN-1: what rides behind MFMA `slot` of row a
                    if (slot < 2) {                  // the two halves of the A fragment AHEAD rows ahead
                        const int an = a + AHEAD;
                        const int buf = an < TMs ? a_rd : a_nx, ar = an < TMs ? an : an - TMs;
                        far[an % RING][slot] = frag_a(smem + buf * C::A_BYTES, ar, slot);
                        return;
                    }
                    if (!copies) return;
                    if (a < COPY_ROWS_A) {
#pragma unroll
                        for (int j = (slot - 2) * CPS_A; j < (slot - 1) * CPS_A; ++j)
                            if (j < CPR_A && a * CPR_A + j < LPT_A) issue_a1(a * CPR_A + j, kt + 2, a_wr, tor);
                    } else if (a >= BR) {
                        const int r = a - BR;
#pragma unroll
                        for (int j = (slot - 2) * CPS_B; j < (slot - 1) * CPS_B; ++j)
                            if (j < CPR_B && r * CPR_B + j < LPT_B) issue_b1(LPT_A + r * CPR_B + j, kt + 2, tor);
                    }
                };
                auto step_barrier = [&]() {
                    __builtin_amdgcn_sched_barrier(0);
                    // lgkmcnt(0) and vmcnt(LPT_A): all but the A copies of this step
                    __builtin_amdgcn_s_waitcnt(waitcnt_vm(LPT_A) & 0xF0FF);
                    phase_barrier();
                };
                if constexpr (PINNED) {
#pragma unroll
                    for (int a = 0; a < TMs; ++a) {
                        if (a == BR) step_barrier();
#pragma unroll
                        for (int h = 0; h < HALVES; ++h) {
#pragma unroll
                            for (int b = 0; b < C::TN; ++b) {
                                mma(a, b, h);
                                // the side instructions of the row, spread over all its MFMAs (behind every
                                // second one where a tile takes two: 16-cycle MFMAs leave room for little more
                                // than one of them with its address arithmetic)
                                if constexpr (HALVES == 2) {
                                    if ((h * C::TN + b) % 2 == 0) side(a, (h * C::TN + b) / 2);
                                } else {
                                    side(a, b);
                                }
                                // B(kt)[b] is dead: its registers take B(kt+1)[b] (where a tile takes two MFMAs:
                                // each half as soon as its MFMA of the last row is out, so the first halves, which
                                // the next step needs first, are read half a row earlier)
                                if constexpr (HALVES == 2) {
                                    if (a == TMs - 1) {
                                        const char *sb_ = smem + B_BASE + ((kt + 1) & 1) * C::B_BYTES - C::A_BYTES;
                                        fbr[b][h] = frag_b(sb_, b, h);
                                    }
                                } else {
                                    if (a == TMs - 1) rd_b(kt + 1, b);
                                }
                            }
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < NT; ++i) {
                        const int a = row_of_tile(i), b = col_of_tile(i);
                        if (i == BR * C::TN) step_barrier();
                        if constexpr (C::BLOCK_SCALE) {
                            // each MFMA starts from zero and gives the partial product of one 128-wide K block; it is
                            // folded into the running sum, scaled, two MFMAs later, so the four FMAs of a tile run
                            // under the MFMAs of the next two (hip_mix_gemm_kernel.cpp:231-244)
                            part[i % (BEHIND + 1)] = mma128<C::ARITH>(fbr[b][0], fbr[b][1], far[a % RING][0], far[a % RING][1],
                                                                      part_t{0, 0, 0, 0});
                            side(a, b);
                            // the factor of a row is formed behind the MFMA that follows the row's first one: it is first
                            // used one MFMA later, and its register was last used (row a-2) one MFMA earlier at the latest
                            const int fr = (JOINT && i >= J0) ? (i == J0 + 1 ? TMs - 2 : (i == J0 + 2 ? TMs - 1 : -1)) : (b == 1 ? a : -1);
                            if (fr >= 0) {
#pragma unroll
                                for (int j = 0; j < NBS; ++j) sc[fr % 2][j] = NBS == 1 ? as_b[fr] : as_b[fr] * bs_c[j];
                            }
                            __builtin_amdgcn_sched_barrier(0);
                            if (i >= BEHIND) fold(i - BEHIND);
                            else if (CARRY && i == 0) fold_left_over();
                            __builtin_amdgcn_sched_barrier(0);
                        } else {
                            mma(a, b, 0);
                            side(a, b);
                        }
                        // B(kt)[b] is dead after its MFMA of the last row: its registers take B(kt+1)[b]
                        if (a == TMs - 1) rd_b(kt + 1, b);
                        if (i == NT - 1 || (!(JOINT && i >= J0) && b == C::TN - 1)) __builtin_amdgcn_sched_barrier(0);
                    }
                }
                if constexpr (C::BLOCK_SCALE) {
#pragma unroll
                    for (int i = TMs * C::TN - BEHIND; i < TMs * C::TN - (CARRY ? 1 : 0); ++i) fold(i);
                    if constexpr (CARRY) left_over = part[(TMs * C::TN - 1) % (BEHIND + 1)];
                    rotate_scales(par ^ 1, kt + 1);
                }
                a_rd = a_nx;
                a_wr = next_buf(a_wr);
            };
            auto first_copies = [&]() {
                const uint32_t tor0 = kt_tail == 0 ? tail_or : 0u, tor1 = kt_tail == 1 ? tail_or : 0u;
#pragma unroll
                for (int i = 0; i < LPT_A; ++i) issue_a1(i, 0, 0, tor0);
#pragma unroll
                for (int i = LPT_A; i < C::LPT; ++i) issue_b1(i, 0, tor0);
                if (nk > 1) {
#pragma unroll
                    for (int i = 0; i < LPT_A; ++i) issue_a1(i, 1, 1, tor1);
#pragma unroll
                    for (int i = LPT_A; i < C::LPT; ++i) issue_b1(i, 1, tor1);
                }
            };
            if constexpr (C::COPYW) {
                if (wave >= C::NW) {
                    // The copying waves: the copies of step(), at the same places between the same barriers (two in
                    // front of the loop, one per step, one behind the loop).  A(kt+2) goes out in front of the barrier
                    // of step kt, into the buffer of A(kt-1), which every computing wave has read before the barrier
                    // of step kt-1; then the wait for everything older, A(kt+1) and B(kt+1), which are first read
                    // behind this barrier; B(kt+2) goes out behind it, into the buffer of B(kt), which is in
                    // registers everywhere since the last row of step kt-1.
                    auto issue_scale_group = [&](int kt) {     // K steps kt .. kt + 3 of this slice, kt a multiple of four
                        if constexpr (SCALES_LDS) {
                            static_assert(C::BM == 64 * C::NPROD, "one copy of 64 rows per copying wave");
                            lds_void *dst = (lds_void *)(smem + SC_BASE + ((kt >> 2) & 3) * (16 * C::BM) + lw * 1024);
                            __builtin_amdgcn_raw_ptr_buffer_load_lds(ras, dst, 16, (row0 + 64 * lw + lane) * p.as_ms * 4,
                                                                     (kbeg + (uint32_t)kt) * 4, 0, 0);
                        }
                    };
                    if (nk > 0) {
                        issue_scale_group(0);
                        first_copies();
                        // (step 0 needs A(0) and B(0); A(1) and B(1) are waited for in front of its barrier)
                        if (nk > 1) __builtin_amdgcn_s_waitcnt(waitcnt_vm(C::LPT));
                        else __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
                        phase_barrier();
                        phase_barrier();
                        int aw = 2;
                        for (int kt = 0; kt < nk; ++kt) {
                            const uint32_t tor = kt + 2 == kt_tail ? tail_or : 0u;
                            if (kt + 2 < nk) {
                                if (((kt + 2) & 3) == 0) issue_scale_group(kt + 2);     // older than the A copies: waited for below
#pragma unroll
                                for (int i = 0; i < LPT_A; ++i) issue_a1(i, kt + 2, aw, tor);
                                __builtin_amdgcn_s_waitcnt(waitcnt_vm(LPT_A));
                            } else {
                                __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
                            }
                            phase_barrier();
                            if (kt + 2 < nk) {
#pragma unroll
                                for (int i = LPT_A; i < C::LPT; ++i) issue_b1(i, kt + 2, tor);
                            }
                            aw = next_buf(aw);
                        }
                        __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
                        phase_barrier();
                    }
                    return;
                }
            }
            if (nk > 0) {
                if constexpr (C::BLOCK_SCALE) {
                    fetch_a_scales(0, 0);
                    fetch_b_scales(0);
                    if constexpr (!SCALES_LDS) rotate_scales(0, 0);
                }
                if constexpr (!C::COPYW) first_copies();
                __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
                phase_barrier();
                if constexpr (SCALES_LDS) rotate_scales(0, 0);      // (the first group of scales is in LDS behind this barrier)
#pragma unroll
                for (int b = 0; b < C::TN; ++b) rd_b(0, b);
#pragma unroll
                for (int r = 0; r < AHEAD; ++r) rd_a(0, r, r);
                // B(0) is in registers everywhere before step 0 starts to overwrite its buffer
                __builtin_amdgcn_s_waitcnt(waitcnt_lgkm0());
                phase_barrier();
                typedef std::integral_constant<bool, true> yes_t;
                typedef std::integral_constant<bool, false> no_t;
                // the step whose copies (for step kt + 2) are those of a partial last step runs in the generic form
                // below, the only place where the copies carry the OR for the lanes past the end of K
                const int kt_tailc = kt_tail >= 2 ? kt_tail - 2 : 0x7fffffff;
                int kt = 0;
                {
                    // Six steps at a time (the A ring has three buffers, B two): inside the group the buffer of every
                    // read and copy is a constant, so the ring arithmetic (two dozen scalar and vector adds per
                    // step) folds into immediate offsets.  With one wave per SIMD what is not issued is MFMA time
                    // (bf16 -1.2 %, fp8 -1.2 %, int8 -0.8 % on 8192^3); the 8-wave block-scaled kernel gains 1.6 %.
                    for (; kt + 6 <= nk && kt + 6 <= kt_tailc; kt += 6) {
#pragma unroll
                        for (int j = 0; j < 6; ++j) {
                            a_rd = j % 3;
                            a_wr = (j + 2) % 3;
                            step(kt + j, j & 1, no_t{}, yes_t{});
                        }
                    }
                    if constexpr (C::BLOCK_SCALE && !PINNED) {       // what the last step of the groups left over
                        const float f = sc[(TMs - 1) % 2][((C::TN - 1) * 16) / 128];
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[TMs - 1][C::TN - 1][r] += (float)left_over[r] * f;
                    }
                    a_rd = 0;            // kt is a multiple of six here
                    a_wr = 2;
                }
                for (; kt + 2 <= nk; kt += 2) {
                    step(kt, 0, yes_t{}, no_t{});
                    step(kt + 1, 1, yes_t{}, no_t{});
                }
                if (kt < nk) step(kt, 0, yes_t{}, no_t{});
                __builtin_amdgcn_s_waitcnt(0x0070);      // copies landed, reads done, before LDS serves the epilogue
                phase_barrier();
                // the MFMAs above are opaque to the compiler's hazard handling: give the last one its wait states
                // before the epilogue reads the accumulators
                if constexpr (PINNED) asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
            }
        }
    } else {
        constexpr int NS = C::NSTAGE;
        // The barrier of a step: the bare s_barrier behind the wave's own wait for its
        // copies (counted, see below): __syncthreads() carries a fence that the compiler turns into "wait for every
        // copy in flight", which empties the ring at every step and leaves the stages issued ahead no time to land
        // under the MFMAs.  Fragment reads are complete before their MFMAs issue, so a wave that reaches the barrier
        // has left the buffers the next copies overwrite.  (The K-major tiles, whose transposing reads the compiler
        // orders behind all copies, take the full barrier.)
        auto ring_barrier = [&]() {
            if constexpr (C::KMAJ == 0) phase_barrier();
            else __syncthreads();
        };
        // Small tiles with a deep ring (NS >= 4): two K steps per barrier.  A workgroup of these is alone or nearly
        // alone on its CU and every step is a chain wait -> barrier -> fragment reads -> a handful of MFMAs, about
        // 0.25 - 0.36 us; taking the steps in pairs pays the barrier and the LDS latency once for two.  Before turn
        // kt (even) stages 0 .. kt+NS-3 have been issued; stages kt and kt+1 are waited for, everybody leaves the
        // buffers of kt-2 and kt-1, and stages kt+NS-2 and kt+NS-1 are issued into them.
        constexpr bool PAIRS = NS >= 4 && !C::BLOCK_SCALE && C::KMAJ == 0 && C::BM * C::BN <= 64 * 128 &&
                               C::KG == 1;
        if constexpr (C::KG == 2) {
            // Two sets of waves half a turn apart, and four waves that copy.  Phase s opens with a barrier; behind it
            // the set s & 1 reads the fragments of stage s while the other set runs the MFMAs of stage s-1 on the
            // fragments it read one phase earlier, and the copying waves issue stage s+NS-1 into the buffer of stage
            // s-1, which everybody has read (a reading wave waits for its fragments before the next barrier).  So
            // the fragment reads of one set and the copies run under the MFMAs of the other set, and a wave about
            // to multiply has nothing else to issue.  That is what the copying waves are for: a stage of copies
            // keeps the CU's vector memory path busy for 360 - 460 cycles, about as long as the 16 MFMAs of a stage
            // take (510), and a wave whose copy instructions queue there issues nothing else meanwhile.  With every
            // wave copying its share right behind the barrier the MFMAs of a stage took twice their time; with the
            // reading set copying between its fragment reads the read phase took 600 - 700 cycles (the LDS queue and
            // the memory queue each hold the wave up in turn).
            // Before the barrier of phase s a copying wave has waited for its quarter of stage s: everything it
            // issued since, NS-2 stages, may stay in flight.  nk + 1 phases, the same barriers for every wave (bare
            // barriers also for K-major tiles: no wave that reads LDS here has copies in flight).
            // (Touching the lines of later stages with plain loads, so that the copies would find them in the L2,
            // was tried and made the loop a quarter slower.)
            // Block scales: each copying wave adds one 4-byte-per-lane copy per stage that brings the a_scale values
            // of 64 tile rows (even waves rows 0 - 63, odd waves rows 64 - 127: the same bytes to the same place from
            // two waves, so that all of them count alike) to the stage's 512 bytes behind the ring.
            // That is one request per row and stage, as many again as the operands' own when the caller's a_scale is
            // K-contiguous (every lane another cache line: 2048 x 2048 x 8192 took 46 us where the same copies at
            // contiguous addresses take 37).  Where the host finds such an a_scale aligned for it (GemmArgs::as_groups)
            // a lane fetches the scales of four K blocks of its row at once, 16 bytes, in front of every fourth stage
            // (waves 0 and 1 of the copying four, 64 rows each), into slot (kt / 4) % 4 of four behind the ring:
            // [row][4 K blocks].  Slot i is refilled for stage 4 i + 16, issued in phase 4 i + 17 - NS, after the last
            // read of stage 4 i + 3.  These copies are not counted: a wave that waits until (NS - 2) * NPC copies are
            // left in flight has then waited for one or two operand copies more than it had to.
            constexpr int NPC = C::NLOAD / C::NPROD;                        // operand copies per stage and copying wave
            constexpr int CPS = NPC + (C::BLOCK_SCALE ? 1 : 0);
            static_assert(C::NPROD == 4 && C::NLOAD % 4 == 0 && C::RBA % 2 == 0 && (NS - 2) * CPS <= 63,
                          "copying waves: an even share each, copies in flight within the 6-bit counter");
            if (kg == 2) {
                // instruction q = pw + 4 * j of the stage (see issue_stage; pw = 0 .. 3, q & 1 = wave & 1): rows
                // 8 * (q & 1) .. + 7 of row block q >> 1, the first RBA row blocks are A's
                const int pw = wave & 3;
                const uint32_t as_voff_k2 = (row0 + 64 * (wave & 1) + lane) * p.as_ms * 4;
                // scalar offset of row block blk of an operand at K step kt: as load_soff
                auto soff_k2 = [&](bool kmajor, uint32_t blk, uint32_t ld, int kt) -> uint32_t {
                    constexpr uint32_t BPP = C::KE / 16;                        // row blocks per panel
                    const uint32_t k = (uint32_t)kpos(kt);
                    if (kmajor) return (k * C::KE + (blk % BPP) * 16) * ld + (blk / BPP) * 128;
                    return blk * 16 * ld + k * C::BKB;
                };
                auto issue_stage_k2 = [&](int kt, auto nt_tag) {          // (nt_tag: B's copies with the streaming hint)
                    constexpr bool B_NT = decltype(nt_tag)::value;
                    char *stage = smem + (kt % NS) * C::STAGE_BYTES + pw * 1024;
                    const bool tl = kpos(kt) == kt_tail;
                    const uint32_t va = tl ? voff_a_t : voff_a, vb = tl ? voff_b_t : voff_b;
#pragma unroll
                    for (int j = 0; j < NPC; ++j) {
                        lds_void *dst = (lds_void *)(stage + j * 4096);
                        const uint32_t blk = (pw >> 1) + 2 * j;
                        if (2 * j < C::RBA)
                            __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, dst, 16, va, soff_k2(C::KMA, blk, p.lda, kt), 0, 0);
                        else
                            __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, dst, 16, vb, soff_k2(C::KMB, blk - C::RBA, p.ldb, kt), 0, B_NT ? 2 : 0);
                    }
                    if constexpr (C::BLOCK_SCALE) {
                        if (!p.as_groups) {
                            lds_void *dst = (lds_void *)(smem + NS * C::STAGE_BYTES + (kt % NS) * 512 + (wave & 1) * 256);
                            __builtin_amdgcn_raw_ptr_buffer_load_lds(ras, dst, 4, as_voff_k2, (kbeg + (uint32_t)kpos(kt)) * p.as_ks * 4, 0, 0);
                        }
                    }
                };
                auto issue_scale_group = [&](int kt) {          // in front of the copies of stage kt
                    if constexpr (C::BLOCK_SCALE) {
                        if (p.as_groups && (kt & 3) == 0 && pw < C::BM / 64) {
                            lds_void *dst = (lds_void *)(smem + NS * C::STAGE_BYTES + ((kt >> 2) & 3) * (16 * C::BM) + pw * 1024);
                            __builtin_amdgcn_raw_ptr_buffer_load_lds(ras, dst, 16, as_voff_k2, (kbeg + (uint32_t)kpos(kt)) * 4, 0, 0);
                        }
                    }
                };
                // (the loop of a copying wave exists twice, with and without the streaming hint on B's copies: chosen per
                // copy inside one loop the branch cost these waves 2 - 4 %)
                auto copy_loop = [&](auto nt_tag) {
#pragma unroll
                    for (int j = 0; j < NS - 1; ++j)
                        if (j < nk) {
                            issue_scale_group(j);
                            issue_stage_k2(j, nt_tag);
                        }
                    const bool counted = !C::BLOCK_SCALE || !p.as_groups;       // the scale copies are among the CPS of a stage
                    for (int ph = 0; ph <= nk; ++ph) {
                        if (ph + NS - 2 >= nk) __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));      // near the end of K fewer are in flight
                        else if (counted) __builtin_amdgcn_s_waitcnt(waitcnt_vm((NS - 2) * CPS));
                        else __builtin_amdgcn_s_waitcnt(waitcnt_vm((NS - 2) * NPC));
                        phase_barrier();
                        if (ph + NS - 1 < nk) {
                            issue_scale_group(ph + NS - 1);
                            issue_stage_k2(ph + NS - 1, nt_tag);
                        }
                    }
                };
                if (p.b_stream) copy_loop(std::integral_constant<bool, true>{});
                else copy_loop(std::integral_constant<bool, false>{});
            } else {
                v4i fa[C::TM][2], fb[C::TN][2];
                auto read_stage = [&](int mine) {
                    if constexpr (C::BLOCK_SCALE) {
                        const int tr = wm * C::WM + (lane & 15);                    // tile row of this lane in row block 0
                        const char *sc = smem + NS * C::STAGE_BYTES +
                                         (p.as_groups ? ((mine >> 2) & 3) * (16 * C::BM) + tr * 16 + (mine & 3) * 4 : (mine % NS) * 512 + tr * 4);
                        const int rb = p.as_groups ? 256 : 64;                      // bytes from one row block to the next
#pragma unroll
                        for (int a = 0; a < C::TM; ++a) as_cur[a] = *(const float *)(sc + a * rb);
                        const uint32_t kb = kbeg + (uint32_t)kpos(mine);
#pragma unroll
                        for (int j = 0; j < NBS; ++j)
                            bs_cur[j] = p.bs[__builtin_amdgcn_readfirstlane(bs_off[j] + kb * p.bs_ks)];
                    }
                    const char *st = smem + (mine % NS) * C::STAGE_BYTES;
#pragma unroll
                    for (int a = 0; a < C::TM; ++a) {
                        fa[a][0] = frag_a(st, a, 0);
                        fa[a][1] = frag_a(st, a, 1);
                    }
#pragma unroll
                    for (int b = 0; b < C::TN; ++b) {
                        fb[b][0] = frag_b(st, b, 0);
                        fb[b][1] = frag_b(st, b, 1);
                    }
                    __builtin_amdgcn_s_waitcnt(waitcnt_lgkm0());   // reads done before the buffer may be refilled
                };
                auto mfma_stage = [&]() {
                    if constexpr (C::BLOCK_SCALE) {
                        // P * (as * bs), then accumulate (hip_mix_gemm_kernel.cpp:241 has (P * as) * bs: the factor
                        // formed first is one multiply per row and K block instead of four per MFMA).  Each MFMA starts
                        // from zero; its partial product is folded into the running sum two MFMAs later, so that the
                        // four FMAs of a tile run under the MFMAs that follow (straight after its own MFMA they would
                        // wait for it, and the next MFMA for them: 60 cycles a tile instead of 32; one MFMA behind, a
                        // register-only loop of this pattern takes 35 cycles a tile, two behind 33).
                        constexpr int NT = C::TM * C::TN, BEHIND = 2;
                        float f[C::TM][NBS];
#pragma unroll
                        for (int a = 0; a < C::TM; ++a)
#pragma unroll
                            for (int j = 0; j < NBS; ++j) f[a][j] = as_cur[a] * bs_cur[j];
                        part_t part[BEHIND + 1];
#pragma unroll
                        for (int i = 0; i < NT + BEHIND; ++i) {
                            if (i < NT) {
                                const int a = i % C::TM, b = i / C::TM;
                                part[i % (BEHIND + 1)] = mma128<C::ARITH>(fb[b][0], fb[b][1], fa[a][0], fa[a][1], part_t{0, 0, 0, 0});
                            }
                            __builtin_amdgcn_sched_barrier(0);       // MFMA i first, the FMAs of tile i-2 under it
                            if (i >= BEHIND) {
                                const int t = i - BEHIND, pa = t % C::TM, pb = t / C::TM;
#pragma unroll
                                for (int r = 0; r < 4; ++r) acc[pa][pb][r] += (float)part[t % (BEHIND + 1)][r] * f[pa][(pb * 16) / 128];
                            }
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    } else {
#pragma unroll
                        for (int b = 0; b < C::TN; ++b)
#pragma unroll
                            for (int a = 0; a < C::TM; ++a)
                                acc[a][b] = mma128<C::ARITH>(fb[b][0], fb[b][1], fa[a][0], fa[a][1], acc[a][b]);
                    }
                };
                int ph = 0;
                if (kg == 1) {                       // phase 0 of the second set: nothing to multiply yet
                    phase_barrier();
                    ph = 1;
                }
                for (; ph <= nk; ph += 2) {
                    phase_barrier();
                    if (ph < nk) read_stage(ph);
                    if (ph + 1 <= nk) {
                        phase_barrier();
                        mfma_stage();
                    }
                }
            }
        } else if constexpr (PAIRS) {
#pragma unroll
            for (int j = 0; j < NS - 2; ++j)
                if (j < nk) issue_stage(j);
            for (int kt = 0; kt < nk; kt += 2) {
                if (kt + NS - 2 <= nk) __builtin_amdgcn_s_waitcnt(waitcnt_vm((NS - 4) * C::LPT));
                else __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));      // near the end of K fewer are in flight
                ring_barrier();
                if (kt + NS - 2 < nk) issue_stage(kt + NS - 2);
                if (kt + NS - 1 < nk) issue_stage(kt + NS - 1);
                const bool two = kt + 1 < nk;
                const char *st0 = smem + (kt % NS) * C::STAGE_BYTES, *st1 = smem + ((kt + 1) % NS) * C::STAGE_BYTES;
                v4i fa[2][C::TM][2], fb[2][C::TN][2];
#pragma unroll
                for (int a = 0; a < C::TM; ++a) {
                    fa[0][a][0] = frag_a(st0, a, 0);
                    fa[0][a][1] = frag_a(st0, a, 1);
                }
#pragma unroll
                for (int b = 0; b < C::TN; ++b) {
                    fb[0][b][0] = frag_b(st0, b, 0);
                    fb[0][b][1] = frag_b(st0, b, 1);
                }
                if (two) {
#pragma unroll
                    for (int a = 0; a < C::TM; ++a) {
                        fa[1][a][0] = frag_a(st1, a, 0);
                        fa[1][a][1] = frag_a(st1, a, 1);
                    }
#pragma unroll
                    for (int b = 0; b < C::TN; ++b) {
                        fb[1][b][0] = frag_b(st1, b, 0);
                        fb[1][b][1] = frag_b(st1, b, 1);
                    }
                }
#pragma unroll
                for (int b = 0; b < C::TN; ++b)
#pragma unroll
                    for (int a = 0; a < C::TM; ++a)
                        acc[a][b] = mma128<C::ARITH>(fb[0][b][0], fb[0][b][1], fa[0][a][0], fa[0][a][1], acc[a][b]);
                if (two) {
#pragma unroll
                    for (int b = 0; b < C::TN; ++b)
#pragma unroll
                        for (int a = 0; a < C::TM; ++a)
                            acc[a][b] = mma128<C::ARITH>(fb[1][b][0], fb[1][b][1], fa[1][a][0], fa[1][a][1], acc[a][b]);
                }
            }
        } else {
        if (nk > 0) {
#pragma unroll
            for (int j = 0; j < NS - 1; ++j)
                if (j < nk) issue_stage(j);
            fetch_scales(0);
        }
        for (int kt = 0; kt < nk; ++kt) {
            // this wave's part of tile kt has landed: everything but the NS-2 stages issued after it
            // (near the end of K fewer are in flight: wait for all)
            if (NS > 2 && kt + NS - 2 < nk) __builtin_amdgcn_s_waitcnt(waitcnt_vm((NS - 2) * C::LPT));
            else __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
            ring_barrier();                                  // ... and everybody else's; tile kt-1 is fully consumed
            expand_scales();
            auto next_stage = [&]() {                        // into the buffer tile kt-1 has just left
                if (kt + NS - 1 < nk) issue_stage(kt + NS - 1);
            };
            // K-major tiles: all fragment reads of the step first, the copies behind them (see GemmCfg)
            constexpr bool READS_FIRST = C::KMAJ != 0;
            if constexpr (!READS_FIRST) next_stage();
            if (kt + 1 < nk) fetch_scales(kt + 1);
            const char *stage = smem + (kt % NS) * C::STAGE_BYTES;
            v4i fa[C::TM][2];
#pragma unroll
            for (int a = 0; a < C::TM; ++a) {
                fa[a][0] = frag_a(stage, a, 0);
                fa[a][1] = frag_a(stage, a, 1);
            }
            part_t part[2];                                  // block scales: the partial products of two tiles
            auto fold_tile = [&](int i) {
                const int pa = i % C::TM, pb = i / C::TM;
                const float f = as_cur[pa] * bs_cur[(pb * 16) / 128];
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[pa][pb][r] += (float)part[i & 1][r] * f;
            };
            v4i fball[READS_FIRST ? C::TN : 1][2];
            if constexpr (READS_FIRST) {
#pragma unroll
                for (int b = 0; b < C::TN; ++b) {
                    fball[b][0] = frag_b(stage, b, 0);
                    fball[b][1] = frag_b(stage, b, 1);
                }
                next_stage();
            }
#pragma unroll
            for (int b = 0; b < C::TN; ++b) {
                v4i fb0, fb1;
                if constexpr (READS_FIRST) {
                    fb0 = fball[b][0];
                    fb1 = fball[b][1];
                } else {
                    fb0 = frag_b(stage, b, 0);
                    fb1 = frag_b(stage, b, 1);
                }
#pragma unroll
                for (int a = 0; a < C::TM; ++a) {
                    if constexpr (C::BLOCK_SCALE) {
                        // P * (as * bs), then accumulate (hip_mix_gemm_kernel.cpp:241 has (P * as) * bs: the factor
                        // formed first is one multiply per row and K block instead of four per MFMA), one MFMA behind:
                        // the four FMAs of a tile go behind the MFMA of the next tile and run under it
                        const int i = b * C::TM + a;
                        part[i & 1] = mma128<C::ARITH>(fb0, fb1, fa[a][0], fa[a][1], part_t{0, 0, 0, 0});
                        if (i > 0) fold_tile(i - 1);
                    } else {
                        acc[a][b] = mma128<C::ARITH>(fb0, fb1, fa[a][0], fa[a][1], acc[a][b]);
                    }
                }
            }
            if constexpr (C::BLOCK_SCALE) fold_tile(C::TM * C::TN - 1);
        }
        }
    }

    QGEMM_STAMP(2);
    // ---- epilogue: lane holds C[m][n0 .. n0+3] of every 16x16 tile
    float scale = 1.0f;
    if (p.per_matrix_scale) scale = p.as[0] * p.bs[0];
    char *Cz = p.C + (size_t)z * p.split_stride * dtype_bytes(p.out_dtype);

    // Fast path: the wave tile lies inside C and rows of C are 16-byte aligned.  The accumulator
    // layout (adjacent lanes = adjacent rows of C) would make every lane of a store its own
    // request; so each 16-row slab goes through this wave's private LDS scratch and leaves as
    // whole 16-byte-per-lane row pieces.  Two scratch slabs per wave: slab a+1 is converted and
    // written while slab a is read back and stored.  The output type is dispatched once, outside
    // the slab loop, so the loop is straight-line code.  LDS is free here: the pipelined variants
    // end their K loop with every wave past a barrier that follows the last fragment read; the
    // simple pipeline needs one more barrier.
    constexpr int EPI_BYTES = 16 * (C::WN * 4 + 64);
    constexpr bool EPI_FITS = C::NW * 2 * EPI_BYTES <= C::LDS_BYTES && C::WN >= 32 && 64 % (C::WN * 2 / 16) == 0 && C::WN <= 256;
    if constexpr (C::KG == 2) {
        // set 1 hands its partial sums to set 0 through LDS (behind the epilogue scratch of set 0) and is done
        static_assert(EPI_FITS && (C::NW / 2) * 2 * EPI_BYTES + (C::NW / 2) * C::TM * C::TN * 1024 <= C::LDS_BYTES, "partial sums in LDS");
        char *part = smem + (C::NW / 2) * 2 * EPI_BYTES + wave_q * (C::TM * C::TN * 1024) + lane * 16;
        __syncthreads();                                   // every fragment read is over
        if (kg == 1) {
#pragma unroll
            for (int a = 0; a < C::TM; ++a)
#pragma unroll
                for (int b = 0; b < C::TN; ++b) *(acc_t *)(part + (a * C::TN + b) * 1024) = acc[a][b];
        }
        __syncthreads();
        if (kg >= 1) return;                               // set 1 and the copying waves are done
#pragma unroll
        for (int a = 0; a < C::TM; ++a)
#pragma unroll
            for (int b = 0; b < C::TN; ++b) {
                const acc_t o = *(const acc_t *)(part + (a * C::TN + b) * 1024);
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[a][b][r] += o[r];
            }
    } else if constexpr (C::PIPE == PIPE_SIMPLE && EPI_FITS) {
        __syncthreads();
    }
    // columns of the wave tile inside C; rows of it inside C (at most WM; none or fewer where the tile sticks out below)
    const bool wave_cols_full = col0 + wn * C::WN + C::WN <= p.N;
    const int wave_rows = (int)p.M - (int)(row0 + wm * C::WM);
    // Every accumulator is read in exactly one place (write_slab): the output type is a uniform branch around
    // the conversion of a slab, and wave tiles that stick out of C sideways or meet unaligned rows take the same way
    // through the scratch and differ only in how a slab leaves it (element by element, bounds checked).  A wave tile
    // that sticks out below C (M is whatever the caller's batch is; N and the alignment come with the weights)
    // keeps the 16-byte stores and leaves out the rows past M; so does one that sticks out sideways when the rows of C
    // end on a 16-byte boundary (its lanes past N leave their pieces out).
    // With the accumulators of a 128 x 128 wave tile pinned in the 256 accumulation registers, several code
    // paths that each name all of them made the register allocator spill two dozen of them to memory here.
    if constexpr (EPI_FITS) {
      const int DT = p.out_dtype;
      // the element size of the output is a compile-time constant of the slab code (two copies of it: the
      // addressing of the scratch depends on it); the type of that size is a uniform branch inside
      auto run = [&](auto es_tag, auto nt_tag) {
        constexpr int ES = decltype(es_tag)::value;
        constexpr bool NT_STORE = decltype(nt_tag)::value;
        // row pitch: 32 bytes (2-byte outputs, 8-byte writes) or 64 bytes (4-byte outputs, 16-byte
        // writes) past a multiple of 256, so the 16 rows a write instruction touches spread over all banks
        constexpr int PITCH = C::WN * ES + (ES == 2 ? 32 : 64);
        constexpr int LPR = C::WN * ES / 16;          // lanes per row when reading back
        constexpr int RPP = 64 / LPR;                 // rows per read instruction
        constexpr int PASSES = 16 / RPP;
        static_assert(16 * PITCH <= EPI_BYTES && PASSES >= 1, "scratch slab");
        char *scratch = smem + wave * (2 * EPI_BYTES);
        const int rd_row = lane / LPR, rd_col = (lane % LPR) * 16;
        const int wr_off = (lane & 15) * PITCH + (lane >> 4) * 4 * ES;
        const size_t c_row_bytes = (size_t)p.ldc * ES;
        const uint32_t wrow0 = row0 + wm * C::WM, wcol0 = col0 + wn * C::WN;
        // 16-byte stores: C and its rows aligned, and every 16-byte piece of a row either inside C or outside
        const bool fast = p.vec_store == 2 && (wave_cols_full || ((size_t)p.N * ES) % 16 == 0);
        const bool lane_in_cols = rd_col < ((int)p.N - (int)wcol0) * ES;
        char *cwave = Cz + ((size_t)wrow0 * p.ldc + wcol0) * ES;
        // Accumulators pinned in the accumulation registers (4-wave solo pipeline) are fetched from there one
        // slab at a time; left to itself the compiler moves all 256 of them into vector registers first.
        constexpr bool ACC_PINNED = C::PIPE == PIPE_SOLO && C::NW == 4 && !C::COPYW;
        auto acc_tile = [&](int a, int b) {
            if constexpr (ACC_PINNED) {
                acc_t t;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    typename std::remove_reference<decltype(t[0])>::type x;
                    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(x) : "a"(acc[a][b][r]));
                    t[r] = x;
                }
                return t;
            } else {
                return acc[a][b];
            }
        };
        auto write_slab = [&](int a) {
            char *wr = scratch + (a & 1) * EPI_BYTES + wr_off;
            if (ES == 4 && DT == QGEMM_DT_I32) {
#pragma unroll
                for (int b = 0; b < C::TN; ++b) *(acc_t *)(wr + b * 16 * 4) = acc_tile(a, b);
            } else {
                v4f v[C::TN];
#pragma unroll
                for (int b = 0; b < C::TN; ++b) {
                    const acc_t t = acc_tile(a, b);
#pragma unroll
                    for (int r = 0; r < 4; ++r) v[b][r] = (float)t[r] * scale;
                }
                if constexpr (ES == 4) {
#pragma unroll
                    for (int b = 0; b < C::TN; ++b) *(v4f *)(wr + b * 16 * 4) = v[b];
                } else if (DT == QGEMM_DT_BF16) {
#pragma unroll
                    for (int b = 0; b < C::TN; ++b)
                        *(v2i *)(wr + b * 16 * 2) = pack4_bf16(v[b][0], v[b][1], v[b][2], v[b][3]);
                } else {
#pragma unroll
                    for (int b = 0; b < C::TN; ++b)
                        *(v2i *)(wr + b * 16 * 2) = pack4_f16(v[b][0], v[b][1], v[b][2], v[b][3]);
                }
            }
        };
        write_slab(0);
#pragma unroll
        for (int a = 0; a < C::TM; ++a) {
            const char *slab = scratch + (a & 1) * EPI_BYTES;
            if (fast) {
                // read slab a back first (its writes were issued a turn ago; the LDS works in order), convert and
                // write slab a+1 while those reads are in flight, then store
                const char *rd = slab + rd_row * PITCH + rd_col;
                v4i v[PASSES];
#pragma unroll
                for (int ps = 0; ps < PASSES; ++ps) v[ps] = *(const v4i *)(rd + ps * RPP * PITCH);
                if (a + 1 < C::TM) write_slab(a + 1);
#pragma unroll
                for (int ps = 0; ps < PASSES; ++ps)
                    if (lane_in_cols && a * 16 + rd_row + ps * RPP < wave_rows) {
                        v4i *dst = (v4i *)(cwave + rd_col + (size_t)(a * 16 + rd_row + ps * RPP) * c_row_bytes);
                        if constexpr (NT_STORE) __builtin_nontemporal_store(v[ps], dst);
                        else *dst = v[ps];
                    }
            } else {
                if (a + 1 < C::TM) write_slab(a + 1);
                // any alignment, any overhang: one element per lane and turn
                for (int e = lane; e < 16 * C::WN; e += 64) {
                    const int r = e / C::WN, cidx = e % C::WN;
                    const uint32_t m = wrow0 + a * 16 + r, n = wcol0 + cidx;
                    if (m >= p.M || n >= p.N) continue;
                    char *dst = cwave + (size_t)(a * 16 + r) * c_row_bytes + (size_t)cidx * ES;
                    const char *src = slab + r * PITCH + cidx * ES;
                    if (ES == 2) *(unsigned short *)dst = *(const unsigned short *)src;
                    else *(uint32_t *)dst = *(const uint32_t *)src;
                }
            }
        }
      };
      // C leaves with non-temporal stores where rounds of tiles follow each other (less dirty L2 in the way of the next
      // round's panels: 1.5 - 3 % at 8192^3), with ordinary ones where the launch is one round at most: the caches then
      // take the burst of every CU writing at once and write it back behind the kernel
      typedef std::integral_constant<bool, true> nt_t;
      typedef std::integral_constant<bool, false> plain_t;
      if (DT == QGEMM_DT_BF16 || DT == QGEMM_DT_F16) {
          run(std::integral_constant<int, 2>{}, nt_t{});
      } else {
          if (p.c_plain) run(std::integral_constant<int, 4>{}, plain_t{});
          else run(std::integral_constant<int, 4>{}, nt_t{});
      }
        QGEMM_STAMP(3);
        QGEMM_STAMP_WRITE(p.dbg_cycles, blockIdx.x * C::NW + wave, 4, lane == 0);
        return;
    }
#pragma unroll
    for (int a = 0; a < C::TM; ++a) {
        const uint32_t m = row0 + wm * C::WM + a * 16 + (lane & 15);
        if (m >= p.M) continue;
#pragma unroll
        for (int b = 0; b < C::TN; ++b) {
            const uint32_t n = col0 + wn * C::WN + b * 16 + (lane >> 4) * 4;
            if (n >= p.N) continue;
            const size_t idx = (size_t)m * p.ldc + n;
            const bool full = p.vec_store && n + 3 < p.N;
            if constexpr (C::ARITH == AR_I8 && !C::BLOCK_SCALE) {
                if (p.out_dtype == QGEMM_DT_I32) {
                    int *dst = (int *)Cz + idx;
                    if (full) *(v4i *)dst = acc[a][b];
                    else
                        for (int r = 0; r < 4; ++r)
                            if (n + r < p.N) dst[r] = acc[a][b][r];
                    continue;
                }
            }
            float v[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] = (float)acc[a][b][r] * scale;
            if (p.out_dtype == QGEMM_DT_F32) {
                float *dst = (float *)Cz + idx;
                if (full) *(v4f *)dst = v4f{v[0], v[1], v[2], v[3]};
                else
                    for (int r = 0; r < 4; ++r)
                        if (n + r < p.N) dst[r] = v[r];
            } else {
                const v2i h = p.out_dtype == QGEMM_DT_BF16 ? pack4_bf16(v[0], v[1], v[2], v[3]) : pack4_f16(v[0], v[1], v[2], v[3]);
                unsigned short *dst = (unsigned short *)Cz + idx;
                if (full) *(v2i *)dst = h;
                else
                    for (int r = 0; r < 4; ++r)
                        if (n + r < p.N) dst[r] = pack4_elem(h, r);
            }
        }
    }
    QGEMM_STAMP(3);
    QGEMM_STAMP_WRITE(p.dbg_cycles, blockIdx.x * C::NW + wave, 4, lane == 0);
#endif
}

}  // namespace qgemm
