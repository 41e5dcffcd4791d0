// MFMA GEMM kernel for gfx950, "NT" operands: A is M x K, B is N x K, both with
// K contiguous.  One template covers int8, fp8-e4m3, bf16 and fp16 inputs.
//
// Replaces the device kernels of the reference:
//   GEMM_kernel_bf16_v1..v5      src/gemm/sm89_gemm_kernel_v{1,2,3,4,5}.cu
//   FP8_GEMM_kernel              src/mix_gemm/hip_mix_gemm_kernel.cpp:249-378
// It is not a translation of either: the tiling, the LDS layout and the load
// path are built around the CDNA4 matrix core.
//
// Data movement
//   * A K step is 128 bytes of every tile row (128 fp8/int8 or 64 bf16/fp16).
//   * Global -> LDS goes through buffer_load_dwordx4 ... lds (no VGPR staging).
//     One such instruction moves a 1 KiB "fragment block": 16 tile rows x 64
//     bytes of K.  Lane l fetches row (l & 15), bytes 16*(l >> 4) .. +16 of the
//     64, and the hardware stores lane l's 16 bytes at block + 16*l.
//   * That is exactly the operand order of the 16-row MFMA instructions (row =
//     lane & 15, K group = lane >> 4), so a fragment is read back with one
//     ds_read_b128 per lane at block + 16*lane: consecutive lanes read
//     consecutive 16-byte words, which is free of bank conflicts by
//     construction and needs no per-read address arithmetic.  (Which K bytes a
//     lane group holds does not matter as long as A and B agree: the
//     contraction index is summed away.)
//   * LDS holds two stages (double buffer).  Tile k+1 is in flight while the
//     matrix cores work on tile k; one s_barrier per K step.
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
#include "common.h"

namespace qgemm {

struct GemmArgs {
    const char *A;        // M x K, row stride lda bytes
    const char *B;        // N x K, row stride ldb bytes
    char *C;              // M x N row-major, ldc elements; split-K: plane z at C + z*split_stride elements
    const float *as;      // per-matrix: 1 float; block: as[m*as_ms + kb*as_ks]
    const float *bs;      // per-matrix: 1 float; block: bs[nb*bs_ns + kb*bs_ks]
    uint32_t M, N;
    uint32_t ksteps;      // K steps of 128 bytes in total
    uint32_t lda, ldb;    // bytes
    uint32_t ldc;         // elements
    uint32_t tiles_m, tiles_n, group_m;
    uint32_t nsplit, ksteps_per_split;
    uint64_t split_stride;
    uint32_t as_ms, as_ks, bs_ns, bs_ks;
    uint32_t nb_max;      // ceil(N/128) - 1
    int out_dtype;        // qgemm_dtype_t of C
    int per_matrix_scale; // multiply by as[0]*bs[0] in the epilogue
    int vec_store;        // C and ldc allow 16-byte (f32/i32) / 8-byte (16-bit) vector stores
};

// How a stage travels from global memory to LDS.
//   LOAD_DMA   buffer_load_dwordx4 ... lds: no VGPR staging, the wave only waits on vmcnt
//   LOAD_VGPR  buffer_load_dwordx4 into registers during the MFMAs of the previous
//              tile, ds_write_b128 afterwards; same LDS layout
enum Loader : int { LOAD_DMA = 0, LOAD_VGPR = 1 };

template <int ARITH_, bool BLOCK_SCALE_, int BM_, int BN_, int WAVES_M_, int WAVES_N_, int LOADER_ = LOAD_DMA>
struct GemmCfg {
    static constexpr int LOADER = LOADER_;
    static constexpr int ARITH = ARITH_;
    static constexpr bool BLOCK_SCALE = BLOCK_SCALE_;
    static constexpr int BM = BM_, BN = BN_, BKB = 128;         // BKB: bytes of K per step
    static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
    static constexpr int NW = WAVES_M * WAVES_N;
    static constexpr int THREADS = NW * kWave;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;  // wave tile
    static constexpr int TM = WM / 16, TN = WN / 16;            // 16x16 MFMA tiles per wave
    static constexpr int NA = BM / 16 * 2, NB = BN / 16 * 2;    // 1 KiB fragment blocks per stage
    static constexpr int LPT = (NA + NB) / NW;                  // DMA instructions per wave per stage
    static constexpr int STAGE_BYTES = (NA + NB) * 1024;
    static constexpr int NSTAGE = 2;
    static constexpr int LDS_BYTES = STAGE_BYTES * NSTAGE;
    static_assert(BM % (16 * WAVES_M) == 0 && BN % (16 * WAVES_N) == 0, "wave tile must be a multiple of 16");
    static_assert((NA + NB) % NW == 0, "fragment blocks must divide evenly over the waves");
    static_assert(!BLOCK_SCALE || ARITH == AR_F8, "block scales are defined for fp8 only");
    static_assert(!BLOCK_SCALE || (128 % WN == 0 || WN % 128 == 0), "wave tile must align with 128-wide scale blocks");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS is 160 KiB per CU");
};

typedef __attribute__((address_space(3))) void lds_void;

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void *base, uint32_t bytes) {
    // raw buffer, 32-bit data format word as used for untyped loads on gfx9
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes, 0x00020000);
}

// vmcnt(n) only (expcnt / lgkmcnt left at "no wait"), gfx9 encoding.
__device__ inline constexpr int waitcnt_vm(int n) { return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8); }

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

template <class C>
__global__ void __launch_bounds__(C::THREADS) gemm_nt_kernel(const GemmArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass only needs the launch stub
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    typedef typename AccT<C::ARITH>::type acc_t;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;

    // ---- which tile, which K slice
    uint32_t wg = blockIdx.x, z = 0;
    if (p.nsplit > 1) {
        z = wg % p.nsplit;
        wg /= p.nsplit;
    }
    uint32_t tm, tn;
    tile_map(wg, p.tiles_m, p.tiles_n, p.group_m, tm, tn);
    const uint32_t row0 = tm * C::BM, col0 = tn * C::BN;
    const uint32_t kbeg = z * p.ksteps_per_split;
    const uint32_t kend = kbeg + p.ksteps_per_split < p.ksteps ? kbeg + p.ksteps_per_split : p.ksteps;
    const int nk = (int)(kend - kbeg);

    // ---- buffer resources: base at this tile's first row and first K byte; the
    // range ends with the last valid row, so rows past M / N read as out of
    // range (never a fault) and only ever feed outputs that are not stored.
    const uint32_t a_rows = p.M - row0 < (uint32_t)C::BM ? p.M - row0 : C::BM;
    const uint32_t b_rows = p.N - col0 < (uint32_t)C::BN ? p.N - col0 : C::BN;
    const uint32_t kbytes = (uint32_t)nk * C::BKB;
    const __amdgpu_buffer_rsrc_t ra =
        make_rsrc(p.A + (size_t)row0 * p.lda + (size_t)kbeg * C::BKB, (a_rows - 1) * p.lda + kbytes);
    const __amdgpu_buffer_rsrc_t rb =
        make_rsrc(p.B + (size_t)col0 * p.ldb + (size_t)kbeg * C::BKB, (b_rows - 1) * p.ldb + kbytes);

    // per-lane byte offsets of the LPT fragment blocks this wave fetches each stage
    uint32_t voff[C::LPT];
    bool isA[C::LPT];
#pragma unroll
    for (int i = 0; i < C::LPT; ++i) {
        const int q = wave + i * C::NW;               // fragment block id within the stage
        isA[i] = q < C::NA;
        const int qq = isA[i] ? q : q - C::NA;
        const uint32_t rowl = (qq >> 1) * 16 + (lane & 15);
        voff[i] = rowl * (isA[i] ? p.lda : p.ldb) + (qq & 1) * 64 + (lane >> 4) * 16;
    }

    auto issue_stage = [&](int kt) {
        char *stage = smem + (kt & 1) * C::STAGE_BYTES;
        const uint32_t soff = (uint32_t)kt * C::BKB;
#pragma unroll
        for (int i = 0; i < C::LPT; ++i) {
            const int q = wave + i * C::NW;
            lds_void *dst = (lds_void *)(stage + q * 1024);
            if (isA[i])
                __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, dst, 16, voff[i], soff, 0, 0);
            else
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, dst, 16, voff[i], soff, 0, 0);
        }
    };

    v4i staged[C::LOADER == LOAD_VGPR ? C::LPT : 1];
    auto fetch_stage = [&](int kt) {       // LOAD_VGPR: global -> registers
        const uint32_t soff = (uint32_t)kt * C::BKB;
#pragma unroll
        for (int i = 0; i < C::LPT; ++i)
            staged[i] = isA[i] ? __builtin_amdgcn_raw_buffer_load_b128(ra, voff[i], soff, 0)
                               : __builtin_amdgcn_raw_buffer_load_b128(rb, voff[i], soff, 0);
    };
    auto commit_stage = [&](int kt) {      // LOAD_VGPR: registers -> LDS, same layout as the DMA path
        char *stage = smem + (kt & 1) * C::STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < C::LPT; ++i) *(v4i *)(stage + (wave + i * C::NW) * 1024 + lane * 16) = staged[i];
    };

    // ---- block scales (fp8 only): a_scale per row of each A fragment, b_scale per 128 columns
    constexpr int NBS = C::BLOCK_SCALE ? (C::WN + 127) / 128 : 1;
    float as_cur[C::TM], as_nxt[C::TM], bs_cur[NBS], bs_nxt[NBS];
    uint32_t as_off[C::TM], bs_off[NBS];
    if constexpr (C::BLOCK_SCALE) {
#pragma unroll
        for (int a = 0; a < C::TM; ++a) {
            uint32_t m = row0 + wm * C::WM + a * 16 + (lane & 15);
            m = m < p.M ? m : p.M - 1;
            as_off[a] = m * p.as_ms;
        }
#pragma unroll
        for (int j = 0; j < NBS; ++j) {
            uint32_t nb = (col0 + wn * C::WN) / 128 + j;
            nb = nb < p.nb_max ? nb : p.nb_max;
            bs_off[j] = nb * p.bs_ns;
        }
    }
    auto load_scales = [&](int kt, float *as_v, float *bs_v) {
        if constexpr (C::BLOCK_SCALE) {
            const uint32_t kb = kbeg + kt;
#pragma unroll
            for (int a = 0; a < C::TM; ++a) as_v[a] = p.as[as_off[a] + kb * p.as_ks];
#pragma unroll
            for (int j = 0; j < NBS; ++j) bs_v[j] = p.bs[bs_off[j] + kb * p.bs_ks];
        }
    };

    acc_t acc[C::TM][C::TN];
#pragma unroll
    for (int a = 0; a < C::TM; ++a)
#pragma unroll
        for (int b = 0; b < C::TN; ++b) acc[a][b] = acc_t{0, 0, 0, 0};

    const int lane_off = lane * 16;
    const int a_frag0 = (wm * C::TM * 2) * 1024 + lane_off;
    const int b_frag0 = (C::NA + wn * C::TN * 2) * 1024 + lane_off;

    // ---- K loop
    if (nk > 0) {
        if constexpr (C::LOADER == LOAD_DMA) {
            issue_stage(0);
        } else {
            fetch_stage(0);
            commit_stage(0);
        }
        load_scales(0, as_nxt, bs_nxt);
    }
    for (int kt = 0; kt < nk; ++kt) {
        if constexpr (C::LOADER == LOAD_DMA)
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));   // this wave's part of tile kt has landed
        __syncthreads();                                 // ... and everybody else's; tile kt-1 is fully consumed
        if constexpr (C::BLOCK_SCALE) {
#pragma unroll
            for (int a = 0; a < C::TM; ++a) as_cur[a] = as_nxt[a];
#pragma unroll
            for (int j = 0; j < NBS; ++j) bs_cur[j] = bs_nxt[j];
        }
        if (kt + 1 < nk) {
            if constexpr (C::LOADER == LOAD_DMA) issue_stage(kt + 1);
            else fetch_stage(kt + 1);
            load_scales(kt + 1, as_nxt, bs_nxt);
        }
        const char *stage = smem + (kt & 1) * C::STAGE_BYTES;
        v4i fa[C::TM][2];
#pragma unroll
        for (int a = 0; a < C::TM; ++a) {
            fa[a][0] = *(const v4i *)(stage + a_frag0 + (a * 2 + 0) * 1024);
            fa[a][1] = *(const v4i *)(stage + a_frag0 + (a * 2 + 1) * 1024);
        }
#pragma unroll
        for (int b = 0; b < C::TN; ++b) {
            const v4i fb0 = *(const v4i *)(stage + b_frag0 + (b * 2 + 0) * 1024);
            const v4i fb1 = *(const v4i *)(stage + b_frag0 + (b * 2 + 1) * 1024);
#pragma unroll
            for (int a = 0; a < C::TM; ++a) {
                if constexpr (C::BLOCK_SCALE) {
                    // (P * as) * bs, then accumulate: hip_mix_gemm_kernel.cpp:241
                    const v4f part = mma128<C::ARITH>(fb0, fb1, fa[a][0], fa[a][1], v4f{0, 0, 0, 0});
                    const float sa = as_cur[a], sb = bs_cur[(b * 16) / 128];
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[a][b][r] += (part[r] * sa) * sb;
                } else {
                    acc[a][b] = mma128<C::ARITH>(fb0, fb1, fa[a][0], fa[a][1], acc[a][b]);
                }
            }
        }
        if constexpr (C::LOADER == LOAD_VGPR) {
            // the other stage was last read in iteration kt-1, which every wave left before this one began
            if (kt + 1 < nk) commit_stage(kt + 1);
        }
    }

    // ---- epilogue: lane holds C[m][n0 .. n0+3] of every 16x16 tile
    float scale = 1.0f;
    if (p.per_matrix_scale) scale = p.as[0] * p.bs[0];
    char *Cz = p.C + (size_t)z * p.split_stride * dtype_bytes(p.out_dtype);
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
            if constexpr (C::ARITH == AR_I8) {
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
                unsigned short h[4];
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    h[r] = p.out_dtype == QGEMM_DT_BF16 ? f32_to_bf16_bits(v[r]) : f32_to_f16_bits(v[r]);
                unsigned short *dst = (unsigned short *)Cz + idx;
                if (full) *(us4 *)dst = us4{h[0], h[1], h[2], h[3]};
                else
                    for (int r = 0; r < 4; ++r)
                        if (n + r < p.N) dst[r] = h[r];
            }
        }
    }
#endif
}

}  // namespace qgemm
