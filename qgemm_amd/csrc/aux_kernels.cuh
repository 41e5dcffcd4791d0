// Kernels around the MFMA GEMM: the any-shape strided GEMM, the transpose, the
// split-K reduction.
#pragma once
#include "common.h"

namespace qgemm {

// ---------------------------------------------------------------------------
// element decode (software; used only by the any-shape kernel)
// ---------------------------------------------------------------------------
__device__ inline float decode_fp8_e4m3(uint8_t b) {
    // OCP e4m3: 1-4-3, bias 7, subnormals m * 2^-9, 0x7F / 0xFF NaN
    const uint32_t sign = (uint32_t)(b & 0x80u) << 24;
    const uint32_t exp = (b >> 3) & 0xFu, mant = b & 7u;
    float mag;
    if (exp == 0) mag = (float)mant * 0.001953125f;
    else if (exp == 15 && mant == 7) mag = __builtin_nanf("");
    else mag = __builtin_bit_cast(float, ((exp + 120u) << 23) | (mant << 20));
    return __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, mag) | sign);
}

template <int IN_DT>
__device__ inline float load_elem(const void *p, size_t i) {
    if constexpr (IN_DT == QGEMM_DT_F8E4M3) return decode_fp8_e4m3(((const uint8_t *)p)[i]);
    else if constexpr (IN_DT == QGEMM_DT_I8) return (float)((const int8_t *)p)[i];
    else if constexpr (IN_DT == QGEMM_DT_BF16)
        return __builtin_bit_cast(float, (uint32_t)((const uint16_t *)p)[i] << 16);
    else return (float)((const _Float16 *)p)[i];
}

__device__ inline void store_out(void *C, size_t idx, float v, int out_dtype) {
    if (out_dtype == QGEMM_DT_F32) ((float *)C)[idx] = v;
    else if (out_dtype == QGEMM_DT_BF16) ((unsigned short *)C)[idx] = f32_to_bf16_bits(v);
    else ((unsigned short *)C)[idx] = f32_to_f16_bits(v);
}

// ---------------------------------------------------------------------------
// Any-shape, any-stride GEMM: one thread per C element.  Carries the shapes the
// MFMA kernel does not take (K not a multiple of 128 bytes).  Same arithmetic
// contract: int32 accumulation for int8, fp32 otherwise; block scales folded in
// per `bk` K elements as (P * as) * bs  (hip_mix_gemm_kernel.cpp:231-244).
// ---------------------------------------------------------------------------
struct StridedArgs {
    const void *A, *B;
    void *C;
    const float *as, *bs;
    uint32_t M, N, K;
    uint64_t a_rs, a_cs, b_ns, b_ks;  // element strides
    uint64_t ldc;
    uint32_t as_ms, as_ks, bs_ns, bs_ks;
    uint32_t bk;                      // K elements per partial product in block mode
    int out_dtype, scale_mode;        // scale_mode: 0 none, 1 per matrix, 2 block
};

template <int IN_DT>
__global__ void __launch_bounds__(256) gemm_strided_kernel(const StridedArgs p) {
    const uint32_t n = blockIdx.x * 16 + (threadIdx.x & 15);
    const uint32_t m = blockIdx.y * 16 + (threadIdx.x >> 4);
    if (m >= p.M || n >= p.N) return;
    const size_t idx = (size_t)m * p.ldc + n;
    if constexpr (IN_DT == QGEMM_DT_I8) {
        const int8_t *a = (const int8_t *)p.A + (size_t)m * p.a_rs;
        const int8_t *b = (const int8_t *)p.B + (size_t)n * p.b_ns;
        if (p.scale_mode == 2) {           // exact int32 partial per 128-wide K block, folded in fp32
            float accf = 0.0f;
            for (uint32_t k0 = 0; k0 < p.K; k0 += kScaleBlock) {
                const uint32_t k1 = k0 + kScaleBlock < p.K ? k0 + kScaleBlock : p.K;
                int part = 0;
                for (uint32_t k = k0; k < k1; ++k) part += (int)a[k * p.a_cs] * (int)b[k * p.b_ks];
                const uint32_t kb = k0 / kScaleBlock;
                accf += ((float)part * p.as[(size_t)m * p.as_ms + (size_t)kb * p.as_ks]) *
                        p.bs[(size_t)(n / kScaleBlock) * p.bs_ns + (size_t)kb * p.bs_ks];
            }
            store_out(p.C, idx, accf, p.out_dtype);
            return;
        }
        int acc = 0;
        for (uint32_t k = 0; k < p.K; ++k) acc += (int)a[k * p.a_cs] * (int)b[k * p.b_ks];
        if (p.out_dtype == QGEMM_DT_I32) {
            ((int *)p.C)[idx] = acc;
            return;
        }
        const float s = p.scale_mode == 1 ? p.as[0] * p.bs[0] : 1.0f;
        store_out(p.C, idx, (float)acc * s, p.out_dtype);
        return;
    }
    float acc = 0.0f;
    if (p.scale_mode == 2) {
        for (uint32_t k0 = 0; k0 < p.K; k0 += p.bk) {
            const uint32_t k1 = k0 + p.bk < p.K ? k0 + p.bk : p.K;
            float part = 0.0f;
            for (uint32_t k = k0; k < k1; ++k)
                part += load_elem<IN_DT>(p.A, (size_t)m * p.a_rs + k * p.a_cs) *
                        load_elem<IN_DT>(p.B, (size_t)n * p.b_ns + k * p.b_ks);
            const uint32_t kb = k0 / kScaleBlock;
            acc += (part * p.as[(size_t)m * p.as_ms + (size_t)kb * p.as_ks]) *
                   p.bs[(size_t)(n / kScaleBlock) * p.bs_ns + (size_t)kb * p.bs_ks];
        }
        store_out(p.C, idx, acc, p.out_dtype);
        return;
    }
    for (uint32_t k = 0; k < p.K; ++k)
        acc += load_elem<IN_DT>(p.A, (size_t)m * p.a_rs + k * p.a_cs) *
               load_elem<IN_DT>(p.B, (size_t)n * p.b_ns + k * p.b_ks);
    const float s = p.scale_mode == 1 ? p.as[0] * p.bs[0] : 1.0f;
    store_out(p.C, idx, acc * s, p.out_dtype);
}

// ---------------------------------------------------------------------------
// Transpose: out[n*M + m] = in[m*N + n]   (src/transpose/transpose.cu:11-58).
// 64 x 64 element tile through LDS, 256 threads.  The LDS tile is stored with
// its 4-byte words XOR-swizzled by the row, so both the row-wise fill and the
// column-wise drain touch 32 distinct banks; no padding column.  Any M, N.
// ---------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256) transpose_kernel(const T *__restrict__ in, T *__restrict__ out, uint32_t M,
                                                        uint32_t N) {
    constexpr int TILE = 64;
    __shared__ T tile[TILE][TILE];
    const uint32_t m0 = blockIdx.y * TILE, n0 = blockIdx.x * TILE;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;   // 64 x 4
    constexpr int PER_WORD = sizeof(T) >= 4 ? 1 : 4 / sizeof(T);
#pragma unroll
    for (int r = ty; r < TILE; r += 4) {
        const uint32_t m = m0 + r, n = n0 + tx;
        if (m < M && n < N) {
            const int word = (tx / PER_WORD) ^ (r & (TILE / PER_WORD - 1));
            tile[r][word * PER_WORD + tx % PER_WORD] = in[(size_t)m * N + n];
        }
    }
    __syncthreads();
#pragma unroll
    for (int r = ty; r < TILE; r += 4) {
        const uint32_t n = n0 + r, m = m0 + tx;   // output row n, column m
        if (n < N && m < M) {
            const int word = (r / PER_WORD) ^ (tx & (TILE / PER_WORD - 1));
            out[(size_t)n * M + m] = tile[tx][word * PER_WORD + r % PER_WORD];
        }
    }
}

// ---------------------------------------------------------------------------
// Byte transpose for shapes with M % 16 == 0, N % 4 == 0 and 16-byte aligned rows (the fp8 / int8
// operands of the reference layout).  128 x 128 tile, 256 threads.  A thread loads 4 x 4 bytes (four
// rows, one dword each: a wave reads whole 128-byte row pieces), transposes the 4 x 4 block in
// registers with byte permutes, and writes the four resulting dwords (4 consecutive m of one n)
// into the LDS tile [n][m]; the tile leaves as 16-byte pieces of output rows, 128 bytes per row.
// ---------------------------------------------------------------------------
// One 128 x 128 tile of the byte transpose (tile_m, tile_n in tiles)
__device__ inline void transpose_bytes_tile(const uint8_t *__restrict__ in, uint8_t *__restrict__ out, uint32_t M,
                                            uint32_t N, uint32_t tile_m, uint32_t tile_n) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr int T = 128, PITCH = T + 16;        // bytes per LDS row
    __shared__ __attribute__((aligned(16))) uint8_t tile[T * PITCH];
    const uint32_t m0 = tile_m * T, n0 = tile_n * T;
    const int cg = threadIdx.x & 31, rg = threadIdx.x >> 5;      // 32 column groups of 4 bytes x 8 row groups of 16
    const uint32_t n = n0 + cg * 4;
#pragma unroll
    for (int ch = 0; ch < 4; ++ch) {
        const uint32_t m = m0 + rg * 16 + ch * 4;
        uint32_t a = 0, b = 0, c = 0, d = 0;
        if (n < N && m < M) {                     // M % 4 == 0: the four rows are all inside or all outside
            const uint8_t *src = in + (size_t)m * N + n;
            a = *(const uint32_t *)src;
            b = *(const uint32_t *)(src + N);
            c = *(const uint32_t *)(src + 2 * (size_t)N);
            d = *(const uint32_t *)(src + 3 * (size_t)N);
        }
        // v_perm_b32: selector byte k picks byte k of the result out of {src1 bytes 0-3, src0 bytes 4-7}
        const uint32_t ab_lo = __builtin_amdgcn_perm(b, a, 0x05010400), ab_hi = __builtin_amdgcn_perm(b, a, 0x07030602);
        const uint32_t cd_lo = __builtin_amdgcn_perm(d, c, 0x05010400), cd_hi = __builtin_amdgcn_perm(d, c, 0x07030602);
        const uint32_t o0 = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100), o1 = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302);
        const uint32_t o2 = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100), o3 = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302);
        uint8_t *dst = tile + (cg * 4) * PITCH + rg * 16 + ch * 4;   // [n - n0][m - m0]
        *(uint32_t *)dst = o0;
        *(uint32_t *)(dst + PITCH) = o1;
        *(uint32_t *)(dst + 2 * PITCH) = o2;
        *(uint32_t *)(dst + 3 * PITCH) = o3;
    }
    __syncthreads();
    const int piece = threadIdx.x & 7, row = threadIdx.x >> 3;   // 8 pieces of 16 bytes per output row, 32 rows per pass
#pragma unroll
    for (int ps = 0; ps < 4; ++ps) {
        const int r = row + ps * 32;
        const uint32_t on = n0 + r, om = m0 + piece * 16;
        if (on < N && om < M) *(v4i *)(out + (size_t)on * M + om) = *(const v4i *)(tile + r * PITCH + piece * 16);
    }
#endif
}

__global__ void __launch_bounds__(256) transpose_bytes_kernel(const uint8_t *__restrict__ in, uint8_t *__restrict__ out,
                                                              uint32_t M, uint32_t N) {
    transpose_bytes_tile(in, out, M, N, blockIdx.y, blockIdx.x);
}

// Two byte transposes in one launch (both operands of the reference fp8 layout: the second launch costs more
// than either transpose takes on mid-size shapes): workgroups 0 .. tiles0-1 take matrix 0, the rest matrix 1.
struct Transpose2Args {
    const uint8_t *in[2];
    uint8_t *out[2];
    uint32_t M[2], N[2], tiles_n[2], tiles0;
};
__global__ void __launch_bounds__(256) transpose_bytes2_kernel(const Transpose2Args a) {
    const uint32_t which = blockIdx.x >= a.tiles0 ? 1u : 0u, t = blockIdx.x - (which ? a.tiles0 : 0u);
    transpose_bytes_tile(a.in[which], a.out[which], a.M[which], a.N[which], t / a.tiles_n[which], t % a.tiles_n[which]);
}

// ---------------------------------------------------------------------------
// 2-byte transpose for shapes with M % 8 == 0, N % 8 == 0 and 16-byte aligned rows (what
// matrix_transpose<bf16 / fp16> of the reference is called with, src/transpose/transpose.cu:60-74).
// No LDS: a lane owns an 8 x 8 block.  It loads eight 16-byte row pieces, interleaves the 16-bit halves
// of vertically adjacent dwords (one v_perm each: 32 per block), and the rest of the transposition is
// which register goes into which output dword.  Lanes 8g..8g+7 hold eight neighbouring column blocks,
// so every load instruction reads 128-byte pieces of 8 rows; lanes g, g+8, .. hold neighbouring row
// blocks, so every store instruction writes 128-byte pieces of 8 output rows.  A wave covers 64 x 64
// elements, a workgroup of four waves 64 rows x 256 columns.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256) transpose_u16_kernel(const uint16_t *__restrict__ in, uint16_t *__restrict__ out,
                                                            uint32_t M, uint32_t N) {
#if defined(__HIP_DEVICE_COMPILE__)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t m = blockIdx.y * 64 + (lane >> 3) * 8;                   // first of this lane's 8 rows
    const uint32_t n = blockIdx.x * 256 + wave * 64 + (lane & 7) * 8;       // first of its 8 columns
    if (m >= M || n >= N) return;                                           // blocks are wholly in or out
    v4i row[8];
    const uint16_t *src = in + (size_t)m * N + n;
#pragma unroll
    for (int j = 0; j < 8; ++j) row[j] = *(const v4i *)(src + (size_t)j * N);
    // pair[i][k] = columns 2k (low perm) and 2k+1 (high perm) of rows 2i, 2i+1
    uint32_t lo[4][4], hi[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t a = (uint32_t)row[2 * i][k], b = (uint32_t)row[2 * i + 1][k];
            lo[i][k] = __builtin_amdgcn_perm(b, a, 0x05040100);     // (a.lo16, b.lo16)
            hi[i][k] = __builtin_amdgcn_perm(b, a, 0x07060302);     // (a.hi16, b.hi16)
        }
    uint16_t *dst = out + (size_t)n * M + m;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const v4i even = {(int)lo[0][k], (int)lo[1][k], (int)lo[2][k], (int)lo[3][k]};
        const v4i odd = {(int)hi[0][k], (int)hi[1][k], (int)hi[2][k], (int)hi[3][k]};
        *(v4i *)(dst + (size_t)(2 * k) * M) = even;
        *(v4i *)(dst + (size_t)(2 * k + 1) * M) = odd;
    }
#endif
}

// ---------------------------------------------------------------------------
// Split-K second pass: C[m,n] = cast(scale * sum_z part[z][m,n]), z ascending
// (a fixed order, so results do not depend on scheduling; int32 stays exact).
// ---------------------------------------------------------------------------
struct ReduceArgs {
    const void *part;      // [nsplit][M][N] f32 or i32
    void *C;
    const float *as, *bs;
    uint32_t M, N, nsplit;
    uint64_t ldc, plane;   // plane = M*N elements
    int part_is_i32, out_dtype, per_matrix_scale;
};

__global__ void __launch_bounds__(256) splitk_reduce_kernel(const ReduceArgs p) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= p.plane) return;
    const uint32_t m = (uint32_t)(i / p.N), n = (uint32_t)(i % p.N);
    const size_t idx = (size_t)m * p.ldc + n;
    if (p.part_is_i32) {
        int acc = 0;
        for (uint32_t z = 0; z < p.nsplit; ++z) acc += ((const int *)p.part)[z * p.plane + i];
        if (p.out_dtype == QGEMM_DT_I32) {
            ((int *)p.C)[idx] = acc;
            return;
        }
        const float s = p.per_matrix_scale ? p.as[0] * p.bs[0] : 1.0f;
        store_out(p.C, idx, (float)acc * s, p.out_dtype);
        return;
    }
    float acc = 0.0f;
    for (uint32_t z = 0; z < p.nsplit; ++z) acc += ((const float *)p.part)[z * p.plane + i];
    const float s = p.per_matrix_scale ? p.as[0] * p.bs[0] : 1.0f;
    store_out(p.C, idx, acc * s, p.out_dtype);
}

// The same for N a multiple of 4 (the planes are 256-byte aligned, so every group of four elements is 16 bytes,
// aligned, inside one row): four elements per thread, the loads of up to eight planes in flight together, then the
// sums in the order of the planes.  The launch is bound by latency, not by the 5 - 30 MB it reads: one element per
// thread with a dependent chain of loads took 4.2 us for 160 x 2048 in four planes, 11 us for 512 x 4096.
// c_vec: C and its rows allow a store of the four outputs at once (16 bytes, or 8 for the 2-byte types).
template <bool IS_I32>
__global__ void __launch_bounds__(256) splitk_reduce4_kernel(const ReduceArgs p, int c_vec) {
    typedef int v4i_ __attribute__((ext_vector_type(4)));
    typedef float v4f_ __attribute__((ext_vector_type(4)));
    typedef typename std::conditional<IS_I32, v4i_, v4f_>::type vec_t;
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= p.plane) return;
    const uint32_t m = (uint32_t)(i / p.N), n = (uint32_t)(i % p.N);
    const size_t idx = (size_t)m * p.ldc + n;
    const vec_t *src = (const vec_t *)((const char *)p.part + i * 4);
    const size_t plane_vecs = p.plane / 4;
    vec_t acc = vec_t{0, 0, 0, 0};
    for (uint32_t z0 = 0; z0 < p.nsplit; z0 += 8) {
        vec_t t[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (z0 + j < p.nsplit) t[j] = __builtin_nontemporal_load(src + (size_t)(z0 + j) * plane_vecs);
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (z0 + j < p.nsplit) acc += t[j];
    }
    if constexpr (IS_I32) {
        if (p.out_dtype == QGEMM_DT_I32) {
            int *dst = (int *)p.C + idx;
            if (c_vec) *(v4i_ *)dst = acc;
            else
                for (int e = 0; e < 4; ++e) dst[e] = acc[e];
            return;
        }
    }
    const float s = p.per_matrix_scale ? p.as[0] * p.bs[0] : 1.0f;
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = (float)acc[e] * s;
    if (p.out_dtype == QGEMM_DT_F32) {
        float *dst = (float *)p.C + idx;
        if (c_vec) *(v4f_ *)dst = v4f_{v[0], v[1], v[2], v[3]};
        else
            for (int e = 0; e < 4; ++e) dst[e] = v[e];
    } else {
        const v2i h = p.out_dtype == QGEMM_DT_BF16 ? pack4_bf16(v[0], v[1], v[2], v[3]) : pack4_f16(v[0], v[1], v[2], v[3]);
        unsigned short *dst = (unsigned short *)p.C + idx;
        if (c_vec) *(v2i *)dst = h;
        else
            for (int e = 0; e < 4; ++e) dst[e] = pack4_elem(h, e);
    }
}

}  // namespace qgemm
