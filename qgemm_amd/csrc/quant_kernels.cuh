// Quantisers: the Q_A / Q_B of C = (A o Q_A) x (B o Q_B) (README.md:1 of the reference, which implements none).
//   per matrix     s = max|x| / 127 (int8) or / 448 (fp8 e4m3);  q = round(x / s), saturated
//   1 x 128 blocks  one scale per row and 128 columns      (the a_scale of hip_mix_gemm_kernel.cpp:149)
//   128 x 128       one scale per 128 x 128 block          (the b_scale of hip_mix_gemm_kernel.cpp:137,164)
// A block (or matrix) of zeros gets s = 1.  x / s is a true division and the rounding is to nearest even,
// so the results are the bits the CPU quantisers give.  All three are bound by HBM traffic.
#pragma once
#include "common.h"

namespace qgemm {

struct QuantArgs {
    const void *x;        // rows x cols, row stride ld elements
    void *q;              // rows x cols bytes, row stride ldq
    float *scales;        // per matrix: 1 float; blocks: scales[ib*scale_rs + jb*scale_cs]
    float *partial;       // per matrix: one partial maximum per workgroup of the first pass
    uint32_t rows, cols, npartial;
    uint64_t ld, ldq, scale_rs, scale_cs;
    int out_dtype;        // QGEMM_DT_I8 or QGEMM_DT_F8E4M3
};

template <int IN_DT>
__device__ inline float load_as_f32(const void *base, size_t idx) {
    if constexpr (IN_DT == QGEMM_DT_F32) return ((const float *)base)[idx];
    else if constexpr (IN_DT == QGEMM_DT_BF16)
        return __builtin_bit_cast(float, (uint32_t)((const unsigned short *)base)[idx] << 16);
    else return (float)((const _Float16 *)base)[idx];
}

// four consecutive elements; `vec` says the address is aligned for one vector load
template <int IN_DT>
__device__ inline v4f load4_as_f32(const void *base, size_t idx, bool vec, uint32_t valid) {
    v4f r = {0, 0, 0, 0};
    if (vec && valid >= 4) {
        if constexpr (IN_DT == QGEMM_DT_F32) {
            r = *(const v4f *)((const float *)base + idx);
        } else {
            const us4 h = *(const us4 *)((const unsigned short *)base + idx);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const unsigned short bits = h[i];     // (a bit_cast applied to a vector element reads element 0)
                if constexpr (IN_DT == QGEMM_DT_BF16) r[i] = __builtin_bit_cast(float, (uint32_t)bits << 16);
                else r[i] = (float)__builtin_bit_cast(_Float16, bits);
            }
        }
        return r;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if ((uint32_t)i < valid) r[i] = load_as_f32<IN_DT>(base, idx + i);
    return r;
}

// |x| with NaN mapped to 0: a NaN never becomes the maximum (the CPU loop's `a > m` ignores it too)
__device__ inline float abs_or_zero(float v) {
    const float a = __builtin_fabsf(v);
    return a == a ? a : 0.0f;
}

// e4m3 (OCP): saturate to +-448, then round to nearest even; NaN -> 0x7F with the sign kept.
// Two values per call: v_cvt_pk_fp8_f32 packs them into the low half of a dword.
__device__ inline uint32_t f32x2_to_fp8(float a, float b) {
    const bool na = a != a, nb = b != b;
    const float ca = __builtin_fminf(__builtin_fmaxf(a, -448.0f), 448.0f);
    const float cb = __builtin_fminf(__builtin_fmaxf(b, -448.0f), 448.0f);
    uint32_t r = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(ca, cb, 0, false) & 0xFFFFu;
    if (na) r = (r & 0xFF00u) | 0x7Fu | ((__builtin_bit_cast(uint32_t, a) >> 24) & 0x80u);
    if (nb) r = (r & 0x00FFu) | ((0x7Fu | ((__builtin_bit_cast(uint32_t, b) >> 24) & 0x80u)) << 8);
    return r;
}

__device__ inline uint32_t f32_to_i8(float v) {
    float r = __builtin_rintf(v);                 // ties to even
    r = r > 127.0f ? 127.0f : r;
    r = r < -127.0f ? -127.0f : r;
    return (uint32_t)(int)r & 0xFFu;              // NaN: the comparisons are false, the cast gives 0
}

// four quantised bytes of (v / s), packed little-endian
__device__ inline uint32_t quant4(v4f v, float s, int out_dtype) {
    const float a = v[0] / s, b = v[1] / s, c = v[2] / s, d = v[3] / s;
    if (out_dtype == QGEMM_DT_F8E4M3) return f32x2_to_fp8(a, b) | (f32x2_to_fp8(c, d) << 16);
    return f32_to_i8(a) | (f32_to_i8(b) << 8) | (f32_to_i8(c) << 16) | (f32_to_i8(d) << 24);
}

__device__ inline void store4(void *q, size_t idx, uint32_t packed, bool vec, uint32_t valid) {
    if (vec && valid >= 4) {
        *(uint32_t *)((uint8_t *)q + idx) = packed;
        return;
    }
    for (uint32_t i = 0; i < 4 && i < valid; ++i) ((uint8_t *)q)[idx + i] = (uint8_t)(packed >> (8 * i));
}

__device__ inline float wave_max(float m) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = __builtin_fmaxf(m, __shfl_xor(m, off, 64));
    return m;
}

__device__ inline float scale_of(float amax, int out_dtype) {
    return amax > 0.0f ? amax / (out_dtype == QGEMM_DT_F8E4M3 ? 448.0f : 127.0f) : 1.0f;
}

// ---- per matrix, pass 1: one partial maximum per workgroup (grid-stride over groups of 4 columns)
template <int IN_DT>
__global__ void __launch_bounds__(256) quant_amax_kernel(const QuantArgs p) {
    __shared__ float red[4];
    const uint32_t groups_per_row = (p.cols + 3) / 4;
    const uint64_t total = (uint64_t)p.rows * groups_per_row;
    const bool vec = p.ld % 4 == 0 && (uintptr_t)p.x % 16 == 0;
    float m = 0.0f;
    for (uint64_t g = (uint64_t)blockIdx.x * 256 + threadIdx.x; g < total; g += (uint64_t)gridDim.x * 256) {
        const uint32_t r = (uint32_t)(g / groups_per_row), c = (uint32_t)(g % groups_per_row) * 4;
        const v4f v = load4_as_f32<IN_DT>(p.x, (size_t)r * p.ld + c, vec, p.cols - c);
#pragma unroll
        for (int i = 0; i < 4; ++i) m = __builtin_fmaxf(m, abs_or_zero(v[i]));
    }
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0)
        p.partial[blockIdx.x] = __builtin_fmaxf(__builtin_fmaxf(red[0], red[1]), __builtin_fmaxf(red[2], red[3]));
}

// ---- per matrix, pass 2: every workgroup reduces the partial maxima again (a few KB, L2 resident), then
// quantises its share; workgroup 0 writes the scale
template <int IN_DT>
__global__ void __launch_bounds__(256) quant_matrix_kernel(const QuantArgs p) {
    __shared__ float red[4];
    float m = 0.0f;
    for (uint32_t i = threadIdx.x; i < p.npartial; i += 256) m = __builtin_fmaxf(m, p.partial[i]);
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    const float amax = __builtin_fmaxf(__builtin_fmaxf(red[0], red[1]), __builtin_fmaxf(red[2], red[3]));
    const float s = scale_of(amax, p.out_dtype);
    if (blockIdx.x == 0 && threadIdx.x == 0) p.scales[0] = s;
    const uint32_t groups_per_row = (p.cols + 3) / 4;
    const uint64_t total = (uint64_t)p.rows * groups_per_row;
    const bool vin = p.ld % 4 == 0 && (uintptr_t)p.x % 16 == 0;
    const bool vout = p.ldq % 4 == 0 && (uintptr_t)p.q % 4 == 0;
    for (uint64_t g = (uint64_t)blockIdx.x * 256 + threadIdx.x; g < total; g += (uint64_t)gridDim.x * 256) {
        const uint32_t r = (uint32_t)(g / groups_per_row), c = (uint32_t)(g % groups_per_row) * 4;
        const v4f v = load4_as_f32<IN_DT>(p.x, (size_t)r * p.ld + c, vin, p.cols - c);
        store4(p.q, (size_t)r * p.ldq + c, quant4(v, s, p.out_dtype), vout, p.cols - c);
    }
}

// ---- 1 x 128 blocks: half a wave (32 lanes x 4 columns) per block, 8 blocks per workgroup
template <int IN_DT>
__global__ void __launch_bounds__(256) quant_row_block_kernel(const QuantArgs p) {
    const uint32_t nbc = (p.cols + 127) / 128;
    const uint64_t nblocks = (uint64_t)p.rows * nbc;
    const uint64_t blk = (uint64_t)blockIdx.x * 8 + (threadIdx.x >> 5);
    if (blk >= nblocks) return;                        // whole half-waves leave together
    const uint32_t r = (uint32_t)(blk / nbc), jb = (uint32_t)(blk % nbc);
    const uint32_t c = jb * 128 + (threadIdx.x & 31) * 4;
    const bool vin = p.ld % 4 == 0 && (uintptr_t)p.x % 16 == 0;
    const bool vout = p.ldq % 4 == 0 && (uintptr_t)p.q % 4 == 0;
    const uint32_t valid = c < p.cols ? p.cols - c : 0;
    const v4f v = load4_as_f32<IN_DT>(p.x, (size_t)r * p.ld + c, vin, valid);
    float m = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) m = __builtin_fmaxf(m, abs_or_zero(v[i]));
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) m = __builtin_fmaxf(m, __shfl_xor(m, off, 32));
    const float s = scale_of(m, p.out_dtype);
    if ((threadIdx.x & 31) == 0) p.scales[(size_t)r * p.scale_rs + (size_t)jb * p.scale_cs] = s;
    if (valid) store4(p.q, (size_t)r * p.ldq + c, quant4(v, s, p.out_dtype), vout, valid);
}

// ---- 128 x 128 blocks: one workgroup per block; a thread holds 4 columns of 16 rows in registers
template <int IN_DT>
__global__ void __launch_bounds__(256) quant_square_block_kernel(const QuantArgs p) {
    __shared__ float red[4];
    const uint32_t nbc = (p.cols + 127) / 128;
    const uint32_t ib = blockIdx.x / nbc, jb = blockIdx.x % nbc;
    const uint32_t c = jb * 128 + (threadIdx.x & 31) * 4;
    const uint32_t r0 = ib * 128 + (threadIdx.x >> 5);            // rows r0, r0 + 8, ...
    const bool vin = p.ld % 4 == 0 && (uintptr_t)p.x % 16 == 0;
    const bool vout = p.ldq % 4 == 0 && (uintptr_t)p.q % 4 == 0;
    const uint32_t valid = c < p.cols ? p.cols - c : 0;
    v4f v[16];
    float m = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const uint32_t r = r0 + i * 8;
        v[i] = v4f{0, 0, 0, 0};
        if (r < p.rows && valid) v[i] = load4_as_f32<IN_DT>(p.x, (size_t)r * p.ld + c, vin, valid);
#pragma unroll
        for (int e = 0; e < 4; ++e) m = __builtin_fmaxf(m, abs_or_zero(v[i][e]));
    }
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    const float amax = __builtin_fmaxf(__builtin_fmaxf(red[0], red[1]), __builtin_fmaxf(red[2], red[3]));
    const float s = scale_of(amax, p.out_dtype);
    if (threadIdx.x == 0) p.scales[(size_t)ib * p.scale_rs + (size_t)jb * p.scale_cs] = s;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const uint32_t r = r0 + i * 8;
        if (r < p.rows && valid) store4(p.q, (size_t)r * p.ldq + c, quant4(v[i], s, p.out_dtype), vout, valid);
    }
}

}  // namespace qgemm
