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

// x / s for many x and one s (a scale: positive, finite).  The compiler expands every fp32 division into a
// reciprocal, two refinements of it and three of the quotient, all on values scaled by v_div_scale so that nothing
// leaves the normal range.  With s between 2^-60 and 2^60 and |x| at most a few hundred s (the quantisers divide by
// max|x| / 448 or / 127) that scaling is the identity unless the quotient is below 2^-100, which every output type
// here turns into a zero of the quotient's sign whatever its low bits: so the reciprocal is refined once per scale
// and the quotient steps are the same fused multiply-adds on the same values: the same bits as x / s, about half
// the instructions per element.  Zeros, infinities and NaNs of x pass through as they are (what the division's
// last step, v_div_fixup, does for a finite positive divisor); scales outside the range take the plain division.
struct Divisor {
    float s, r;
    bool in_range;
};
__device__ inline Divisor make_divisor(float s) {
    Divisor d;
    d.s = s;
    d.in_range = s >= 0x1p-60f && s <= 0x1p60f;
    const float r0 = __builtin_amdgcn_rcpf(s);
    d.r = __builtin_fmaf(__builtin_fmaf(-s, r0, 1.0f), r0, r0);
    return d;
}
__device__ inline float div_by(float x, const Divisor &d) {
    if (!d.in_range) return x / d.s;
    float q = x * d.r;
    q = __builtin_fmaf(__builtin_fmaf(-d.s, q, x), d.r, q);
    q = __builtin_fmaf(__builtin_fmaf(-d.s, q, x), d.r, q);
    const float ax = __builtin_fabsf(x);
    return (ax > 0.0f && ax < __builtin_inff()) ? q : x;
}

// four quantised bytes of (v / s), packed little-endian
__device__ inline uint32_t quant4(v4f v, const Divisor &dv, int out_dtype) {
    const float a = div_by(v[0], dv), b = div_by(v[1], dv), c = div_by(v[2], dv), d = div_by(v[3], dv);
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

// maximum over each half of the wave (lanes 0-31, 32-63), in every lane, on the vector ALU alone: lane exchanges
// inside a row of 16 ride on the max instruction (DPP), the two rows of a half are exchanged with one lane swap.
// (Five __shfl_xor per block are five trips through the LDS crossbar with their address arithmetic.)
__device__ inline float half_wave_max(float m) {
    auto dpp = [](float v, auto ctrl) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), decltype(ctrl)::value, 0xF, 0xF, true));
    };
    m = __builtin_fmaxf(m, dpp(m, std::integral_constant<int, 0xB1>{}));      // quad_perm [1,0,3,2]: lane ^ 1
    m = __builtin_fmaxf(m, dpp(m, std::integral_constant<int, 0x4E>{}));      // quad_perm [2,3,0,1]: lane ^ 2
    m = __builtin_fmaxf(m, dpp(m, std::integral_constant<int, 0x141>{}));     // row_half_mirror: lane -> 7 - lane within 8
    m = __builtin_fmaxf(m, dpp(m, std::integral_constant<int, 0x140>{}));     // row_mirror: lane -> 15 - lane within 16
    const unsigned u = __builtin_bit_cast(unsigned, m);
    const auto sw = __builtin_amdgcn_permlane16_swap(u, u, false, false);      // (R0 R0 R2 R2), (R1 R1 R3 R3)
    const unsigned even = sw[0], odd = sw[1];          // (a bit_cast applied to a vector element reads element 0)
    return __builtin_fmaxf(__builtin_bit_cast(float, even), __builtin_bit_cast(float, odd));
}

__device__ inline float scale_of(float amax, int out_dtype) {
    return amax > 0.0f ? amax / (out_dtype == QGEMM_DT_F8E4M3 ? 448.0f : 127.0f) : 1.0f;
}

// ---- per matrix, pass 1: one partial maximum per workgroup (grid-stride over groups of 4 columns)
template <int IN_DT>
__global__ void __launch_bounds__(256) quant_amax_kernel(const QuantArgs p) {
    __shared__ float red[4];
    const uint32_t groups_per_row = (p.cols + 3) / 4;
    const bool vec = p.ld % 4 == 0 && (uintptr_t)p.x % 16 == 0;
    float m = 0.0f;
    // rows in turn over the workgroups, groups of four columns in turn over the threads: no division per element
    for (uint32_t r = blockIdx.x; r < p.rows; r += gridDim.x) {
        for (uint32_t g = threadIdx.x; g < groups_per_row; g += 256) {
            const uint32_t c = g * 4;
            const v4f v = load4_as_f32<IN_DT>(p.x, (size_t)r * p.ld + c, vec, p.cols - c);
#pragma unroll
            for (int i = 0; i < 4; ++i) m = __builtin_fmaxf(m, abs_or_zero(v[i]));
        }
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
    const bool vin = p.ld % 4 == 0 && (uintptr_t)p.x % 16 == 0;
    const bool vout = p.ldq % 4 == 0 && (uintptr_t)p.q % 4 == 0;
    const Divisor dv = make_divisor(s);
    for (uint32_t r = blockIdx.x; r < p.rows; r += gridDim.x) {
        for (uint32_t g = threadIdx.x; g < groups_per_row; g += 256) {
            const uint32_t c = g * 4;
            const v4f v = load4_as_f32<IN_DT>(p.x, (size_t)r * p.ld + c, vin, p.cols - c);
            store4(p.q, (size_t)r * p.ldq + c, quant4(v, dv, p.out_dtype), vout, p.cols - c);
        }
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
    m = half_wave_max(m);
    const float s = scale_of(m, p.out_dtype);
    if ((threadIdx.x & 31) == 0) p.scales[(size_t)r * p.scale_rs + (size_t)jb * p.scale_cs] = s;
    if (valid) store4(p.q, (size_t)r * p.ldq + c, quant4(v, make_divisor(s), p.out_dtype), vout, valid);
}

// ---- 1 x 128 blocks, the common case: whole blocks (cols a multiple of 128), x and q aligned for vector access,
// fp8 out.  Grid (rows, ceil(blocks per row / 8)): half wave h of workgroup (r, g) takes block 8 g + h of row r, so
// there is no division to find the block and no bounds check per element.  (The general kernel above spends more
// instructions on those than on the quantisation: 6144 x 7168 fp32 54 -> 40 us, the same for bf16 input, which
// says the kernel is bound by instruction issue, not by memory.)
template <int IN_DT>
__global__ void __launch_bounds__(256) quant_row_block_whole_kernel(const QuantArgs p) {
    const uint32_t nbc = p.cols / 128;
    const uint32_t r = blockIdx.x, jb = blockIdx.y * 8 + (threadIdx.x >> 5);
    if (jb >= nbc) return;                             // whole half-waves leave together
    const uint32_t c = jb * 128 + (threadIdx.x & 31) * 4;
    const v4f v = load4_as_f32<IN_DT>(p.x, (size_t)r * p.ld + c, true, 4);
    float m = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) m = __builtin_fmaxf(m, abs_or_zero(v[i]));
    m = half_wave_max(m);
    const float s = scale_of(m, QGEMM_DT_F8E4M3);
    if ((threadIdx.x & 31) == 0) p.scales[(size_t)r * p.scale_rs + (size_t)jb * p.scale_cs] = s;
    *(uint32_t *)((uint8_t *)p.q + (size_t)r * p.ldq + c) = quant4(v, make_divisor(s), QGEMM_DT_F8E4M3);
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
    const Divisor dv = make_divisor(s);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const uint32_t r = r0 + i * 8;
        if (r < p.rows && valid) store4(p.q, (size_t)r * p.ldq + c, quant4(v[i], dv, p.out_dtype), vout, valid);
    }
}

// ---- 128 x 128 blocks, whole blocks (rows and cols multiples of 128), x and q aligned for vector access, fp8 out:
// as above without the bounds checks
template <int IN_DT>
__global__ void __launch_bounds__(256) quant_square_block_whole_kernel(const QuantArgs p) {
    __shared__ float red[4];
    const uint32_t ib = blockIdx.y, jb = blockIdx.x;
    const uint32_t c = jb * 128 + (threadIdx.x & 31) * 4;
    const uint32_t r0 = ib * 128 + (threadIdx.x >> 5);            // rows r0, r0 + 8, ...
    const size_t x0 = (size_t)r0 * p.ld + c, q0 = (size_t)r0 * p.ldq + c;
    v4f v[16];
    float m = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = load4_as_f32<IN_DT>(p.x, x0 + (size_t)i * 8 * p.ld, true, 4);
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) m = __builtin_fmaxf(m, abs_or_zero(v[i][e]));
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    const float amax = __builtin_fmaxf(__builtin_fmaxf(red[0], red[1]), __builtin_fmaxf(red[2], red[3]));
    const float s = scale_of(amax, QGEMM_DT_F8E4M3);
    if (threadIdx.x == 0) p.scales[(size_t)ib * p.scale_rs + (size_t)jb * p.scale_cs] = s;
    const Divisor dv = make_divisor(s);
#pragma unroll
    for (int i = 0; i < 16; ++i)
        *(uint32_t *)((uint8_t *)p.q + q0 + (size_t)i * 8 * p.ldq) = quant4(v[i], dv, QGEMM_DT_F8E4M3);
}

}  // namespace qgemm
