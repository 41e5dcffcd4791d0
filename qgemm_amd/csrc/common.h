// Shared device/host definitions for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/qgemm.h"

namespace qgemm {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef unsigned short us4 __attribute__((ext_vector_type(4)));

// Arithmetic families of the MFMA kernels.
enum Arith : int { AR_I8 = 0, AR_F8 = 1, AR_BF16 = 2, AR_F16 = 3 };

constexpr int kWave = 64;          // include/gpu_type.h:23 (WAVE_SIZE)
constexpr int kXcds = 8;           // include/gpu_type.h:24 (XCD_SWIZZLE)
constexpr int kScaleBlock = 128;   // hip_mix_gemm_kernel.cpp:46 (SCALE_BLOCK_SIZE)

__host__ __device__ inline int dtype_bytes(int dt) {
    switch (dt) {
        case QGEMM_DT_F32: case QGEMM_DT_I32: return 4;
        case QGEMM_DT_BF16: case QGEMM_DT_F16: return 2;
        case QGEMM_DT_I8: case QGEMM_DT_F8E4M3: return 1;
        default: return 0;
    }
}

// float -> bf16 bits, round to nearest even with a NaN guard: the intent of
// src/include/fast_quat.h:4-12 (which has no guard).  The compiler lowers the
// cast to v_cvt_pk_bf16_f32 on gfx950.
__device__ inline unsigned short f32_to_bf16_bits(float f) {
    __bf16 h = (__bf16)f;
    return __builtin_bit_cast(unsigned short, h);
}
__device__ inline unsigned short f32_to_f16_bits(float f) {
    _Float16 h = (_Float16)f;
    return __builtin_bit_cast(unsigned short, h);
}
// Four floats -> four bf16 / fp16 values in 8 bytes, element 0 in the low half of component 0.  Two elements per
// v_cvt_pk_*: half the instructions of four scalar conversions, and no packing step afterwards.  (The packing the
// compiler picks for two 16-bit scalars, v_pack_b32_f16, treats its inputs as fp16 numbers and quiets what looks
// like a signalling NaN: a bf16 pattern 0x7c01 .. 0x7dff, a finite value of 2^121 and more, came out with bit 9
// set.  The vector conversions never hold a lone 16-bit value in a register.)
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ inline v2i pack4_bf16(float a, float b, float c, float d) {
    return v2i{__builtin_bit_cast(int, __builtin_convertvector(f32x2_t{a, b}, bf16x2_t)),
               __builtin_bit_cast(int, __builtin_convertvector(f32x2_t{c, d}, bf16x2_t))};
}
__device__ inline v2i pack4_f16(float a, float b, float c, float d) {
    return v2i{__builtin_bit_cast(int, __builtin_convertvector(f32x2_t{a, b}, f16x2_t)),
               __builtin_bit_cast(int, __builtin_convertvector(f32x2_t{c, d}, f16x2_t))};
}
// element e (0 .. 3) of such a pack
__device__ inline unsigned short pack4_elem(v2i p, int e) { return (unsigned short)((unsigned)p[e >> 1] >> ((e & 1) * 16)); }

// Linear workgroup id -> (tile_m, tile_n).
// Step 1 (XCD remap): the dispatcher deals workgroups to the 8 XCDs round
// robin, so ids {x, x+8, x+16, ..} share an L2.  Renumber so that each XCD
// owns one contiguous range of the raster.
// Step 2 (GROUP_M raster, sm89_gemm_kernel_v3.cu:169-183): walk `group_m`
// tile rows column by column, so that concurrently resident tiles share A
// panels and B panels.  The group-size clamp uses the tile count (the
// reference clamps with M in rows).
__host__ __device__ inline void tile_map(uint32_t wg, uint32_t tiles_m, uint32_t tiles_n, uint32_t group_m,
                                         uint32_t &tm, uint32_t &tn) {
    const uint32_t total = tiles_m * tiles_n;
    uint32_t id = wg;
    if (total >= (uint32_t)kXcds * 2) {
        const uint32_t per = (total + kXcds - 1) / kXcds;           // ids owned by a "tall" XCD
        const uint32_t tall = total % kXcds ? total % kXcds : kXcds;  // XCDs that own `per` ids
        const uint32_t xcd = wg % kXcds, local = wg / kXcds;
        id = xcd < tall ? xcd * per + local : tall * per + (xcd - tall) * (per - 1) + local;
    }
    if (group_m <= 1) {
        tm = id / tiles_n;
        tn = id % tiles_n;
        return;
    }
    const uint32_t per_group = group_m * tiles_n;
    const uint32_t g = id / per_group;
    const uint32_t start_m = g * group_m;
    const uint32_t gsize = tiles_m - start_m < group_m ? tiles_m - start_m : group_m;
    const uint32_t in_group = id % per_group;
    tm = start_m + in_group % gsize;
    tn = in_group / gsize;
}

}  // namespace qgemm
