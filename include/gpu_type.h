// Element type aliases of the host API.  Same names as the reference's
// include/gpu_type.h:20-31, with the fp8 type switched from the gfx942 "fnuz"
// flavour to OCP e4m3, which is what gfx950 MFMA decodes.
#pragma once
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <hip/hip_fp8.h>

#include <cstdint>

#define __FP8_TYPE __hip_fp8_e4m3
#define __FP8x4_TYPE __hip_fp8x4_e4m3
#define __BF16_TYPE __hip_bfloat16
#define __BF16x2_TYPE __hip_bfloat162
#define __FP16_TYPE __half
#define __INT16_TYPE int16_t
#define __FP32_TYPE float

constexpr inline int WAVE_SIZE = 64;
constexpr inline int XCD_SWIZZLE = 8;
