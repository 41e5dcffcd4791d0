"""qgemm_amd -- MI355X (gfx950) scaled mixed-precision GEMM.

The product is the C-ABI library qgemm_amd/libqgemm.so (HIP kernels, declared
in include/qgemm.h).  This package is the thin Python host side over that ABI:
torch is used for device memory and streams only.
"""
from .lib import QgemmError, load_library, load_torch_extension, library_path  # noqa: F401
from .ops import (  # noqa: F401
    DT_BF16, DT_F16, DT_F32, DT_F8E4M3, DT_I8, DT_I32,
    LAYOUT_K_CONTIGUOUS, LAYOUT_REFERENCE, QUANT_BLOCK_128x128, QUANT_BLOCK_1x128, QUANT_PER_MATRIX,
    SCALE_BLOCK128, SCALE_PER_MATRIX,
    bf16_mm, fp8_mm, gemm, int8_mm, int8_mm_block, last_config, matrix_transpose, plan, quantize, scaled_gemm, selftest_layouts,
    force_config, set_option, tile_map, variant_names,
)
