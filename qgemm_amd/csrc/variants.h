// Table of compiled MFMA GEMM variants (one row per tile shape, loader and
// arithmetic family).  Plays the role of the reference's constexpr tile tables
// (src/include/gemm_config.h:30-36,65-71) and of its divisibility dispatch
// (hip_mix_gemm_kernel.cpp:442-505), but is chosen at run time from the shape.
#pragma once
#include "gemm_mfma.cuh"

namespace qgemm {

struct Variant {
    const char *name;
    int arith;
    bool block_scale;
    int bm, bn, threads, lds_bytes, loader;
    bool auto_ok;   // the shape heuristic may pick this row (the others are reachable through force_config)
    int kgroups;    // 2: two sets of waves per workgroup, each computing every other K step (GemmCfg::KG);
                    // 8: the skinny-M kernel, eight waves each computing every eighth K step (gemm_skinny.cuh)
    bool a_scale_k_contiguous;   // block scales: the kernel also reads a_scale[m * ld + kb] as the caller has it
                                 // (the others want it rows-contiguous, a_scale[m + kb * ld])
    bool a_scale_any_stride;     // block scales: the kernel reads a_scale[m * ms + kb * ks] for any ms, ks
    hipError_t (*launch)(const GemmArgs &, uint32_t grid, hipStream_t);
};

// one translation unit per arithmetic family defines one of these
const Variant *variants_i8(int *count);
const Variant *variants_f8(int *count);
const Variant *variants_f8_block(int *count);
const Variant *variants_bf16(int *count);
const Variant *variants_f16(int *count);
// K-major operand storage (GemmCfg::KMAJ): the reference's fp8 layout (A is K x M, B is K x N) and "NN" 16-bit GEMMs
const Variant *variants_f8_block_tn(int *count);
const Variant *variants_bf16_nn(int *count);
const Variant *variants_f16_nn(int *count);

}  // namespace qgemm
