// Table of compiled MFMA GEMM variants (one row per tile shape and schedule, one table per arithmetic
// family).  Plays the role of the reference's constexpr tile tables (src/include/gemm_config.h:30-36,65-71)
// and of its divisibility dispatch (hip_mix_gemm_kernel.cpp:442-505), but is chosen at run time from the shape.
// Rows are addressed by name (unique inside a family): no caller depends on the order of a table.
#pragma once
#include "gemm_mfma.cuh"

namespace qgemm {

struct Variant {
    const char *name;
    int arith;
    bool block_scale;
    int bm, bn, threads, lds_bytes;
    bool auto_ok;   // the shape heuristic may pick this row (the others are reachable by name, option "force_config")
    bool copy_waves;   // solo schedule with four computing and four copying waves (GemmCfg::COPYW)
    int kgroups;    // 2: two sets of waves per workgroup, each computing every other K step (GemmCfg::KG);
                    // 8: the skinny-M kernel, eight waves each computing every eighth K step (gemm_skinny.cuh)
    bool a_scale_k_contiguous;   // block scales: the kernel reads a_scale[m * ld + kb] as QGEMM_LAYOUT_K_CONTIGUOUS passes
                                 // it (the others want it rows-contiguous, a_scale[m + kb * ld], or take any strides)
    bool a_scale_any_stride;     // block scales: the kernel reads a_scale[m * ms + kb * ks] for any ms, ks
    // Pair of rows that differ only in the arrangement of a_scale they read (GemmCfg::ASK): index, in the same table,
    // of the other row of the pair (-1: none), and how many K blocks the K-contiguous one fetches per load (2 or 4:
    // the caller's a_scale rows, K and every K slice have to be multiples of that many blocks, and rows aligned to
    // as many floats).
    int twin;
    int ks_blocks;
    hipError_t (*launch)(const GemmArgs &, uint32_t grid, hipStream_t);
};

// one translation unit per arithmetic family defines one of these
const Variant *variants_i8(int *count);
const Variant *variants_f8(int *count);
const Variant *variants_f8_block(int *count);
const Variant *variants_i8_block(int *count);
const Variant *variants_bf16(int *count);
const Variant *variants_f16(int *count);
// K-major operand storage (GemmCfg::KMAJ): the reference's fp8 layout (A is K x M, B is K x N) and "NN" 16-bit GEMMs
const Variant *variants_f8_block_tn(int *count);
const Variant *variants_bf16_nn(int *count);
const Variant *variants_f16_nn(int *count);

}  // namespace qgemm
