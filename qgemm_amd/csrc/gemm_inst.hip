// Instantiates the MFMA GEMM template for one arithmetic family.  Compiled once
// per family with -DINST_ARITH=<Arith> -DINST_BLOCK=<0|1> -DINST_FN=<table fn>,
// so the families build in parallel.
#include "variants.h"
#include "gemm_skinny.cuh"

#include <type_traits>

#ifndef INST_ARITH
#error "compile with -DINST_ARITH=... -DINST_BLOCK=... -DINST_FN=... [-DINST_KMAJ=1|2|3]"
#endif
#ifndef INST_KMAJ
#define INST_KMAJ 0      // bit 0: A stored K x M, bit 1: B stored K x N (see GemmCfg::KMAJ)
#endif

namespace qgemm {

template <class C>
static hipError_t launch_variant(const GemmArgs &a, uint32_t grid, hipStream_t s) {
    static bool attr_done = false;
    if (!attr_done) {
        // more than 64 KiB of dynamic LDS has to be asked for explicitly
        hipError_t e = hipFuncSetAttribute((const void *)gemm_nt_kernel<C>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           C::LDS_BYTES);
        if (e != hipSuccess) return e;
        attr_done = true;
    }
    hipLaunchKernelGGL(gemm_nt_kernel<C>, dim3(grid), dim3(C::THREADS), C::LDS_BYTES, s, a);
    return hipGetLastError();
}

template <class C>
static hipError_t launch_skinny(const GemmArgs &a, uint32_t grid, hipStream_t s) {
    static bool attr_done = false;
    if (!attr_done) {
        hipError_t e = hipFuncSetAttribute((const void *)gemm_skinny_kernel<C>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           C::LDS_BYTES);
        if (e != hipSuccess) return e;
        attr_done = true;
    }
    hipLaunchKernelGGL(gemm_skinny_kernel<C>, dim3(grid), dim3(C::THREADS), C::LDS_BYTES, s, a);
    return hipGetLastError();
}
// row of the skinny-M kernel (gemm_skinny.cuh): 16 * TM rows x 32 columns, eight waves splitting K between them.
// Picked by choose_variant in place of the narrow simple-pipeline tiles, never by the table scan (auto_ok = false).
template <int TM, int TN = 2>
static Variant skinny_row(const char *name) {
    using C = SkinnyCfg<INST_ARITH, TM, (bool)INST_BLOCK, TN>;
    return Variant{name, C::ARITH, C::BLOCK_SCALE, C::BM, C::BN, C::THREADS, C::LDS_BYTES, LOAD_DMA, false, 8, false,
                   C::BLOCK_SCALE, &launch_skinny<C>};
}

#define CFG(BM, BN, WM_, WN_, LD, PP) GemmCfg<INST_ARITH, (bool)INST_BLOCK, BM, BN, WM_, WN_, LD, PP, 0, (PP) != PIPE_SIMPLE, INST_KMAJ>

// A K-major operand needs whole 128-byte panels of its tile side, four waves and the simple pipeline (GemmCfg's
// static_asserts); rows of the table that cannot have that are aliases of the 128 x 128 row in such a family,
// so that force_config indices agree across families, and are never picked by the heuristic.
constexpr int kElemBytes = (INST_ARITH == AR_BF16 || INST_ARITH == AR_F16) ? 2 : 1;
constexpr bool kmajor_can(int bm, int bn, int nw, int pipe) {
    return INST_KMAJ == 0 || (pipe == PIPE_SIMPLE && nw % 4 == 0 && (!(INST_KMAJ & 1) || (bm * kElemBytes) % 128 == 0) &&
                              (!(INST_KMAJ & 2) || (bn * kElemBytes) % 128 == 0));
}
template <bool OK, class C, class Fallback>
static Variant row_of(const char *name, bool auto_ok) {
    using P = std::conditional_t<OK, C, Fallback>;
    return Variant{OK ? name : "128x128_w2x2_dma", P::ARITH, P::BLOCK_SCALE, P::BM, P::BN, P::THREADS, P::LDS_BYTES,
                   P::LOADER, OK && auto_ok, P::KG, P::ASK, P::AS_ANY_STRIDE, &launch_variant<P>};
}
#define ROWP(NAME, BM, BN, WM_, WN_, LD, PP, AUTO) \
    row_of<kmajor_can(BM, BN, (WM_) * (WN_), PP), CFG(BM, BN, WM_, WN_, LD, PP), CFG(128, 128, 2, 2, LOAD_DMA, PIPE_SIMPLE)>(NAME, AUTO)
#define ROW(NAME, BM, BN, WM_, WN_, LD, AUTO) ROWP(NAME, BM, BN, WM_, WN_, LD, PIPE_SIMPLE, AUTO)

// force_config indexes this table; the heuristic only considers the rows marked auto.
static const Variant kTable[] = {
    ROW("256x256_w2x4_dma", 256, 256, 2, 4, LOAD_DMA, false),
    ROW("256x128_w2x2_dma", 256, 128, 2, 2, LOAD_DMA, false),
    ROW("128x128_w2x2_dma", 128, 128, 2, 2, LOAD_DMA, true),
    ROW("64x128_w1x4_dma", 64, 128, 1, 4, LOAD_DMA, true),
    ROW("32x128_w1x4_dma", 32, 128, 1, 4, LOAD_DMA, true),
    ROW("16x128_w1x2_dma", 16, 128, 1, 2, LOAD_DMA, true),
    ROW("256x256_w2x4_vgpr", 256, 256, 2, 4, LOAD_VGPR, false),
    ROW("128x128_w2x2_vgpr", 128, 128, 2, 2, LOAD_VGPR, false),
    ROW("32x128_w1x4_vgpr", 32, 128, 1, 4, LOAD_VGPR, false),
    ROWP("256x256_w4x2_pingpong", 256, 256, 4, 2, LOAD_DMA, PIPE_PINGPONG, false),
    ROWP("256x256_w2x4_pingpong", 256, 256, 2, 4, LOAD_DMA, PIPE_PINGPONG, false),
    // The 256 x 256 tile the heuristic uses: fp8 per-matrix runs fastest on the 4-wave solo schedule (a third
    // fewer LDS reads: 3 % in interleaved runs); for int8 and the 16-bit types the table marks the 8-wave one and
    // choose_variant swaps in the 4-wave one where the tiles fill whole rounds of CUs (1 % faster there, 1 - 6 %
    // slower in partly filled rounds); block scales need the 8-wave form.
#if INST_BLOCK   // no block-scaled form of the 4-wave solo pipeline: the row is an alias, so indices agree across families
    ROWP("256x256_w4x2_pingpong", 256, 256, 4, 2, LOAD_DMA, PIPE_PINGPONG, false),
#else
    ROWP("256x256_w2x2_solo", 256, 256, 2, 2, LOAD_DMA, PIPE_SOLO, INST_ARITH == AR_F8 && INST_KMAJ == 0),
#endif
    ROWP("256x256_w2x4_solo8", 256, 256, 2, 4, LOAD_DMA, PIPE_SOLO, INST_BLOCK || INST_ARITH != AR_F8),
    // narrow tiles for skinny M: N / 32 workgroups stream disjoint strips of B over the whole of K, so no
    // K split (and no second pass over partial sums) is needed to occupy the CUs
    ROW("128x32_w4x1_dma", 128, 32, 4, 1, LOAD_DMA, true),
    ROW("64x32_w4x1_dma", 64, 32, 4, 1, LOAD_DMA, true),
    ROW("16x32_w1x2_dma", 16, 32, 1, 2, LOAD_DMA, true),
    // 128 x 128 with eight computing waves in two K groups and four copying waves (GemmCfg::KG), five stages (160 KiB,
    // one workgroup per CU; four with block scales, whose a_scale values take 2 KiB behind the ring): for shapes with
    // no more tiles than CUs, where the two-stage row above would sit alone on its CU
    // (K-major families too: the waves that read the tile with the transposing LDS reads have no copies in flight)
    row_of<kmajor_can(128, 128, 4, PIPE_SIMPLE),
           GemmCfg<INST_ARITH, (bool)INST_BLOCK, 128, 128, 2, 2, LOAD_DMA, PIPE_SIMPLE, 0, false, INST_KMAJ, INST_BLOCK ? 4 : 5, 2>,
           CFG(128, 128, 2, 2, LOAD_DMA, PIPE_SIMPLE)>("128x128_w2x2_k2", true),
    // the same for the 64 x 128 tile, with six stages
    row_of<kmajor_can(64, 128, 4, PIPE_SIMPLE),
           GemmCfg<INST_ARITH, (bool)INST_BLOCK, kmajor_can(64, 128, 4, PIPE_SIMPLE) ? 64 : 128, 128, kmajor_can(64, 128, 4, PIPE_SIMPLE) ? 1 : 2,
                   kmajor_can(64, 128, 4, PIPE_SIMPLE) ? 4 : 2, LOAD_DMA, PIPE_SIMPLE, 0, false, INST_KMAJ,
                   kmajor_can(64, 128, 4, PIPE_SIMPLE) ? 6 : (INST_BLOCK ? 4 : 5), 2>,
           CFG(128, 128, 2, 2, LOAD_DMA, PIPE_SIMPLE)>("64x128_w1x4_k2", true),
    // skinny M (gemm_skinny.cuh): the K split inside the workgroup, no staging, no barrier in the K loop
#if INST_KMAJ      // (no K-major form: aliases, so indices agree across families)
    ROW("128x128_w2x2_dma", 128, 128, 2, 2, LOAD_DMA, false),
    ROW("128x128_w2x2_dma", 128, 128, 2, 2, LOAD_DMA, false),
    ROW("128x128_w2x2_dma", 128, 128, 2, 2, LOAD_DMA, false),
    ROW("128x128_w2x2_dma", 128, 128, 2, 2, LOAD_DMA, false),
#else
    skinny_row<1>("skinny_16x32_k8"),
    skinny_row<2>("skinny_32x32_k8"),
    skinny_row<4>("skinny_64x32_k8"),
    skinny_row<8>("skinny_128x32_k8"),
#endif
    // the block-scaled 8-wave solo kernel reading a_scale with the K blocks contiguous, as QGEMM_LAYOUT_K_CONTIGUOUS
    // passes it (GemmCfg::ASK): launch_nt swaps it in for the row above of the same name when the scales allow it,
    // which saves a transposed copy of a_scale (the simple and ping-pong pipelines read it through strides)
#if INST_BLOCK && !INST_KMAJ
    row_of<true, GemmCfg<INST_ARITH, true, 256, 256, 2, 4, LOAD_DMA, PIPE_SOLO, 0, true, 0, 0, 1, true>,
           CFG(128, 128, 2, 2, LOAD_DMA, PIPE_SIMPLE)>("256x256_w2x4_solo8_ks", false),
#else
    ROW("128x128_w2x2_dma", 128, 128, 2, 2, LOAD_DMA, false),
#endif
    // the skinny-M kernel on a 64 x 64 tile: for shapes with a few row tiles whose 64 x 64 tiles fit one round of CUs
#if INST_KMAJ      // (K-contiguous operands only: alias, so indices agree across families)
    ROW("128x128_w2x2_dma", 128, 128, 2, 2, LOAD_DMA, false),
#else
    skinny_row<4, 4>("skinny_64x64_k8"),
#endif
    // 256 x 128 on the solo schedule with four computing waves (128 x 64 wave tiles, one per SIMD) and four copying
    // waves (GemmCfg::COPYW): block scales and K-major operands on a large tile, and its twin for K-contiguous a_scale
    row_of<true, GemmCfg<INST_ARITH, (bool)INST_BLOCK, 256, 128, 2, 2, LOAD_DMA, PIPE_SOLO, 0, true, INST_KMAJ, 0, 1, false, true>,
           CFG(128, 128, 2, 2, LOAD_DMA, PIPE_SIMPLE)>("256x128_w2x2_cw", true),
#if INST_BLOCK && !INST_KMAJ
    row_of<true, GemmCfg<INST_ARITH, true, 256, 128, 2, 2, LOAD_DMA, PIPE_SOLO, 0, true, 0, 0, 1, true, true>,
           CFG(128, 128, 2, 2, LOAD_DMA, PIPE_SIMPLE)>("256x128_w2x2_cw_ks", false),
#else
    ROW("128x128_w2x2_dma", 128, 128, 2, 2, LOAD_DMA, false),
#endif
    // 192 x 256 on the 8-wave solo schedule (96 x 64 wave tiles): for row counts whose 256-row tiles would leave
    // a round of CUs partly empty (3072 rows against 4096 columns: 256 tiles instead of 192), and its twin for
    // K-contiguous a_scale.  K-contiguous operands only.
#if INST_KMAJ
    ROW("128x128_w2x2_dma", 128, 128, 2, 2, LOAD_DMA, false),
    ROW("128x128_w2x2_dma", 128, 128, 2, 2, LOAD_DMA, false),
#else
    ROWP("192x256_w2x4_solo8", 192, 256, 2, 4, LOAD_DMA, PIPE_SOLO, true),
#if INST_BLOCK
    row_of<true, GemmCfg<INST_ARITH, true, 192, 256, 2, 4, LOAD_DMA, PIPE_SOLO, 0, true, 0, 0, 1, true>,
           CFG(128, 128, 2, 2, LOAD_DMA, PIPE_SIMPLE)>("192x256_w2x4_solo8_ks", false),
#else
    ROW("128x128_w2x2_dma", 128, 128, 2, 2, LOAD_DMA, false),
#endif
#endif
};

const Variant *INST_FN(int *count) {
    *count = (int)(sizeof(kTable) / sizeof(kTable[0]));
    return kTable;
}

}  // namespace qgemm
