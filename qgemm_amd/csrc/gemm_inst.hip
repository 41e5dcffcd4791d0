// Instantiates the MFMA GEMM template for one arithmetic family.  Compiled once
// per family with -DINST_ARITH=<Arith> -DINST_BLOCK=<0|1> -DINST_FN=<table fn>,
// so the families build in parallel.
#include "variants.h"
#include "gemm_skinny.cuh"

#include <atomic>
#include <cstring>
#include <vector>

#ifndef INST_ARITH
#error "compile with -DINST_ARITH=... -DINST_BLOCK=... -DINST_FN=... [-DINST_KMAJ=1|2|3]"
#endif
#ifndef INST_KMAJ
#define INST_KMAJ 0      // bit 0: A stored K x M, bit 1: B stored K x N (see GemmCfg::KMAJ)
#endif

namespace qgemm {

// More than 64 KiB of dynamic LDS has to be asked for explicitly, once per kernel and device.
template <class K>
static hipError_t allow_lds(K kernel, int bytes) {
    static std::atomic<uint64_t> done{0};          // one bit per device
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const uint64_t bit = (uint64_t)1 << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
    e = hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
    return e;
}

template <class C>
static hipError_t launch_variant(const GemmArgs &a, uint32_t grid, hipStream_t s) {
    hipError_t e = allow_lds(gemm_nt_kernel<C>, C::LDS_BYTES);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(gemm_nt_kernel<C>, dim3(grid), dim3(C::THREADS), C::LDS_BYTES, s, a);
    return hipGetLastError();
}

template <class C>
static hipError_t launch_skinny(const GemmArgs &a, uint32_t grid, hipStream_t s) {
    hipError_t e = allow_lds(gemm_skinny_kernel<C>, C::LDS_BYTES);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(gemm_skinny_kernel<C>, dim3(grid), dim3(C::THREADS), C::LDS_BYTES, s, a);
    return hipGetLastError();
}

constexpr int kElemBytes = (INST_ARITH == AR_BF16 || INST_ARITH == AR_F16) ? 2 : 1;
constexpr bool kBlock = (bool)INST_BLOCK;
// A K-major operand needs whole 128-byte panels of its tile side and a multiple of four waves (GemmCfg's
// static_asserts); tiles that cannot have that are left out of a K-major family.
constexpr bool kmajor_can(int bm, int bn, int nw) {
    return INST_KMAJ == 0 || (nw % 4 == 0 && (!(INST_KMAJ & 1) || (bm * kElemBytes) % 128 == 0) &&
                              (!(INST_KMAJ & 2) || (bn * kElemBytes) % 128 == 0));
}

template <class C>
static Variant gemm_row(const char *name, bool auto_ok) {
    return Variant{name, C::ARITH, C::BLOCK_SCALE, C::BM, C::BN, C::THREADS, C::LDS_BYTES, auto_ok, C::COPYW, C::KG, C::ASK,
                   C::AS_ANY_STRIDE, -1, 0, &launch_variant<C>};
}
// row of the skinny-M kernel (gemm_skinny.cuh): 16 * TM rows x 16 * TN columns, eight waves splitting K between them.
// Picked by choose_variant in place of the narrow simple-pipeline tiles, never by the table scan (auto_ok = false).
template <int TM, int TN = 2>
static Variant skinny_row(const char *name) {
    using C = SkinnyCfg<INST_ARITH, TM, kBlock, TN>;
    return Variant{name, C::ARITH, C::BLOCK_SCALE, C::BM, C::BN, C::THREADS, C::LDS_BYTES, false, false, 8, false, C::BLOCK_SCALE,
                   -1, 0, &launch_skinny<C>};
}

// simple pipeline
template <int BM, int BN, int WM, int WN, int STAGES = 0, int KG = 1>
using Simple = GemmCfg<INST_ARITH, kBlock, BM, BN, WM, WN, PIPE_SIMPLE, INST_KMAJ, STAGES, KG>;
// solo pipeline (ASK: the twin that reads a_scale K-contiguous; COPYW: four copying waves beside four computing ones)
template <int BM, int BN, int WM, int WN, bool ASK = false, bool COPYW = false>
using Solo = GemmCfg<INST_ARITH, kBlock, BM, BN, WM, WN, PIPE_SOLO, INST_KMAJ, 0, 1, ASK, COPYW>;

static std::vector<Variant> build_table() {
    std::vector<Variant> t;
    auto add = [&](const Variant &v) { t.push_back(v); };
    // a row and its twin for K-contiguous a_scale (block-scaled, K-contiguous families only)
    auto add_pair = [&](const Variant &base, const Variant &ks, int ks_blocks) {
        const int i = (int)t.size();
        t.push_back(base);
        t.push_back(ks);
        t[i].twin = i + 1;
        t[i + 1].twin = i;
        t[i + 1].ks_blocks = ks_blocks;
    };
    if constexpr (kmajor_can(128, 128, 4)) add(gemm_row<Simple<128, 128, 2, 2>>("128x128_w2x2_dma", true));
    if constexpr (kmajor_can(64, 128, 4)) add(gemm_row<Simple<64, 128, 1, 4>>("64x128_w1x4_dma", true));
    if constexpr (kmajor_can(32, 128, 4)) add(gemm_row<Simple<32, 128, 1, 4>>("32x128_w1x4_dma", true));
    if constexpr (kmajor_can(16, 128, 2)) add(gemm_row<Simple<16, 128, 1, 2>>("16x128_w1x2_dma", true));
    // narrow tiles for skinny M: N / 32 workgroups stream disjoint strips of B over the whole of K, so no
    // K split (and no second pass over partial sums) is needed to occupy the CUs
    if constexpr (kmajor_can(128, 32, 4)) add(gemm_row<Simple<128, 32, 4, 1>>("128x32_w4x1_dma", true));
    if constexpr (kmajor_can(64, 32, 4)) add(gemm_row<Simple<64, 32, 4, 1>>("64x32_w4x1_dma", true));
    if constexpr (kmajor_can(16, 32, 2)) add(gemm_row<Simple<16, 32, 1, 2>>("16x32_w1x2_dma", true));
    // 128 x 128 with eight computing waves in two K groups and four copying waves (GemmCfg::KG), five stages (160 KiB,
    // one workgroup per CU; four with block scales, whose a_scale values take 2 KiB behind the ring): for shapes with
    // no more tiles than CUs, where the two-stage row above would sit alone on its CU
    // (K-major families too: the waves that read the tile with the transposing LDS reads have no copies in flight)
    if constexpr (kmajor_can(128, 128, 4)) add(gemm_row<Simple<128, 128, 2, 2, kBlock ? 4 : 5, 2>>("128x128_w2x2_k2", true));
    // the same for the 64 x 128 tile, with six stages
    if constexpr (kmajor_can(64, 128, 4)) add(gemm_row<Simple<64, 128, 1, 4, 6, 2>>("64x128_w1x4_k2", true));
    if constexpr (INST_KMAJ == 0) {
        // The 256 x 256 tile: fp8 per-matrix runs fastest on the 4-wave solo schedule (a third fewer LDS reads: 3 % in
        // interleaved runs); for int8 and the 16-bit types the table marks the 8-wave one and choose_variant swaps in
        // the 4-wave one where the tiles fill whole rounds of CUs; block scales need the 8-wave form (accumulators in
        // vector registers), which has a twin reading a_scale with the K blocks contiguous, two per load.
        if constexpr (!kBlock) add(gemm_row<Solo<256, 256, 2, 2>>("256x256_w2x2_solo", INST_ARITH == AR_F8));
        if constexpr (kBlock)
            add_pair(gemm_row<Solo<256, 256, 2, 4>>("256x256_w2x4_solo8", true),
                     gemm_row<Solo<256, 256, 2, 4, true>>("256x256_w2x4_solo8_ks", false), 2);
        else
            add(gemm_row<Solo<256, 256, 2, 4>>("256x256_w2x4_solo8", INST_ARITH != AR_F8));
        // 192 x 256 on the 8-wave solo schedule (96 x 64 wave tiles): for row counts whose 256-row tiles would leave
        // a round of CUs partly empty (3072 rows against 4096 columns: 256 tiles instead of 192)
        if constexpr (kBlock)
            add_pair(gemm_row<Solo<192, 256, 2, 4>>("192x256_w2x4_solo8", true),
                     gemm_row<Solo<192, 256, 2, 4, true>>("192x256_w2x4_solo8_ks", false), 2);
        else
            add(gemm_row<Solo<192, 256, 2, 4>>("192x256_w2x4_solo8", true));
        // skinny M (gemm_skinny.cuh): the K split inside the workgroup, no staging, no barrier in the K loop; on a
        // 64 x 64 tile for shapes with a few row tiles whose 64 x 64 tiles fit one round of CUs
        add(skinny_row<1>("skinny_16x32_k8"));
        add(skinny_row<2>("skinny_32x32_k8"));
        add(skinny_row<4>("skinny_64x32_k8"));
        add(skinny_row<8>("skinny_128x32_k8"));
        add(skinny_row<4, 4>("skinny_64x64_k8"));
        add(skinny_row<1, 1>("skinny_16x16_k8"));
        add(skinny_row<2, 1>("skinny_32x16_k8"));
    }
    // 256 x 128 on the solo schedule with four computing waves (128 x 64 wave tiles, one per SIMD) and four copying
    // waves (GemmCfg::COPYW): block scales and K-major operands on a large tile; its twin for K-contiguous a_scale
    // takes the scales of four K blocks per copy
    if constexpr (kBlock && INST_KMAJ == 0)
        add_pair(gemm_row<Solo<256, 128, 2, 2, false, true>>("256x128_w2x2_cw", true),
                 gemm_row<Solo<256, 128, 2, 2, true, true>>("256x128_w2x2_cw_ks", false), 4);
    else
        add(gemm_row<Solo<256, 128, 2, 2, false, true>>("256x128_w2x2_cw", true));
    return t;
}

const Variant *INST_FN(int *count) {
    static const std::vector<Variant> table = build_table();
    *count = (int)table.size();
    return table.data();
}

}  // namespace qgemm
