/*! \file gemm.h
    \brief Host API of the matrix multiply entry points (drop-in for the reference's include/gemm.h).

    Same template names and the same 9-argument shape as include/gemm.h:25-66 of the reference:

        template <typename typeIn, typename typeOut>
        void GEMM_kernel_vN(const typeIn* A, size_t ldA, const typeIn* B, size_t ldB,
                            typeOut* C, size_t ldC, size_t M, size_t N, size_t K);

    v1 .. v5 take B as K x N row-major ("NN", src/include/gemm_utils.cuh:93,108); v3_1 and v4_1 take
    B as N x K row-major ("NT", gemm_utils.cuh:259,271).  In the reference the seven names are seven
    stages of one CUDA kernel; here they all forward to the one gfx950 MFMA kernel through the C ABI
    (include/qgemm.h), which picks its own tiling.  All pointers are device pointers; work is
    enqueued on the default stream and the call returns without synchronising.

    Error behaviour follows the reference: v1 / v2 report nothing; v3 and later print the failure to
    std::cerr and continue (src/gemm/sm89_gemm_kernel_v3.cu:294-298).

    The reference instantiates <bf16, float> only.  Supported here: typeIn in {__hip_bfloat16, __half,
    int8_t, __hip_fp8_e4m3}, typeOut in {float, __hip_bfloat16, __half} (and int32_t for int8_t).
*/
#pragma once
#include "common.h"
#include "gpu_type.h"
#include "qgemm.h"

namespace qgemm_host {

template <typename T> struct dtype_of;
template <> struct dtype_of<float> { static constexpr int value = QGEMM_DT_F32; };
template <> struct dtype_of<__hip_bfloat16> { static constexpr int value = QGEMM_DT_BF16; };
template <> struct dtype_of<__half> { static constexpr int value = QGEMM_DT_F16; };
template <> struct dtype_of<int8_t> { static constexpr int value = QGEMM_DT_I8; };
template <> struct dtype_of<int32_t> { static constexpr int value = QGEMM_DT_I32; };
template <> struct dtype_of<__hip_fp8_e4m3> { static constexpr int value = QGEMM_DT_F8E4M3; };

// The reference's launchers accept ldA and ldB and never use them: every loader indexes A with K and B with N
// ("NN", src/include/gemm_utils.cuh:93,108,208,220) or with K ("NT", :259,271; the v3.1 launcher passes K in the
// place of ldB, sm80_gemm_kernel_v3.1.cu:292), and the reference's harness calls every entry, the NT ones
// included, with ldB = N (tests/includes/test_config.h:238).  The drop-ins do the same: dense A and B whatever
// ldA / ldB say; only ldC is honoured (sm89_gemm_kernel_v3.cu:258).  Strided operands are available through
// qgemm_gemm itself.
template <typename typeIn, typename typeOut>
inline int gemm_forward(int layout_b, const typeIn *A, size_t /*ldA*/, const typeIn *B, size_t /*ldB*/, typeOut *C,
                        size_t ldC, size_t M, size_t N, size_t K, bool report) {
    const int st = qgemm_gemm(dtype_of<typeIn>::value, dtype_of<typeOut>::value, layout_b, A, K, B,
                              layout_b == QGEMM_B_KN ? N : K, C, ldC, M, N, K, nullptr);
    if (st != QGEMM_OK && report)
        std::cerr << "HIP kernel launch error: " << qgemm_status_string(st) << std::endl;
    return st;
}

}  // namespace qgemm_host

#define QGEMM_DEFINE_ENTRY(NAME, LAYOUT, REPORT)                                                              \
    template <typename typeIn, typename typeOut>                                                              \
    inline void NAME(const typeIn *A, size_t ldA, const typeIn *B, size_t ldB, typeOut *C, size_t ldC,        \
                     size_t M, size_t N, size_t K) {                                                          \
        (void)qgemm_host::gemm_forward<typeIn, typeOut>(LAYOUT, A, ldA, B, ldB, C, ldC, M, N, K, REPORT);     \
    }

QGEMM_DEFINE_ENTRY(GEMM_kernel_v1, QGEMM_B_KN, false)
QGEMM_DEFINE_ENTRY(GEMM_kernel_v2, QGEMM_B_KN, false)
QGEMM_DEFINE_ENTRY(GEMM_kernel_v3, QGEMM_B_KN, true)
QGEMM_DEFINE_ENTRY(GEMM_kernel_v3_1, QGEMM_B_NK, true)
QGEMM_DEFINE_ENTRY(GEMM_kernel_v4, QGEMM_B_KN, true)
QGEMM_DEFINE_ENTRY(GEMM_kernel_v4_1, QGEMM_B_NK, true)
QGEMM_DEFINE_ENTRY(GEMM_kernel_v5, QGEMM_B_KN, true)

#undef QGEMM_DEFINE_ENTRY
