// Scaled mixed-precision GEMM entry points of src/mix_gemm (drop-in).
//
//   select_BLOCK_TILE_SIZE_M(A, B, as, bs, C, M, N, K)   hip_mix_gemm_kernel.cpp:489-505
//       raw-pointer entry of the FP8 128-block-scaled GEMM, with the reference's storage
//       contract (:425-439): A[m + k*M], B[k*N + n], as[m + kb*M], bs[nb + kb*ceil(N/128)],
//       C[m*N + n] bf16.  Throws std::runtime_error with the reference's message when M, N or
//       K is not a multiple of 32 (:460,485,503).
//   fp8_mm(a, b, as, bs, c)                               hip_mix_gemm_kernel.cpp:508-516
//       the torch::Tensor wrapper (needs <torch/extension.h> included first).
//   int8_mm / fp8_mm_per_matrix                            src/gemm/sm80_gemm_kernel.cu:14-22 (stub)
//       per-matrix scaled GEMMs on K-contiguous operands: A[m*K + k], B[n*K + k].
//
// The element type of the reference is the gfx942 "fnuz" fp8; gfx950 decodes OCP e4m3.
#pragma once
#include <stdexcept>
#include <string>

#include "common.h"
#include "gpu_type.h"
#include "qgemm.h"

namespace qgemm_host {

inline void throw_on_status(int st, size_t M, size_t N, size_t K) {
    switch (st) {
        case QGEMM_OK: return;
        case QGEMM_ERR_NOT_DIVISIBLE_M:
            throw std::runtime_error("M (" + std::to_string(M) +
                                     ") is not divisible by any predefined BLOCK_TILE_SIZE_M in the list.");
        case QGEMM_ERR_NOT_DIVISIBLE_N:
            throw std::runtime_error("N (" + std::to_string(N) +
                                     ") is not divisible by any predefined BLOCK_TILE_SIZE_N in the list.");
        case QGEMM_ERR_NOT_DIVISIBLE_K:
            throw std::runtime_error("K (" + std::to_string(K) +
                                     ") is not divisible by any predefined BLOCK_TILE_SIZE_K in the list.");
        default: throw std::runtime_error(std::string("qgemm: ") + qgemm_status_string(st));
    }
}

}  // namespace qgemm_host

inline void select_BLOCK_TILE_SIZE_M(const __hip_fp8_e4m3 *A, const __hip_fp8_e4m3 *B, const float *as, const float *bs,
                                     __hip_bfloat16 *C, size_t M, size_t N, size_t K) {
    qgemm_host::throw_on_status(
        qgemm_scaled_gemm(QGEMM_DT_F8E4M3, QGEMM_DT_BF16, QGEMM_SCALE_BLOCK128, QGEMM_LAYOUT_REFERENCE, A, B, as, bs, C,
                          N, M, N, K, 0, nullptr),
        M, N, K);
}

// C = (sA * sB) * (A x B^T), int32 accumulation; typeOut float / __hip_bfloat16 / __half / int32_t (raw accumulators)
template <typename typeOut>
inline void int8_mm(const int8_t *A, const int8_t *B, const float *as, const float *bs, typeOut *C, size_t M, size_t N,
                    size_t K);
template <> inline void int8_mm<float>(const int8_t *A, const int8_t *B, const float *as, const float *bs, float *C,
                                       size_t M, size_t N, size_t K) {
    qgemm_host::throw_on_status(qgemm_scaled_gemm(QGEMM_DT_I8, QGEMM_DT_F32, QGEMM_SCALE_PER_MATRIX,
                                                  QGEMM_LAYOUT_K_CONTIGUOUS, A, B, as, bs, C, N, M, N, K, 0, nullptr),
                                M, N, K);
}
template <> inline void int8_mm<int32_t>(const int8_t *A, const int8_t *B, const float *as, const float *bs,
                                         int32_t *C, size_t M, size_t N, size_t K) {
    qgemm_host::throw_on_status(qgemm_scaled_gemm(QGEMM_DT_I8, QGEMM_DT_I32, QGEMM_SCALE_PER_MATRIX,
                                                  QGEMM_LAYOUT_K_CONTIGUOUS, A, B, as, bs, C, N, M, N, K, 0, nullptr),
                                M, N, K);
}
template <> inline void int8_mm<__hip_bfloat16>(const int8_t *A, const int8_t *B, const float *as, const float *bs,
                                                __hip_bfloat16 *C, size_t M, size_t N, size_t K) {
    qgemm_host::throw_on_status(qgemm_scaled_gemm(QGEMM_DT_I8, QGEMM_DT_BF16, QGEMM_SCALE_PER_MATRIX,
                                                  QGEMM_LAYOUT_K_CONTIGUOUS, A, B, as, bs, C, N, M, N, K, 0, nullptr),
                                M, N, K);
}

// per-matrix scaled fp8, K-contiguous operands, bf16 out
inline void fp8_mm_per_matrix(const __hip_fp8_e4m3 *A, const __hip_fp8_e4m3 *B, const float *as, const float *bs,
                              __hip_bfloat16 *C, size_t M, size_t N, size_t K) {
    qgemm_host::throw_on_status(qgemm_scaled_gemm(QGEMM_DT_F8E4M3, QGEMM_DT_BF16, QGEMM_SCALE_PER_MATRIX,
                                                  QGEMM_LAYOUT_K_CONTIGUOUS, A, B, as, bs, C, N, M, N, K, 0, nullptr),
                                M, N, K);
}

#if defined(TORCH_EXTENSION_NAME) || defined(TORCH_API_INCLUDE_EXTENSION_H)
// m = a.size(0), n = b.size(0), k = a.size(1), exactly as the reference reads them
inline void fp8_mm(torch::Tensor a, torch::Tensor b, torch::Tensor as, torch::Tensor bs, torch::Tensor c) {
    const size_t m = a.size(0), n = b.size(0), k = a.size(1);
    select_BLOCK_TILE_SIZE_M(static_cast<const __hip_fp8_e4m3 *>(a.data_ptr()),
                             static_cast<const __hip_fp8_e4m3 *>(b.data_ptr()), as.data_ptr<float>(),
                             bs.data_ptr<float>(), static_cast<__hip_bfloat16 *>(c.data_ptr()), m, n, k);
}
#endif
