// qgemm_python: the torch extension module the reference's packaging names (setup.py:73) and its
// HIP source begins (void fp8_mm(torch::Tensor a, b, as, bs, c), hip_mix_gemm_kernel.cpp:508-516;
// bf16_mm / int8_mm are the commented intent of src/gemm/sm80_gemm_kernel.cu:4-22).  Host code only:
// every function checks its tensors and forwards their data pointers, with torch's current stream, to the
// C ABI of libqgemm.so.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>

#include <stdexcept>
#include <string>

#include "../../include/qgemm.h"

namespace {

void *current_stream() { return (void *)c10::hip::getCurrentHIPStream().stream(); }

void check(int status, const char *what) {
    if (status != QGEMM_OK) throw std::runtime_error(std::string(what) + ": " + qgemm_status_string(status));
}

int dtype_of(const torch::Tensor &t) {
    switch (t.scalar_type()) {
        case torch::kFloat32: return QGEMM_DT_F32;
        case torch::kBFloat16: return QGEMM_DT_BF16;
        case torch::kFloat16: return QGEMM_DT_F16;
        case torch::kInt8: return QGEMM_DT_I8;
        case torch::kInt32: return QGEMM_DT_I32;
        case torch::kFloat8_e4m3fn: return QGEMM_DT_F8E4M3;
        case torch::kUInt8: return QGEMM_DT_F8E4M3;      // raw e4m3 codes
        default: throw std::runtime_error("qgemm_python: unsupported tensor dtype");
    }
}

void need_device(const torch::Tensor &t, const char *name) {
    if (!t.is_cuda()) throw std::runtime_error(std::string("qgemm_python: ") + name + " must be a device tensor");
}

// The kernels decode OCP e4m3 (torch.float8_e4m3fn or raw codes as uint8); the gfx942 "fnuz" encoding has another
// bias and another NaN and is refused.
void need_fp8(const torch::Tensor &t, const char *name) {
    if (t.scalar_type() != torch::kFloat8_e4m3fn && t.scalar_type() != torch::kUInt8)
        throw std::runtime_error(std::string("qgemm_python: ") + name + " must be float8_e4m3fn (OCP e4m3) or uint8 codes");
}

// c is [m, n] with unit inner stride; its row stride becomes ldC
void need_out(const torch::Tensor &c, size_t m, size_t n) {
    if (c.dim() != 2 || (size_t)c.size(0) != m || (size_t)c.size(1) != n || c.stride(1) != 1 || (m > 1 && (size_t)c.stride(0) < n))
        throw std::runtime_error("qgemm_python: c must be [m, n] with unit inner stride");
}

// The reference's contract (hip_mix_gemm_kernel.cpp:425-439): a is [m, k] column-major (storage a[i + j*m]),
// b is [n, k] column-major (storage [k, n] row-major), a_scale [m, k/128] and b_scale [n/128, k/128]
// column-major, c [m, n] row-major bf16; m = a.size(0), n = b.size(0), k = a.size(1).
void fp8_mm(torch::Tensor a, torch::Tensor b, torch::Tensor as, torch::Tensor bs, torch::Tensor c) {
    need_device(a, "a"); need_device(b, "b"); need_device(as, "a_scale"); need_device(bs, "b_scale"); need_device(c, "c");
    const size_t m = a.size(0), n = b.size(0), k = a.size(1);
    need_fp8(a, "a"); need_fp8(b, "b");
    need_out(c, m, n);
    check(qgemm_scaled_gemm(QGEMM_DT_F8E4M3, dtype_of(c), QGEMM_SCALE_BLOCK128, QGEMM_LAYOUT_REFERENCE, a.data_ptr(),
                            b.data_ptr(), as.data_ptr<float>(), bs.data_ptr<float>(), c.data_ptr(), c.stride(0), m, n, k, 0,
                            current_stream()),
          "fp8_mm");
}

// K-contiguous operands (a [m, k], b [n, k] row-major), one fp32 scale each; c fp32 / bf16 / fp16 (or int32 for
// the raw int8 accumulators).
void scaled_mm(torch::Tensor a, torch::Tensor b, torch::Tensor as, torch::Tensor bs, torch::Tensor c, const char *what) {
    need_device(a, "a"); need_device(b, "b"); need_device(as, "a_scale"); need_device(bs, "b_scale"); need_device(c, "c");
    if (!a.is_contiguous() || !b.is_contiguous() || a.size(1) != b.size(1))
        throw std::runtime_error(std::string(what) + ": a [m, k] and b [n, k] must be contiguous with equal k");
    const size_t m = a.size(0), n = b.size(0), k = a.size(1);
    need_out(c, m, n);
    check(qgemm_scaled_gemm(dtype_of(a), dtype_of(c), QGEMM_SCALE_PER_MATRIX, QGEMM_LAYOUT_K_CONTIGUOUS, a.data_ptr(),
                            b.data_ptr(), as.data_ptr<float>(), bs.data_ptr<float>(), c.data_ptr(), c.stride(0), m, n, k, 0,
                            current_stream()),
          what);
}
void int8_mm(torch::Tensor a, torch::Tensor b, torch::Tensor as, torch::Tensor bs, torch::Tensor c) {
    if (a.scalar_type() != torch::kInt8 || b.scalar_type() != torch::kInt8)
        throw std::runtime_error("qgemm_python: int8_mm takes int8 operands");
    scaled_mm(a, b, as, bs, c, "int8_mm");
}
void fp8_mm_per_matrix(torch::Tensor a, torch::Tensor b, torch::Tensor as, torch::Tensor bs, torch::Tensor c) {
    need_fp8(a, "a"); need_fp8(b, "b");
    scaled_mm(a, b, as, bs, c, "fp8_mm_per_matrix");
}

// c [m, n] = a [m, k] x b [n, k]^T, 16-bit operands, fp32 accumulation
void bf16_mm(torch::Tensor a, torch::Tensor b, torch::Tensor c) {
    need_device(a, "a"); need_device(b, "b"); need_device(c, "c");
    if (a.size(1) != b.size(1) || a.stride(1) != 1 || b.stride(1) != 1 || c.stride(1) != 1)
        throw std::runtime_error("bf16_mm: a [m, k] and b [n, k] with unit inner strides");
    need_out(c, a.size(0), b.size(0));
    check(qgemm_gemm(dtype_of(a), dtype_of(c), QGEMM_B_NK, a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0), c.data_ptr(),
                     c.stride(0), a.size(0), b.size(0), a.size(1), current_stream()),
          "bf16_mm");
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "MI355X scaled mixed-precision GEMM (torch-facing entry points over libqgemm.so)";
    m.def("fp8_mm", &fp8_mm, "block-scaled fp8 GEMM, reference layout: fp8_mm(a, b, a_scale, b_scale, c)");
    m.def("fp8_mm_per_matrix", &fp8_mm_per_matrix, "per-matrix scaled fp8 GEMM, K-contiguous operands");
    m.def("int8_mm", &int8_mm, "per-matrix scaled int8 GEMM, K-contiguous operands");
    m.def("bf16_mm", &bf16_mm, "bf16 / fp16 GEMM, b stored [n, k]");
}
