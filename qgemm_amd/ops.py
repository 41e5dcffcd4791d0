"""Host-side mirror of the reference's operator interface, over the C ABI.

  fp8_mm(a, b, as, bs, c)      src/mix_gemm/hip_mix_gemm_kernel.cpp:508-516
  int8_mm / bf16_mm            the stubs in src/gemm/sm80_gemm_kernel.cu:4-22
  int8_mm_block                int8 operands with the 128-block scales of fp8_mm (no counterpart in the reference)
  matrix_transpose(in, out)    src/transpose/transpose.cu:60-74
  gemm(...)                    GEMM_kernel_v*<In, Out> of include/gemm.h:25-66
  quantize(x, ...)             the Q_A / Q_B of README.md:1 (the reference has no quantiser)

Tensors are torch CUDA(HIP) tensors; only their data pointers and the current
stream cross the boundary."""
import ctypes as C

import torch

from .lib import check, load_library

DT_F32, DT_BF16, DT_F16, DT_I8, DT_F8E4M3, DT_I32 = 0, 1, 2, 3, 4, 5
B_KN, B_NK = 0, 1
SCALE_PER_MATRIX, SCALE_BLOCK128 = 1, 2
LAYOUT_K_CONTIGUOUS, LAYOUT_REFERENCE = 0, 1
QUANT_PER_MATRIX, QUANT_BLOCK_1x128, QUANT_BLOCK_128x128 = 1, 2, 3

_TORCH_DT = {
    torch.float32: DT_F32, torch.bfloat16: DT_BF16, torch.float16: DT_F16, torch.int8: DT_I8,
    torch.int32: DT_I32, torch.float8_e4m3fn: DT_F8E4M3,
}


def _dt(t, fp8_as_uint8=False):
    if t.dtype == torch.uint8 and fp8_as_uint8:
        return DT_F8E4M3
    try:
        return _TORCH_DT[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported tensor dtype {t.dtype}") from None


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need_gpu(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise ValueError("qgemm operates on device tensors only (there is no CPU path)")


def set_option(key, value):
    check(load_library().qgemm_set_option(key.encode(), int(value)))


def force_config(name=None):
    """Pin the row `name` of the variant tables for the GEMM calls that follow (None: back to the heuristic)."""
    check(load_library().qgemm_force_config(name.encode() if name else None))


def variant_names(in_dtype, scale_mode=0, k_major=0):
    """Names of the rows of the family that serves (in_dtype, scale_mode, k_major); arguments as for plan()."""
    lib = load_library()
    out = []
    for i in range(lib.qgemm_variant_count(in_dtype, scale_mode, k_major)):
        buf = C.create_string_buffer(64)
        check(lib.qgemm_variant_name(in_dtype, scale_mode, k_major, i, buf, 64))
        out.append(buf.value.decode())
    return out


def plan(in_dtype, scale_mode, k_major, M, N, K):
    """Name of the kernel configuration the library would choose (no launch, no device needed)."""
    buf = C.create_string_buffer(128)
    check(load_library().qgemm_plan(in_dtype, scale_mode, k_major, M, N, K, buf, 128))
    return buf.value.decode()


def last_config():
    buf = C.create_string_buffer(128)
    check(load_library().qgemm_last_config(buf, 128))
    return buf.value.decode()


def selftest_layouts():
    """-> (ok, report)"""
    buf = C.create_string_buffer(4096)
    st = load_library().qgemm_selftest_layouts(buf, 4096)
    return st == 0, buf.value.decode()


def tile_map(wg, tiles_m, tiles_n, group_m):
    tm, tn = C.c_uint32(), C.c_uint32()
    check(load_library().qgemm_tile_map(wg, tiles_m, tiles_n, group_m, C.byref(tm), C.byref(tn)))
    return tm.value, tn.value


def gemm(A, B, C_out, layout_b="nk", M=None, N=None, K=None, ldA=None, ldB=None, ldC=None):
    """C[M,N] = A[M,K] @ B.  layout_b "kn": B is [K,N] (GEMM_kernel_v1..v5);
    "nk": B is [N,K] (GEMM_kernel_v3_1 / v4_1)."""
    _need_gpu(A, B, C_out)
    lb = {"kn": B_KN, "nk": B_NK}[layout_b]
    M = A.shape[0] if M is None else M
    K = A.shape[1] if K is None else K
    N = (B.shape[1] if lb == B_KN else B.shape[0]) if N is None else N
    ldA = A.stride(0) if ldA is None else ldA
    ldB = B.stride(0) if ldB is None else ldB
    ldC = C_out.stride(0) if ldC is None else ldC
    check(load_library().qgemm_gemm(_dt(A, True), _dt(C_out), lb, A.data_ptr(), ldA, B.data_ptr(), ldB,
                                    C_out.data_ptr(), ldC, M, N, K, _stream()))
    return C_out


def scaled_gemm(A, B, a_scale, b_scale, C_out, M, N, K, scale_mode, layout=LAYOUT_K_CONTIGUOUS, split_k=0,
                in_dtype=None, ldC=None):
    _need_gpu(A, B, a_scale, b_scale, C_out)
    in_dtype = _dt(A, True) if in_dtype is None else in_dtype
    ldC = C_out.stride(0) if ldC is None else ldC
    check(load_library().qgemm_scaled_gemm(
        in_dtype, _dt(C_out), scale_mode, layout, A.data_ptr(), B.data_ptr(),
        a_scale.data_ptr() if a_scale is not None else None, b_scale.data_ptr() if b_scale is not None else None,
        C_out.data_ptr(), ldC, M, N, K, split_k, _stream()))
    return C_out


def _need_fp8(*ts):
    """The kernels decode OCP e4m3 (torch.float8_e4m3fn, or its raw codes as uint8).  The gfx942 "fnuz" encoding
    the reference's fp8_mm names has another bias and another NaN: refuse it rather than compute with every value
    doubled."""
    for t in ts:
        if t.dtype not in (torch.float8_e4m3fn, torch.uint8):
            raise TypeError(f"fp8 operands must be torch.float8_e4m3fn (OCP e4m3) or uint8 codes, got {t.dtype}")


def _need_out(c, m, n):
    if c.dim() != 2 or tuple(c.shape) != (m, n) or c.stride(1) != 1 or (m > 1 and c.stride(0) < n):
        raise ValueError(f"c must be [{m}, {n}] with unit inner stride, got shape {tuple(c.shape)} strides {c.stride()}")


def fp8_mm(a, b, a_scale, b_scale, c):
    """The reference entry (hip_mix_gemm_kernel.cpp:425-439, 508-516):
      a        [m, k] fp8, column-major  (storage a[i + j*m])
      b        [n, k] fp8, column-major  (storage b[n + k*n_total], i.e. [k, n] row-major)
      a_scale  [m, k/128] fp32, column-major;  b_scale [n/128, k/128] fp32, column-major
      c        [m, n] bf16, row-major
    m = a.size(0), n = b.size(0), k = a.size(1) exactly as the reference reads them."""
    m, n, k = a.size(0), b.size(0), a.size(1)
    _need_fp8(a, b)
    _need_out(c, m, n)
    return scaled_gemm(a, b, a_scale, b_scale, c, m, n, k, SCALE_BLOCK128, LAYOUT_REFERENCE, in_dtype=DT_F8E4M3,
                       ldC=c.stride(0))


def int8_mm(a, b, a_scale, b_scale, c, split_k=0):
    """Per-matrix scaled int8 GEMM: a [m,k] int8, b [n,k] int8 (both K-contiguous), one fp32 scale each,
    c [m,n] fp32 / bf16 / fp16, or int32 for the raw accumulators."""
    m, k = a.shape
    n = b.shape[0]
    if a.dtype != torch.int8 or b.dtype != torch.int8:
        raise TypeError(f"int8_mm takes int8 operands, got {a.dtype} and {b.dtype}")
    _need_out(c, m, n)
    return scaled_gemm(a, b, a_scale, b_scale, c, m, n, k, SCALE_PER_MATRIX, split_k=split_k, in_dtype=DT_I8,
                       ldC=c.stride(0))


def int8_mm_block(a, b, a_scale, b_scale, c, split_k=0):
    """int8 GEMM with 128-block scales, the int8 twin of fp8_mm's arithmetic (hip_mix_gemm_kernel.cpp:231-244) on
    K-contiguous operands: a [m,k] int8, b [n,k] int8, a_scale [m, ceil(k/128)] and b_scale [ceil(n/128), ceil(k/128)]
    fp32 row-major, c [m,n] fp32 / bf16 / fp16.  Every 128-wide K block's exact int32 partial is folded into an fp32
    sum with a_scale[m, kb] * b_scale[n // 128, kb]."""
    m, k = a.shape
    n = b.shape[0]
    if a.dtype != torch.int8 or b.dtype != torch.int8:
        raise TypeError(f"int8_mm_block takes int8 operands, got {a.dtype} and {b.dtype}")
    _need_out(c, m, n)
    return scaled_gemm(a, b, a_scale, b_scale, c, m, n, k, SCALE_BLOCK128, split_k=split_k, in_dtype=DT_I8, ldC=c.stride(0))


def bf16_mm(a, b, c):
    """a [m,k], b [n,k] (K-contiguous), c [m,n]; plain GEMM with fp32 accumulation."""
    return gemm(a, b, c, "nk")


def matrix_transpose(idata, odata, M=None, N=None):
    """odata[N, M] = idata[M, N]^T for 1-, 2- or 4-byte elements."""
    _need_gpu(idata, odata)
    M = idata.shape[0] if M is None else M
    N = idata.shape[1] if N is None else N
    check(load_library().qgemm_transpose(idata.element_size(), idata.data_ptr(), odata.data_ptr(), M, N, _stream()))
    return odata


def quantize(x, out_dtype=torch.float8_e4m3fn, mode=QUANT_PER_MATRIX, rows_contiguous_scales=False):
    """q, scales = quantise(x): x [rows, cols] fp32 / bf16 / fp16 (row stride free), q [rows, cols] int8 or
    fp8-e4m3.  scales: [1] for QUANT_PER_MATRIX; [rows, ceil(cols/128)] for QUANT_BLOCK_1x128 (or its
    transpose, storage [ceil(cols/128), rows], with rows_contiguous_scales: the a_scale arrangement of the
    reference layout); [ceil(rows/128), ceil(cols/128)] for QUANT_BLOCK_128x128 (transposed likewise)."""
    _need_gpu(x)
    assert x.dim() == 2 and x.stride(1) == 1
    rows, cols = x.shape
    q = torch.empty((rows, cols), dtype=out_dtype, device=x.device)
    if mode == QUANT_PER_MATRIX:
        scales = torch.empty(1, dtype=torch.float32, device=x.device)
        rs = cs = 0
    else:
        nbr = rows if mode == QUANT_BLOCK_1x128 else (rows + 127) // 128
        nbc = (cols + 127) // 128
        if rows_contiguous_scales:
            scales = torch.empty((nbc, nbr), dtype=torch.float32, device=x.device)
            rs, cs = 1, nbr
        else:
            scales = torch.empty((nbr, nbc), dtype=torch.float32, device=x.device)
            rs, cs = nbc, 1
    ld = x.stride(0) if rows > 1 else max(cols, 1)          # the stride of a single row is arbitrary
    check(load_library().qgemm_quantize(_dt(x), _dt(q, True), mode, x.data_ptr(), ld, rows, cols, q.data_ptr(),
                                        cols, scales.data_ptr(), rs, cs, _stream()))
    return q, scales
