"""ctypes front end of the CPU oracle (oracle/cpu_ref.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  The product package never imports this module.

All arrays are numpy, C-contiguous.  Layout strings:
  "nt"  A[m,k] row-major, B[n,k] row-major        (both K-contiguous)
  "nn"  A[m,k] row-major, B[k,n] row-major
  "tn"  A stored [k,m] (M-contiguous), B[k,n]      (fp8_mm's contract,
        hip_mix_gemm_kernel.cpp:96,111)
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# QGEMM_ORACLE_LIB names another build of the same source (the sanitizer build of `make -C oracle asan`)
_LIB_PATH = os.environ.get("QGEMM_ORACLE_LIB") or os.path.join(_HERE, "libcpu_ref.so")


def build(force=False):
    if os.environ.get("QGEMM_ORACLE_LIB"):
        return _LIB_PATH
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libcpu_ref.so"])
    return _LIB_PATH


def _load():
    build()
    lib = C.CDLL(_LIB_PATH)
    sz, f32, u64, vp = C.c_size_t, C.c_float, C.c_uint64, C.c_void_p
    sig = {
        "ref_num_threads": (C.c_int, []),
        "ref_set_num_threads": (None, [C.c_int]),
        "ref_fill_uniform": (None, [vp, sz, u64, f32, f32]),
        "ref_fill_normal": (None, [vp, sz, u64]),
        "ref_fill_pattern": (None, [vp, sz, C.c_int]),
        "ref_f32_to_bf16": (C.c_uint16, [f32]),
        "ref_bf16_to_f32": (f32, [C.c_uint16]),
        "ref_f32_to_f16": (C.c_uint16, [f32]),
        "ref_f16_to_f32": (f32, [C.c_uint16]),
        "ref_fp8_e4m3_to_f32": (f32, [C.c_uint8]),
        "ref_f32_to_fp8_e4m3": (C.c_uint8, [f32]),
        "ref_decode_fp8": (None, [vp, vp, sz]),
        "ref_encode_fp8": (None, [vp, vp, sz]),
        "ref_encode_bf16": (None, [vp, vp, sz]),
        "ref_decode_bf16": (None, [vp, vp, sz]),
        "ref_encode_f16": (None, [vp, vp, sz]),
        "ref_decode_f16": (None, [vp, vp, sz]),
        "ref_amax": (f32, [vp, sz]),
        "ref_quantize_int8": (f32, [vp, vp, sz]),
        "ref_quantize_fp8": (f32, [vp, vp, sz]),
        "ref_quantize_fp8_block": (None, [vp, vp, vp, sz, sz, sz, sz]),
        "ref_quantize_int8_block": (None, [vp, vp, vp, sz, sz, sz, sz]),
        "ref_transpose": (None, [vp, vp, sz, sz, sz]),
        "ref_gemm_i8_i32": (None, [vp, sz, sz, vp, sz, sz, vp, sz, sz, sz, sz]),
        "ref_scale_i32_to_f32": (None, [vp, vp, sz, f32, f32]),
        "ref_gemm_f32acc": (None, [vp, sz, sz, vp, sz, sz, vp, sz, sz, sz, sz]),
        "ref_gemm_f64acc": (None, [vp, sz, sz, vp, sz, sz, vp, sz, sz, sz, sz]),
        "ref_gemm_fp8_block": (None, [vp, sz, sz, vp, sz, sz, vp, sz, sz, vp, sz, sz, vp, sz, sz, sz, sz, sz]),
        "ref_gemm_i8_block": (None, [vp, sz, sz, vp, sz, sz, vp, sz, sz, vp, sz, sz, vp, sz, sz, sz, sz]),
        "ref_gemm_fp8_block_f64": (None, [vp, sz, sz, vp, sz, sz, vp, sz, sz, vp, sz, sz, vp, sz, sz, sz, sz]),
        "ref_select_tile": (sz, [sz, C.c_int]),
        "ref_block_swizzle": (None, [sz, sz, sz, sz, C.POINTER(sz), C.POINTER(sz)]),
        "ref_max_abs_diff": (C.c_double, [vp, vp, sz]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    return lib


lib = _load()


def _p(a):
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be C-contiguous"
    return a.ctypes.data


def num_threads():
    return lib.ref_num_threads()


def set_num_threads(n):
    lib.ref_set_num_threads(int(n))


# ---------------------------------------------------------------- inputs
def fill_uniform(shape, seed, lo=-1.0, hi=1.0):
    out = np.empty(shape, np.float32)
    lib.ref_fill_uniform(_p(out), out.size, seed, lo, hi)
    return out


def fill_normal(shape, seed):
    out = np.empty(shape, np.float32)
    lib.ref_fill_normal(_p(out), out.size, seed)
    return out


def fill_pattern(shape, which):
    out = np.empty(shape, np.float32)
    lib.ref_fill_pattern(_p(out), out.size, int(which))
    return out


# ---------------------------------------------------------------- codecs
def encode_fp8(x):
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(x.shape, np.uint8)
    lib.ref_encode_fp8(_p(x), _p(out), x.size)
    return out


def decode_fp8(q):
    q = np.ascontiguousarray(q, np.uint8)
    out = np.empty(q.shape, np.float32)
    lib.ref_decode_fp8(_p(q), _p(out), q.size)
    return out


def encode_bf16(x):
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib.ref_encode_bf16(_p(x), _p(out), x.size)
    return out


def decode_bf16(h):
    h = np.ascontiguousarray(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib.ref_decode_bf16(_p(h), _p(out), h.size)
    return out


def encode_f16(x):
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib.ref_encode_f16(_p(x), _p(out), x.size)
    return out


def decode_f16(h):
    h = np.ascontiguousarray(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib.ref_decode_f16(_p(h), _p(out), h.size)
    return out


# ------------------------------------------------------------ quantisers
def amax(x):
    x = np.ascontiguousarray(x, np.float32)
    return float(lib.ref_amax(_p(x), x.size))


def quantize_int8(x):
    x = np.ascontiguousarray(x, np.float32)
    q = np.empty(x.shape, np.int8)
    s = lib.ref_quantize_int8(_p(x), _p(q), x.size)
    return q, np.float32(s)


def quantize_fp8(x):
    x = np.ascontiguousarray(x, np.float32)
    q = np.empty(x.shape, np.uint8)
    s = lib.ref_quantize_fp8(_p(x), _p(q), x.size)
    return q, np.float32(s)


def quantize_fp8_block(x, br, bc):
    x = np.ascontiguousarray(x, np.float32)
    rows, cols = x.shape
    q = np.empty(x.shape, np.uint8)
    s = np.empty(((rows + br - 1) // br, (cols + bc - 1) // bc), np.float32)
    lib.ref_quantize_fp8_block(_p(x), _p(q), _p(s), rows, cols, br, bc)
    return q, s


def quantize_int8_block(x, br, bc):
    x = np.ascontiguousarray(x, np.float32)
    rows, cols = x.shape
    q = np.empty(x.shape, np.int8)
    s = np.empty(((rows + br - 1) // br, (cols + bc - 1) // bc), np.float32)
    lib.ref_quantize_int8_block(_p(x), _p(q), _p(s), rows, cols, br, bc)
    return q, s


# -------------------------------------------------------------- transpose
def transpose(a):
    a = np.ascontiguousarray(a)
    M, N = a.shape
    out = np.empty((N, M), a.dtype)
    lib.ref_transpose(_p(a), _p(out), M, N, a.dtype.itemsize)
    return out


# ------------------------------------------------------------------ GEMMs
def _strides(layout, A, B):
    """-> (M, N, K, a_rs, a_cs, b_ns, b_ks) in elements."""
    if layout == "nt":
        (M, K), (N, K2) = A.shape, B.shape
        s = (K, 1, K, 1)
    elif layout == "nn":
        (M, K), (K2, N) = A.shape, B.shape
        s = (K, 1, 1, N)
    elif layout == "tn":
        (K, M), (K2, N) = A.shape, B.shape
        s = (1, M, 1, N)
    else:
        raise ValueError(layout)
    assert K == K2, "inner dimensions differ"
    return (M, N, K) + s


def gemm_i8_i32(A, B, layout="nt"):
    A = np.ascontiguousarray(A, np.int8)
    B = np.ascontiguousarray(B, np.int8)
    M, N, K, ars, acs, bns, bks = _strides(layout, A, B)
    Cm = np.empty((M, N), np.int32)
    lib.ref_gemm_i8_i32(_p(A), ars, acs, _p(B), bns, bks, _p(Cm), N, M, N, K)
    return Cm


def scale_i32_to_f32(acc, sa, sb):
    acc = np.ascontiguousarray(acc, np.int32)
    out = np.empty(acc.shape, np.float32)
    lib.ref_scale_i32_to_f32(_p(acc), _p(out), acc.size, float(sa), float(sb))
    return out


def gemm_f32acc(A, B, layout="nt"):
    A = np.ascontiguousarray(A, np.float32)
    B = np.ascontiguousarray(B, np.float32)
    M, N, K, ars, acs, bns, bks = _strides(layout, A, B)
    Cm = np.empty((M, N), np.float32)
    lib.ref_gemm_f32acc(_p(A), ars, acs, _p(B), bns, bks, _p(Cm), N, M, N, K)
    return Cm


def gemm_f64acc(A, B, layout="nt"):
    A = np.ascontiguousarray(A, np.float32)
    B = np.ascontiguousarray(B, np.float32)
    M, N, K, ars, acs, bns, bks = _strides(layout, A, B)
    Cm = np.empty((M, N), np.float64)
    lib.ref_gemm_f64acc(_p(A), ars, acs, _p(B), bns, bks, _p(Cm), N, M, N, K)
    return Cm


def _scale_strides(scale_layout, as_, bs, M, N, K):
    kb = (K + 127) // 128
    nb = (N + 127) // 128
    if scale_layout == "row":      # as [M, K/128], bs [N/128, K/128], row-major
        assert as_.shape == (M, kb) and bs.shape == (nb, kb), (as_.shape, bs.shape)
        return (kb, 1, kb, 1)
    if scale_layout == "col":      # reference contract: as[m + kb*M], bs[nb + kb*ceil(N/128)]
        assert as_.shape == (kb, M) and bs.shape == (kb, nb), (as_.shape, bs.shape)
        return (1, M, 1, nb)
    raise ValueError(scale_layout)


def gemm_fp8_block(A, B, as_, bs, layout="nt", scale_layout="row", bk=None):
    """A, B: fp32 arrays holding decoded fp8 values.  Returns fp32 accumulators."""
    A = np.ascontiguousarray(A, np.float32)
    B = np.ascontiguousarray(B, np.float32)
    as_ = np.ascontiguousarray(as_, np.float32)
    bs = np.ascontiguousarray(bs, np.float32)
    M, N, K, ars, acs, bns, bks = _strides(layout, A, B)
    sms, sks, tns, tks = _scale_strides(scale_layout, as_, bs, M, N, K)
    if bk is None:
        bk = lib.ref_select_tile(K, 2) or 128
    Cm = np.empty((M, N), np.float32)
    lib.ref_gemm_fp8_block(_p(A), ars, acs, _p(B), bns, bks, _p(as_), sms, sks, _p(bs), tns, tks,
                           _p(Cm), N, M, N, K, bk)
    return Cm


def gemm_i8_block(A, B, as_, bs, layout="nt", scale_layout="row"):
    """A, B: int8.  Exact int32 partial per 128-wide K block, folded in fp32 like gemm_fp8_block.  Returns fp32."""
    A = np.ascontiguousarray(A, np.int8)
    B = np.ascontiguousarray(B, np.int8)
    as_ = np.ascontiguousarray(as_, np.float32)
    bs = np.ascontiguousarray(bs, np.float32)
    M, N, K, ars, acs, bns, bks = _strides(layout, A, B)
    sms, sks, tns, tks = _scale_strides(scale_layout, as_, bs, M, N, K)
    Cm = np.empty((M, N), np.float32)
    lib.ref_gemm_i8_block(_p(A), ars, acs, _p(B), bns, bks, _p(as_), sms, sks, _p(bs), tns, tks, _p(Cm), N, M, N, K)
    return Cm


def gemm_fp8_block_f64(A, B, as_, bs, layout="nt", scale_layout="row"):
    A = np.ascontiguousarray(A, np.float32)
    B = np.ascontiguousarray(B, np.float32)
    as_ = np.ascontiguousarray(as_, np.float32)
    bs = np.ascontiguousarray(bs, np.float32)
    M, N, K, ars, acs, bns, bks = _strides(layout, A, B)
    sms, sks, tns, tks = _scale_strides(scale_layout, as_, bs, M, N, K)
    Cm = np.empty((M, N), np.float64)
    lib.ref_gemm_fp8_block_f64(_p(A), ars, acs, _p(B), bns, bks, _p(as_), sms, sks, _p(bs), tns, tks,
                               _p(Cm), N, M, N, K)
    return Cm


def select_tile(dim, which):
    return int(lib.ref_select_tile(dim, {"m": 0, "n": 1, "k": 2}[which]))


def block_swizzle(bid, tiles_m, tiles_n, group):
    tm, tn = C.c_size_t(), C.c_size_t()
    lib.ref_block_swizzle(bid, tiles_m, tiles_n, group, C.byref(tm), C.byref(tn))
    return tm.value, tn.value


def max_abs_diff(c, ref):
    c = np.ascontiguousarray(c, np.float32)
    ref = np.ascontiguousarray(ref, np.float32)
    return float(lib.ref_max_abs_diff(_p(c), _p(ref), c.size))
