"""qgemm_scaled_gemm_static: the entry point that allocates nothing (static device scratch instead of the
library workspace), against qgemm_scaled_gemm on the same operands, bit for bit, two calls in a row with the
second one smaller."""
import ctypes as C

import numpy as np
import pytest
import torch

import qgemm_amd as Q
from oracle import cpu_ref as R
from qgemm_amd import lib as L
from tests.util import dev, fp8_inputs, fp8_tensor, int8_inputs, say, scalar

pytestmark = pytest.mark.gpu


def _memory_state():
    """(library workspace base, its size, free device memory): what a call that allocates would change."""
    base, size = C.c_void_p(), C.c_size_t()
    L.check(L.load_library().qgemm_workspace_info(C.byref(base), C.byref(size)))
    torch.cuda.synchronize()
    return base.value, size.value, torch.cuda.mem_get_info()[0]


def _call(static, in_dt, scale_mode, layout, a, b, sa, sb, c, M, N, K, split):
    lib = L.load_library()
    fn = lib.qgemm_scaled_gemm_static if static else lib.qgemm_scaled_gemm
    before = _memory_state() if static else None
    st = fn(in_dt, Q.ops._dt(c), scale_mode, layout, a.data_ptr(), b.data_ptr(), sa.data_ptr(), sb.data_ptr(),
            c.data_ptr(), c.stride(0), M, N, K, split, C.c_void_p(torch.cuda.current_stream().cuda_stream))
    if static:
        # the property in the entry's name: neither the library's workspace nor the device's free memory moved
        assert _memory_state() == before, (before, _memory_state())
    return st


def _int8_case(M, N, K, split, seed):
    qa, sa, qb, sb = int8_inputs(M, N, K, seed)
    a, b, s1, s2 = dev(qa), dev(qb), scalar(sa), scalar(sb)
    want = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    assert _call(False, Q.DT_I8, Q.SCALE_PER_MATRIX, Q.LAYOUT_K_CONTIGUOUS, a, b, s1, s2, want, M, N, K, split) == 0
    assert "splitk" in Q.last_config()
    got = torch.full((M, N), -5.0, dtype=torch.float32, device="cuda")
    assert _call(True, Q.DT_I8, Q.SCALE_PER_MATRIX, Q.LAYOUT_K_CONTIGUOUS, a, b, s1, s2, got, M, N, K, split) == 0
    assert "splitk" in Q.last_config()
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert np.array_equal(got.cpu().numpy(), R.scale_i32_to_f32(R.gemm_i8_i32(qa, qb), sa, sb))


def _block_case(M, N, K, seed, layout):
    """fp8 block scales: K-contiguous scales go through a transposed copy of a_scale in the scratch; the
    reference layout (with the K-major kernels switched off) through transposed copies of both operands."""
    qa, _, qb, _ = fp8_inputs(M, N, K, seed)
    as_ = R.fill_uniform((M, K // 128), seed + 2, 0.5, 2.0) / np.float32(448)
    bs = R.fill_uniform((N // 128, K // 128), seed + 3, 0.5, 2.0) / np.float32(448)
    if layout == Q.LAYOUT_REFERENCE:
        a, b = fp8_tensor(np.ascontiguousarray(qa.T)), fp8_tensor(np.ascontiguousarray(qb.T))
        sa, sb = dev(np.ascontiguousarray(as_.T)), dev(np.ascontiguousarray(bs.T))
    else:
        a, b, sa, sb = fp8_tensor(qa), fp8_tensor(qb), dev(as_), dev(bs)
    want = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    assert _call(False, Q.DT_F8E4M3, Q.SCALE_BLOCK128, layout, a, b, sa, sb, want, M, N, K, 0) == 0
    got = torch.full((M, N), -5.0, dtype=torch.bfloat16, device="cuda")
    assert _call(True, Q.DT_F8E4M3, Q.SCALE_BLOCK128, layout, a, b, sa, sb, got, M, N, K, 0) == 0
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    ref = R.gemm_fp8_block(R.decode_fp8(qa), R.decode_fp8(qb), as_, bs)
    err = np.abs(got.float().cpu().numpy() - ref)
    assert np.all(err <= 1e-2 + 2e-2 * np.abs(ref))


def test_static_scratch_entry_matches_the_allocating_one():
    say("no-alloc entry: int8 split-K, larger then smaller")
    _int8_case(128, 1024, 4096, 4, seed=601)          # 2 MiB of partial planes
    _int8_case(48, 200, 1024, 3, seed=603)            # smaller, ragged: the scratch still holds the first call's planes
    say("no-alloc entry: fp8 block scales, K-contiguous scales (transposed a_scale in the scratch)")
    _block_case(512, 384, 1024, seed=605, layout=Q.LAYOUT_K_CONTIGUOUS)
    _block_case(160, 128, 512, seed=609, layout=Q.LAYOUT_K_CONTIGUOUS)
    say("no-alloc entry: reference layout through the transposes")
    Q.set_option("kmajor", 0)
    try:
        _block_case(256, 384, 1024, seed=613, layout=Q.LAYOUT_REFERENCE)
        _block_case(64, 128, 256, seed=617, layout=Q.LAYOUT_REFERENCE)
    finally:
        Q.set_option("kmajor", 1)


def test_static_scratch_entry_refuses_what_does_not_fit():
    say("no-alloc entry: too large")
    M, N, K = 2048, 4096, 1024                         # 4 planes of 32 MiB > 32 MiB of scratch
    a = torch.zeros((M, K), dtype=torch.int8, device="cuda")
    b = torch.zeros((N, K), dtype=torch.int8, device="cuda")
    c = torch.full((M, N), 3, dtype=torch.int32, device="cuda")
    s = scalar(1)
    assert _call(True, Q.DT_I8, Q.SCALE_PER_MATRIX, Q.LAYOUT_K_CONTIGUOUS, a, b, s, s, c, M, N, K, 4) == 10
    torch.cuda.synchronize()
    assert bool(torch.all(c == 3))                     # nothing was launched
    assert b"static scratch" in L.load_library().qgemm_status_string(10)
    # the room for transposed operands counts too: reference layout through the transposes, A^T + B^T = 40 MiB
    say("no-alloc entry: too large, transposed operands")
    M, N, K = 4096, 6144, 4096
    a = torch.zeros((K, M), dtype=torch.uint8, device="cuda")
    b = torch.zeros((K, N), dtype=torch.uint8, device="cuda")
    sa = torch.ones((K // 128, M), dtype=torch.float32, device="cuda")
    sb = torch.ones((K // 128, N // 128), dtype=torch.float32, device="cuda")
    cb = torch.full((M, N), 3.0, dtype=torch.bfloat16, device="cuda")
    Q.set_option("kmajor", 0)
    try:
        assert _call(True, Q.DT_F8E4M3, Q.SCALE_BLOCK128, Q.LAYOUT_REFERENCE, a, b, sa, sb, cb, M, N, K, 1) == 10
    finally:
        Q.set_option("kmajor", 1)
    torch.cuda.synchronize()
    assert bool(torch.all(cb == 3.0))
    # ... and the room for a transposed a_scale: 131072 rows x 72 K blocks of floats = 36 MiB
    say("no-alloc entry: too large, transposed a_scale")
    M, N, K = 131072, 128, 72 * 128 + 128
    KB = K // 128                                      # 73: the row with copying waves fetches four K blocks a copy or wants a_scale rows-contiguous, through a copy
    a = torch.zeros((M, K), dtype=torch.uint8, device="cuda")
    b = torch.zeros((N, K), dtype=torch.uint8, device="cuda")
    sa = torch.ones((M, KB), dtype=torch.float32, device="cuda")
    sb = torch.ones((1, KB), dtype=torch.float32, device="cuda")
    cb = torch.full((M, N), 3.0, dtype=torch.bfloat16, device="cuda")
    Q.force_config("256x128_w2x2_cw")
    try:
        assert _call(True, Q.DT_F8E4M3, Q.SCALE_BLOCK128, Q.LAYOUT_K_CONTIGUOUS, a, b, sa, sb, cb, M, N, K, 1) == 10
    finally:
        Q.force_config(None)
    torch.cuda.synchronize()
    assert bool(torch.all(cb == 3.0))
