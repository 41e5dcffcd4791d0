"""qgemm_python, the torch-facing module (reference setup.py:73; fp8_mm of hip_mix_gemm_kernel.cpp:508-516):
loads on the CPU with its four functions; on the GPU each one gives the bits of the ctypes path (same
library entry, same kernel) and agrees with the CPU oracle to rtol 2e-2 / atol 1e-2 (int32 bit-exact)."""
import numpy as np
import pytest
import torch

import qgemm_amd as Q
from oracle import cpu_ref as R

RTOL, ATOL = 2e-2, 1e-2


def test_module_loads_and_exports():
    mod = Q.load_torch_extension()
    for name in ("fp8_mm", "fp8_mm_per_matrix", "int8_mm", "bf16_mm"):
        assert callable(getattr(mod, name))
    # host tensors are refused before anything touches a device
    t = torch.zeros(2, 2)
    with pytest.raises(RuntimeError, match="device tensor"):
        mod.bf16_mm(t, t, t)


def _dev(x):
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def _close(got, ref):
    return np.all(np.abs(got - ref) <= ATOL + RTOL * np.abs(ref) + 1e-5 * np.abs(ref).max())


@pytest.mark.gpu
def test_fp8_mm_reference_layout():
    mod = Q.load_torch_extension()
    m, n, k = 256, 512, 1024
    a = R.fill_normal((m, k), 11)
    b = R.fill_normal((n, k), 12)
    qa, sa = R.quantize_fp8_block(a, 1, 128)          # [m, k/128]
    qb, sb = R.quantize_fp8_block(b, 128, 128)        # [n/128, k/128]
    ref = R.gemm_fp8_block(R.decode_fp8(qa), R.decode_fp8(qb), sa, sb)
    # reference layout: a [m, k] column-major, b [n, k] column-major, scales column-major
    a_t = _dev(qa.T).view(torch.float8_e4m3fn).t()     # shape [m, k], strides (1, m)
    b_t = _dev(qb.T).view(torch.float8_e4m3fn).t()
    as_t = _dev(sa.T).t()
    bs_t = _dev(sb.T).t()
    c = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    mod.fp8_mm(a_t, b_t, as_t, bs_t, c)
    c2 = torch.zeros_like(c)
    Q.fp8_mm(a_t, b_t, as_t, bs_t, c2)
    torch.cuda.synchronize()
    assert torch.equal(c, c2)
    assert _close(c.float().cpu().numpy(), ref)
    # the reference's dispatch contract: dimensions divisible by 32 or it throws (hip_mix_gemm_kernel.cpp:460,485,503)
    with pytest.raises(RuntimeError):
        mod.fp8_mm(a_t[:100], b_t, as_t[:100], bs_t, c[:100])


@pytest.mark.gpu
def test_int8_fp8_per_matrix_and_bf16():
    mod = Q.load_torch_extension()
    m, n, k = 192, 320, 512
    scalar = lambda v: _dev(np.array([v], np.float32))
    qa, sa = R.quantize_int8(R.fill_normal((m, k), 21))
    qb, sb = R.quantize_int8(R.fill_normal((n, k), 22))
    ci = torch.zeros((m, n), dtype=torch.int32, device="cuda")
    mod.int8_mm(_dev(qa), _dev(qb), scalar(sa), scalar(sb), ci)
    cf = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    mod.int8_mm(_dev(qa), _dev(qb), scalar(sa), scalar(sb), cf)
    torch.cuda.synchronize()
    acc = R.gemm_i8_i32(qa, qb)
    assert np.array_equal(ci.cpu().numpy(), acc)
    assert _close(cf.cpu().numpy(), acc.astype(np.float32) * np.float32(sa * sb))

    fa, ta = R.quantize_fp8(R.fill_normal((m, k), 23))
    fb, tb = R.quantize_fp8(R.fill_normal((n, k), 24))
    cb = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    mod.fp8_mm_per_matrix(_dev(fa).view(torch.float8_e4m3fn), _dev(fb).view(torch.float8_e4m3fn), scalar(ta), scalar(tb), cb)
    torch.cuda.synchronize()
    ref = R.gemm_f32acc(R.decode_fp8(fa), R.decode_fp8(fb)) * np.float32(ta * tb)
    assert _close(cb.float().cpu().numpy(), ref)

    # a side stream is honoured: the module launches on torch's current stream
    x = torch.randn(m, k, device="cuda").bfloat16()
    y = torch.randn(n, k, device="cuda").bfloat16()
    out = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        mod.bf16_mm(x, y, out)
    side.synchronize()
    ref = x.float().cpu().numpy() @ y.float().cpu().numpy().T
    assert _close(out.float().cpu().numpy(), ref)
