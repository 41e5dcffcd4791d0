"""Quantisers on the GPU (through the C ABI) against the CPU oracle: scales and quantised bytes
bit for bit (x / s is a true division and the rounding is to nearest even on both sides)."""
import numpy as np
import pytest
import torch

import qgemm_amd as Q
from oracle import cpu_ref as R
from tests.util import assert_close, dev, host, say

pytestmark = pytest.mark.gpu


def _u8(t):
    torch.cuda.synchronize()
    return t.view(torch.uint8).cpu().numpy()


@pytest.mark.parametrize("shape", [(64, 256), (100, 300), (1, 5), (513, 1027), (2048, 4096)])
def test_per_matrix_int8_and_fp8_bit_exact(shape):
    say("quantize per-matrix", shape)
    x = R.fill_normal(shape, 7)
    qi, si = R.quantize_int8(x)
    g, s = Q.quantize(dev(x), torch.int8, Q.QUANT_PER_MATRIX)
    assert host(s)[0] == si
    assert np.array_equal(host(g), qi)
    qf, sf = R.quantize_fp8(x)
    g, s = Q.quantize(dev(x), torch.float8_e4m3fn, Q.QUANT_PER_MATRIX)
    assert host(s)[0] == sf
    assert np.array_equal(_u8(g), qf)


def test_fp8_encode_every_rounding_case():
    """All of e4m3's grid points, their midpoints and neighbours, overflow, infinities, NaN and
    subnormals go through the quantiser with s = 1 (the matrix maximum is made 448)."""
    say("quantize fp8 special values")
    grid = R.decode_fp8(np.arange(256, dtype=np.uint8)).astype(np.float64)
    grid = np.sort(grid[np.isfinite(grid)])
    mids = (grid[1:] + grid[:-1]) / 2
    vals = np.concatenate([grid, mids, np.nextafter(mids.astype(np.float32), np.float32(np.inf)),
                           np.nextafter(mids.astype(np.float32), np.float32(-np.inf)),
                           [0.0, -0.0, 447.9, 448.0, 2.0 ** -10, 2.0 ** -9, 3 * 2.0 ** -10, 1e-30, np.nan]])
    vals = vals.astype(np.float32)
    vals = np.concatenate([vals, np.full(7, 448.0, np.float32)])[None, :]      # amax = 448 exactly -> s = 1
    q, s = R.quantize_fp8(vals)
    assert s == 1.0
    g, gs = Q.quantize(dev(vals), torch.float8_e4m3fn, Q.QUANT_PER_MATRIX)
    assert host(gs)[0] == 1.0
    assert np.array_equal(_u8(g), q)
    # block quantiser on values beyond the block maximum cannot happen; saturation is reached through inf
    big = np.array([[np.inf, 1.0, -np.inf, 3.0]], np.float32)
    qb, sb = R.quantize_fp8(big)
    g, gs = Q.quantize(dev(big), torch.float8_e4m3fn, Q.QUANT_PER_MATRIX)
    assert np.array_equal(host(gs).view(np.uint32), np.array([sb]).view(np.uint32))
    assert np.array_equal(_u8(g), qb)


@pytest.mark.parametrize("shape", [(32, 256), (100, 300), (3, 129), (256, 1024), (130, 260)])
def test_block_quantisers_bit_exact(shape):
    say("quantize blocks", shape)
    x = R.fill_normal(shape, 9) * np.float32(3.0)
    x[0, :] = 0.0                                            # an all-zero 1 x 128 block: s = 1
    for mode, br in ((Q.QUANT_BLOCK_1x128, 1), (Q.QUANT_BLOCK_128x128, 128)):
        q, s = R.quantize_fp8_block(x, br, 128)
        g, gs = Q.quantize(dev(x), torch.float8_e4m3fn, mode)
        assert np.array_equal(host(gs), s), mode
        assert np.array_equal(_u8(g), q), mode
        g2, gt = Q.quantize(dev(x), torch.float8_e4m3fn, mode, rows_contiguous_scales=True)
        assert np.array_equal(host(gt), s.T) and np.array_equal(_u8(g2), q)
    if shape[0] > 8:
        assert host(Q.quantize(dev(x), torch.float8_e4m3fn, Q.QUANT_BLOCK_1x128)[1])[0, 0] == 1.0


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_16_bit_inputs_and_row_stride(dt):
    say("quantize 16-bit input", dt)
    base = torch.from_numpy(R.fill_normal((96, 400), 21)).to(dt).cuda()
    x = base[:, 8:392]                                       # row stride 400, 384 columns, 16-byte aligned start
    xf = x.float().cpu().numpy()
    q, s = R.quantize_fp8_block(xf, 1, 128)
    g, gs = Q.quantize(x, torch.float8_e4m3fn, Q.QUANT_BLOCK_1x128)
    assert np.array_equal(host(gs), s) and np.array_equal(_u8(g), q)
    y = base[:, 3:390]                                       # misaligned start, ragged width: scalar path
    yf = y.float().cpu().numpy()
    qi, si = R.quantize_int8(yf)
    g, gs = Q.quantize(y, torch.int8, Q.QUANT_PER_MATRIX)
    assert host(gs)[0] == si and np.array_equal(host(g), qi)


def test_errors_and_empty():
    say("quantize errors")
    x = torch.zeros((16, 128), device="cuda")
    with pytest.raises(Q.QgemmError) as e:                   # the output is int8 or e4m3
        Q.quantize(x, torch.int32, Q.QUANT_BLOCK_1x128)
    assert e.value.status == 2
    q, s = Q.quantize(x, torch.float8_e4m3fn, Q.QUANT_PER_MATRIX)      # all zeros: s = 1
    assert host(s)[0] == 1.0 and not _u8(q).any()
    q, s = Q.quantize(torch.zeros((0, 128), device="cuda"), torch.int8, Q.QUANT_PER_MATRIX)
    assert host(s)[0] == 1.0


def test_quantise_then_multiply_block_scaled():
    """The whole path on the GPU: 1 x 128 quantiser for A (scales written rows-contiguous, the form the
    kernel consumes), 128 x 128 for B, block-scaled GEMM; against the oracle doing the same on the CPU."""
    M, N, K = 256, 384, 1024
    say("quantize + block-scaled GEMM", (M, N, K))
    a = R.fill_normal((M, K), 31)
    b = R.fill_normal((N, K), 32)
    qa, sa = R.quantize_fp8_block(a, 1, 128)
    qb, sb = R.quantize_fp8_block(b, 128, 128)
    ref = R.gemm_fp8_block(R.decode_fp8(qa), R.decode_fp8(qb), sa, sb)
    ga, gsa = Q.quantize(dev(a), torch.float8_e4m3fn, Q.QUANT_BLOCK_1x128)
    gb, gsb = Q.quantize(dev(b), torch.float8_e4m3fn, Q.QUANT_BLOCK_128x128)
    c = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    Q.scaled_gemm(ga, gb, gsa, gsb, c, M, N, K, Q.SCALE_BLOCK128)
    assert_close(host(c), ref, what=Q.last_config())
    # the result only differs from a GEMM on the unquantised operands by the quantisation error
    exact = a.astype(np.float64) @ b.astype(np.float64).T
    assert np.abs(host(c) - exact).max() < 0.06 * np.abs(exact).max()


def test_division_by_the_scale_is_the_ieee_division():
    """The quantisers divide every element of a block by one scale and share the reciprocal's refinement between
    the elements; the quotients have to be those of the IEEE division the oracle does, bit for bit after encoding.
    Random mantissas over twelve octaves below the block maximum (ties of the e4m3 and int8 rounding are hit
    through the sheer number: 4 M elements), blocks whose scale lies on both sides of the range the shared form
    covers (2^-60 .. 2^60) and far outside, elements that make quotients below 2^-100, signed zeros, infinities
    and NaNs of both signs."""
    rng = np.random.default_rng(1234)
    rows, cols = 2048, 2048
    mant = rng.integers(0, 1 << 23, (rows, cols), dtype=np.uint32)
    expo = rng.integers(115, 128, (rows, cols), dtype=np.uint32)          # 2^-12 .. 2^0
    sign = rng.integers(0, 2, (rows, cols), dtype=np.uint32) << 31
    x = (sign | (expo << 23) | mant).view(np.float32)
    # per row a magnitude: the scales of the 1 x 128 blocks then run from far below 2^-60 to far above 2^60
    row_exp = np.linspace(-100, 100, rows).round().astype(np.int32)
    x = np.ldexp(x, row_exp[:, None]).astype(np.float32)
    # specials sprinkled in: tiny elements (quotient < 2^-100), signed zeros, infinities, NaNs
    x[:, 5] = np.ldexp(np.float32(1.5), row_exp - 120).astype(np.float32)
    x[:, 6] = -x[:, 5]
    x[:, 130] = 0.0
    x[:, 131] = -0.0
    x[::7, 300] = np.inf
    x[::11, 301] = -np.inf
    x[::5, 400] = np.nan
    x[::9, 401] = np.float32(-np.nan)
    say("quantize: division by the shared scale", x.shape)
    for mode, br in ((Q.QUANT_BLOCK_1x128, 1), (Q.QUANT_BLOCK_128x128, 128)):
        q, s = R.quantize_fp8_block(x, br, 128)
        g, gs = Q.quantize(dev(x), torch.float8_e4m3fn, mode)
        assert np.array_equal(host(gs).view(np.uint32), s.view(np.uint32)), mode
        assert np.array_equal(_u8(g), q), mode
    # per matrix: one scale for everything; slices of rows keep the scale inside and outside the range
    for lo, hi in ((0, 64), (1000, 1064), (2000, 2048), (400, 420)):
        part = np.ascontiguousarray(x[lo:hi])
        part = np.where(np.isfinite(part), part, np.float32(0)).astype(np.float32) if lo != 1000 else part
        q, s = R.quantize_fp8(part)
        g, gs = Q.quantize(dev(part), torch.float8_e4m3fn, Q.QUANT_PER_MATRIX)
        assert host(gs).view(np.uint32)[0] == np.array([s], np.float32).view(np.uint32)[0]
        assert np.array_equal(_u8(g), q), (lo, hi)
        part = np.where(np.isfinite(part), part, np.float32(0)).astype(np.float32)
        qi, si = R.quantize_int8(part)
        gi, gsi = Q.quantize(dev(part), torch.int8, Q.QUANT_PER_MATRIX)
        assert host(gsi).view(np.uint32)[0] == np.array([si], np.float32).view(np.uint32)[0]
        assert np.array_equal(host(gi), qi), (lo, hi)
