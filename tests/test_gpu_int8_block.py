"""int8 operands with 128-block scales: the int8 twin of the reference's FP8_GEMM_kernel arithmetic
(hip_mix_gemm_kernel.cpp:231-244; the reference's own int8 path is a stub, src/gemm/sm80_gemm_kernel.cu:14-22).  The
partial product of a 128-wide K block is an exact int32, converted to fp32 once and folded in with
a_scale[m, kb] * b_scale[n / 128, kb].  Power-of-two scales keep every step exact (partials below 2^24), so every row
of the variant table has to give the oracle's bits; random scales to the stated tolerance; both storages; a partial
last K block; the block quantiser for int8; config 4's shape."""
import numpy as np
import pytest
import torch

import qgemm_amd as Q
from oracle import cpu_ref as R
from tests.util import assert_close, dev, host, say

pytestmark = pytest.mark.gpu
ROWS = Q.variant_names(Q.DT_I8, Q.SCALE_BLOCK128)


@pytest.fixture(autouse=True)
def _reset_options():
    yield
    Q.force_config(None)
    for k, v in (("force_split", 0), ("kmajor", 1)):
        Q.set_option(k, v)


def _call(qa, qb, as_, bs, c, M, N, K, layout=Q.LAYOUT_K_CONTIGUOUS, split=0):
    return Q.scaled_gemm(dev(qa), dev(qb), dev(as_), dev(bs), c, M, N, K, Q.SCALE_BLOCK128, layout=layout, split_k=split,
                         in_dtype=Q.DT_I8)


@pytest.mark.parametrize("variant", [None] + ROWS)
def test_power_of_two_scales_bit_exact_every_row(variant):
    rng = np.random.default_rng(11)
    for (M, N, K) in ((272, 392, 768), (64, 256, 1200), (300, 200, 160)):       # (the last two: a partial last K block)
        KB = (K + 127) // 128
        for split in ((1, 2) if KB >= 6 else (1,)):
            say("int8 block pow2", (M, N, K), variant, "split", split)
            Q.force_config(variant)
            Q.set_option("force_split", split)
            # small integers and power-of-two scales: every term and every partial sum is exact in fp32 in any order
            # (the rows with K groups, the skinny-M kernel and a K split add the blocks in other orders than the oracle)
            qa = rng.integers(-3, 4, size=(M, K)).astype(np.int8)
            qb = rng.integers(-3, 4, size=(N, K)).astype(np.int8)
            as_ = (2.0 ** rng.integers(-3, 4, size=(M, KB))).astype(np.float32)
            bs = (2.0 ** rng.integers(-3, 4, size=((N + 127) // 128, KB))).astype(np.float32)
            ref = R.gemm_i8_block(qa, qb, as_, bs)
            c = torch.full((M, N), -7.0, dtype=torch.float32, device="cuda")
            _call(qa, qb, as_, bs, c, M, N, K)
            assert "strided" not in Q.last_config()
            assert np.array_equal(host(c), ref), (Q.last_config(), (M, N, K), split)
            # the whole int8 range against unit scales: the exact int32 product (|sums| < 2^24 at these K)
            qa = rng.integers(-127, 128, size=(M, K)).astype(np.int8)
            qb = rng.integers(-127, 128, size=(N, K)).astype(np.int8)
            c.fill_(-7.0)
            _call(qa, qb, np.ones_like(as_), np.ones_like(bs), c, M, N, K)
            assert np.array_equal(host(c), R.gemm_i8_i32(qa, qb).astype(np.float32)), (Q.last_config(), (M, N, K), split)


@pytest.mark.parametrize("variant", [None, "256x256_w2x4_solo8", "128x128_w2x2_dma", "skinny_64x32_k8", "256x128_w2x2_cw", "128x128_w2x2_k2"])
def test_random_scales_tolerance_and_outputs(variant):
    M, N, K = 320, 384, 1024
    say("int8 block random", (M, N, K), variant)
    qa, _ = R.quantize_int8_block(R.fill_normal((M, K), 21), 1, 128)
    qb, _ = R.quantize_int8_block(R.fill_normal((N, K), 22), 128, 128)
    as_ = R.fill_uniform((M, K // 128), 23, 0.5, 2.0) / np.float32(127)
    bs = R.fill_uniform((N // 128, K // 128), 24, 0.5, 2.0) / np.float32(127)
    ref = R.gemm_i8_block(qa, qb, as_, bs)
    Q.force_config(variant)
    for dt in (torch.float32, torch.bfloat16, torch.float16):
        c = torch.zeros((M, N), dtype=dt, device="cuda")
        _call(qa, qb, as_, bs, c, M, N, K)
        # the kernels fold P * (as * bs), the oracle (P * as) * bs: one rounding of difference per block
        assert_close(host(c).astype(np.float32), ref, rtol=2e-2, atol=1e-2, what=f"{Q.last_config()} {dt}")
    c = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    Q.int8_mm_block(dev(qa), dev(qb), dev(as_), dev(bs), c)
    assert np.max(np.abs(host(c) - ref)) <= 2e-5 * np.max(np.abs(ref))


def test_reference_storage_and_any_shape():
    """A stored K x M, B K x N, scales K-block-major (the layout contract of fp8_mm, hip_mix_gemm_kernel.cpp:425-439):
    through the transposes; K not a multiple of 16: the any-shape kernel; same bits as the K-contiguous call."""
    rng = np.random.default_rng(12)
    for (M, N, K) in ((160, 224, 512), (96, 128, 200)):
        KB = (K + 127) // 128
        qa = rng.integers(-3, 4, size=(M, K)).astype(np.int8)
        qb = rng.integers(-3, 4, size=(N, K)).astype(np.int8)
        as_ = (2.0 ** rng.integers(-3, 4, size=(M, KB))).astype(np.float32)
        bs = (2.0 ** rng.integers(-3, 4, size=((N + 127) // 128, KB))).astype(np.float32)
        ref = R.gemm_i8_block(qa, qb, as_, bs)
        say("int8 block, reference storage", (M, N, K))
        c = torch.full((M, N), -7.0, dtype=torch.float32, device="cuda")
        if K % 32 == 0:
            Q.scaled_gemm(dev(np.ascontiguousarray(qa.T)), dev(np.ascontiguousarray(qb.T)), dev(np.ascontiguousarray(as_.T)),
                          dev(np.ascontiguousarray(bs.T)), c, M, N, K, Q.SCALE_BLOCK128, layout=Q.LAYOUT_REFERENCE, in_dtype=Q.DT_I8)
            assert np.array_equal(host(c), ref), Q.last_config()
        c.fill_(-7.0)
        _call(qa, qb, as_, bs, c, M, N, K)
        assert (Q.last_config() == "strided_any_shape") == (K % 16 != 0)
        assert np.array_equal(host(c), ref), Q.last_config()
    with pytest.raises(Q.QgemmError) as e:               # there is no int32 sum of scaled blocks
        _call(qa, qb, as_, bs, torch.zeros((M, N), dtype=torch.int32, device="cuda"), M, N, K)
    assert e.value.status == 2


@pytest.mark.parametrize("shape", [(64, 256), (130, 300), (256, 1024)])
def test_block_quantiser_int8_bit_exact(shape):
    say("int8 block quantiser", shape)
    x = R.fill_normal(shape, 31) * np.float32(3.0)
    for mode, br in ((Q.QUANT_BLOCK_1x128, 1), (Q.QUANT_BLOCK_128x128, 128)):
        q, s = R.quantize_int8_block(x, br, 128)
        g, gs = Q.quantize(dev(x), torch.int8, mode)
        assert np.array_equal(host(gs), s), mode
        assert np.array_equal(host(g), q), mode


def test_quantise_then_multiply_config4_shape():
    """fp32 operands -> int8 with 1 x 128 / 128 x 128 block scales on the GPU -> block-scaled GEMM at config 4's shape, bf16
    out: oracle on 12 full rows and the columns of one 128-block, and every scale doubled doubles... every output x 4."""
    M, N, K = 6144, 4608, 7168
    say("int8 block, config 4 shape")
    a, b = R.fill_normal((M, K), 41), R.fill_normal((N, K), 42)
    ga, gsa = Q.quantize(dev(a), torch.int8, Q.QUANT_BLOCK_1x128)
    gb, gsb = Q.quantize(dev(b), torch.int8, Q.QUANT_BLOCK_128x128)
    qa, sa = R.quantize_int8_block(a, 1, 128)
    qb, sb = R.quantize_int8_block(b, 128, 128)
    assert np.array_equal(host(ga), qa) and np.array_equal(host(gsa), sa)
    assert np.array_equal(host(gb), qb) and np.array_equal(host(gsb), sb)
    c = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    Q.scaled_gemm(ga, gb, gsa, gsb, c, M, N, K, Q.SCALE_BLOCK128, in_dtype=Q.DT_I8)
    name = Q.last_config()
    assert name.startswith("256x256_w2x4_solo8"), name
    got = host(c)
    rows = np.sort(np.random.default_rng(5).choice(M, 12, replace=False))
    assert_close(got[rows], R.gemm_i8_block(qa[rows], qb, sa[rows], sb), what=name)
    nb = 20
    sel = np.arange(nb * 128, nb * 128 + 128, 11)
    assert_close(got[:, sel], R.gemm_i8_block(qa, qb[sel], sa, sb[nb:nb + 1]), what=name + " cols")
    # against the product of the unquantised operands: the quantisation error of int8 with block scales
    full = a[rows].astype(np.float64) @ b.astype(np.float64).T
    assert np.max(np.abs(got[rows] - full)) <= 0.05 * np.sqrt(K)
    c2 = torch.zeros_like(c)
    Q.scaled_gemm(ga, gb, gsa * 2, gsb * 2, c2, M, N, K, Q.SCALE_BLOCK128, in_dtype=Q.DT_I8)
    assert torch.equal(c2.float(), 4 * c.float())
