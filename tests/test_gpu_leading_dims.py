"""Leading dimensions on the MFMA path: ldC > N (the one stride the reference honours,
src/gemm/sm89_gemm_kernel_v3.cu:258), ldA > K and ldB > K, through every way a tile leaves the kernel
(16-byte row pieces from whole and from ragged tiles, element by element from an unaligned tile, the tiles without
LDS staging),
with and without a K split.  The padding columns of C and a guard row behind it are filled with a poison
value that has to survive."""
import numpy as np
import pytest
import torch

import qgemm_amd as Q
from oracle import cpu_ref as R
from tests.util import assert_close, dev, fp8_inputs, fp8_tensor, host, int8_inputs, say, scalar

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _reset_options():
    yield
    Q.set_option("force_config", -1)
    Q.set_option("force_split", 0)


def _padded_c(M, N, pad, dtype, poison):
    """-> (whole allocation [M + 1, N + pad] filled with poison, view [M, N] with row stride N + pad)"""
    whole = torch.full((M + 1, N + pad), poison, dtype=dtype, device="cuda")
    return whole, whole[:M, :N]


def _poison_intact(whole, M, N, poison):
    w = whole.cpu()
    return bool(torch.all(w[:M, N:] == poison)) and bool(torch.all(w[M] == poison))


# variant rows (gemm_inst.hip): 128x128 (staged epilogue), 256x256 4-wave solo, 8-wave solo, 128x32 and 16x32 (no LDS
# staging of C), 128x128 with two K groups, 256x128 with copying waves, 192x256 (8-wave solo)
EXITS = ["128x128_w2x2_dma", "256x256_w2x2_solo", "256x256_w2x4_solo8", "128x32_w4x1_dma", "16x32_w1x2_dma",
         "128x128_w2x2_k2", "256x128_w2x2_cw", "192x256_w2x4_solo8"]


@pytest.mark.parametrize("pad", [8, 5])
@pytest.mark.parametrize("variant", EXITS)
# whole wave tiles / ragged / ragged with rows that end on a 16-byte boundary (16-byte stores, rows and lanes left out)
@pytest.mark.parametrize("shape", [(256, 512, 256), (300, 333, 256), (300, 328, 256)])
@pytest.mark.parametrize("split", [1, 2])
def test_int8_padded_ldc(pad, variant, shape, split):
    M, N, K = shape
    say("ldC int8", shape, "pad", pad, "variant", variant, "split", split)
    qa, sa, qb, sb = int8_inputs(M, N, K, seed=900 + EXITS.index(variant))
    acc = R.gemm_i8_i32(qa, qb)
    Q.force_config(variant)
    for dt, ref, poison in ((torch.int32, acc, -77), (torch.float32, R.scale_i32_to_f32(acc, sa, sb), -77.0)):
        whole, c = _padded_c(M, N, pad, dt, poison)
        Q.int8_mm(dev(qa), dev(qb), scalar(sa), scalar(sb), c, split_k=split)
        assert np.array_equal(host(c), ref), Q.last_config()
        assert _poison_intact(whole, M, N, poison), Q.last_config()


@pytest.mark.parametrize("pad", [8, 5])
@pytest.mark.parametrize("variant", EXITS)
@pytest.mark.parametrize("shape", [(256, 512, 256), (300, 333, 256), (300, 328, 256)])
def test_fp8_bf16_out_padded_ldc(pad, variant, shape):
    M, N, K = shape
    say("ldC fp8 -> bf16", shape, "pad", pad, "variant", variant)
    qa, sa, qb, sb = fp8_inputs(M, N, K, seed=920 + EXITS.index(variant))
    ref = R.gemm_f32acc(R.decode_fp8(qa), R.decode_fp8(qb)) * np.float32(sa * sb)
    Q.force_config(variant)
    whole, c = _padded_c(M, N, pad, torch.bfloat16, -77.0)
    Q.scaled_gemm(fp8_tensor(qa), fp8_tensor(qb), scalar(sa), scalar(sb), c, M, N, K, Q.SCALE_PER_MATRIX, split_k=1)
    assert_close(host(c.contiguous()), ref, what=Q.last_config())
    assert _poison_intact(whole, M, N, -77.0), Q.last_config()
    # the same padded C must hold the bits of the dense call
    dense = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    Q.scaled_gemm(fp8_tensor(qa), fp8_tensor(qb), scalar(sa), scalar(sb), dense, M, N, K, Q.SCALE_PER_MATRIX, split_k=1)
    assert torch.equal(dense, c.contiguous())


@pytest.mark.parametrize("pad", [8, 5])
@pytest.mark.parametrize("variant", ["128x128_w2x2_dma", "256x256_w2x4_solo8", "128x32_w4x1_dma", "256x128_w2x2_cw",
                                     "192x256_w2x4_solo8"])
def test_fp8_block_scaled_padded_ldc(pad, variant):
    M, N, K = 256, 384, 512
    say("ldC fp8 block", "pad", pad, "variant", variant)
    qa, _, qb, _ = fp8_inputs(M, N, K, seed=940)
    as_ = R.fill_uniform((M, K // 128), 941, 0.5, 2.0) / np.float32(448)
    bs = R.fill_uniform((N // 128, K // 128), 942, 0.5, 2.0) / np.float32(448)
    ref = R.gemm_fp8_block(R.decode_fp8(qa), R.decode_fp8(qb), as_, bs)
    Q.force_config(variant)
    whole, c = _padded_c(M, N, pad, torch.bfloat16, -77.0)
    Q.scaled_gemm(fp8_tensor(qa), fp8_tensor(qb), dev(as_), dev(bs), c, M, N, K, Q.SCALE_BLOCK128, split_k=1)
    assert_close(host(c.contiguous()), ref, what=Q.last_config())
    assert _poison_intact(whole, M, N, -77.0), Q.last_config()


@pytest.mark.parametrize("variant", EXITS)
@pytest.mark.parametrize("pads", [(16, 16, 8), (32, 16, 5), (16, 48, 0)])
def test_bf16_padded_lda_ldb_ldc(variant, pads):
    """ldA = K + pa, ldB = K + pb (B stored N x K), ldC = N + pc; the padding of A and B holds large values that
    must never reach a sum; small integers so the result has to equal numpy's integer product bit for bit."""
    pa, pb, pc = pads
    M, N, K = 264, 392, 320
    say("ldA/ldB/ldC bf16", pads, "variant", variant)
    rng = np.random.default_rng(960 + EXITS.index(variant))
    a = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
    b = rng.integers(-4, 5, size=(N, K)).astype(np.float32)
    ref = (a.astype(np.int64) @ b.astype(np.int64).T).astype(np.float32)
    a_pad = torch.full((M, K + pa), 1000.0, dtype=torch.bfloat16, device="cuda")
    b_pad = torch.full((N, K + pb), 1000.0, dtype=torch.bfloat16, device="cuda")
    a_pad[:, :K] = torch.from_numpy(a).cuda().bfloat16()
    b_pad[:, :K] = torch.from_numpy(b).cuda().bfloat16()
    Q.force_config(variant)
    whole, c = _padded_c(M, N, pc, torch.float32, -77.0)
    Q.gemm(a_pad[:, :K], b_pad[:, :K], c, "nk")
    assert "strided" not in Q.last_config(), Q.last_config()
    assert np.array_equal(host(c), ref), Q.last_config()
    assert _poison_intact(whole, M, N, -77.0), Q.last_config()
