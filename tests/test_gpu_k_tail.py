"""K whose bytes are not a multiple of 128 (the unit of a K step) on the MFMA kernels.  The reference's dispatch keeps
every K % 32 == 0 on the matrix cores through its 64- and 32-wide K tiles (hip_mix_gemm_kernel.cpp:442-463); here the
last K step is partial and the lanes whose 16-byte chunk lies past the end of a row fetch zeros instead of the next
row's bytes.  Every row of every variant table, every place the partial step can fall in a pipeline (first copies, the
unrolled groups' hand-over, the last slice of a K split), ragged M and N, rows padded with values that must never
reach a sum.  Small integers (and power-of-two block scales) sum exactly, so the results have to equal the CPU
oracle bit for bit: one byte of the next row, or one missing chunk, cannot hide."""
import numpy as np
import pytest
import torch

import qgemm_amd as Q
from oracle import cpu_ref as R
from tests.util import assert_close, dev, fp8_inputs, fp8_tensor, host, int8_inputs, say, scalar

pytestmark = pytest.mark.gpu

I8_ROWS = Q.variant_names(Q.DT_I8, Q.SCALE_PER_MATRIX)
F8_ROWS = Q.variant_names(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX)
F8B_ROWS = Q.variant_names(Q.DT_F8E4M3, Q.SCALE_BLOCK128)
F8B_TN_ROWS = Q.variant_names(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 3)
BF16_ROWS = Q.variant_names(Q.DT_BF16)
BF16_NN_ROWS = Q.variant_names(Q.DT_BF16, 0, 2)
# K in bytes: one partial step; one whole and one partial; three steps; eight and nine steps (the partial step's copies
# issued in the first step behind an unrolled group of six); ten steps
KBYTES = (96, 160, 272, 1008, 1136, 1200)


@pytest.fixture(autouse=True)
def _reset_options():
    yield
    Q.force_config(None)
    for k, v in (("force_split", 0), ("kmajor", 1), ("k_rot", -1)):
        Q.set_option(k, v)


def _ints(rng, shape):
    return rng.integers(-3, 4, size=shape).astype(np.float32)


def _mfma(name):
    assert "strided" not in name, name


@pytest.mark.parametrize("variant", [None] + I8_ROWS)
def test_int8_every_row(variant):
    M, N = 300, 328
    for K in KBYTES:
        for split in ((1, 2) if K >= 1136 else (1,)):
            say("k tail int8", (M, N, K), variant, "split", split)
            Q.force_config(variant)
            Q.set_option("force_split", split)
            qa, sa, qb, sb = int8_inputs(M, N, K, seed=K + split)
            # rows of A and B padded to a multiple of 128 bytes with a value that would show in any sum
            a_pad = torch.full((M, K + 48), 99, dtype=torch.int8, device="cuda")
            b_pad = torch.full((N, K + 48), 99, dtype=torch.int8, device="cuda")
            a_pad[:, :K], b_pad[:, :K] = dev(qa), dev(qb)
            ref = R.gemm_i8_i32(qa, qb)
            c = torch.full((M, N), -7, dtype=torch.int32, device="cuda")
            Q.int8_mm(dev(qa), dev(qb), scalar(sa), scalar(sb), c)            # dense rows: the next row follows at once
            _mfma(Q.last_config())
            assert np.array_equal(host(c), ref), (Q.last_config(), K, split)
            c2 = torch.full((M, N), -7, dtype=torch.int32, device="cuda")
            L = Q.load_library()
            st = L.qgemm_gemm(Q.DT_I8, Q.DT_I32, 1, a_pad.data_ptr(), K + 48, b_pad.data_ptr(), K + 48, c2.data_ptr(), N, M, N, K,
                              None)
            assert st == 0
            _mfma(Q.last_config())
            assert np.array_equal(host(c2), ref), (Q.last_config(), K, split, "padded rows")


@pytest.mark.parametrize("variant", [None] + F8_ROWS)
def test_fp8_per_matrix_every_row(variant):
    M, N = 272, 392
    rng = np.random.default_rng(3)
    for K in KBYTES:
        say("k tail fp8", (M, N, K), variant)
        Q.force_config(variant)
        a, b = _ints(rng, (M, K)), _ints(rng, (N, K))
        ref = R.gemm_f32acc(a, b)
        for dt in (torch.float32, torch.bfloat16):
            c = torch.full((M, N), -7.0, dtype=dt, device="cuda")
            Q.scaled_gemm(fp8_tensor(R.encode_fp8(a)), fp8_tensor(R.encode_fp8(b)), scalar(1), scalar(1), c, M, N, K,
                          Q.SCALE_PER_MATRIX, split_k=1)
            _mfma(Q.last_config())
            want = ref if dt == torch.float32 else R.decode_bf16(R.encode_bf16(ref))
            assert np.array_equal(host(c), want), (Q.last_config(), K, dt)


@pytest.mark.parametrize("variant", [None] + F8B_ROWS)
def test_fp8_block_scales_every_row(variant):
    """The last 128-block of K is partial: its products are scaled with a_scale[m, K // 128] and b_scale[n // 128, K // 128]
    like those of a whole block.  Both arrangements of a_scale (an even and an odd number of K blocks per row: the
    kernels' twins for K-contiguous scales and the copy into the rows-contiguous order)."""
    M, N = 300, 392
    rng = np.random.default_rng(4)
    for K in KBYTES + (1456,):
        KB = (K + 127) // 128
        for split in ((1, 2) if KB >= 9 else (1,)):
            say("k tail fp8 block", (M, N, K), variant, "split", split)
            Q.force_config(variant)
            Q.set_option("force_split", split)
            a, b = _ints(rng, (M, K)), _ints(rng, (N, K))
            as_ = (2.0 ** rng.integers(-3, 4, size=(M, KB))).astype(np.float32)
            bs = (2.0 ** rng.integers(-3, 4, size=((N + 127) // 128, KB))).astype(np.float32)
            ref = R.gemm_fp8_block(a, b, as_, bs)
            c = torch.full((M, N), -7.0, dtype=torch.float32, device="cuda")
            Q.scaled_gemm(fp8_tensor(R.encode_fp8(a)), fp8_tensor(R.encode_fp8(b)), dev(as_), dev(bs), c, M, N, K,
                          Q.SCALE_BLOCK128)
            _mfma(Q.last_config())
            assert np.array_equal(host(c), ref), (Q.last_config(), K, split)


@pytest.mark.parametrize("variant", [None] + F8B_TN_ROWS)
def test_fp8_mm_reference_storage(variant):
    """fp8_mm's own storage (A is K x M, B is K x N): K % 32 == 0 is all the reference asks for.  As stored (the k rows
    past the end of K lie past the end of the buffer range) and through the transposes."""
    M, N = 288, 352
    rng = np.random.default_rng(5)
    for K in (96, 160, 288, 1184):
        KB = (K + 127) // 128
        a, b = _ints(rng, (M, K)), _ints(rng, (N, K))
        as_ = (2.0 ** rng.integers(-3, 4, size=(M, KB))).astype(np.float32)
        bs = (2.0 ** rng.integers(-3, 4, size=((N + 127) // 128, KB))).astype(np.float32)
        ref = R.gemm_fp8_block(a, b, as_, bs)
        a_t = fp8_tensor(np.ascontiguousarray(R.encode_fp8(a).T)).t()
        b_t = fp8_tensor(np.ascontiguousarray(R.encode_fp8(b).T)).t()
        as_t, bs_t = dev(np.ascontiguousarray(as_.T)).t(), dev(np.ascontiguousarray(bs.T)).t()
        for kmajor in (2, 0):
            say("k tail fp8_mm", (M, N, K), variant, "kmajor", kmajor)
            Q.force_config(variant)
            Q.set_option("kmajor", kmajor)
            c = torch.full((M, N), -7.0, dtype=torch.float32, device="cuda")
            Q.fp8_mm(a_t, b_t, as_t, bs_t, c)
            _mfma(Q.last_config())
            assert ("_tn" in Q.last_config()) == (kmajor == 2), Q.last_config()
            assert np.array_equal(host(c), ref), (Q.last_config(), K)


@pytest.mark.parametrize("variant", [None] + BF16_ROWS)
def test_bf16_every_row(variant):
    M, N = 264, 392
    rng = np.random.default_rng(6)
    for K in (8, 72, 136, 504, 568, 1000):              # 16, 144, 272, 1008, 1136, 2000 bytes
        say("k tail bf16", (M, N, K), variant)
        Q.force_config(variant)
        a, b = _ints(rng, (M, K)), _ints(rng, (N, K))
        ref = (a.astype(np.int64) @ b.astype(np.int64).T).astype(np.float32)
        a_pad = torch.full((M, K + 24), 1000.0, dtype=torch.bfloat16, device="cuda")       # the next 48 bytes of a row: poison
        b_pad = torch.full((N, K + 8), 1000.0, dtype=torch.bfloat16, device="cuda")
        a_pad[:, :K] = torch.from_numpy(a).cuda().bfloat16()
        b_pad[:, :K] = torch.from_numpy(b).cuda().bfloat16()
        c = torch.full((M, N), -7.0, dtype=torch.float32, device="cuda")
        Q.gemm(a_pad[:, :K], b_pad[:, :K], c, "nk")
        _mfma(Q.last_config())
        assert np.array_equal(host(c), ref), (Q.last_config(), K)


@pytest.mark.parametrize("variant", [None] + BF16_NN_ROWS)
def test_bf16_b_stored_k_by_n(variant):
    """GEMM_kernel_v1..v5 storage with a partial last K step: A K-contiguous (chunks past the end of a row zeroed), B
    K x N as stored (k rows past the end out of range)."""
    M, N = 200, 264
    rng = np.random.default_rng(7)
    for K in (72, 200, 1000):
        for kmajor in (2, 0):
            say("k tail bf16 kn", (M, N, K), variant, "kmajor", kmajor)
            Q.force_config(variant)
            Q.set_option("kmajor", kmajor)
            a, b = _ints(rng, (M, K)), _ints(rng, (K, N))
            ref = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
            c = torch.full((M, N), -7.0, dtype=torch.float32, device="cuda")
            Q.gemm(torch.from_numpy(a).cuda().bfloat16(), torch.from_numpy(b).cuda().bfloat16(), c, "kn")
            _mfma(Q.last_config())
            assert ("_nn" in Q.last_config()) == (kmajor == 2), Q.last_config()
            assert np.array_equal(host(c), ref), (Q.last_config(), K)


def test_values_next_to_the_tail_never_count():
    """Random fp8 data (tolerance against the oracle) with NaN codes in the bytes that follow every row: a K-contiguous
    operand whose rows are longer than K.  One chunk of them in a sum and the result is NaN."""
    M, N, ld = 256, 384, 1024
    for K in (912, 944):
        say("k tail, NaN behind the rows", (M, N, K))
        qa, sa, qb, sb = fp8_inputs(M, N, K, seed=K)
        a_pad = torch.full((M, ld), 0x7F, dtype=torch.uint8, device="cuda")
        b_pad = torch.full((N, ld), 0x7F, dtype=torch.uint8, device="cuda")
        a_pad[:, :K], b_pad[:, :K] = dev(qa), dev(qb)
        ref = R.gemm_f32acc(R.decode_fp8(qa), R.decode_fp8(qb))
        c = torch.zeros((M, N), dtype=torch.float32, device="cuda")
        st = Q.load_library().qgemm_gemm(Q.DT_F8E4M3, Q.DT_F32, 1, a_pad.data_ptr(), ld, b_pad.data_ptr(), ld, c.data_ptr(), N,
                                         M, N, K, None)
        assert st == 0
        _mfma(Q.last_config())
        got = host(c)
        assert not np.isnan(got).any(), Q.last_config()
        # (the operands are raw e4m3 codes up to 448: bring the sums to O(1), as the scaled GEMM would, for the tolerance)
        assert_close(got * np.float32(sa * sb), ref * np.float32(sa * sb), what=Q.last_config())


def test_what_is_left_for_the_any_shape_kernel():
    """K bytes not a multiple of 16, or operands that are not 16-byte aligned: the one-thread-per-element kernel, and
    qgemm_plan says so."""
    assert Q.plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 64, 64, 100) == "strided_any_shape"
    assert Q.plan(Q.DT_BF16, 0, 0, 64, 64, 100) == "strided_any_shape"           # 200 bytes
    assert Q.plan(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX, 0, 64, 64, 96) != "strided_any_shape"
    assert Q.plan(Q.DT_BF16, 0, 0, 64, 64, 72) != "strided_any_shape"
    M, N, K = 64, 96, 160
    qa, sa, qb, sb = int8_inputs(M, N, K, seed=9)
    whole = torch.zeros(M * K + 16, dtype=torch.int8, device="cuda")
    whole[1:1 + M * K] = dev(qa).flatten()
    a_off = whole[1:1 + M * K].view(M, K)                    # A starts one byte past a 16-byte boundary
    c = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    Q.int8_mm(a_off, dev(qb), scalar(sa), scalar(sb), c)
    assert Q.last_config() == "strided_any_shape"
    assert np.array_equal(host(c), R.gemm_i8_i32(qa, qb))
