"""The five BASELINE configurations at their full sizes.

Where the CPU oracle cannot finish the whole problem in seconds, the check is the oracle on
sampled full rows and full columns of C, plus size-independent properties of the whole matrix:
int32 results are identical bit for bit between two different tile configurations; scaling an
operand's scale by a power of two scales C exactly; a K split leaves int32 results unchanged."""
import numpy as np
import pytest
import torch

import qgemm_amd as Q
from oracle import cpu_ref as R
from tests.util import assert_close, dev, fp8_tensor, host, say, scalar

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _reset_options():
    yield
    Q.set_option("force_config", -1)
    Q.set_option("force_split", 0)
    Q.set_option("row_split", 1)


def _sample(n, count, seed):
    return np.sort(np.random.default_rng(seed).choice(n, size=count, replace=False))


def test_cfg1_fp16_1024_b_stored_transposed():
    """FP16 GEMM M=N=K=1024, A MxK, B stored NxK, uniform[-1,1], fp32 accumulate, fp16 out; whole matrix."""
    M = N = K = 1024
    say("cfg1 fp16 1024^3")
    ha, hb = R.encode_f16(R.fill_uniform((M, K), 42)), R.encode_f16(R.fill_uniform((N, K), 43))
    ref = R.gemm_f32acc(R.decode_f16(ha), R.decode_f16(hb))
    a, b = dev(ha.view(np.int16)).view(torch.float16), dev(hb.view(np.int16)).view(torch.float16)
    c = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    Q.gemm(a, b, c, "nk")
    # fp16 output: half an ulp (2^-11 relative) on top of accumulation-order slack
    assert_close(host(c).astype(np.float32), ref, rtol=2.0 ** -10, atol=2e-3, what=Q.last_config())


def test_cfg2_int8_4096_bit_exact():
    """INT8 per-matrix 4096^3: int32 accumulators bit-exact on 64 full rows and 64 full columns against the
    oracle, identical over the whole matrix between two tile configurations and a K split; fp32 output equals
    float(acc) * (sA * sB) bit for bit."""
    M = N = K = 4096
    say("cfg2 int8 4096^3")
    qa, sa = R.quantize_int8(R.fill_normal((M, K), 42))
    qb, sb = R.quantize_int8(R.fill_normal((N, K), 43))
    da, db_ = dev(qa), dev(qb)
    c = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    Q.int8_mm(da, db_, scalar(sa), scalar(sb), c)
    name0 = Q.last_config()
    got = host(c)
    rows, cols = _sample(M, 64, 1), _sample(N, 64, 2)
    assert np.array_equal(got[rows], R.gemm_i8_i32(qa[rows], qb)), name0
    assert np.array_equal(got[:, cols], R.gemm_i8_i32(qa, qb[cols])), name0
    # another tile configuration and a K split: the same integers everywhere
    Q.force_config("128x128_w2x2_dma")
    c2 = torch.zeros_like(c)
    Q.int8_mm(da, db_, scalar(sa), scalar(sb), c2)
    assert Q.last_config() != name0 and torch.equal(c, c2)
    Q.force_config(None)
    c3 = torch.zeros_like(c)
    Q.int8_mm(da, db_, scalar(sa), scalar(sb), c3, split_k=4)
    assert "splitk" in Q.last_config() and torch.equal(c, c3)
    cf = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    Q.int8_mm(da, db_, scalar(sa), scalar(sb), cf)
    assert np.array_equal(host(cf), R.scale_i32_to_f32(got, sa, sb))


def test_cfg3_fp8_per_matrix_8192():
    """FP8 e4m3 per-matrix 8192^3, bf16 out: rtol 2e-2 / atol 1e-2 against the fp32-accumulate oracle on 32 full
    rows and 32 full columns; doubling sA doubles every output exactly; two tile configurations agree to bf16
    rounding."""
    M = N = K = 8192
    say("cfg3 fp8 8192^3")
    qa, sa = R.quantize_fp8(R.fill_normal((M, K), 42))
    qb, sb = R.quantize_fp8(R.fill_normal((N, K), 43))
    assert R.decode_fp8(qa).__abs__().max() == 448.0          # max|x| maps to 448
    da, db_ = fp8_tensor(qa), fp8_tensor(qb)
    c = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    Q.scaled_gemm(da, db_, scalar(sa), scalar(sb), c, M, N, K, Q.SCALE_PER_MATRIX)
    name0 = Q.last_config()
    got = host(c)
    rows, cols = _sample(M, 32, 3), _sample(N, 32, 4)
    fb = R.decode_fp8(qb)
    assert_close(got[rows], R.gemm_f32acc(R.decode_fp8(qa[rows]), fb) * np.float32(sa * sb), what=name0 + " rows")
    del fb
    assert_close(got[:, cols], R.gemm_f32acc(R.decode_fp8(qa), R.decode_fp8(qb[cols])) * np.float32(sa * sb),
                 what=name0 + " cols")
    c2 = torch.zeros_like(c)
    Q.scaled_gemm(da, db_, scalar(2 * sa), scalar(sb), c2, M, N, K, Q.SCALE_PER_MATRIX)
    assert torch.equal(c2.float(), 2 * c.float())              # power-of-two scale: exact
    Q.force_config("256x256_w2x4_solo8")
    c3 = torch.zeros_like(c)
    Q.scaled_gemm(da, db_, scalar(sa), scalar(sb), c3, M, N, K, Q.SCALE_PER_MATRIX)
    assert Q.last_config() != name0
    # same products, different fp32 summation order: at most one bf16 ulp apart
    assert torch.all((c3.float() - c.float()).abs() <= 2.0 ** -7 * c.float().abs() + 1e-3)


def test_cfg4_fp8_block_scaled_6144x4608x7168():
    """FP8 block-scaled M=6144 N=4608 K=7168: a_scale [M, K/128], b_scale [N/128, K/128] uniform[0.5, 2], bf16
    out; oracle (per-128-block partial, then (P*as)*bs) on 24 full rows and 24 full columns."""
    M, N, K = 6144, 4608, 7168
    say("cfg4 fp8 block-scaled")
    qa, _ = R.quantize_fp8(R.fill_normal((M, K), 42))
    qb, _ = R.quantize_fp8(R.fill_normal((N, K), 43))
    # scales uniform[0.5, 2], times the 1/448 a quantiser would have produced, so C is O(sqrt(K))
    as_ = R.fill_uniform((M, K // 128), 44, 0.5, 2.0) * np.float32(5.0 / 448.0)
    bs = R.fill_uniform((N // 128, K // 128), 45, 0.5, 2.0) * np.float32(5.0 / 448.0)
    c = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    Q.scaled_gemm(fp8_tensor(qa), fp8_tensor(qb), dev(as_), dev(bs), c, M, N, K, Q.SCALE_BLOCK128)
    got = host(c)
    rows, cols = _sample(M, 24, 5), _sample(N, 24, 6)
    fb = R.decode_fp8(qb)
    assert_close(got[rows], R.gemm_fp8_block(R.decode_fp8(qa[rows]), fb, as_[rows], bs), what=Q.last_config())
    del fb
    # a column sample needs the b_scale row of each sampled column's 128-block: evaluate per block
    fa = R.decode_fp8(qa)
    for nb in np.unique(cols // 128):
        sel = cols[cols // 128 == nb]
        ref = R.gemm_fp8_block(fa, R.decode_fp8(qb[sel]), as_, bs[nb:nb + 1])
        assert_close(got[:, sel], ref, what=f"{Q.last_config()} cols of block {nb}")


def test_cfg4_shape_with_k_7200_stays_on_the_matrix_cores():
    """Config 4's shape with K = 7200 (56 whole K blocks and a quarter of one; K % 32 == 0 is all the reference's
    dispatch asks for, hip_mix_gemm_kernel.cpp:442-463), in both storages: the pipelined MFMA kernels, not the any-shape
    kernel; oracle on 16 full rows and the columns of one 128-block."""
    M, N, K = 6144, 4608, 7200
    say("cfg4 shape, K = 7200")
    KB = (K + 127) // 128
    assert Q.plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 0, M, N, K).startswith("256x256_w2x4_solo8")
    assert "strided" not in Q.plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 3, M, N, K)
    qa, _ = R.quantize_fp8(R.fill_normal((M, K), 42))
    qb, _ = R.quantize_fp8(R.fill_normal((N, K), 43))
    as_ = R.fill_uniform((M, KB), 44, 0.5, 2.0) * np.float32(5.0 / 448.0)
    bs = R.fill_uniform((N // 128, KB), 45, 0.5, 2.0) * np.float32(5.0 / 448.0)
    c = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    Q.scaled_gemm(fp8_tensor(qa), fp8_tensor(qb), dev(as_), dev(bs), c, M, N, K, Q.SCALE_BLOCK128)
    name = Q.last_config()
    assert name.startswith("256x256_w2x4_solo8"), name
    got = host(c)
    rows = _sample(M, 16, 5)
    fb = R.decode_fp8(qb)
    assert_close(got[rows], R.gemm_fp8_block(R.decode_fp8(qa[rows]), fb, as_[rows], bs), what=name)
    del fb
    nb = 17
    sel = np.arange(nb * 128, nb * 128 + 128, 9)
    assert_close(got[:, sel], R.gemm_fp8_block(R.decode_fp8(qa), R.decode_fp8(qb[sel]), as_, bs[nb:nb + 1]), what=name + " cols")
    # the reference's storage: A is K x M, B is K x N, scales K-block-major
    c2 = torch.zeros_like(c)
    Q.fp8_mm(fp8_tensor(np.ascontiguousarray(qa.T)).t(), fp8_tensor(np.ascontiguousarray(qb.T)).t(),
             dev(np.ascontiguousarray(as_.T)).t(), dev(np.ascontiguousarray(bs.T)).t(), c2)
    assert "strided" not in Q.last_config(), Q.last_config()
    assert_close(host(c2)[rows], got[rows], rtol=2.0 ** -7, atol=1e-3, what="reference storage against K-contiguous")


@pytest.mark.parametrize("M", [16, 64, 128])
def test_cfg5_skinny_split_k(M):
    """Skinny M, N=7168, K=2048, int8 (bit-exact) and fp8 (tolerance) with per-matrix scales; whole matrix.
    Once the way the heuristic runs it (narrow tiles over the whole of K) and once with K split in four."""
    N, K = 7168, 2048
    say("cfg5 skinny", M)
    qa, sa = R.quantize_int8(R.fill_normal((M, K), 42))
    qb, sb = R.quantize_int8(R.fill_normal((N, K), 43))
    acc = R.gemm_i8_i32(qa, qb)
    c = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    Q.int8_mm(dev(qa), dev(qb), scalar(sa), scalar(sb), c)
    assert np.array_equal(host(c), acc), Q.last_config()
    c.fill_(-1)
    Q.int8_mm(dev(qa), dev(qb), scalar(sa), scalar(sb), c, split_k=4)
    assert "splitk4" in Q.last_config(), Q.last_config()
    assert np.array_equal(host(c), acc), Q.last_config()
    cf = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    Q.int8_mm(dev(qa), dev(qb), scalar(sa), scalar(sb), cf)
    assert np.array_equal(host(cf), R.scale_i32_to_f32(acc, sa, sb))
    fa, ta = R.quantize_fp8(R.fill_normal((M, K), 44))
    fb, tb = R.quantize_fp8(R.fill_normal((N, K), 45))
    cb = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    Q.scaled_gemm(fp8_tensor(fa), fp8_tensor(fb), scalar(ta), scalar(tb), cb, M, N, K, Q.SCALE_PER_MATRIX)
    fref = R.gemm_f32acc(R.decode_fp8(fa), R.decode_fp8(fb)) * np.float32(ta * tb)
    assert_close(host(cb), fref, what=Q.last_config())
    Q.scaled_gemm(fp8_tensor(fa), fp8_tensor(fb), scalar(ta), scalar(tb), cb, M, N, K, Q.SCALE_PER_MATRIX, split_k=4)
    assert_close(host(cb), fref, what=Q.last_config())


@pytest.mark.parametrize("shape", [(16, 7168, 2048), (96, 7168, 2048), (128, 7168, 2048 + 128), (37, 2080, 2048),
                                   (512, 2048, 4096), (300, 1000, 2048 + 128)])        # (the last two: 64 x 64 tiles)
def test_block_scaled_skinny_m(shape):
    """The skinny-M kernel with 128-block scales (the arithmetic of FP8_GEMM_kernel, hip_mix_gemm_kernel.cpp:231-244,
    at decode-sized M): the whole matrix against the oracle with a_scale K-contiguous (QGEMM_LAYOUT_K_CONTIGUOUS) and,
    in the reference's storage (QGEMM_LAYOUT_REFERENCE), rows-contiguous: the kernel reads it through strides, so the two give the same
    bits.  K steps that do not divide by the 16 of a round, a ragged last strip and a last b_scale block that is not
    whole; and power-of-two scales on small integers, where every product and sum is exact, bit for bit."""
    M, N, K = shape
    say("block-scaled skinny", shape)
    KB, NB = K // 128, (N + 127) // 128
    qa, _ = R.quantize_fp8(R.fill_normal((M, K), 61))
    qb, _ = R.quantize_fp8(R.fill_normal((N, K), 62))
    as_ = R.fill_uniform((M, KB), 63, 0.5, 2.0) / np.float32(448)
    bs = R.fill_uniform((NB, KB), 64, 0.5, 2.0) / np.float32(448)
    assert Q.plan(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 0, M, N, K).startswith("skinny")
    ref = R.gemm_fp8_block(R.decode_fp8(qa), R.decode_fp8(qb), as_, bs)
    c = torch.full((M, N), 7.0, dtype=torch.bfloat16, device="cuda")
    Q.scaled_gemm(fp8_tensor(qa), fp8_tensor(qb), dev(as_), dev(bs), c, M, N, K, Q.SCALE_BLOCK128)
    name = Q.last_config()
    assert name.startswith("skinny"), name
    assert_close(host(c), ref, what=name)
    # the reference's storage: operands and scales transposed; the NT kernel behind the operand transposes reads
    # a_scale rows-contiguous
    if M % 32 == 0 and N % 32 == 0:       # (the reference's dispatch refuses other shapes in its own layout: mix_gemm.h)
        Q.set_option("kmajor", 0)
        try:
            c2 = torch.full((M, N), 9.0, dtype=torch.bfloat16, device="cuda")
            Q.scaled_gemm(fp8_tensor(np.ascontiguousarray(qa.T)), fp8_tensor(np.ascontiguousarray(qb.T)),
                          dev(np.ascontiguousarray(as_.T)), dev(np.ascontiguousarray(bs.T)), c2, M, N, K, Q.SCALE_BLOCK128,
                          layout=Q.LAYOUT_REFERENCE)
            assert "skinny" in Q.last_config(), Q.last_config()
            assert torch.equal(c, c2), Q.last_config()
        finally:
            Q.set_option("kmajor", 1)
    # power-of-two scales, small integers: exact in any order of summation
    rng = np.random.default_rng(65)
    ia = rng.integers(-4, 5, (M, K)).astype(np.float32)
    ib = rng.integers(-4, 5, (N, K)).astype(np.float32)
    as2 = np.exp2(rng.integers(-3, 4, (M, KB))).astype(np.float32)
    bs2 = np.exp2(rng.integers(-3, 4, (NB, KB))).astype(np.float32)
    ref2 = R.gemm_fp8_block(ia, ib, as2, bs2)
    cx = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    Q.scaled_gemm(fp8_tensor(R.encode_fp8(ia)), fp8_tensor(R.encode_fp8(ib)), dev(as2), dev(bs2), cx, M, N, K, Q.SCALE_BLOCK128)
    assert Q.last_config().startswith("skinny"), Q.last_config()
    assert np.array_equal(host(cx), ref2)


def test_row_split_of_a_partly_empty_last_round():
    """4608 x 7680 are 540 tiles of 256 x 256 on 256 CUs: the rows of the two full rounds (4352) go to the 256 x 256
    kernel, the 256 rows below to a second launch with smaller tiles.  int8: the same integers as the single
    launch, everywhere, and the oracle's on sampled rows on both sides of the seam; fp8 block-scaled and bf16:
    within tolerance of the oracle on rows of both parts, and of the single launch everywhere."""
    M, N, K = 4608, 7680, 2048
    M1 = 4352
    say("row split int8", M, N, K)
    assert "+" in Q.plan(Q.DT_I8, Q.SCALE_PER_MATRIX, 0, M, N, K)
    rng = np.random.default_rng(21)
    qa = rng.integers(-127, 128, (M, K), dtype=np.int8)
    qb = rng.integers(-127, 128, (N, K), dtype=np.int8)
    da, db_ = dev(qa), dev(qb)
    c = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    Q.int8_mm(da, db_, scalar(1.0), scalar(1.0), c)
    name = Q.last_config()
    assert "+" in name, name
    rows = np.concatenate([_sample(M1, 12, 5), M1 + _sample(M - M1, 12, 6), [M1 - 1, M1, M - 1]])
    assert np.array_equal(host(c)[rows], R.gemm_i8_i32(qa[rows], qb)), name
    Q.set_option("row_split", 0)
    c1 = torch.zeros_like(c)
    Q.int8_mm(da, db_, scalar(1.0), scalar(1.0), c1)
    assert "+" not in Q.last_config() and torch.equal(c, c1)
    Q.set_option("row_split", 1)

    say("row split fp8 block-scaled", M, N, K)
    qa8, _ = R.quantize_fp8(R.fill_normal((M, K), 31))
    qb8, _ = R.quantize_fp8(R.fill_normal((N, K), 32))
    as_ = R.fill_uniform((M, K // 128), 33, 0.5, 2.0) / np.float32(448)
    bs = R.fill_uniform((N // 128, K // 128), 34, 0.5, 2.0) / np.float32(448)
    cb = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    Q.scaled_gemm(fp8_tensor(qa8), fp8_tensor(qb8), dev(as_), dev(bs), cb, M, N, K, Q.SCALE_BLOCK128)
    name = Q.last_config()
    assert "+" in name, name
    ref = R.gemm_fp8_block(R.decode_fp8(qa8[rows]), R.decode_fp8(qb8), as_[rows], bs)
    assert_close(host(cb)[rows], ref, what=name)
    Q.set_option("row_split", 0)
    cb1 = torch.zeros_like(cb)
    Q.scaled_gemm(fp8_tensor(qa8), fp8_tensor(qb8), dev(as_), dev(bs), cb1, M, N, K, Q.SCALE_BLOCK128)
    assert "+" not in Q.last_config()
    assert torch.all((cb1.float() - cb.float()).abs() <= 2.0 ** -7 * cb.float().abs() + 1e-3)
    Q.set_option("row_split", 1)

    say("row split bf16", M, N, K)
    ha, hb = R.encode_bf16(R.fill_uniform((M, K), 41)), R.encode_bf16(R.fill_uniform((N, K), 42))
    a16, b16 = dev(ha.view(np.int16)).view(torch.bfloat16), dev(hb.view(np.int16)).view(torch.bfloat16)
    c16 = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    Q.gemm(a16, b16, c16, "nk")
    name = Q.last_config()
    assert "+" in name, name
    assert_close(host(c16)[rows], R.gemm_f32acc(R.decode_bf16(ha[rows]), R.decode_bf16(hb)), rtol=1e-4, atol=1e-3, what=name)


def test_column_split_of_a_partly_empty_last_round():
    """4096 x 4608 are 16 x 18 = 288 tiles of 256 x 256 on 256 CUs, and no whole number of row bands makes a full round:
    the 16 column bands of one full round (4096 columns) go to the 256 x 256 kernel, the 512 columns to their right to a
    second launch (plan "a|b"), whose B, b_scale blocks and C start 4096 columns in.  int8: the integers of the single
    launch everywhere and the oracle's on sampled rows (all columns, so both sides of the seam); fp8 block-scaled (the
    right part must pick up b_scale at block row 32) and bf16: the oracle within tolerance on the same rows, and the
    single launch everywhere."""
    M, N, K = 4096, 4608, 2048
    N1 = 4096
    say("column split int8", M, N, K)
    plan = Q.plan(Q.DT_I8, Q.SCALE_PER_MATRIX, 0, M, N, K)
    assert "|" in plan and "+" not in plan, plan
    rng = np.random.default_rng(23)
    qa = rng.integers(-127, 128, (M, K), dtype=np.int8)
    qb = rng.integers(-127, 128, (N, K), dtype=np.int8)
    da, db_ = dev(qa), dev(qb)
    c = torch.full((M, N), -7, dtype=torch.int32, device="cuda")
    Q.int8_mm(da, db_, scalar(1.0), scalar(1.0), c)
    name = Q.last_config()
    assert name == plan, (name, plan)
    rows = np.concatenate([_sample(M, 20, 5), [0, M - 1]])
    got = host(c)
    assert np.array_equal(got[rows], R.gemm_i8_i32(qa[rows], qb)), name
    cols = np.array([0, N1 - 1, N1, N1 + 127, N1 + 128, N - 1])
    assert np.array_equal(got[:, cols], R.gemm_i8_i32(qa, qb[cols])), name
    Q.set_option("row_split", 0)
    c1 = torch.full((M, N), -8, dtype=torch.int32, device="cuda")
    Q.int8_mm(da, db_, scalar(1.0), scalar(1.0), c1)
    assert "|" not in Q.last_config() and "+" not in Q.last_config() and torch.equal(c, c1)
    Q.set_option("row_split", 1)

    say("column split fp8 block-scaled", M, N, K)
    qa8, _ = R.quantize_fp8(R.fill_normal((M, K), 35))
    qb8, _ = R.quantize_fp8(R.fill_normal((N, K), 36))
    as_ = R.fill_uniform((M, K // 128), 37, 0.5, 2.0) / np.float32(448)
    bs = R.fill_uniform((N // 128, K // 128), 38, 0.5, 2.0) / np.float32(448)
    cb = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    Q.scaled_gemm(fp8_tensor(qa8), fp8_tensor(qb8), dev(as_), dev(bs), cb, M, N, K, Q.SCALE_BLOCK128)
    name = Q.last_config()
    assert "|" in name, name
    ref = R.gemm_fp8_block(R.decode_fp8(qa8[rows]), R.decode_fp8(qb8), as_[rows], bs)
    assert_close(host(cb)[rows], ref, what=name)
    Q.set_option("row_split", 0)
    cb1 = torch.zeros_like(cb)
    Q.scaled_gemm(fp8_tensor(qa8), fp8_tensor(qb8), dev(as_), dev(bs), cb1, M, N, K, Q.SCALE_BLOCK128)
    assert "|" not in Q.last_config()
    assert torch.all((cb1.float() - cb.float()).abs() <= 2.0 ** -7 * cb.float().abs() + 1e-3)
    Q.set_option("row_split", 1)

    say("column split bf16, C with a leading dimension", M, N, K)
    ha, hb = R.encode_bf16(R.fill_uniform((M, K), 43)), R.encode_bf16(R.fill_uniform((N, K), 44))
    a16, b16 = dev(ha.view(np.int16)).view(torch.bfloat16), dev(hb.view(np.int16)).view(torch.bfloat16)
    wide = torch.full((M, N + 64), -3.0, dtype=torch.float32, device="cuda")
    c16 = wide[:, :N]
    Q.gemm(a16, b16, c16, "nk")
    name = Q.last_config()
    assert "|" in name, name
    assert_close(host(c16)[rows], R.gemm_f32acc(R.decode_bf16(ha[rows]), R.decode_bf16(hb)), rtol=1e-4, atol=1e-3, what=name)
    assert torch.all(wide[:, N:] == -3.0)


def test_forced_row_and_column_splits_on_ragged_shapes_match_the_single_launch():
    """Ragged M and N (not multiples of the tiles, of 128 or of 16), with the rows and then the columns of the full
    rounds forced into a launch of their own wherever the geometry has such a split: the int32 results are those of
    the single launch, element for element, and nothing is written beyond column N of a wider C.  fp8 with block
    scales (ragged N: the last b_scale block row is partial) stays within a bf16 ulp of the single launch."""
    rng = np.random.default_rng(2025)
    shapes = [(4097, 4609, 640), (6000, 4500, 512), (3333, 9001, 384), (8200, 2300, 768), (5121, 5119, 400)]
    seen = set()
    try:
        for (M, N, K) in shapes:
            say("forced splits int8", M, N, K)
            da = dev(rng.integers(-127, 128, (M, K), dtype=np.int8))
            db_ = dev(rng.integers(-127, 128, (N, K), dtype=np.int8))
            outs = {}
            for mode in (0, 2, 3):
                Q.set_option("row_split", mode)
                wide = torch.full((M, N + 3), -9, dtype=torch.int32, device="cuda")
                Q.int8_mm(da, db_, scalar(1.0), scalar(1.0), wide[:, :N])
                name = Q.last_config()
                assert torch.all(wide[:, N:] == -9), name
                outs[mode] = wide[:, :N].clone()
                seen.add("+" if "+" in name else ("|" if "|" in name else "one"))
                assert mode != 0 or ("+" not in name and "|" not in name), name
            assert torch.equal(outs[0], outs[2]) and torch.equal(outs[0], outs[3]), (M, N, K)
        assert seen == {"+", "|", "one"}, seen

        M, N, K = 4200, 4500, 640
        say("forced splits fp8 block-scaled", M, N, K)
        KB, NB = K // 128, (N + 127) // 128
        qa8, _ = R.quantize_fp8(R.fill_normal((M, K), 61))
        qb8, _ = R.quantize_fp8(R.fill_normal((N, K), 62))
        as_ = dev(R.fill_uniform((M, KB), 63, 0.5, 2.0) / np.float32(448))
        bs = dev(R.fill_uniform((NB, KB), 64, 0.5, 2.0) / np.float32(448))
        a8, b8 = fp8_tensor(qa8), fp8_tensor(qb8)
        outs = {}
        for mode in (0, 2, 3):
            Q.set_option("row_split", mode)
            c = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
            Q.scaled_gemm(a8, b8, as_, bs, c, M, N, K, Q.SCALE_BLOCK128)
            outs[mode] = (c.float(), Q.last_config())
        assert "+" in outs[2][1] and "|" in outs[3][1], (outs[2][1], outs[3][1])
        for mode in (2, 3):
            assert torch.all((outs[mode][0] - outs[0][0]).abs() <= 2.0 ** -7 * outs[0][0].abs() + 1e-3), outs[mode][1]
    finally:
        Q.set_option("row_split", 1)


@pytest.mark.parametrize("shape,m_main,rest", [((4184, 4096, 2048), 4096, "skinny_64x64_k8"),      # 88 rows below one full round
                                               ((5000, 4096, 2048), 4096, "128x128")])            # single launch: 128 x 128 tiles
def test_row_split_with_a_short_rest_and_against_smaller_tiles(shape, m_main, rest):
    """Row split where the rows below the full rounds are at most 128 (they go to the skinny-M kernel) and where a
    single launch would have taken smaller tiles for everything.  int8: the integers of the single launch
    everywhere and the oracle's on rows of both parts and at the seam; fp8 per-matrix to bf16: the oracle within
    tolerance on the same rows."""
    M, N, K = shape
    say("row split", shape)
    plan = Q.plan(Q.DT_I8, Q.SCALE_PER_MATRIX, 0, M, N, K)
    assert plan.startswith("256x256") and "+" in plan and rest in plan.split("+")[1], plan
    rng = np.random.default_rng(77)
    qa = rng.integers(-127, 128, (M, K), dtype=np.int8)
    qb = rng.integers(-127, 128, (N, K), dtype=np.int8)
    da, db_ = dev(qa), dev(qb)
    c = torch.full((M, N), -5, dtype=torch.int32, device="cuda")
    Q.int8_mm(da, db_, scalar(1.0), scalar(1.0), c)
    name = Q.last_config()
    assert name == plan, (name, plan)
    rows = np.concatenate([_sample(m_main, 10, 5), m_main + _sample(M - m_main, 10, 6), [m_main - 1, m_main, M - 1]])
    assert np.array_equal(host(c)[rows], R.gemm_i8_i32(qa[rows], qb)), name
    Q.set_option("row_split", 0)
    c1 = torch.full((M, N), -6, dtype=torch.int32, device="cuda")
    Q.int8_mm(da, db_, scalar(1.0), scalar(1.0), c1)
    assert "+" not in Q.last_config() and torch.equal(c, c1)
    Q.set_option("row_split", 1)

    qa8, sa = R.quantize_fp8(R.fill_normal((M, K), 51))
    qb8, sb = R.quantize_fp8(R.fill_normal((N, K), 52))
    cb = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    Q.scaled_gemm(fp8_tensor(qa8), fp8_tensor(qb8), scalar(sa), scalar(sb), cb, M, N, K, Q.SCALE_PER_MATRIX)
    name = Q.last_config()
    assert "+" in name, name
    ref = R.gemm_f32acc(R.decode_fp8(qa8[rows]), R.decode_fp8(qb8)) * np.float32(sa * sb)
    assert_close(host(cb)[rows], ref, what=name)


def test_one_round_of_256x128_tiles_int8_and_block_scales():
    """2048 x 4096 x 4096, a shape the heuristic gives to the row with copying waves (256 tiles of 256 x 128): int32
    accumulators identical over the whole matrix to those of a 128 x 128 tile and of a K split, and bit-exact
    against the oracle on sampled rows and columns; with 128-block scales, sampled rows against the oracle and an
    exact factor of four when every a_scale is doubled and every b_scale too."""
    M, N, K = 2048, 4096, 4096
    say("one round of 256x128 tiles", (M, N, K))
    qa, sa = R.quantize_int8(R.fill_normal((M, K), 52))
    qb, sb = R.quantize_int8(R.fill_normal((N, K), 53))
    da, db_ = dev(qa), dev(qb)
    c = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    Q.int8_mm(da, db_, scalar(sa), scalar(sb), c)
    assert Q.last_config() == "256x128_w2x2_cw", Q.last_config()
    got = host(c)
    rows, cols = _sample(M, 32, 3), _sample(N, 32, 4)
    assert np.array_equal(got[rows], R.gemm_i8_i32(qa[rows], qb))
    assert np.array_equal(got[:, cols], R.gemm_i8_i32(qa, qb[cols]))
    for force, split in (("128x128_w2x2_dma", 1), ("256x128_w2x2_cw", 2)):
        Q.force_config(force)
        Q.set_option("force_split", split)
        c2 = torch.zeros_like(c)
        Q.int8_mm(da, db_, scalar(sa), scalar(sb), c2)
        assert torch.equal(c, c2), Q.last_config()
    Q.set_option("force_config", -1)
    Q.set_option("force_split", 0)
    # block scales
    rng = np.random.default_rng(54)
    a8 = R.encode_fp8(np.clip(R.fill_normal((M, K), 55), -4, 4))
    b8 = R.encode_fp8(np.clip(R.fill_normal((N, K), 56), -4, 4))
    as_ = (0.5 + rng.random((M, K // 128))).astype(np.float32)
    bs = (0.5 + rng.random((N // 128, K // 128))).astype(np.float32)
    ta, tb = fp8_tensor(a8), fp8_tensor(b8)
    cf = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    Q.scaled_gemm(ta, tb, dev(as_), dev(bs), cf, M, N, K, Q.SCALE_BLOCK128)
    assert Q.last_config() == "256x128_w2x2_cw_ks", Q.last_config()
    gotf = host(cf)
    rows = _sample(M, 8, 5)
    ref = R.gemm_fp8_block(R.decode_fp8(a8[rows]), R.decode_fp8(b8), as_[rows], bs)
    # (every kernel of the library lands within 4.2e-3 of the exact sums here, rms 9e-4 at |C| around 55: that is the
    # MFMA's own accumulation of 128 products, the fp32 oracle is within 6e-5; the stated tolerance covers it)
    assert_close(gotf[rows], ref, what=Q.last_config())
    cf4 = torch.zeros_like(cf)
    Q.scaled_gemm(ta, tb, dev(2 * as_), dev(2 * bs), cf4, M, N, K, Q.SCALE_BLOCK128)
    assert torch.equal(cf4, 4 * cf)
