"""GPU parity tests: the HIP path, called through the C ABI, against the CPU
oracle on the same seeded inputs.  Integer results bit-exact; float results
within rtol 2e-2 / atol 1e-2 of the fp32-accumulate oracle (tests/util.py).

Sizes here are ones the oracle finishes in seconds; the full BASELINE sizes are
in test_gpu_full_size.py."""
import numpy as np
import pytest
import torch

import qgemm_amd as Q
from oracle import cpu_ref as R
from tests.util import (assert_close, dev, fp8_inputs, fp8_tensor, host, int8_inputs, say, scalar)

pytestmark = pytest.mark.gpu

# rows of the variant tables, by name, as the library reports them (one table per family)
I8_ROWS = Q.variant_names(Q.DT_I8, Q.SCALE_PER_MATRIX)
F8_ROWS = Q.variant_names(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX)
F8B_ROWS = Q.variant_names(Q.DT_F8E4M3, Q.SCALE_BLOCK128)
F8B_TN_ROWS = Q.variant_names(Q.DT_F8E4M3, Q.SCALE_BLOCK128, 3)
ROWS_16 = {"bf16": Q.variant_names(Q.DT_BF16), "f16": Q.variant_names(Q.DT_F16)}
ROWS_16_NN = {"bf16": Q.variant_names(Q.DT_BF16, 0, 2), "f16": Q.variant_names(Q.DT_F16, 0, 2)}
@pytest.mark.parametrize("shape", [(130, 1000, 4096), (130, 1530, 6144), (200, 1530, 5120), (40, 1000, 4096), (64, 2040, 5120)])
def test_small_tiles_over_several_row_tiles_instead_of_a_k_split(shape):
    """17 .. 256 rows, few columns, 32 .. 48 K steps: the planner takes small tiles of the skinny-M kernel, several over
    the rows, where it used to take a taller tile and a K split (option "small_tiles", 0 gives the old choice).  int32
    accumulators of both choices bit for bit against the oracle, ragged M and N."""
    M, N, K = shape
    row = Q.plan(Q.DT_I8, Q.SCALE_PER_MATRIX, 0, M, N, K)
    say("small tiles", shape, row)
    assert row.startswith("skinny_") and "splitk" not in row and int(row.split("_")[1].split("x")[0]) < M, row
    qa, sa, qb, sb = int8_inputs(M, N, K, seed=321)
    ref = R.gemm_i8_i32(qa, qb)
    c = torch.full((M, N), -7, dtype=torch.int32, device="cuda")
    Q.int8_mm(dev(qa), dev(qb), scalar(sa), scalar(sb), c)
    assert Q.last_config() == row and np.array_equal(host(c), ref)
    Q.set_option("small_tiles", 0)
    try:
        c0 = torch.full((M, N), -8, dtype=torch.int32, device="cuda")
        Q.int8_mm(dev(qa), dev(qb), scalar(sa), scalar(sb), c0)
        assert Q.last_config() != row and np.array_equal(host(c0), ref), Q.last_config()
    finally:
        Q.set_option("small_tiles", 1)


PAIRS_16 = [(d, v) for d in ("f16", "bf16") for v in ROWS_16[d]]
PAIRS_16_NN = [(d, v) for d in ("f16", "bf16") for v in ROWS_16_NN[d]]


@pytest.fixture(autouse=True)
def _reset_options():
    yield
    Q.force_config(None)
    Q.set_option("force_split", 0)
    Q.set_option("group_m", 0)
    Q.set_option("kmajor", 1)
    Q.set_option("k_rot", -1)


def test_selftest_layouts():
    """The hardware behaviour the kernels assume: LDS-DMA placement (also above 64 KiB),
    MFMA operand and accumulator lane layouts for i8 / f8 / bf16 / f16."""
    say("selftest_layouts")
    ok, report = Q.selftest_layouts()
    print(report, flush=True)
    assert ok, report
    # tile rows past M / N are kept out of reach by the buffer range check, scalar offset included
    assert "soffset IS part of the buffer range check" in report


# ----------------------------------------------------------------- int8
@pytest.mark.parametrize("variant", I8_ROWS)
@pytest.mark.parametrize("shape", [(256, 256, 256), (300, 202, 384), (16, 128, 128), (520, 1000, 640)])
def test_int8_accumulators_bit_exact_every_variant(variant, shape):
    M, N, K = shape
    say("int8 i32", shape, "variant", variant)
    qa, sa, qb, sb = int8_inputs(M, N, K, seed=100 + I8_ROWS.index(variant))
    ref = R.gemm_i8_i32(qa, qb)
    Q.force_config(variant)
    c = torch.full((M, N), -7, dtype=torch.int32, device="cuda")
    Q.int8_mm(dev(qa), dev(qb), scalar(sa), scalar(sb), c, split_k=1)
    assert np.array_equal(host(c), ref), Q.last_config()


@pytest.mark.parametrize("shape", [(512, 384, 1024), (100, 36, 256)])
def test_int8_per_matrix_f32_bit_exact(shape):
    M, N, K = shape
    say("int8 f32", shape)
    qa, sa, qb, sb = int8_inputs(M, N, K, seed=7)
    ref = R.scale_i32_to_f32(R.gemm_i8_i32(qa, qb), sa, sb)
    c = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    Q.int8_mm(dev(qa), dev(qb), scalar(sa), scalar(sb), c)
    assert np.array_equal(host(c), ref), Q.last_config()      # one rounding each side: identical bits


def test_int8_extremes_do_not_overflow():
    M, N, K = 32, 128, 8192
    say("int8 extremes", (M, N, K))
    a = torch.full((M, K), 127, dtype=torch.int8, device="cuda")
    b = torch.full((N, K), -127, dtype=torch.int8, device="cuda")
    c = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    Q.int8_mm(a, b, scalar(1), scalar(1), c)
    assert torch.all(c == -127 * 127 * K)


@pytest.mark.parametrize("nsplit", [2, 3, 8])
def test_int8_split_k_bit_exact(nsplit):
    M, N, K = 64, 384, 2048
    say("int8 split-k", nsplit)
    qa, sa, qb, sb = int8_inputs(M, N, K, seed=11)
    acc = R.gemm_i8_i32(qa, qb)
    c32 = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    Q.int8_mm(dev(qa), dev(qb), scalar(sa), scalar(sb), c32, split_k=nsplit)
    assert "splitk" in Q.last_config()
    assert np.array_equal(host(c32), acc)
    cf = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    Q.int8_mm(dev(qa), dev(qb), scalar(sa), scalar(sb), cf, split_k=nsplit)
    assert np.array_equal(host(cf), R.scale_i32_to_f32(acc, sa, sb))


# ------------------------------------------------------------------ fp8
@pytest.mark.parametrize("variant", F8_ROWS)
def test_fp8_per_matrix_every_variant(variant):
    M, N, K = 272, 392, 512
    say("fp8 per-matrix", (M, N, K), "variant", variant)
    qa, sa, qb, sb = fp8_inputs(M, N, K, seed=200 + F8_ROWS.index(variant))
    ref = R.gemm_f32acc(R.decode_fp8(qa), R.decode_fp8(qb)) * np.float32(sa * sb)
    Q.force_config(variant)
    for dt in (torch.bfloat16, torch.float32, torch.float16):
        c = torch.zeros((M, N), dtype=dt, device="cuda")
        Q.scaled_gemm(fp8_tensor(qa), fp8_tensor(qb), scalar(sa), scalar(sb), c, M, N, K, Q.SCALE_PER_MATRIX,
                      split_k=1)
        assert_close(host(c).astype(np.float32), ref, what=f"{Q.last_config()} {dt}")


def test_fp8_exact_on_small_integers():
    """Products of small integers sum exactly in fp32: the GPU result must equal the oracle bit for bit,
    which pins operand order and the K mapping without any tolerance."""
    M, N, K = 128, 256, 1024
    say("fp8 exact integers")
    rng = np.random.default_rng(5)
    a = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
    b = rng.integers(-4, 5, size=(N, K)).astype(np.float32)
    qa, qb = R.encode_fp8(a), R.encode_fp8(b)
    ref = R.gemm_f32acc(a, b)
    c = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    Q.scaled_gemm(fp8_tensor(qa), fp8_tensor(qb), scalar(1), scalar(1), c, M, N, K, Q.SCALE_PER_MATRIX)
    assert np.array_equal(host(c), ref)


def test_fp8_every_code_decodes_like_the_oracle():
    """Row i of A holds code i on the diagonal position i: C = A * I picks every finite e4m3 code once."""
    say("fp8 all codes")
    codes = np.array([b for b in range(256) if (b & 0x7F) != 0x7F], np.uint8)
    M, K, N = 256, 256, 256
    qa = np.zeros((M, K), np.uint8)
    for i, cde in enumerate(codes):
        qa[i, i] = cde
    qb = np.zeros((N, K), np.uint8)
    qb[np.arange(N), np.arange(N)] = 0x38          # 1.0
    c = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    Q.scaled_gemm(fp8_tensor(qa), fp8_tensor(qb), scalar(1), scalar(1), c, M, N, K, Q.SCALE_PER_MATRIX)
    got = host(c)
    assert np.array_equal(np.diag(got)[: len(codes)], R.decode_fp8(codes))


@pytest.mark.parametrize("variant", F8B_ROWS)
def test_fp8_block_scaled_every_variant(variant):
    M, N, K = 160, 384, 512
    say("fp8 block-scaled", (M, N, K), "variant", variant)
    qa, _, qb, _ = fp8_inputs(M, N, K, seed=300 + F8B_ROWS.index(variant))
    as_ = R.fill_uniform((M, K // 128), 301, 0.5, 2.0)
    bs = R.fill_uniform((N // 128, K // 128), 302, 0.5, 2.0)
    # bring the products to O(1) so atol means something
    as_ *= np.float32(1.0 / 448.0)
    bs *= np.float32(1.0 / 448.0)
    ref = R.gemm_fp8_block(R.decode_fp8(qa), R.decode_fp8(qb), as_, bs)
    Q.force_config(variant)
    c = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    Q.scaled_gemm(fp8_tensor(qa), fp8_tensor(qb), dev(as_), dev(bs), c, M, N, K, Q.SCALE_BLOCK128, split_k=1)
    assert_close(host(c), ref, what=Q.last_config())


@pytest.mark.parametrize("variant", [None] + F8B_ROWS)
@pytest.mark.parametrize("shape", [(64, 256, 512), (272, 392, 768)])
def test_fp8_block_scaled_power_of_two_scales_bit_exact(variant, shape):
    """Power-of-two scales commute exactly with fp32 arithmetic, and small-integer products sum exactly:
    the scaled result must equal the oracle bit for bit, in every tile variant and pipeline (a wrong scale
    index, row or K block, cannot hide behind a tolerance).  Ragged M and N in the second shape."""
    M, N, K = shape
    say("fp8 block pow2", shape, "variant", variant)
    Q.force_config(variant)
    rng = np.random.default_rng(6 + ([None] + F8B_ROWS).index(variant))
    a = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
    b = rng.integers(-3, 4, size=(N, K)).astype(np.float32)
    as_ = (2.0 ** rng.integers(-3, 4, size=(M, K // 128))).astype(np.float32)
    bs = (2.0 ** rng.integers(-3, 4, size=((N + 127) // 128, K // 128))).astype(np.float32)
    ref = R.gemm_fp8_block(a, b, as_, bs)
    c = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    Q.scaled_gemm(fp8_tensor(R.encode_fp8(a)), fp8_tensor(R.encode_fp8(b)), dev(as_), dev(bs), c, M, N, K,
                  Q.SCALE_BLOCK128, split_k=1 if variant else 0)
    assert np.array_equal(host(c), ref), Q.last_config()


@pytest.mark.parametrize("case", [(512, 512, 1024, 0), (300, 520, 768, 0), (256, 256, 1536, 2),
                                  (256, 256, 1280, 2), (256, 256, 384, 0), (512, 256, 7168, 0), (300, 256, 7296, 3)])
def test_fp8_block_scaled_k_contiguous_scale_twin(case):
    """The block-scaled 8-wave kernel reads a_scale as QGEMM_LAYOUT_K_CONTIGUOUS passes it, two K blocks per 8-byte
    load, whatever the number of K blocks per row (an odd one puts every other row at a 4-byte aligned address and
    lets the pair behind a row's last block reach into the next row, or past the end of the array, where the buffer
    range check returns zero for it) and per K slice; bit-exact on small integers and power-of-two scales, so a scale
    taken from the wrong K block or row cannot pass."""
    M, N, K, split = case
    say("fp8 block, K-contiguous a_scale", case)
    rng = np.random.default_rng(17)
    a = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
    b = rng.integers(-3, 4, size=(N, K)).astype(np.float32)
    as_ = (2.0 ** rng.integers(-3, 4, size=(M, K // 128))).astype(np.float32)
    bs = (2.0 ** rng.integers(-3, 4, size=((N + 127) // 128, K // 128))).astype(np.float32)
    ref = R.gemm_fp8_block(a, b, as_, bs)
    Q.force_config("256x256_w2x4_solo8")
    Q.set_option("force_split", split)
    c = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    Q.scaled_gemm(fp8_tensor(R.encode_fp8(a)), fp8_tensor(R.encode_fp8(b)), dev(as_), dev(bs), c, M, N, K, Q.SCALE_BLOCK128)
    assert "solo8_ks" in Q.last_config(), Q.last_config()
    assert np.array_equal(host(c), ref), Q.last_config()
    # scales that start at a 4-byte aligned address, with NaNs in front of and behind the array: nothing outside it
    # may reach a result
    as_off = torch.full((as_.size + 2,), float("nan"), dtype=torch.float32, device="cuda")
    as_off[1:-1] = dev(as_).flatten()
    c.zero_()
    Q.scaled_gemm(fp8_tensor(R.encode_fp8(a)), fp8_tensor(R.encode_fp8(b)), as_off[1:-1], dev(bs), c, M, N, K, Q.SCALE_BLOCK128)
    assert "solo8_ks" in Q.last_config(), Q.last_config()
    assert np.array_equal(host(c), ref), Q.last_config()


def test_fp8_mm_reference_layout():
    """fp8_mm(a, b, as, bs, c) with the reference's column-major contract
    (hip_mix_gemm_kernel.cpp:425-439): same numbers as the K-contiguous call."""
    M, N, K = 128, 192, 384
    say("fp8_mm reference layout")
    qa, _, qb, _ = fp8_inputs(M, N, K, seed=31)
    as_ = R.fill_uniform((M, K // 128), 32, 0.5, 2.0) / np.float32(448)
    bs = R.fill_uniform(((N + 127) // 128, K // 128), 33, 0.5, 2.0) / np.float32(448)
    ref = R.gemm_fp8_block(R.decode_fp8(qa), R.decode_fp8(qb), as_, bs)
    # column-major [m,k] == row-major [k,m]; torch views with the reference's sizes and strides
    a_t = fp8_tensor(np.ascontiguousarray(qa.T)).t()          # size (M,K), stride (1,M)
    b_t = fp8_tensor(np.ascontiguousarray(qb.T)).t()          # size (N,K), stride (1,N)
    as_t = dev(np.ascontiguousarray(as_.T)).t()
    bs_t = dev(np.ascontiguousarray(bs.T)).t()
    c = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    Q.fp8_mm(a_t, b_t, as_t, bs_t, c)
    assert_close(host(c), ref, what=Q.last_config())
    # the oracle in the reference's own layout gives the same numbers
    tn = R.gemm_fp8_block(R.decode_fp8(np.ascontiguousarray(qa.T)), R.decode_fp8(np.ascontiguousarray(qb.T)),
                          np.ascontiguousarray(as_.T), np.ascontiguousarray(bs.T), "tn", "col")
    assert np.array_equal(tn, ref)


@pytest.mark.parametrize("variant", F8B_TN_ROWS)
@pytest.mark.parametrize("shape", [(160, 224, 512), (288, 544, 384)])
def test_fp8_mm_reference_layout_native_every_variant(variant, shape):
    """The reference storage (A is K x M, B is K x N, hip_mix_gemm_kernel.cpp:96,111) read as it lies, through
    the K-major tiles and the transposing LDS reads, for every tile variant; against the oracle, and against
    the route through the transpose utility (same kernel arithmetic, other summation order inside an MFMA)."""
    M, N, K = shape
    say("fp8_mm reference layout, native", shape, "variant", variant)
    qa, _, qb, _ = fp8_inputs(M, N, K, seed=500 + F8B_TN_ROWS.index(variant))
    as_ = R.fill_uniform((M, K // 128), 501, 0.5, 2.0) / np.float32(448)
    bs = R.fill_uniform(((N + 127) // 128, K // 128), 502, 0.5, 2.0) / np.float32(448)
    ref = R.gemm_fp8_block(R.decode_fp8(qa), R.decode_fp8(qb), as_, bs)
    a_t = fp8_tensor(np.ascontiguousarray(qa.T)).t()
    b_t = fp8_tensor(np.ascontiguousarray(qb.T)).t()
    as_t = dev(np.ascontiguousarray(as_.T)).t()
    bs_t = dev(np.ascontiguousarray(bs.T)).t()
    Q.force_config(variant)
    c = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    Q.fp8_mm(a_t, b_t, as_t, bs_t, c)
    assert Q.last_config() == variant + "_tn", Q.last_config()
    assert_close(host(c), ref, what=Q.last_config())
    Q.set_option("kmajor", 0)
    c2 = torch.zeros_like(c)
    Q.fp8_mm(a_t, b_t, as_t, bs_t, c2)
    assert not Q.last_config().endswith("_tn")
    assert_close(host(c), host(c2), rtol=1e-4, atol=1e-4, what="native against transposed")


def test_fp8_mm_reference_layout_native_exact_and_split():
    """Small-integer operands and power-of-two scales: every product and sum is exact, so the K-major path has
    to give the oracle's bits whatever the order inside an MFMA; also with K split over workgroups."""
    M, N, K = 96, 160, 1024
    say("fp8_mm reference layout, native, exact")
    rng = np.random.default_rng(9)
    a = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
    b = rng.integers(-3, 4, size=(N, K)).astype(np.float32)
    as_ = (2.0 ** rng.integers(-3, 4, size=(M, K // 128))).astype(np.float32)
    bs = (2.0 ** rng.integers(-3, 4, size=((N + 127) // 128, K // 128))).astype(np.float32)
    ref = R.gemm_fp8_block(a, b, as_, bs)
    a_t = fp8_tensor(np.ascontiguousarray(R.encode_fp8(a).T)).t()
    b_t = fp8_tensor(np.ascontiguousarray(R.encode_fp8(b).T)).t()
    as_t, bs_t = dev(np.ascontiguousarray(as_.T)).t(), dev(np.ascontiguousarray(bs.T)).t()
    for split in (0, 2, 4):
        Q.set_option("force_split", split)
        c = torch.zeros((M, N), dtype=torch.float32, device="cuda")
        Q.fp8_mm(a_t, b_t, as_t, bs_t, c)
        assert "_tn" in Q.last_config(), Q.last_config()
        assert np.array_equal(host(c), ref), Q.last_config()


def test_fp8_mm_dispatch_errors_like_the_reference():
    """hip_mix_gemm_kernel.cpp:460,485,503: dimensions not divisible by 32 throw."""
    say("fp8_mm errors")
    z = torch.zeros(1, device="cuda")
    for (m, n, k), status in (((48, 64, 128), 6), ((64, 48, 128), 7), ((64, 64, 80), 8)):
        a = torch.zeros((k, m), dtype=torch.uint8, device="cuda").view(torch.float8_e4m3fn).t()
        b = torch.zeros((k, n), dtype=torch.uint8, device="cuda").view(torch.float8_e4m3fn).t()
        c = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
        with pytest.raises(Q.QgemmError) as e:
            Q.fp8_mm(a, b, z, z, c)
        assert e.value.status == status and "not divisible" in str(e.value)


@pytest.mark.parametrize("shape", [(64, 64, 100), (32, 96, 168), (33, 17, 50)])
def test_any_shape_kernel_k_not_multiple_of_16(shape):
    M, N, K = shape
    say("any-shape", shape)
    qa, sa, qb, sb = int8_inputs(M, N, K, seed=41)
    c = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    Q.int8_mm(dev(qa), dev(qb), scalar(sa), scalar(sb), c)
    assert Q.last_config() == "strided_any_shape"
    assert np.array_equal(host(c), R.gemm_i8_i32(qa, qb))
    qa, sa, qb, sb = fp8_inputs(M, N, K, seed=42)
    if M % 32 == 0 and N % 32 == 0:
        as_ = R.fill_uniform((M, (K + 127) // 128), 43, 0.5, 2.0) / np.float32(448)
        bs = R.fill_uniform(((N + 127) // 128, (K + 127) // 128), 44, 0.5, 2.0) / np.float32(448)
        ref = R.gemm_fp8_block(R.decode_fp8(qa), R.decode_fp8(qb), as_, bs)      # bk by the reference's dispatch
        cb = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
        Q.scaled_gemm(fp8_tensor(qa), fp8_tensor(qb), dev(as_), dev(bs), cb, M, N, K, Q.SCALE_BLOCK128)
        assert_close(host(cb), ref)
    ref = R.gemm_f32acc(R.decode_fp8(qa), R.decode_fp8(qb)) * np.float32(sa * sb)
    cf = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    Q.scaled_gemm(fp8_tensor(qa), fp8_tensor(qb), scalar(sa), scalar(sb), cf, M, N, K, Q.SCALE_PER_MATRIX)
    assert_close(host(cf), ref)


@pytest.mark.parametrize("nsplit", [2, 4])
def test_fp8_split_k(nsplit):
    M, N, K = 16, 512, 2048
    say("fp8 split-k", nsplit)
    qa, sa, qb, sb = fp8_inputs(M, N, K, seed=51)
    ref = R.gemm_f32acc(R.decode_fp8(qa), R.decode_fp8(qb)) * np.float32(sa * sb)
    c = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    Q.scaled_gemm(fp8_tensor(qa), fp8_tensor(qb), scalar(sa), scalar(sb), c, M, N, K, Q.SCALE_PER_MATRIX,
                  split_k=nsplit)
    assert "splitk" in Q.last_config()
    assert_close(host(c), ref)
    # block-scaled + split: partial planes are already scaled
    as_ = R.fill_uniform((M, K // 128), 52, 0.5, 2.0) / np.float32(448)
    bs = R.fill_uniform((N // 128, K // 128), 53, 0.5, 2.0) / np.float32(448)
    refb = R.gemm_fp8_block(R.decode_fp8(qa), R.decode_fp8(qb), as_, bs)
    Q.scaled_gemm(fp8_tensor(qa), fp8_tensor(qb), dev(as_), dev(bs), c, M, N, K, Q.SCALE_BLOCK128, split_k=nsplit)
    assert_close(host(c), refb)


def _stratified_f32():
    """fp32 bit patterns that exercise a narrowing conversion: NaNs, infinities, zeros, fp32 subnormals, exact ties
    of the bf16 rounding (low half 0x8000 under an even and an odd upper half) and their neighbours, the fp16
    overflow boundary (65504, 65520 and neighbours), the fp16 subnormal range with its ties, and random patterns
    of every exponent."""
    rng = np.random.default_rng(2024)
    bits = [0x7FC00000, 0xFFC00000, 0x7F800001, 0x7FFFFFFF, 0x7F800000, 0xFF800000, 0x00000000, 0x80000000,
            0x00000001, 0x80000001, 0x007FFFFF, 0x00008000, 0x00018000, 0x7F7FFFFF, 0xFF7FFFFF, 0x7F7F8000, 0x7F7F7FFF]
    for upper in (0x3F80, 0x3F81, 0x4049, 0xC2F7, 0x0001, 0x0002, 0x7F7E):
        for low in (0x7FFF, 0x8000, 0x8001, 0x0000, 0xFFFF):
            bits.append((upper << 16) | low)
    for v in (65504.0, 65519.996, 65520.0, 65536.0, 1e9, -65519.996, -65520.0):
        bits.append(int(np.float32(v).view(np.uint32)))
    for e in range(-26, -13):                       # fp16 subnormals and the smallest normals: quarter steps and ties
        for m in (1.0, 1.25, 1.5, 1.75, 1.0009765625, 1.00048828125, 1.001464843750):
            for sgn in (1.0, -1.0):
                bits.append(int(np.float32(sgn * m * 2.0 ** e).view(np.uint32)))
    rnd = rng.integers(0, 1 << 32, size=3600, dtype=np.uint64).astype(np.uint32)
    all_bits = np.concatenate([np.array(bits, np.uint64).astype(np.uint32), rnd])
    return all_bits.view(np.float32)


@pytest.mark.parametrize("variant", [None, "256x256_w2x4_solo8", "128x128_w2x2_dma", "skinny_128x32_k8", "256x128_w2x2_cw"])
def test_epilogue_conversions_match_the_oracle_codecs(variant):
    """The float -> bf16 / fp16 conversion of the epilogues (f32_to_bf16_bits / f32_to_f16_bits, csrc/common.h: the
    NaN-guarded form of src/include/fast_quat.h:3-12) on a stratified fp32 sample, bit for bit against the oracle's
    codecs.  The sample travels as a_scale of a block-scaled GEMM whose only product per row is 1.0 * 1.0, so that
    the accumulator the epilogue converts is exactly the sample value (fma(1, x, 0) = x)."""
    x = _stratified_f32()
    M, N, K = len(x), 128, 128
    say("epilogue conversions", (M, N, K), "variant", variant)
    qa = np.zeros((M, K), np.uint8)
    qa[:, 0] = 0x38                                  # 1.0
    qb = np.zeros((N, K), np.uint8)
    qb[:, 0] = 0x38
    as_ = x.reshape(M, 1).copy()
    bs = np.ones((1, 1), np.float32)
    with np.errstate(all="ignore"):
        acc = x + np.float32(0.0)                    # what the fold leaves: -0 becomes +0, everything else is itself
    nan = np.isnan(acc)
    Q.force_config(variant)
    for dt, enc in ((torch.bfloat16, R.encode_bf16), (torch.float16, R.encode_f16), (torch.float32, None)):
        c = torch.zeros((M, N), dtype=dt, device="cuda")
        Q.scaled_gemm(fp8_tensor(qa), fp8_tensor(qb), dev(as_), dev(bs), c, M, N, K, Q.SCALE_BLOCK128, split_k=1)
        torch.cuda.synchronize()
        if enc is None:
            got = c.cpu().numpy()
            assert np.array_equal(got[~nan].view(np.uint32), np.broadcast_to(acc[:, None], got.shape)[~nan].view(np.uint32))
            assert np.all(np.isnan(got[nan]))
            continue
        got = c.view(torch.int16).cpu().numpy().view(np.uint16)
        want = enc(acc)
        bad = (got[~nan] != want[~nan, None])
        assert not bad.any(), (Q.last_config(), dt, [hex(int(v)) for v in acc[~nan].view(np.uint32)[np.nonzero(bad.any(axis=1))[0][:8]]])
        # NaN in, NaN out (payload free): exponent all ones, mantissa non-zero
        g = got[nan].astype(np.uint32)
        if dt == torch.bfloat16:
            assert np.all(((g & 0x7F80) == 0x7F80) & ((g & 0x007F) != 0))
        else:
            assert np.all(((g & 0x7C00) == 0x7C00) & ((g & 0x03FF) != 0))


def test_rotated_k_start_changes_only_the_summation_order():
    """With at most 256 rows the workgroups of column tile i start their K loops 3 i steps in (option "k_rot"): the
    same products summed in another order.  Random fp8 data: with and without the rotation the results agree to the
    stated tolerance with the oracle and to a few fp32 ulps of the sum's magnitude with each other; identical rows of
    A against identical columns of B give identical bits at every column position only with k_rot = 0."""
    M, N, K = 64, 1024, 4096
    say("k_rot on / off", (M, N, K))
    qa, sa, qb1, sb = fp8_inputs(M, 128, K, seed=77)
    qb = np.tile(qb1, (N // 128, 1))                 # every 128-column block of B holds the same columns
    ref = R.gemm_f32acc(R.decode_fp8(qa), R.decode_fp8(qb)) * np.float32(sa * sb)
    out = {}
    for rot in (-1, 0):
        Q.set_option("k_rot", rot)
        c = torch.zeros((M, N), dtype=torch.float32, device="cuda")
        Q.scaled_gemm(fp8_tensor(qa), fp8_tensor(qb), scalar(sa), scalar(sb), c, M, N, K, Q.SCALE_PER_MATRIX)
        out[rot] = host(c)
        assert_close(out[rot], ref, what=f"k_rot {rot} {Q.last_config()}")
    Q.set_option("k_rot", -1)
    assert np.max(np.abs(out[-1] - out[0])) <= 1e-4 * np.max(np.abs(ref))
    blocks0 = out[0].reshape(M, N // 128, 128)
    assert np.array_equal(blocks0, np.broadcast_to(blocks0[:, :1], blocks0.shape))     # position-independent sums


# ---------------------------------------------------------- plain fp16 / bf16
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("layout_b", ["nk", "kn"])
@pytest.mark.parametrize("shape", [(256, 256, 256), (136, 200, 192)])
def test_plain_gemm_16bit(dtype, layout_b, shape):
    M, N, K = shape
    say("plain", dtype, layout_b, shape)
    enc, dec, tdt = ((R.encode_f16, R.decode_f16, torch.float16) if dtype == "f16"
                     else (R.encode_bf16, R.decode_bf16, torch.bfloat16))
    ha, hb = enc(R.fill_uniform((M, K), 61)), enc(R.fill_uniform((N, K), 62))     # cfg 1: uniform[-1, 1]
    ref = R.gemm_f32acc(dec(ha), dec(hb))
    a = dev(ha.view(np.int16)).view(tdt)
    b_nk = dev(hb.view(np.int16)).view(tdt)
    b = b_nk if layout_b == "nk" else b_nk.t().contiguous()
    for out_dt in (tdt, torch.float32):
        c = torch.zeros((M, N), dtype=out_dt, device="cuda")
        Q.gemm(a, b, c, layout_b)
        got = host(c).astype(np.float32) if out_dt != torch.bfloat16 else host(c)
        # 16-bit output: half an ulp of the output type on top of the accumulation-order slack
        rtol = 2.0 ** -8 if out_dt == torch.bfloat16 else (2.0 ** -10 if out_dt == torch.float16 else 1e-5)
        assert_close(got, ref, rtol=rtol, atol=1e-3, what=f"{Q.last_config()} {out_dt}")


@pytest.mark.parametrize("dtype,variant", PAIRS_16)
def test_plain_gemm_16bit_every_variant(dtype, variant):
    """Every tile variant on 16-bit operands (the big tiles use the 32 x 32 x 16 MFMA and their own fragment and
    accumulator layouts): small integers, so sums are exact and the bits must equal numpy's integer product,
    ragged M and N, 16-bit and fp32 outputs."""
    M, N, K = 300, 328, 384
    say("plain 16-bit", dtype, "variant", variant)
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    rng = np.random.default_rng(40 + ROWS_16[dtype].index(variant))
    a = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
    b = rng.integers(-4, 5, size=(N, K)).astype(np.float32)
    ref = (a.astype(np.int64) @ b.astype(np.int64).T).astype(np.float32)       # |ref| <= 16 * 384: exact in fp32
    Q.force_config(variant)
    c = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    Q.gemm(torch.from_numpy(a).cuda().to(tdt), torch.from_numpy(b).cuda().to(tdt), c, "nk")
    assert np.array_equal(host(c), ref), Q.last_config()
    # a row-aligned shape takes the vectorised way out; 16-bit output (values up to 2^8 * 24 are exact in neither
    # type in general: compare against the rounded reference)
    M2, N2 = 256, 512
    c2 = torch.zeros((M2, N2), dtype=tdt, device="cuda")
    a2 = rng.integers(-2, 3, size=(M2, K)).astype(np.float32)
    b2 = rng.integers(-2, 3, size=(N2, K)).astype(np.float32)
    Q.gemm(torch.from_numpy(a2).cuda().to(tdt), torch.from_numpy(b2).cuda().to(tdt), c2, "nk")
    ref2 = torch.from_numpy((a2.astype(np.int64) @ b2.astype(np.int64).T).astype(np.float32)).to(tdt)
    assert torch.equal(c2.cpu(), ref2), Q.last_config()


@pytest.mark.parametrize("dtype,variant", PAIRS_16_NN)
def test_plain_gemm_nn_native_every_variant(dtype, variant):
    """GEMM_kernel_v1..v5 storage (B is K x N, include/gemm.h:25-66) read as it lies through the K-major B tile,
    every tile variant, ragged M and N, a padded leading dimension of B, against the oracle."""
    M, N, K, ldB = 200, 264, 320, 272
    say("plain NN native", dtype, "variant", variant)
    enc, dec, tdt = ((R.encode_f16, R.decode_f16, torch.float16) if dtype == "f16"
                     else (R.encode_bf16, R.decode_bf16, torch.bfloat16))
    ha, hb = enc(R.fill_uniform((M, K), 71 + ROWS_16_NN[dtype].index(variant))), enc(R.fill_uniform((K, N), 72))
    ref = R.gemm_f32acc(dec(ha), dec(hb), "nn")
    a = dev(ha.view(np.int16)).view(tdt)
    b_pad = torch.full((K, ldB), 7.0, dtype=tdt, device="cuda")          # columns N .. ldB-1 must never matter
    b_pad[:, :N] = dev(hb.view(np.int16)).view(tdt)
    Q.force_config(variant)
    c = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    Q.gemm(a, b_pad[:, :N], c, "kn")
    assert Q.last_config() == variant + "_nn", Q.last_config()
    assert_close(host(c), ref, rtol=1e-5, atol=1e-3, what=Q.last_config())
    # the route through the transpose utility needs ldB == N
    Q.set_option("kmajor", 0)
    c2 = torch.zeros_like(c)
    Q.gemm(a, b_pad[:, :N].contiguous(), c2, "kn")
    assert not Q.last_config().endswith("_nn")
    assert_close(host(c), host(c2), rtol=1e-5, atol=1e-4, what="native against transposed")


def test_plain_gemm_nn_native_exact_integers():
    """Small integers: exact in bf16 and in the fp32 sums, so the bits must match numpy's integer product."""
    M, N, K = 256, 384, 512
    say("plain NN native, exact")
    rng = np.random.default_rng(12)
    a = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
    b = rng.integers(-4, 5, size=(K, N)).astype(np.float32)
    ref = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    for split in (0, 3):
        Q.set_option("force_split", split)
        c = torch.zeros((M, N), dtype=torch.float32, device="cuda")
        Q.gemm(torch.from_numpy(a).cuda().bfloat16(), torch.from_numpy(b).cuda().bfloat16(), c, "kn")
        assert "_nn" in Q.last_config(), Q.last_config()
        assert np.array_equal(host(c), ref), Q.last_config()


def test_plain_gemm_reference_pattern_inputs():
    """The harness's closed-form inputs and check (tests/includes/test_config.h:251-258, 161-169):
    bf16 in, fp32 out, NN layout, max |C - ref| < 5e-2."""
    M = N = K = 256
    say("pattern inputs", (M, N, K))
    ha = R.encode_bf16(R.fill_pattern((M, K), 0))
    hb = R.encode_bf16(R.fill_pattern((K, N), 1))
    ref = R.gemm_f32acc(R.decode_bf16(ha), R.decode_bf16(hb), "nn")
    c = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    Q.gemm(dev(ha.view(np.int16)).view(torch.bfloat16), dev(hb.view(np.int16)).view(torch.bfloat16), c, "kn")
    assert R.max_abs_diff(host(c), ref) < 5e-2


# ------------------------------------------------------------------ transpose
@pytest.mark.parametrize("dt", [torch.uint8, torch.int16, torch.float32])
@pytest.mark.parametrize("shape", [(64, 32), (128, 256), (100, 36), (1, 77), (1024, 1024), (48, 100), (400, 260),
                                   (8, 8), (72, 264), (264, 8), (520, 72)])
def test_transpose(dt, shape):
    M, N = shape
    say("transpose", dt, shape)
    lo, hi = {torch.uint8: (0, 256), torch.int16: (-32768, 32768)}.get(dt, (0, 30000))
    a = np.random.default_rng(1).integers(lo, hi, size=(M, N))
    x = torch.from_numpy(a).to(dt).cuda()
    y = torch.zeros((N, M), dtype=dt, device="cuda")
    Q.matrix_transpose(x, y)
    assert torch.equal(y, x.t().contiguous())
    assert np.array_equal(host(y), R.transpose(host(x)))
    back = torch.zeros_like(x)
    Q.matrix_transpose(y, back)
    assert torch.equal(back, x)                      # involution


def test_empty_and_invalid_arguments():
    say("empty / invalid")
    z = torch.zeros((0, 16), dtype=torch.int8, device="cuda")
    b = torch.zeros((16, 16), dtype=torch.int8, device="cuda")
    c = torch.zeros((0, 16), dtype=torch.int32, device="cuda")
    Q.int8_mm(z, b, scalar(1), scalar(1), c)          # M == 0: nothing to do, no error
    with pytest.raises(Q.QgemmError) as e:            # int32 output is only defined for int8 input
        Q.scaled_gemm(b.view(torch.float8_e4m3fn), b.view(torch.float8_e4m3fn), scalar(1), scalar(1),
                      torch.zeros((16, 16), dtype=torch.int32, device="cuda"), 16, 16, 16, Q.SCALE_PER_MATRIX)
    assert e.value.status == 2
    with pytest.raises(ValueError):
        Q.int8_mm(torch.zeros((16, 16), dtype=torch.int8), b, scalar(1), scalar(1), c)   # host tensor
