"""Pins the CPU oracle (oracle/cpu_ref.c) against closed forms, library casts
and brute force, so that a dropped term, wrong index or transposed operand in
the oracle fails here before the oracle is trusted to judge the GPU path.

The reference holds no golden vectors for this path (its only oracle is
cuBLAS on a GPU, tests/includes/test_config.h:29-52); what it does fix is the
closed-form input pattern (:251-258), reproduced below."""
import numpy as np
import pytest
import torch

from oracle import cpu_ref as R


# ------------------------------------------------------------------ fp8 codec
def _e4m3_table():
    """OCP e4m3 written from the format definition: 1-4-3, bias 7."""
    t = np.zeros(256, np.float64)
    for b in range(256):
        s = -1.0 if b & 0x80 else 1.0
        e, m = (b >> 3) & 0xF, b & 7
        if e == 15 and m == 7:
            t[b] = np.nan
        elif e == 0:
            t[b] = s * m * 2.0 ** -9
        else:
            t[b] = s * (1 + m / 8.0) * 2.0 ** (e - 7)
    return t


def test_fp8_decode_table_closed_form():
    t = _e4m3_table()
    got = R.decode_fp8(np.arange(256, dtype=np.uint8)).astype(np.float64)
    assert np.array_equal(np.isnan(t), np.isnan(got))
    ok = ~np.isnan(t)
    assert np.array_equal(t[ok], got[ok])
    assert got[0x7E] == 448.0 and got[0xFE] == -448.0 and got[0x08] == 2.0 ** -6 and got[0x01] == 2.0 ** -9


def test_fp8_decode_matches_torch_e4m3fn():
    codes = torch.arange(256, dtype=torch.uint8)
    ref = codes.view(torch.float8_e4m3fn).to(torch.float32).numpy()
    got = R.decode_fp8(codes.numpy())
    ok = ~np.isnan(ref)
    assert np.array_equal(np.isnan(ref), np.isnan(got))
    assert np.array_equal(ref[ok], got[ok])


def test_fp8_encode_roundtrip_every_finite_code():
    codes = np.array([b for b in range(256) if (b & 0x7F) != 0x7F], np.uint8)
    vals = R.decode_fp8(codes)
    back = R.encode_fp8(vals)
    # -0.0 keeps its sign bit
    assert np.array_equal(back, codes)


def test_fp8_encode_ties_to_even_and_saturation():
    t = _e4m3_table()
    pos = np.array([b for b in range(0x7F)], np.uint8)
    v = t[pos]
    mids = (v[:-1] + v[1:]) / 2            # exact in double, and in float (<= 5 significant bits)
    enc = R.encode_fp8(mids.astype(np.float32))
    expect = np.where(pos[:-1] % 2 == 0, pos[:-1], pos[1:])
    assert np.array_equal(enc, expect)
    eps = np.float32(1.0) + np.float32(2.0 ** -20)
    assert np.array_equal(R.encode_fp8((mids * eps).astype(np.float32)), pos[1:])
    assert np.array_equal(R.encode_fp8((mids / eps).astype(np.float32)), pos[:-1])
    # clamp-then-round: everything at or above 448 (inf included) saturates, NaN stays NaN
    x = np.array([448, 449, 463.9, 464, 500, 1e9, np.inf, -460, -np.inf], np.float32)
    assert np.array_equal(R.encode_fp8(x), np.array([0x7E] * 7 + [0xFE] * 2, np.uint8))
    assert R.encode_fp8(np.array([np.nan], np.float32))[0] & 0x7F == 0x7F


def test_fp8_encode_matches_torch_below_saturation():
    x = R.fill_uniform((1 << 16,), seed=7, lo=-448.0, hi=448.0)
    x = np.concatenate([x, R.fill_uniform((1 << 14,), seed=8, lo=-0.05, hi=0.05)])
    ref = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(R.encode_fp8(x), ref)


def test_fp8_encode_monotone():
    x = np.sort(R.fill_uniform((1 << 15,), seed=9, lo=0.0, hi=500.0))
    d = R.decode_fp8(R.encode_fp8(x))
    assert np.all(np.diff(d) >= 0)


# ------------------------------------------------------------ bf16 / fp16 codec
def _strat_sample(n, seed):
    bits = np.random.default_rng(seed).integers(0, 1 << 32, size=n, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    return x[np.isfinite(x)]


def test_bf16_encode_matches_torch():
    x = _strat_sample(1 << 18, 1)
    ref = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(R.encode_bf16(x), ref)
    assert np.array_equal(R.decode_bf16(ref), torch.from_numpy(x).to(torch.bfloat16).float().numpy())
    # the bit trick of fast_quat.h on a hand case: 1 + 2^-8 is a tie -> even (1.0); 1 + 3*2^-8 -> 1 + 2^-6
    assert R.encode_bf16(np.array([1 + 2.0 ** -8, 1 + 3 * 2.0 ** -8], np.float32)).tolist() == [0x3F80, 0x3F82]
    assert np.isnan(R.decode_bf16(R.encode_bf16(np.array([np.nan], np.float32))))[0]


def test_f16_codec_matches_numpy():
    x = _strat_sample(1 << 18, 2)
    x = np.concatenate([x, R.fill_uniform((1 << 16,), 3, -70000.0, 70000.0), R.fill_uniform((1 << 16,), 4, -1e-4, 1e-4)])
    with np.errstate(over="ignore"):
        ref = x.astype(np.float16)
    assert np.array_equal(R.encode_f16(x), ref.view(np.uint16))
    allh = np.arange(1 << 16, dtype=np.uint16)
    got = R.decode_f16(allh)
    exp = allh.view(np.float16).astype(np.float32)
    ok = ~np.isnan(exp)
    assert np.array_equal(got[ok], exp[ok]) and np.array_equal(np.isnan(got), np.isnan(exp))


# ------------------------------------------------------------------- inputs
def test_pattern_inputs_closed_form():
    # tests/includes/test_config.h:251-258
    i = np.arange(5000)
    a = ((i % 43).astype(np.float32).astype(np.float64) / 20.0 + 0.2 + (i % 19)).astype(np.float32)
    b = ((i % 43).astype(np.float32).astype(np.float64) / 20.0 + 0.2 + (i % 37)).astype(np.float32)
    assert np.array_equal(R.fill_pattern((5000,), 0), a)
    assert np.array_equal(R.fill_pattern((5000,), 1), b)
    assert R.fill_pattern((1,), 0)[0] == np.float32(0.2)


def test_prng_is_counter_based_and_sane():
    a = R.fill_uniform((1000,), seed=42)
    b = R.fill_uniform((2000,), seed=42)
    assert np.array_equal(a, b[:1000])                 # value i depends on (seed, i) only
    assert not np.array_equal(a, R.fill_uniform((1000,), seed=43))
    assert a.min() >= -1.0 and a.max() < 1.0
    n = R.fill_normal((1 << 18,), seed=42)
    assert abs(n.mean()) < 0.01 and abs(n.std() - 1.0) < 0.01
    assert np.array_equal(n[:100], R.fill_normal((100,), seed=42))
    R.set_num_threads(1)
    n1 = R.fill_normal((1 << 12,), seed=5)
    R.set_num_threads(8)
    assert np.array_equal(n1, R.fill_normal((1 << 12,), seed=5))


# --------------------------------------------------------------- quantisers
def test_quantize_int8_closed_form():
    x = R.fill_normal((257, 131), seed=11)
    q, s = R.quantize_int8(x)
    assert s == np.float32(np.abs(x).max()) / np.float32(127.0)
    exp = np.clip(np.rint(x / s), -127, 127).astype(np.int8)   # np.rint: ties to even
    assert np.array_equal(q, exp)
    assert np.all(np.abs(x - s * q.astype(np.float32)) <= s / 2 * (1 + 1e-6))
    assert np.abs(q).max() == 127
    t = np.array([0.5, 1.5, 2.5, -0.5, -1.5, 127.0], np.float32)  # s == 1 exactly
    assert R.quantize_int8(t)[0].tolist() == [0, 2, 2, 0, -2, 127]


def test_quantize_fp8_per_matrix_and_block():
    x = R.fill_normal((256, 384), seed=12)
    q, s = R.quantize_fp8(x)
    assert s == np.float32(np.abs(x).max()) / np.float32(448.0)
    assert np.array_equal(q, R.encode_fp8(x / s))
    assert R.decode_fp8(q).__abs__().max() == 448.0
    qb, sb = R.quantize_fp8_block(x, 128, 128)
    assert sb.shape == (2, 3)
    for i in range(2):
        for j in range(3):
            blk = x[i * 128:(i + 1) * 128, j * 128:(j + 1) * 128]
            assert sb[i, j] == np.float32(np.abs(blk).max()) / np.float32(448.0)
            assert np.array_equal(qb[i * 128:(i + 1) * 128, j * 128:(j + 1) * 128], R.encode_fp8(blk / sb[i, j]))
    qa, sa = R.quantize_fp8_block(x, 1, 128)
    assert sa.shape == (256, 3)
    assert sa[5, 2] == np.float32(np.abs(x[5, 256:]).max()) / np.float32(448.0)


# ---------------------------------------------------------------- transpose
def test_transpose_is_numpy_T_and_involution():
    for dt in (np.uint8, np.uint16, np.float32):
        a = np.random.default_rng(0).integers(0, 200, size=(96, 160)).astype(dt)
        t = R.transpose(a)
        assert np.array_equal(t, a.T)
        assert np.array_equal(R.transpose(t), a)


# ----------------------------------------------------------------- int8 GEMM
def _brute_i32(A, B):
    M, K = A.shape
    N = B.shape[0]
    out = np.zeros((M, N), np.int64)
    for m in range(M):
        for n in range(N):
            s = 0
            for k in range(K):
                s += int(A[m, k]) * int(B[n, k])
            out[m, n] = s
    return out


def test_int8_gemm_bruteforce_and_layouts():
    rng = np.random.default_rng(3)
    A = rng.integers(-127, 128, size=(5, 19), dtype=np.int8)
    B = rng.integers(-127, 128, size=(7, 19), dtype=np.int8)
    exp = _brute_i32(A, B)
    assert np.array_equal(R.gemm_i8_i32(A, B, "nt"), exp)
    assert np.array_equal(R.gemm_i8_i32(A, np.ascontiguousarray(B.T), "nn"), exp)
    assert np.array_equal(R.gemm_i8_i32(np.ascontiguousarray(A.T), np.ascontiguousarray(B.T), "tn"), exp)
    # a transposed-operand mistake cannot hide: M != N != K and A != B
    assert not np.array_equal(exp[:5, :5], exp[:5, :5].T)


def test_int8_gemm_identities_and_extremes():
    K = 8192
    A = np.full((2, K), 127, np.int8)
    B = np.full((3, K), -127, np.int8)
    assert np.all(R.gemm_i8_i32(A, B) == -127 * 127 * K)          # largest magnitude stays inside int32
    assert 127 * 127 * 8192 < 2 ** 31
    ones = np.ones((4, 300), np.int8)
    assert np.all(R.gemm_i8_i32(ones, ones) == 300)
    eye = np.eye(64, dtype=np.int8)
    Bm = np.random.default_rng(1).integers(-127, 128, size=(48, 64), dtype=np.int8)
    assert np.array_equal(R.gemm_i8_i32(eye, Bm), Bm.T.astype(np.int32))
    # any K split sums to the same integers
    A = np.random.default_rng(2).integers(-127, 128, size=(16, 512), dtype=np.int8)
    Bk = np.random.default_rng(4).integers(-127, 128, size=(24, 512), dtype=np.int8)
    full = R.gemm_i8_i32(A, Bk)
    parts = sum(R.gemm_i8_i32(A[:, s:s + 128], Bk[:, s:s + 128]) for s in range(0, 512, 128))
    assert np.array_equal(full, parts)
    assert np.array_equal(full, A.astype(np.int64) @ Bk.astype(np.int64).T)


def test_int8_scale_epilogue_single_roundings():
    acc = np.array([[123456789, -7, 0, 2 ** 31 - 1]], np.int32)
    sa, sb = np.float32(0.0123), np.float32(0.0456)
    exp = acc.astype(np.float32) * np.float32(sa * sb)
    assert np.array_equal(R.scale_i32_to_f32(acc, sa, sb), exp)


# ------------------------------------------------------------------- fp GEMM
def test_fp_gemm_exact_on_representable_inputs_and_layouts():
    rng = np.random.default_rng(5)
    A = rng.integers(-8, 9, size=(9, 40)).astype(np.float32)
    B = rng.integers(-8, 9, size=(11, 40)).astype(np.float32)
    exp = (A.astype(np.float64) @ B.astype(np.float64).T)
    for fn in (R.gemm_f32acc, R.gemm_f64acc):
        assert np.array_equal(fn(A, B, "nt"), exp)
        assert np.array_equal(fn(A, np.ascontiguousarray(B.T), "nn"), exp)
        assert np.array_equal(fn(np.ascontiguousarray(A.T), np.ascontiguousarray(B.T), "tn"), exp)


def test_fp_gemm_f32acc_within_bound_of_f64():
    A = R.fill_uniform((32, 1024), 21)
    B = R.fill_uniform((48, 1024), 22)
    c32 = R.gemm_f32acc(A, B).astype(np.float64)
    c64 = R.gemm_f64acc(A, B)
    assert np.allclose(c64, A.astype(np.float64) @ B.astype(np.float64).T, rtol=0, atol=1e-9)
    bound = 1024 * 2.0 ** -24 * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64).T)
    assert np.all(np.abs(c32 - c64) <= bound)


def test_fp_gemm_pattern_inputs_small_case():
    # the harness's own inputs (test_config.h:251-258), bf16-rounded as typeIn = bf16 does
    M = N = K = 64
    A = R.decode_bf16(R.encode_bf16(R.fill_pattern((M, K), 0)))
    B = R.decode_bf16(R.encode_bf16(R.fill_pattern((K, N), 1)))
    c = R.gemm_f32acc(A, B, "nn")
    ref = (torch.from_numpy(A).double() @ torch.from_numpy(B).double()).numpy()
    assert np.max(np.abs(c - ref)) < 5e-2          # the harness tolerance, test_config.h:64


# ------------------------------------------------------------- block-scaled
def _fp8_vals(shape, seed):
    return R.decode_fp8(R.quantize_fp8(R.fill_normal(shape, seed))[0])


def test_block_scaled_bruteforce_reference_order():
    M, N, K = 32, 256, 256
    A, B = _fp8_vals((M, K), 31), _fp8_vals((N, K), 32)
    as_ = R.fill_uniform((M, K // 128), 33, 0.5, 2.0)
    bs = R.fill_uniform((N // 128, K // 128), 34, 0.5, 2.0)
    got = R.gemm_fp8_block(A, B, as_, bs)
    exp = np.zeros((M, N), np.float32)
    for m in range(0, M, 7):                    # brute force a lattice of entries in pure python floats
        for n in range(0, N, 13):
            acc = np.float32(0)
            for kb in range(K // 128):
                p = np.float32(0)
                for k in range(kb * 128, kb * 128 + 128):
                    p = np.float32(p + np.float32(A[m, k] * B[n, k]))
                acc = np.float32(acc + np.float32(np.float32(p * as_[m, kb]) * bs[n // 128, kb]))
            assert got[m, n] == acc
    f64 = R.gemm_fp8_block_f64(A, B, as_, bs)
    assert np.allclose(got, f64, rtol=2e-5, atol=1.0)
    # a transposed scale index must show: as varies along m, bs along n-blocks
    assert not np.allclose(got, R.gemm_fp8_block(A, B, as_[::-1].copy(), bs), rtol=1e-3)
    assert not np.allclose(got, R.gemm_fp8_block(A, B, as_, bs[::-1].copy()), rtol=1e-3)


def test_block_scaled_reductions():
    M, N, K = 32, 128, 384
    A, B = _fp8_vals((M, K), 41), _fp8_vals((N, K), 42)
    one_a, one_b = np.ones((M, 3), np.float32), np.ones((1, 3), np.float32)
    plain = R.gemm_fp8_block(A, B, one_a, one_b)
    # scales == 1 -> a plain GEMM accumulated per 128 block
    blocks = sum(R.gemm_f32acc(A[:, s:s + 128], B[:, s:s + 128]).astype(np.float64) for s in range(0, K, 128))
    assert np.allclose(plain, blocks, rtol=2e-5, atol=1.0)       # |c| ~ 1e5: fp32 ulp ~ 1e-2
    assert np.allclose(plain, R.gemm_f64acc(A, B), rtol=2e-5, atol=1.0)
    # power-of-two scales commute exactly with fp32 arithmetic
    assert np.array_equal(R.gemm_fp8_block(A, B, one_a * 4, one_b * 0.5), plain * 2)
    # constant scales == per-matrix scaling
    sa, sb = np.float32(1.37), np.float32(0.61)
    pm = R.gemm_fp8_block(A, B, one_a * sa, one_b * sb).astype(np.float64)
    assert np.allclose(pm, R.gemm_f64acc(A, B) * float(sa) * float(sb), rtol=2e-5, atol=1.0)
    # doubling one K block's scale doubles only that block's contribution (exact in binary fp)
    as2 = one_a.copy()
    as2[:, 1] = 2
    only1 = R.gemm_fp8_block(A[:, 128:256], B[:, 128:256], np.ones((M, 1), np.float32), np.ones((1, 1), np.float32))
    assert np.allclose(R.gemm_fp8_block(A, B, as2, one_b).astype(np.float64), plain.astype(np.float64) + only1,
                       rtol=2e-5, atol=1.0)


def test_block_scaled_reference_layouts_agree():
    M, N, K = 32, 256, 256
    A, B = _fp8_vals((M, K), 51), _fp8_vals((N, K), 52)
    as_ = R.fill_uniform((M, 2), 53, 0.5, 2.0)
    bs = R.fill_uniform((2, 2), 54, 0.5, 2.0)
    nt = R.gemm_fp8_block(A, B, as_, bs, "nt", "row")
    tn = R.gemm_fp8_block(np.ascontiguousarray(A.T), np.ascontiguousarray(B.T), np.ascontiguousarray(as_.T),
                          np.ascontiguousarray(bs.T), "tn", "col")
    assert np.array_equal(nt, tn)


def test_int8_block_scaled_pinned_without_itself():
    """ref_gemm_i8_block (int8 operands, 128-block scales): brute force in Python integers and numpy float32 steps on a
    lattice of entries (a dropped block, a scale taken from the wrong row / K block / column block, or a partial
    converted too late shows); unit scales give the exact int32 GEMM; power-of-two scales commute exactly; equal scales
    are the per-matrix product up to one rounding per block; a partial last K block; both storages agree."""
    M, N, K = 24, 256, 400                              # K: three whole blocks and one of 16
    KB = (K + 127) // 128
    qa = R.quantize_int8(R.fill_normal((M, K), 61))[0]
    qb = R.quantize_int8(R.fill_normal((N, K), 62))[0]
    as_ = R.fill_uniform((M, KB), 63, 0.5, 2.0)
    bs = R.fill_uniform((N // 128, KB), 64, 0.5, 2.0)
    got = R.gemm_i8_block(qa, qb, as_, bs)
    for m in range(0, M, 5):
        for n in range(0, N, 37):
            acc = np.float32(0)
            for kb in range(KB):
                p = sum(int(qa[m, k]) * int(qb[n, k]) for k in range(kb * 128, min(K, kb * 128 + 128)))   # exact
                acc = np.float32(acc + np.float32(np.float32(np.float32(p) * as_[m, kb]) * bs[n // 128, kb]))
            assert got[m, n] == acc, (m, n)
    exact = R.gemm_i8_i32(qa, qb)
    ones_a, ones_b = np.ones((M, KB), np.float32), np.ones((N // 128, KB), np.float32)
    assert np.array_equal(R.gemm_i8_block(qa, qb, ones_a, ones_b), exact.astype(np.float32))     # |acc| < 2^24 here
    assert np.abs(exact).max() < 2 ** 24
    assert np.array_equal(R.gemm_i8_block(qa, qb, ones_a * 8, ones_b * 0.25), exact.astype(np.float32) * 2)
    sa, sb = np.float32(1.37), np.float32(0.61)
    pm = R.gemm_i8_block(qa, qb, ones_a * sa, ones_b * sb).astype(np.float64)
    assert np.allclose(pm, exact.astype(np.float64) * float(sa) * float(sb), rtol=1e-6, atol=1e-2)
    assert not np.allclose(got, R.gemm_i8_block(qa, qb, as_[::-1].copy(), bs), rtol=1e-3)
    assert not np.allclose(got, R.gemm_i8_block(qa, qb, as_, bs[::-1].copy()), rtol=1e-3)
    assert not np.allclose(got, R.gemm_i8_block(qa, qb, as_[:, ::-1].copy(), bs), rtol=1e-3)
    tn = R.gemm_i8_block(np.ascontiguousarray(qa.T), np.ascontiguousarray(qb.T), np.ascontiguousarray(as_.T),
                         np.ascontiguousarray(bs.T), "tn", "col")
    assert np.array_equal(got, tn)


def test_reference_tile_dispatch_and_swizzle():
    # hip_mix_gemm_kernel.cpp:442-505
    assert [R.select_tile(d, "m") for d in (6144, 192, 96, 48)] == [128, 64, 32, 0]
    assert [R.select_tile(d, "n") for d in (4608, 96, 48)] == [64, 32, 0]
    assert [R.select_tile(d, "k") for d in (7168, 192, 96, 40)] == [128, 64, 32, 0]
    for tm, tn, g in ((8, 8, 4), (7, 5, 4), (1, 9, 4), (32, 32, 8)):
        seen = {R.block_swizzle(b, tm, tn, g) for b in range(tm * tn)}
        assert seen == {(i, j) for i in range(tm) for j in range(tn)}
    assert R.block_swizzle(1, 8, 8, 4) == (1, 0) and R.block_swizzle(4, 8, 8, 4) == (0, 1)
