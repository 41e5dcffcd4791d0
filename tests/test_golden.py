"""The committed golden vectors (tests/golden/, written by tests/golden/make_golden.py from
numpy's closed forms and float64 / int64 brute force, independent of the oracle and of the
HIP library) against the CPU oracle -- and, in the GPU half, against the HIP path through
the C ABI.  The reference itself holds no vectors for this path."""
import json
import os

import numpy as np
import pytest

from oracle import cpu_ref as R

HERE = os.path.dirname(os.path.abspath(__file__))
G = np.load(os.path.join(HERE, "golden", "gemm_cases.npz"), allow_pickle=False)
RTOL, ATOL = 2e-2, 1e-2


def _table():
    with open(os.path.join(HERE, "golden", "fp8_e4m3_decode.json")) as f:
        return np.array([np.nan if v is None else v for v in json.load(f)["decode"]], np.float64)


def test_golden_fp8_decode_table():
    t = _table()
    got = R.decode_fp8(np.arange(256, dtype=np.uint8)).astype(np.float64)
    assert np.array_equal(np.isnan(got), np.isnan(t))
    assert np.array_equal(got[~np.isnan(t)], t[~np.isnan(t)])
    assert t[0x7E] == 448.0 and t[0x01] == 2.0 ** -9 and np.isnan(t[0x7F]) and np.isnan(t[0xFF])


def test_golden_int8():
    acc = R.gemm_i8_i32(G["i8_a"], G["i8_b"])
    assert np.array_equal(acc, G["i8_c"])
    sa, sb = G["i8_scales"]
    c = R.scale_i32_to_f32(acc, sa, sb)
    assert np.array_equal(c.astype(np.float64), G["i8_c"].astype(np.float64) * float(sa) * float(sb))


def test_golden_fp8_per_matrix():
    sa, sb = G["f8_scales"]
    c = R.gemm_f32acc(R.decode_fp8(G["f8_a"]), R.decode_fp8(G["f8_b"])).astype(np.float64) * (float(sa) * float(sb))
    ref = G["f8_c"]
    # fp32 accumulation of K = 256 exact products: a few ulp of the largest partial sum
    assert np.max(np.abs(c - ref)) <= 1e-5 * np.max(np.abs(ref))


def test_golden_fp8_block_reference_storage():
    c = R.gemm_fp8_block(R.decode_fp8(G["blk_a"]), R.decode_fp8(G["blk_b"]), G["blk_as"], G["blk_bs"], "tn", "col")
    ref = G["blk_c"]
    assert np.max(np.abs(c - ref)) <= 1e-5 * np.max(np.abs(ref))
    c64 = R.gemm_fp8_block_f64(R.decode_fp8(G["blk_a"]), R.decode_fp8(G["blk_b"]), G["blk_as"], G["blk_bs"], "tn", "col")
    assert np.max(np.abs(c64 - ref)) <= 1e-12 * np.max(np.abs(ref))


def test_golden_pattern_inputs_bf16():
    a = R.decode_bf16(G["pat_a_bf16"])
    b = R.decode_bf16(G["pat_b_bf16"])
    # the oracle's own pattern generator and bf16 rounding reproduce the stored bits
    assert np.array_equal(R.encode_bf16(R.fill_pattern(a.shape, 0)), G["pat_a_bf16"])
    assert np.array_equal(R.encode_bf16(R.fill_pattern(b.shape, 1)), G["pat_b_bf16"])
    c = R.gemm_f32acc(a, b, "nn").astype(np.float64)
    assert np.max(np.abs(c - G["pat_c"])) <= 1e-5 * np.max(np.abs(G["pat_c"]))


# ------------------------------------------------------------------ GPU half
def _close(got, ref, what):
    """rtol / atol of the parity bar, plus the noise floor of fp32 accumulation itself: the stored
    results are float64 truth, and where terms of size max|ref| cancel, an fp32-accumulate result
    (the oracle's included, see test_golden_fp8_per_matrix) is only good to ~1e-5 of that size."""
    err = np.abs(np.asarray(got, np.float64) - ref)
    bound = ATOL + RTOL * np.abs(ref) + 1e-5 * np.max(np.abs(ref))
    assert np.all(err <= bound), f"{what}: max excess {(err - bound).max()}"


@pytest.mark.gpu
def test_gpu_golden_int8():
    import torch
    import qgemm_amd as Q
    from tests.util import dev, host, say, scalar
    say("golden int8")
    sa, sb = G["i8_scales"]
    c = torch.zeros(G["i8_c"].shape, dtype=torch.int32, device="cuda")
    Q.int8_mm(dev(G["i8_a"]), dev(G["i8_b"]), scalar(sa), scalar(sb), c)
    assert np.array_equal(host(c), G["i8_c"]), Q.last_config()
    cf = torch.zeros(G["i8_c"].shape, dtype=torch.float32, device="cuda")
    Q.int8_mm(dev(G["i8_a"]), dev(G["i8_b"]), scalar(sa), scalar(sb), cf)
    assert np.array_equal(host(cf).astype(np.float64), G["i8_c"].astype(np.float64) * float(sa) * float(sb))


@pytest.mark.gpu
def test_gpu_golden_fp8_per_matrix():
    import torch
    import qgemm_amd as Q
    from tests.util import fp8_tensor, host, say, scalar
    say("golden fp8 per-matrix")
    M, K = G["f8_a"].shape
    N = G["f8_b"].shape[0]
    sa, sb = G["f8_scales"]
    for dt in (torch.float32, torch.bfloat16):
        c = torch.zeros((M, N), dtype=dt, device="cuda")
        Q.scaled_gemm(fp8_tensor(G["f8_a"]), fp8_tensor(G["f8_b"]), scalar(sa), scalar(sb), c, M, N, K,
                      Q.SCALE_PER_MATRIX)
        _close(host(c), G["f8_c"], f"{dt} {Q.last_config()}")


@pytest.mark.gpu
def test_gpu_golden_fp8_block_reference_storage():
    import torch
    import qgemm_amd as Q
    from tests.util import dev, fp8_tensor, host, say
    say("golden fp8 block-scaled, reference storage")
    K, M = G["blk_a"].shape
    N = G["blk_b"].shape[1]
    a_t = fp8_tensor(G["blk_a"]).t()          # size (M, K), strides (1, M): the reference's column-major a
    b_t = fp8_tensor(G["blk_b"]).t()          # size (N, K), strides (1, N)
    as_t = dev(G["blk_as"]).t()
    bs_t = dev(G["blk_bs"]).t()
    c = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    Q.fp8_mm(a_t, b_t, as_t, bs_t, c)
    _close(host(c), G["blk_c"], Q.last_config())


@pytest.mark.gpu
def test_gpu_golden_pattern_inputs_bf16():
    import torch
    import qgemm_amd as Q
    from tests.util import dev, host, say
    say("golden pattern bf16 NN")
    a = dev(G["pat_a_bf16"].view(np.int16)).view(torch.bfloat16)
    b = dev(G["pat_b_bf16"].view(np.int16)).view(torch.bfloat16)
    c = torch.zeros(G["pat_c"].shape, dtype=torch.float32, device="cuda")
    Q.gemm(a, b, c, "kn")
    ref = G["pat_c"]
    # fp32 accumulation over K = 96 of values up to ~60: relative 1e-5 of the largest entry
    assert np.max(np.abs(host(c).astype(np.float64) - ref)) <= 1e-5 * np.max(np.abs(ref)), Q.last_config()
