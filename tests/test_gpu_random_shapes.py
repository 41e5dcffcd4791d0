"""Seeded random sweep over what the dispatch can combine: family (int8 / fp8 per matrix / fp8 block scales in both
storages / int8 block scales / bf16 / fp16 with B stored N x K or K x N), shape (ragged, down to one row), tile variant (the
heuristic's or a forced row of the table), K split and output type.  Every case is checked against the CPU oracle:
int32 accumulators bit for bit, float outputs to rtol 2e-2 / atol 1e-2 (plus half an ulp of a 16-bit output)."""
import numpy as np
import pytest
import torch

import qgemm_amd as Q
from oracle import cpu_ref as R
from tests.util import assert_close, dev, fp8_tensor, host, say, scalar

pytestmark = pytest.mark.gpu
# rows of the variant table of each family, by name, as the library reports them
ROWS = {
    "i8": Q.variant_names(Q.DT_I8, Q.SCALE_PER_MATRIX), "f8": Q.variant_names(Q.DT_F8E4M3, Q.SCALE_PER_MATRIX),
    "f8_block": Q.variant_names(Q.DT_F8E4M3, Q.SCALE_BLOCK128), "f8_block_ref": Q.variant_names(Q.DT_F8E4M3, Q.SCALE_BLOCK128),
    "i8_block": Q.variant_names(Q.DT_I8, Q.SCALE_BLOCK128),
    "bf16_nk": Q.variant_names(Q.DT_BF16), "bf16_kn": Q.variant_names(Q.DT_BF16),
    "f16_nk": Q.variant_names(Q.DT_F16), "f16_kn": Q.variant_names(Q.DT_F16),
}


@pytest.fixture(autouse=True)
def _reset_options():
    yield
    for k, v in (("force_config", -1), ("force_split", 0), ("group_m", 0), ("kmajor", 1)):
        Q.set_option(k, v)


def _draw(rng):
    fam = rng.choice(["i8", "f8", "f8_block", "f8_block_ref", "i8_block", "bf16_nk", "bf16_kn", "f16_nk", "f16_kn"])
    kq = {"i8": 128, "f8": 128, "f8_block": 128, "f8_block_ref": 128, "i8_block": 128}.get(fam, 64)     # elements of a 128-byte K step
    K = int(rng.integers(1, 9)) * kq
    if rng.random() < 0.25:                         # a long K: several rounds of the skinny-M kernel, deep rings
        K = int(rng.integers(9, 41)) * kq
    if rng.random() < 0.3:                          # a partial last K step: whole 16-byte chunks (fp8_mm: K % 32 == 0)
        unit = 32 if fam == "f8_block_ref" else kq // 8
        K += int(rng.integers(1, kq // unit)) * unit
    if rng.random() < 0.3:
        M = int(rng.choice([1, 7, 16, 33, 100, 128]))
    else:
        M = int(rng.integers(1, 40)) * 16 + int(rng.choice([0, 0, 5, 8]))
    N = int(rng.integers(1, 40)) * 16 + int(rng.choice([0, 0, 8]))
    if fam == "f8_block_ref":                       # the reference's contract: multiples of 32
        M, N = max(32, M // 32 * 32), max(32, N // 32 * 32)
    if fam.endswith("_kn"):
        N = max(8, N // 8 * 8)                      # rows of B are 16-byte aligned either way
    # (a K-major call whose family lacks the forced row goes through the transposes to the K-contiguous row of that name)
    variant = str(rng.choice(ROWS[fam])) if rng.random() < 0.6 else None
    split = int(rng.choice([0, 0, 0, 2, 3])) if K // kq >= 4 else 0
    if "block" in fam and split and (K + 127) // 128 < 2 * split:
        split = 0
    return fam, M, N, K, variant, split


@pytest.mark.parametrize("seed", range(192))
def test_random_case(seed):
    rng = np.random.default_rng(1000 + seed)
    fam, M, N, K, variant, split = _draw(rng)
    say("random", seed, fam, (M, N, K), "variant", variant, "split", split)
    Q.force_config(variant)
    Q.set_option("force_split", split)
    if fam == "i8":
        qa, sa = R.quantize_int8(R.fill_normal((M, K), seed))
        qb, sb = R.quantize_int8(R.fill_normal((N, K), seed + 500))
        acc = R.gemm_i8_i32(qa, qb)
        c = torch.full((M, N), -3, dtype=torch.int32, device="cuda")
        Q.int8_mm(dev(qa), dev(qb), scalar(sa), scalar(sb), c)
        assert np.array_equal(host(c), acc), Q.last_config()
        cf = torch.zeros((M, N), dtype=torch.float32, device="cuda")
        Q.int8_mm(dev(qa), dev(qb), scalar(sa), scalar(sb), cf)
        assert np.array_equal(host(cf), R.scale_i32_to_f32(acc, sa, sb)), Q.last_config()
        return
    out_dt = [torch.bfloat16, torch.float16, torch.float32][int(rng.integers(0, 3))]
    extra_rtol = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -10, torch.float32: 0.0}[out_dt]
    c = torch.full((M, N), 7.0, dtype=out_dt, device="cuda")
    if fam == "f8":
        qa, sa = R.quantize_fp8(R.fill_normal((M, K), seed))
        qb, sb = R.quantize_fp8(R.fill_normal((N, K), seed + 500))
        ref = R.gemm_f32acc(R.decode_fp8(qa), R.decode_fp8(qb)) * np.float32(sa * sb)
        Q.scaled_gemm(fp8_tensor(qa), fp8_tensor(qb), scalar(sa), scalar(sb), c, M, N, K, Q.SCALE_PER_MATRIX)
    elif fam == "i8_block":
        qa, _ = R.quantize_int8(R.fill_normal((M, K), seed))
        qb, _ = R.quantize_int8(R.fill_normal((N, K), seed + 500))
        as_ = R.fill_uniform((M, (K + 127) // 128), seed + 1, 0.5, 2.0) / np.float32(127)
        bs = R.fill_uniform(((N + 127) // 128, (K + 127) // 128), seed + 2, 0.5, 2.0) / np.float32(127)
        ref = R.gemm_i8_block(qa, qb, as_, bs)
        Q.int8_mm_block(dev(qa), dev(qb), dev(as_), dev(bs), c)
    elif fam in ("f8_block", "f8_block_ref"):
        qa, _ = R.quantize_fp8(R.fill_normal((M, K), seed))
        qb, _ = R.quantize_fp8(R.fill_normal((N, K), seed + 500))
        as_ = R.fill_uniform((M, (K + 127) // 128), seed + 1, 0.5, 2.0) / np.float32(448)
        bs = R.fill_uniform(((N + 127) // 128, (K + 127) // 128), seed + 2, 0.5, 2.0) / np.float32(448)
        ref = R.gemm_fp8_block(R.decode_fp8(qa), R.decode_fp8(qb), as_, bs)
        if fam == "f8_block":
            Q.scaled_gemm(fp8_tensor(qa), fp8_tensor(qb), dev(as_), dev(bs), c, M, N, K, Q.SCALE_BLOCK128)
        else:
            Q.set_option("kmajor", int(rng.integers(0, 2)))
            Q.fp8_mm(fp8_tensor(np.ascontiguousarray(qa.T)).t(), fp8_tensor(np.ascontiguousarray(qb.T)).t(),
                     dev(np.ascontiguousarray(as_.T)).t(), dev(np.ascontiguousarray(bs.T)).t(), c)
    else:
        enc, dec, tdt = ((R.encode_f16, R.decode_f16, torch.float16) if fam.startswith("f16")
                         else (R.encode_bf16, R.decode_bf16, torch.bfloat16))
        ha, hb = enc(R.fill_uniform((M, K), seed)), enc(R.fill_uniform((N, K), seed + 500))
        ref = R.gemm_f32acc(dec(ha), dec(hb))
        a = dev(ha.view(np.int16)).view(tdt)
        b = dev(hb.view(np.int16)).view(tdt)
        if fam.endswith("_kn"):
            Q.set_option("kmajor", int(rng.integers(0, 2)))
            Q.gemm(a, b.t().contiguous(), c, "kn")
        else:
            Q.gemm(a, b, c, "nk")
    assert_close(host(c).astype(np.float32), ref, rtol=2e-2 + extra_rtol, atol=1e-2, what=f"{fam} {Q.last_config()} {out_dt}")
