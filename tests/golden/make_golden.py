#!/usr/bin/env python3
"""Writes the golden vectors of tests/golden/ (run once; the outputs are committed).

Nothing here uses the oracle or the HIP library: inputs come from numpy's PCG64 with a
fixed seed and expected outputs from the closed forms / float64 and int64 brute force,
so the fixtures are an independent pin for both.  The reference holds no vectors of its
own for this path; its closed-form input pattern (tests/includes/test_config.h:251-258)
and its index formulas (src/mix_gemm/hip_mix_gemm_kernel.cpp:96,111,137,149,241) are
what the cases restate.

  python tests/golden/make_golden.py
"""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def e4m3_decode_table():
    """OCP FP8 E4M3: 1-4-3, bias 7, subnormals m * 2^-9, no inf, NaN = S.1111.111, max 448."""
    out = []
    for code in range(256):
        s = -1.0 if code & 0x80 else 1.0
        e, m = (code >> 3) & 0xF, code & 7
        if e == 0xF and m == 7:
            out.append(float("nan"))
        elif e == 0:
            out.append(s * m * 2.0 ** -9)
        else:
            out.append(s * (1.0 + m / 8.0) * 2.0 ** (e - 7))
    return out


def finite_codes(rng, shape):
    c = rng.integers(0, 256, size=shape, dtype=np.uint8)
    c[(c & 0x7F) == 0x7F] = 0x3C          # replace NaN codes by 1.5
    return c


def main():
    rng = np.random.default_rng(42)
    table = e4m3_decode_table()
    with open(os.path.join(HERE, "fp8_e4m3_decode.json"), "w") as f:
        json.dump({"format": "OCP FP8 E4M3 (e4m3fn)", "decode": [None if v != v else v for v in table]}, f)
    dec = np.array(table, dtype=np.float64)

    out = {}
    # int8, NT operands (A M x K, B N x K), exact
    M, N, K = 48, 80, 192
    a = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    b = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    out["i8_a"], out["i8_b"] = a, b
    out["i8_c"] = (a.astype(np.int64) @ b.astype(np.int64).T).astype(np.int32)
    out["i8_scales"] = np.array([0.03125, 0.0078125], dtype=np.float32)          # powers of two: C_f32 exact

    # fp8 per-matrix, NT operands; truth in float64 (every product is exact there)
    M, N, K = 64, 128, 256
    a = finite_codes(rng, (M, K))
    b = finite_codes(rng, (N, K))
    sa, sb = np.float32(0.0123), np.float32(0.0456)
    out["f8_a"], out["f8_b"], out["f8_scales"] = a, b, np.array([sa, sb], dtype=np.float32)
    out["f8_c"] = (dec[a] @ dec[b].T) * (float(sa) * float(sb))

    # fp8 block-scaled in the reference's storage: A[m + k*M], B[k*N + n], as[m + kb*M], bs[nb + kb*ceil(N/128)],
    # acc += (P * as) * bs per 128-block of K
    M, N, K = 32, 256, 256
    a = finite_codes(rng, (K, M))          # stored K x M: element (m, k) at a[k, m]
    b = finite_codes(rng, (K, N))
    a_s = rng.uniform(0.5, 2.0, size=(K // 128, M)).astype(np.float32)
    b_s = rng.uniform(0.5, 2.0, size=(K // 128, N // 128)).astype(np.float32)
    c = np.zeros((M, N))
    for kb in range(K // 128):
        p = dec[a[kb * 128:(kb + 1) * 128]].T @ dec[b[kb * 128:(kb + 1) * 128]]
        c += p * a_s[kb].astype(np.float64)[:, None] * np.repeat(b_s[kb].astype(np.float64), 128)[None, :]
    out["blk_a"], out["blk_b"], out["blk_as"], out["blk_bs"], out["blk_c"] = a, b, a_s, b_s, c

    # the reference harness's closed-form inputs, 16-bit GEMM, NN operands (B is K x N)
    M, N, K = 32, 64, 96
    i = np.arange(M * K, dtype=np.float64)
    j = np.arange(K * N, dtype=np.float64)
    pa = ((i % 43) / 20.0 + 0.2 + (i % 19)).astype(np.float32).reshape(M, K)
    pb = ((j % 43) / 20.0 + 0.2 + (j % 37)).astype(np.float32).reshape(K, N)

    def bf16_bits(x):                      # round to nearest even on the upper 16 bits (src/include/fast_quat.h:3-12)
        u = x.view(np.uint32).astype(np.uint64)
        return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)

    def bf16_value(h):
        return (h.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    ha, hb = bf16_bits(pa), bf16_bits(pb)
    out["pat_a_bf16"], out["pat_b_bf16"] = ha, hb
    out["pat_c"] = bf16_value(ha) @ bf16_value(hb)
    np.savez_compressed(os.path.join(HERE, "gemm_cases.npz"), **out)
    print("wrote", sorted(out))


if __name__ == "__main__":
    main()
