"""The rows with two K groups per workgroup (two sets of computing waves half a turn apart, copying waves beside them):
every number of K steps from one up to past twice the ring, so that the first phases (nothing to multiply yet), the
last ones (nothing left to read or copy) and every ring position are hit; with and without a K split; on ragged
tiles.  Small integers (and power-of-two block scales) sum exactly in fp32 and int32, so the results must equal the
CPU oracle bit for bit: a stage read too early, a buffer refilled too soon or a step left out cannot hide."""
import numpy as np
import pytest
import torch

import qgemm_amd as Q
from oracle import cpu_ref as R
from tests.util import dev, fp8_tensor, host, say, scalar

pytestmark = pytest.mark.gpu
ROWS = ["128x128_w2x2_k2", "64x128_w1x4_k2"]                # rows of the variant table, by name


@pytest.fixture(autouse=True)
def _reset_options():
    yield
    for k, v in (("force_config", -1), ("force_split", 0), ("kmajor", 1), ("k_rot", -1), ("as_groups", 1)):
        Q.set_option(k, v)


@pytest.mark.parametrize("row", sorted(ROWS))
@pytest.mark.parametrize("fam", ["f8", "f8_block", "i8", "bf16"])
def test_every_number_of_k_steps(row, fam):
    M, N = 200, 328                                          # ragged in both directions, several tiles
    for ksteps in range(1, 14):
        for split in ((0, 2) if ksteps >= 4 else (0,)):
            K = ksteps * (64 if fam == "bf16" else 128)
            say("k groups", row, fam, (M, N, K), "split", split)
            Q.force_config(row)
            Q.set_option("force_split", split if split else 1)
            rng = np.random.default_rng(100 * ksteps + split)
            a = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
            b = rng.integers(-3, 4, size=(N, K)).astype(np.float32)
            if fam == "i8":
                c = torch.full((M, N), -7, dtype=torch.int32, device="cuda")
                Q.int8_mm(dev(a.astype(np.int8)), dev(b.astype(np.int8)), scalar(1), scalar(1), c)
                ref = R.gemm_i8_i32(a.astype(np.int8), b.astype(np.int8))
            elif fam == "bf16":
                c = torch.full((M, N), -7.0, dtype=torch.float32, device="cuda")
                Q.gemm(dev(a).bfloat16(), dev(b).bfloat16(), c, "nk")
                ref = R.gemm_f32acc(a, b)
            elif fam == "f8":
                c = torch.full((M, N), -7.0, dtype=torch.float32, device="cuda")
                Q.scaled_gemm(fp8_tensor(R.encode_fp8(a)), fp8_tensor(R.encode_fp8(b)), scalar(1), scalar(1), c, M, N, K,
                              Q.SCALE_PER_MATRIX)
                ref = R.gemm_f32acc(a, b)
            else:
                as_ = (2.0 ** rng.integers(-3, 4, size=(M, ksteps))).astype(np.float32)
                bs = (2.0 ** rng.integers(-3, 4, size=((N + 127) // 128, ksteps))).astype(np.float32)
                c = torch.full((M, N), -7.0, dtype=torch.float32, device="cuda")
                Q.scaled_gemm(fp8_tensor(R.encode_fp8(a)), fp8_tensor(R.encode_fp8(b)), dev(as_), dev(bs), c, M, N, K,
                              Q.SCALE_BLOCK128)
                ref = R.gemm_fp8_block(a, b, as_, bs)
            name = Q.last_config()
            assert name.startswith(row), name
            assert ("splitk" in name) == (split > 1), name
            assert np.array_equal(host(c), ref), (name, ksteps, split)


@pytest.mark.parametrize("fam,row", [("f8_block_ref", "128x128_w2x2_k2"), ("bf16_kn", "128x128_w2x2_k2"), ("bf16_kn", "64x128_w1x4_k2")])
def test_every_number_of_k_steps_k_major(fam, row):
    """The same with the operands stored K-major and read as stored (transposing LDS reads in the computing waves,
    the copying waves walking rows of k): the reference's fp8 layout with block scales, and B of a plain GEMM
    stored K x N."""
    M, N = 192, 320                                          # fp8_mm takes multiples of 32, as the reference does
    Q.set_option("kmajor", 2)                                # as stored, whatever the estimate says
    for ksteps in range(1, 14):
        K = ksteps * (64 if fam == "bf16_kn" else 128)
        say("k groups, K-major", row, fam, (M, N, K))
        Q.force_config(row)
        Q.set_option("force_split", 1)
        rng = np.random.default_rng(7000 + ksteps)
        a = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
        b = rng.integers(-3, 4, size=(N, K)).astype(np.float32)
        c = torch.full((M, N), -7.0, dtype=torch.float32, device="cuda")
        if fam == "bf16_kn":
            Q.gemm(dev(a).bfloat16(), dev(np.ascontiguousarray(b.T)).bfloat16(), c, "kn")
            ref = R.gemm_f32acc(a, b)
            suffix = "_nn"
        else:
            as_ = (2.0 ** rng.integers(-3, 4, size=(M, ksteps))).astype(np.float32)
            bs = (2.0 ** rng.integers(-3, 4, size=((N + 127) // 128, ksteps))).astype(np.float32)
            Q.fp8_mm(fp8_tensor(np.ascontiguousarray(R.encode_fp8(a).T)).t(), fp8_tensor(np.ascontiguousarray(R.encode_fp8(b).T)).t(),
                     dev(np.ascontiguousarray(as_.T)).t(), dev(np.ascontiguousarray(bs.T)).t(), c)
            ref = R.gemm_fp8_block(a, b, as_, bs)
            suffix = "_tn"
        name = Q.last_config()
        assert name == row + suffix, name
        assert np.array_equal(host(c), ref), (name, ksteps)


@pytest.mark.parametrize("row", sorted(ROWS))
def test_block_scales_four_k_blocks_a_copy(row):
    """K-contiguous a_scale, rows and K slices at multiples of four blocks: the copying waves bring four K blocks of a
    row at once into one of four slots.  More than four groups (the slots are reused), a K split whose slices are
    (8) and are not (6, 10) multiples of four, the rotated start by four steps, by three (the single-block copies take
    over) and none, an a_scale whose rows are not 16-byte aligned (the same), and the option that switches it off:
    every result equals the oracle bit for bit."""
    M, N = 200, 328
    for ksteps in (4, 8, 12, 16, 20, 40):
        for split, k_rot, groups, shift in ((1, -1, 1, 0), (1, 0, 1, 0), (1, 4, 1, 0), (1, 8, 1, 0), (1, 3, 1, 0),
                                            (2, -1, 1, 0), (1, -1, 0, 0), (1, -1, 1, 1), (2, 4, 1, 1)):
            K = ksteps * 128
            say("k groups, a_scale in groups", row, (M, N, K), "split", split, "k_rot", k_rot, "groups", groups, "shift", shift)
            Q.force_config(row)
            Q.set_option("force_split", split)
            Q.set_option("k_rot", k_rot)
            Q.set_option("as_groups", groups)
            rng = np.random.default_rng(31 * ksteps + split + 7 * shift)
            a = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
            b = rng.integers(-3, 4, size=(N, K)).astype(np.float32)
            as_ = (2.0 ** rng.integers(-3, 4, size=(M, ksteps))).astype(np.float32)
            bs = (2.0 ** rng.integers(-3, 4, size=((N + 127) // 128, ksteps))).astype(np.float32)
            as_dev = torch.empty(M * ksteps + 4, dtype=torch.float32, device="cuda")[shift:shift + M * ksteps]
            as_dev.copy_(dev(as_).reshape(-1))
            c = torch.full((M, N), -7.0, dtype=torch.float32, device="cuda")
            Q.scaled_gemm(fp8_tensor(R.encode_fp8(a)), fp8_tensor(R.encode_fp8(b)), as_dev, dev(bs), c, M, N, K, Q.SCALE_BLOCK128)
            name = Q.last_config()
            assert name.startswith(row) and ("splitk" in name) == (split > 1), name
            assert np.array_equal(host(c), R.gemm_fp8_block(a, b, as_, bs)), (name, ksteps, split, k_rot, groups, shift)
