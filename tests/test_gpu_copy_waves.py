"""The 256 x 128 row whose four computing waves leave every copy to four copying waves (`256x128_w2x2_cw`, its twin
for K-contiguous a_scale and its K-major forms): every number of K steps from one up to past the point where the
three A buffers and two B buffers have all been reused, with and without a K split, on one tile, on ragged tiles and
on several tiles.  Small integers (and power-of-two block scales) sum exactly, so the results must equal the CPU
oracle bit for bit: a buffer refilled before its last read, a copy waited for too late or a step left out cannot
hide."""
import numpy as np
import pytest
import torch

import qgemm_amd as Q
from oracle import cpu_ref as R
from tests.util import dev, fp8_tensor, host, say, scalar

pytestmark = pytest.mark.gpu
ROW = "256x128_w2x2_cw"                                      # row of the variant table


@pytest.fixture(autouse=True)
def _reset_options():
    yield
    for k, v in (("force_config", -1), ("force_split", 0), ("kmajor", 1)):
        Q.set_option(k, v)


@pytest.mark.parametrize("fam", ["f8", "f8_block", "i8", "bf16", "f8_block_ref", "bf16_kn"])
def test_every_number_of_k_steps(fam):
    want = {"f8_block_ref": "256x128_w2x2_cw_tn", "bf16_kn": "256x128_w2x2_cw_nn"}.get(fam, "256x128_w2x2_cw")
    for (M, N) in ((256, 128), (300, 200), (512, 384)):
        if fam == "f8_block_ref":                            # fp8_mm takes multiples of 32, as the reference does
            M, N = (M + 31) // 32 * 32, (N + 31) // 32 * 32
        for ksteps in (1, 2, 3, 4, 5, 6, 7, 8, 9, 13, 16):
            for split in ((1, 2) if ksteps >= 4 else (1,)):
                K = ksteps * (64 if fam.startswith("bf16") else 128)
                say("copying waves", fam, (M, N, K), "split", split)
                Q.force_config(ROW)
                Q.set_option("force_split", split)
                Q.set_option("kmajor", 2)                    # K-major operands as stored, whatever the estimate says
                rng = np.random.default_rng(100 * ksteps + split)
                a = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
                b = rng.integers(-3, 4, size=(N, K)).astype(np.float32)
                c = torch.full((M, N), -7.0, dtype=torch.float32, device="cuda")
                if fam == "i8":
                    c = torch.full((M, N), -7, dtype=torch.int32, device="cuda")
                    Q.int8_mm(dev(a.astype(np.int8)), dev(b.astype(np.int8)), scalar(1), scalar(1), c)
                    ref = R.gemm_i8_i32(a.astype(np.int8), b.astype(np.int8))
                elif fam == "bf16":
                    Q.gemm(dev(a).bfloat16(), dev(b).bfloat16(), c, "nk")
                    ref = R.gemm_f32acc(a, b)
                elif fam == "bf16_kn":
                    Q.gemm(dev(a).bfloat16(), dev(np.ascontiguousarray(b.T)).bfloat16(), c, "kn")
                    ref = R.gemm_f32acc(a, b)
                elif fam == "f8":
                    Q.scaled_gemm(fp8_tensor(R.encode_fp8(a)), fp8_tensor(R.encode_fp8(b)), scalar(1), scalar(1), c, M, N, K,
                                  Q.SCALE_PER_MATRIX)
                    ref = R.gemm_f32acc(a, b)
                else:
                    as_ = (2.0 ** rng.integers(-3, 4, size=(M, ksteps))).astype(np.float32)
                    bs = (2.0 ** rng.integers(-3, 4, size=((N + 127) // 128, ksteps))).astype(np.float32)
                    if fam == "f8_block":                    # (even K block counts take the twin that reads a_scale as given)
                        Q.scaled_gemm(fp8_tensor(R.encode_fp8(a)), fp8_tensor(R.encode_fp8(b)), dev(as_), dev(bs), c, M, N, K,
                                      Q.SCALE_BLOCK128)
                    else:
                        Q.fp8_mm(fp8_tensor(np.ascontiguousarray(R.encode_fp8(a).T)).t(),
                                 fp8_tensor(np.ascontiguousarray(R.encode_fp8(b).T)).t(),
                                 dev(np.ascontiguousarray(as_.T)).t(), dev(np.ascontiguousarray(bs.T)).t(), c)
                    ref = R.gemm_fp8_block(a, b, as_, bs)
                name = Q.last_config()
                assert name.replace("_ks", "").startswith(want), name
                assert ("splitk" in name) == (split > 1), name
                assert np.array_equal(host(c), ref), (name, ksteps, split)


@pytest.mark.parametrize("fam", ["f8", "f8_block", "i8", "bf16"])
def test_192_row_tile_every_number_of_k_steps(fam):
    """The 192 x 256 row of the 8-wave solo schedule (wave tiles of six row blocks, a fragment ring of three slots,
    three A copies and four B copies per wave and step): the same sweep over K steps, K splits and ragged tiles."""
    for (M, N) in ((192, 256), (300, 200), (576, 512)):
        for ksteps in (1, 2, 3, 4, 5, 6, 7, 8, 9, 13, 16):
            for split in ((1, 2) if ksteps >= 4 else (1,)):
                K = ksteps * (64 if fam == "bf16" else 128)
                say("192-row tile", fam, (M, N, K), "split", split)
                Q.force_config("192x256_w2x4_solo8")
                Q.set_option("force_split", split)
                rng = np.random.default_rng(300 * ksteps + split)
                a = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
                b = rng.integers(-3, 4, size=(N, K)).astype(np.float32)
                c = torch.full((M, N), -7.0, dtype=torch.float32, device="cuda")
                if fam == "i8":
                    c = torch.full((M, N), -7, dtype=torch.int32, device="cuda")
                    Q.int8_mm(dev(a.astype(np.int8)), dev(b.astype(np.int8)), scalar(1), scalar(1), c)
                    ref = R.gemm_i8_i32(a.astype(np.int8), b.astype(np.int8))
                elif fam == "bf16":
                    Q.gemm(dev(a).bfloat16(), dev(b).bfloat16(), c, "nk")
                    ref = R.gemm_f32acc(a, b)
                elif fam == "f8":
                    Q.scaled_gemm(fp8_tensor(R.encode_fp8(a)), fp8_tensor(R.encode_fp8(b)), scalar(1), scalar(1), c, M, N, K,
                                  Q.SCALE_PER_MATRIX)
                    ref = R.gemm_f32acc(a, b)
                else:
                    as_ = (2.0 ** rng.integers(-3, 4, size=(M, ksteps))).astype(np.float32)
                    bs = (2.0 ** rng.integers(-3, 4, size=((N + 127) // 128, ksteps))).astype(np.float32)
                    Q.scaled_gemm(fp8_tensor(R.encode_fp8(a)), fp8_tensor(R.encode_fp8(b)), dev(as_), dev(bs), c, M, N, K,
                                  Q.SCALE_BLOCK128)
                    ref = R.gemm_fp8_block(a, b, as_, bs)
                name = Q.last_config()
                assert name.replace("_ks", "").startswith("192x256_w2x4_solo8"), name
                assert ("splitk" in name) == (split > 1), name
                assert np.array_equal(host(c), ref), (name, ksteps, split)
