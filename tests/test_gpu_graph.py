"""Launches recorded into a HIP graph replay to the eager results.

Every entry point launches on the caller's stream and, once the workspace has grown to what a
shape needs, allocates nothing and records no memset, so a serving loop can capture its GEMMs
after one eager warm-up call.  Each graph is replayed several times with eager launches and
synchronisations in between, on operands rewritten between the replays, and every replay is
compared with the eager result for the same operands: int32 bit for bit, floats bit for bit as
well (same kernel, same order of accumulation)."""
import numpy as np
import pytest
import torch

import qgemm_amd as Q
from oracle import cpu_ref as R
from tests.util import dev, fp8_tensor, host, say, scalar

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _reset_options():
    yield
    Q.set_option("force_config", -1)
    Q.set_option("force_split", 0)


def _capture(fn):
    fn()                               # warm-up: grows the workspace outside the capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    return g


def _replays(g, fn, out, rewrite, rounds=3):
    for r in range(rounds):
        rewrite(r)
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        got = out.clone()
        out.zero_()
        fn()                           # the program's own eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.uint8), out.view(torch.uint8)), "replay %d differs from eager" % r


@pytest.mark.parametrize("split", [0, 4])
def test_int8_graph_replay(split):
    """int8 per-matrix GEMM with and without a K split (two launches and the workspace inside the graph)."""
    M, N, K = 192, 320, 2048
    say("graph int8", M, N, K, "split", split)
    rng = np.random.default_rng(7)
    a = dev(rng.integers(-127, 128, (M, K), dtype=np.int8))
    b = dev(rng.integers(-127, 128, (N, K), dtype=np.int8))
    sa, sb = scalar(0.01), scalar(0.02)
    c = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    fn = lambda: Q.int8_mm(a, b, sa, sb, c, split_k=split)

    def rewrite(r):
        a.copy_(dev(np.random.default_rng(100 + r).integers(-127, 128, (M, K), dtype=np.int8)))

    g = _capture(fn)
    _replays(g, fn, c, rewrite)
    # and the last replay's operands against the oracle
    assert np.array_equal(host(c), R.gemm_i8_i32(host(a), host(b)))


def test_fp8_reference_layout_graph_replay():
    """fp8 block-scaled GEMM in the reference's storage (K x M and K x N operands): the operand transposes, the
    GEMM and the scale handling replay as one graph."""
    M, N, K = 256, 384, 1024
    say("graph fp8 reference layout", M, N, K)
    rng = np.random.default_rng(11)
    qa, _ = R.quantize_fp8(R.fill_normal((M, K), 1))
    qb, _ = R.quantize_fp8(R.fill_normal((N, K), 2))
    a_t = fp8_tensor(np.ascontiguousarray(qa.T)).t()            # [m, k], storage k x m
    b_t = fp8_tensor(np.ascontiguousarray(qb.T)).t()
    a_s = dev(rng.uniform(0.5, 1.5, (K // 128, M)).astype(np.float32))
    b_s = dev(rng.uniform(0.5, 1.5, (K // 128, N // 128)).astype(np.float32))
    c = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    fn = lambda: Q.fp8_mm(a_t, b_t, a_s.t(), b_s.t(), c)

    def rewrite(r):
        a_s.copy_(dev(np.random.default_rng(200 + r).uniform(0.5, 1.5, (K // 128, M)).astype(np.float32)))

    for kmajor in (0, 1):
        Q.set_option("kmajor", kmajor)
        try:
            g = _capture(fn)
            _replays(g, fn, c, rewrite)
        finally:
            Q.set_option("kmajor", 1)


def test_quantize_graph_replay():
    """Per-matrix quantiser (two passes through the workspace) followed by the GEMM on its output."""
    M, N, K = 128, 256, 512
    say("graph quantize + gemm", M, N, K)
    x = dev(R.fill_normal((M, K), 5))
    w = fp8_tensor(R.quantize_fp8(R.fill_normal((N, K), 6))[0])
    sw = scalar(0.01)
    c = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    hold = {}

    def fn():
        q, s = Q.quantize(x, torch.float8_e4m3fn, Q.QUANT_PER_MATRIX)
        hold["q"], hold["s"] = q, s          # keeps the graph's private allocations alive
        Q.scaled_gemm(q, w, s, sw, c, M, N, K, Q.SCALE_PER_MATRIX)

    def rewrite(r):
        x.copy_(dev(R.fill_normal((M, K), 50 + r)))

    g = _capture(fn)
    _replays(g, fn, c, rewrite)
