"""The library workspace: never freed under a caller's feet, shared safely between streams, never grown during
a graph capture."""
import ctypes as C

import numpy as np
import pytest
import torch

import qgemm_amd as Q
from oracle import cpu_ref as R
from qgemm_amd import lib as L
from tests.util import dev, fp8_inputs, fp8_tensor, host, int8_inputs, say, scalar

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _reset_options():
    yield
    Q.set_option("force_config", -1)
    Q.set_option("force_split", 0)
    Q.set_option("kmajor", 1)


def _info():
    base, size = C.c_void_p(), C.c_size_t()
    L.check(L.load_library().qgemm_workspace_info(C.byref(base), C.byref(size)))
    return base.value, size.value


def test_growth_keeps_earlier_graphs_valid():
    """A graph captured while the workspace was small replays to the same bits after a later, larger call has
    made the library move to a bigger block: the old block is retired, not freed."""
    say("workspace growth under a captured graph")
    M, N, K = 64, 384, 2048
    qa, sa, qb, sb = int8_inputs(M, N, K, seed=77)
    a, b, s1, s2 = dev(qa), dev(qb), scalar(sa), scalar(sb)
    c = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    fn = lambda: Q.int8_mm(a, b, s1, s2, c, split_k=4)
    fn()
    torch.cuda.synchronize()
    base0, size0 = _info()
    assert base0 and size0 >= M * N * 4 * 4
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    ref = R.gemm_i8_i32(qa, qb)
    # a call that needs more than the current block: reference-layout transposes of a larger problem
    big = size0 + (8 << 20)
    L.check(L.load_library().qgemm_reserve_workspace(big))
    base1, size1 = _info()
    assert size1 >= big and base1 != base0
    # scribble over the new block with other work, then replay the old graph
    M2, N2 = 128, 512
    qa2, sa2, qb2, sb2 = int8_inputs(M2, N2, K, seed=78)
    c2 = torch.zeros((M2, N2), dtype=torch.int32, device="cuda")
    Q.int8_mm(dev(qa2), dev(qb2), scalar(sa2), scalar(sb2), c2, split_k=8)
    for _ in range(3):
        c.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(host(c), ref)
    assert np.array_equal(host(c2), R.gemm_i8_i32(qa2, qb2))
    # same-size calls never move the block
    Q.int8_mm(dev(qa2), dev(qb2), scalar(sa2), scalar(sb2), c2, split_k=8)
    assert _info() == (base1, size1)


def test_no_allocation_during_capture():
    """A call that would have to grow the workspace while its stream is being captured fails with
    QGEMM_ERR_ALLOC (5) and leaves the block alone."""
    say("workspace growth refused during capture")
    base0, size0 = _info()
    M, N = 4096, 4096                                # planes of 64 MiB: as many as it takes to outgrow the block
    nsplit = size0 // (M * N * 4) + 2
    K = 128 * 4 * nsplit
    a = torch.zeros((M, K), dtype=torch.int8, device="cuda")
    b = torch.zeros((N, K), dtype=torch.int8, device="cuda")
    c = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    s = scalar(1)
    g = torch.cuda.CUDAGraph()
    status = []
    with torch.cuda.graph(g):
        try:
            Q.int8_mm(a, b, s, s, c, split_k=nsplit)
            status.append(0)
        except Q.QgemmError as e:
            status.append(e.status)
    assert status == [5]
    assert _info() == (base0, size0)


def test_two_streams_share_the_workspace_in_order():
    """Split-K int8 on one stream interleaved with reference-layout fp8 (two operand transposes in the workspace)
    on another, no host synchronisation in between: every result equals the serial one bit for bit."""
    say("two streams, one workspace")
    M, N, K = 256, 512, 2048
    qa, sa, qb, sb = int8_inputs(M, N, K, seed=81)
    a8, b8, s8a, s8b = dev(qa), dev(qb), scalar(sa), scalar(sb)
    fa, _, fb, _ = fp8_inputs(M, N, K, seed=83)
    as_ = R.fill_uniform((M, K // 128), 84, 0.5, 2.0) / np.float32(448)
    bs = R.fill_uniform((N // 128, K // 128), 85, 0.5, 2.0) / np.float32(448)
    a_t = fp8_tensor(np.ascontiguousarray(fa.T)).t()
    b_t = fp8_tensor(np.ascontiguousarray(fb.T)).t()
    as_t, bs_t = dev(np.ascontiguousarray(as_.T)).t(), dev(np.ascontiguousarray(bs.T)).t()
    Q.set_option("kmajor", 0)                         # force the route through the transposes (workspace)
    # serial results
    ci_ref = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    cf_ref = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    Q.int8_mm(a8, b8, s8a, s8b, ci_ref, split_k=8)
    assert "splitk" in Q.last_config()
    Q.fp8_mm(a_t, b_t, as_t, bs_t, cf_ref)
    assert not Q.last_config().endswith("_tn")
    torch.cuda.synchronize()
    assert np.array_equal(host(ci_ref), R.gemm_i8_i32(qa, qb))
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    rounds = 12
    ci = [torch.zeros_like(ci_ref) for _ in range(rounds)]
    cf = [torch.zeros_like(cf_ref) for _ in range(rounds)]
    for r in range(rounds):
        with torch.cuda.stream(s1):
            Q.int8_mm(a8, b8, s8a, s8b, ci[r], split_k=8)
        with torch.cuda.stream(s2):
            Q.fp8_mm(a_t, b_t, as_t, bs_t, cf[r])
    torch.cuda.synchronize()
    for r in range(rounds):
        assert torch.equal(ci[r], ci_ref), f"int8 round {r}"
        assert torch.equal(cf[r].view(torch.int16), cf_ref.view(torch.int16)), f"fp8 round {r}"
