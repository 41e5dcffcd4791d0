"""Shared helpers of the GPU parity tests: seeded inputs from the oracle's
counter-based PRNG, host<->device plumbing, tolerance checks."""
import sys

import numpy as np
import torch

from oracle import cpu_ref as R

# float outputs vs the fp32-accumulate oracle: the tolerance the task states
RTOL, ATOL = 2e-2, 1e-2


def say(*a):
    """Name the case before it touches the GPU, flushed, so a lost box still says where it was."""
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def dev(x):
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def fp8_tensor(q_u8):
    """uint8 codes -> device tensor viewed as torch.float8_e4m3fn"""
    return dev(q_u8).view(torch.float8_e4m3fn)


def host(t):
    torch.cuda.synchronize()
    if t.dtype == torch.bfloat16:
        return t.float().cpu().numpy()
    return t.cpu().numpy()


def int8_inputs(M, N, K, seed):
    """cfg-2 style: fp32 N(0,1), symmetric per-matrix quantisation."""
    qa, sa = R.quantize_int8(R.fill_normal((M, K), seed))
    qb, sb = R.quantize_int8(R.fill_normal((N, K), seed + 1))
    return qa, sa, qb, sb


def fp8_inputs(M, N, K, seed):
    """cfg-3 style: fp32 N(0,1) scaled so max|x| maps to 448."""
    qa, sa = R.quantize_fp8(R.fill_normal((M, K), seed))
    qb, sb = R.quantize_fp8(R.fill_normal((N, K), seed + 1))
    return qa, sa, qb, sb


def scalar(x):
    return dev(np.array([x], np.float32))


def assert_close(got, ref, rtol=RTOL, atol=ATOL, what=""):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    err = np.abs(got - ref)
    bound = atol + rtol * np.abs(ref)
    bad = err > bound
    if bad.any():
        i = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(f"{what}: {bad.sum()} of {bad.size} outside rtol={rtol} atol={atol}; worst at {i}: "
                             f"got {got[i]} ref {ref[i]}")


def bf16_round(x):
    return R.decode_bf16(R.encode_bf16(x))
