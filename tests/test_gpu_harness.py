"""Runs the C++ harness (tests/harness/hip_benchmark, built over the drop-in headers
include/gemm.h, mix_gemm.h, matrix_transpose.h, blas.h) on the GPU and checks every row PASSes."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "harness", "hip_benchmark")


def test_cpp_harness_rows_pass():
    assert os.path.exists(EXE), "build it first: make -C tests/harness (or __graft_entry__.build())"
    print("[case] hip_benchmark --quick", flush=True)
    out = subprocess.run([EXE, "--quick"], capture_output=True, text=True, timeout=300)
    print(out.stdout[-4000:], out.stderr[-2000:], flush=True)
    assert out.returncode == 0
    rows = [l.split() for l in out.stdout.splitlines() if l.startswith("GEMM_kernel_v") or l.startswith("fp8_mm")]
    assert len(rows) >= 15                       # 7 entry points x 2 shapes + the fp8 row
    # row format of the reference harness: name time tflops bandwidth PASS|FAIL max_err speedup
    for r in rows:
        assert len(r) == 7 and r[4] == "PASS", r
        float(r[1]); float(r[2]); float(r[3]); float(r[5]); float(r[6])
    assert "matrix_transpose<bf16> 192x96: PASS" in out.stdout
    assert "dispatch error for M=48: PASS" in out.stdout
