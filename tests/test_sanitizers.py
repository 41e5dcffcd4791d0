"""Host code under AddressSanitizer and UndefinedBehaviorSanitizer (no GPU involved; device code is never
sanitized): the CPU oracle, and the part of the C-ABI library that runs before a kernel is launched.  The
reference builds with -Wall -Wextra only (CMakeLists.txt:14).

  make -C oracle asan          oracle/_asan/oracle_asan (driver oracle/asan_main.c), oracle/_asan/libcpu_ref_ubsan.so
  make -C qgemm_amd/csrc asan  qgemm_amd/csrc/build_asan/libqgemm_asan.so, tests/asan/capi_host_asan
"""
import os
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ENV = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")


def _run(cmd, **kw):
    out = subprocess.run(cmd, capture_output=True, text=True, env=kw.pop("env", ENV), timeout=600, **kw)
    text = out.stdout + out.stderr
    assert out.returncode == 0, text[-4000:]
    assert "AddressSanitizer" not in text and "runtime error" not in text, text[-4000:]
    return text


@pytest.fixture(scope="module")
def oracle_asan():
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    _run(["make", "-C", os.path.join(ROOT, "oracle"), "asan"])
    return os.path.join(ROOT, "oracle", "_asan")


def test_oracle_under_asan_and_ubsan(oracle_asan):
    """Every oracle function on exactly-sized heap buffers (ragged shapes, all three operand storages, padded
    leading dimensions), each result checked against a plain loop in the driver."""
    assert "oracle_asan: clean" in _run([os.path.join(oracle_asan, "oracle_asan")])


def test_oracle_python_tests_against_the_ubsan_build(oracle_asan):
    """tests/test_oracle.py and the CPU half of tests/test_golden.py, with the oracle library replaced by its
    UndefinedBehaviorSanitizer build (any finding aborts the child)."""
    env = dict(ENV, QGEMM_ORACLE_LIB=os.path.join(oracle_asan, "libcpu_ref_ubsan.so"))
    text = _run([sys.executable, "-m", "pytest", "-q", "-m", "not gpu", "-p", "no:cacheprovider",
                 os.path.join(ROOT, "tests", "test_oracle.py"), os.path.join(ROOT, "tests", "test_golden.py")], env=env, cwd=ROOT)
    assert " passed" in text and "failed" not in text


def test_capi_host_layer_under_asan_and_ubsan():
    """Argument validation, option table, tile raster and the planner (qgemm_plan over 5000 shape / type / storage
    combinations, forced rows and splits) of a library build whose host code is sanitized; no device is touched."""
    hipcc = "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc) or not os.path.exists(os.path.join(ROOT, "qgemm_amd", "csrc", "build", "inst_f8.o")):
        pytest.skip("needs hipcc and the kernel objects of a library build (make -C qgemm_amd/csrc)")
    _run(["make", "-C", os.path.join(ROOT, "qgemm_amd", "csrc"), "asan"])
    assert "capi_host_asan: clean" in _run([os.path.join(ROOT, "tests", "asan", "capi_host_asan")])
