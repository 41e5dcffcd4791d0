"""tests/harness/benchmark_to_md.py: the row format of the reference's harness (test_config.h:210-226) goes in,
TFLOPS / speedup / percent-of-peak tables come out."""
import importlib.util
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
spec = importlib.util.spec_from_file_location("benchmark_to_md", os.path.join(ROOT, "tests", "harness", "benchmark_to_md.py"))
md = importlib.util.module_from_spec(spec)
spec.loader.exec_module(md)

TEXT = """HIP gfx950 GEMM Benchmark
GPU: AMD Instinct MI355X

=== GEMM Benchmark ===
Problem size: M=512, N=512, K=512
Precision: bf16
Warmup runs: 5
Benchmark runs: 10
==========================================================================================
Function                 Time(ms)    TFLOPS      Bandwidth(GB/s)Correctness Max Error       Speedup
------------------------------------------------------------------------------------------
reference_cpu_oracle     12.500      0.021       0.126          PASS        0.00e+00        1.00e+00
GEMM_kernel_v1           0.010       25.000      150.000        PASS        1.20e-02        1.25e+03
GEMM_kernel_v3.1         0.020       12.500      75.000         FAIL        9.00e+00        6.25e+02
==========================================================================================

=== GEMM Benchmark ===
Problem size: M=256, N=384, K=512
Precision: fp8 e4m3 (OCP), 128-block scales, bf16 out
Warmup runs: 5
Benchmark runs: 10
fp8_mm(select_BLOCK..)   0.010       50.000      40.000         PASS        3.00e-03        1.00e+00
dispatch error for M=48: PASS
"""


def test_parse_and_tables():
    blocks, names = md.parse(TEXT.splitlines())
    assert list(blocks) == [("M=512, N=512, K=512", "bf16"), ("M=256, N=384, K=512", "fp8")]
    assert names == ["reference_cpu_oracle", "GEMM_kernel_v1", "GEMM_kernel_v3.1", "fp8_mm(select_BLOCK..)"]
    assert blocks[("M=512, N=512, K=512", "bf16")]["GEMM_kernel_v1"]["tflops"] == 25.0
    out = md.render(TEXT.splitlines())
    assert "| M=512, N=512, K=512 | bf16 | 0.021 | 25.000 | 12.500 (FAIL) | - |" in out
    assert "| M=512, N=512, K=512 | bf16 | 1.00x | 1250.00x | 625.00x (FAIL) | - |" in out
    assert "| M=512, N=512, K=512 | bf16 | 0.00 % | 1.00 % | 0.50 % (FAIL) | - |" in out      # of 2500 TFLOP/s
    assert "| M=256, N=384, K=512 | fp8 | - | - | - | 1.00 % |" in out                          # of 5000 TFLOP/s
    assert out.rstrip().endswith("4 rows, 1 failed.")


def test_kernel_stats(tmp_path):
    p = tmp_path / "x_kernel_stats.csv"
    p.write_text('"Name","Calls","TotalDurationNs","AverageNs","Percentage","MinNs","MaxNs","StdDev"\n'
                 '"gemm_nt_kernel<Cfg>",25,10000000,400000.0,92.5,376925,480155,31705.0\n')
    out = md.render(TEXT.splitlines(), str(p))
    assert "| `gemm_nt_kernel<Cfg>` | 25 | 400.00 | 376.93 | 480.15 | 92.50 |" in out


def test_empty_input():
    assert md.render([]) == "No benchmark rows found.\n"
