#!/usr/bin/env python3
"""Benchmark of the scaled-GEMM hot path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one pass of the hot path over one batch of synthetic input already
resident in HBM: one fp8-e4m3 per-matrix-scaled GEMM, M = N = K = 8192, fp32
accumulation, bf16 output (BASELINE.json config 3, the shape the metric is quoted
on).  Prints ONE JSON line.  `value` is TFLOP/s = 2*M*N*K / time.

Timing protocol: W warm-up launches, then K launches bracketed by
torch.cuda.synchronize() (wall clock, `ms_per_step`) and by a pair of HIP events
on the launch stream (`roofline.achieved`): the reference harness's protocol
(tests/includes/test_config.h:110-135, simple_timer.h:27-41) with its TFLOPS
formula (:146-147).  That window is taken twice: as the first GPU work of the
process (`cold_start`: the part was idle and its clock is still rising), and
again behind the other configs and 300 more launches of the same GEMM, with no
pause (`value`: the part under load).  See LOAD_MS in bench_util.py.  The tuning and
probing modes (--shape, --vendor-sweep, --mid-sweep, --stream-sweep, --split-sweep, --skinny-probe) live in
bench_modes.py.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import bench_modes  # noqa: E402
from bench_util import (LOAD_MS, PEAK_HBM_GBS, PEAK_TFLOPS, _graph_time, _quant_fp8, _quant_i8, _time_each_launch,  # noqa: E402
                        _time_launches, _time_under_load)

# HBM-side bytes per launch of the headline kernel, from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE (KiB per dispatch) scaled by what the same counters read for a plain copy of
# known size (`--copy-calibration`).  Measured offline (bench.py cannot run under its own
# profiler); the summaries with the commands are profiles/gemm_nt_f8_256x256_solo8_8192.md and
# profiles/gemm_nt_f8_256x256_solo_8192.md.  Keyed by (kernel name, M): None where no counter run exists.
FETCH_FACTOR = 2.0     # copy of 262144 KiB reads FETCH_SIZE = 131084
WRITE_FACTOR = 1.0     # copy of 262144 KiB reads WRITE_SIZE = 262144
MEASURED_TRAFFIC_BYTES = {      # (FETCH_SIZE KiB * factor + WRITE_SIZE KiB * factor) * 1024, and where the readings are kept
    ("256x256_w2x4_solo8", 8192): ((405763.0 * FETCH_FACTOR + 131072.0 * WRITE_FACTOR) * 1024.0,
                                   "profiles/gemm_nt_f8_256x256_solo8_8192.md"),
    ("256x256_w2x2_solo", 8192): ((399561.0 * FETCH_FACTOR + 131206.0 * WRITE_FACTOR) * 1024.0,
                                  "profiles/gemm_nt_f8_256x256_solo_8192.md"),
}


def measured_traffic(kernel, M):
    """-> (bytes per launch or None, where the figure comes from).  The figure is a constant read off two offline
    rocprofv3 --pmc runs, not measured by this run; a kernel without such a run says so loudly instead of a bare null."""
    hit = MEASURED_TRAFFIC_BYTES.get((kernel, M))
    if hit:
        return hit[0], "constant from offline rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE), %s" % hit[1]
    print("bench.py: WARNING: no HBM traffic counters on record for kernel %r at M=%d; roofline.traffic is null. "
          "Run the two --pmc commands of profiles/gemm_nt_f8_256x256_solo_8192.md for it and add the readings to "
          "MEASURED_TRAFFIC_BYTES." % (kernel, M), file=sys.stderr, flush=True)
    return None, "MISSING: no rocprofv3 --pmc run on record for kernel %s at M=%d" % (kernel, M)


def cpu_baseline(a_q, b_q, sa, sb, rows):
    """The CPU oracle (a port: the reference has no CPU GEMM) on the first `rows` rows of C,
    full N and K, all host cores.  Timed: fp8 decode of the operands + fp32-accumulate GEMM."""
    import numpy as np
    from oracle import cpu_ref as R
    a = a_q[:rows].view(__import__("torch").uint8).cpu().numpy()
    b = b_q.view(__import__("torch").uint8).cpu().numpy()
    N, K = b.shape
    R.gemm_f32acc(R.decode_fp8(a[:8]), R.decode_fp8(b[:64]))       # warm the library and the threads
    t0 = time.perf_counter()
    c = R.gemm_f32acc(R.decode_fp8(a), R.decode_fp8(b)) * np.float32(sa * sb)
    dt = time.perf_counter() - t0
    return {
        "value": 2.0 * rows * N * K / dt / 1e12, "unit": "TFLOP/s", "cores": R.num_threads(), "kind": "port",
        "sample": f"first {rows} rows of C (full N={N}, K={K}) of the same fp8 workload, fp8 decode + fp32-accumulate "
                  f"GEMM, {dt:.2f} s; extrapolated full problem {dt * (a_q.shape[0] / rows):.0f} s",
    }, c


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # defaults long enough to time the steady state: the first launches on an idle part run at boost clock, the
    # next twenty far below it while the power management settles (per-launch trace in profiles/)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--size", type=int, default=8192, help="M = N = K of the headline workload")
    ap.add_argument("--cpu-rows", type=int, default=8192, help="rows of C the CPU baseline computes (0 = skip)")
    ap.add_argument("--no-extra", action="store_true", help="skip the other BASELINE configs")
    ap.add_argument("--no-steady", action="store_true", help="skip the 100 + 200 launch steady-state block")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run three plain device copies of 256 MiB (the known-size kernel the FETCH_SIZE / "
                         "WRITE_SIZE counters are scaled against) and exit")
    ap.add_argument("--vendor-sweep", action="store_true",
                    help="only time this library against the vendor library (torch.matmul, torch._scaled_mm, "
                         "torch._int_mm) over a list of shapes, interleaved, print one JSON line and exit")
    ap.add_argument("--stream-sweep", action="store_true",
                    help="only time decode-size shapes whose weights are streamed out of HBM, this library and the vendor "
                         "library from replayed graphs, print one JSON line and exit")
    ap.add_argument("--mid-sweep", action="store_true",
                    help="only time 160 ... 3072 rows against six weight shapes, this library and the vendor library from "
                         "replayed graphs, print one JSON line and exit")
    ap.add_argument("--split-sweep", action="store_true",
                    help="only time shapes with a partly empty last round of 256 x 256 tiles as one launch, split by rows, "
                         "split by columns and as the planner has it, print one JSON line and exit")
    ap.add_argument("--shape", default="",
                    help="only run this library on one shape, e.g. fp8:2048x2048x8192 (fp8 | fp8block | int8 | int8f32 | bf16 | fp16), "
                         "--steps launches from a replayed graph; print one JSON line and exit")
    ap.add_argument("--skinny-probe", action="store_true",
                    help="only probe where the skinny-M kernel (config 5) spends its time, print one JSON line and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus must be 1 (no multi-GPU path exists).", file=sys.stderr)
        return 2

    import torch
    import qgemm_amd as Q
    Q.load_library()                      # fails loudly if libqgemm.so is missing: there is no fallback
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    if args.copy_calibration:
        n = 1 << 28
        src = torch.full((n,), 3, dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": {"bytes_read": n, "bytes_written": n, "launches": 3}}))
        return 0
    torch.manual_seed(42)                 # seed of the reference harness, tests/includes/test_config.h:64
    dev = "cuda:0"
    if args.shape:
        print(json.dumps({"shape": bench_modes.one_shape(Q, torch, dev, args.shape, max(1, min(args.steps, 200)))}))
        return 0
    if args.stream_sweep:
        print(json.dumps({"stream_sweep": bench_modes.stream_sweep(Q, torch, dev)}))
        return 0
    if args.vendor_sweep:
        print(json.dumps({"vendor_sweep": bench_modes.vendor_sweep(Q, torch, dev)}))
        return 0
    if args.mid_sweep:
        print(json.dumps({"mid_sweep": bench_modes.mid_sweep(Q, torch, dev)}))
        return 0
    if args.split_sweep:
        print(json.dumps({"split_sweep": bench_modes.split_sweep(Q, torch, dev)}))
        return 0
    if args.skinny_probe:
        print(json.dumps({"skinny_probe": bench_modes.skinny_probe(Q, torch, dev)}))
        return 0
    M = N = K = args.size

    # ---- headline: fp8 per-matrix 8192^3 -> bf16
    a_q, sa = _quant_fp8(torch.randn(M, K, device=dev))
    b_q, sb = _quant_fp8(torch.randn(N, K, device=dev))
    c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    run = lambda: Q.scaled_gemm(a_q, b_q, sa, sb, c, M, N, K, Q.SCALE_PER_MATRIX)
    # the driver's window on a part that was idle until now: W launches, then K timed
    cold_wall, cold_ev, cold_per = _time_each_launch(run, args.steps, args.warmup)
    cfg_name = Q.last_config()
    flops = 2.0 * M * N * K
    out = {}

    # ---- the other configs (parity for them is in tests/).  One policy for every entry: 30 timed launches between two
    # HIP events behind LOAD_MS of untimed launches of the same call (at least 10); shapes whose kernel is shorter
    # than a Python call (configs 1 and 5) by replaying a captured graph of 24 launches.
    if not args.no_extra:
        XW, XS = 10, 30
        extra = {"timing": "every entry: %d timed launches between two HIP events behind %.0f ms of untimed launches of the "
                           "same call (at least %d); cfg1, cfg5 and the streamed decode shapes: microseconds per launch of a "
                           "captured graph of 24 launches, replayed 20 times behind 3 untimed replays; the mid_* shapes: graph "
                           "of 8 launches behind %.0f ms of untimed replays" % (XS, LOAD_MS, XW, LOAD_MS)}
        tx = lambda fn: _time_under_load(fn, XS, XW)

        def gemm_entry(ms, fl, peak):
            return {"tflops": fl / ms / 1e9, "frac_of_peak": fl / ms / 1e9 / peak, "ms": ms, "kernel": Q.last_config()}
        ai, sai = _quant_i8(torch.randn(M, K, device=dev))
        bi, sbi = _quant_i8(torch.randn(N, K, device=dev))
        cf = torch.empty(M, N, dtype=torch.float32, device=dev)
        extra["int8_per_matrix_%d" % M] = gemm_entry(tx(lambda: Q.int8_mm(ai, bi, sai, sbi, cf)), flops, PEAK_TFLOPS["i8"])
        # the same product with bf16 output (half the bytes of C; what the headline's fp8 run writes)
        cb16 = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
        extra["int8_per_matrix_%d_bf16_out" % M] = gemm_entry(tx(lambda: Q.int8_mm(ai, bi, sai, sbi, cb16)), flops,
                                                             PEAK_TFLOPS["i8"])
        del ai, bi, cf, cb16
        # cfg 2: int8 4096^3 -> f32
        m2 = 4096
        ai, sai = _quant_i8(torch.randn(m2, m2, device=dev))
        bi, sbi = _quant_i8(torch.randn(m2, m2, device=dev))
        cf = torch.empty(m2, m2, dtype=torch.float32, device=dev)
        extra["cfg2_int8_4096"] = gemm_entry(tx(lambda: Q.int8_mm(ai, bi, sai, sbi, cf)), 2.0 * m2 ** 3, PEAK_TFLOPS["i8"])
        del ai, bi, cf
        # cfg 1: fp16 1024^3, B stored N x K (launch-bound: graph replay)
        m1 = 1024
        ah = (torch.rand(m1, m1, device=dev) * 2 - 1).half()
        bh = (torch.rand(m1, m1, device=dev) * 2 - 1).half()
        ch = torch.empty(m1, m1, dtype=torch.float16, device=dev)
        us = _graph_time([lambda: Q.gemm(ah, bh, ch, "nk")] * 24)
        extra["cfg1_fp16_1024"] = dict(gemm_entry(us * 1e-3, 2.0 * m1 ** 3, PEAK_TFLOPS["f16"]), us_per_launch=us)
        # cfg 4: fp8 block-scaled 6144 x 4608 x 7168
        m4, n4, k4 = 6144, 4608, 7168
        f4 = 2.0 * m4 * n4 * k4
        a4, _ = _quant_fp8(torch.randn(m4, k4, device=dev))
        b4, _ = _quant_fp8(torch.randn(n4, k4, device=dev))
        as4 = torch.rand(m4, k4 // 128, device=dev) * 1.5 + 0.5
        bs4 = torch.rand(n4 // 128, k4 // 128, device=dev) * 1.5 + 0.5
        c4 = torch.empty(m4, n4, dtype=torch.bfloat16, device=dev)
        extra["cfg4_fp8_block_6144x4608x7168"] = gemm_entry(
            tx(lambda: Q.scaled_gemm(a4, b4, as4, bs4, c4, m4, n4, k4, Q.SCALE_BLOCK128)), f4, PEAK_TFLOPS["f8"])
        del a4, b4
        # the same shape with K = 7200: 56 whole K blocks and a quarter of one (K % 32 == 0 is all the reference's
        # dispatch asks for); rows of 7200 bytes are not 128-byte aligned, so every K step of a row spans two lines
        k4t = 7200
        a4t, _ = _quant_fp8(torch.randn(m4, k4t, device=dev))
        b4t, _ = _quant_fp8(torch.randn(n4, k4t, device=dev))
        kb4t = (k4t + 127) // 128
        as4t = torch.rand(m4, kb4t, device=dev) * 1.5 + 0.5
        bs4t = torch.rand(n4 // 128, kb4t, device=dev) * 1.5 + 0.5
        extra["cfg4_shape_k7200_partial_last_k_block"] = gemm_entry(
            tx(lambda: Q.scaled_gemm(a4t, b4t, as4t, bs4t, c4, m4, n4, k4t, Q.SCALE_BLOCK128)), 2.0 * m4 * n4 * k4t, PEAK_TFLOPS["f8"])
        del a4t, b4t
        # int8 operands with the same 128-block scales (each K block's exact int32 partial folded into an fp32 sum): the
        # int8 twin of the reference's block-scaled arithmetic, config 4's shape
        a4i, _ = _quant_i8(torch.randn(m4, k4, device=dev))
        b4i, _ = _quant_i8(torch.randn(n4, k4, device=dev))
        extra["cfg4_shape_int8_block_scales"] = gemm_entry(
            tx(lambda: Q.int8_mm_block(a4i, b4i, as4, bs4, c4)), f4, PEAK_TFLOPS["i8"])
        del a4i, b4i, c4
        # cfg 5: skinny M, N = 7168, K = 2048, int8 (f32 out) and fp8 (bf16 out); bandwidth-bound: GB/s of algorithmic
        # bytes.  "rotated": every launch of the graph reads another B (24 buffers, 352 MB: more than the Infinity
        # Cache holds); "resident": all 24 launches read the same B.
        n5, k5 = 7168, 2048
        nbuf = 24
        for fam in ("fp8", "int8"):
            quant, out_dt, in_dt = ((_quant_fp8, torch.bfloat16, Q.DT_F8E4M3) if fam == "fp8"
                                    else (_quant_i8, torch.float32, Q.DT_I8))
            b5s = [quant(torch.randn(n5, k5, device=dev)) for _ in range(nbuf)]
            for m5 in (16, 64, 128):
                a5, s5a = quant(torch.randn(m5, k5, device=dev))
                c5 = torch.empty(m5, n5, dtype=out_dt, device=dev)
                mk = lambda bq, sbq: (lambda: Q.scaled_gemm(a5, bq, s5a, sbq, c5, m5, n5, k5, Q.SCALE_PER_MATRIX,
                                                            in_dtype=in_dt))
                us_rot = _graph_time([mk(bq, sbq) for (bq, sbq) in b5s])
                us_res = _graph_time([mk(*b5s[0])] * nbuf)
                us_rot_load = _graph_time([mk(bq, sbq) for (bq, sbq) in b5s], load_ms=LOAD_MS)
                # option b_stream = 1: the streaming hint on the copies of B, which the library puts on by itself only
                # for a B of 32 MiB or more (a caller that loops over one small B would find it in the memory-side cache)
                Q.set_option("b_stream", 1)
                us_rot_stream = _graph_time([mk(bq, sbq) for (bq, sbq) in b5s])
                Q.set_option("b_stream", -1)
                nbytes = n5 * k5 + m5 * k5 + m5 * n5 * c5.element_size()
                extra["cfg5_%s_skinny_M%d" % (fam, m5)] = {
                    "us_per_launch_rotated": us_rot, "us_per_launch_resident": us_res,
                    "us_per_launch_rotated_behind_%d_ms_of_replays" % LOAD_MS: us_rot_load,
                    "us_per_launch_rotated_with_option_b_stream": us_rot_stream,
                    "GBps": nbytes / us_rot / 1e3, "frac_of_hbm_peak": nbytes / us_rot / 1e3 / PEAK_HBM_GBS,
                    "GBps_resident": nbytes / us_res / 1e3, "tflops": 2.0 * m5 * n5 * k5 / us_rot / 1e6,
                    "algorithmic_bytes": nbytes, "kernel": Q.last_config()}
            del b5s
        # the same shapes with 128-block scales (the reference's FP8_GEMM_kernel arithmetic at decode-sized M): the
        # skinny-M kernel with the fold in its K loop; bytes as above plus the scales
        b5s = [_quant_fp8(torch.randn(n5, k5, device=dev))[0] for _ in range(nbuf)]
        bs5 = torch.rand(n5 // 128, k5 // 128, device=dev) * 1.5 + 0.5
        for m5 in (16, 64, 128):
            a5, _ = _quant_fp8(torch.randn(m5, k5, device=dev))
            as5 = torch.rand(m5, k5 // 128, device=dev) * 1.5 + 0.5
            c5 = torch.empty(m5, n5, dtype=torch.bfloat16, device=dev)
            mk = lambda bq: (lambda: Q.scaled_gemm(a5, bq, as5, bs5, c5, m5, n5, k5, Q.SCALE_BLOCK128))
            us_rot = _graph_time([mk(bq) for bq in b5s])
            us_res = _graph_time([mk(b5s[0])] * nbuf)
            nbytes = n5 * k5 + m5 * k5 + m5 * n5 * 2 + as5.numel() * 4 + bs5.numel() * 4
            extra["skinny_fp8_block_M%d" % m5] = {
                "us_per_launch_rotated": us_rot, "us_per_launch_resident": us_res,
                "GBps": nbytes / us_rot / 1e3, "frac_of_hbm_peak": nbytes / us_rot / 1e3 / PEAK_HBM_GBS,
                "GBps_resident": nbytes / us_res / 1e3, "algorithmic_bytes": nbytes, "kernel": Q.last_config()}
        del b5s
        # cfg 4 in the reference's own storage (A is K x M, B is K x N, scales [K/128, M] and [K/128, N/128])
        a4r, _ = _quant_fp8(torch.randn(k4, m4, device=dev))
        b4r, _ = _quant_fp8(torch.randn(k4, n4, device=dev))
        as4r = torch.rand(k4 // 128, m4, device=dev) * 1.5 + 0.5
        bs4r = torch.rand(k4 // 128, n4 // 128, device=dev) * 1.5 + 0.5
        c4r = torch.empty(m4, n4, dtype=torch.bfloat16, device=dev)
        extra["cfg4_reference_layout_fp8_mm"] = gemm_entry(
            tx(lambda: Q.fp8_mm(a4r.t(), b4r.t(), as4r.t(), bs4r.t(), c4r)), f4, PEAK_TFLOPS["f8"])
        del a4r, b4r, c4r
        # decode-size rows against large weights streamed out of HBM (B rotates through more buffers than the memory-side
        # cache holds): HBM-bound, bytes = B + A + C
        for (ms_, ns_, ks_) in ((16, 28672, 8192), (128, 28672, 4096)):
            nb_ = int(700e6 // (ns_ * ks_)) + 1
            bs_ = [_quant_fp8(torch.randn(ns_, ks_, device=dev))[0] for _ in range(nb_)]
            as_, sas_ = _quant_fp8(torch.randn(ms_, ks_, device=dev))
            one_ = torch.ones(1, device=dev)
            cs_ = torch.empty(ms_, ns_, dtype=torch.bfloat16, device=dev)
            us = _graph_time([(lambda bq=bq: Q.scaled_gemm(as_, bq, sas_, one_, cs_, ms_, ns_, ks_, Q.SCALE_PER_MATRIX)) for bq in bs_])
            nbytes = ns_ * ks_ + ms_ * ks_ + ms_ * ns_ * 2
            extra["stream_fp8_%dx%dx%d" % (ms_, ns_, ks_)] = {
                "us_per_launch": us, "GBps": nbytes / us / 1e3, "frac_of_hbm_peak": nbytes / us / 1e3 / PEAK_HBM_GBS,
                "buffers": nb_, "algorithmic_bytes": nbytes, "kernel": Q.last_config()}
            del bs_
        # mid-size shapes with no more 128 x 128 tiles than CUs (the rows with two K groups per workgroup), microseconds
        # per launch of a replayed graph: fp8 per-matrix, bf16, and fp8 with block scales in the reference's own storage
        # (read as stored)
        mm, nm_, km = 2048, 2048, 8192
        am, sam = _quant_fp8(torch.randn(mm, km, device=dev)); bm_, sbm = _quant_fp8(torch.randn(nm_, km, device=dev))
        cm = torch.empty(mm, nm_, dtype=torch.bfloat16, device=dev)
        us = _graph_time([lambda: Q.scaled_gemm(am, bm_, sam, sbm, cm, mm, nm_, km, Q.SCALE_PER_MATRIX)] * 8, load_ms=LOAD_MS)
        extra["mid_fp8_2048x2048x8192"] = {"us_per_launch": us, "tflops": 2.0 * mm * nm_ * km / us / 1e6,
                                           "frac_of_peak": 2.0 * mm * nm_ * km / us / 1e6 / PEAK_TFLOPS["f8"], "kernel": Q.last_config()}
        asm_ = (torch.rand(mm, km // 128, device=dev) + 0.5) / 448; bsm_ = (torch.rand(nm_ // 128, km // 128, device=dev) + 0.5) / 448
        us = _graph_time([lambda: Q.scaled_gemm(am, bm_, asm_, bsm_, cm, mm, nm_, km, Q.SCALE_BLOCK128)] * 8, load_ms=LOAD_MS)
        extra["mid_fp8_block_2048x2048x8192"] = {"us_per_launch": us, "tflops": 2.0 * mm * nm_ * km / us / 1e6,
                                                 "frac_of_peak": 2.0 * mm * nm_ * km / us / 1e6 / PEAK_TFLOPS["f8"], "kernel": Q.last_config()}
        # one round of 256 x 128 tiles (the row with copying waves): 2048 x 4096 x 4096, per-matrix and block scales
        nw_, kw_ = 4096, 4096
        aw_, saw_ = _quant_fp8(torch.randn(mm, kw_, device=dev)); bw_, sbw_ = _quant_fp8(torch.randn(nw_, kw_, device=dev))
        cw_ = torch.empty(mm, nw_, dtype=torch.bfloat16, device=dev)
        us = _graph_time([lambda: Q.scaled_gemm(aw_, bw_, saw_, sbw_, cw_, mm, nw_, kw_, Q.SCALE_PER_MATRIX)] * 8, load_ms=LOAD_MS)
        extra["mid_fp8_2048x4096x4096"] = {"us_per_launch": us, "tflops": 2.0 * mm * nw_ * kw_ / us / 1e6,
                                           "frac_of_peak": 2.0 * mm * nw_ * kw_ / us / 1e6 / PEAK_TFLOPS["f8"], "kernel": Q.last_config()}
        asw_ = (torch.rand(mm, kw_ // 128, device=dev) + 0.5) / 448; bsw_ = (torch.rand(nw_ // 128, kw_ // 128, device=dev) + 0.5) / 448
        us = _graph_time([lambda: Q.scaled_gemm(aw_, bw_, asw_, bsw_, cw_, mm, nw_, kw_, Q.SCALE_BLOCK128)] * 8, load_ms=LOAD_MS)
        extra["mid_fp8_block_2048x4096x4096"] = {"us_per_launch": us, "tflops": 2.0 * mm * nw_ * kw_ / us / 1e6,
                                                 "frac_of_peak": 2.0 * mm * nw_ * kw_ / us / 1e6 / PEAK_TFLOPS["f8"], "kernel": Q.last_config()}
        del aw_, bw_, cw_
        # a partly filled round of 256 x 256 tiles that 192-row tiles fill: 3072 x 4096 x 4096
        mp_ = 3072
        ap_, sap_ = _quant_fp8(torch.randn(mp_, kw_, device=dev)); bp_, sbp_ = _quant_fp8(torch.randn(nw_, kw_, device=dev))
        cp_ = torch.empty(mp_, nw_, dtype=torch.bfloat16, device=dev)
        us = _graph_time([lambda: Q.scaled_gemm(ap_, bp_, sap_, sbp_, cp_, mp_, nw_, kw_, Q.SCALE_PER_MATRIX)] * 8, load_ms=LOAD_MS)
        extra["mid_fp8_3072x4096x4096"] = {"us_per_launch": us, "tflops": 2.0 * mp_ * nw_ * kw_ / us / 1e6,
                                           "frac_of_peak": 2.0 * mp_ * nw_ * kw_ / us / 1e6 / PEAK_TFLOPS["f8"], "kernel": Q.last_config()}
        del ap_, bp_, cp_
        ab16, bb16 = torch.randn(mm, km, device=dev).bfloat16(), torch.randn(nm_, km, device=dev).bfloat16()
        us = _graph_time([lambda: Q.bf16_mm(ab16, bb16, cm)] * 8, load_ms=LOAD_MS)
        extra["mid_bf16_2048x2048x8192"] = {"us_per_launch": us, "tflops": 2.0 * mm * nm_ * km / us / 1e6,
                                            "frac_of_peak": 2.0 * mm * nm_ * km / us / 1e6 / PEAK_TFLOPS["bf16"], "kernel": Q.last_config()}
        del ab16, bb16
        kr = 2048
        amr, _ = _quant_fp8(torch.randn(kr, mm, device=dev)); bmr, _ = _quant_fp8(torch.randn(kr, nm_, device=dev))
        asr = torch.rand(kr // 128, mm, device=dev) * 1.5 + 0.5; bsr = torch.rand(kr // 128, nm_ // 128, device=dev) * 1.5 + 0.5
        us = _graph_time([lambda: Q.fp8_mm(amr.t(), bmr.t(), asr.t(), bsr.t(), cm)] * 8, load_ms=LOAD_MS)
        extra["mid_fp8_mm_reference_layout_2048"] = {"us_per_launch": us, "tflops": 2.0 * mm * nm_ * kr / us / 1e6,
                                                     "frac_of_peak": 2.0 * mm * nm_ * kr / us / 1e6 / PEAK_TFLOPS["f8"], "kernel": Q.last_config()}
        del am, bm_, cm, amr, bmr
        # transpose utility (HBM-bound: 2 * M * N * element bytes)
        for (mt, nt, dtt, nm) in ((8192, 8192, torch.bfloat16, "2B"), (7168, 6144, torch.uint8, "1B")):
            xt = torch.randint(0, 100, (mt, nt), device=dev).to(dtt)
            yt = torch.empty(nt, mt, dtype=dtt, device=dev)
            ms = tx(lambda: Q.matrix_transpose(xt, yt))
            gbs = 2.0 * mt * nt * xt.element_size() / ms / 1e6
            extra["transpose_%s_%dx%d" % (nm, mt, nt)] = {"GBps": gbs, "frac_of_hbm_peak": gbs / PEAK_HBM_GBS, "ms": ms}
        # quantisers (HBM-bound): bytes = input (twice for the two-pass per-matrix form) + one output byte
        xq = torch.randn(m4, k4, device=dev)
        for (mode, nm, passes) in ((Q.QUANT_PER_MATRIX, "per_matrix", 2), (Q.QUANT_BLOCK_1x128, "1x128", 1),
                                   (Q.QUANT_BLOCK_128x128, "128x128", 1)):
            ms = tx(lambda: Q.quantize(xq, torch.float8_e4m3fn, mode))
            gbs = m4 * k4 * (4.0 * passes + 1.0) / ms / 1e6
            extra["quantize_fp8_%s_f32_%dx%d" % (nm, m4, k4)] = {"GBps": gbs, "frac_of_hbm_peak": gbs / PEAK_HBM_GBS, "ms": ms}
        del xq
        # bf16 8192^3 through this library, and the vendor library on the same box in the role cuBLAS plays in
        # the reference's harness (tests/cuda_benchmark.cpp): torch.matmul (bf16) and torch._scaled_mm (fp8,
        # the headline operands), both hipBLASLt underneath, interleaved with this library's kernels.  Reported
        # beside, never part of `value`.
        xb = torch.randn(M, K, device=dev).bfloat16()
        yb = torch.randn(N, K, device=dev).bfloat16()
        cb = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
        extra["bf16_%d" % M] = gemm_entry(tx(lambda: Q.bf16_mm(xb, yb, cb)), flops, PEAK_TFLOPS["bf16"])
        # the same product with B stored K x N (the storage of GEMM_kernel_v1..v5)
        ybt = yb.t().contiguous()
        extra["bf16_nn_%d" % M] = gemm_entry(tx(lambda: Q.gemm(xb, ybt, cb, "kn")), flops, PEAK_TFLOPS["bf16"])
        del ybt
        # interleaved blocks of ten launches, this library and the vendor's in turn, so both see the same clocks
        def interleaved(ours, theirs, rounds=10, per_block=10):
            for _ in range(3):
                ours(); theirs()
            _time_under_load(ours, 1, 2)
            t_ours = t_theirs = 0.0
            for _ in range(rounds):
                t_ours += _time_launches(ours, per_block, 0)[1]
                t_theirs += _time_launches(theirs, per_block, 0)[1]
            return t_ours / rounds, t_theirs / rounds
        vendor = {}
        try:
            mo, mv = interleaved(lambda: Q.bf16_mm(xb, yb, cb), lambda: torch.matmul(xb, yb.t(), out=cb), rounds=6, per_block=5)
            vendor["bf16_%d" % M] = {"this_library_tflops": flops / mo / 1e9, "torch_matmul_tflops": flops / mv / 1e9,
                                     "this_library_ms": mo, "torch_matmul_ms": mv}
        except Exception as e:                      # a library row that does not run is reported, not hidden
            vendor["bf16_%d" % M] = {"error": str(e)[:200]}
        try:
            mo, mv = interleaved(run, lambda: torch._scaled_mm(a_q, b_q.t(), scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16))
            vendor["fp8_per_matrix_%d" % M] = {"this_library_tflops": flops / mo / 1e9, "torch_scaled_mm_tflops": flops / mv / 1e9,
                                               "this_library_ms": mo, "torch_scaled_mm_ms": mv}
        except Exception as e:
            vendor["fp8_per_matrix_%d" % M] = {"error": str(e)[:200]}
        extra["vendor_library"] = vendor
        del xb, yb, cb
        out["extra"] = extra

    # ---- headline: the same operands once the part is under load, as a GEMM inside a training or serving loop finds
    # it.  The 100 + 200 launches of the steady-state block come first (they alone are longer than the 45 ms the clock
    # needs), then, with no pause, the window the command line asks for: W launches, then K timed ones.  The same
    # window on the idle part is `cold_start` above; both are on the line.
    if not args.no_steady:
        _, ss_ms = _time_launches(run, 200, 100)
        out["steady_state"] = {"launches": 200, "warmup": 100, "kernel_ms": ss_ms, "tflops": flops / ss_ms / 1e9,
                               "frac": flops / ss_ms / 1e9 / PEAK_TFLOPS["f8"]}
    wall_ms, ev_ms, per_launch_ms = _time_each_launch(run, args.steps, args.warmup)
    assert Q.last_config() == cfg_name
    tflops_wall = flops / (wall_ms * 1e-3) / 1e12
    tflops_ev = flops / (ev_ms * 1e-3) / 1e12
    traffic, traffic_source = measured_traffic(cfg_name, M)
    head = {
        "metric": "scaled-GEMM TFLOP/s (fp8 e4m3 per-matrix scales, M=N=K=%d), 1 GPU" % M,
        "value": tflops_wall, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall_ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f8e4m3 (fp32 accumulate, bf16 out)", "data": "synthetic",
        "config": {"workload": f"fp8-e4m3 per-matrix-scaled GEMM M=N=K={M}, A MxK and B NxK K-contiguous, bf16 out",
                   "kernel": cfg_name,
                   "timed": "W + K launches with no pause behind the launches of the other configs and of the steady-state "
                            "block (the part under load); cold_start: the same window on a part that was idle"},
        "roofline": {"bound": "mfma", "achieved": tflops_ev, "peak": PEAK_TFLOPS["f8"], "unit": "TFLOP/s",
                     "frac": tflops_ev / PEAK_TFLOPS["f8"], "traffic": traffic, "traffic_source": traffic_source,
                     "traffic_unit": "bytes per launch (L2 <-> fabric, rocprofv3 FETCH_SIZE + WRITE_SIZE, calibrated)",
                     "algorithmic_bytes": float(M * K + N * K + 2 * M * N),
                     "kernel_ms": ev_ms, "flops_per_launch": flops},
        # launch-to-launch period of every timed launch, in order (HIP events between the launches)
        "per_launch_ms": [round(t, 4) for t in per_launch_ms],
        # the same W + K launches as the first GPU work of the process, on a part that was idle: the clock is still on
        # its way up (see LOAD_MS)
        "cold_start": {"ms_per_step": cold_wall, "kernel_ms": cold_ev, "tflops": flops / cold_ev / 1e9,
                       "frac": flops / cold_ev / 1e9 / PEAK_TFLOPS["f8"], "per_launch_ms": [round(t, 4) for t in cold_per]},
    }
    out = dict(head, **out)

    # ---- CPU baseline beside it (bounded sample), and a parity spot check of the timed kernel against it
    if args.cpu_rows > 0:
        rows = min(args.cpu_rows, M)
        base, cref = cpu_baseline(a_q, b_q, float(sa), float(sb), rows)
        out["cpu_baseline"] = base
        import numpy as np
        got = c[:rows].float().cpu().numpy()
        ok = bool(np.all(np.abs(got - cref) <= 1e-2 + 2e-2 * np.abs(cref)))
        out["parity_spot_check"] = {"rows": rows, "rtol": 2e-2, "atol": 1e-2, "pass": ok}
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
