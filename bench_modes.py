"""Tuning and probing modes of bench.py (one JSON line each; none of them is on the path of a plain `python bench.py`
run): --vendor-sweep, --shape, --stream-sweep, --mid-sweep, --skinny-probe.  The summaries in profiles/ cite them as
their commands."""
import json
import sys

from bench_util import LOAD_MS, _graph_time, _quant_fp8, _quant_i8, _time_launches, _time_under_load

# the shapes of the reference's report (TechniqueReport.md:117-121, 151-155) and a few that do not tile evenly
SWEEP_SHAPES = [(1024, 512, 2048), (2048, 2048, 2048), (4096, 4096, 4096), (8192, 4096, 2048), (8192, 4096, 4096),
                (8192, 8192, 8192), (6144, 6144, 6144), (6144, 4608, 7168), (4096, 14336, 4096), (4000, 4000, 4096),
                (512, 4096, 4096), (2048, 2048, 8192), (2048, 4096, 4096), (1024, 8192, 8192),
                # row counts that are whatever a batch holds, against weight shapes
                (1000, 4096, 4096), (3000, 8192, 4096), (5000, 4096, 7168), (7000, 7168, 2048), (200, 7168, 4096)]


def vendor_sweep(Q, torch, dev):
    """Median over eight interleaved blocks of ten launches each, this library and the vendor's in turn (so both see
    the same clocks), per shape and input type.  Times are microseconds per call as a Python caller sees them on an
    otherwise idle stream: below about 25 us the vendor figure is torch's dispatch, not its kernel."""
    def med(fn_a, fn_b, rounds=8, per_block=10):
        for _ in range(3):
            fn_a(); fn_b()
        ta, tb = [], []
        for _ in range(rounds):
            ta.append(_time_launches(fn_a, per_block, 0)[1] * 1e3)
            tb.append(_time_launches(fn_b, per_block, 0)[1] * 1e3)
        ta.sort(); tb.sort()
        return ta[rounds // 2], tb[rounds // 2]
    rows = []
    for fam in ("fp8", "int8", "bf16"):
        for (M, N, K) in SWEEP_SHAPES:
            if fam == "fp8":
                a, sa = _quant_fp8(torch.randn(M, K, device=dev)); b, sb = _quant_fp8(torch.randn(N, K, device=dev))
                c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
                ours = lambda: Q.scaled_gemm(a, b, sa, sb, c, M, N, K, Q.SCALE_PER_MATRIX)
                theirs = lambda: torch._scaled_mm(a, b.t(), scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)
            elif fam == "int8":
                a, sa = _quant_i8(torch.randn(M, K, device=dev)); b, sb = _quant_i8(torch.randn(N, K, device=dev))
                c = torch.empty(M, N, dtype=torch.int32, device=dev)
                ours = lambda: Q.int8_mm(a, b, sa, sb, c)
                theirs = lambda: torch._int_mm(a, b.t())
            else:
                a = torch.randn(M, K, device=dev).bfloat16(); b = torch.randn(N, K, device=dev).bfloat16()
                c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
                ours = lambda: Q.bf16_mm(a, b, c)
                theirs = lambda: torch.matmul(a, b.t(), out=c)
            row = {"type": fam, "M": M, "N": N, "K": K}
            try:
                t_ours, t_theirs = med(ours, theirs)
                row.update({"this_library_us": round(t_ours, 1), "vendor_us": round(t_theirs, 1),
                            "ratio": round(t_ours / t_theirs, 3), "kernel": Q.last_config()})
            except Exception as e:                  # a vendor row that does not run is reported, not hidden
                row["error"] = str(e)[:200]
            rows.append(row)
            print("[sweep]", json.dumps(row), file=sys.stderr, flush=True)
    return rows


def one_shape(Q, torch, dev, spec, launches):
    """`--shape fp8:2048x2048x8192` (fp8 | fp8block | int8 | bf16 | fp16): this library alone on one shape, `launches`
    calls from a replayed graph after as many to warm up (and, for kernels of 20 us or more, LOAD_MS of further untimed
    replays); for profiling a single kernel, or for trying a shape."""
    fam, dims = spec.split(":")
    M, N, K = (int(x) for x in dims.lower().split("x"))
    c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    if fam == "fp8":
        a, sa = _quant_fp8(torch.randn(M, K, device=dev)); b, sb = _quant_fp8(torch.randn(N, K, device=dev))
        fn = lambda: Q.scaled_gemm(a, b, sa, sb, c, M, N, K, Q.SCALE_PER_MATRIX)
    elif fam == "fp8block":
        a, _ = _quant_fp8(torch.randn(M, K, device=dev)); b, _ = _quant_fp8(torch.randn(N, K, device=dev))
        KB = (K + 127) // 128
        sa = (torch.rand(M, KB, device=dev) + 0.5) / 448; sb = (torch.rand((N + 127) // 128, KB, device=dev) + 0.5) / 448
        fn = lambda: Q.scaled_gemm(a, b, sa, sb, c, M, N, K, Q.SCALE_BLOCK128)
    elif fam in ("int8", "int8f32"):                        # int8: bf16 out; int8f32: fp32 out (config 2's output type)
        a, sa = _quant_i8(torch.randn(M, K, device=dev)); b, sb = _quant_i8(torch.randn(N, K, device=dev))
        if fam == "int8f32":
            c = torch.empty(M, N, dtype=torch.float32, device=dev)
        fn = lambda: Q.int8_mm(a, b, sa, sb, c)
    elif fam in ("bf16", "fp16"):
        dt = torch.bfloat16 if fam == "bf16" else torch.float16
        a = torch.randn(M, K, device=dev).to(dt); b = torch.randn(N, K, device=dev).to(dt)
        c = torch.empty(M, N, dtype=dt, device=dev)
        fn = lambda: Q.gemm(a, b, c, "nk")
    else:
        raise SystemExit("bench.py --shape: type must be fp8, fp8block, int8, int8f32, bf16 or fp16")
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(launches):
            fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(); g.replay(); e1.record()
    torch.cuda.synchronize()
    # kernels of 20 us or more: LOAD_MS of untimed replays first, so that the clock of a part that was idle has settled
    # (bench_util.LOAD_MS; shorter kernels run slower, not faster, behind a long run of nothing but themselves)
    first_ms = e0.elapsed_time(e1)
    heavy = first_ms * 1e3 / launches >= 20.0
    if heavy:
        for _ in range(int(LOAD_MS / first_ms) + 1):
            g.replay()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(); g.replay(); e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / launches
    out = {"type": fam, "M": M, "N": N, "K": K, "kernel": Q.last_config(), "launches": launches, "us_per_launch": round(us, 2),
           "tflops": round(2.0 * M * N * K / us / 1e6, 1)}
    # With the measurement build of the library (QGEMM_LIBRARY=qgemm_amd/libqgemm_dbg.so, `make DEBUG=1`): the time
    # stamps gemm_nt_kernel takes per wave (start, K loop entered, K loop left, end; a 100 MHz clock all CUs share) of
    # one eager launch that follows twenty untimed ones (kernels of 20 us or more: LOAD_MS of them), summarised per round of workgroups (CUs at a time).
    try:
        Q.set_option("dbg_ptr", 0)
    except Q.QgemmError:
        return out
    if "+" in out["kernel"] or "|" in out["kernel"] or "skinny" in out["kernel"] or "splitk" in out["kernel"]:
        return out
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    slots = 1 << 16                                          # workgroups x waves of any variant on any shape tried here
    buf = torch.zeros(slots * 4, dtype=torch.int64, device=dev)
    Q.set_option("dbg_ptr", buf.data_ptr())
    for _ in range(max(20, int(LOAD_MS * 1e3 / us) if heavy else 0)):
        fn()
    buf.zero_()
    torch.cuda.synchronize()
    fn()
    torch.cuda.synchronize()
    Q.set_option("dbg_ptr", 0)
    t = buf.view(slots, 4).double() * 10.0                   # ticks -> ns
    used = t[:, 3] > 0
    n_waves = int(used.sum())
    t = t[:n_waves]
    t0 = float(t[:, 0].min())
    # stamps of a workgroup = those of its first wave
    nw = 8 if "w2x4" in out["kernel"] or "w1x4_k2" in out["kernel"] else 4
    nw = {"128x128_w2x2_k2": 12, "64x128_w1x4_k2": 12, "256x128_w2x2_cw": 8, "256x128_w2x2_cw_ks": 8}.get(out["kernel"].replace("_tn", "").replace("_nn", ""), nw)
    w = t[::nw]
    n_wg = w.shape[0]
    rounds = []
    for r0 in range(0, n_wg, cus):
        g = w[r0:r0 + cus]
        rounds.append({"workgroups": int(g.shape[0]), "start_us": round(float(g[:, 0].mean() - t0) / 1e3, 2),
                       "to_k_loop_us": round(float((g[:, 1] - g[:, 0]).mean()) / 1e3, 2),
                       "k_loop_us": round(float((g[:, 2] - g[:, 1]).mean()) / 1e3, 2),
                       "us_per_k_step": round(float((g[:, 2] - g[:, 1]).mean()) / 1e3 / ((K * (2 if fam in ("bf16", "fp16") else 1) + 127) // 128), 3),
                       "k_loop_end_us": round(float(g[:, 2].mean() - t0) / 1e3, 2),
                       "epilogue_us": round(float((g[:, 3] - g[:, 2]).mean()) / 1e3, 2),
                       "end_us_mean": round(float(g[:, 3].mean() - t0) / 1e3, 2), "end_us_last": round(float(g[:, 3].max() - t0) / 1e3, 2)})
    out["stamps"] = {"waves": n_waves, "workgroups": n_wg, "waves_per_workgroup": nw, "rounds_of_%d_CUs" % cus: rounds}
    return out


STREAM_SHAPES = [(1, 8192, 8192), (16, 4096, 4096), (16, 4096, 14336), (64, 4096, 14336), (16, 8192, 8192), (64, 8192, 8192),
                 (128, 8192, 8192), (16, 14336, 4096), (32, 14336, 4096), (64, 14336, 4096), (128, 14336, 4096),
                 (16, 28672, 8192), (64, 28672, 8192), (128, 28672, 4096), (32, 8192, 28672), (16, 7168, 2048),
                 (64, 7168, 2048), (128, 7168, 2048),
                 # few columns (grouped-query K / V projections, small experts): where the tile choice fills the CUs with
                 # small tiles or narrow strips instead of a K split across workgroups
                 (16, 1024, 8192), (64, 1024, 8192), (64, 1024, 4096), (128, 1024, 4096), (128, 2048, 4096), (256, 2048, 4096)]


def stream_sweep(Q, torch, dev):
    """Decode-size row counts against weight matrices streamed out of HBM: B rotates through enough buffers (700 MB) that
    no launch finds its B in the 256 MB memory-side cache; this library and the vendor library, each as a replayed graph
    of one launch per buffer.  Microseconds per launch and TB/s of algorithmic bytes (B + A + C)."""
    rows = []
    for fam in ("fp8", "bf16"):
        for (M, N, K) in STREAM_SHAPES:
            es = 1 if fam == "fp8" else 2
            nbuf = max(2, int(700e6 // (N * K * es)) + 1)
            c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
            if fam == "fp8":
                bs = [_quant_fp8(torch.randn(N, K, device=dev))[0] for _ in range(nbuf)]
                a, sa = _quant_fp8(torch.randn(M, K, device=dev))
                sb = torch.ones(1, device=dev)
                ours = [(lambda b=b: Q.scaled_gemm(a, b, sa, sb, c, M, N, K, Q.SCALE_PER_MATRIX)) for b in bs]
                theirs = [(lambda b=b: torch._scaled_mm(a, b.t(), scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)) for b in bs]
            else:
                bs = [torch.randn(N, K, device=dev).bfloat16() for _ in range(nbuf)]
                a = torch.randn(M, K, device=dev).bfloat16()
                ours = [(lambda b=b: Q.bf16_mm(a, b, c)) for b in bs]
                theirs = [(lambda b=b: torch.matmul(a, b.t(), out=c)) for b in bs]
            nbytes = (N * K + M * K) * es + M * N * 2
            row = {"type": fam, "M": M, "N": N, "K": K, "buffers": nbuf}
            t_ours = _graph_time(ours, reps=6)
            row.update({"this_library_us": round(t_ours, 1), "this_library_TBps": round(nbytes / t_ours / 1e6, 2), "kernel": Q.last_config()})
            try:
                t_theirs = _graph_time(theirs, reps=6)
                row.update({"vendor_us": round(t_theirs, 1), "vendor_TBps": round(nbytes / t_theirs / 1e6, 2), "ratio": round(t_ours / t_theirs, 3)})
            except Exception as e:                  # a vendor row that does not run is reported, not hidden
                row["error"] = str(e)[:200]
            rows.append(row)
            print("[stream]", json.dumps(row), file=sys.stderr, flush=True)
            del bs
    return rows


MID_ROWS = (160, 256, 512, 768, 1024, 1536, 2048, 2560, 3072)
MID_WEIGHTS = ((4096, 4096), (14336, 4096), (4096, 14336), (7168, 2048), (2048, 7168), (8192, 8192))      # N x K


def mid_sweep(Q, torch, dev):
    """Mid-size row counts against weight shapes (9 x 6 shapes, fp8 per-matrix and bf16): this library and the vendor
    library, each as a replayed graph of eight launches on resident operands, so that torch's dispatch does not count.
    Microseconds per launch."""
    rows = []
    for fam in ("fp8", "bf16"):
        for (N, K) in MID_WEIGHTS:
            if fam == "fp8":
                b, sb = _quant_fp8(torch.randn(N, K, device=dev))
            else:
                b = torch.randn(N, K, device=dev).bfloat16()
            for M in MID_ROWS:
                c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
                if fam == "fp8":
                    a, sa = _quant_fp8(torch.randn(M, K, device=dev))
                    ours = lambda: Q.scaled_gemm(a, b, sa, sb, c, M, N, K, Q.SCALE_PER_MATRIX)
                    theirs = lambda: torch._scaled_mm(a, b.t(), scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)
                else:
                    a = torch.randn(M, K, device=dev).bfloat16()
                    ours = lambda: Q.bf16_mm(a, b, c)
                    theirs = lambda: torch.matmul(a, b.t(), out=c)
                row = {"type": fam, "M": M, "N": N, "K": K}
                t_ours = _graph_time([ours] * 8, reps=5)
                row.update({"this_library_us": round(t_ours, 1), "kernel": Q.last_config()})
                try:
                    t_theirs = _graph_time([theirs] * 8, reps=5)
                    row.update({"vendor_us": round(t_theirs, 1), "ratio": round(t_ours / t_theirs, 3)})
                except Exception as e:                  # a vendor row that does not run is reported, not hidden
                    row["error"] = str(e)[:200]
                rows.append(row)
                print("[mid]", json.dumps(row), file=sys.stderr, flush=True)
    return rows


SPLIT_SHAPES = [(6144, 4608, 7168), (4096, 14336, 4096), (4096, 14336, 7168), (8192, 7168, 4096), (8192, 4608, 4096),
                (8192, 4608, 2048), (4096, 4608, 4096), (2048, 28672, 4096), (6144, 6144, 6144), (5120, 5120, 5120),
                (3072, 14336, 4096), (7000, 7168, 2048)]


def split_sweep(Q, torch, dev):
    """Shapes whose 256 x 256 tiles leave a partly empty last round of CUs: one launch, the rows of the full rounds and
    the rows below as two launches, the same with columns, and what the planner takes (option "row_split" 0 / 2 / 3 /
    1), fp8 per-matrix, fp8 with block scales and bf16; microseconds per launch, ten launches behind LOAD_MS of the
    same call, the four settings in turn, twice; the vendor library beside them where it has the type."""
    rows = []
    for fam in ("fp8", "fp8block", "bf16"):
        for (M, N, K) in SPLIT_SHAPES:
            c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
            vend = None
            if fam == "bf16":
                a = torch.randn(M, K, device=dev).bfloat16(); b = torch.randn(N, K, device=dev).bfloat16()
                fn = lambda: Q.bf16_mm(a, b, c)
                vend = lambda: torch.matmul(a, b.t(), out=c)
            else:
                a, sa = _quant_fp8(torch.randn(M, K, device=dev)); b, sb = _quant_fp8(torch.randn(N, K, device=dev))
                if fam == "fp8":
                    fn = lambda: Q.scaled_gemm(a, b, sa, sb, c, M, N, K, Q.SCALE_PER_MATRIX)
                    vend = lambda: torch._scaled_mm(a, b.t(), scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)
                else:
                    KB = (K + 127) // 128
                    sa = (torch.rand(M, KB, device=dev) + 0.5) / 448; sb = (torch.rand((N + 127) // 128, KB, device=dev) + 0.5) / 448
                    fn = lambda: Q.scaled_gemm(a, b, sa, sb, c, M, N, K, Q.SCALE_BLOCK128)
            row = {"type": fam, "M": M, "N": N, "K": K}
            try:
                for rep in range(2):
                    for key, mode in (("one_launch", 0), ("rows", 2), ("columns", 3), ("planner", 1)):
                        Q.set_option("row_split", mode)
                        row.setdefault(key + "_us", []).append(round(_time_under_load(fn, 10, 3) * 1e3, 1))
                        row[key] = Q.last_config()
                    if vend is not None:
                        row.setdefault("vendor_us", []).append(round(_time_under_load(vend, 10, 3) * 1e3, 1))
            finally:
                Q.set_option("row_split", 1)
            rows.append(row)
            print("[split]", json.dumps(row), file=sys.stderr, flush=True)
    return rows


def skinny_probe(Q, torch, dev):
    """Where a launch of the skinny-M kernel spends its time (config 5 shapes, fp8):
      * graph-replay time per launch with B resident against the number of 32-column strips (= workgroups), K and
        M unchanged: tells a limit inside a CU from one in the L2 / fabric;
      * with the measurement build of the library (QGEMM_LIBRARY=qgemm_amd/libqgemm_dbg.so, `make DEBUG=1`): the
        kernel's own time stamps (100 MHz clock shared by all CUs), means over all waves of eager launches."""
    K = 2048
    out = {"resident_us_by_strips": {}, "stamps_ns": {}}
    for M in (16, 64, 128):
        a, sa = _quant_fp8(torch.randn(M, K, device=dev))
        for N in (896, 1792, 3584, 7168):
            b, sb = _quant_fp8(torch.randn(N, K, device=dev))
            c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
            us = _graph_time([lambda: Q.scaled_gemm(a, b, sa, sb, c, M, N, K, Q.SCALE_PER_MATRIX, split_k=1)] * 24)
            out["resident_us_by_strips"]["M%d_strips%d" % (M, N // 32)] = round(us, 2)
    # every row of the skinny-M kernel that can run each M of config 5, forced by name: what a workgroup pulls through
    # its CU's load path (its rows of A and its columns of B, K bytes each) against the time of a launch
    N, nbuf = 7168, 24
    bs = [_quant_fp8(torch.randn(N, K, device=dev)) for _ in range(nbuf)]
    out["by_row"] = {}
    for M, rows in ((16, ("skinny_16x32_k8",)), (32, ("skinny_32x32_k8",)), (64, ("skinny_64x32_k8", "skinny_64x64_k8")),
                    (128, ("skinny_128x32_k8", "skinny_64x64_k8"))):
        a, sa = _quant_fp8(torch.randn(M, K, device=dev))
        c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
        for name in rows:
            tm, tn = (int(v) for v in name.split("_")[1].split("x"))
            Q.force_config(name)
            mk = lambda bq, sbq: (lambda: Q.scaled_gemm(a, bq, sa, sbq, c, M, N, K, Q.SCALE_PER_MATRIX, split_k=1))
            us_rot = _graph_time([mk(*p) for p in bs])
            us_res = _graph_time([mk(*bs[0])] * nbuf)
            assert Q.last_config() == name, (Q.last_config(), name)
            out["by_row"]["M%d_%s" % (M, name)] = {
                "workgroups": ((M + tm - 1) // tm) * (N // tn), "kib_per_workgroup": (min(M, tm) + tn) * K // 1024,
                "us_rotated": round(us_rot, 2), "us_resident": round(us_res, 2)}
    Q.force_config(None)
    del bs
    try:
        Q.set_option("dbg_ptr", 0)
    except Q.QgemmError:
        out["stamps_ns"] = "needs the measurement build: QGEMM_LIBRARY=qgemm_amd/libqgemm_dbg.so"
        return out
    N, NS, nbuf = 7168, 6, 24
    buf = torch.zeros(224 * 8 * NS, dtype=torch.int64, device=dev)
    Q.set_option("dbg_ptr", buf.data_ptr())
    bs = [_quant_fp8(torch.randn(N, K, device=dev)) for _ in range(nbuf)]
    names = ("wave_start", "copies_issued", "unused", "k_loop_done", "past_barrier", "kernel_end")
    for M in (16, 64, 128):
        a, sa = _quant_fp8(torch.randn(M, K, device=dev))
        c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
        for mode in ("rotated", "resident"):
            acc, last = None, 0.0
            for r in range(30):
                b, sb = bs[r % nbuf] if mode == "rotated" else bs[0]
                buf.zero_()
                torch.cuda.synchronize()
                Q.scaled_gemm(a, b, sa, sb, c, M, N, K, Q.SCALE_PER_MATRIX)
                torch.cuda.synchronize()
                if r < 6:
                    continue
                t = buf.view(224 * 8, NS).double() * 10.0             # 100 MHz ticks -> ns
                rel = t - t[:, 0].min()
                row = rel.mean(dim=0)
                acc = row if acc is None else acc + row
                last += float(rel[:, 5].max())
            acc /= 24
            out["stamps_ns"]["M%d_%s" % (M, mode)] = dict(
                {n: round(float(v)) for n, v in zip(names, acc.tolist()) if n != "unused"}, last_wave_end=round(last / 24))
    Q.set_option("dbg_ptr", 0)
    return out
