"""Timing helpers and synthetic operands shared by bench.py and its tuning modes (bench_modes.py)."""
import time

# MI355X published dense peaks
PEAK_TFLOPS = {"f8": 5000.0, "i8": 5000.0, "bf16": 2500.0, "f16": 2500.0}
PEAK_HBM_GBS = 8000.0


def _time_launches(fn, steps, warmup):
    """-> (wall ms per step, event ms per launch)"""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    return wall, e0.elapsed_time(e1) / steps


def _time_each_launch(fn, steps, warmup):
    """-> (wall ms per step, event ms per launch, [ms of every timed launch]): one HIP event between consecutive
    launches, so the launch-to-launch period of each timed launch is on record."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    ev[0].record()
    for i in range(steps):
        fn()
        ev[i + 1].record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    return wall, ev[0].elapsed_time(ev[steps]) / steps, [ev[i].elapsed_time(ev[i + 1]) for i in range(steps)]


# A part that was idle for 10 ms or longer runs its next launches below the clock it settles at: the launch-to-launch
# period of the headline GEMM reads 0.49 ms ten launches in, 0.42 after twenty, 0.38 after fifty and 0.355 from about
# 120 launches (45 ms) on, whatever ran before the pause.  Everything but `cold_start` is therefore timed behind
# LOAD_MS of untimed launches of the same call.
LOAD_MS = 50.0


def _time_under_load(fn, steps, min_warmup):
    """-> event ms per launch of `steps` launches that follow at least LOAD_MS (and `min_warmup` launches) of the same call"""
    _, d = _time_launches(fn, max(2, min_warmup), 2)
    n = int(min(5000, LOAD_MS / max(d, 1e-3)))
    return _time_launches(fn, steps, n)[1]


def _graph_time(fns, reps=20, load_ms=0.0):
    """Microseconds per launch of the launches `fns`, captured once into a HIP graph and replayed `reps` times behind
    three untimed replays and `load_ms` more of them: what a caller that captures its GEMMs sees, without one Python
    call per 5-microsecond kernel.  (Kernels of a few microseconds that are bound by launch and memory latency run
    slower, not faster, behind a long run of nothing but themselves: config 5 at M = 16 reads 5.6 us per launch behind
    0 or 5 ms of its own replays, 6.0 - 6.8 behind 50 ms and 7.4 - 7.9 behind 200 ms.  They are timed behind the three
    replays, as in every earlier record of this file's figures, and config 5 behind LOAD_MS as well.)"""
    import torch
    for f in fns:
        f()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for f in fns:
            f()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(3):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    for _ in range(int(min(5000, load_ms / max(e0.elapsed_time(e1) / 3, 1e-3)))):
        g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / (reps * len(fns))


def _quant_fp8(x):
    import torch
    s = (x.abs().max() / 448.0).float().reshape(1)
    return (x / s).to(torch.float8_e4m3fn), s


def _quant_i8(x):
    import torch
    s = (x.abs().max() / 127.0).float().reshape(1)
    return torch.clamp(torch.round(x / s), -127, 127).to(torch.int8), s
