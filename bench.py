#!/usr/bin/env python3
"""Benchmark of TMQ's GPU hot path on one MI355X. The headline is the fused soft-staircase pass; the
other legs of the metric (ternary GEMV / GEMM, ResNet-18 inference, the TMQ share of a ResNet-18 QAT
step) ride along under "also", each with its own `roofline` and `cpu_baseline`.

Workload (BASELINE.json configs[1]): a flat fp32 tensor of 2^26 weights, uniform in [-1,1] with
10 % of the elements placed within +-0.02 of a ternary level, an N(0,1) upstream gradient, and a
sweep over five hardness values of the default schedule. One "step" is one fused pass
(y = S(w), dw = g*S'(w) + gl*Q'(w), loss sum, clamp(w)) over the whole tensor at the next hardness
value of the sweep. Inputs are resident in HBM before the timed region starts.

Prints ONE JSON line: metric soft-step fwd+bwd GB/s on the algorithmic 20 B/element, with a
`roofline` object for the dominant kernel (HIP-event timed per launch) and a `cpu_baseline`
object (the op-for-op torch CPU restatement of the reference path, timed on this host's cores
on a bounded sample).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|softstep|linear|pack|resnet_infer|resnet_qat]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HARDNESS = [0.1, 1.1684210526315788, 3.0004, 4.72, 6.0]   # default schedule, epochs 0/21/79/88/149 of 150
SHARPNESS, STRENGTH = 5.0, 5e-4
HBM_PEAK_GBS = 8000.0
MFMA_FP16_PEAK_TFLOPS = 2500.0


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def timed_cpu(torch, fn, threads, budget_s, min_reps=3, max_reps=15):
    """Median seconds of fn() on `threads` host threads: one warm-up, then repetitions until the
    budget is spent (at least min_reps)."""
    prev = torch.get_num_threads()
    torch.set_num_threads(threads)
    try:
        fn()
        times, t_start = [], time.perf_counter()
        while len(times) < min_reps or (time.perf_counter() - t_start < budget_s and len(times) < max_reps):
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
    finally:
        torch.set_num_threads(prev)
    times.sort()
    return times[len(times) // 2], len(times)
BYTES_PER_ELEM = 20                                        # load w, g; store y, dw, clamp(w)


def measured_traffic(path, n=1 << 26, default_n=1 << 26, key="traffic_bytes"):
    """HBM bytes per launch of a kernel as measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs,
    each scaled by what the same counter reads for a plain copy of known size). Counters cannot be read from
    inside a timed run, so the figure comes from the committed profile summary of the same workload (a line
    `<key>: <bytes>`), and is only handed out for the workload size it was measured at."""
    try:
        if n != default_n:
            return None
        for line in open(os.path.join(ROOT, "profiles", path)):
            if line.startswith(key + ":"):
                return int(line.split(":")[1].split()[0])
    except (OSError, ValueError):
        pass
    return None


def make_inputs(n, torch):
    """Seeded CPU generation (identical bits for the CPU baseline and the GPU)."""
    gen = lambda s: torch.Generator(device="cpu").manual_seed(s)
    w = 2 * torch.rand(n, generator=gen(1)) - 1
    mask = torch.rand(n, generator=gen(2)) < 0.10
    level = torch.randint(-1, 2, (n,), generator=gen(3)).float()
    offset = 0.04 * torch.rand(n, generator=gen(4)) - 0.02
    w[mask] = (level + offset)[mask]
    g = torch.randn(n, generator=gen(5))
    return w, g


def cpu_baseline(torch, sample_n, budget_s=8.0):
    """The reference's CPU op chain (oracle/torch_path.py) on the first sample_n elements of the
    same workload, on all host threads torch uses and on one; GB/s on the same 20 B/element."""
    from oracle import torch_path as tp
    w, g = make_inputs(sample_n, torch)
    gl = 1.0 / sample_n
    threads = torch.get_num_threads()
    k = [0]

    def one():
        tp.fused_step(w, g, HARDNESS[k[0] % len(HARDNESS)], SHARPNESS, STRENGTH, gl, -1.0, 1.0)
        k[0] += 1
    med, reps = timed_cpu(torch, one, threads, budget_s, min_reps=5, max_reps=25)
    med1, reps1 = timed_cpu(torch, one, 1, budget_s / 2, min_reps=3, max_reps=10)
    return {"value": round(sample_n * BYTES_PER_ELEM / med / 1e9, 3), "unit": "GB/s", "cores": threads,
            "kind": "port", "value_1_thread": round(sample_n * BYTES_PER_ELEM / med1 / 1e9, 3), "cpu": cpu_model(),
            "sample": f"first {sample_n} elements of the workload, {reps} ({reps1} on one thread) timed fused steps over "
                      f"the hardness sweep, median; torch {torch.__version__} CPU ops in the reference's op order"}


def bench_softstep(args, torch):
    from tmq_amd import ops, _capi
    dev = torch.device("cuda:0")
    n = args.elements
    w, g = make_inputs(n, torch)
    tw, tg = w.to(dev), g.to(dev)
    del w, g
    gl = float(torch.tensor(1.0, dtype=torch.float32) / torch.tensor(float(n), dtype=torch.float32))
    lib = _capi.load()
    y, dw, wc = torch.empty_like(tw), torch.empty_like(tw), torch.empty_like(tw)
    loss = torch.empty(1, dtype=torch.float64, device=dev)
    ws = torch.empty(lib.tmq_softstep_fused_workspace_bytes(n), dtype=torch.uint8, device=dev)
    out = (y, dw, wc, loss, ws)
    in_launch = not args.two_launch_loss

    def step(i):
        # the loss sum is finished by the pass itself (one launch per step); --two-launch-loss: block partial sums
        # to a workspace and a finalisation launch behind every pass
        ops.softstep_fused(tw, tg, HARDNESS[i % len(HARDNESS)], SHARPNESS, STRENGTH, gl, -1.0, 1.0, out=out,
                           in_launch=in_launch)

    if args.copy_calibration:
        # A plain copy of known size (n*4 B read + n*4 B written) for scaling rocprofv3's
        # FETCH_SIZE / WRITE_SIZE counters; not part of the timed region.
        y.copy_(tw)
    # Let clocks settle: a fixed 60 ms of the same kernel before the W warm-up steps (not timed).
    t_settle = time.perf_counter()
    while time.perf_counter() - t_settle < args.settle_ms * 1e-3:
        step(0)
        torch.cuda.synchronize()
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    # One HIP-event pair on the launch stream around the K timed steps (per-launch event pairs would
    # put a barrier between launches and time the dispatch gaps instead of the kernel).
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for i in range(args.steps):
        step(i)
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    avg_ms = e0.elapsed_time(e1) / args.steps
    bytes_per_launch = n * BYTES_PER_ELEM
    value = bytes_per_launch * args.steps / wall / 1e9
    achieved = bytes_per_launch / (avg_ms * 1e-3) / 1e9
    res = {
        "metric": "soft-step fwd+bwd GB/s", "value": round(value, 2), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall / args.steps * 1e3, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: fused soft-step fwd+bwd+qloss+clamp, flat fp32 tensor, hardness sweep "
                               "over 5 schedule values", "elements": n, "bytes_per_element": BYTES_PER_ELEM,
                   "hardness": HARDNESS, "sharpness": SHARPNESS, "strength": STRENGTH},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": measured_traffic("softstep_fused_2p26.md", n),
                     "algorithmic_bytes": bytes_per_launch,
                     "kernel": "stream_kernel<FusedOp<15>, Single, InLaunch> (the loss sum finished inside the launch)"
                               if in_launch else "stream_kernel<FusedOp<15>> (+ 1-block loss finalisation in the same call)",
                     "avg_launch_us": round(avg_ms * 1e3, 3)},
    }
    if not args.no_cpu:
        res["cpu_baseline"] = cpu_baseline(torch, args.cpu_sample)
    return res


def bench_linear(args, torch):
    """BASELINE configs[2]: y = x W^T, K = N = 4096, 2-bit packed ternary W (P(0) = .5), fp16 x, one
    fp32 scale per output channel, fp32 accumulation; M in {1, 16, 256, 4096}. M = 1 rotates over
    distinct weight buffers (> 256 MB in total) so that the packed weights come from HBM, not
    from L2 / Infinity Cache."""
    from tmq_amd import ops
    dev = torch.device("cuda:0")
    K = N = 4096
    gen = lambda s: torch.Generator(device="cpu").manual_seed(s)
    u = torch.rand(N, K, generator=gen(10))
    W = torch.where(u < .25, 1.0, torch.where(u < .5, -1.0, 0.0))
    packed = ops.compactify_ternary(W.to(dev))
    scale = (0.5 + torch.rand(N, generator=gen(11))).to(dev)
    nrot = 72 if args.rotate else 1
    natives = [ops.NativeWeights(packed.clone(), N) for _ in range(nrot)]
    if args.copy_calibration:
        # a plain copy of known size (64 MiB read + 64 MiB written) for scaling rocprofv3's FETCH_SIZE / WRITE_SIZE
        cal = torch.empty(1 << 24, dtype=torch.float32, device=dev)
        torch.empty_like(cal).copy_(cal)
    out = {}
    for M in [int(m) for m in args.m_list.split(",")]:
        x = torch.randn(M, K, generator=gen(12)).half().to(dev)
        reps = args.steps if M < 4096 else max(10, args.steps // 4)
        for i in range(max(args.warmup, 3)):
            ops.ternary_linear(x, natives[i % nrot], scale)
        torch.cuda.synchronize()
        # One pass over the rotating weight buffers is captured in a HIP graph (kernel launches only),
        # so that the figure is the kernel's own rate and not the Python call overhead between launches.
        graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
        per_graph = nrot if M < 4096 else 4
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                for i in range(per_graph):
                    ops.ternary_linear(x, natives[i % nrot], scale)
        replays = max(2, reps // per_graph)
        t_settle = time.perf_counter()
        while time.perf_counter() - t_settle < args.settle_ms * 1e-3:
            graph.replay()
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(replays):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) / (replays * per_graph) * 1e3
        flops = 2.0 * M * N * K
        byts = K * N / 4 + 2 * M * K + 4 * M * N + 4 * N
        out[str(M)] = {"us": round(us, 3), "tflops": round(flops / us / 1e6, 3), "gbs": round(byts / us / 1e3, 2),
                       "frac_hbm": round(byts / us / 1e3 / HBM_PEAK_GBS, 4),
                       "frac_mfma_fp16": round(flops / us / 1e6 / 2500.0, 4)}
    extra = {}
    if args.gemv_floor:
        extra = _gemv_floor_and_large(args, torch, natives)
        # fp32 activations, the reference's own calling convention (tmq/tmq.py:680-683 hands fp32 rows to its kernels):
        # ops.ternary_linear splits them into fp16 row pairs in a workspace (one launch, inside the timed call) and
        # runs the fp16 kernels once over twice the rows -- 22 significant bits per value
        f32 = {}
        for M in (256, 4096):
            x = torch.randn(M, K, generator=gen(13)).to(dev)
            per_graph = 24 if M < 4096 else 4

            def run32(x=x, per_graph=per_graph):
                for i in range(per_graph):
                    ops.ternary_linear(x, natives[i % nrot], scale)
                return per_graph
            run32()
            us = _graph_time_us(torch, run32, max(2, args.steps // 8), args.settle_ms)
            f32[str(M)] = {"us": round(us, 3), "tflops": round(2.0 * M * N * K / us / 1e6, 3)}
        extra["by_M_fp32_rows"] = f32
    res = {"metric": "ternary-GEMM eff. TFLOP/s (K=N=4096)", "unit": "TFLOP/s", "n_gpus": 1, "dtype": "f16",
           "data": "synthetic", "config": {"workload": "configs[2]: ternary linear K=N=4096", "rotate_buffers": nrot},
           "value": out.get("4096", {}).get("tflops"), "by_M": out, **extra}
    if "4096" in out:
        o = out["4096"]
        res["roofline"] = {"bound": "mfma", "achieved": o["tflops"], "peak": MFMA_FP16_PEAK_TFLOPS, "unit": "TFLOP/s",
                           "frac": o["frac_mfma_fp16"],
                           "traffic": measured_traffic("ternary_linear_k4096_n4096.md", key="traffic_bytes_m4096"),
                           "algorithmic_bytes": int(K * N / 4 + 2 * 4096 * K + 4 * 4096 * N + 4 * N),
                           "algorithmic_flops": 2.0 * 4096 * N * K,
                           "kernel": "tile_solo_kernel<128 x 512> (M = 4096)", "avg_launch_us": o["us"]}
    if "1" in out:
        o = out["1"]
        res["roofline_gemv"] = {"bound": "hbm", "achieved": o["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                "frac": o["frac_hbm"],
                                "traffic": measured_traffic("ternary_linear_k4096_n4096.md", key="traffic_bytes_gemv_4096"),
                                "algorithmic_bytes": int(K * N / 4 + 2 * K + 8 * N),
                                "kernel": "gemv8_kernel (M = 1, fp8 x bf8 MFMA), %d rotating weight buffers" % nrot,
                                "avg_launch_us": o["us"]}
    if "gemv_16384" in extra:
        o = extra["gemv_16384"]
        res["roofline_gemv_16384"] = {"bound": "hbm", "achieved": o["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                      "frac": o["frac_hbm"],
                                      "traffic": measured_traffic("ternary_linear_k4096_n4096.md", key="traffic_bytes_gemv_16384"),
                                      "algorithmic_bytes": int(16384 * 16384 / 4 + 2 * 16384 + 8 * 16384),
                                      "kernel": "gemv8_kernel (M = 1, K = N = 16384, fp8 x bf8 MFMA), 6 rotating weight buffers",
                                      "avg_launch_us": o["us"]}
    if not args.no_cpu:
        res["cpu_baseline"] = cpu_baseline_linear(torch, W, scale.cpu())
    return res


def cpu_baseline_linear(torch, W, scale):
    """The reference's CPU inference of a ternary layer: fp32 F.linear on ternary-valued fp32 weights
    (it has no CPU path for packed weights), then the per-channel scale. M = 4096 and M = 1 at
    K = N = 4096, all host threads and one thread (one thread: 512 of the 4096 rows)."""
    F = torch.nn.functional
    K = W.shape[1]
    threads = torch.get_num_threads()
    gen = torch.Generator(device="cpu").manual_seed(12)
    x = torch.randn(4096, K, generator=gen)
    x1 = x[:1].contiguous()
    xs = x[:512].contiguous()
    t_all, r_all = timed_cpu(torch, lambda: F.linear(x, W) * scale, threads, 4.0)
    t_one, r_one = timed_cpu(torch, lambda: F.linear(xs, W) * scale, 1, 4.0)
    t_v, _ = timed_cpu(torch, lambda: F.linear(x1, W) * scale, threads, 1.0, min_reps=10, max_reps=50)
    t_v1, _ = timed_cpu(torch, lambda: F.linear(x1, W) * scale, 1, 1.0, min_reps=10, max_reps=50)
    fl = 2.0 * W.shape[0] * K
    return {"value": round(fl * 4096 / t_all / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "value_1_thread": round(fl * 512 / t_one / 1e12, 4), "cpu": cpu_model(),
            "gemv_tflops": round(fl / t_v / 1e12, 5), "gemv_tflops_1_thread": round(fl / t_v1 / 1e12, 5),
            "gemv_us": round(t_v * 1e6, 1),
            "sample": f"fp32 F.linear on ternary-valued fp32 weights, K = N = 4096: M = 4096 on {threads} threads "
                      f"({r_all} reps), M = 512 on one thread ({r_one} reps), M = 1 on both; medians; torch {torch.__version__}"}


def _graph_time_us(torch, calls, replays, settle_ms):
    """Capture the launches `calls` issue into one HIP graph and time its replays with events."""
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            n = calls()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < settle_ms * 1e-3:
        graph.replay()
        torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(replays):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / (replays * n) * 1e3


def _gemv_floor_and_large(args, torch, natives):
    """Two reference points for the M = 1 figure: (1) the read floor -- a kernel that only streams the
    same packed bytes with the same launch geometry (tmq_probe_stream_read) -- and (2) the same GEMV at
    K = N = 16384 (64 MiB of packed weights per launch, rotating over 6 buffers), where a launch is
    long enough for bandwidth rather than latency to decide."""
    import ctypes
    from tmq_amd import ops, _capi
    dev = torch.device("cuda:0")
    lib = _capi.load()
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    res = {}

    def probe_calls(bufs):
        def run():
            s = _capi.stream_of(sink)
            for b in bufs:
                _capi.check(lib.tmq_probe_stream_read(_capi.ptr(b), ctypes.c_size_t(b.numel()), _capi.ptr(sink), s), "probe")
            return len(bufs)
        return run

    small = [nw.buf for nw in natives]
    run = probe_calls(small)
    run()
    res["read_floor_4MiB_us"] = round(_graph_time_us(torch, run, max(2, args.steps // len(small)), args.settle_ms), 3)

    K = N = 16384
    W = torch.randint(-1, 2, (N, K), dtype=torch.int8, device=dev)
    packed = ops.compactify_ternary(W)
    del W
    big = [ops.NativeWeights(packed.clone(), N) for _ in range(6)]
    x = torch.randn(1, K, device=dev).half()
    scale = (0.5 + torch.rand(N, device=dev))

    def gemv():
        for nw in big:
            ops.ternary_linear(x, nw, scale)
        return len(big)
    gemv()
    us = _graph_time_us(torch, gemv, max(2, args.steps // 12), args.settle_ms)
    byts = K * N / 4 + 2 * K + 8 * N
    run = probe_calls([nw.buf for nw in big])
    run()
    floor = _graph_time_us(torch, run, max(2, args.steps // 12), args.settle_ms)
    res["gemv_16384"] = {"us": round(us, 3), "gbs": round(byts / us / 1e3, 1), "frac_hbm": round(byts / us / 1e3 / HBM_PEAK_GBS, 4),
                         "read_floor_us": round(floor, 3), "read_floor_gbs": round(K * N / 4 / floor / 1e3, 1)}
    # the same GEMV on activation planes made beforehand (tmq_gemv8_prepare, NOT in the timed region): what a vector
    # multiplied with several layers, or emitted in this form by its producer, costs per layer; and with the
    # preparation launch in front of every GEMV
    planes = ops.gemv8_prepare(x)

    def gemv_planes():
        for nw in big:
            ops.ternary_linear_planes(planes, nw, scale)
        return len(big)

    def gemv_prepare_and_planes():
        for nw in big:
            ops.ternary_linear_planes(ops.gemv8_prepare(x), nw, scale)
        return len(big)
    gemv_planes()
    us_p = _graph_time_us(torch, gemv_planes, max(2, args.steps // 12), args.settle_ms)
    us_pp = _graph_time_us(torch, gemv_prepare_and_planes, max(2, args.steps // 12), args.settle_ms)
    res["gemv_16384"]["planes_prepared_beforehand_us"] = round(us_p, 3)
    res["gemv_16384"]["planes_prepared_beforehand_frac_hbm"] = round(byts / us_p / 1e3 / HBM_PEAK_GBS, 4)
    res["gemv_16384"]["prepare_launch_plus_gemv_us"] = round(us_pp, 3)
    # the same layer against 4 and 16 rows (batched decoding): the weights are still read once
    for rows in (4, 16):
        xr = torch.randn(rows, K, device=dev).half()

        def few(xr=xr):
            for nw in big:
                ops.ternary_linear(xr, nw, scale)
            return len(big)
        few()
        us = _graph_time_us(torch, few, max(2, args.steps // 12), args.settle_ms)
        byts = K * N / 4 + 2 * rows * K + 4 * N + 4 * rows * N
        res["rows%d_16384" % rows] = {"us": round(us, 3), "gbs": round(byts / us / 1e3, 1),
                                      "frac_hbm": round(byts / us / 1e3 / HBM_PEAK_GBS, 4)}
    # fp32 rows, the reference's own convention (tmq/tmq_cuda.cu:242-286 takes an fp32 vector): one row is scaled and
    # split into its two fp16 terms inside the GEMV; four rows are split once into fp16 row pairs (a launch of its
    # own, inside the timed call) and take one pass of the fp16 weight stream
    for rows in (1, 4):
        xr = torch.randn(rows, K, device=dev)

        def few32(xr=xr):
            for nw in big:
                ops.ternary_linear(xr, nw, scale)
            return len(big)
        few32()
        us = _graph_time_us(torch, few32, max(2, args.steps // 12), args.settle_ms)
        byts = K * N / 4 + 4 * rows * K + 4 * N + 4 * rows * N
        res["rows%d_16384_fp32" % rows] = {"us": round(us, 3), "gbs": round(byts / us / 1e3, 1),
                                           "frac_hbm": round(byts / us / 1e3 / HBM_PEAK_GBS, 4)}
    # 17 and 32 rows: ops.ternary_linear brings a workspace, so the product runs with its reduction cut across
    # workgroups (tmq_ternary_linear_ws: partial sums + an ordered second launch, both inside the timed call); the same
    # rows through the entry point without a workspace beside it
    for rows in (17, 32):
        xr = torch.randn(rows, K, device=dev).half()
        ys = torch.empty((rows, N), dtype=torch.float32, device=dev)
        ep = _capi.Epilogue(scale.data_ptr(), None, None, 0, _capi.F32)

        def with_ws(xr=xr):
            for nw in big:
                ops.ternary_linear(xr, nw, scale)
            return len(big)

        def without_ws(xr=xr):
            s = _capi.stream_of(xr)
            for nw in big:
                _capi.check(lib.tmq_ternary_linear(_capi.ptr(xr), _capi.F16, rows, K, _capi.ptr(nw.buf), N, ctypes.byref(ep),
                                                   _capi.ptr(ys), s), "ternary_linear")
            return len(big)
        with_ws()
        without_ws()
        us = _graph_time_us(torch, with_ws, max(2, args.steps // 12), args.settle_ms)
        us0 = _graph_time_us(torch, without_ws, max(2, args.steps // 12), args.settle_ms)
        byts = K * N / 4 + 2 * rows * K + 4 * N + 4 * rows * N
        res["rows%d_16384" % rows] = {"us": round(us, 3), "without_workspace_us": round(us0, 3), "gbs": round(byts / us / 1e3, 1),
                                      "frac_hbm": round(byts / us / 1e3 / HBM_PEAK_GBS, 4),
                                      "kernel": "rows_split_kernel + splitk_reduce_kernel (tmq_ternary_linear_ws)"}
    return res


def bench_layers(args, torch):
    """The layer types beside Linear / Conv2d (groups == 1): depthwise convolutions (tmq/tmq_cuda.cu:166-238) and
    transposed convolutions (tmq/tmq.py:978-1087) from 2-bit weights, fp16 NHWC. Memory-bound (one multiply-add per loaded
    element for the depthwise ones): reported as bytes of input + output per second against the HBM peak. Rotating
    inputs, HIP-graph replays."""
    import tmq_amd as t
    from tmq_amd import ops
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(7)
    res = {"metric": "depthwise / transposed ternary layers", "unit": "us", "n_gpus": 1, "dtype": "f16", "data": "synthetic",
           "config": {"workload": "batch 64, 128 channels, 56 x 56 depthwise windows; ConvTranspose2d 128 -> 64, 4 x 4 / 2, 56 x 56, batch 32; first layer 3 -> 64, 3 x 3 / 1, 32 x 32, batch 128"}}
    B, C, H, W = 64, 128, 56, 56
    xs = [torch.randn((B, C, H, W), device=dev, generator=g).half().contiguous(memory_format=torch.channels_last) for _ in range(4)]
    for name, k, pad, dil in (("dw3x3", (3, 3), 1, 1), ("dw3x5", (3, 5), (1, 2), 1), ("dw3x3_dilated2", (3, 3), 2, 2), ("dw5x5", (5, 5), 2, 1)):
        Wt = torch.randint(-1, 2, (C, 1) + k, device=dev, generator=g).float()
        words = ops.compactify_ternary(Wt)

        def run(words=words, k=k, pad=pad, dil=dil):
            for x in xs:
                ops.ternary_dwconv2d(x, words, k, 1, pad, dil, out_dtype=torch.float16)
            return len(xs)
        run()
        us = _graph_time_us(torch, run, max(2, args.steps // 4), args.settle_ms)
        byts = 2 * xs[0].numel() * 2
        res[name] = {"us": round(us, 3), "gbs": round(byts / us / 1e3, 1), "frac_hbm": round(byts / us / 1e3 / HBM_PEAK_GBS, 4)}
    # depthwise transposed convolution (tmq/tmq_cuda.cu:118-162), 128 channels, 28 x 28 -> 56 x 56, 4 x 4 / 2, gathered
    # per output position
    xh = [torch.randn((B, C, 28, 28), device=dev, generator=g).half().contiguous(memory_format=torch.channels_last) for _ in range(4)]
    words_t = ops.compactify_ternary(torch.randint(-1, 2, (C, 1, 4, 4), device=dev, generator=g).float())

    def run_dwt():
        for x in xh:
            ops.ternary_dwconvtrans2d(x, words_t, 4, 2, 1, 0, 1, out_dtype=torch.float16)
        return len(xh)
    run_dwt()
    us = _graph_time_us(torch, run_dwt, max(2, args.steps // 4), args.settle_ms)
    byts = 5 * xh[0].numel() * 2
    res["dwconvtrans4x4s2"] = {"us": round(us, 3), "gbs": round(byts / us / 1e3, 1), "frac_hbm": round(byts / us / 1e3 / HBM_PEAK_GBS, 4)}
    net = torch.nn.Sequential(torch.nn.ConvTranspose2d(128, 64, 4, 2, 1, bias=True))
    ctrl = t.QuantizationControl()
    t.quantize_model(net, ctrl)
    net.to(dev).eval()
    ctrl.quantize()
    t.compressed_state_dict(net, strong=False)
    prev = t.set_compact_output_dtype(torch.float16)
    try:
        xt = [torch.randn((32, 128, 56, 56), device=dev, generator=g).half().contiguous(memory_format=torch.channels_last) for _ in range(4)]
        with torch.no_grad():
            y = net(xt[0])

            def run_t():
                for x in xt:
                    net(x)
                return len(xt)
            us = _graph_time_us(torch, run_t, max(2, args.steps // 4), args.settle_ms)
    finally:
        t.set_compact_output_dtype(prev)
    byts = (xt[0].numel() + y.numel()) * 2
    res["convtranspose_128_64_k4s2"] = {"us": round(us, 3), "launches": 4, "out_MB": round(y.numel() * 2 / 1e6, 1), "gbs": round(byts / us / 1e3, 1),
                                        "note": "one stride-1 implicit-GEMM convolution per output phase, written in place (tmq_ternary_conv2d_view)"}
    # a small-image network's opening (3 -> 64, 3 x 3, stride 1, 32 x 32, batch 128, NCHW fp16 in, fp16 NHWC out): the
    # pixel-pair form of Conv2d.compact_forward (repack launch + one convolution launch; tmq/tmq.py:822-871)
    first = torch.nn.Sequential(torch.nn.Conv2d(3, 64, 3, 1, 1, bias=True))
    ctrl = t.QuantizationControl()
    t.quantize_model(first, ctrl)
    first.to(dev).eval()
    ctrl.quantize()
    t.compressed_state_dict(first, strong=False)
    prev = t.set_compact_output_dtype(torch.float16)
    try:
        xf = [torch.randn((128, 3, 32, 32), device=dev, generator=g).half() for _ in range(4)]
        with torch.no_grad():
            yf = first[0].compact_forward(xf[0], relu=True)

            def run_f():
                for x in xf:
                    first[0].compact_forward(x, relu=True)
                return len(xf)
            us = _graph_time_us(torch, run_f, max(2, args.steps // 4), args.settle_ms)
    finally:
        t.set_compact_output_dtype(prev)
    byts = (xf[0].numel() + yf.numel()) * 2
    res["first_layer_3_64_k3s1"] = {"us": round(us, 3), "launches": 2, "gbs": round(byts / us / 1e3, 1),
                                    "note": "input pixel pairs as 8 channels, output pixel pairs as 128 filters (Conv2d._pixelpair_plan)"}
    res["value"] = res["dw3x3"]["us"]
    res["roofline"] = {"bound": "hbm", "achieved": res["dw3x3"]["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": res["dw3x3"]["frac_hbm"],
                       "traffic": measured_traffic("depthwise_layers_batch64.md", key="traffic_bytes_dw3x3"),
                       "algorithmic_bytes": 2 * xs[0].numel() * 2, "kernel": "dwconv_square_image_kernel<3, 4, 1, 1, 3>",
                       "avg_launch_us": res["dw3x3"]["us"]}
    return res


def bench_pack(args, torch):
    """2-bit pack / unpack of a 4096 x 4096 fp32 weight matrix (the layer of BASELINE configs[2]): 4.25 B per
    weight (4 on the fp32 side, 1/4 on the packed side). Rotates over distinct fp32 buffers (> 256 MB in total)
    so that nothing comes from L2 / Infinity Cache; HIP-graph replays, events on the launch stream."""
    from tmq_amd import _capi
    lib = _capi.load()
    dev = torch.device("cuda:0")
    N = K = 4096
    nb = 7
    Ws = [torch.randint(-1, 2, (N, K), device=dev).float() for _ in range(nb)]
    outs = [torch.empty((K, N // 16), dtype=torch.int32, device=dev) for _ in range(nb)]
    if args.copy_calibration:
        Ws[1].copy_(Ws[0])          # a copy of known size (64 MiB read + 64 MiB written) for scaling the traffic counters

    def pack():
        s = _capi.stream_of(Ws[0])
        for w, o in zip(Ws, outs):
            _capi.check(lib.tmq_pack_ternary(_capi.ptr(w), _capi.F32, N, K, _capi.ptr(o), s), "pack")
        return nb

    def unpack():
        s = _capi.stream_of(Ws[0])
        for w, o in zip(Ws, outs):
            _capi.check(lib.tmq_unpack_ternary(_capi.ptr(o), N, K, _capi.ptr(w), s), "unpack")
        return nb
    pack()
    torch.cuda.synchronize()
    byts = N * K * 4.25
    res = {"metric": "2-bit pack / unpack GB/s", "unit": "GB/s", "n_gpus": 1, "dtype": "u32", "data": "synthetic",
           "config": {"workload": "pack / unpack of a 4096 x 4096 fp32 matrix, %d rotating buffers" % nb}}
    for name, fn in (("pack", pack), ("unpack", unpack)):
        us = _graph_time_us(torch, fn, max(3, args.steps // nb), args.settle_ms)
        res[name] = {"us": round(us, 3), "gbs": round(byts / us / 1e3, 1)}
        res["roofline" if name == "pack" else "roofline_unpack"] = {
            "bound": "hbm", "achieved": round(byts / us / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(byts / us / 1e3 / HBM_PEAK_GBS, 4),
            "traffic": measured_traffic("pack_4096.md", key="traffic_bytes_" + name), "algorithmic_bytes": int(byts),
            "kernel": ("pack_wide_kernel<float, 4, 1>" if name == "pack" else "unpack_wide_kernel<8>"), "avg_launch_us": round(us, 3)}
    res["value"] = res["pack"]["gbs"]
    if not args.no_cpu:
        res["cpu_baseline"] = cpu_baseline_pack(torch, N, K)
    return res


def cpu_baseline_pack(torch, N, K):
    """The reference's packer on the host: compactify_ternary of tmq/tmq_native.cpp:418-425 (a scalar double
    loop, matrixTo2BitTernary 152-171) from the reference's own file compiled under oracle/_ref when that
    library is in the tree ("reference"), else the C restatement of the same loop in oracle/ ("port"). One
    host thread (the loop has no parallel form), the whole 4096 x 4096 matrix, GB/s on the same 4.25 B/weight."""
    import importlib.util
    gen = torch.Generator(device="cpu").manual_seed(10)
    W = torch.randint(-1, 2, (N, K), generator=gen).float()
    so = os.path.join(ROOT, "oracle", "_ref", "tmq_native.so")
    kind, fn = "port", None
    if os.path.exists(so):
        try:
            spec = importlib.util.spec_from_file_location("tmq_native", so)
            mod = importlib.util.module_from_spec(spec)
            spec.loader.exec_module(mod)
            kind, fn = "reference", (lambda: mod.compactify_ternary(W))
        except (ImportError, OSError):
            fn = None
    if fn is None:
        from tests import oracle_lib
        Wn = W.numpy()
        fn = lambda: oracle_lib.pack(Wn)
    t, reps = timed_cpu(torch, fn, 1, 6.0)
    return {"value": round(N * K * 4.25 / t / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": kind, "cpu": cpu_model(),
            "ms": round(t * 1e3, 2),
            "sample": f"compactify_ternary of the whole {N} x {K} fp32 matrix, one thread, {reps} reps, median"}


def _resnet_for_inference(torch, dev, calibrated):
    """ResNet-18 / 102 classes with i.i.d. ternary weights (P(0) = .5), every layer switched to compact weights.
    calibrated=False: BatchNorm exactly as BASELINE configs[3] words it (running_mean ~ N(0, 0.1), running_var ~
    U(0.5, 2), gamma 1, beta 0). calibrated=True: BatchNorm statistics taken from the batch, so that the
    activations are finite and of order one in every layer (bench_models.calibrate_batchnorm_)."""
    import tmq_amd as t
    from bench_models import ResNet18, randomize_ternary_, calibrate_batchnorm_
    torch.manual_seed(20)
    model = ResNet18(102)
    t.quantize_model(model, t.QuantizationControl())
    randomize_ternary_(model, torch.Generator().manual_seed(20))
    model.to(dev)
    if calibrated:
        xc = torch.randn(8, 3, 224, 224, generator=torch.Generator().manual_seed(20)).half().to(dev)
        calibrate_batchnorm_(model, xc, torch.Generator().manual_seed(21))
    model.eval()
    t.compressed_state_dict(model, strong=False)              # switches every layer to compact weights
    return model


def bench_resnet_infer(args, torch):
    """BASELINE configs[3]: ResNet-18 (102 classes) ternary inference, batch 64 of 3x224x224 fp16.

    Two networks are timed. `value` / `modes` are the configuration as BASELINE words it. With unscaled ternary
    weights and running_var ~ U(0.5, 2) every 3 x 3 convolution multiplies the activation scale by ~17, so from
    the end of layer1 on its fp16 activations are Inf / NaN (`output_finite` false): the kernels do all the work,
    but on degenerate data. `calibrated` is the same network with BatchNorm statistics taken from the batch
    (finite activations of order one in every layer, `output_finite` true); it is the figure to compare kernels by."""
    import tmq_amd as t
    dev = torch.device("cuda:0")
    B = args.batch or 64
    x = torch.randn(B, 3, 224, 224, generator=torch.Generator().manual_seed(20)).half().to(dev)

    def timed(fn, reps):
        with torch.no_grad():
            for _ in range(max(2, args.warmup // 4)):
                out = fn()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0 = time.perf_counter()
            e0.record()
            for _ in range(reps):
                out = fn()
            e1.record()
            torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / reps
        finite = bool(torch.isfinite(out.float()).all().item())     # after the timed loop, not inside it
        return {"ms": round(dt * 1e3, 4), "gpu_ms": round(e0.elapsed_time(e1) / reps, 4), "img_s": round(B / dt, 1),
                "tflops": round(3.627e9 * B / dt / 1e12, 2), "output_finite": finite}

    few = max(3, args.steps // 4)
    if args.resnet_variant == "calibrated_fused":      # for profiling: the runner on finite activations and nothing else
        runner = t.ResNetRunner(_resnet_for_inference(torch, dev, calibrated=True))
        f = timed(lambda: runner(x), args.steps)
        return {"metric": "ResNet-18 img/s", "value": f["img_s"], "unit": "img/s", "n_gpus": 1, "dtype": "f16",
                "data": "synthetic", "config": {"workload": "configs[3]: ResNet-18/102 ternary inference, calibrated BatchNorm, "
                                                              "tmq_amd.ResNetRunner only", "batch": B}, "calibrated": {"fused": f}}
    # ---- the configuration as worded
    model = _resnet_for_inference(torch, dev, calibrated=False)
    runner = t.ResNetRunner(model)
    out = {"fused": timed(lambda: runner(x), args.steps)}
    out["drop_in"] = timed(lambda: model(x), few)
    t.fold_batchnorm(model)                                   # BatchNorm into the convolutions' epilogues
    out["drop_in_bn_folded"] = timed(lambda: model(x), few)
    prev = t.set_compact_output_dtype(torch.float16)          # fp16 channels_last between the layers
    try:
        out["drop_in_bn_folded_fp16"] = timed(lambda: model(x), few)
        t.use_native_pooling(model)                           # the library's fp16 NHWC max-pool / average pool
        out["drop_in_bn_folded_fp16_pooling"] = timed(lambda: model(x), few)
        gm = t.fuse_epilogues(model)[0]                       # ReLU / residual add into the kernels' epilogues (torch.fx)
        out["drop_in_fused_graph"] = timed(lambda: gm(x), few)
        replay = t.GraphedForward(gm)                         # ... and the whole forward recorded as one HIP graph
        out["drop_in_fused_graph_replayed"] = timed(lambda: replay(x), args.steps)
    finally:
        t.set_compact_output_dtype(prev)
    del model, gm, replay
    # ---- the same network with finite activations
    model = _resnet_for_inference(torch, dev, calibrated=True)
    runner = t.ResNetRunner(model)
    cal = {"fused": timed(lambda: runner(x), args.steps)}
    session = t.optimize_for_inference(model)                 # fold + fp16 + pooling + fx fusion + HIP graph in one call
    cal["optimize_for_inference"] = timed(lambda: session(x), args.steps)
    best = max(out, key=lambda k: out[k]["img_s"])
    f = cal["fused"]
    res = {"metric": "ResNet-18 img/s", "value": out["fused"]["img_s"], "unit": "img/s", "n_gpus": 1, "dtype": "f16",
           "data": "synthetic", "config": {"workload": "configs[3]: ResNet-18/102 ternary inference", "batch": B},
           "output_finite": out["fused"]["output_finite"],
           "note": "value: BatchNorm statistics as BASELINE words them -- fp16 activations overflow after layer1, so most "
                   "convolutions multiply Inf / NaN; `calibrated`: the same network with BatchNorm statistics from the "
                   "batch, finite activations in every layer",
           "modes": out, "calibrated": cal, "value_calibrated": f["img_s"],
           "roofline": {"bound": "mfma", "achieved": f["tflops"], "peak": MFMA_FP16_PEAK_TFLOPS,
                        "unit": "TFLOP/s", "frac": round(f["tflops"] / MFMA_FP16_PEAK_TFLOPS, 4), "traffic": None,
                        "algorithmic_flops": 3.627e9 * B,
                        "kernel": "whole forward of tmq_amd.ResNetRunner on the calibrated network (finite activations): 20 "
                                  "ternary implicit-GEMM convolutions, fc, pooling, the input read from its NCHW planes by the opening kernel (21 launches)",
                        "avg_launch_us": round(f["gpu_ms"] * 1e3, 2)},
           "fastest_mode": best}
    if not args.no_cpu:
        res["cpu_baseline"] = cpu_baseline_resnet(torch)
    return res


def cpu_baseline_resnet(torch):
    """The reference's CPU inference mode for a ternarised network: the fp32 model with ternary-valued
    weights through F.conv2d / F.linear (samples/resnet_train.py:255-264), eval-mode BatchNorm. A
    bounded sample of the batch: 16 images on all host threads, 4 on one."""
    from bench_models import ResNet18, randomize_ternary_
    torch.manual_seed(20)
    model = ResNet18(102)
    randomize_ternary_(model, torch.Generator().manual_seed(20))
    model.eval()
    x = torch.randn(16, 3, 224, 224, generator=torch.Generator().manual_seed(20))
    threads = torch.get_num_threads()
    with torch.no_grad():
        t_all, r_all = timed_cpu(torch, lambda: model(x), threads, 5.0)
        t_one, r_one = timed_cpu(torch, lambda: model(x[:4]), 1, 5.0)
    return {"value": round(16 / t_all, 2), "unit": "img/s", "cores": threads, "kind": "port",
            "value_1_thread": round(4 / t_one, 2), "cpu": cpu_model(),
            "sample": f"fp32 ResNet-18/102 with ternary-valued weights (F.conv2d / F.linear, eval BatchNorm): 16 images on "
                      f"{threads} threads ({r_all} reps), 4 images on one thread ({r_one} reps), medians; torch {torch.__version__}"}


def bench_resnet_qat(args, torch):
    """BASELINE configs[4]: one ResNet-18 QAT step, batch 128 fp32, hardness 2.236133, penalty 5e-4."""
    import tmq_amd as t
    from bench_models import ResNet18
    from torch import nn
    dev = torch.device("cuda:0")
    torch.manual_seed(30)
    model = ResNet18(102)
    ctrl = t.QuantizationControl(epoch_knots=t.QuantizationScheduleBuilder.default_schedule(150),
                                 qpenalty_range=(5e-4, 5e-4))
    t.quantize_model(model, ctrl)
    model.to(dev).train()
    for e in range(76):
        ctrl.step(e)
    B = args.batch or 128
    x = torch.randn(B, 3, 224, 224, generator=torch.Generator().manual_seed(30)).to(dev)
    labels = torch.randint(0, 102, (B,), generator=torch.Generator().manual_seed(31)).to(dev)
    opt = torch.optim.Adam(model.parameters(), lr=0.1)

    def step():
        opt.zero_grad(set_to_none=True)
        loss = nn.functional.cross_entropy(model(x), labels) + ctrl.quantization_loss()
        loss.backward()
        opt.step()
        ctrl.clamp()

    reps = max(3, args.steps // 10)
    for _ in range(3):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / reps

    # The TMQ kernels of one step on their own, exactly the launches the step above issues: the
    # multi-tensor soft-step forward with the quantization loss, the multi-tensor backward
    # (g S'(w) + loss gradient), the multi-tensor clamp. Eager (Python call overhead included, what a
    # loop of these calls alone costs) and as HIP-graph replays (the kernels' own time).
    from tmq_amd import tmq as tmq_mod
    b = tmq_mod._b
    ws = [node.weight.data for node in ctrl._registry.values()]
    gs = [torch.randn_like(w) for w in ws]
    up = torch.ones((), device=dev)
    d, sharp, p = ctrl.digamma, float(ctrl.qpenalty_sharpness), float(ctrl.qpenalty)
    n_w = sum(w.numel() for w in ws)
    parts = {"fwd_loss": (lambda: b.softstep_fwd_all(ws, d, True, sharp, p), 8),
             "bwd": (lambda: b.softstep_bwd_all(ws, gs, up, d, sharp, p), 12),
             "clamp": (lambda: ctrl.clamp(), 8)}

    def tmq_only():
        for fn, _ in parts.values():
            fn()
        return 1

    for _ in range(3):
        tmq_only()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(20):
        tmq_only()
    e1.record()
    torch.cuda.synchronize()
    eager_ms = e0.elapsed_time(e1) / 20
    tmq_ms = _graph_time_us(torch, tmq_only, 50, args.settle_ms) / 1e3
    per = {}
    for name, (fn, bpe) in parts.items():
        us = _graph_time_us(torch, lambda fn=fn: (fn(), 1)[1], 50, 10.0)
        per[name] = {"us": round(us, 2), "gbs": round(n_w * bpe / us / 1e3, 1)}
    nbytes = n_w * 28
    res = {"metric": "ResNet-18 QAT step time", "value": round(dt * 1e3, 3), "unit": "ms", "higher_is_better": False,
           "n_gpus": 1, "dtype": "f32", "data": "synthetic",
           "config": {"workload": "configs[4]: ResNet-18 QAT step", "batch": B, "digamma": ctrl.digamma,
                      "qpenalty": ctrl.qpenalty, "quantized_weights": n_w, "layers": len(ws)},
           "tmq_kernels_ms": round(tmq_ms, 4), "tmq_share": round(tmq_ms / (dt * 1e3), 5),
           "tmq_calls_eager_ms": round(eager_ms, 4), "tmq_algorithmic_bytes": nbytes, "tmq_launches": per,
           "roofline": {"bound": "hbm", "achieved": round(nbytes / tmq_ms / 1e6, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": round(nbytes / tmq_ms / 1e6 / HBM_PEAK_GBS, 4), "traffic": None,
                        "algorithmic_bytes": nbytes,
                        "kernel": "the step's TMQ launches: multi-tensor soft-step forward + loss (8 B/weight; the sum "
                                  "finished inside the launch), multi-tensor backward (12 B/weight), multi-tensor clamp (8 B/weight)",
                        "avg_launch_us": round(tmq_ms * 1e3, 2)}}
    if not args.no_cpu:
        res["cpu_baseline"] = cpu_baseline_qat(torch, [w.cpu() for w in ws], d, sharp, p)
    return res


def cpu_baseline_qat(torch, ws, d, sharp, p):
    """The TMQ part of the same step on the reference's CPU op chains (oracle/torch_path.py), layer by
    layer: soft-step forward and backward, loss and its gradient, clamp."""
    from oracle import torch_path as tp
    gs = [torch.randn_like(w) for w in ws]
    threads = torch.get_num_threads()

    def one():
        for w, g in zip(ws, gs):
            tp.fused_step(w, g, d, sharp, p, 1.0 / w.numel(), -1.0, 1.0)
    t_all, r_all = timed_cpu(torch, one, threads, 4.0)
    t_one, r_one = timed_cpu(torch, one, 1, 4.0, min_reps=2)
    return {"value": round(t_all * 1e3, 2), "unit": "ms of TMQ work per step", "cores": threads, "kind": "port",
            "value_1_thread": round(t_one * 1e3, 2), "cpu": cpu_model(),
            "sample": f"all {len(ws)} weight tensors of the network ({sum(w.numel() for w in ws)} weights), {r_all} reps on "
                      f"{threads} threads, {r_one} on one; medians; torch {torch.__version__} CPU ops in the reference's op order"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--settle-ms", type=float, default=60.0)
    ap.add_argument("--copy-calibration", action="store_true")
    ap.add_argument("--two-launch-loss", action="store_true", help="soft-step: finalise the loss in a second launch")
    ap.add_argument("--workload", default="all")
    ap.add_argument("--elements", type=int, default=1 << 26)
    ap.add_argument("--cpu-sample", type=int, default=1 << 22)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--m-list", default="1,16,256,4096")
    ap.add_argument("--rotate", type=int, default=1)
    ap.add_argument("--gemv-floor", type=int, default=1, help="linear workload: also time the read floor and a 16384^2 GEMV")
    ap.add_argument("--batch", type=int, default=0)
    ap.add_argument("--resnet-variant", default="all", help="resnet_infer: all | calibrated_fused (that runner only, for profiling)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build targets one GPU; --gpus N with N > 1 is not supported (the path has no "
              "cross-GPU work).", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    if args.workload == "all":
        # the headline line (soft-step) with the other legs of the metric riding along under "also"
        res = bench_softstep(args, torch)
        torch.cuda.empty_cache()
        res["also"] = {}
        for name, leg in (("linear", bench_linear), ("pack", bench_pack), ("resnet_infer", bench_resnet_infer),
                          ("resnet_qat", bench_resnet_qat), ("layers", bench_layers)):
            res["also"][name] = leg(args, torch)
            torch.cuda.empty_cache()
    elif args.workload == "softstep":
        res = bench_softstep(args, torch)
    elif args.workload == "linear":
        res = bench_linear(args, torch)
    elif args.workload == "pack":
        res = bench_pack(args, torch)
    elif args.workload == "layers":
        res = bench_layers(args, torch)
    elif args.workload == "resnet_infer":
        res = bench_resnet_infer(args, torch)
    elif args.workload == "resnet_qat":
        res = bench_resnet_qat(args, torch)
    else:
        print(f"bench.py: unknown workload {args.workload}", file=sys.stderr)
        sys.exit(2)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
