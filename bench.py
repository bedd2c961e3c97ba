#!/usr/bin/env python3
"""Headline benchmark: the fused soft-staircase pass on one MI355X.

Workload (BASELINE.json configs[1]): a flat fp32 tensor of 2^26 weights, uniform in [-1,1] with
10 % of the elements placed within +-0.02 of a ternary level, an N(0,1) upstream gradient, and a
sweep over five hardness values of the default schedule. One "step" is one fused pass
(y = S(w), dw = g*S'(w) + gl*Q'(w), loss sum, clamp(w)) over the whole tensor at the next hardness
value of the sweep. Inputs are resident in HBM before the timed region starts.

Prints ONE JSON line: metric soft-step fwd+bwd GB/s on the algorithmic 20 B/element, with a
`roofline` object for the dominant kernel (HIP-event timed per launch) and a `cpu_baseline`
object (the op-for-op torch CPU restatement of the reference path, timed on this host's cores
on a bounded sample).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload softstep|gemv|gemm|...]
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
BYTES_PER_ELEM = 20                                        # load w, g; store y, dw, clamp(w)


def measured_traffic(path, n, default_n=1 << 26):
    """HBM bytes per launch of the dominant kernel as measured with rocprofv3 --pmc FETCH_SIZE /
    WRITE_SIZE (scaled by a copy of known size); the figure lives in the committed profile summary.
    Only valid for the workload size it was measured at."""
    try:
        if n != default_n:
            return None
        for line in open(os.path.join(ROOT, "profiles", path)):
            if line.startswith("traffic_bytes:"):
                return int(line.split(":")[1])
    except OSError:
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


def cpu_baseline(torch, sample_n, budget_s=15.0):
    """The reference's CPU op chain (oracle/torch_path.py) on the first sample_n elements of the
    same workload, all host cores torch uses; GB/s on the same 20 B/element."""
    from oracle import torch_path as tp
    w, g = make_inputs(sample_n, torch)
    gl = 1.0 / sample_n
    threads = torch.get_num_threads()
    times = []
    t_start = time.perf_counter()
    reps = 0
    while True:
        d = HARDNESS[reps % len(HARDNESS)]
        t0 = time.perf_counter()
        tp.fused_step(w, g, d, SHARPNESS, STRENGTH, gl, -1.0, 1.0)
        dt = time.perf_counter() - t0
        if reps >= 1:                      # first repetition is the warm-up
            times.append(dt)
        reps += 1
        if (len(times) >= 5 and time.perf_counter() - t_start > budget_s) or len(times) >= 25:
            break
    times.sort()
    med = times[len(times) // 2]
    return {"value": round(sample_n * BYTES_PER_ELEM / med / 1e9, 3), "unit": "GB/s", "cores": threads,
            "kind": "port",
            "sample": f"first {sample_n} elements of the workload, {len(times)} timed fused steps over the hardness "
                      f"sweep, median; torch {torch.__version__} CPU ops in the reference's op order"}


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

    def step(i):
        ops.softstep_fused(tw, tg, HARDNESS[i % len(HARDNESS)], SHARPNESS, STRENGTH, gl, -1.0, 1.0, out=out)

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
                     "kernel": "stream_kernel<FusedOp<15>> (+ 1-block loss finalisation in the same call)",
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
    return {"metric": "ternary-GEMM eff. TFLOP/s (K=N=4096)", "unit": "TFLOP/s", "n_gpus": 1, "dtype": "f16",
            "data": "synthetic", "config": {"workload": "configs[2]: ternary linear K=N=4096", "rotate_buffers": nrot},
            "value": out.get("4096", {}).get("tflops"), "by_M": out, **extra}


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
    return res


def bench_resnet_infer(args, torch):
    """BASELINE configs[3]: ResNet-18 (102 classes) ternary inference, batch 64 of 3x224x224 fp16."""
    import tmq_amd as t
    from bench_models import ResNet18, randomize_ternary_, FusedTernaryResNet18
    dev = torch.device("cuda:0")
    torch.manual_seed(20)
    model = ResNet18(102)
    ctrl = t.QuantizationControl()
    t.quantize_model(model, ctrl)
    randomize_ternary_(model, torch.Generator().manual_seed(20))
    model.to(dev).eval()
    t.compressed_state_dict(model, strong=False)              # switches every layer to compact weights
    B = args.batch or 64
    x = torch.randn(B, 3, 224, 224, generator=torch.Generator().manual_seed(20)).half().to(dev)
    fused = FusedTernaryResNet18(model)
    out, graph = {}, [None]
    for name, fn, reps in (("fused", lambda: fused(x), args.steps), ("drop_in", lambda: model(x), max(3, args.steps // 4)),
                           ("drop_in_bn_folded", lambda: model(x), max(3, args.steps // 4)),
                           ("drop_in_bn_folded_fp16", lambda: model(x), max(3, args.steps // 4)),
                           ("drop_in_bn_folded_fp16_pooling", lambda: model(x), max(3, args.steps // 4)),
                           ("drop_in_fused_graph", lambda: graph[0](x), max(3, args.steps // 4))):
        if name == "drop_in_bn_folded":
            t.fold_batchnorm(model)                           # BatchNorm into the convolutions' epilogues
        if name == "drop_in_bn_folded_fp16":
            t.set_compact_output_dtype(torch.float16)         # fp16 channels_last between the layers
        if name == "drop_in_bn_folded_fp16_pooling":
            t.use_native_pooling(model)                       # the library's fp16 NHWC max-pool / average pool
        if name == "drop_in_fused_graph":
            graph[0] = t.fuse_epilogues(model)[0]             # ReLU / residual add into the kernels' epilogues (torch.fx)
        with torch.no_grad():
            for _ in range(max(2, args.warmup // 4)):
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(reps):
                fn()
            torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / reps
        out[name] = {"ms": round(dt * 1e3, 4), "img_s": round(B / dt, 1), "tflops": round(3.627e9 * B / dt / 1e12, 2)}
    t.set_compact_output_dtype(torch.float32)
    return {"metric": "ResNet-18 img/s", "value": out["fused"]["img_s"], "unit": "img/s", "n_gpus": 1, "dtype": "f16",
            "data": "synthetic", "config": {"workload": "configs[3]: ResNet-18/102 ternary inference", "batch": B},
            "modes": out}


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

    # The TMQ kernels of one step on their own (GPU time between events): soft-step forward and backward
    # of each of the 21 layers, the multi-tensor quantization loss and its gradient, the multi-tensor clamp.
    from tmq_amd import tmq as tmq_mod
    b = tmq_mod._b
    ws = [node.weight for node in ctrl._registry.values()]
    gs = [torch.randn_like(w) for w in ws]

    def tmq_only():
        for w, g in zip(ws, gs):
            b.fwd_softstep(w.data, ctrl.digamma)
            b.bwd_softstep(w.data, ctrl.digamma, 1.0, g)
        ctrl.quantization_loss().backward()
        ctrl.clamp()

    for _ in range(3):
        tmq_only()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        tmq_only()
    e1.record()
    torch.cuda.synchronize()
    tmq_ms = e0.elapsed_time(e1) / reps
    nbytes = sum(w.numel() for w in ws) * (8 + 12 + 4 + 12 + 8)   # fwd, bwd, loss, loss gradient (accumulating), clamp
    return {"metric": "ResNet-18 QAT step time", "value": round(dt * 1e3, 3), "unit": "ms", "higher_is_better": False,
            "n_gpus": 1, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "configs[4]: ResNet-18 QAT step", "batch": B, "digamma": ctrl.digamma,
                       "qpenalty": ctrl.qpenalty, "quantized_weights": 11219136},
            "tmq_kernels_ms": round(tmq_ms, 4), "tmq_share": round(tmq_ms / (dt * 1e3), 4),
            "tmq_algorithmic_bytes": nbytes, "tmq_gbs": round(nbytes / tmq_ms / 1e6, 1)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--settle-ms", type=float, default=60.0)
    ap.add_argument("--copy-calibration", action="store_true")
    ap.add_argument("--workload", default="softstep")
    ap.add_argument("--elements", type=int, default=1 << 26)
    ap.add_argument("--cpu-sample", type=int, default=1 << 22)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--m-list", default="1,16,256,4096")
    ap.add_argument("--rotate", type=int, default=1)
    ap.add_argument("--gemv-floor", type=int, default=1, help="linear workload: also time the read floor and a 16384^2 GEMV")
    ap.add_argument("--batch", type=int, default=0)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build targets one GPU; --gpus N with N > 1 is not supported (the path has no "
              "cross-GPU work).", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    if args.workload == "softstep":
        res = bench_softstep(args, torch)
    elif args.workload == "linear":
        res = bench_linear(args, torch)
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
