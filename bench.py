"""Benchmark of the dense-contraction path on one MI355X.

One "step" is one launch of the hot kernel on inputs already resident in HBM.
The headline workload is the fp16 GEMM M=N=K=4096 (A row-major, B column-major,
fp32 accumulate, fp16 output); the 3x3 implicit-GEMM convolution and the
FlashAttention-2 forward named by the metric are timed in the same run and
reported under "also".  Prints one JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload gemm|gemm_nonsquare|gemm_rowmajor|gemm_f32|gemm_f32_4096|conv|attention|attention_causal|conv_transpose|resnet18_b1|resnet18_b32|copy]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = 2500.0  # MI355X dense fp16/bf16 MFMA peak
PEAKS = {"f16": 2500.0, "bf16": 2500.0, "f32": 157.3}  # dense MFMA peak of the type a workload computes in
FLOP_PER_CLK_PER_CU = {"f16": 4096.0, "bf16": 4096.0, "f32": 256.0}  # dense MFMA rate of one compute unit
# What the roofline blocks take from the rocprofv3 counter runs: HBM-side bytes per launch of a
# workload's dominant kernel (FETCH_SIZE / WRITE_SIZE scaled by a copy of known size) and the shader
# clock that kernel ran at (SQ_BUSY_CYCLES over its duration).  The table is written by
# `python -m tracea_amd.profile_summary` from the counter files of the commands that
# profiles/bench_kernels_mi355x.md lists, and names the kernel each row was measured on.
ROOFLINE_INPUTS = os.path.join(ROOT, "profiles", "roofline_inputs.json")
KERNEL_OF = {"gemm": "gemm", "gemm_nonsquare": "gemm", "gemm_rowmajor": "gemm", "conv": "conv2d",
             "attention": "attention", "attention_causal": "attention"}  # operator whose variant a workload runs
METRIC = "TFLOPS + % fp16 MFMA peak: GEMM 4096^3, 3x3 implicit-GEMM conv, FA2 fwd"


def make_workload(name, torch, ops):
    """Returns (label, flops per step, algorithmic bytes per step, dtype, step function)."""
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(0x7ACEA000)
    if name == "gemm":
        m = n = k = 4096
        a = (torch.randn(m, k, device=dev, generator=g) / k ** 0.5).half()
        bt = (torch.randn(n, k, device=dev, generator=g) / k ** 0.5).half()  # column-major B
        c = torch.empty(m, n, device=dev, dtype=torch.float16)
        b = bt.t()
        return ("fp16 GEMM 4096x4096x4096, A row-major, B column-major, fp32 acc, fp16 out",
                2.0 * m * n * k, 2.0 * (m * k + k * n + m * n), "f16", lambda: ops.gemm(a, b, out=c))
    if name == "gemm_nonsquare":
        # the second shape of the fp16 GEMM configuration, there to exercise the choice of tile shape
        m, n, k = 8192, 2048, 8192
        a = (torch.randn(m, k, device=dev, generator=g) / k ** 0.5).half()
        bt = (torch.randn(n, k, device=dev, generator=g) / k ** 0.5).half()
        c = torch.empty(m, n, device=dev, dtype=torch.float16)
        b = bt.t()
        return ("fp16 GEMM 8192x2048x8192, A row-major, B column-major, fp32 acc, fp16 out",
                2.0 * m * n * k, 2.0 * (m * k + k * n + m * n), "f16", lambda: ops.gemm(a, b, out=c))
    if name == "gemm_rowmajor":
        # the same product with B stored [K,N] row-major, the layout the reference's tracea_gemm documents
        m = n = k = 4096
        a = (torch.randn(m, k, device=dev, generator=g) / k ** 0.5).half()
        b = (torch.randn(k, n, device=dev, generator=g) / k ** 0.5).half()
        c = torch.empty(m, n, device=dev, dtype=torch.float16)
        return ("fp16 GEMM 4096x4096x4096, A and B row-major, fp32 acc, fp16 out",
                2.0 * m * n * k, 2.0 * (m * k + k * n + m * n), "f16", lambda: ops.gemm(a, b, out=c))
    if name in ("gemm_f32", "gemm_f32_4096"):
        # the reference's CPU-runnable case on the device: fp32, row-major, uniform[-1,1] (fp32 MFMA peak 157.3 TFLOP/s)
        m = n = k = 1024 if name == "gemm_f32" else 4096
        a = torch.rand(m, k, device=dev, generator=g) * 2 - 1
        b = torch.rand(k, n, device=dev, generator=g) * 2 - 1
        c = torch.empty(m, n, device=dev)
        return ("fp32 GEMM %dx%dx%d, row-major, uniform[-1,1]" % (m, n, k), 2.0 * m * n * k,
                4.0 * (m * k + k * n + m * n), "f32", lambda: ops.gemm(a, b, out=c))
    if name == "conv":
        n, h, w, cin, cout = 32, 56, 56, 64, 64
        x = torch.randn(n, h, w, cin, device=dev, generator=g).half()
        wt = (torch.randn(cout, 3, 3, cin, device=dev, generator=g) * (2.0 / 576) ** 0.5).half()
        bias = torch.randn(cout, device=dev, generator=g) * 0.1
        y = torch.empty(n, h, w, cout, device=dev, dtype=torch.float16)
        return ("fp16 NHWC conv N32 56x56x64->64 3x3 s1 p1, bias+ReLU",
                2.0 * n * h * w * cout * 9 * cin, 2.0 * (x.numel() + wt.numel() + y.numel()), "f16",
                lambda: ops.conv2d(x, wt, bias=bias, stride=1, padding=1, epilogue="bias+relu", out=y))
    if name in ("attention", "attention_causal"):
        causal = name.endswith("causal")
        b, h, s, d = 4, 32, 4096, 128
        q, k, v = [torch.randn(b, h, s, d, device=dev, generator=g).bfloat16() for _ in range(3)]
        o = torch.empty_like(q)
        flops = 4.0 * b * h * d * (s * (s + 1) / 2.0 if causal else float(s) * s)
        return ("bf16 FA2 forward B4 H32 S4096 D128 %s" % ("causal" if causal else "dense"),
                flops, 2.0 * 4 * q.numel(), "bf16", lambda: ops.attention(q, k, v, causal=causal, out=o))
    if name in ("conv_transpose", "conv_transpose_cached"):
        # the reference's VAE decoder layer at batch 8 (src/optimizer/benchmark.rs:572-575); FLOPs are
        # the products that are not structurally zero, 1/stride^2 of the reference's 2*M*N*K count
        n, h, w, cin, cout, r, st, pd = 8, 32, 32, 512, 256, 4, 2, 1
        x = torch.randn(n, h, w, cin, device=dev, generator=g).half()
        wt = (torch.randn(cin, r, r, cout, device=dev, generator=g) * (1.0 / (4 * cin)) ** 0.5).half()
        ho = (h - 1) * st - 2 * pd + r
        y = torch.empty(n, ho, ho, cout, device=dev, dtype=torch.float16)
        from tracea_amd import capi
        cached = name.endswith("cached")  # the regrouped filter bank kept between calls (constant filters)

        def step():
            capi.lib().tracea_set_conv_transpose_filter_cache(1 if cached else 0)
            ops.conv_transpose2d(x, wt, stride=st, padding=pd, out=y)
            capi.lib().tracea_set_conv_transpose_filter_cache(0)
        return ("fp16 NHWC transposed conv N8 32x32x512->64x64x256 4x4 s2 p1" + (", filter cache on" if cached else ""),
                2.0 * n * h * w * cin * r * r * cout, 2.0 * (x.numel() + wt.numel() + y.numel()), "f16", step)
    if name in ("resnet18_b1", "resnet18_b32"):
        # the reference's network benchmark graph (src/bin/network_bench.rs:41-215), fused, compiled into
        # an execution plan and replayed as one HIP graph; random weights, BatchNorm parameters near identity
        from tracea_amd import graph as G, plan as P
        batch = 1 if name.endswith("b1") else 32
        graph, info = G.resnet18_graph(batch)
        plan = P.Plan(G.fuse(graph))
        image = torch.zeros(batch, 224, 224, 8, device=dev, dtype=torch.float16)
        image[..., :3] = torch.randn(batch, 224, 224, 3, device=dev, generator=g).half()
        plan.bind(info["input"], image)
        flops = 0.0
        for node in graph["operators"]:
            (kind, body), = node.items()
            if kind == "Conv2d":
                ho = (body["h"] + 2 * body["padding"] - body["r"]) // body["stride"] + 1
                flops += 2.0 * body["n"] * ho * ho * body["k"] * body["r"] * body["s"] * (3 if body["c"] == 8 else body["c"])
        flops += 2.0 * batch * 512 * 1000
        for oid, (k, r, s_, c) in info["convs"].items():
            w = (torch.randn(k, r, s_, c, device=dev, generator=g) * (2.0 / (r * s_ * c)) ** 0.5).half()
            plan.bind(oid, w, "weight")
        for oid, (params, c) in info["bn"].items():
            vals = [torch.rand(c, device=dev, generator=g) * 0.5 + 0.75, torch.randn(c, device=dev, generator=g) * 0.1,
                    torch.randn(c, device=dev, generator=g) * 0.1, torch.rand(c, device=dev, generator=g) * 0.5 + 0.75]
            for pid, v in zip(params, vals):
                plan.bind(pid, v)
        plan.bind(info["fc"], (torch.randn(512, 1000, device=dev, generator=g) * 512 ** -0.5).half(), "weight")
        plan.capture()
        return ("fp16 ResNet-18 forward, batch %d, 224x224, %d fused launches replayed as one HIP graph"
                % (batch, len(plan.describe()["steps"])), flops, 0.0, "f16", plan.replay)
    if name in ("basic_block", "downsample_block"):
        # the reference's fused ResNet basic block, N=32: conv3x3+BN+ReLU -> conv3x3+BN+residual+ReLU on 128
        # channels at 28x28, and the downsampling form (64ch 56x56 -> 128ch 28x28, stride-2 first convolution,
        # 1x1 stride-2 shortcut convolution with BN); BN folded to scale/shift, every operator in an epilogue
        from tracea_amd import capi
        n = 32
        down = name == "downsample_block"
        cin, hin = (64, 56) if down else (128, 28)
        ch, ho = 128, 28
        x = torch.randn(n, hin, hin, cin, device=dev, generator=g).half()
        w1 = (torch.randn(ch, 3, 3, cin, device=dev, generator=g) * (2.0 / (9 * cin)) ** 0.5).half()
        w2 = (torch.randn(ch, 3, 3, ch, device=dev, generator=g) * (2.0 / (9 * ch)) ** 0.5).half()
        ws = (torch.randn(ch, 1, 1, cin, device=dev, generator=g) * (2.0 / cin) ** 0.5).half()
        bn = [(torch.rand(ch, device=dev, generator=g) + 0.5, torch.randn(ch, device=dev, generator=g) * 0.1) for _ in range(3)]
        y1 = torch.empty(n, ho, ho, ch, device=dev, dtype=torch.float16)
        sc = torch.empty_like(y1)
        y2 = torch.empty_like(y1)

        def block():
            ops.conv2d_ex(x, w1, [(capi.OP_SCALE_SHIFT,) + bn[0], (capi.OP_RELU,)], stride=2 if down else 1, padding=1, out=y1)
            skip = x
            if down:
                ops.conv2d_ex(x, ws, [(capi.OP_SCALE_SHIFT,) + bn[2]], stride=2, padding=0, out=sc)
                skip = sc
            ops.conv2d_ex(y1, w2, [(capi.OP_SCALE_SHIFT,) + bn[1], (capi.OP_RESIDUAL_ADD, skip), (capi.OP_RELU,)],
                          stride=1, padding=1, out=y2)
        m = n * ho * ho
        flops = 2.0 * m * ch * 9 * cin + 2.0 * m * ch * 9 * ch + (2.0 * m * ch * cin if down else 0.0)
        byts = 2.0 * (x.numel() * (2 if not down else 2) + w1.numel() + w2.numel() + 2 * y1.numel() + y2.numel())
        return ("fp16 NHWC fused ResNet %s block N32 -> 128ch 28x28 (%d launches)" % ("downsampling" if down else "basic", 3 if down else 2),
                flops, byts, "f16", block)
    if name == "gemm_tiles_half":
        # the headline product restricted to a random half of its 128x128 output tiles through a tile
        # list (the reference's examples/ttg_sparse_experiment.rs at full size); FLOPs count listed tiles
        # only.  (With 256x256 tiles half of the list is 124 workgroups for 256 CUs and takes as long as one
        # tile's walk over K, 96 us.)
        from tracea_amd.ttg import TileLayout, gemm_ttg
        m = n = k = 4096
        a = (torch.randn(m, k, device=dev, generator=g) / k ** 0.5).half()
        bt = (torch.randn(n, k, device=dev, generator=g) / k ** 0.5).half()
        c = torch.zeros(m, n, device=dev, dtype=torch.float16)
        lay = TileLayout.from_random(m, n, k, 128, 128, 64, 0.5, seed=11)
        tiles = lay.num_active_tiles
        return ("fp16 GEMM 4096x4096x4096 over a tile list: %d of 1024 tiles of 128x128" % tiles,
                2.0 * tiles * 128 * 128 * k, 2.0 * (m * k + k * n + tiles * 128 * 128), "f16",
                lambda: gemm_ttg(a, bt.t(), lay, c))
    if name == "copy":
        # calibration workload for the HBM traffic counters: a plain device copy of known size
        n = 256 << 20
        src = torch.empty(n, device=dev, dtype=torch.uint8).fill_(1)
        dst = torch.empty(n, device=dev, dtype=torch.uint8)
        return ("device copy of 256 MiB (counter calibration)", 0.0, 2.0 * n, "u8", lambda: dst.copy_(src))
    raise SystemExit("unknown workload " + name)


def roofline_inputs():
    try:
        with open(ROOFLINE_INPUTS) as f:
            return json.load(f).get("workloads", {})
    except (OSError, ValueError):
        return {}


def measure_clock(torch, capi, step, dev_s):
    """Shader clock (GHz) while `step` runs: a one-wave probe kernel on a stream of its own samples the shader's
    tick counter and the constant 100 MHz counter for about 3.5 ms while launches of `step` fill 6 ms or more of
    the main stream; the median of the tick/time slopes over windows of 64 samples is the clock the launches
    ran at (the probe's first windows, taken before the launches reach the device, fall outside the median)."""
    import numpy as np
    samples, gap = 1500, 1
    buf = torch.zeros(2 * samples, dtype=torch.int64, device="cuda:0")
    side = torch.cuda.Stream()
    launches = max(8, int(6e-3 / max(dev_s, 1e-6)) + 1)
    for _ in range(3):
        step()
    torch.cuda.synchronize()
    capi.check("tracea_clock_probe", capi.lib().tracea_clock_probe(buf.data_ptr(), samples, gap, side.cuda_stream))
    for _ in range(launches):
        step()
    torch.cuda.synchronize()
    t = buf.cpu().numpy().reshape(-1, 2).astype(np.float64)
    w = 64
    dticks, dreal = t[w:, 0] - t[:-w, 0], (t[w:, 1] - t[:-w, 1]) * 1e-8  # the real-time counter ticks at 100 MHz
    ok = dreal > 0
    if not ok.any():
        return None
    return float(np.median(dticks[ok] / dreal[ok]) / 1e9)


def roofline_block(name, flops, dev_s, dtype, cus, variant, inputs, clock_ghz=None):
    """achieved = algorithmic flops / HIP-event time per launch; peak = the published one; the peak at the
    clock the kernel ran at uses the clock measured beside the launches of this run (measure_clock); traffic
    comes from the counter table, with `stale` set when the kernel that just ran is not the one the table's
    row was measured on."""
    peak = PEAKS.get(dtype, PEAK_TFLOPS)
    row = inputs.get(name) or {}
    achieved = flops / dev_s / 1e12
    block = {"bound": "mfma", "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s",
             "frac": round(achieved / peak, 4), "traffic": row.get("traffic_bytes")}
    clock, source = clock_ghz, "probe kernel beside the launches, this run (shader ticks over the 100 MHz counter)"
    if not clock and row.get("clock_ghz"):
        clock, source = row["clock_ghz"], "profiles/roofline_inputs.json (another run)"
    if clock:
        at_clock = cus * FLOP_PER_CLK_PER_CU.get(dtype, 4096.0) * clock * 1e9 / 1e12
        block["peak_at_measured_clock"] = round(at_clock, 1)
        block["clock_ghz"] = round(clock, 3)
        block["clock_from"] = source
        # the probe reads the clock of the one CU it sits on, averaged over windows of some 150 us: an upper
        # bound for launches that leave that CU a free wave slot or whose phases alternate (stamps written by
        # the kernels themselves read 1.7-1.9 GHz over a causal attention wave's life and 1.75 GHz over the
        # convolution's main loop where the probe reads 2.4 and 2.2)
        if name in ("conv", "attention_causal"):
            block["clock_is_upper_bound"] = True
        block["frac_of_peak_at_measured_clock"] = round(achieved / at_clock, 4)
    if row:
        block["counters_from"] = row.get("variant")
        block["stale"] = bool(variant) and row.get("variant") not in (None, variant)
    return block


def time_steps(torch, step, steps, warmup):
    """Wall clock around exactly `steps` launches, plus HIP-event time on the launch stream."""
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()  # the kernels are enqueued on torch's current stream, the one these events see
    for _ in range(steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall / steps, e0.elapsed_time(e1) * 1e-3 / steps


def launch_stats(torch, step, launches=50, cold_trials=5):
    """Per-launch figures of the timing protocol: median and minimum over `launches` back-to-back
    launches (one event between each pair; caches are not flushed between them), and the median of
    `cold_trials` single launches that each follow a 1 GiB fill, which leaves nothing of the
    operands in the 32 MB of L2 or the 256 MB memory-side cache."""
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(launches + 1)]
    ev[0].record()
    for i in range(launches):
        step()
        ev[i + 1].record()
    torch.cuda.synchronize()
    ts = sorted(ev[i].elapsed_time(ev[i + 1]) * 1e3 for i in range(launches))
    flush = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0")
    cold = []
    for i in range(cold_trials):
        flush.fill_(i)
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        step()
        e1.record()
        torch.cuda.synchronize()
        cold.append(e0.elapsed_time(e1) * 1e3)
    del flush
    return {"median": round(ts[len(ts) // 2], 2), "min": round(ts[0], 2), "cold_cache": round(sorted(cold)[len(cold) // 2], 2),
            "launches": launches}


def time_steps_graph(torch, step, steps):
    """The same launches recorded once into a HIP graph and replayed: device time per launch without
    the host's per-call cost (about 15 us per call from Python here, which is longer than the shorter
    kernels themselves).  Split-K scratch is sized by the warm-up launches on the capture stream."""
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for _ in range(steps):
            step()
    graph.replay()
    torch.cuda.synchronize()
    best = None
    for _ in range(3):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        t = e0.elapsed_time(e1) * 1e-3 / steps
        best = t if best is None or t < best else best
    return best


def cpu_baseline():
    """The reference's CPU SIMD GEMM (restated gemm_cpu_packed, hero tiling) on the host cores,
    protocol of examples/cpu_bench.rs:34-57: one warm-up call, three timed calls."""
    import numpy as np

    import oracle
    threads = oracle.default_threads()
    out = {}
    for size in (1024, 4096):
        rng = np.random.default_rng(0x7ACEA001)
        a = rng.uniform(-1, 1, (size, size)).astype(np.float32)
        b = rng.uniform(-1, 1, (size, size)).astype(np.float32)
        c = np.zeros((size, size), np.float32)
        oracle.gemm_cpu_packed(a, b, c, nthreads=threads)
        t0 = time.perf_counter()
        for _ in range(3):
            oracle.gemm_cpu_packed(a, b, c, nthreads=threads)
        out[size] = 2.0 * size ** 3 / ((time.perf_counter() - t0) / 3) / 1e12
    return {"value": round(out[4096], 4), "unit": "TFLOPS", "cores": threads, "kind": "port",
            "sample": "fp32 packed AVX2 SGEMM (Mc=Nc=128,Kc=256,Mr=6,Nr=16), 1 warm-up + 3 timed calls at "
                      "4096^3 (value) and at the reference's 1024^3 (%.4f TFLOPS)" % out[1024]}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="gemm")
    ap.add_argument("--no-extras", action="store_true", help="skip the conv/attention/CPU legs")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)")

    import torch

    from tracea_amd import capi, ops
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a HIP device")
    capi.init()

    # Order of the legs: CPU baseline, side workloads, then the headline.  After an idle period
    # the device needs some 20 ms of load before its clocks settle (4096^3: 129 us per launch over the
    # first 50 launches, 116 us from the 150th on); with the side workloads first the headline's
    # warm-up and timed steps run on a device that is already in its steady state.
    cpu = also = None
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    inputs = roofline_inputs()
    if not args.no_extras:
        cpu = cpu_baseline()
        also = {}
        for name in ("gemm", "gemm_nonsquare", "gemm_rowmajor", "gemm_f32", "gemm_f32_4096", "conv", "basic_block", "downsample_block", "attention", "attention_causal",
                     "conv_transpose", "conv_transpose_cached", "resnet18_b1", "resnet18_b32", "gemm_tiles_half"):
            if name == args.workload:
                continue
            lab, fl, by, dt, st = make_workload(name, torch, ops)
            # (two passes, the faster one counts and both are listed: a single host-side stall of tens of
            # milliseconds, seen once per process in the HIP runtime after the CPU leg, would otherwise be a whole
            # leg's figure.  The headline below is one pass.)
            _, d1 = time_steps(torch, st, max(5, args.steps // 2), max(2, args.warmup // 2))
            d2 = time_steps(torch, st, max(5, args.steps // 2), 0)[1]
            d = min(d1, d2)
            also[name] = {"workload": lab, "tflops": round(fl / d / 1e12, 2),
                          "pct_of_peak": round(100.0 * fl / d / 1e12 / PEAKS.get(dt, PEAK_TFLOPS), 2),
                          "us_per_launch": round(d * 1e6, 2), "dtype": dt,
                          "passes_us": [round(d1 * 1e6, 2), round(d2 * 1e6, 2)], "stat": "min of 2 passes"}
            dk = d
            if name in ("conv", "gemm_f32", "basic_block", "downsample_block"):  # launches shorter than the host's per-call cost: also as a replayed graph
                dg = time_steps_graph(torch, st, 40)
                also[name]["us_per_launch_graph"] = round(dg * 1e6, 2)
                also[name]["tflops_graph"] = round(fl / dg / 1e12, 2)
                dk = min(d, dg)
            if name in ("conv", "attention", "attention_causal", "gemm"):  # the workloads the metric names
                # the kernel's duration: events over back-to-back launches, from Python or (where a Python
                # call takes longer than the kernel) over the replayed graph
                also[name]["roofline"] = roofline_block(name, fl, dk, dt, cus, capi.last_variant(KERNEL_OF[name]), inputs,
                                                        measure_clock(torch, capi, st, dk))
                also[name]["roofline"]["timed"] = "graph replay" if dk < d else "stream launches"
            del st
            torch.cuda.empty_cache()

    label, flops, bytes_, dtype, step = make_workload(args.workload, torch, ops)
    wall, dev_s = time_steps(torch, step, args.steps, args.warmup)
    tflops = flops / wall / 1e12
    stats = launch_stats(torch, step)
    clock = measure_clock(torch, capi, step, dev_s)
    line = {
        "metric": METRIC, "value": round(tflops, 2), "unit": "TFLOPS", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall * 1e3, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype,
        "data": "synthetic", "config": {"workload": label, "variant": capi.last_variant(KERNEL_OF[args.workload]) if args.workload in KERNEL_OF else None},
        "pct_of_peak": round(100.0 * tflops / PEAKS.get(dtype, PEAK_TFLOPS), 2),
        "roofline": roofline_block(args.workload, flops, dev_s, dtype, cus,
                                   capi.last_variant(KERNEL_OF[args.workload]) if args.workload in KERNEL_OF else None, inputs, clock),
    }
    line["roofline"]["hbm_GBps_algorithmic"] = round(bytes_ / dev_s / 1e9, 1)
    line["launch_us"] = stats
    if not args.no_extras:
        line["also"] = also
        line["cpu_baseline"] = cpu
    print(json.dumps(line))


if __name__ == "__main__":
    main()
