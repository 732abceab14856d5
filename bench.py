#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

Default workload (BASELINE.json configs[1]): the W4A16 GEMM at the four
Llama-3-8B linear shapes (qkv, o, gate_up, down) with M = 16 fp16 activations,
int4 weights, group size 128.  One *step* = one pass over the four layers.
Weights rotate through enough distinct copies to exceed twice the 256 MB
Infinity Cache, so every step streams its weights from HBM.  Steps are captured
in a HIP graph (launch gaps would otherwise dominate microsecond kernels) and
timed with HIP events on the launch stream.

Prints ONE JSON line: whole-job GB/s of algorithmic bytes, the roofline
fraction of the dominant kernel, and the CPU oracle timed on the host cores.
The same line carries the rest of the metric: the M = 1 .. 2048 sweep over the
four shapes (``sweep``), the W8A8 int8 GEMM of configs[2] with its own roofline
block and CPU baseline (``w8a8_int8``), and the two fused-MoE layers of
configs[3] / configs[4] (``moe_w4a16``, ``moe_fp8_block``), each with the CPU
oracle timed on a stated sample.  ``--quick`` leaves those legs out.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

LLAMA3_8B = [("qkv", 4096, 6144), ("o", 4096, 4096), ("gate_up", 4096, 28672), ("down", 14336, 4096)]
GROUP = 128
HBM_PEAK_GBPS = 8000.0
FP16_PEAK_TFLOPS = 2500.0
INT8_PEAK_TOPS = 5000.0

# HBM bytes per launch of w4a16_stream_kernel in the default workload, mean over
# the four layers, from two `rocprofv3 --pmc` runs of this script (FETCH_SIZE,
# then WRITE_SIZE), each scaled by what the same counter reads for the 256 MiB
# copy of --calibrate-copy (FETCH_SIZE: 2 KiB per unit, WRITE_SIZE: 1 KiB per
# unit).  Keyed by (M, --split-k); other settings were not profiled.
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = {(16, 0): 34022694}
# the build the figure was taken on, and the work split (tiles per workgroup, K splits) it belongs to: the
# line carries `traffic` only while the library still plans the four layers that way (a different split
# moves the traffic: re-measure with the commands in profiles/w4a16_stream_kernel_llama3_8b_m16.txt)
MEASURED_TRAFFIC_COMMIT = "1cb0412"
MEASURED_TRAFFIC_PLAN = {"qkv": (2, 1), "o": (1, 1), "gate_up": (8, 1), "down": (4, 4)}


def stream_plans(M):
    """(tiles per workgroup, K splits) the library takes for the four layers at M rows on this device."""
    import ctypes
    from vllm_gcu_amd import _lib
    lib = _lib.load()
    out = {}
    for name, K, N in LLAMA3_8B:
        nt, sp = ctypes.c_int(0), ctypes.c_int(0)
        _lib.check(lib.mi355q_w4a16_stream_plan(M, K, N, GROUP, ctypes.byref(nt), ctypes.byref(sp)), "stream_plan")
        out[name] = (nt.value, sp.value)
    return out


def w4a16_bytes(M, K, N, g=GROUP):
    """Algorithmic bytes of one W4A16 GEMM: packed weights + fp16 scales +
    packed int4 zeros + fp16 activations in + fp16 out."""
    return K * N // 2 + (K // g) * N * 2 + (K // g) * N // 2 + 2 * M * K + 2 * M * N


def make_layer(K, N, copies, dev, seed):
    import torch
    g = torch.Generator(device="cpu").manual_seed(seed)
    layers = []
    for c in range(copies):
        # random bits are as good as any int4 matrix; they are in slab order already
        qw = torch.randint(-2**31, 2**31 - 1, (K // 8, N), dtype=torch.int32, generator=g).to(dev)
        zp = torch.randint(-2**31, 2**31 - 1, (K // GROUP, N // 8), dtype=torch.int32, generator=g).to(dev)
        sc = (torch.rand(K // GROUP, N, generator=g) * 0.009 + 0.001).to(torch.float16).to(dev)
        layers.append((qw, zp, sc))
    return layers


def time_graph(fn_list, steps, warmup, stream):
    """Time exactly `steps` steps, step i running fn_list[i % len(fn_list)].

    One HIP graph holds len(fn_list) consecutive steps (so the kernels run back
    to back without host launch gaps); it is replayed steps // len times and a
    second graph holds the remainder.  HIP events on `stream` bracket the timed
    region.  Returns seconds for all steps."""
    import torch
    n = len(fn_list)

    def capture(k):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            for i in range(k):
                fn_list[i]()
        return g

    with torch.cuda.stream(stream):
        for fn in fn_list:
            fn()                                    # warm (allocates workspaces on this stream)
        stream.synchronize()
        full = capture(n)
        rem = capture(steps % n) if steps % n else None
        for _ in range(max(1, -(-warmup // n))):
            full.replay()
        stream.synchronize()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(steps // n):
            full.replay()
        if rem is not None:
            rem.replay()
        e1.record(stream)
        e1.synchronize()
        torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e-3


def cpu_baseline_w4a16(M, target_s=12.0):
    """The CPU oracle (dequantize + torch.matmul, fp32) on the same four
    shapes, all host threads: whole passes over the four layers are repeated
    until about target_s seconds of CPU work are done.  Returns GB/s of the
    same algorithmic bytes."""
    import numpy as np
    import torch
    from oracle import w4 as ow4
    torch.set_num_threads(os.cpu_count() or 1)
    rng = np.random.default_rng(0)
    cases = []
    for name, K, N in LLAMA3_8B:
        q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
        z = rng.integers(0, 16, size=(K // GROUP, N), dtype=np.uint8)
        s = rng.uniform(0.001, 0.01, size=(K // GROUP, N)).astype(np.float16)
        x = rng.standard_normal((M, K)).astype(np.float16)
        cases.append((K, N, q, z, s, x))
    tot_b, tot_t, passes = 0, 0.0, 0
    while tot_t < target_s and passes < 200:
        for K, N, q, z, s, x in cases:
            t0 = time.time()
            ow4.w4a16_gemm(x, q, z, s, GROUP)
            tot_t += time.time() - t0
            tot_b += w4a16_bytes(M, K, N)
        passes += 1
    return {"value": round(tot_b / tot_t / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"{passes} passes of oracle.w4.w4a16_gemm (numpy dequantize + torch fp32 matmul) over the "
                      f"four layers at M={M}; {tot_t:.1f} s of CPU work"}


def device_report(dev):
    """Peaks re-derived from what the device reports, beside the published ones the fractions use:
    matrix peak = compute units x core clock x dense MFMA operations per unit and clock (4096 for
    fp16 / bf16, 8192 for fp8 / int8 on CDNA4), HBM peak = 2 x memory clock x bus width."""
    import torch
    p = torch.cuda.get_device_properties(dev)
    cus, ghz = p.multi_processor_count, getattr(p, "clock_rate", 0) / 1e6
    if not ghz:
        # the runtime reports no clock here: take the GPU agent's "Max Clock Freq. (MHz)" of rocminfo
        import re
        import subprocess
        try:
            txt = subprocess.run(["rocminfo"], capture_output=True, text=True, timeout=30).stdout
            for agent in txt.split("*******")[1:]:
                if re.search(r"Device Type:\s+GPU", agent):
                    m = re.search(r"Max Clock Freq\. \(MHz\):\s*(\d+)", agent)
                    if m:
                        ghz = int(m.group(1)) / 1e3
                        break
        except (OSError, subprocess.SubprocessError):
            pass
    rep = {"name": p.name, "arch": getattr(p, "gcnArchName", ""), "compute_units": cus, "core_clock_GHz": round(ghz, 3),
           "hbm_GiB": round(p.total_memory / 2**30, 1),
           "derived_peak_TFLOPs": {"f16_bf16": round(cus * ghz * 4096 / 1e3, 1), "fp8_int8": round(cus * ghz * 8192 / 1e3, 1)}}
    mem_khz, width = getattr(p, "memory_clock_rate", 0), getattr(p, "memory_bus_width", 0)
    if mem_khz and width:
        rep["derived_peak_hbm_GBps"] = round(2 * mem_khz * 1e3 * width / 8 / 1e9, 1)
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    rep["host_cpu"] = {"model": model, "os_cpu_count": os.cpu_count(), "torch_threads": torch.get_num_threads()}
    return rep


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--m", type=int, default=16, help="activation rows of the default workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--sweep", action="store_true", help="(default now) time every (shape, M) of the config")
    ap.add_argument("--quick", action="store_true",
                    help="headline, per-layer detail and CPU baseline only: no sweep, no W8A8, no MoE legs")
    ap.add_argument("--extras", action="store_true",
                    help="also the decode-sized MoE layer, the w4a8 experts, norm + quant and the fp8 dense linear")
    ap.add_argument("--split-k", type=int, default=0)
    ap.add_argument("--family", type=int, default=0,
                    help="W4A16 kernel of the headline leg: 0 the library's choice, 1 streaming, 2 MFMA tiles of 64 rows, "
                         "3 the 128-row ring kernel")
    ap.add_argument("--no-w8a8", action="store_true", help="skip the W8A8 int8 GEMM leg")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run a 256 MiB device copy at the end (reference reading for rocprofv3 --pmc)")
    ap.add_argument("--moe", action="store_true", help="(default now) time the two fused-MoE layers of the config")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no sharding, no collectives); "
              "use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from vllm_gcu_amd.kernels import _custom_ops as ops
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.Stream(device=dev)
    M = args.m

    set_bytes = sum(K * N // 2 for _, K, N in LLAMA3_8B)
    copies = max(2, -(-2 * 256 * 2**20 // set_bytes) + 1)
    layers = {name: make_layer(K, N, copies, dev, seed=i) for i, (name, K, N) in enumerate(LLAMA3_8B)}
    xs = {K: torch.randn(M, K, dtype=torch.float16, device=dev) for K in {k for _, k, _ in LLAMA3_8B}}

    def layer_call(name, K, c):
        qw, zp, sc = layers[name][c]
        return ops.w4a16_gemm(xs[K], qw, sc, zp, None, GROUP, split_k=args.split_k, family=args.family)

    def make_step(c):
        def step():
            for name, K, N in LLAMA3_8B:
                layer_call(name, K, c)
        return step

    step_fns = [make_step(c) for c in range(copies)]
    step_bytes = sum(w4a16_bytes(M, K, N) for _, K, N in LLAMA3_8B)

    # per-layer detail (each layer timed alone, its weights rotating the same way)
    per_layer = {}
    for name, K, N in LLAMA3_8B:
        fns = [(lambda name=name, K=K, c=c: layer_call(name, K, c)) for c in range(copies)]
        n = max(args.steps, 100)
        t = time_graph(fns, n, args.warmup, stream) / n
        b = w4a16_bytes(M, K, N)
        per_layer[name] = {"K": K, "N": N, "us": round(t * 1e6, 3), "GBps": round(b / t / 1e9, 1),
                           "frac_hbm": round(b / t / 1e9 / HBM_PEAK_GBPS, 4)}
    # floor: a plain streaming read (no arithmetic, 16-byte loads, nothing stored) of each layer's
    # packed weights, timed the same way; the best of several grid sizes is quoted
    import ctypes
    from vllm_gcu_amd.kernels import _runtime as rt
    probe = ctypes.CDLL(os.path.join(ROOT, "vllm-gcu_amd", "libmi355q_bench.so"))
    probe.mi355q_bench_stream_read.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p,
                                               ctypes.c_void_p]
    sink = torch.zeros(16, dtype=torch.uint8, device=dev)
    floor_us = 0.0
    for name, K, N in LLAMA3_8B:
        nbytes = K * N // 2
        best = None
        for wgs in (256, 512, 1024, 2048):
            def read(c, name=name, nbytes=nbytes, wgs=wgs):
                rc = probe.mi355q_bench_stream_read(layers[name][c][0].data_ptr(), nbytes, wgs, sink.data_ptr(),
                                                    rt.stream_ptr())
                assert rc == 0
            fns = [(lambda c=c, read=read: read(c)) for c in range(copies)]
            n = max(args.steps, 100)
            t = time_graph(fns, n, args.warmup, stream) / n
            if best is None or t < best[0]:
                best = (t, wgs)
        t = best[0]
        per_layer[name]["read_floor_us"] = round(t * 1e6, 3)
        per_layer[name]["read_floor_workgroups"] = best[1]
        per_layer[name]["time_over_read_floor"] = round(per_layer[name]["us"] / (t * 1e6), 3)
        floor_us += t * 1e6
    # The headline: --warmup untimed steps, then exactly --steps timed ones.  It comes after the per-layer and
    # read-floor legs above so that it meets the card in the state a serving loop keeps it in (the first
    # GPU work after start-up runs about 3 % slower than the same steps a few hundred milliseconds later).
    secs = time_graph(step_fns, args.steps, args.warmup, stream)
    ms_per_step = secs / args.steps * 1e3
    value = step_bytes * args.steps / secs / 1e9
    # the same step timed over at least 200 steps after at least 20 warm-up steps, whatever --steps says
    # (a short --steps run is one or two graph replays: consistent, but noisier)
    n_long = max(args.steps, 200)
    secs_long = time_graph(step_fns, n_long, max(args.warmup, 20), stream)
    for name in per_layer:
        per_layer[name]["time_over_read_floor"] = round(per_layer[name]["us"] / per_layer[name]["read_floor_us"], 3)

    # Every launch of a step is the same kernel (w4a16_stream_kernel), so the
    # dominant kernel's average launch is a quarter of a step: algorithmic bytes
    # per launch / average launch duration over the timed region.
    launches = len(LLAMA3_8B)
    launch_us = ms_per_step * 1e3 / launches
    achieved = step_bytes / launches / (launch_us * 1e-6) / 1e9
    traffic = MEASURED_TRAFFIC_BYTES_PER_LAUNCH.get((M, args.split_k))
    plans = stream_plans(M) if M <= 64 else {}
    provenance = None
    if traffic is not None:
        if plans == MEASURED_TRAFFIC_PLAN:
            provenance = {"measured_on_commit": MEASURED_TRAFFIC_COMMIT, "work_split": {k: list(v) for k, v in plans.items()},
                          "how": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, commands and per-layer figures in "
                                 "profiles/w4a16_stream_kernel_llama3_8b_m16.txt; the streaming kernel's loads and "
                                 "work split are unchanged since that commit"}
        else:
            print(f"bench.py: the library plans {plans}, the traffic figure was measured on {MEASURED_TRAFFIC_PLAN}: "
                  "traffic left out, re-measure it", file=sys.stderr)
            traffic = None
    roofline = {"bound": "hbm", "kernel": "w4a16_stream_kernel", "launches_per_step": launches,
                "avg_launch_us": round(launch_us, 3), "algorithmic_bytes_per_launch": step_bytes // launches,
                "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic,
                "traffic_provenance": provenance}
    if M > 64:
        # --m above the decode range: the launches are the MFMA kernels (64-row tiles or the 128-row ring kernel,
        # chosen per layer) and the bound is the fp16 matrix peak
        step_flops = sum(2.0 * M * K * N for _, K, N in LLAMA3_8B)
        tf = step_flops / launches / (launch_us * 1e-6) / 1e12
        roofline = {"bound": "mfma", "kernel": "w4a16_mid_kernel / w4a16_tile_kernel", "launches_per_step": launches,
                    "avg_launch_us": round(launch_us, 3), "algorithmic_flops_per_launch": step_flops / launches,
                    "achieved": round(tf, 1), "peak": 2500.0, "unit": "TFLOP/s", "frac": round(tf / 2500.0, 4),
                    "traffic": None}

    out = {
        "metric": "W4A16 GEMM HBM GB/s (algorithmic bytes / time), Llama-3-8B linear shapes",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"W4A16 GEMM, Llama-3-8B shapes qkv/o/gate_up/down, M={M}, int4 g=128, "
                               f"fp16 act, fp32 accumulate; one step = the 4 layers once",
                   "weight_copies_rotated": copies, "bytes_per_step": step_bytes},
        "frac_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
        "per_layer": per_layer,
        "stable": {"steps": n_long, "ms_per_step": round(secs_long / n_long * 1e3, 5),
                   "value": round(step_bytes * n_long / secs_long / 1e9, 2),
                   "frac_hbm_peak": round(step_bytes * n_long / secs_long / 1e9 / HBM_PEAK_GBPS, 4)},
        "read_floor": {"what": "plain streaming read of the packed weights only (best of 256..2048 workgroups), one launch "
                               "per layer, same graph timing",
                       "us_per_step": round(floor_us, 3),
                       "step_time_over_floor": round(ms_per_step * 1e3 / floor_us, 3)},
        "roofline": roofline,
    }
    out["device"] = device_report(dev)
    if not args.no_w8a8 and not args.quick:
        out["w8a8_int8"] = w8a8_gemm_bench(ops, dev, stream, cpu=not args.no_cpu)
        torch.cuda.empty_cache()
    if not args.quick:
        out["yardsticks"] = yardsticks(dev, stream)
        torch.cuda.empty_cache()
        out["sweep"] = sweep(ops, dev, stream, args)
        out["moe_w4a16"] = moe_bench(ops, dev, stream, "w4a16", cpu=not args.no_cpu)
        torch.cuda.empty_cache()
        out["moe_fp8_block"] = moe_bench(ops, dev, stream, "fp8", cpu=not args.no_cpu)
        torch.cuda.empty_cache()
    if args.extras:
        out["moe_w4a16_decode"] = moe_bench(ops, dev, stream, "w4a16", tokens=16)
        import torch as _torch
        out["moe_w4a16_bf16"] = moe_bench(ops, dev, stream, "w4a16", tokens=512, act_dtype=_torch.bfloat16)
        torch.cuda.empty_cache()
        # the DeepSeek-V3-style layer at a prefill token count (128 rows per expert: blocks of 256 slots on the
        # MFMA tile kernel with gathered rows)
        out["moe_fp8_block_prefill"] = moe_bench(ops, dev, stream, "fp8", iters=6, tokens=4096)
        torch.cuda.empty_cache()
        out["moe_w4a8"] = moe_bench(ops, dev, stream, "w4a8")
        torch.cuda.empty_cache()
        # unquantised experts at prefill token counts (blocks of 256 slots on the MFMA tile kernel, 16-bit operands)
        out["moe_f16_prefill"] = {str(t): moe_bench(ops, dev, stream, "f16", iters=8, tokens=t) for t in (512, 2048)}
        torch.cuda.empty_cache()
        out["norm_quant"] = glue_bench(ops, dev, stream)
        torch.cuda.empty_cache()
        out["fp8_dense"] = fp8_dense_bench(ops, dev, stream)
        torch.cuda.empty_cache()
        out["w4a16_variants"] = variants_bench(ops, dev, stream)
    if args.calibrate_copy:
        # a plain copy of known size: its FETCH_SIZE / WRITE_SIZE readings scale
        # the counters of the profiled kernels to bytes
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        out["calibration_copy_bytes"] = int(src.numel())
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_w4a16(M)
    print(json.dumps(out))


def cpu_baseline_w8a8(x16, w_nk, ws, rows=2048):
    """The CPU oracle of configs[2] on the first `rows` token rows against the whole weight: dynamic
    per-token quantisation, exact int32 GEMM (fp32 matmul over K chunks of 1024), scale epilogue."""
    import numpy as np
    import torch
    from oracle import w8a8 as o8
    torch.set_num_threads(os.cpu_count() or 1)
    x = x16[:rows].cpu().numpy()
    w_kn = np.ascontiguousarray(w_nk.cpu().numpy().T)
    wsn = ws.cpu().numpy()
    t0 = time.time()
    xq, xs = o8.dynamic_scaled_int8_quant(x)
    acc = o8.int8_gemm_i32(xq, w_kn)
    o8.scaled_mm_epilogue(acc, xs, wsn).astype(np.float16)
    dt = time.time() - t0
    K, N = w_kn.shape
    return {"value": round(2.0 * rows * K * N / dt / 1e12, 4), "unit": "TOP/s", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"oracle.w8a8 (per-token quant + exact int32 GEMM + epilogue) on {rows} of the 2048 token rows "
                      f"against the whole [8192, 28672] weight, 1 repetition, {dt:.2f} s of CPU work"}


def w8a8_gemm_bench(ops, dev, stream, iters=30, warmup=40, cpu=False):
    """BASELINE configs[2]: W8A8 int8 GEMM, M=2048, K=8192, N=28672 (one
    Llama-3-70B MLP layer), per-token x per-channel scales fused, fp16 out."""
    import torch
    M, K, N = 2048, 8192, 28672
    g = torch.Generator(device="cpu").manual_seed(0)
    x = torch.randn(M, K, generator=g).to(torch.float16).to(dev)
    xq, xs, _ = ops.scaled_int8_quant(x)
    w_nk = torch.randint(-127, 128, (N, K), dtype=torch.int8, generator=g).to(dev)
    ws = (torch.rand(N, generator=g) * 0.019 + 0.001).float().to(dev)
    out = torch.empty(M, N, dtype=torch.float16, device=dev)
    # three weight copies in turn (3 x 235 MB against a 256 MB last-level cache), as the decode legs do
    wts = [w_nk.t(), w_nk.roll(1, 0).t(), w_nk.roll(2, 0).t()]
    # long warm-up: the core clock settles (it drops under sustained MFMA load and
    # recovers part of the way) only after some tens of launches
    # (several launches per graph: a graph of one short kernel would time the replay gap with it)
    t = time_graph([(lambda wt=wt: torch.ops._C.cutlass_scaled_mm(out, xq, wt, xs, ws, None)) for wt in wts] * 2,
                   iters, warmup, stream) / iters
    tq = time_graph([lambda: ops.scaled_int8_quant(x)] * 10, iters, 10, stream) / iters
    ops_ = 2.0 * M * K * N
    # decode: 16 tokens against the same layer, weights as the linear method keeps them after
    # loading (kslab order); three weight copies in turn so that none is served from a cache
    from vllm_gcu_amd.kernels.quantization import rearrange
    Md = 16
    ksl = [rearrange.to_kslab(w_nk if i == 0 else w_nk.roll(i, 0)) for i in range(3)]
    outd = torch.empty(Md, N, dtype=torch.float16, device=dev)
    fns = [(lambda w=w: torch.ops._C.cutlass_scaled_mm(outd, xq[:Md], w.t(), xs[:Md], ws, None)) for w in ksl]
    td = time_graph(fns * 2, iters, 6, stream) / iters
    res_cpu = cpu_baseline_w8a8(x, w_nk, ws) if cpu else None
    return {"workload": "W8A8 int8 GEMM M=2048 K=8192 N=28672, fused per-token x per-channel scales, fp16 out, "
                        "three weight copies in turn",
            "gemm_us": round(t * 1e6, 1), "TOPs": round(ops_ / t / 1e12, 1),
            "frac_int8_mfma_peak": round(ops_ / t / 1e12 / INT8_PEAK_TOPS, 4),
            "roofline": {"bound": "mfma", "kernel": "w8a8_int8_gemm_kernel", "avg_launch_us": round(t * 1e6, 1),
                         "algorithmic_ops_per_launch": ops_, "achieved": round(ops_ / t / 1e12, 1),
                         "peak": INT8_PEAK_TOPS, "unit": "TOP/s", "frac": round(ops_ / t / 1e12 / INT8_PEAK_TOPS, 4),
                         "timed_launches": iters, "warmup_launches": warmup,
                         "note": "one GEMM = two launches of the kernel at this shape (three full rounds of 256 x 256 "
                                 "tiles, then the remaining columns as one round of 256 x 128 tiles); avg_launch_us is "
                                 "the pair"},
            "cpu_baseline": res_cpu,
            "dynamic_quant_us": round(tq * 1e6, 1),
            "dynamic_quant_GBps": round((2 * M * K + M * K + 4 * M) / tq / 1e9, 1),
            "decode_m16_us": round(td * 1e6, 1),
            "decode_m16_GBps": round((N * K + Md * K + 2 * Md * N) / td / 1e9, 1)}


def cpu_baseline_moe_w4a16(x, logits, w13, z13, s13, w2, z2, s2, T):
    """The CPU oracle of configs[3]: routing + the naive per-expert loop over dequantised experts, all 512
    tokens, 1 repetition (the experts are dequantised inside the timed region, as the oracle does)."""
    import numpy as np
    import torch
    from oracle import moe as om
    from oracle import w4 as ow4
    torch.set_num_threads(os.cpu_count() or 1)
    xh = x.cpu().numpy()
    lg = logits.cpu().numpy()
    W13, Z13, S13 = w13.cpu().numpy(), z13.cpu().numpy(), s13.cpu().numpy()
    W2, Z2, S2 = w2.cpu().numpy(), z2.cpu().numpy(), s2.cpu().numpy()

    def expert(wq, zq, sc, e):
        # the bench's random words are slab-order words; as a timing of unpack + dequantise they stand
        # for any int4 matrix (values are not compared here)
        return ow4.dequantize(ow4.gptq_unpack_weight(wq[e]), ow4.gptq_unpack_zeros(zq[e]), sc[e], GROUP)

    def f16(a):
        return a.astype(np.float16).astype(np.float32)
    t0 = time.time()
    tw, ids, _ = om.topk_softmax(lg, T, True)
    om.fused_experts(xh.astype(np.float32), lambda e: expert(W13, Z13, S13, e), lambda e: expert(W2, Z2, S2, e),
                     tw, ids, f16)
    dt = time.time() - t0
    M, H = xh.shape
    I = W2.shape[1] * 8
    flops = 2.0 * M * T * (H * 2 * I + I * H)
    return {"value": round(flops / dt / 1e12, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle.moe.fused_experts on all {M} tokens (routing, unpack + dequantise of the 8 experts, fp32 "
                      f"matmuls, SiLU gate, weighted sum), 1 repetition, {dt:.1f} s of CPU work"}


def cpu_baseline_moe_fp8(x, tw, ids, w13, s13, w2, s2, tokens=2):
    """The CPU oracle of configs[4] on the first `tokens` tokens (their 8 experts each are dequantised)."""
    import numpy as np
    import torch
    from oracle import fp8 as of8
    from oracle import moe as om
    torch.set_num_threads(os.cpu_count() or 1)
    xf = x[:tokens].float().cpu().numpy()
    twn, idn = tw[:tokens].cpu().numpy(), ids[:tokens].cpu().numpy()
    need = sorted(set(idn.reshape(-1).tolist()))
    c13 = {e: w13[e].view(torch.uint8).cpu().numpy() for e in need}
    c2 = {e: w2[e].view(torch.uint8).cpu().numpy() for e in need}
    b13 = {e: s13[e].cpu().numpy() for e in need}
    b2 = {e: s2[e].cpu().numpy() for e in need}

    def deq(codes, sc):
        return (of8.from_e4m3fn(codes) * np.repeat(np.repeat(sc, 128, 0), 128, 1)).T

    def qdq(a):
        qa, sa = of8.per_token_group_quant_fp8(a, 128)
        return of8.from_e4m3fn(qa) * np.repeat(sa, 128, -1)

    def bf16(a):
        return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).float().numpy()
    t0 = time.time()
    om.fused_experts(qdq(xf), lambda e: deq(c13[e], b13[e]), lambda e: deq(c2[e], b2[e]), twn, idn, bf16, quant_a2=qdq)
    dt = time.time() - t0
    H, I = xf.shape[1], w2.shape[2]
    nbytes = len(need) * (3 * H * I)
    return {"value": round(nbytes / dt / 1e9, 4), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle.moe.fused_experts on the first {tokens} of 256 tokens ({len(need)} experts dequantised from "
                      f"fp8 codes and block scales, fp32 matmuls), 1 repetition, {dt:.1f} s of CPU work; bytes = those "
                      f"experts' weights"}


def moe_bench(ops, dev, stream, which, iters=20, tokens=None, cpu=False, act_dtype=None):
    """BASELINE configs[3] (Mixtral-8x7B layer, W4A16) and configs[4]
    (DeepSeek-V3-style layer, fp8 block-scaled): routing + the whole
    fused-experts sequence, one layer."""
    import torch
    from vllm_gcu_amd.kernels import fused_moe
    from vllm_gcu_amd.kernels.modular_experts import TritonExpertsPad
    from vllm_gcu_amd.kernels.modular_kernel import FusedMoEModularKernel
    from vllm_gcu_amd.kernels.prepare_finalize import MoEPrepareAndFinalizeNoEP
    g = torch.Generator(device="cpu").manual_seed(0)

    def rnd_i32(*shape):
        # random words filled on the device (the tensors are hundreds of MB)
        return torch.randint(-2**31, 2**31 - 1, shape, dtype=torch.int32, device=dev)

    if which == "w4a16":
        M, H, E, I, T = tokens or 512, 4096, 8, 14336, 2
        w13, w2 = rnd_i32(E, H // 8, 2 * I), rnd_i32(E, I // 8, H)
        z13, z2 = rnd_i32(E, H // 128, 2 * I // 8), rnd_i32(E, I // 128, H // 8)
        adt = act_dtype or torch.float16             # (configs[3] states fp16; bf16 is the type Mixtral ships in)
        s13 = (torch.rand(E, H // 128, 2 * I, device=dev) * 0.009 + 0.001).to(adt)
        s2 = (torch.rand(E, I // 128, H, device=dev) * 0.009 + 0.001).to(adt)
        x = torch.randn(M, H, generator=g).to(adt).to(dev)
        logits = torch.randn(M, E, generator=g).to(dev)
        moe = FusedMoEModularKernel(MoEPrepareAndFinalizeNoEP(), TritonExpertsPad(use_int4_w4a16=True, block_shape=[0, 128]))
        kw = dict(w1_scale=s13, w2_scale=s2, w1_zp=z13, w2_zp=z2)

        def step():
            tw, ids = ops.fused_topk(x, logits, T, True)
            return moe(x, w13, w2, tw, ids, **kw)
        flops = 2.0 * M * T * (H * 2 * I + I * H)
        bytes_ = E * (H * 2 * I + I * H) // 2 + E * (H // 128 * 2 * I + I // 128 * H) * 2 \
            + E * (H // 128 * 2 * I + I // 128 * H) // 2 + 2 * M * H * 2
        name = f"fused MoE W4A16, Mixtral-8x7B layer: {M} tok, hidden 4096, 8 experts, inter 14336, top-2" + \
            (", bf16 activations" if adt == torch.bfloat16 else "")
    elif which == "f16":
        # the Mixtral-8x7B layer of configs[3] with unquantised fp16 experts (fused_moe_kernel)
        M, H, E, I, T = tokens or 512, 4096, 8, 14336, 2
        w13 = torch.empty(E, 2 * I, H, device=dev, dtype=torch.float16).normal_(0, 0.02)
        w2 = torch.empty(E, H, I, device=dev, dtype=torch.float16).normal_(0, 0.02)
        x = torch.randn(M, H, generator=g).half().to(dev)
        logits = torch.randn(M, E, generator=g).to(dev)
        moe = FusedMoEModularKernel(MoEPrepareAndFinalizeNoEP(), TritonExpertsPad())
        kw = {}

        def step():
            tw, ids = ops.fused_topk(x, logits, T, True)
            return moe(x, w13, w2, tw, ids, **kw)
        flops = 2.0 * M * T * (H * 2 * I + I * H)
        bytes_ = E * (H * 2 * I + I * H) * 2 + 2 * M * H * 2
        name = f"fused MoE, unquantised fp16 experts, Mixtral-8x7B layer shape: {M} tok, hidden 4096, 8 experts, inter 14336, top-2"
    elif which == "w4a8":
        # the Mixtral-8x7B layer of configs[3] with w4a8-fp8 experts: fp8 activations with one
        # static scale per GEMM, symmetric int4 weights, fp32 group scales
        M, H, E, I, T = 512, 4096, 8, 14336, 2
        w13, w2 = rnd_i32(E, H // 8, 2 * I), rnd_i32(E, I // 8, H)
        s13 = torch.rand(E, H // 128, 2 * I, device=dev) * 0.009 + 0.001
        s2 = torch.rand(E, I // 128, H, device=dev) * 0.009 + 0.001
        a1, a2 = torch.tensor([0.02], device=dev), torch.tensor([0.5], device=dev)
        x = torch.randn(M, H, generator=g).half().to(dev)
        logits = torch.randn(M, E, generator=g).to(dev)
        moe = FusedMoEModularKernel(MoEPrepareAndFinalizeNoEP(), TritonExpertsPad(use_fp8_w8a8=True, block_shape=None))
        kw = dict(w1_scale=s13, w2_scale=s2, a1_scale=a1, a2_scale=a2, a1_scale_rec=1.0 / a1, a2_scale_rec=1.0 / a2)

        def step():
            tw, ids = ops.fused_topk(x, logits, T, True)
            return moe(x, w13, w2, tw, ids, **kw)
        flops = 2.0 * M * T * (H * 2 * I + I * H)
        bytes_ = E * (H * 2 * I + I * H) // 2 + E * (H // 128 * 2 * I + I // 128 * H) * 4 + 2 * M * H * 2
        name = "fused MoE w4a8-fp8, Mixtral-8x7B layer shape: 512 tok, hidden 4096, 8 experts, inter 14336, top-2"
    else:
        M, H, E, I, T = tokens or 256, 7168, 256, 2048, 8

        def block_fp8(n, k):
            """[E, n, k] weights ~ N(0, 0.02) quantised to fp8-e4m3 with one fp32 scale per 128 x 128 block
            (scale = block absmax / 448), as BASELINE configs[4] states; one expert at a time on the device."""
            codes = torch.empty((E, n, k), dtype=torch.float8_e4m3fn, device=dev)
            scales = torch.empty((E, n // 128, k // 128), dtype=torch.float32, device=dev)
            gg = torch.Generator(device=dev).manual_seed(n + k)
            for e in range(E):
                w = torch.randn(n, k, device=dev, generator=gg) * 0.02
                blk = w.view(n // 128, 128, k // 128, 128)
                sc = blk.abs().amax(dim=(1, 3)).clamp_min(1e-12) / 448.0
                codes[e] = (blk / sc[:, None, :, None]).view(n, k).to(torch.float8_e4m3fn)
                scales[e] = sc
            return codes, scales
        w13, s13 = block_fp8(2 * I, H)
        w2, s2 = block_fp8(H, I)
        x = torch.randn(M, H, generator=g).to(torch.bfloat16).to(dev)
        logits = torch.randn(M, E, generator=g).to(dev)
        moe = FusedMoEModularKernel(MoEPrepareAndFinalizeNoEP(), TritonExpertsPad(use_fp8_w8a8=True, block_shape=[128, 128]))
        kw = dict(w1_scale=s13, w2_scale=s2)

        def step():
            tw, ids = fused_moe.grouped_topk(x, logits, T, True, 8, 4, "softmax", None)
            return moe(x, w13, w2, tw, ids, **kw)
        tw, ids = fused_moe.grouped_topk(x, logits, T, True, 8, 4, "softmax", None)
        hit = int(torch.unique(ids).numel())
        flops = 2.0 * M * T * (H * 2 * I + I * H)
        bytes_ = hit * (2 * I * H + H * I + 4 * (2 * I // 128 * H // 128 + H // 128 * I // 128)) \
            + M * H + M * H // 128 * 4 + M * H * 2
        name = (f"fused MoE fp8 block-scaled, DeepSeek-V3-style layer: {M} tok, hidden 7168, 256 experts ({hit} hit), inter 2048, "
                "top-8; weights ~ N(0, 0.02) quantised per 128 x 128 block")
    time_graph([step], 5, 3, stream)
    t = time_graph([step], iters, 0, stream) / iters
    res = {"workload": name, "us": round(t * 1e6, 1), "compulsory_bytes": int(bytes_),
           "GBps": round(bytes_ / t / 1e9, 1), "frac_hbm": round(bytes_ / t / 1e9 / HBM_PEAK_GBPS, 4),
           "TFLOPs": round(flops / t / 1e12, 1),
           "frac_mfma_peak": round(flops / t / 1e12 / (5000.0 if which == "fp8" else FP16_PEAK_TFLOPS), 4)}
    if cpu and which == "w4a16" and tokens is None:
        res["cpu_baseline"] = cpu_baseline_moe_w4a16(x, logits, w13, z13, s13, w2, z2, s2, T)
    if cpu and which == "fp8":
        res["cpu_baseline"] = cpu_baseline_moe_fp8(x, tw, ids, w13, s13, w2, s2)
    return res


def glue_bench(ops, dev, stream, iters=50):
    """The norm + quantise prologue of a block-fp8 layer: 2048 tokens of hidden 7168, bf16 ->
    fp8 with one scale per 128 values, with and without the residual add.  HBM-bound."""
    import torch
    rows, K = 2048, 7168
    x = torch.randn(rows, K, device=dev).to(torch.bfloat16)
    r = torch.randn(rows, K, device=dev).to(torch.bfloat16)
    w = torch.ones(K, device=dev, dtype=torch.bfloat16)
    q = torch.empty((rows, K), dtype=torch.float8_e4m3fn, device=dev)
    s = torch.empty((rows, K // 128), dtype=torch.float32, device=dev)
    out = {}
    for name, fn, nbytes in (
            ("rms_norm_per_token_group_quant_fp8",
             lambda: torch.ops._C.rms_norm_per_token_group_quant_fp8(q, s, x, w, 1e-6, 128),
             rows * K * 3 + rows * K // 128 * 4),
            ("fused_add_rms_norm_per_token_group_quant_fp8",
             lambda: torch.ops._C.fused_add_rms_norm_per_token_group_quant_fp8(q, r, s, x, w, 1e-6, 128),
             rows * K * 7 + rows * K // 128 * 4)):
        t = time_graph([fn], iters, 5, stream) / iters
        out[name] = {"shape": [rows, K], "us": round(t * 1e6, 2), "GBps": round(nbytes / t / 1e9, 1),
                     "frac_hbm": round(nbytes / t / 1e9 / HBM_PEAK_GBPS, 4)}
    return out


def fp8_dense_bench(ops, dev, stream, iters=12):
    """fp8 block-scaled dense linear (linear_quant), K=8192 N=28672, weights in the kslab order,
    three copies in turn: decode (M=16, weight-streaming kernel, HBM-bound) and prefill
    (M=2048, MFMA tile kernel)."""
    import torch
    from vllm_gcu_amd.kernels.quantization import rearrange
    K, N = 8192, 28672
    ws_ = [rearrange.to_kslab((torch.randn(N, K, device=dev) * 0.5).to(torch.float8_e4m3fn)) for _ in range(3)]
    wsc = torch.rand(N // 128, K // 128, device=dev) * 0.05 + 0.02
    out = {}
    for M in (16, 2048):
        x = torch.randn(M, K, device=dev, dtype=torch.bfloat16)
        xq, xs = ops.per_token_group_quant_fp8(x, 128)
        o = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
        fns = [(lambda w=w: torch.ops._C.linear_quant(o, xq, w, None, xs, wsc)) for w in ws_]
        time_graph(fns, iters, 3, stream)
        t = time_graph(fns, iters, 0, stream) / iters
        nbytes = N * K + M * K + 4 * M * (K // 128) + 4 * (N // 128) * (K // 128) + 2 * M * N
        out[f"M{M}"] = {"us": round(t * 1e6, 1), "GBps": round(nbytes / t / 1e9, 1),
                        "frac_hbm": round(nbytes / t / 1e9 / HBM_PEAK_GBPS, 4),
                        "TFLOPs": round(2.0 * M * N * K / t / 1e12, 1),
                        "frac_fp8_mfma_peak": round(2.0 * M * N * K / t / 1e12 / 5000.0, 4)}
    # the same layer with per-token x per-channel scales (cutlass_scaled_mm on fp8 operands)
    wch = torch.rand(N, 1, device=dev) * 0.019 + 0.001
    pc = {}
    for M in (16, 128, 2048):
        x = torch.randn(M, K, device=dev, dtype=torch.bfloat16)
        xq, xs = ops.scaled_fp8_quant(x, None, use_per_token_if_dynamic=True)
        o = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
        fns = [(lambda w=w: torch.ops._C.cutlass_scaled_mm(o, xq, w.t(), xs, wch, None)) for w in ws_]
        time_graph(fns, iters, 3, stream)
        t = time_graph(fns, iters, 0, stream) / iters
        nbytes = N * K + M * K + 4 * M + 4 * N + 2 * M * N
        pc[f"M{M}"] = {"us": round(t * 1e6, 1), "GBps": round(nbytes / t / 1e9, 1),
                       "frac_hbm": round(nbytes / t / 1e9 / HBM_PEAK_GBPS, 4),
                       "TFLOPs": round(2.0 * M * N * K / t / 1e12, 1),
                       "frac_fp8_mfma_peak": round(2.0 * M * N * K / t / 1e12 / 5000.0, 4)}
    return {"workload": "fp8 block-scaled dense linear K=8192 N=28672, bf16 out", **out,
            "per_token_per_channel": {"workload": "fp8 per-token x per-channel scaled GEMM (cutlass_scaled_mm), same layer",
                                      **pc}}


def yardsticks(dev, stream, iters=30):
    """What the chip and the vendor's own library reach on the same shapes and the same kind of data,
    beside the published peaks: (a) a loop of matrix instructions on register-resident operands
    (nothing loaded or stored in the loop; fp16: A ~ N(0,1), B ~ N(0, 0.02); int8: uniform), two
    wavefronts per SIMD; (b) torch.matmul (fp16, dense weights, no dequantisation) at the Llama-3-8B shapes for
    M = 128 and 2048 and torch._int_mm (int8 -> int32, no scales) at the W8A8 shape."""
    import ctypes
    import torch
    from vllm_gcu_amd.kernels import _runtime as rt
    probe = ctypes.CDLL(os.path.join(ROOT, "vllm-gcu_amd", "libmi355q_bench.so"))
    probe.mi355q_bench_mfma_rate.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                             ctypes.c_void_p, ctypes.c_void_p]
    clk = torch.zeros(2, dtype=torch.int64, device=dev)
    sink = torch.zeros(16, dtype=torch.uint8, device=dev)
    # launches of about half a millisecond, timed like the GEMMs (the sustained rate over tens of
    # milliseconds is lower still: the clock keeps dropping under matrix load)
    wgs, loops = 2 * 256, 800
    res = {"what": yardsticks.__doc__.split("\n\n")[0].replace("\n    ", " ")}
    # operands as the GEMMs see them: activations N(0,1), weights N(0, 0.02) (fp16); uniform int8 on both sides
    f16_src = torch.cat([torch.randn(1 << 20, device=dev), torch.randn(1 << 20, device=dev) * 0.02]).half()
    for kind, name, src, per in ((0, "mfma_f32_16x16x32_f16", f16_src, 2 * 16 * 16 * 32),
                                 (1, "mfma_i32_16x16x64_i8",
                                  torch.randint(-127, 128, (4 << 20,), dtype=torch.int8, device=dev), 2 * 16 * 16 * 64)):
        def run(kind=kind, src=src):
            assert probe.mi355q_bench_mfma_rate(src.data_ptr(), kind, wgs, loops, sink.data_ptr(), clk.data_ptr(),
                                                rt.stream_ptr()) == 0
        t = time_graph([run], iters, 10, stream) / iters
        rate = wgs * 4 * loops * 32 * per / t / 1e12
        peak = FP16_PEAK_TFLOPS if kind == 0 else INT8_PEAK_TOPS
        ticks = clk.cpu().tolist()
        # core clock inside the loop: shader-clock ticks per tick of the 100 MHz reference counter
        ghz = ticks[0] / max(1, ticks[1]) * 0.1
        res[name] = {"T_per_s": round(rate, 1), "frac_of_published_peak": round(rate / peak, 4),
                     "core_clock_GHz_in_loop": round(ghz, 3),
                     "cycles_per_instruction_per_SIMD": round(ticks[0] / (2.0 * loops * 32), 2)}
    vend = []
    for name, K, N in LLAMA3_8B:
        w = [(torch.randn(K, N, device=dev) * 0.02).half() for _ in range(2)]
        for M in (128, 2048):
            x = torch.randn(M, K, device=dev).half()
            outs = [torch.empty(M, N, dtype=torch.float16, device=dev) for _ in range(2)]
            fns = [(lambda c=c: torch.matmul(x, w[c], out=outs[c])) for c in range(2)]
            n = 100 if M <= 128 else iters
            t = time_graph(fns, n, 10, stream) / n
            vend.append({"layer": name, "K": K, "N": N, "M": M, "us": round(t * 1e6, 2),
                         "TFLOPs": round(2.0 * M * K * N / t / 1e12, 1)})
        del w
        torch.cuda.empty_cache()
    res["vendor_fp16_gemm"] = vend
    M, K, N = 2048, 8192, 28672
    a = torch.randint(-127, 128, (M, K), dtype=torch.int8, device=dev)
    b = torch.randint(-127, 128, (N, K), dtype=torch.int8, device=dev).t()
    try:
        t = time_graph([lambda: torch._int_mm(a, b)], iters, 40, stream) / iters
        res["vendor_int8_mm"] = {"M": M, "K": K, "N": N, "us": round(t * 1e6, 1), "TOPs": round(2.0 * M * K * N / t / 1e12, 1)}
    except RuntimeError as e:
        res["vendor_int8_mm"] = {"error": str(e)[:120]}
    return res


def variants_bench(ops, dev, stream):
    """W4A16 away from the headline's type and group size: bf16 activations, and quantisation groups of 64
    and 32, on two Llama-3-8B layers at prefill heights (weights rotated past the last-level cache)."""
    import torch
    res = []
    for name, K, N in (("gate_up", 4096, 28672), ("down", 14336, 4096)):
        copies = max(2, -(-2 * 256 * 2**20 // (K * N // 2)) + 1)
        gen = torch.Generator(device="cpu").manual_seed(11)
        qws = [torch.randint(-2**31, 2**31 - 1, (K // 8, N), dtype=torch.int32, generator=gen).to(dev) for _ in range(copies)]
        for dt, g in ((torch.float16, 128), (torch.bfloat16, 128), (torch.float16, 64), (torch.float16, 32)):
            zp = torch.randint(-2**31, 2**31 - 1, (K // g, N // 8), dtype=torch.int32, generator=gen).to(dev)
            sc = (torch.rand(K // g, N, generator=gen) * 0.009 + 0.001).to(dt).to(dev)
            for M in ((128, 2048, 8192) if dt == torch.bfloat16 else (128, 2048)):
                x = torch.randn(M, K, dtype=dt, device=dev)
                fns = [(lambda qw=qw: ops.w4a16_gemm(x, qw, sc, zp, None, g)) for qw in qws]
                n = 30
                t = time_graph(fns, n, 6, stream) / n
                fl = 2.0 * M * K * N
                res.append({"layer": name, "M": M, "dtype": str(dt).split(".")[-1], "group_size": g,
                            "us": round(t * 1e6, 1), "TFLOPs": round(fl / t / 1e12, 1),
                            "frac_fp16_mfma": round(fl / t / 1e12 / FP16_PEAK_TFLOPS, 4)})
        del qws
        torch.cuda.empty_cache()
    return res


def sweep(ops, dev, stream, args):
    """Every (shape, M) of BASELINE configs[1]: GB/s and TFLOP/s."""
    import torch
    res = []
    for name, K, N in LLAMA3_8B:
        copies = max(2, -(-2 * 256 * 2**20 // (K * N // 2)) + 1)
        lay = make_layer(K, N, copies, dev, seed=7)
        for M in (1, 8, 16, 32, 128, 2048):
            x = torch.randn(M, K, dtype=torch.float16, device=dev)
            fns = [(lambda c=c: ops.w4a16_gemm(x, lay[c][0], lay[c][2], lay[c][1], None, GROUP))
                   for c in range(copies)]
            try:
                n = 200 if M <= 128 else 30
                t = time_graph(fns, n, 10, stream) / n
            except RuntimeError as e:       # kernel family not available for this M
                res.append({"layer": name, "M": M, "error": str(e)[:80]})
                continue
            b, fl = w4a16_bytes(M, K, N), 2.0 * M * K * N
            res.append({"layer": name, "K": K, "N": N, "M": M, "us": round(t * 1e6, 2),
                        "GBps": round(b / t / 1e9, 1), "frac_hbm": round(b / t / 1e9 / HBM_PEAK_GBPS, 4),
                        "TFLOPs": round(fl / t / 1e12, 2),
                        "frac_fp16_mfma": round(fl / t / 1e12 / FP16_PEAK_TFLOPS, 4)})
        del lay
        torch.cuda.empty_cache()
    return res


if __name__ == "__main__":
    main()
