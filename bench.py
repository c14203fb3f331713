#!/usr/bin/env python3
"""Benchmark of the w4g64 quantized-linear path on one MI355X.

Headline (`value`): batch-1 QMV over a decode layer's seven projections
(q 4096->4096, k and v 4096->1024, o 4096->4096, gate and up 4096->12288,
down 12288->4096), in GB/s of ALGORITHMIC bytes (packed codes + scales + biases
+ x + y, each once).  A step is one pass over the seven projections of one
layer; consecutive steps use different layers' weights (8 layers, 868 MB in
rotation) so that no pass finds its weights in the 256 MB last-level cache.
By default q|k|v go out as one grouped launch and so do gate|up (the reference's
fused-QKV dispatch: same seven results, four launches); `--launch separate`
times seven launches, and the other mode's time is reported beside `value`.
The timed region is one HIP graph of `steps` passes, replayed between two
events on the launch stream with inputs already resident in HBM.

Also reported on the same JSON line: the roofline fraction of the QMV kernel
(timed region / launches), per-shape kernel durations of eager launches
(hipExtLaunchKernel events), the small-batch and video-DiT configurations,
QMM at M = 2048 in TFLOP/s, and the CPU baseline (the oracle's dequant + fp32
matmul on the host cores) on a bounded sample.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
MFMA_BF16_PEAK_TF = 2500.0  # MI355X dense bf16
# HBM-side bytes per decode layer of the default workload (all its QMV launches together) come from the
# committed summary of two rocprofv3 --pmc passes (FETCH_SIZE, WRITE_SIZE per dispatch, scaled by what the
# same counters read for a device-to-device copy of known size); the file states the build it was taken from.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "qmv_flow_kernel_decode_layer_m1_hbm_traffic_pmc.txt")
QMM_TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "qmm_big_kernel_m2048_mfma_lds_traffic_pmc.txt")
DIT_TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "qmm_big_kernel_dit_m16320_lora_r32.txt")


def traffic_from_profile(path=TRAFFIC_PROFILE, key="traffic_bytes_per_layer:"):
    """(bytes under `key`, text naming the profiled build) from a committed summary, or (None, None)."""
    try:
        text = open(path).read()
    except OSError:
        return None, None
    val, build = None, None
    for line in text.splitlines():
        if line.startswith(key):
            val = float(line.split(":", 1)[1])
        if line.startswith("build:"):
            build = line.split(":", 1)[1].strip()
    return val, build

DECODE_LAYER = [("q", 4096, 4096), ("k", 4096, 1024), ("v", 4096, 1024), ("o", 4096, 4096),
                ("gate", 4096, 12288), ("up", 4096, 12288), ("down", 12288, 4096)]
PREFILL = [("gate_up", 4096, 12288), ("down", 12288, 4096), ("attn", 4096, 4096)]
SMALL_BATCH = [(5120, 5120), (5120, 17408), (17408, 5120), (5120, 151936)]
DIT = [(5120, 5120), (5120, 20480), (20480, 5120)]


def alg_bytes(K, N, M):
    return N * K * 9 // 16 + 2 * M * K + 2 * M * N


def make_weight(torch, N, K, dev, gen):
    w = torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 8), dtype=torch.int32, device=dev, generator=gen)
    s = torch.empty((N, K // 64), dtype=torch.float32, device=dev).uniform_(0.005, 0.02, generator=gen).bfloat16()
    z = torch.randn((N, K // 64), dtype=torch.float32, device=dev, generator=gen)
    b = (-8.0 * s.float() * (1.0 + 0.05 * z)).bfloat16()
    return w, s, b


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--layers", type=int, default=8, help="distinct weight sets in rotation")
    ap.add_argument("--variant", type=int, default=0, help="QMV kernel variant (0 = automatic)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-qmm", action="store_true", help="skip the QMM section")
    ap.add_argument("--only", action="store_true",
                    help="run nothing but the selected launch mode of the decode-layer set (for a profiler: every "
                         "QMV launch in the trace then belongs to the timed workload)")
    ap.add_argument("--only-qmm", action="store_true",
                    help="run nothing but the fused QMM kernel on the three M=2048 projections and print their "
                         "timings (for a profiler: every qmm_tile_kernel dispatch then belongs to that workload)")
    ap.add_argument("--only-small", type=int, default=0, metavar="M",
                    help="run nothing but the small-batch QMV set (BASELINE config 3: four shapes) at M rows, weights "
                         "rotated through HBM (for a profiler: every QMV dispatch then belongs to that workload)")
    ap.add_argument("--only-dit", action="store_true",
                    help="run nothing but the video-DiT QMM set (BASELINE config 5: three shapes at M = 16320) with "
                         "the rank-32 adapter (for a profiler)")
    ap.add_argument("--no-extras", action="store_true", help="skip the small-batch QMV and video-DiT QMM sections")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches instead of a HIP graph")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three 256 MiB device-to-device copies (a kernel of known traffic, to scale "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--launch", choices=["grouped", "separate", "concurrent"], default="grouped",
                    help="how a layer's seven projections are launched (default: q|k|v and gate|up grouped)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import vpipe_amd

    L = vpipe_amd.load()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(0x5EED0002)
    st = L.vpq_init()
    if st != 0:
        raise vpipe_amd.VpqError(st, "vpq_init")

    def copy_calibration():
        """Three 256 MiB device-to-device copies: a kernel of known traffic beside the profiled ones."""
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(generator=gen)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()

    if args.only_qmm:
        M, res = 2048, {}
        for name, K, N in PREFILL:
            w, s, b = make_weight(torch, N, K, dev, gen)
            x = torch.randn((M, K), device=dev, generator=gen).bfloat16()
            y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
            for _ in range(150):                       # ~40 ms: the clocks settle
                vpipe_amd.qmm_w4g64(w, s, b, x, K, N, M, out=y)
            torch.cuda.synchronize()
            t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0.record()
            for _ in range(20):
                vpipe_amd.qmm_w4g64(w, s, b, x, K, N, M, out=y)
            t1.record()
            torch.cuda.synchronize()
            us = t0.elapsed_time(t1) * 1e3 / 20
            res[name] = {"K": K, "N": N, "M": M, "us": round(us, 2),
                         "TFLOPs": round(2.0 * M * N * K / (us * 1e-6) / 1e12, 1)}
        if args.copy_calibration:
            copy_calibration()
        print(json.dumps({"qmm_m2048_fused_kernel_only": res, "build": vpipe_amd.build_id()}))
        return

    if args.only_small:
        M, res = args.only_small, {}
        for K, N in SMALL_BATCH:
            copies = max(2, min(8, int(600e6 // (N * K * 9 // 16))))
            packs = [make_weight(torch, N, K, dev, gen) for _ in range(copies)]
            x = torch.randn((M, K), device=dev, generator=gen).bfloat16()
            y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
            ws = vpipe_amd.qmv_workspace(K, N, M, dev)
            for i in range(4 * copies):
                w, s, b = packs[i % copies]
                vpipe_amd.qmv_w4g64(w, s, b, x, K, N, M, out=y, ws=ws)
            torch.cuda.synchronize()
            res["%d->%d" % (K, N)] = {"launches": 4 * copies, "algorithmic_bytes": alg_bytes(K, N, M)}
            del packs
        if args.copy_calibration:
            copy_calibration()
        print(json.dumps({"qmv_small_batch_only": res, "M": M, "build": vpipe_amd.build_id()}))
        return
    if args.only_dit:
        M, r, res = 16320, 32, {}
        for K, N in DIT:
            w, s, b = make_weight(torch, N, K, dev, gen)
            x = torch.randn((M, K), device=dev, generator=gen).bfloat16()
            y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
            A = (torch.randn((r, K), device=dev, generator=gen) * 0.02).bfloat16()
            B = (torch.randn((N, r), device=dev, generator=gen) * 0.02).bfloat16()
            t = torch.empty((M, r), dtype=torch.bfloat16, device=dev)
            for _ in range(6):
                vpipe_amd.qmm_w4g64(w, s, b, x, K, N, M, out=y, lora_A=A, lora_B=B, r=r, alpha=1.0, t_ws=t)
            torch.cuda.synchronize()
            res["%d->%d" % (K, N)] = {"launches": 6, "flops": 2.0 * M * N * K, "lora_flops": 2.0 * M * r * (K + N)}
            del w, s, b, x, y, A, B, t
        if args.copy_calibration:
            copy_calibration()
        print(json.dumps({"qmm_dit_only": res, "M": M, "r": r, "build": vpipe_amd.build_id()}))
        return

    # ---- inputs, resident in HBM ------------------------------------------------
    layers = []
    for _ in range(args.layers):
        layers.append([make_weight(torch, N, K, dev, gen) for _, K, N in DECODE_LAYER])
    xs = {K: torch.randn((1, K), device=dev, generator=gen).bfloat16() for K in (4096, 12288)}
    ys = [torch.empty((1, N), dtype=torch.bfloat16, device=dev) for _, _, N in DECODE_LAYER]
    wss = [vpipe_amd.qmv_workspace(K, N, 1, dev) for _, K, N in DECODE_LAYER]
    layer_bytes = sum(alg_bytes(K, N, 1) for _, K, N in DECODE_LAYER)

    def project(li, j):
        _, K, N = DECODE_LAYER[j]
        w, s, b = layers[li][j]
        vpipe_amd.qmv_w4g64(w, s, b, xs[K], K, N, 1, out=ys[j], ws=wss[j], variant=args.variant)

    groups = {}

    def group(li, js):
        if (li, js) not in groups:
            K = DECODE_LAYER[js[0]][1]
            packs = [layers[li][j] + (DECODE_LAYER[j][2],) for j in js]
            groups[(li, js)] = vpipe_amd.capi.QmvGroup(packs, xs[K], K, 1, [ys[j] for j in js])
        groups[(li, js)].launch()

    def pass_separate(li):
        """Seven launches, one per projection."""
        for j in range(len(DECODE_LAYER)):
            project(li, j)

    def pass_grouped(li):
        """Four launches: q|k|v read the same x and go out as ONE grouped launch, so do gate|up
        (the reference's fused-QKV dispatch, gpu-kernels/metal/quant/affine_qmv.metal:405-516);
        o and down are single launches.  Same seven results, bit for bit."""
        group(li, (0, 1, 2))
        project(li, 3)
        group(li, (4, 5))
        project(li, 6)

    side = [torch.cuda.Stream(device=dev), torch.cuda.Stream(device=dev)]

    def pass_concurrent(li):
        """Seven launches with q|k|v and gate|up as concurrent graph branches (the reference's
        ConcurrentScope, apple-silicon/metal-compute/compute-encoder.h).  Measured slower than one
        stream on MI355X (55.7 vs 42.5 us per layer); kept for reproduction."""
        main = torch.cuda.current_stream()
        side[0].wait_stream(main)
        side[1].wait_stream(main)
        project(li, 0)
        with torch.cuda.stream(side[0]):
            project(li, 1)
        with torch.cuda.stream(side[1]):
            project(li, 2)
        main.wait_stream(side[0])
        main.wait_stream(side[1])
        project(li, 3)
        side[0].wait_stream(main)
        project(li, 4)
        with torch.cuda.stream(side[0]):
            project(li, 5)
        main.wait_stream(side[0])
        project(li, 6)

    def time_steps(layer_pass, steps, use_graph, repeats=7):
        """ms per step of `steps` passes: one HIP graph replayed between two events (or eager), the median of
        `repeats` such timings (and all of them, for the spread)."""
        graph = None
        if use_graph:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for i in range(steps):
                    layer_pass(i % args.layers)
            graph.replay()                      # untimed: first replay uploads the graph
            torch.cuda.synchronize()
        times = []
        for _ in range(repeats):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            if graph is not None:
                graph.replay()
            else:
                for i in range(steps):
                    layer_pass(i % args.layers)
            e1.record()
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1) / steps)
        return float(np.median(times)), times

    def kernel_durations(layer_pass, launches_per_pass):
        """Per-kernel durations (hipExtLaunchKernel events: kernel start -> end), us [pass, launch]."""
        passes = max(4 * args.layers, 32)
        n_launch = passes * launches_per_pass
        st = L.vpq_profile_enable(n_launch)
        if st != 0:
            raise vpipe_amd.VpqError(st, "vpq_profile_enable")
        for i in range(passes):
            layer_pass(i % args.layers)
        buf = (ctypes.c_float * n_launch)()
        got = L.vpq_profile_read(buf, n_launch)
        L.vpq_profile_enable(0)
        assert got == n_launch, got
        return np.array(buf[:], dtype=np.float64).reshape(passes, launches_per_pass) * 1e3

    modes = {"grouped": (pass_grouped, 4, "q|k|v and gate|up as grouped launches (4 launches per layer)"),
             "separate": (pass_separate, 7, "one launch per projection (7 launches per layer)"),
             "concurrent": (pass_concurrent, 7, "7 launches, q|k|v and gate|up as concurrent graph branches")}
    if args.variant != 0 and args.launch == "grouped":
        args.launch = "separate"                # a forced kernel variant only exists per projection
    layer_pass, launches_per_layer, launch_text = modes[args.launch]
    use_graph = not args.no_graph

    if args.only:
        args.no_qmm = args.no_extras = args.no_cpu = True
    for i in range(args.warmup):
        if not args.only:
            pass_separate(i % args.layers)
        layer_pass(i % args.layers)
    torch.cuda.synchronize()

    # ---- timed region ---------------------------------------------------------------
    ms_per_step, ms_all = time_steps(layer_pass, args.steps, use_graph)
    value = layer_bytes / (ms_per_step * 1e-3) / 1e9
    launch = ("hipgraph, " if use_graph else "eager, ") + launch_text
    other = "separate" if args.launch != "separate" else "grouped"
    ms_other = time_steps(modes[other][0], args.steps, use_graph)[0] if args.variant == 0 and not args.only else None

    # ---- what this GPU gives to ANY kernel at these launch sizes, measured in this run the same way ----
    # A kernel that only reads (the library's measurement aid: 16-byte loads, all requested up front) over the
    # same byte counts per launch as the layer's launches, from a rotating buffer larger than the last-level
    # cache, as the same kind of HIP graph; and a kernel that does nothing.
    ceilings = None
    if not args.only:
        sink = torch.zeros((4,), dtype=torch.int32, device=dev)
        if launches_per_layer == 4:
            launch_bytes = [sum(alg_bytes(K, N, 1) for _, K, N in DECODE_LAYER[0:3]), alg_bytes(4096, 4096, 1),
                            sum(alg_bytes(K, N, 1) for _, K, N in DECODE_LAYER[4:6]), alg_bytes(12288, 4096, 1)]
        else:
            launch_bytes = [alg_bytes(K, N, 1) for _, K, N in DECODE_LAYER]
        launch_bytes = [(b + 15) // 16 * 16 for b in launch_bytes]
        per_layer = sum(launch_bytes)
        pool = torch.empty((args.layers * per_layer + 4096,), dtype=torch.uint8, device=dev).random_(generator=gen)
        base = (pool.data_ptr() + 255) // 256 * 256

        def pass_read(li):
            off = base + li * per_layer
            for nb in launch_bytes:
                st_ = L.vpq_profile_read_kernel(vpipe_amd.capi._stream(), ctypes.c_void_p(off), nb, ctypes.c_void_p(sink.data_ptr()))
                if st_ != 0:
                    raise vpipe_amd.VpqError(st_, "vpq_profile_read_kernel")
                off += nb

        def pass_empty(li):
            for _ in launch_bytes:
                L.vpq_profile_empty_kernel(vpipe_amd.capi._stream(), ctypes.c_void_p(sink.data_ptr()))

        for i in range(args.layers):
            pass_read(i)
            pass_empty(i)
        torch.cuda.synchronize()
        ms_read, _ = time_steps(pass_read, args.steps, use_graph)
        ms_empty, _ = time_steps(pass_empty, args.steps, use_graph)
        dur_read = kernel_durations(pass_read, len(launch_bytes))
        dur_empty = kernel_durations(pass_empty, len(launch_bytes))
        ceilings = {"read_only_kernel_us_per_layer": round(ms_read * 1e3, 3),
                    "read_only_kernel_GBps": round(per_layer / (ms_read * 1e-3) / 1e9, 1),
                    "empty_kernel_us_per_launch_in_graph": round(ms_empty * 1e3 / len(launch_bytes), 3),
                    "read_only_eager_kernel_us": {"%.1f MB" % (nb / 1e6): round(float(dur_read[:, i].mean()), 3)
                                                  for i, nb in enumerate(launch_bytes)},
                    "empty_eager_kernel_us": round(float(dur_empty.mean()), 3),
                    "bytes_per_launch": launch_bytes}
        # the lm_head-sized launch (config 3's 5120 -> 151936): one read of 438 MB, eager kernel duration
        big = alg_bytes(5120, 151936, 1) // 16 * 16
        bigpool = torch.empty((2 * big + 256,), dtype=torch.uint8, device=dev).random_(generator=gen)
        bbase = (bigpool.data_ptr() + 255) // 256 * 256
        L.vpq_profile_enable(8)
        for i in range(8):
            L.vpq_profile_read_kernel(vpipe_amd.capi._stream(), ctypes.c_void_p(bbase + (i % 2) * big), big, ctypes.c_void_p(sink.data_ptr()))
        kb = (ctypes.c_float * 8)()
        n = L.vpq_profile_read(kb, 8)
        L.vpq_profile_enable(0)
        us_big = float(np.median(kb[2:n])) * 1e3
        ceilings["read_only_eager_kernel_us"]["%.1f MB" % (big / 1e6)] = round(us_big, 2)
        ceilings["read_only_GBps_at_438MB"] = round(big / (us_big * 1e-6) / 1e9, 1)
        del pool, bigpool

    # ---- roofline of the dominant kernel ------------------------------------------------
    # Every launch of the timed region is the same kernel (qmv_mfma_kernel); its average launch
    # duration is the timed region (events on the launch stream around the graph replay) divided
    # by the launches in it -- back-to-back kernels of one stream, so launch gaps are included.
    avg_launch_us = ms_per_step * 1e3 / launches_per_layer
    achieved = (layer_bytes / launches_per_layer) / (avg_launch_us * 1e-6) / 1e9
    # Per-launch detail from hipExtLaunchKernel start/stop events of eager launches (these run
    # slower than the same kernels inside the graph when the host cannot keep the queue full).
    dur = kernel_durations(layer_pass, launches_per_layer)
    kernel_us_per_layer = float(dur.sum(axis=1).mean())
    per_shape = {}
    if launches_per_layer == 7 or not args.only:
        dur7 = dur if launches_per_layer == 7 else kernel_durations(pass_separate, 7)
        for j, (name, K, N) in enumerate(DECODE_LAYER):
            us = float(dur7[:, j].mean())
            per_shape[name] = {"K": K, "N": N, "us": round(us, 3),
                               "GBps": round(alg_bytes(K, N, 1) / (us * 1e-6) / 1e9, 1)}
    default_workload = args.variant == 0
    traffic_layer, traffic_build = traffic_from_profile()
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": (traffic_layer / launches_per_layer) if (default_workload and traffic_layer and launches_per_layer == 4) else None,
                "traffic_profile": ("profiles/" + os.path.basename(TRAFFIC_PROFILE) + " (" + str(traffic_build) + ")") if traffic_layer else None,
                "kernel": "qmv_flow_kernel (all %d launches of a layer)" % launches_per_layer,
                "avg_launch_us": round(avg_launch_us, 3),
                "bytes_per_launch": layer_bytes / launches_per_layer,
                "launches_timed": args.steps * launches_per_layer,
                "timing": "median of %d replays of one HIP graph of %d steps; all replays, us per layer: %s"
                          % (len(ms_all), args.steps, [round(t * 1e3, 3) for t in ms_all])}
    if ceilings is not None:
        roofline["measured_ceilings"] = ceilings
        roofline["frac_of_read_only_kernel"] = round(ceilings["read_only_kernel_us_per_layer"] / (ms_per_step * 1e3), 4)
    if launches_per_layer == 4:
        roofline["eager_launch_us"] = {n: round(float(dur[:, i].mean()), 3)
                                       for i, n in enumerate(("q|k|v", "o", "gate|up", "down"))}

    build = vpipe_amd.build_id()
    roofline["build"] = build
    if traffic_layer:
        roofline["traffic_profile_is_of_this_build"] = bool(traffic_build) and str(traffic_build).split()[0] == build
    out = {
        "metric": "4-bit QMV HBM GB/s at batch 1 (decode-layer projection set)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "decode-layer QMV set, M=1, w4g64: q,o 4096->4096; k,v 4096->1024; "
                               "gate,up 4096->12288; down 12288->4096",
                   "layers_in_rotation": args.layers, "launch": launch,
                   "algorithmic_bytes_per_step": layer_bytes},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "us_per_layer": round(ms_per_step * 1e3, 3),
        "eager_kernel_us_per_layer": round(kernel_us_per_layer, 3),
        "per_shape": per_shape,
        "roofline": roofline,
    }
    if ms_other is not None:
        out["us_per_layer_" + other] = round(ms_other * 1e3, 3)

    def steady_us(fn, iters, warm_ms=40.0):
        """us per call of fn at the clocks the box settles at: the calls run back to back for warm_ms before the
        timed ones (the first milliseconds after an idle spell run at lower clocks), then `iters` calls between
        two events on the stream."""
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        fn()
        torch.cuda.synchronize()
        t0.record()
        fn()
        t1.record()
        torch.cuda.synchronize()
        n_warm = max(2, int(warm_ms / max(t0.elapsed_time(t1), 1e-3)))
        for _ in range(n_warm):
            fn()
        t0.record()
        for _ in range(iters):
            fn()
        t1.record()
        torch.cuda.synchronize()
        return t0.elapsed_time(t1) * 1e3 / iters

    def dense_gemm_us(w, s, b, x, y, K, N, iters=20):
        """Yardstick, not product: the vendor library's dense bf16 GEMM (torch.matmul) on the SAME
        operands with the weight expanded to bf16 beforehand -- what a GEMM with no dequantization
        at all reaches on this box with these (non-trivial) values."""
        wdeq = vpipe_amd.dequant_w4g64(w, s, b, K, N)
        return steady_us(lambda: torch.matmul(x, wdeq.t(), out=y), iters)

    def dense_route_us(w, s, b, x, y, K, N, M, iters):
        """The library's own dequant-once route: (expansion + dense GEMM per call, dense GEMM alone
        when the expansion is kept), us per call from events on the stream."""
        wdeq = torch.empty((N, K), dtype=torch.bfloat16, device=dev)
        return [steady_us(lambda: vpipe_amd.qmm_dense_route_w4g64(w, s, b, x, K, N, M, wdeq, expand=expand, out=y), iters)
                for expand in (True, False)]

    # ---- QMM at M = 2048 ---------------------------------------------------------------
    if not args.no_qmm:
        M = 2048
        qmm = {}
        tot_flops, tot_us = 0.0, 0.0
        for name, K, N in PREFILL:
            w, s, b = make_weight(torch, N, K, dev, gen)
            x = torch.randn((M, K), device=dev, generator=gen).bfloat16()
            y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
            us = steady_us(lambda: vpipe_amd.qmm_w4g64(w, s, b, x, K, N, M, out=y), 20)
            flops = 2.0 * M * N * K
            qmm[name] = {"K": K, "N": N, "M": M, "us": round(us, 2), "TFLOPs": round(flops / (us * 1e-6) / 1e12, 1),
                         "vendor_dense_bf16_TFLOPs": round(flops / (dense_gemm_us(w, s, b, x, y, K, N) * 1e-6) / 1e12, 1)}
            dr = dense_route_us(w, s, b, x, y, K, N, M, 20)
            qmm[name]["dense_route_TFLOPs"] = round(flops / (dr[0] * 1e-6) / 1e12, 1)
            qmm[name]["dense_route_kept_expansion_TFLOPs"] = round(flops / (dr[1] * 1e-6) / 1e12, 1)
            tot_flops += flops
            tot_us += us
            del w, s, b, x, y
        ach = tot_flops / (tot_us * 1e-6) / 1e12
        out["qmm_m2048"] = qmm
        qmm_traffic, qmm_traffic_build = traffic_from_profile(QMM_TRAFFIC_PROFILE, "traffic_bytes_4096x12288_m2048:")
        out["roofline_qmm"] = {"bound": "mfma", "achieved": round(ach, 1), "peak": MFMA_BF16_PEAK_TF,
                               "unit": "TFLOP/s", "frac": round(ach / MFMA_BF16_PEAK_TF, 4), "traffic": qmm_traffic,
                               "traffic_of": "one 4096->12288 launch at M = 2048 (fetched + written; algorithmic 95.4 MB), "
                                             "profiles/" + os.path.basename(QMM_TRAFFIC_PROFILE) + " (" + str(qmm_traffic_build) + ")",
                               "traffic_profile_is_of_this_build": bool(qmm_traffic_build) and
                                                                   str(qmm_traffic_build).split()[0] == vpipe_amd.build_id(),
                               "kernel": "qmm_big_kernel<3,false,0> (4096->12288: 256x192 tiles) and qmm_big_kernel<2,false,0> "
                                         "(12288->4096, 4096->4096: 256x128 tiles); flops of the three over their time",
                               "timing": "us per call over 20 back-to-back calls after 40 ms of the same calls "
                                         "(the clocks the box settles at), events on the stream",
                               "note": "vendor_dense_bf16_TFLOPs in qmm_m2048 = torch.matmul on the expanded "
                                       "weight, same operands, timed the same way: the dense-GEMM rate this box "
                                       "sustains on real data"}

    # ---- the other configurations, as context (not part of `value`) -----------------------
    if not args.no_extras:
        def kernel_us(fn, iters):
            for _ in range(2):
                fn(0)
            torch.cuda.synchronize()
            L.vpq_profile_enable(8 * iters)
            for i in range(iters):
                fn(i)
            kb = (ctypes.c_float * (8 * iters))()
            n = L.vpq_profile_read(kb, 8 * iters)
            L.vpq_profile_enable(0)
            return float(np.sum(kb[:n])) * 1e3 / iters     # all kernels of a call (LoRA: two, the sampler: five)

        # small-batch QMV of a 5120-hidden model, weights rotated so that they come from HBM
        small, small_bytes, small_us = {}, 0.0, 0.0
        for K, N in SMALL_BATCH:
            copies = max(2, min(8, int(600e6 // (N * K * 9 // 16))))
            packs = [make_weight(torch, N, K, dev, gen) for _ in range(copies)]
            row = {}
            for M in (1, 2, 4, 8, 16):
                x = torch.randn((M, K), device=dev, generator=gen).bfloat16()
                y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)

                ws = vpipe_amd.qmv_workspace(K, N, M, dev)     # lets the library split K across workgroups where that pays

                def call(i, x=x, y=y, M=M, ws=ws):
                    w, s, b = packs[i % copies]
                    vpipe_amd.qmv_w4g64(w, s, b, x, K, N, M, out=y, ws=ws)
                # as the headline is timed: one HIP graph of back-to-back calls over the rotating packs between two
                # events, median of 5 replays (launch gaps included, 1.6-1.7 us per launch in a graph); beside it
                # the kernel's own duration from events around each eager launch (their floor is ~4 us)
                n_calls = 8 * copies
                saved_layers, args.layers = args.layers, n_calls
                ms, _ = time_steps(call, n_calls, use_graph, repeats=5)
                args.layers = saved_layers
                us = ms * 1e3
                us_ev = kernel_us(call, 2 * copies)
                row["M=%d" % M] = {"us": round(us, 2), "GBps": round(alg_bytes(K, N, M) / (us * 1e-6) / 1e9, 1),
                                   "eager_event_us": round(us_ev, 2)}
                small_bytes += alg_bytes(K, N, M)
                small_us += us
            small["%d->%d" % (K, N)] = row
            del packs
        out["qmv_small_batch"] = small
        out["roofline_small_batch"] = {
            "bound": "hbm", "achieved": round(small_bytes / (small_us * 1e-6) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(small_bytes / (small_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4), "traffic": None,
            "kernel": "qmv_flow_kernel_1 (M = 1), qmv_ring_kernel (2..16 rows), qmv_stream_kernel (2..4 rows over "
                      "5120->151936): the 20 (shape, M) cases of BASELINE config 3, algorithmic bytes of all over "
                      "the time of all",
            "timing": "per case one HIP graph of 8 x (packs in rotation) calls, median of 5 replays",
            "profile": "profiles/qmv_small_batch_m1_m4_m16.txt (rocprofv3 kernel trace + FETCH_SIZE / WRITE_SIZE)"}

        # video-DiT QMM with the fused rank-32 LoRA (flops of the base contraction only)
        M, r, alpha = 16320, 32, 1.0
        dit = {}
        for K, N in DIT:
            w, s, b = make_weight(torch, N, K, dev, gen)
            x = torch.randn((M, K), device=dev, generator=gen).bfloat16()
            y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
            A = (torch.randn((r, K), device=dev, generator=gen) * 0.02).bfloat16()
            B = (torch.randn((N, r), device=dev, generator=gen) * 0.02).bfloat16()
            t = torch.empty((M, r), dtype=torch.bfloat16, device=dev)
            us0 = steady_us(lambda: vpipe_amd.qmm_w4g64(w, s, b, x, K, N, M, out=y), 5)
            us1 = steady_us(lambda: vpipe_amd.qmm_w4g64(w, s, b, x, K, N, M, out=y, lora_A=A, lora_B=B, r=r,
                                                        alpha=alpha, t_ws=t), 5)
            flops = 2.0 * M * N * K
            dit["%d->%d" % (K, N)] = {"us": round(us0, 1), "TFLOPs": round(flops / (us0 * 1e-6) / 1e12, 1),
                                      "us_with_lora": round(us1, 1),
                                      "TFLOPs_with_lora": round(flops / (us1 * 1e-6) / 1e12, 1),
                                      "vendor_dense_bf16_TFLOPs": round(
                                          flops / (dense_gemm_us(w, s, b, x, y, K, N, iters=5) * 1e-6) / 1e12, 1)}
            dr = dense_route_us(w, s, b, x, y, K, N, M, 5)
            dit["%d->%d" % (K, N)]["dense_route_TFLOPs"] = round(flops / (dr[0] * 1e-6) / 1e12, 1)
            dit["%d->%d" % (K, N)]["dense_route_kept_expansion_TFLOPs"] = round(flops / (dr[1] * 1e-6) / 1e12, 1)
            # the same route with the adapter in the dense GEMM's accumulators (the bits of the fused call)
            wdeq = torch.empty((N, K), dtype=torch.bfloat16, device=dev)
            drl = [steady_us(lambda: vpipe_amd.qmm_dense_route_w4g64(w, s, b, x, K, N, M, wdeq, expand=e, out=y, lora_A=A,
                                                                     lora_B=B, r=r, alpha=alpha, t_ws=t), 5)
                   for e in (True, False)]
            dit["%d->%d" % (K, N)]["dense_route_with_lora_TFLOPs"] = round(flops / (drl[0] * 1e-6) / 1e12, 1)
            dit["%d->%d" % (K, N)]["dense_route_kept_expansion_with_lora_TFLOPs"] = round(flops / (drl[1] * 1e-6) / 1e12, 1)
            dit["%d->%d" % (K, N)]["us_dense_route_with_lora"] = round(drl[0], 1)
            del w, s, b, x, y, A, B, t, wdeq
        out["qmm_dit_m16320_lora_r32"] = dit
        dit_flops = sum(2.0 * M * N * K for K, N in DIT)
        dit_us = sum(v["us"] for v in dit.values())
        dit_us_lora = sum(v["us_with_lora"] for v in dit.values())
        dit_traffic, dit_traffic_build = traffic_from_profile(DIT_TRAFFIC_PROFILE,
                                                              "traffic_bytes_per_launch_mean_of_the_three_shapes:")
        dit_alg = sum(2.0 * M * K + N * K * 9 / 16.0 + 2.0 * M * N for K, N in DIT) / len(DIT)
        out["roofline_qmm_dit"] = {
            "bound": "mfma", "achieved": round(dit_flops / (dit_us * 1e-6) / 1e12, 1), "peak": MFMA_BF16_PEAK_TF,
            "unit": "TFLOP/s", "frac": round(dit_flops / (dit_us * 1e-6) / 1e12 / MFMA_BF16_PEAK_TF, 4),
            "traffic": dit_traffic,
            "traffic_of": "mean over the three shapes of one qmm_big_kernel<4,true,0> launch with the rank-32 adapter "
                          "(fetched + written; algorithmic mean %.1f MB: x, the pack and y once), profiles/%s (%s)"
                          % (dit_alg / 1e6, os.path.basename(DIT_TRAFFIC_PROFILE), dit_traffic_build),
            "traffic_profile_is_of_this_build": bool(dit_traffic_build) and
                                                str(dit_traffic_build).split()[0] == vpipe_amd.build_id(),
            "achieved_with_lora_r32": round(dit_flops / (dit_us_lora * 1e-6) / 1e12, 1),
            "achieved_with_lora_r32_dense_route": round(
                dit_flops / (sum(v["us_dense_route_with_lora"] for v in dit.values()) * 1e-6) / 1e12, 1),
            "kernel": "qmm_big_kernel<4,*,0> (256 x 256 tiles) + lora_a_dma_kernel; flops of the three base "
                      "contractions (2 M N K) over their time, the adapter's flops not counted",
            "timing": "us per call over 5 back-to-back calls after 40 ms of the same calls, events on the stream",
            "profile": "profiles/qmm_big_kernel_dit_m16320_lora_r32.txt (rocprofv3 kernel trace + MFMA busy)"}

    # ---- fused gate|up + SwiGLU (interleaved pack), as context ------------------------------
    if not args.no_extras:
        fused = []
        for li in range(args.layers):
            fused.append(vpipe_amd.interleave_gate_up(layers[li][4], layers[li][5]))
        y_mlp = torch.empty((1, 12288), dtype=torch.bfloat16, device=dev)

        def pass_fused_mlp(li):
            """q|k|v grouped, o, gate|up + SwiGLU as one launch over the interleaved pack, down."""
            group(li, (0, 1, 2))
            project(li, 3)
            w, s, b = fused[li]
            vpipe_amd.qmv_swiglu_w4g64(w, s, b, xs[4096], 4096, 24576, 1, out=y_mlp)
            project(li, 6)

        for i in range(args.layers):
            pass_fused_mlp(i)
        torch.cuda.synchronize()
        ms_f, _ = time_steps(pass_fused_mlp, args.steps, use_graph)
        fm = {"us_per_layer": round(ms_f * 1e3, 3), "GBps": round((layer_bytes - 2 * 12288) / (ms_f * 1e-3) / 1e9, 1),
              "launches_per_layer": 4}
        M = 2048
        w, s, b = fused[0]
        x = torch.randn((M, 4096), device=dev, generator=gen).bfloat16()
        y = torch.empty((M, 12288), dtype=torch.bfloat16, device=dev)
        us = steady_us(lambda: vpipe_amd.qmm_swiglu_w4g64(w, s, b, x, 4096, 24576, M, out=y), 20)
        fm["qmm_swiglu_m2048_4096->2x12288"] = {"us": round(us, 2),
                                               "TFLOPs": round(2.0 * M * 24576 * 4096 / (us * 1e-6) / 1e12, 1)}
        out["fused_mlp_swiglu"] = fm
        del fused, x, y

        # dense expansion (the a1 kernel): 9/16 B read and 2 B written per weight
        dq = {}
        for K, N in ((4096, 4096), (4096, 12288), (5120, 20480)):
            w, s, b = make_weight(torch, N, K, dev, gen)
            wdeq = torch.empty((N, K), dtype=torch.bfloat16, device=dev)
            us = kernel_us(lambda i: vpipe_amd.dequant_w4g64(w, s, b, K, N, out=wdeq), 6)
            nbytes = N * K * 9 // 16 + 2 * N * K
            dq["%dx%d" % (N, K)] = {"us": round(us, 2), "GBps": round(nbytes / (us * 1e-6) / 1e9, 1)}
            del w, s, b, wdeq
        out["dequant_w4g64"] = dq

        # 8-bit twin, general kernel (one wavefront per row): 17/16 B per weight
        w8 = {}
        for K, N in ((4096, 4096), (5120, 151936)):
            copies = max(2, min(8, int(600e6 // (N * K * 17 // 16))))
            packs = []
            for _ in range(copies):
                w = torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 4), dtype=torch.int32, device=dev, generator=gen)
                s = torch.empty((N, K // 64), dtype=torch.float32, device=dev).uniform_(0.0003, 0.0012, generator=gen).bfloat16()
                packs.append((w, s, (-128.0 * s.float()).bfloat16()))
            x = torch.randn((1, K), device=dev, generator=gen).bfloat16()
            y = torch.empty((1, N), dtype=torch.bfloat16, device=dev)

            def call8(i, x=x, y=y, K=K, N=N):
                w, s, b = packs[i % copies]
                vpipe_amd.qmv_w8g64(w, s, b, x, K, N, 1, out=y)
            us = kernel_us(call8, 2 * copies)
            nbytes = N * K * 17 // 16 + 2 * K + 2 * N
            w8["%d->%d" % (K, N)] = {"us": round(us, 2), "GBps": round(nbytes / (us * 1e-6) / 1e9, 1)}
            del packs
        out["qmv_w8g64_m1"] = w8

        # 8-bit fused gate|up + SwiGLU (interleaved pack 4096 -> 2 x 12288) and the 8-bit MoE gathers of the
        # decode block below (hidden 2048, inner 768, 128 experts, top-8); IEEE binary16 elements on the
        # general kernel (one wavefront per row)
        w8g = {}
        K, F = 4096, 12288
        packs = []
        for _ in range(3):
            w = torch.randint(-2 ** 31, 2 ** 31 - 1, (2 * F, K // 4), dtype=torch.int32, device=dev, generator=gen)
            s = torch.empty((2 * F, K // 64), dtype=torch.float32, device=dev).uniform_(0.0003, 0.0012, generator=gen).bfloat16()
            packs.append((w, s, (-128.0 * s.float()).bfloat16()))
        x = torch.randn((1, K), device=dev, generator=gen).bfloat16()
        y = torch.empty((1, F), dtype=torch.bfloat16, device=dev)
        us = kernel_us(lambda i: vpipe_amd.qmv_gated_w8g64(*packs[i % 3], x, K, 2 * F, 1, out=y), 6)
        w8g["gate|up+swiglu 4096->2x12288"] = {"us": round(us, 2),
                                               "GBps": round((2 * F * K * 17 // 16) / (us * 1e-6) / 1e9, 1)}
        del packs
        H8, I8, E8, k8 = 2048, 768, 128, 8
        gw8 = torch.randint(-2 ** 31, 2 ** 31 - 1, (E8, 2 * I8, H8 // 4), dtype=torch.int32, device=dev, generator=gen)
        gs8 = torch.empty((E8, 2 * I8, H8 // 64), dtype=torch.float32, device=dev).uniform_(0.0003, 0.0012, generator=gen).bfloat16()
        gb8 = (-128.0 * gs8.float()).bfloat16()
        ids8 = [torch.randperm(E8, device=dev, generator=gen)[:k8].to(torch.int32).contiguous() for _ in range(16)]
        xm8 = torch.randn((1, H8), device=dev, generator=gen).bfloat16()
        act8 = torch.empty((k8, I8), dtype=torch.bfloat16, device=dev)
        us = kernel_us(lambda i: vpipe_amd.gather_qmv_gated_w8g64(gw8, gs8, gb8, xm8, H8, 2 * I8, ids8[i % 16], k8, E8, out=act8), 16)
        w8g["moe gather gate|up+swiglu 2048->2x768, top-8 of 128"] = {
            "us": round(us, 2), "GBps": round(k8 * (2 * I8 * H8 * 17 // 16) / (us * 1e-6) / 1e9, 1)}
        del gw8, gs8, gb8
        out["qmv_w8g64_gated_and_gathered"] = w8g

        # fused 8-bit GEMM at M = 2048 (the large-tile kernel with byte codes; the tile kernel beside it), clocks settled
        K, N, M8 = 4096, 12288, 2048
        w = torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 4), dtype=torch.int32, device=dev, generator=gen)
        s = torch.empty((N, K // 64), dtype=torch.float32, device=dev).uniform_(0.0003, 0.0012, generator=gen).bfloat16()
        b = (-128.0 * s.float()).bfloat16()
        x = torch.randn((M8, K), device=dev, generator=gen).bfloat16()
        y = torch.empty((M8, N), dtype=torch.bfloat16, device=dev)
        us = steady_us(lambda: vpipe_amd.qmm_w8g64(w, s, b, x, K, N, M8, out=y), 10)
        us_t = steady_us(lambda: vpipe_amd.qmm_w8g64(w, s, b, x, K, N, M8, out=y, tile_n=128), 10)
        out["qmm_w8g64_m2048_4096->12288"] = {"us": round(us, 2), "TFLOPs": round(2.0 * M8 * N * K / (us * 1e-6) / 1e12, 1),
                                              "tile_kernel_TFLOPs": round(2.0 * M8 * N * K / (us_t * 1e-6) / 1e12, 1)}
        del w, s, b
        # the group-32 pack on the same shape
        w = torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 8), dtype=torch.int32, device=dev, generator=gen)
        s = torch.empty((N, K // 32), dtype=torch.float32, device=dev).uniform_(0.005, 0.02, generator=gen).bfloat16()
        b = (-8.0 * s.float()).bfloat16()
        us = steady_us(lambda: vpipe_amd.qmm_w4g32(w, s, b, x, K, N, M8, out=y), 10)
        us_t = steady_us(lambda: vpipe_amd.qmm_w4g32(w, s, b, x, K, N, M8, out=y, tile_n=128), 10)
        out["qmm_w4g32_m2048_4096->12288"] = {"us": round(us, 2), "TFLOPs": round(2.0 * M8 * N * K / (us * 1e-6) / 1e12, 1),
                                              "tile_kernel_TFLOPs": round(2.0 * M8 * N * K / (us_t * 1e-6) / 1e12, 1)}
        del w, s, b, x, y

        f16 = {}
        for K, N in ((4096, 4096), (4096, 12288)):
            packs = []
            for _ in range(4):
                w = torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 8), dtype=torch.int32, device=dev, generator=gen)
                s = torch.empty((N, K // 64), dtype=torch.float32, device=dev).uniform_(0.005, 0.02, generator=gen).half()
                packs.append((w, s, (-8.0 * s.float()).half()))
            x = torch.randn((1, K), device=dev, generator=gen).half()
            y = torch.empty((1, N), dtype=torch.float16, device=dev)
            us = kernel_us(lambda i, x=x, y=y, K=K, N=N: vpipe_amd.qmv_w4g64_f16(*packs[i % 4], x, K, N, 1, out=y), 8)
            f16["%d->%d" % (K, N)] = {"us": round(us, 2), "GBps": round((N * K * 9 // 16 + 2 * K + 2 * N) / (us * 1e-6) / 1e9, 1)}
            del packs
        out["qmv_f16_elements_m1"] = f16

        # the fused GEMM on binary16 elements (the large-tile kernel with the f16 MFMA), clocks settled
        K, N, M16 = 4096, 12288, 2048
        w = torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 8), dtype=torch.int32, device=dev, generator=gen)
        s = torch.empty((N, K // 64), dtype=torch.float32, device=dev).uniform_(0.005, 0.02, generator=gen).half()
        b = (-8.0 * s.float()).half()
        x = torch.randn((M16, K), device=dev, generator=gen).half()
        y = torch.empty((M16, N), dtype=torch.float16, device=dev)
        us = steady_us(lambda: vpipe_amd.qmm_w4g64_f16(w, s, b, x, K, N, M16, out=y), 10)
        out["qmm_f16_elements_m2048_4096->12288"] = {"us": round(us, 2),
                                                     "TFLOPs": round(2.0 * M16 * N * K / (us * 1e-6) / 1e12, 1)}
        del w, s, b, x, y

        # group-32 twin (GGUF Q4_0 repacked), M=1: affine form (5/8 B per weight) and scale-only form
        # (bias never read: 9/16 B per weight)
        g32 = {}
        for K, N in ((4096, 4096), (4096, 12288)):
            copies = max(2, min(8, int(600e6 // (N * K * 5 // 8))))
            packs = []
            for _ in range(copies):
                w = torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 8), dtype=torch.int32, device=dev, generator=gen)
                s = torch.empty((N, K // 32), dtype=torch.float32, device=dev).uniform_(0.005, 0.02, generator=gen).bfloat16()
                packs.append((w, s, (-8.0 * s.float()).bfloat16()))
            x = torch.randn((1, K), device=dev, generator=gen).bfloat16()
            y = torch.empty((1, N), dtype=torch.bfloat16, device=dev)

            def call32(i, x=x, y=y, K=K, N=N, so=False):
                w, s, b = packs[i % copies]
                vpipe_amd.qmv_w4g32(w, s, None if so else b, x, K, N, 1, out=y, scale_only=so)
            us_a = kernel_us(call32, 2 * copies)
            us_q = kernel_us(lambda i: call32(i, so=True), 2 * copies)
            g32["%d->%d" % (K, N)] = {
                "affine": {"us": round(us_a, 2), "GBps": round((N * K * 5 // 8 + 2 * K + 2 * N) / (us_a * 1e-6) / 1e9, 1)},
                "q40_scale_only": {"us": round(us_q, 2),
                                   "GBps": round((N * K * 9 // 16 + 2 * K + 2 * N) / (us_q * 1e-6) / 1e9, 1)}}
            del packs
        out["qmv_w4g32_m1"] = g32

        # greedy tail: argmax over the lm_head's 151936 bf16 logits (both launches of the two-stage form)
        lg = torch.randn((1, 151936), device=dev, generator=gen).bfloat16()
        tok = torch.empty((1,), dtype=torch.int32, device=dev)
        out["argmax_v151936"] = {
            "two_stage_us": round(kernel_us(lambda i: vpipe_amd.argmax_bf16(lg, out=tok, two_stage=True), 16), 2),
            "one_workgroup_us": round(kernel_us(lambda i: vpipe_amd.argmax_bf16(lg, out=tok, two_stage=False), 16), 2)}
        # stochastic tail: the one-workgroup sampler (top-k 50, top-p 0.9, 24 bisection steps each) over the same logits
        seen_b = torch.zeros((151936,), dtype=torch.uint8, device=dev)
        ws_b = torch.empty((151936,), dtype=torch.bfloat16, device=dev)
        n_slabs = vpipe_amd.sample_hist_slabs(151936)
        work_b = torch.empty((int(L.vpq_sample_hist_workspace_bytes(n_slabs)) // 4,), dtype=torch.float32, device=dev)
        out["sample_topp_v151936"] = {
            "one_workgroup_us": round(kernel_us(lambda i: vpipe_amd.sample_topp_bf16(lg.view(-1), seen_b, 0.8, 0.9, 1000 + i,
                                                                                      ws=ws_b, out=tok, top_k=50), 8), 1),
            # the same draw over n_slabs workgroups with histogram thresholds: all five launches of a call
            "histogram_slabs": n_slabs,
            "histogram_us": round(kernel_us(lambda i: vpipe_amd.sample_hist_bf16(lg.view(-1), seen_b, 0.8, 0.9, 1000 + i,
                                                                                 ws=ws_b, out=tok, work=work_b, n_slabs=n_slabs,
                                                                                 top_k=50), 8), 1)}

        # MoE decode block, pair-batched gathers (hidden 2048, expert inner 768, 128 experts, top-8,
        # one token): 8 of the 128 gate|up slabs and 8 down slabs per step, a fresh random set of
        # experts each launch over two layers' batches (679 MB, so the slabs come from HBM)
        H, I, E, top_k = 2048, 768, 128, 8
        batches = []
        for _ in range(2):
            gw = torch.randint(-2 ** 31, 2 ** 31 - 1, (E, 2 * I, H // 8), dtype=torch.int32, device=dev, generator=gen)
            gs = torch.empty((E, 2 * I, H // 64), dtype=torch.float32, device=dev).uniform_(0.005, 0.02, generator=gen).bfloat16()
            dw = torch.randint(-2 ** 31, 2 ** 31 - 1, (E, H, I // 8), dtype=torch.int32, device=dev, generator=gen)
            ds = torch.empty((E, H, I // 64), dtype=torch.float32, device=dev).uniform_(0.005, 0.02, generator=gen).bfloat16()
            batches.append((gw, gs, (-8.0 * gs.float()).bfloat16(), dw, ds, (-8.0 * ds.float()).bfloat16()))
        ids = [torch.randperm(E, device=dev, generator=gen)[:top_k].to(torch.int32).contiguous() for _ in range(16)]
        xm = torch.randn((1, H), device=dev, generator=gen).bfloat16()
        actm = torch.empty((top_k, I), dtype=torch.bfloat16, device=dev)
        partm = torch.empty((top_k, H), dtype=torch.bfloat16, device=dev)

        def call_gu(i):
            gw, gs, gb, _, _, _ = batches[i % 2]
            vpipe_amd.gather_qmv_gated_w4g64(gw, gs, gb, xm, H, 2 * I, ids[i % 16], top_k, E, out=actm)

        def call_dn(i):
            _, _, _, dw, ds, db = batches[i % 2]
            vpipe_amd.gather_down_qmv_w4g64(dw, ds, db, actm, I, H, ids[i % 16], E, out=partm)
        us_gu = kernel_us(call_gu, 16)
        us_dn = kernel_us(call_dn, 16)
        b_gu = top_k * (2 * I * H * 9 // 16) + 2 * H + 2 * top_k * I
        b_dn = top_k * (H * I * 9 // 16) + 2 * top_k * (I + H)
        out["moe_gather_decode_top8_of_128"] = {
            "gate|up+swiglu 2048->2x768": {"us": round(us_gu, 2), "GBps": round(b_gu / (us_gu * 1e-6) / 1e9, 1)},
            "down 768->2048": {"us": round(us_dn, 2), "GBps": round(b_dn / (us_dn * 1e-6) / 1e9, 1)}}

        # MoE prefill block of the same model, 2048 tokens (16384 pairs): the pair sort, then the two
        # expert-sorted GEMMs; beside them the pair-batched gathers (one QMV per pair) on the same pairs.
        # TFLOPs count the pairs' flops only, not the padding slots'.
        T = 2048
        eid = torch.randint(0, E, (T * top_k,), dtype=torch.int32, device=dev, generator=gen)
        xt = torch.randn((T, H), device=dev, generator=gen).bfloat16()
        gw, gs, gb, dw, ds, db = batches[0]
        sorted_ = {}

        def call_sort(i):
            sorted_["v"] = vpipe_amd.moe_sort_pairs(eid, top_k, E)
        us_sort = kernel_us(call_sort, 8)
        t2e, srow, sdst, ntiles = sorted_["v"]
        npad = srow.numel()
        gact = torch.empty((npad, I), dtype=torch.bfloat16, device=dev)
        partp = torch.empty((T * top_k, H), dtype=torch.bfloat16, device=dev)
        us_ggu = kernel_us(lambda i: vpipe_amd.qmm_grouped_gated_w4g64(gw, gs, gb, xt, H, 2 * I, t2e, srow, E, out=gact), 8)
        us_gdn = kernel_us(lambda i: vpipe_amd.qmm_grouped_down_w4g64(dw, ds, db, gact, I, H, t2e, sdst, E, out=partp), 8)
        actp = torch.empty((T * top_k, I), dtype=torch.bfloat16, device=dev)
        us_pgu = kernel_us(lambda i: vpipe_amd.gather_qmv_gated_w4g64(gw, gs, gb, xt, H, 2 * I, eid, top_k, E, out=actp), 4)
        us_pdn = kernel_us(lambda i: vpipe_amd.gather_down_qmv_w4g64(dw, ds, db, actp, I, H, eid, E, out=partp), 4)
        f_gu = 2.0 * T * top_k * 2 * I * H
        f_dn = 2.0 * T * top_k * H * I
        out["moe_grouped_prefill_t2048_top8_of_128"] = {
            "blocks_in_use": int(ntiles.cpu()[0]), "slots": int(ntiles.cpu()[0]) * vpipe_amd.grouped_block_rows(),
            "pairs": T * top_k,
            "pair_sort_us": round(us_sort, 2),
            "gate|up+swiglu 2048->2x768": {"us": round(us_ggu, 2), "TFLOPs": round(f_gu / (us_ggu * 1e-6) / 1e12, 1),
                                           "pair_gather_qmv_us": round(us_pgu, 2)},
            "down 768->2048": {"us": round(us_gdn, 2), "TFLOPs": round(f_dn / (us_gdn * 1e-6) / 1e12, 1),
                               "pair_gather_qmv_us": round(us_pdn, 2)}}
        del batches

    # ---- CPU baseline: the oracle's dequant + fp32 matmul on the host cores ------------
    # The reference's CPU path (quantize-module expansion + plain fp32 dot, OpenMP over output rows) restated in
    # oracle/vpq_oracle.c, timed here on this box's host cores.  `cpu_baseline` is the headline workload
    # (config 2); `cpu_baseline_configs` holds configs 1 (the three forms timed separately), 3 (every shape and
    # M, one call each) and 4-5 (a 64-row subsample of M, scaled linearly: extrapolated).
    if not args.no_cpu:
        from oracle import oracle
        host = []
        for j, (_, K, N) in enumerate(DECODE_LAYER):
            w, s, b = layers[0][j]
            host.append((w.cpu().numpy().view(np.uint32), s.view(torch.int16).cpu().numpy().view(np.uint16),
                         b.view(torch.int16).cpu().numpy().view(np.uint16),
                         xs[K].view(torch.int16).cpu().numpy().view(np.uint16),
                         np.empty((N, K), dtype=np.float32), np.empty((1, K), dtype=np.float32)))
        def cpu_pass():
            for j, (_, K, N) in enumerate(DECODE_LAYER):
                w, s, b, x, wdeq, xf = host[j]
                oracle.cpu_dequant_matmul(w, s, b, x, K, N, 1, wdeq=wdeq, xf=xf)
        cpu_pass()
        t0 = time.perf_counter()
        n_pass = 0
        while True:
            cpu_pass()
            n_pass += 1
            el = time.perf_counter() - t0
            if el > 6.0 or n_pass >= 200:
                break
        cpu_model = "unknown"
        try:
            for line in open("/proc/cpuinfo"):
                if line.startswith("model name"):
                    cpu_model = line.split(":", 1)[1].strip()
                    break
        except OSError:
            pass
        out["cpu_baseline"] = {"value": round(layer_bytes * n_pass / el / 1e9, 2), "unit": "GB/s",
                               "cores": oracle.num_threads(), "kind": "port",
                               "sample": "%d passes of the same decode-layer set (one layer's weights), "
                                         "dequant to fp32 [N,K] + fp32 dot, OpenMP over N" % n_pass,
                               "ms_per_step": round(el / n_pass * 1e3, 3),
                               "nproc": os.cpu_count(), "omp_max_threads": oracle.num_threads(), "cpu_model": cpu_model}

        def timed(fn, min_s=0.25, max_calls=50):
            fn()
            t0 = time.perf_counter()
            n = 0
            while True:
                fn()
                n += 1
                el = time.perf_counter() - t0
                if el > min_s or n >= max_calls:
                    return el / n

        def host_pack(N, K, seed):
            rng = np.random.default_rng(seed)
            w = rng.integers(0, 2 ** 32, size=(N, K // 8), dtype=np.uint32)
            sf = rng.uniform(0.005, 0.02, size=(N, K // 64)).astype(np.float32)
            s = torch.from_numpy(sf).bfloat16().view(torch.int16).numpy().view(np.uint16)
            bf = (-8.0 * sf * (1.0 + 0.05 * rng.standard_normal((N, K // 64)))).astype(np.float32)
            b = torch.from_numpy(bf).bfloat16().view(torch.int16).numpy().view(np.uint16)
            return w, s, b

        def host_x(M, K, seed):
            rng = np.random.default_rng(seed)
            return torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).bfloat16().view(torch.int16).numpy().view(np.uint16)

        cfg = {}
        # config 1: one 4096 -> 4096 QMV, the three forms separately
        K, N = 4096, 4096
        w, s, b = host_pack(N, K, 1)
        x = host_x(1, K, 2)
        wdeq, xf = np.empty((N, K), dtype=np.float32), np.empty((1, K), dtype=np.float32)
        t_dq = timed(lambda: oracle.cpu_dequant_f32(w, s, b, K, N, wdeq))
        t_mv = timed(lambda: oracle.cpu_matmul_f32(wdeq, x, K, N, 1, xf=xf))
        t_fu = timed(lambda: oracle.cpu_fused_qmv(w, s, b, x, K, N, 1, xf=xf))
        ab = alg_bytes(K, N, 1)
        cfg["config1_qmv_4096x4096_m1"] = {
            "dequant_to_fp32_us": round(t_dq * 1e6, 1), "fp32_gemv_us": round(t_mv * 1e6, 1),
            "fused_dequant_dot_us": round(t_fu * 1e6, 1),
            "GBps_dequant_plus_gemv": round(ab / (t_dq + t_mv) / 1e9, 2), "GBps_fused": round(ab / t_fu / 1e9, 2)}
        # config 3: every shape and M, one call each (the expansion dominates and does not depend on M)
        c3 = {}
        for K, N in SMALL_BATCH:
            w, s, b = host_pack(N, K, 3 + N)
            wdeq = np.empty((N, K), dtype=np.float32)
            row = {}
            for M in (1, 2, 4, 8, 16):
                x = host_x(M, K, 4 + M)
                xf = np.empty((M, K), dtype=np.float32)
                big = N * K > 200e6
                t = timed(lambda: oracle.cpu_dequant_matmul(w, s, b, x, K, N, M, wdeq=wdeq, xf=xf),
                          min_s=0.0 if big else 0.1, max_calls=1 if big else 5)
                row["M=%d" % M] = {"us": round(t * 1e6, 1), "GBps": round(alg_bytes(K, N, M) / t / 1e9, 2)}
            c3["%d->%d" % (K, N)] = row
            del w, s, b, wdeq
        cfg["config3_small_batch"] = c3
        # configs 4-5: 64 rows of x, scaled to M (extrapolated)
        for name, shapes, M in (("config4_prefill_m2048", [(K, N) for _, K, N in PREFILL], 2048),
                                ("config5_dit_m16320", DIT, 16320)):
            res = {}
            for K, N in shapes:
                w, s, b = host_pack(N, K, 5 + N)
                x = host_x(64, K, 6)
                wdeq, xf = np.empty((N, K), dtype=np.float32), np.empty((64, K), dtype=np.float32)
                t_dq = timed(lambda: oracle.cpu_dequant_f32(w, s, b, K, N, wdeq), min_s=0.0, max_calls=1)
                t_mm = timed(lambda: oracle.cpu_matmul_f32(wdeq, x, K, N, 64, xf=xf), min_s=0.0, max_calls=1)
                t_full = t_dq + t_mm * (M / 64.0)
                res["%d->%d" % (K, N)] = {"extrapolated_ms": round(t_full * 1e3, 1),
                                          "extrapolated_TFLOPs": round(2.0 * M * N * K / t_full / 1e12, 4),
                                          "measured": "expansion %.1f ms + 64 rows of x %.1f ms, scaled by M/64" % (t_dq * 1e3, t_mm * 1e3)}
                del w, s, b, wdeq
            cfg[name] = res
        out["cpu_baseline_configs"] = cfg

    if args.copy_calibration:
        copy_calibration()
        out["copy_calibration"] = {"bytes_read": 256 << 20, "bytes_written": 256 << 20, "copies": 3}

    print(json.dumps(out))


if __name__ == "__main__":
    main()
