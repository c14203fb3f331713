#!/usr/bin/env python3
"""Benchmark of the w4g64 quantized-linear path on one MI355X.

Headline (`value`): batch-1 QMV over a decode layer's seven projections
(q 4096->4096, k and v 4096->1024, o 4096->4096, gate and up 4096->12288,
down 12288->4096), in GB/s of ALGORITHMIC bytes (packed codes + scales + biases
+ x + y, each once).  A step is one pass over the seven projections of one
layer; consecutive steps use different layers' weights (8 layers, 868 MB in
rotation) so that no pass finds its weights in the 256 MB last-level cache.
The timed region is one HIP graph of `steps` passes, replayed between two
events on the launch stream with inputs already resident in HBM.

Also reported on the same JSON line: the per-kernel roofline fraction (kernel
durations from hipExtLaunchKernel events, no launch gaps), per-shape numbers,
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
# HBM-side bytes per QMV launch of the default workload (average over a layer's seven launches),
# from two rocprofv3 --pmc passes (FETCH_SIZE, WRITE_SIZE per dispatch).  FETCH_SIZE reads half
# the bytes of a 256 MiB device-to-device copy on this part, so it is scaled by 2.0; WRITE_SIZE
# by 1.0.  109.68 MB fetched per layer, writes below the counter's resolution.
TRAFFIC_PER_LAUNCH = 15.67e6

DECODE_LAYER = [("q", 4096, 4096), ("k", 4096, 1024), ("v", 4096, 1024), ("o", 4096, 4096),
                ("gate", 4096, 12288), ("up", 4096, 12288), ("down", 12288, 4096)]
PREFILL = [("gate_up", 4096, 12288), ("down", 12288, 4096), ("attn", 4096, 4096)]


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
    ap.add_argument("--no-graph", action="store_true", help="time eager launches instead of a HIP graph")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three 256 MiB device-to-device copies (a kernel of known traffic, to scale "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--concurrent", action="store_true",
                    help="capture q|k|v and gate|up as concurrent graph branches (measured slower than one "
                         "stream on MI355X: 55.7 vs 42.5 us per layer)")
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

    def layer_pass(li):
        for j in range(len(DECODE_LAYER)):
            project(li, j)

    side = [torch.cuda.Stream(device=dev), torch.cuda.Stream(device=dev)]

    def layer_pass_concurrent(li):
        """The layer's dataflow: q|k|v are independent of each other, so are gate|up (the reference
        encodes them in a concurrent scope, apple-silicon/metal-compute/compute-encoder.h,
        ConcurrentScope); o follows the attention, down follows gate|up."""
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

    for i in range(args.warmup):
        layer_pass(i % args.layers)
    torch.cuda.synchronize()

    # ---- timed region ---------------------------------------------------------------
    concurrent = args.concurrent and not args.no_graph
    launch = "hipgraph, q|k|v and gate|up as concurrent branches" if concurrent else "hipgraph, one stream"
    graph = None
    if not args.no_graph:
        try:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for i in range(args.steps):
                    (layer_pass_concurrent if concurrent else layer_pass)(i % args.layers)
            graph.replay()                      # untimed: first replay uploads the graph
            torch.cuda.synchronize()
        except Exception as e:                  # capture unsupported: fall back to eager, say so
            print("bench.py: graph capture failed (%s); timing eager launches" % e, file=sys.stderr)
            graph = None
    if graph is None:
        launch = "eager"
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    if graph is not None:
        graph.replay()
    else:
        for i in range(args.steps):
            layer_pass(i % args.layers)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1)
    ms_per_step = ms / args.steps
    value = layer_bytes / (ms_per_step * 1e-3) / 1e9

    # ---- per-kernel durations (hipExtLaunchKernel events: kernel start -> end) --------
    passes = max(4 * args.layers, 32)
    n_launch = passes * len(DECODE_LAYER)
    st = L.vpq_profile_enable(n_launch)
    if st != 0:
        raise vpipe_amd.VpqError(st, "vpq_profile_enable")
    for i in range(passes):
        layer_pass(i % args.layers)
    buf = (ctypes.c_float * n_launch)()
    got = L.vpq_profile_read(buf, n_launch)
    L.vpq_profile_enable(0)
    assert got == n_launch, got
    dur = np.array(buf[:], dtype=np.float64).reshape(passes, len(DECODE_LAYER)) * 1e3   # us
    per_shape = {}
    for j, (name, K, N) in enumerate(DECODE_LAYER):
        us = float(dur[:, j].mean())
        per_shape[name] = {"K": K, "N": N, "us": round(us, 3),
                           "GBps": round(alg_bytes(K, N, 1) / (us * 1e-6) / 1e9, 1)}
    kernel_us_per_layer = float(dur.sum(axis=1).mean())
    avg_launch_us = kernel_us_per_layer / len(DECODE_LAYER)
    achieved = layer_bytes / (kernel_us_per_layer * 1e-6) / 1e9
    default_workload = args.variant == 0
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": TRAFFIC_PER_LAUNCH if default_workload else None,
                "kernel": "qmv_mfma_kernel (all seven launches of a layer)", "avg_launch_us": round(avg_launch_us, 3),
                "bytes_per_launch": layer_bytes / len(DECODE_LAYER),
                "launches_timed": n_launch}

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
        "kernel_us_per_layer": round(kernel_us_per_layer, 3),
        "per_shape": per_shape,
        "roofline": roofline,
    }

    # ---- QMM at M = 2048 ---------------------------------------------------------------
    if not args.no_qmm:
        M = 2048
        qmm = {}
        tot_flops, tot_us = 0.0, 0.0
        for name, K, N in PREFILL:
            w, s, b = make_weight(torch, N, K, dev, gen)
            x = torch.randn((M, K), device=dev, generator=gen).bfloat16()
            y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
            for _ in range(3):
                vpipe_amd.qmm_w4g64(w, s, b, x, K, N, M, out=y)
            torch.cuda.synchronize()
            iters = 10
            L.vpq_profile_enable(iters)
            for _ in range(iters):
                vpipe_amd.qmm_w4g64(w, s, b, x, K, N, M, out=y)
            kb = (ctypes.c_float * iters)()
            n = L.vpq_profile_read(kb, iters)
            L.vpq_profile_enable(0)
            us = float(np.mean(kb[:n])) * 1e3
            flops = 2.0 * M * N * K
            qmm[name] = {"K": K, "N": N, "M": M, "us": round(us, 2), "TFLOPs": round(flops / (us * 1e-6) / 1e12, 1)}
            tot_flops += flops
            tot_us += us
            del w, s, b, x, y
        ach = tot_flops / (tot_us * 1e-6) / 1e12
        out["qmm_m2048"] = qmm
        out["roofline_qmm"] = {"bound": "mfma", "achieved": round(ach, 1), "peak": MFMA_BF16_PEAK_TF,
                               "unit": "TFLOP/s", "frac": round(ach / MFMA_BF16_PEAK_TF, 4), "traffic": None,
                               "kernel": "qmm_tile_kernel<false>"}

    # ---- CPU baseline: the oracle's dequant + fp32 matmul on the host cores ------------
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
            if el > 10.0 or n_pass >= 200:
                break
        out["cpu_baseline"] = {"value": round(layer_bytes * n_pass / el / 1e9, 2), "unit": "GB/s",
                               "cores": oracle.num_threads(), "kind": "port",
                               "sample": "%d passes of the same decode-layer set (one layer's weights), "
                                         "dequant to fp32 [N,K] + fp32 dot, OpenMP over N" % n_pass,
                               "ms_per_step": round(el / n_pass * 1e3, 3)}

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(generator=gen)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        out["copy_calibration"] = {"bytes_read": 256 << 20, "bytes_written": 256 << 20, "copies": 3}

    print(json.dumps(out))


if __name__ == "__main__":
    main()
