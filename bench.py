#!/usr/bin/env python3
"""Benchmark of the int4 decode GEMV (BASELINE.json config 2) on one MI355X.

Workload: FullyConnected, 1 token, K=4096, N=14336, int4 per-channel weights in the packed
I4O4 layout, fp16 activations / scales / output, fp32 accumulation.  One step = one launch
of the op over one activation batch.  The packed weights (29.4 MB) would sit in the 256 MB
Infinity Cache if one buffer were reused, so the steps rotate over a ring of weight copies
larger than that cache, the way the reference's own perf harness does behind
kUseMultipleWeights (cl/testing/perf_util.cc:2247-2253).

Prints ONE JSON line.  `value` is algorithmic bytes * steps / wall time of the timed region
(a HIP-graph replay of the steps, inputs resident in HBM); `roofline.achieved` divides the
same algorithmic bytes by the average launch duration measured with HIP events on the
launch stream over that region.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "ml-drift_amd", "python"))
sys.path.insert(0, ROOT)

import numpy as np

HBM_PEAK_GBS = 8000.0


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=4000)
    p.add_argument("--warmup", type=int, default=400)
    p.add_argument("--ring", type=int, default=16, help="distinct weight copies (16 x 29.4 MB > 256 MB)")
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--no-graph", action="store_true", help="time an eager launch loop instead of a graph replay")
    p.add_argument("--cpu-seconds", type=float, default=12.0)
    p.add_argument("--traffic-probe", action="store_true",
                   help="for `rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE`: a 256 MiB device copy (the known-size "
                        "reference dispatch) followed by 64 launches over the weight ring, then exit")
    return p.parse_args()


def cpu_baseline(case, seconds):
    """The CPU restatement of the reference's generated kernel (oracle/, OpenMP over output
    slices) on the same case; repeated whole-GEMV passes for about `seconds`."""
    from oracle import oracle as o
    n, k, m = case["n"], case["k"], case["m"]
    ns = (n + 3) // 4
    packed = o.int8_as_uint4(case["w"], o.LAYOUT_I4O4, ns)
    act = o.f32_to_f16_bits(o.to_slices(case["act"]))
    sc = np.zeros(ns * 4, np.float32)
    sc[:n] = case["scale"][:, 0]
    sc = o.f32_to_f16_bits(sc)
    cores = os.cpu_count() or 1
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        pass
    threads = int(os.environ.get("OMP_NUM_THREADS", cores))
    reps, t0 = 0, time.perf_counter()
    o.fc_kernel(act, packed, m, k, n, o.PREC_F32F16, 4, o.SCALE_LINEAR, sc, threads=threads)  # warm
    t0 = time.perf_counter()
    while True:
        o.fc_kernel(act, packed, m, k, n, o.PREC_F32F16, 4, o.SCALE_LINEAR, sc, threads=threads)
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= seconds or reps >= 1000:
            break
    return reps, dt, threads


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU part (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import torch
    import mldhip as M
    import workloads as W

    if not torch.cuda.is_available():
        print("no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    cfg = W.CONFIGS["c2"]
    case = W.make_fc_case(**cfg)
    m, k, n = case["m"], case["k"], case["n"]

    # ring of ops: copy 0 holds the seeded case, the others random packed bytes (every byte
    # pattern is a valid pair of int4 codes)
    devs = [W.FcDevice(case)]
    gen = torch.Generator(device="cuda").manual_seed(1)
    ops = [devs[0].op]
    weights = [devs[0].weights]
    for r in range(1, args.ring):
        wt = torch.randint(0, 256, devs[0].weights.shape, dtype=torch.uint8, device="cuda", generator=gen)
        op = M.fc_create(M.PRECISION_F32_F16, M.FLOAT16, M.FLOAT16, n, k, devs[0].desc, scale_shape=(n, 1),
                         max_tokens=m)
        op.bind([devs[0].act, wt, devs[0].scale], [devs[0].out])
        op.set_shape(1, 1, m)
        ops.append(op)
        weights.append(wt)
    algo_bytes, flops = ops[0].cost()

    stream = torch.cuda.Stream()  # default priority
    s = stream.cuda_stream
    with torch.cuda.stream(stream):
        # correctness spot check of copy 0 (fp16 tolerance of the path: 2e-2 of the output RMS)
        ops[0].launch(s)
        stream.synchronize()
        got = devs[0].result()
        ref = case["act"].astype(np.float64) @ W.dequantized_weights(case).T
        rel = np.abs(got - ref).max() / np.sqrt(np.mean(ref ** 2))
        if not rel <= 2e-2:
            print("result check failed: max|err|/rms = %g" % rel, file=sys.stderr)
            sys.exit(1)
        kernel = ops[0].kernel_name

        if args.traffic_probe:
            src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").fill_(7)
            dst = torch.empty_like(src)
            for _ in range(3):
                dst.copy_(src)
            for i in range(64):
                ops[i % args.ring].launch(s)
            stream.synchronize()
            print(json.dumps({"traffic_probe": "done", "copy_bytes": 256 << 20, "kernel": kernel}))
            return

        for i in range(max(args.warmup, args.ring)):  # every op allocates its workspace on first use
            ops[i % args.ring].launch(s)
        stream.synchronize()

        use_graph = not args.no_graph
        graph = None
        if use_graph:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                cs = torch.cuda.current_stream().cuda_stream
                for i in range(args.steps):
                    ops[i % args.ring].launch(cs)
            graph.replay()  # untimed: first replay uploads the graph
            stream.synchronize()

        ev0 = torch.cuda.Event(enable_timing=True)
        ev1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev0.record(stream)
        if use_graph:
            graph.replay()
        else:
            for i in range(args.steps):
                ops[i % args.ring].launch(s)
        ev1.record(stream)
        stream.synchronize()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        ev_ms = ev0.elapsed_time(ev1)

    ms_per_step = wall * 1e3 / args.steps
    value = algo_bytes * args.steps / wall / 1e9
    launch_us = ev_ms * 1e3 / args.steps
    achieved = algo_bytes / (launch_us * 1e-6) / 1e9

    # HBM bytes per launch from the committed rocprofv3 --pmc summary (FETCH_SIZE + WRITE_SIZE,
    # scaled by a known-size copy); null when no summary is there
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "fc_w4_stream_c2.md")
    if os.path.exists(tpath):
        import re
        mt = re.search(r"^hbm_bytes_per_launch = (\d+)", open(tpath).read(), re.M)
        traffic = int(mt.group(1)) if mt else None

    out = {
        "metric": "int4_decode_gemv_hbm_bandwidth",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u4 weights x f16 activations, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "c2: FullyConnected decode GEMV M=1 K=4096 N=14336 int4 per-channel, fp16 act/out",
                   "weight_ring": args.ring, "timed_region": "hipGraph replay" if use_graph else "eager launch loop",
                   "algorithmic_bytes_per_step": algo_bytes, "flops_per_step": flops,
                   "pct_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2)},
        "roofline": {"bound": "hbm", "kernel": kernel, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "avg_launch_us": round(launch_us, 3)},
    }
    if not args.no_cpu_baseline:
        reps, dt, threads = cpu_baseline(case, args.cpu_seconds)
        out["cpu_baseline"] = {"value": round(algo_bytes * reps / dt / 1e9, 3), "unit": "GB/s", "cores": threads,
                               "kind": "port",
                               "sample": "%d full passes of the same c2 GEMV (oracle restatement of the reference's "
                                         "generated kernel, OpenMP over output slices) in %.1f s" % (reps, dt)}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
