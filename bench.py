#!/usr/bin/env python3
"""Benchmark of the int4 decode GEMV (benchmark configuration 2) on one MI355X.

Workload: FullyConnected, 1 token, K=4096, N=14336, int4 per-channel weights in the packed
I4O4 layout, fp16 activations / scales / output, fp32 accumulation.  One step = one launch
of the op over one activation batch.  The packed weights (29.4 MB) would sit in the 256 MB
Infinity Cache if one buffer were reused, so the steps rotate over a ring of weight copies
larger than that cache, the way the reference's own perf harness does behind
kUseMultipleWeights (cl/testing/perf_util.cc:2247-2253).

Prints ONE JSON line.  The timed region is one replay of a HIP graph that holds R x steps launches
(inputs resident in HBM; R such that the region lasts at least 25 ms, so that the replay's own host
cost does not weigh on a 20-step run); it is timed 5 times and the median region is reported.  `value` is algorithmic bytes / (wall time of
the region / launches in it); `roofline.achieved` divides the same bytes by the average launch
duration measured with HIP events on the launch stream over the same region.
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
    p.add_argument("--steps", type=int, default=None, help="default 4000 (c2, c1, f2), 2000 (moe), 200 (c3, c4), 20 (c5-*)")
    p.add_argument("--warmup", type=int, default=None, help="default steps / 10")
    p.add_argument("--workload", default="c2", choices=["c2", "c1", "c3", "c4", "c5-decode", "c5-prefill", "f2", "moe", "gemv"],
                   help="c2 (default) is the headline line; the others time the remaining configurations "
                        "the same way (one JSON line each, no CPU baseline)")
    p.add_argument("--tokens", type=int, default=128,
                   help="c5-prefill: tokens per step (the configuration is quoted at 128; larger chunks show the "
                        "kernels away from the launch-bound regime)")
    p.add_argument("--shape", default="", help="c3: another GEMM shape as M,K,N,GROUP (tokens, input channels, output "
                   "channels, input channels per scale group), e.g. 8192,4096,14336,32 for a large prefill chunk; "
                   "gemv: the shape of the few-token FullyConnected to time (GROUP = K: per-channel scales)")
    p.add_argument("--bits", type=int, default=4, choices=[4, 8], help="gemv: weight bits")
    p.add_argument("--ring", type=int, default=16, help="distinct weight copies (16 x 29.4 MB > 256 MB)")
    p.add_argument("--layout", default="default", choices=["default", "library", "reference", "decode"],
                   help="c2: int4 weights in the layout mldhip_fc_int4_weights_desc asks for (output groups of 16 "
                        "slices; the default) or in the reference's own FullyConnected layout (one output group). "
                        "c5-decode: the weights as mldhip_fc_int4_weights_desc_decode asks for them (the default) or, "
                        "with 'library', in the layout mldhip_fc_int4_weights_desc asks for; c5-prefill with 'decode': "
                        "the prefill step over the decode ops' layout (one copy of the weights for both graphs)")
    p.add_argument("--tune", default="", help="tuning knobs for the run, e.g. gemv_ksplit=1,gemm_dual=0 (mldhip_set_tuning)")
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--no-graph", action="store_true", help="time an eager launch loop instead of a graph replay")
    p.add_argument("--cpu-seconds", type=float, default=12.0)
    p.add_argument("--traffic-probe", action="store_true",
                   help="for `rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE`: a 256 MiB device copy (the known-size "
                        "reference dispatch) followed by 64 launches over the weight ring, then exit")
    a = p.parse_args()
    if a.steps is None:
        a.steps = {"c2": 4000, "c1": 4000, "f2": 4000, "moe": 2000, "gemv": 2000, "c3": 200, "c4": 200}.get(a.workload, 20)
    if a.warmup is None:
        a.warmup = max(1, a.steps // 10)
    return a


# The timed region is at least this long, whatever --steps says.  (Long enough for the host side
# too: on this stack a stream synchronisation that waits between about 5 and 8 ms returns after
# 8 ms, which would inflate a 5 ms region by half; at 25 ms wall clock and HIP events agree to 0.3 %.)
MIN_REGION_MS = 25.0
REGIONS = 5          # the region is timed this many times; the median one is reported


def time_graph(torch, stream, launch_step, steps, warmup, use_graph=True, ring=1):
    """`warmup` eager steps, then the timed region: ONE replay of a HIP graph that holds the steps.
    A replay of a short graph is dominated by its own host and synchronisation cost (tens of
    microseconds, and back-to-back replays of one graph do not overlap: each waits for the one
    before and leaves the GPU idle while it is submitted), so the graph holds R * steps launches,
    R chosen from an untimed replay of a `steps`-launch graph such that the region lasts at least
    MIN_REGION_MS (rounded up to whole turns of the weight ring, so that every weight copy comes
    back only after all the others).  The region is timed REGIONS times and the median one is
    reported.  Returns (wall seconds per step, event microseconds per step, {R, launches}): both
    are region / launches in it, the wall clock bracketed by synchronisations, the HIP events
    recorded on `stream` around the same replay."""
    s = stream.cuda_stream

    def build(launches):
        if not use_graph:
            def run():
                for i in range(launches):
                    launch_step(s, i)
            return run
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            cs = torch.cuda.current_stream().cuda_stream
            for i in range(launches):
                launch_step(cs, i)
        return graph.replay

    def timed(run):
        ev0 = torch.cuda.Event(enable_timing=True)
        ev1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev0.record(stream)
        run()
        ev1.record(stream)
        stream.synchronize()
        torch.cuda.synchronize()
        return time.perf_counter() - t0, ev0.elapsed_time(ev1)

    with torch.cuda.stream(stream):
        for i in range(warmup):
            launch_step(s, i)
        stream.synchronize()
        launches = -(-steps // ring) * ring
        run = build(launches)
        run()  # untimed: the first replay uploads the graph
        stream.synchronize()
        _, one_ms = timed(run)
        reps = max(1, min(5000, int(np.ceil(MIN_REGION_MS / max(one_ms, 1e-3)))))
        if reps > 1:
            launches = reps * launches
            run = build(launches)
            run()
            stream.synchronize()
        regions = [timed(run) for _ in range(REGIONS)]
    # the median region: a host hiccup of a millisecond (seen on shared boxes) drops out
    wall, event_ms = sorted(regions)[REGIONS // 2]
    fastest_us = min(r[1] for r in regions) * 1e3 / launches
    return wall / launches, event_ms * 1e3 / launches, {"steps_multiple": reps, "launches_in_region": launches,
                                                         "timed_regions": REGIONS, "reported_region": "median by wall time",
                                                         "fastest_region_us_per_step": round(fastest_us, 3)}


def run_other(args, torch, M, W):
    """The configurations other than c2: same timing method, metric of their own roofline."""
    stream = torch.cuda.Stream()
    base = {"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "data": "synthetic"}
    if args.workload in ("c1", "f2"):
        # decode GEMVs over a ring of weight copies larger than the 256 MB cache
        if args.workload == "c1":
            case = W.make_fc_case(**W.CONFIGS["c1"])
            # the weights as mldhip_fc_int8_weights_desc_decode asks for them (--layout reference: the
            # reference's one output group)
            dev0 = W.FcDevice(case, decode_layout=args.layout not in ("reference", "library"))
            m, k, n = case["m"], case["k"], case["n"]
            ring = max(args.ring, 80)  # 80 x 4.2 MB
            gen = torch.Generator(device="cuda").manual_seed(1)
            ops, keep = [dev0.op], [dev0]
            for r in range(1, ring):
                wt = torch.randint(0, 256, dev0.weights.shape, dtype=torch.uint8, device="cuda", generator=gen)
                op = M.fc_create(M.PRECISION_F32, M.FLOAT32, M.FLOAT32, n, k, dev0.desc, scale_shape=(n, 1), max_tokens=m)
                op.bind([dev0.act, wt, dev0.scale], [dev0.out])
                op.set_shape(1, 1, m)
                ops.append(op)
                keep.append(wt)
            nbytes = n * k + k * 4 + n * 4 + n * 4  # W + act + scale + out (fp32 tensors)
            label = ("c1: FullyConnected decode GEMV M=1 K=2048 N=2048 int8 per-channel, fp32 act/out, "
                     "kOSpatialIOGroupI4O4 output_group_size %d" % dev0.desc.output_group_size)
            metric, dtype = "int8_decode_gemv_hbm_bandwidth", "u8 weights x f32 activations, f32 accumulate"
        else:
            m, k, n = 1, 4096, 14336
            rng = np.random.default_rng(0)
            w = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
            src = rng.integers(-128, 128, size=(m, k), dtype=np.int8)
            desc = M.fc_int4_weights_desc(n, k, reference=args.layout == "reference")
            packed = torch.from_numpy(M.rearrange_int8_as_uint4(w, desc))
            act = torch.from_numpy(W.to_slices(src)).cuda()
            out_t = torch.zeros(((n + 3) // 4, m, 4), dtype=torch.int32, device="cuda")
            ring = args.ring
            ops, keep = [], []
            for r in range(ring):
                wt = packed.cuda() if r == 0 else torch.randint(0, 256, packed.shape, dtype=torch.uint8, device="cuda")
                op = M.fc_create(M.PRECISION_F32, M.INT8, M.INT32, n, k, desc, max_tokens=m)
                op.bind([act, wt], [out_t])
                op.set_shape(1, 1, m)
                ops.append(op)
                keep.append(wt)
            nbytes = n * k // 2 + k + n * 4  # W + int8 act + int32 out
            label = ("f2: int8-math FullyConnected decode GEMV M=1 K=4096 N=14336, int8 act x uint4 weights -> int32, "
                     "kOSpatialIOGroupI4O4 output_group_size %d" % desc.output_group_size)
            metric, dtype = "int8_math_decode_gemv_hbm_bandwidth", "i8 x u4, i32 accumulate (v_dot4)"
        wall, us, reg = time_graph(torch, stream, lambda s, i: ops[i % len(ops)].launch(s), args.steps, args.warmup,
                                   ring=len(ops))
        out = dict(base, metric=metric, value=round(nbytes / wall / 1e9, 1), unit="GB/s",
                   ms_per_step=round(wall * 1e3, 6), dtype=dtype,
                   config=dict({"workload": label, "weight_ring": len(ops), "algorithmic_bytes_per_step": nbytes}, **reg),
                   roofline={"bound": "hbm", "kernel": ops[0].kernel_name, "achieved": round(nbytes / us / 1e3, 1),
                             "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                             "traffic": None, "avg_launch_us": round(us, 3)})
    elif args.workload == "gemv":
        # a FullyConnected of 1..16 tokens at a shape of the caller's choice (fp16 tensors, symmetric weights), over a
        # ring of weight copies larger than the 256 MB cache: the few-token figures quoted beside the configurations
        if not args.shape:
            print("--workload gemv needs --shape M,K,N,GROUP", file=sys.stderr)
            sys.exit(2)
        sm, sk, sn, sg = [int(v) for v in args.shape.split(",")]
        groups = 1 if sg >= sk else sk // sg
        case = W.make_fc_case(seed=0, m=sm, k=sk, n=sn, weight_bits=args.bits, tensor_dtype=np.float16, groups=groups)
        dev0 = W.FcDevice(case, reference_layout=args.layout == "reference", decode_layout=args.layout == "decode")
        wbytes = dev0.weights.numel()
        ring = max(2, min(100, -(-(300 << 20) // wbytes)))
        gen = torch.Generator(device="cuda").manual_seed(1)
        ops, keep = [dev0.op], [dev0]
        for r in range(1, ring):
            wt = torch.randint(0, 256, dev0.weights.shape, dtype=torch.uint8, device="cuda", generator=gen)
            op = M.fc_create(M.PRECISION_F32_F16, M.FLOAT16, M.FLOAT16, sn, sk, dev0.desc, scale_shape=(sn, groups), max_tokens=sm)
            op.bind([dev0.act, wt, dev0.scale], [dev0.out])
            op.set_shape(1, 1, sm)
            ops.append(op)
            keep.append(wt)
        nbytes, _ = ops[0].cost()
        wall, us, reg = time_graph(torch, stream, lambda s, i: ops[i % len(ops)].launch(s), args.steps, args.warmup,
                                   ring=len(ops))
        out = dict(base, metric="decode_gemv_hbm_bandwidth", value=round(nbytes / wall / 1e9, 1), unit="GB/s",
                   ms_per_step=round(wall * 1e3, 6), dtype="u%d weights x f16 activations, f32 accumulate" % args.bits,
                   config=dict({"workload": "gemv: FullyConnected M=%d K=%d N=%d int%d, %s, fp16 act/out" % (
                                    sm, sk, sn, args.bits, "per-channel" if groups == 1 else "group-%d" % sg),
                                "weights_layout": "kOSpatialIOGroupI4O4, output_group_size %d" % dev0.desc.output_group_size,
                                "weight_ring": len(ops), "algorithmic_bytes_per_step": nbytes}, **reg),
                   roofline={"bound": "hbm", "kernel": ops[0].kernel_name, "achieved": round(nbytes / us / 1e3, 1),
                             "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                             "traffic": None, "avg_launch_us": round(us, 3)})
    elif args.workload == "moe":
        # FullyConnected with batched weights selected by runtime ids: one token, 2 of 8 expert
        # matrices of the c2 shape per step.  Successive steps take other pairs of experts and the
        # weights exist twice, so a matrix comes back after 470 MB of other weights.
        m, k, n, experts, top = 1, 4096, 14336, 8, 2
        ns = (n + 3) // 4
        # the matrices in the layout mldhip_fc_int4_weights_desc asks for (--layout reference: one output
        # group, one matrix after the other, as the reference's kernel reads them)
        desc = M.fc_int4_weights_desc(n, k, reference=args.layout == "reference")
        rng = np.random.default_rng(0)
        act = torch.from_numpy(W.to_slices(rng.standard_normal((m, k)).astype(np.float16))).cuda()
        scale = torch.from_numpy(M.scale_to_tensor_batched(
            (np.abs(rng.normal(0.0, 0.02, size=(n, experts, 1))) / 7.0).astype(np.float32), M.FLOAT16).view(np.float16)).cuda()
        out_t = torch.zeros((ns, top * m, 4), dtype=torch.float16, device="cuda")
        ops, keep = [], []
        for copy in range(2):
            wt = torch.randint(0, 256, (experts * (k // 4) * ns * 8,), dtype=torch.uint8, device="cuda")
            for pair in range(experts // top):
                ids = torch.tensor([pair * top + j for j in range(top)], dtype=torch.int32, device="cuda")
                op = M.fc_create(M.PRECISION_F32_F16, M.FLOAT16, M.FLOAT16, n, k, desc, scale_shape=(n, 1),
                                 max_tokens=top * m, weights_batch=experts, shared_src=True)
                op.bind([act, ids, wt, scale], [out_t])
                op.set_shape(1, top, m)
                ops.append(op)
                keep += [ids, wt]
        nbytes = top * (n * k // 2 + n * 2 + n * 2 * m) + k * 2 * m + top * 4  # W + scale + out per row, act, ids
        wall, us, reg = time_graph(torch, stream, lambda s, i: ops[i % len(ops)].launch(s), args.steps, args.warmup,
                                   ring=len(ops))
        out = dict(base, metric="int4_moe_decode_gemv_hbm_bandwidth", value=round(nbytes / wall / 1e9, 1),
                   unit="GB/s", ms_per_step=round(wall * 1e3, 6),
                   dtype="u4 weights x f16 activations, f32 accumulate",
                   config=dict({"workload": "moe: FullyConnected with batched weights by runtime ids, 1 token, 2 of 8 "
                                            "matrices K=4096 N=14336 int4 per-channel, fp16 act/out",
                                "weights_layout": "kOSpatialIOGroupI4O4, output_group_size %d" % desc.output_group_size,
                                "weight_ring": len(ops), "algorithmic_bytes_per_step": nbytes}, **reg),
                   roofline={"bound": "hbm", "kernel": ops[0].kernel_name, "achieved": round(nbytes / us / 1e3, 1),
                             "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                             "traffic": None, "avg_launch_us": round(us, 3)})
    elif args.workload == "c3":
        cfg = dict(W.CONFIGS["c3"])
        label = "c3: FullyConnected prefill GEMM M=512 K=4096 N=4096 int4 group-32, fp16 act/out"
        if args.shape:
            sm, sk, sn, sg = [int(v) for v in args.shape.split(",")]
            cfg.update(m=sm, k=sk, n=sn, groups=sk // sg)
            label = "c3 at another shape: FullyConnected prefill GEMM M=%d K=%d N=%d int4 group-%d, fp16 act/out" % (sm, sk, sn, sg)
        case = W.make_fc_case(**cfg)
        dev = W.FcDevice(case)
        wall, us, reg = time_graph(torch, stream, lambda s, i: dev.op.launch(s), args.steps, args.warmup)
        flops = 2.0 * case["m"] * case["k"] * case["n"]
        out = dict(base, metric="int4_prefill_gemm_throughput", value=round(flops / wall / 1e12, 1),
                   unit="TFLOP/s", ms_per_step=round(wall * 1e3, 6),
                   dtype="u4 weights x f16 activations, f32 accumulate (fp16 MFMA)",
                   config=dict({"workload": label, "flops_per_step": flops}, **reg),
                   roofline={"bound": "mfma", "kernel": dev.op.kernel_name, "achieved": round(flops / us / 1e6, 1),
                             "peak": 2500.0, "unit": "TFLOP/s", "frac": round(flops / us / 1e6 / 2500.0, 4),
                             "traffic": None, "avg_launch_us": round(us, 3)})
    elif args.workload == "c4":
        cfg = W.CONFIGS["c4"]
        m, k, n = cfg["m"], cfg["k"], cfg["n"]
        rng = np.random.default_rng(cfg["seed"])
        x = rng.standard_normal((m, k)).astype(np.float16)
        w = rng.integers(-127, 128, size=(n, k), dtype=np.int8)
        src = torch.from_numpy(W.to_slices(x)).cuda()
        k16, ns = (k + 15) // 16, (n + 3) // 4
        codes = torch.zeros((k16, m, 16), dtype=torch.int8, device="cuda")
        params = torch.zeros((m, 4), dtype=torch.float32, device="cuda")
        q = M.quantization_create(M.FLOAT16, M.PACKED_INT8C16, k, calculate_sum=False, symmetric=True, max_tokens=m)
        q.bind([src], [codes, params])
        q.set_shape(1, 1, m)
        wd = M.conv_int8_weights_desc(n, k)
        wt = torch.from_numpy(M.rearrange_int8(w, wd)).cuda()
        wsum = torch.from_numpy(np.pad(w.astype(np.int32).sum(axis=1), (0, ns * 4 - n)).astype(np.int32)).cuda()
        wscale = torch.full((ns * 4,), 1e-4, dtype=torch.float32, device="cuda")
        out_t = torch.zeros((ns, m, 4), dtype=torch.float16, device="cuda")
        conv = M.conv_int8_create(M.FLOAT16, n, k, wd, max_tokens=m)
        conv.bind([codes, wt, params, wsum, wscale], [out_t])
        conv.set_shape(1, 1, m)

        def step(s, i):
            q.launch(s)
            conv.launch(s)
        wall, _, reg = time_graph(torch, stream, step, args.steps, args.warmup)
        _, us, _ = time_graph(torch, stream, lambda s, i: conv.launch(s), args.steps, args.warmup)
        _, q_us, _ = time_graph(torch, stream, lambda s, i: q.launch(s), args.steps, args.warmup)
        # the same step with the reference's default, asymmetric quantization (the rescale then adds
        # w_scale * offset * sum_i(w) per token and channel)
        codes_a, params_a = torch.zeros_like(codes), torch.zeros_like(params)
        out_a = torch.zeros_like(out_t)
        qa = M.quantization_create(M.FLOAT16, M.PACKED_INT8C16, k, calculate_sum=False, symmetric=False, max_tokens=m)
        qa.bind([src], [codes_a, params_a])
        qa.set_shape(1, 1, m)
        conv_a = M.conv_int8_create(M.FLOAT16, n, k, wd, max_tokens=m)
        conv_a.bind([codes_a, wt, params_a, wsum, wscale], [out_a])
        conv_a.set_shape(1, 1, m)

        def step_a(s, i):
            qa.launch(s)
            conv_a.launch(s)
        wall_a, _, _ = time_graph(torch, stream, step_a, args.steps, args.warmup)
        # codes that round-to-nearest-even (the wording of the configuration) would change: the library
        # follows the reference's floor(x * scale + 128.5)
        codes_e, params_e = torch.zeros_like(codes), torch.zeros_like(params)
        qe = M.quantization_create(M.FLOAT16, M.PACKED_INT8C16, k, calculate_sum=False, symmetric=True, max_tokens=m,
                                   round_to_nearest_even=True)
        qe.bind([src], [codes_e, params_e])
        qe.set_shape(1, 1, m)
        q.launch(stream.cuda_stream)
        qe.launch(stream.cuda_stream)
        stream.synchronize()
        differing = int((codes_e[:, :, :] != codes[:, :, :]).sum().item())
        ops = 2.0 * m * k * n
        out = dict(base, metric="int8_dynamic_gemm_throughput", value=round(ops / wall / 1e12, 1),
                   unit="TOP/s", ms_per_step=round(wall * 1e3, 6),
                   dtype="i8 x i8, i32 accumulate (int8 MFMA), f32 rescale",
                   config=dict({"workload": "c4: per-token int8 quantization + int8 x int8 GEMM M=2048 K=2048 N=8192, fp16 out",
                                "ops_per_step": ops, "quantize_us": round(q_us, 3),
                                "asymmetric_quantization_ms_per_step": round(wall_a * 1e3, 6),
                                "codes_changed_by_round_to_nearest_even": "%d of %d" % (differing, m * k)}, **reg),
                   roofline={"bound": "mfma", "kernel": conv.kernel_name, "achieved": round(ops / us / 1e6, 1),
                             "peak": 5000.0, "unit": "TOP/s", "frac": round(ops / us / 1e6 / 5000.0, 4),
                             "traffic": None, "avg_launch_us": round(us, 3)})
    else:
        from decoder_stack import DecoderStack
        tokens = 1 if args.workload == "c5-decode" else max(5, args.tokens)
        # a decode step runs over the weights as a decode graph's ops ask for them (--layout library:
        # the one layout that serves both graphs)
        decode_layout = (tokens == 1 and args.layout != "library") or args.layout == "decode"
        st = DecoderStack(max_tokens=max(128, tokens), keep_host=False, decode_layout=decode_layout)
        st.set_tokens(tokens)
        wall, us, reg = time_graph(torch, stream, lambda s, i: st.launch(s), args.steps, args.warmup)
        wb, fl = st.weight_bytes(), st.flops(tokens)
        if tokens == 1:
            out = dict(base, metric="int4_decoder_stack_decode_hbm_bandwidth", value=round(wb / wall / 1e9, 1),
                       unit="GB/s", roofline={"bound": "hbm", "kernel": "%s (126 FCs per step; q/k/v and gate/up share a launch)" % " + ".join(sorted(set(st.kernel_names()))),
                                              "achieved": round(wb / us / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                              "frac": round(wb / us / 1e3 / HBM_PEAK_GBS, 4), "traffic": None,
                                              "avg_step_us": round(us, 1)})
        else:
            out = dict(base, metric="int4_decoder_stack_prefill_throughput", value=round(fl / wall / 1e12, 1),
                       unit="TFLOP/s", roofline={"bound": "mfma", "kernel": "fc_w4_mfma_gemm_kernel (126 FCs per step)",
                                                 "achieved": round(fl / us / 1e6, 1), "peak": 2500.0, "unit": "TFLOP/s",
                                                 "frac": round(fl / us / 1e6 / 2500.0, 4), "traffic": None,
                                                 "avg_step_us": round(us, 1)})
        out.update(ms_per_step=round(wall * 1e3, 6), dtype="u4 weights x f16 activations, f32 accumulate",
                   config=dict({"workload": "c5: 18 layers x (q,k,v,o,gate,up,down) int4 group-32, hidden 2048, %d token(s) "
                                            "per step" % tokens, "weight_bytes_per_step": wb, "flops_per_step": fl,
                                "weights_layout": "decode ops' layout (mldhip_fc_int4_weights_desc_decode)" if decode_layout
                                else "mldhip_fc_int4_weights_desc"}, **reg))
    print(json.dumps(out))


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(case, seconds):
    """The CPU restatement of the reference's generated kernel (oracle/: gcc -O3, eight output
    channels at a time with AVX2 + hardware fp16 conversion where the CPU has them, OpenMP over
    output slices) on the same case: whole-GEMV passes for about `seconds` / 2 on one thread, then
    on all the cores this process may use.  Returns {threads: (passes, seconds)}, the path taken."""
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
    cores = int(os.environ.get("OMP_NUM_THREADS", cores))
    runs = {}
    for threads in (1, cores):
        o.fc_kernel(act, packed, m, k, n, o.PREC_F32F16, 4, o.SCALE_LINEAR, sc, threads=threads)  # warm
        reps, t0 = 0, time.perf_counter()
        while True:
            o.fc_kernel(act, packed, m, k, n, o.PREC_F32F16, 4, o.SCALE_LINEAR, sc, threads=threads)
            reps += 1
            dt = time.perf_counter() - t0
            if dt >= seconds / 2 or reps >= 2000:
                break
        runs[threads] = (reps, dt)
    return runs, cores, o.last_fc_path


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
    for item in filter(None, args.tune.split(",")):
        name, value = item.split("=")
        M.check(M.lib().mldhip_set_tuning(name.encode(), int(value)))
    if args.workload != "c2":
        run_other(args, torch, M, W)
        return
    cfg = W.CONFIGS["c2"]
    case = W.make_fc_case(**cfg)
    m, k, n = case["m"], case["k"], case["n"]

    # ring of ops: copy 0 holds the seeded case, the others random packed bytes (every byte
    # pattern is a valid pair of int4 codes)
    devs = [W.FcDevice(case, reference_layout=args.layout == "reference")]
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
        # per-channel symmetric weights: y = (x . q) * s, in float64
        ref = (case["act"].astype(np.float64) @ case["w"].astype(np.float64).T) * case["scale"][:, 0].astype(np.float64)
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

        wall, launch_us, reg = time_graph(torch, stream, lambda st, i: ops[i % args.ring].launch(st), args.steps,
                                          max(args.warmup, args.ring), use_graph=not args.no_graph, ring=args.ring)
    use_graph = not args.no_graph
    ms_per_step = wall * 1e3
    value = algo_bytes / wall / 1e9
    achieved = algo_bytes / (launch_us * 1e-6) / 1e9

    # HBM bytes per launch are not measured by this run (hardware counters need rocprofv3 around the
    # process): `traffic` stays null, and the figure of the committed rocprofv3 --pmc summary (FETCH_SIZE
    # + WRITE_SIZE, scaled by a known-size copy) is passed on under a name that says where it is from
    traffic = None
    traffic_from_profile = None
    tname = "fc_w4_stream_c2.md" if args.layout == "reference" else "fc_w4_strip_c2.md"
    tpath = os.path.join(ROOT, "profiles", tname)
    if os.path.exists(tpath):
        import re
        mt = re.search(r"^hbm_bytes_per_launch = (\d+)", open(tpath).read(), re.M)
        traffic_from_profile = {"bytes": int(mt.group(1)), "source": "profiles/" + tname} if mt else None

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
                   "weights_layout": "kOSpatialIOGroupI4O4, output_group_size %d" % devs[0].desc.output_group_size,
                   "weight_ring": args.ring, "timed_region": "hipGraph replays" if use_graph else "eager launch loop",
                   "steps_multiple": reg["steps_multiple"], "launches_in_region": reg["launches_in_region"],
                   "timed_regions": reg["timed_regions"], "reported_region": reg["reported_region"],
                   "algorithmic_bytes_per_step": algo_bytes, "flops_per_step": flops,
                   "pct_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2)},
        "roofline": {"bound": "hbm", "kernel": kernel, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "traffic_from_profile": traffic_from_profile, "avg_launch_us": round(launch_us, 3)},
    }
    if not args.no_cpu_baseline:
        runs, cores, path = cpu_baseline(case, args.cpu_seconds)
        rate = {t: algo_bytes * r / dt / 1e9 for t, (r, dt) in runs.items()}
        out["cpu_baseline"] = {"value": round(rate[cores], 3), "unit": "GB/s", "cores": cores, "kind": "port",
                               "value_1t": round(rate[1], 3), "cpu_model": cpu_model(),
                               "code_path": "avx2+fma+f16c, 8 channels at a time" if path == 1 else "scalar, software fp16",
                               "sample": "full passes of the same c2 GEMV (oracle restatement of the reference's "
                                         "generated kernel, gcc -O3, OpenMP over output slices): %d in %.1f s on 1 "
                                         "thread, %d in %.1f s on %d threads" % (runs[1] + runs[cores] + (cores,))}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
