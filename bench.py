#!/usr/bin/env python3
"""Benchmark of the real-quantised segmented linear on one MI355X.

A step is one pass of the hot path (activation quantise -> segmented MFMA GEMM
with fused de-quantisation and bias) over every linear of the workload, on
synthetic inputs already resident in HBM.  The default workload is the FLUX.1
double-stream block at M = 4608, INT8 W8A8 (the configuration the headline
metric is quoted on).  Prints one JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TOPS = {"int8": 5000.0, "fpe4m3": 5000.0}  # dense MFMA, TOP/s
PEAK_HBM = 8000.0                               # GB/s
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "gemm_hbm_traffic_configs_1_to_5.txt")


def recorded_traffic(config):
    """HBM-side bytes per GEMM launch from the last rocprofv3 counter runs of this workload
    (counters cannot be read from inside this process): profiles/gemm_hbm_traffic_configs_1_to_5.txt, written by
    `python -m segquant_amd.profile_counters`.  (bytes or None, where the figure comes from)."""
    try:
        rec = json.load(open(TRAFFIC_FILE)).get(str(config))
    except (OSError, ValueError):
        rec = None
    if not rec:
        return None, "no counter run recorded for this workload"
    return rec["traffic_bytes_per_launch"], f"profiles/gemm_hbm_traffic_configs_1_to_5.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE at commit {rec.get('commit', '?')})"


def cpu_baseline(specs, rows, repeats=5):
    """The fake-quant path (fp32 quantise->de-quantise + torch matmul) on the
    host cores, on the first ``rows`` tokens of every linear of the workload
    (0: all of them)."""
    import torch
    from oracle import fake_path_torch as F
    from segquant_amd import workloads as W
    cores = os.cpu_count() or 1
    threads = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(threads)
    work = []
    ops = 0
    for sp in specs:
        rows_sp = min(rows, sp.M) if rows > 0 else sp.M
        x = W.make_input(sp, M=rows_sp)
        w = W.make_weight(sp)
        # weights are fake-quantised once, offline, and stored de-quantised
        if sp.weight_axis == 1 and sp.weight_group:
            wg = w.reshape(w.shape[0], -1, sp.weight_group)
            w_hat = F.fake_quant(wg, sp.weight, F.scale_of(wg.abs().amax(dim=2, keepdim=True), sp.weight)).reshape(w.shape)
        elif sp.weight_axis == 1:
            ws = F.scale_of(w.abs().amax(dim=1, keepdim=True), sp.weight)
            w_hat = F.fake_quant(w, sp.weight, ws)
        elif sp.seg_mode == "weight" and sp.chunksizes:
            w_hat = torch.cat([F.fake_quant(b, sp.weight, F.scale_of(b.abs().amax(), sp.weight))
                               for b in w.split(sp.chunksizes, dim=0)])
        else:
            w_hat = F.fake_quant(w, sp.weight, F.scale_of(w.abs().amax(), sp.weight))
        bounds = W.segment_bounds(sp)
        n_in = len(bounds) - 1
        dual = [i in sp.dual_segments for i in range(n_in)]
        work.append((x, w_hat, W.make_bias(sp), sp.act, bounds, dual, sp.act_axis == -1))
        ops += 2 * rows_sp * sp.N * sp.K
    times = []
    for it in range(repeats + 1):
        t0 = time.perf_counter()
        for args in work:
            F.fake_linear(*args)
        t1 = time.perf_counter()
        if it:  # first pass is the warm-up
            times.append(t1 - t0)
    t = sorted(times)[len(times) // 2]
    return {"value": ops / t / 1e12, "unit": "TOP/s", "cores": threads, "kind": "port",
            "sample": (f"first {rows} tokens" if rows > 0 else "all tokens") +
                      f" of each linear of the workload ({specs[0].M} for the first), fp32 fake-quant + torch.matmul, "
                      f"median of {repeats} passes, {t:.3f} s per pass"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--ramp", type=int, default=30,
                    help="untimed steps before the warm-up: the first ~25 steps after start-up run ~10 %% slower "
                         "(measured: 606 us against 547 us per step) while clocks and page tables settle")
    ap.add_argument("--config", type=int, default=3, help="benchmark configuration 1..5 (default: FLUX int8, M=4608)")
    ap.add_argument("--cpu-rows", type=int, default=0,
                    help="tokens per linear in the CPU baseline sample (0: the whole workload; a few seconds for config 3)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-e4m3", action="store_true", help="skip the supplementary e4m3 pass over the config-3 shapes")
    ap.add_argument("--producers", action="store_true",
                    help="config 5 only: also time every linear fed by its two producers (attention output, MLP output before "
                         "its GELU) through forward_parts, against torch's GELU + concatenation in front of the ordinary forward")
    ap.add_argument("--overlap", action="store_true",
                    help="also time the steps with each linear's quantise kernel on a second stream under the previous linear's "
                         "GEMM (measured on config 3: 7 %% slower than in sequence, the chip being held by its power limit)")
    ap.add_argument("--graph", action="store_true",
                    help="also time the steps replayed from captured HIP graphs (one graph per rotating input set, at most 32): "
                         "what a serving loop pays when the host's enqueue time is off the path")
    ap.add_argument("--pair", action="store_true",
                    help="config 2 only: also time fc1 -> GELU(tanh) -> fc2 as chained linears (forward_into: fc1's GEMM epilogue writes "
                         "fc2's DualScale codes; no float tensor and no quantise launch between the two GEMMs)")
    ap.add_argument("--lib", default=None,
                    help="load this build of the library instead of segquant_amd/libsegq.so (measurement variants made by "
                         "`make -C segquant_amd/csrc variant`, whose results may be wrong on purpose: timings only)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also launch one plain 256 MiB -> 256 MiB elementwise copy, the yardstick for HBM byte counters")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch
    if args.lib:
        from segquant_amd import _lib as _L
        _L.LIB_PATH = os.path.abspath(args.lib)
    from segquant_amd import ops, workloads as W
    from segquant_amd._lib import lib
    lib()  # fail loudly if the HIP library is missing
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    dev = "cuda:0"
    torch.cuda.set_device(0)

    specs = W.config_linears(args.config)
    layers, inputs = [], []
    bytes_per_set = 0
    for sp in specs:
        layer, x = W.build_layer(sp, device=dev, real_quant=True)
        assert layer.optimizer.real_quant
        layers.append(layer)
        inputs.append(x.to(sp.x_dtype))
        bytes_per_set += sp.M * sp.K * (x.to(sp.x_dtype).element_size() + 1) + sp.M * sp.N * 2
    # rotate over enough input copies that a step never finds its operands in the
    # 256 MB last-level cache left there by the previous step
    n_sets = max(2, -(-(768 << 20) // bytes_per_set))
    sets = [[x.to(dev).clone() for x in inputs] for _ in range(n_sets)]

    biases = [layer.bias_data if layer.bias else None for layer in layers]

    def step(i):
        xs = sets[i % n_sets]
        for layer, x in zip(layers, xs):
            layer(x)

    side = torch.cuda.Stream()  # default priority, like the main stream

    def step_overlapped(i):
        """The same launches with the quantise kernel of linear l + 1 enqueued on a second stream,
        so that it runs (bound by HBM) under the GEMM of linear l (bound by the matrix cores).
        The linears of a step are independent, which is what makes this legal here."""
        xs = sets[i % n_sets]
        work = [layer.optimizer.fused_launches(x, b, fresh=True) for layer, x, b in zip(layers, xs, biases)]
        main = torch.cuda.current_stream()
        side.wait_stream(main)  # buffers the allocator hands out again were last used on the main stream
        ops.quantize_launch(work[0][0])
        ready = None
        for l, (q, g, ws) in enumerate(work):
            nxt = None
            if l + 1 < len(work):
                with torch.cuda.stream(side):
                    ops.quantize_launch(work[l + 1][0])
                    nxt = torch.cuda.Event()
                    nxt.record(side)
            if ready is not None:
                main.wait_event(ready)
            ops.gemm_launch(g, ws)
            ready = nxt

    if args.calib_copy:
        src = torch.zeros(64 << 20, dtype=torch.int32, device=dev)
        dst = torch.empty_like(src)
        torch.mul(src, 1, out=dst)
        torch.cuda.synchronize()
        del src, dst
    # untimed: ramp, then warm-up.  The first ramp steps are clocked on their own, so that the
    # line also says what a step costs right after start-up
    n_cold = min(10, args.ramp)
    torch.cuda.synchronize()
    t_c0 = time.perf_counter()
    for i in range(n_cold):
        step(i)
    torch.cuda.synchronize()
    cold_ms = (time.perf_counter() - t_c0) / n_cold * 1e3 if n_cold else None
    for i in range(n_cold, args.ramp + args.warmup):
        step(i)
    torch.cuda.synchronize()
    # the timed region: exactly args.steps steps, nothing else on the stream
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(args.ramp + args.warmup + i)
    t_host = time.perf_counter()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    wall = t1 - t0
    total_ops = sum(sp.ops for sp in specs)
    value = total_ops * args.steps / wall / 1e12
    wall_ov = None
    if args.overlap:
        # the same steps with quantise launches overlapped with the previous linear's GEMM
        for i in range(args.warmup):
            step_overlapped(i)
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        for i in range(args.steps):
            step_overlapped(args.warmup + i)
        torch.cuda.synchronize()
        wall_ov = time.perf_counter() - t2
    graph_res = None
    if args.graph:
        n_g = min(n_sets, 32)
        cap = torch.cuda.Stream()
        cap.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(cap):  # buffers, workspaces and kernel attributes of this stream exist before the capture
            for i in range(2):
                step(i)
        torch.cuda.current_stream().wait_stream(cap)
        torch.cuda.synchronize()
        graphs = []
        for i in range(n_g):
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr, stream=cap):
                step(i)
            graphs.append(gr)
        for i in range(args.warmup):
            graphs[i % n_g].replay()
        torch.cuda.synchronize()
        tg0 = time.perf_counter()
        for i in range(args.steps):
            graphs[i % n_g].replay()
        torch.cuda.synchronize()
        wall_g = time.perf_counter() - tg0
        graph_res = {"value": round(total_ops * args.steps / wall_g / 1e12, 2), "unit": "TOP/s", "ms_per_step": round(wall_g / args.steps * 1e3, 4),
                     "graphs": n_g, "how": "each step replayed from a HIP graph captured over one of the rotating input sets"}
        del graphs
    pair_res = None
    if args.pair and args.config == 2:
        fc1, fc2 = layers
        xs1 = [s_[0] for s_ in sets]
        for i in range(args.warmup):
            fc1.forward_into(fc2, xs1[i % n_sets], pre_op="gelu_tanh")
        torch.cuda.synchronize()
        tp0 = time.perf_counter()
        for i in range(args.steps):
            fc1.forward_into(fc2, xs1[i % n_sets], pre_op="gelu_tanh")
        torch.cuda.synchronize()
        wall_p = time.perf_counter() - tp0
        with ops.record_launches() as plog:
            for i in range(args.steps):
                fc1.forward_into(fc2, xs1[i % n_sets], pre_op="gelu_tanh")
            torch.cuda.synchronize()
        per = {}
        for j, (kind, e0, e1, info) in enumerate(plog):
            per.setdefault(("fc1_quantize", "fc1_gemm_codes_out", "fc2_gemm")[j % 3], []).append(e0.elapsed_time(e1) * 1e3)
        pair_res = {"value": round(total_ops * args.steps / wall_p / 1e12, 2), "unit": "TOP/s", "ms_per_step": round(wall_p / args.steps * 1e3, 4),
                    "launches_per_step": 3, "quantize_launches_per_step": 1,
                    "kernel_us": {k: round(sum(v) / len(v), 2) for k, v in per.items()},
                    "how": "fc1.forward_into(fc2, x, pre_op='gelu_tanh'): fc1 quantise, fc1 GEMM writing fc2's two code tensors, fc2 GEMM"}
    # Per-kernel durations for the roofline figures, outside the timed region.  GEMM: the same
    # steps with a HIP event pair around every launch (the records cost a few microseconds per
    # launch, little against a GEMM).  Quantise: the kernels are ~10-30 us, so each linear's
    # quantise launch is instead repeated back to back over the rotating inputs between ONE event
    # pair; its average includes the gaps between launches and agrees with the kernel trace.
    with ops.record_launches() as log:
        for i in range(args.steps):
            step(args.ramp + args.warmup + args.steps + i)
        torch.cuda.synchronize()
    q_t = q_bytes = 0.0
    n_q = 0
    q_detail = []
    q_sets = []
    for li, layer in enumerate(layers):
        # enough distinct inputs (and outputs) that no launch finds its operands in the 256 MB
        # last-level cache: the rotation of the timed steps is too short when one kernel runs alone
        sp = specs[li]
        per_launch = sp.M * sp.K * (inputs[li].element_size() + 1)
        copies = [xs[li] for xs in sets]
        while len(copies) * per_launch < (640 << 20):
            copies.append(copies[0].clone())
        qs = [layer.optimizer.fused_launches(x, biases[li], fresh=True)[0] for x in copies]
        q_sets.append(qs)
        reps = max(1, -(-args.steps // len(qs)))
        for q in qs:
            ops.quantize_launch(q)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            for q in qs:
                ops.quantize_launch(q)
        e1.record()
        torch.cuda.synchronize()
        info = qs[0][2]
        nb = info["rows"] * info["cols"] * (info["x_bytes"] + info["code_bytes"] * info["tensors"]) + (4 * info["rows"] if info["dynamic"] else 0)
        t = e0.elapsed_time(e1) * 1e-3
        q_t += t
        q_bytes += nb * reps * len(qs)
        n_q += reps * len(qs)
        q_detail.append({"rows": info["rows"], "cols": info["cols"], "us": round(t / (reps * len(qs)) * 1e6, 2),
                         "GB/s": round(nb * reps * len(qs) / t / 1e9, 1)})
        del qs, copies

    g_t = g_ops = g_exec = g_bytes = 0.0
    n_g = 0
    for kind, e0, e1, info in log:
        if kind != "gemm":
            continue
        ms = e0.elapsed_time(e1)
        g_t += ms * 1e-3
        g_ops += 2.0 * info["m"] * info["n"] * info["k_alg"] * info["batch"]
        g_exec += 2.0 * info["m"] * info["n"] * info["k_exec"] * info["batch"]
        g_bytes += info["batch"] * (info["m"] * info["k_alg"] + info["n"] * info["k_alg"] * (0.5 if info["b_fmt"] == "int4" else 1.0)
                                    + 2.0 * info["m"] * info["n"])
        n_g += 1
    # Supplementary: linears whose inputs are of one kind (same shape and dtype, dynamic per-row
    # scales) quantised through segq_quantize_many, which lets them share a launch.  Not part of
    # the step: in a block these inputs are produced one after the other.
    q_batched = None
    kinds = {}
    for li, qs in enumerate(q_sets):
        info = qs[0][2]
        if info["dynamic"] and info["tensors"] == 1:
            kinds.setdefault((info["rows"], info["cols"], info["x_bytes"], info["code_bytes"]), []).append(li)
    for kind, lis in kinds.items():
        if len(lis) < 2:
            continue
        n = min(len(q_sets[li]) for li in lis)
        groups = [[q_sets[li][i] for li in lis] for i in range(n)]
        for grp in groups:
            ops.quantize_many(grp)
        torch.cuda.synchronize()
        passes = []   # median of three passes: one pass is a few hundred microseconds, within reach of a single stall
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for grp in groups:
                ops.quantize_many(grp)
            e1.record()
            torch.cuda.synchronize()
            passes.append(e0.elapsed_time(e1))
        nb = kind[0] * kind[1] * (kind[2] + kind[3]) + 4 * kind[0]
        t = sorted(passes)[1] * 1e-3 / (n * len(lis))
        q_batched = {"linears": [specs[li].name for li in lis], "rows": kind[0], "cols": kind[1], "us_per_tensor": round(t * 1e6, 2),
                     "GB/s": round(nb / t / 1e9, 1), "frac": round(nb / t / 1e9 / PEAK_HBM, 4)}
        break
    # the kernels the library picks for these linears, asked of the library itself
    kernels = []
    for layer, x, b in zip(layers, sets[0], biases):
        q, g, ws = layer.optimizer.fused_launches(x, b)
        plan = ops.gemm_plan(g, ws)
        kernels.append(plan["kernel"] + (f" x{plan['splits']} K shares" if plan["splits"] > 1 else "") + (" parked ranges" if plan["parked"] else ""))
    fmt = specs[0].act
    peak = PEAK_TOPS[fmt]
    # the same peak from the device itself: CUs x 4 SIMDs x 2048 8-bit ops per clock and SIMD (one
    # 16x16x64 int8 or 16x16x128 fp8 MFMA every 16 / 32 clocks) x the highest engine clock it reports
    import ctypes
    from segquant_amd import _lib as L_
    dev_cus, dev_khz = ctypes.c_int32(0), ctypes.c_int32(0)
    L_.check(lib().segq_device_info(ctypes.byref(dev_cus), ctypes.byref(dev_khz)))
    clock_ghz = dev_khz.value / 1e6
    peak_dev = dev_cus.value * 4 * 2048 * clock_ghz / 1e3
    g_tops = g_ops / g_t / 1e12
    q_gbs = q_bytes / q_t / 1e9
    traffic, traffic_source = recorded_traffic(args.config)
    out = {
        "metric": "seg-GEMM TOPS + % MFMA peak (FLUX shapes, M=4608); quantize kernel GB/s",
        "value": round(value, 2), "unit": "TOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ramp_steps": args.ramp,
        "cold_start_ms_per_step": None if cold_ms is None else round(cold_ms, 4),
        "ms_per_step": round(wall / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8" if fmt == "int8" else "fp8_e4m3", "data": "synthetic",
        "config": {"workload": f"config {args.config}: " + ", ".join(f"{s.name} M{s.M} K{s.K} N{s.N} {s.kernel_type}" for s in specs),
                   "step": "activation quantize + segmented GEMM with fused dequant+bias, per linear",
                   "input_dtype": str(specs[0].x_dtype).replace("torch.", ""), "output_dtype": str(specs[0].x_dtype).replace("torch.", "")},
        "roofline": {"bound": "mfma", "kernel": " / ".join(dict.fromkeys(kernels)) + f" ({fmt})", "achieved": round(g_tops, 2), "peak": peak,
                     "unit": "TFLOP/s", "frac": round(g_tops / peak, 4), "traffic": traffic, "traffic_source": traffic_source,
                     "peak_from_device": {"compute_units": dev_cus.value, "max_engine_clock_GHz": round(clock_ghz, 3),
                                          "ops_per_clock_per_cu": 8192, "TOP/s": round(peak_dev, 1)},
                     "launches": n_g, "avg_launch_us": round(g_t / max(n_g, 1) * 1e6, 2),
                     "algorithmic_bytes_per_launch": round(g_bytes / max(n_g, 1)),
                     "executed_tops": round(g_exec / g_t / 1e12, 2),
                     # the same launches against the HBM roof (the bound of the small-M shapes)
                     "hbm_GBps": round(g_bytes / g_t / 1e9, 1), "hbm_frac": round(g_bytes / g_t / 1e9 / PEAK_HBM, 4)},
        "quantize": {"bound": "hbm", "kernel": "segq::quant_dynamic_row_kernel / quant_dynamic_kernel / quant_static_kernel", "achieved": round(q_gbs, 1),
                     "peak": PEAK_HBM, "unit": "GB/s", "frac": round(q_gbs / PEAK_HBM, 4), "launches": n_q,
                     "avg_launch_us": round(q_t / max(n_q, 1) * 1e6, 2), "per_linear": q_detail,
                     "shared_launch": q_batched},
        # host time to enqueue one linear (descriptor fill + one library call), from the timed region
        "host_us_per_linear": round((t_host - t0) / (args.steps * len(layers)) * 1e6, 2),
    }
    if args.lib:
        out["library"] = args.lib
    # every GEMM launch of the instrumented pass by linear (events on the launching stream)
    per_gemm = {}
    gi = 0
    for kind, e0, e1, info in log:
        if kind == "gemm":
            per_gemm.setdefault(specs[gi % len(specs)].name, []).append(e0.elapsed_time(e1) * 1e3)
            gi += 1
    out["roofline"]["per_linear_us"] = {k: round(sum(v) / len(v), 2) for k, v in per_gemm.items()}
    if args.producers and args.config == 5:
        import torch.nn.functional as Fn
        res = []
        for sp, layer in zip(specs, layers):
            k0 = sp.chunksizes[0]
            pre = W.make_input(sp, activated=False).to(sp.x_dtype)
            n_c = max(2, -(-(768 << 20) // (sp.M * sp.K * 3)))
            parts = [(pre[:, :k0].to(dev).contiguous(), pre[:, k0:].to(dev).contiguous()) for _ in range(n_c)]

            def torch_front(i):
                a, m = parts[i % n_c]
                return layer(torch.cat([a, Fn.gelu(m, approximate="tanh")], dim=1))

            def fused_front(i):
                a, m = parts[i % n_c]
                return layer.forward_parts([a, m], pre_ops=[None, "gelu_tanh"])

            t = {}
            for name, fn in (("torch_gelu_cat_then_linear", torch_front), ("forward_parts", fused_front)):
                for i in range(5):
                    fn(i)
                torch.cuda.synchronize()
                ta = time.perf_counter()
                for i in range(args.steps):
                    fn(i)
                torch.cuda.synchronize()
                t[name] = (time.perf_counter() - ta) / args.steps * 1e6
            res.append({"linear": sp.name, **{k: round(v, 1) for k, v in t.items()}})
            del parts
        out["producer_fusion_us"] = res
    if graph_res is not None:
        out["graph_replay"] = graph_res
    if pair_res is not None:
        out["chained_pair"] = pair_res
    out["quantize"]["launches_per_step"] = len(layers)
    if wall_ov is not None:
        out["overlapped"] = {"value": round(total_ops * args.steps / wall_ov / 1e12, 2), "unit": "TOP/s",
                             "ms_per_step": round(wall_ov / args.steps * 1e3, 4),
                             "how": "quantise of linear l+1 on a second stream under the GEMM of linear l (the linears of a step are independent)"}
    if args.config == 3 and not args.no_e4m3:
        # Supplementary: the same three shapes with e4m3 codes on both sides (the metric names
        # int8 and fp8 peaks alike), GEMM launches only, same rotation of operands.
        import dataclasses
        del sets, layers
        torch.cuda.empty_cache()
        specs8 = [dataclasses.replace(sp, act="fpe4m3", weight="fpe4m3") for sp in specs]
        layers8 = [W.build_layer(sp, device=dev, real_quant=True)[0] for sp in specs8]
        sets8 = [[x.to(dev).clone() for x in inputs] for _ in range(n_sets)]
        for i in range(20):
            for layer, x in zip(layers8, sets8[i % n_sets]):
                layer(x)
        with ops.record_launches() as log8:
            for i in range(20):
                for layer, x in zip(layers8, sets8[i % n_sets]):
                    layer(x)
            torch.cuda.synchronize()
        t8 = sum(e0.elapsed_time(e1) for kind, e0, e1, _ in log8 if kind == "gemm") * 1e-3
        n8 = sum(1 for kind, *_ in log8 if kind == "gemm")
        ops8 = sum(2.0 * info["m"] * info["n"] * info["k_alg"] for kind, _, _, info in log8 if kind == "gemm")
        k8 = []
        for layer, x in zip(layers8, sets8[0]):
            q, g, ws = layer.optimizer.fused_launches(x, layer.bias_data if layer.bias else None)
            k8.append(ops.gemm_plan(g, ws)["kernel"])
        out["e4m3_same_shapes"] = {"bound": "mfma", "kernel": " / ".join(dict.fromkeys(k8)) + " (fpe4m3)",
                                   "achieved": round(ops8 / t8 / 1e12, 2), "peak": PEAK_TOPS["fpe4m3"], "unit": "TFLOP/s",
                                   "frac": round(ops8 / t8 / 1e12 / PEAK_TOPS["fpe4m3"], 4), "launches": n8,
                                   "avg_launch_us": round(t8 / max(n8, 1) * 1e6, 2)}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(specs, args.cpu_rows)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
