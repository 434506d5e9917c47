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
# HBM-side bytes per GEMM launch (fetched + written), from the two rocprofv3 --pmc runs
# summarised in profiles/gemm_pipe_int8_flux_m4608.md (FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 KiB,
# factors from a 256 MiB copy).  Counters cannot be read from inside this process.
# the GEMM kernels the tile heuristic picks for each configuration's linears (rocprofv3 traces, profiles/)
GEMM_KERNELS = {
    1: "segq::gemm_kernel (int8, general)",
    2: "segq::gemm_pipe_kernel<128,128> / <256,128, two ranges> (e4m3)",
    3: "segq::gemm_pipe_kernel<192,288> / <288,192> (int8)",
    4: "segq::gemm_pipe_kernel<128,128, group factors> (int8 x int4 expanded to int8)",
    5: "segq::gemm_pipe_kernel<288,192> / <128,128> (int8 with parked ranges, e4m3 rescaled in place)",
}
MEASURED_TRAFFIC_BYTES = {3: 343.5e6}


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
    ap.add_argument("--calib-copy", action="store_true",
                    help="also launch one plain 256 MiB -> 256 MiB elementwise copy, the yardstick for HBM byte counters")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch
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

    def step(i):
        xs = sets[i % n_sets]
        for layer, x in zip(layers, xs):
            layer(x)

    if args.calib_copy:
        src = torch.zeros(64 << 20, dtype=torch.int32, device=dev)
        dst = torch.empty_like(src)
        torch.mul(src, 1, out=dst)
        torch.cuda.synchronize()
        del src, dst
    for i in range(args.ramp + args.warmup):
        step(i)
    torch.cuda.synchronize()
    # the timed region: exactly args.steps steps, nothing else on the stream
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(args.ramp + args.warmup + i)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    wall = t1 - t0
    total_ops = sum(sp.ops for sp in specs)
    value = total_ops * args.steps / wall / 1e12
    # A second pass of the same steps with a HIP event pair around every launch gives the
    # per-kernel durations for the roofline figures.  It is kept out of the timed region:
    # the twelve event records per step cost ~50 us of a ~500 us step.
    with ops.record_launches() as log:
        for i in range(args.steps):
            step(args.ramp + args.warmup + args.steps + i)
        torch.cuda.synchronize()

    g_t = g_ops = g_exec = g_bytes = q_t = q_bytes = 0.0
    n_g = n_q = 0
    for kind, e0, e1, info in log:
        ms = e0.elapsed_time(e1)
        if kind == "gemm":
            g_t += ms * 1e-3
            g_ops += 2.0 * info["m"] * info["n"] * info["k_alg"] * info["batch"]
            g_exec += 2.0 * info["m"] * info["n"] * info["k_exec"] * info["batch"]
            g_bytes += info["batch"] * (info["m"] * info["k_alg"] + info["n"] * info["k_alg"] * (0.5 if info["b_fmt"] == "int4" else 1.0)
                                        + 2.0 * info["m"] * info["n"])
            n_g += 1
        else:
            q_t += ms * 1e-3
            q_bytes += info["rows"] * info["cols"] * (info["x_bytes"] + info["code_bytes"] * info["tensors"])
            n_q += 1
    fmt = specs[0].act
    peak = PEAK_TOPS[fmt]
    g_tops = g_ops / g_t / 1e12
    q_gbs = q_bytes / q_t / 1e9
    out = {
        "metric": "seg-GEMM TOPS + % MFMA peak (FLUX shapes, M=4608); quantize kernel GB/s",
        "value": round(value, 2), "unit": "TOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ramp_steps": args.ramp,
        "ms_per_step": round(wall / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8" if fmt == "int8" else "fp8_e4m3", "data": "synthetic",
        "config": {"workload": f"config {args.config}: " + ", ".join(f"{s.name} M{s.M} K{s.K} N{s.N} {s.kernel_type}" for s in specs),
                   "step": "activation quantize + segmented GEMM with fused dequant+bias, per linear",
                   "input_dtype": str(specs[0].x_dtype).replace("torch.", ""), "output_dtype": str(specs[0].x_dtype).replace("torch.", "")},
        "roofline": {"bound": "mfma", "kernel": GEMM_KERNELS.get(args.config, "segq::gemm_pipe_kernel"), "achieved": round(g_tops, 2), "peak": peak,
                     "unit": "TFLOP/s", "frac": round(g_tops / peak, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(args.config),
                     "launches": n_g, "avg_launch_us": round(g_t / max(n_g, 1) * 1e6, 2),
                     "algorithmic_bytes_per_launch": round(g_bytes / max(n_g, 1)),
                     "executed_tops": round(g_exec / g_t / 1e12, 2)},
        "quantize": {"bound": "hbm", "kernel": "segq::quant_*_kernel", "achieved": round(q_gbs, 1), "peak": PEAK_HBM,
                     "unit": "GB/s", "frac": round(q_gbs / PEAK_HBM, 4), "launches": n_q,
                     "avg_launch_us": round(q_t / max(n_q, 1) * 1e6, 2)},
    }
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
        out["e4m3_same_shapes"] = {"bound": "mfma", "kernel": "segq::gemm_pipe_kernel<192,288> / <288,192> (e4m3)",
                                   "achieved": round(ops8 / t8 / 1e12, 2), "peak": PEAK_TOPS["fpe4m3"], "unit": "TFLOP/s",
                                   "frac": round(ops8 / t8 / 1e12 / PEAK_TOPS["fpe4m3"], 4), "launches": n8,
                                   "avg_launch_us": round(t8 / max(n8, 1) * 1e6, 2)}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(specs, args.cpu_rows)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
