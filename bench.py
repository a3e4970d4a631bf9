#!/usr/bin/env python3
"""Benchmark of the hot path: BERT-base encoder (batch 1, seq 128, fp32) planned like the reference's
Executor (plain_greedy by default) and replayed as HIP launches over one HBM arena.

A "step" is one inference: one replay of the whole launch plan (416 graph nodes issued as a few dozen kernel
launches after launch-level fusion) on inputs that are already resident in HBM.  Prints ONE JSON line:
`value` = inferences/s over the timed replays; `roofline` = the contraction kernel's flops over its launch
durations (dispatch begin/end timestamps) against the fp32 MFMA peak, `roofline.traffic` = the HBM bytes per
launch the tracked profiler summary (`roofline.traffic_source`) holds for exactly this workload, else null;
`cpu_baseline` = the oracle's scalar loop nests on one host core for a bounded sample;
`peak_hbm_bytes` = arena + constants + interface staging.  The default run adds `configs`: the same
measurement (GPU legs only) for the other five configurations and for BERT-base under the DP executor.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config NAME] [--executor plain_greedy|dp_greedy]
                    [--no-cpu-baseline] [--per-kernel] [--per-launch] [--bf16] [--hbm-kernels] [--mfma-kernels]
"""
import argparse
import json
import os
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

FP32_MFMA_PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix peak
HBM_PEAK_GBS = 8000.0

# HBM bytes per launch of the contraction kernel come from the tracked profiler summary of the default workload
# (BERT-base, seq 128, 12 layers, plain_greedy, fusion on): rocprofv3 FETCH_SIZE / WRITE_SIZE per dispatch, each
# scaled by what the same counter reads for the identity-copy kernel.  The summary carries one line
# "traffic_bytes_per_launch = N" for bench.py; any other workload reports null.
TRAFFIC_SUMMARY = os.path.join("profiles", "matmul_bert_base_s128.md")


def traffic_from_summary():
    import re

    try:
        text = open(os.path.join(ROOT, TRAFFIC_SUMMARY)).read()
    except OSError:
        return None
    m = re.search(r"traffic_bytes_per_launch\s*=\s*([0-9][0-9,_]*)", text)
    return int(m.group(1).replace(",", "").replace("_", "")) if m else None


def host_cores():
    try:
        return len(os.sched_getaffinity(0))
    except AttributeError:
        return os.cpu_count() or 1


# what the CPU figure is and is not
ORACLE_CAVEAT = ("the oracle is a scalar restatement of the reference's loop nests built with gcc -O2 -ffp-contract=off (accumulate in "
                 "memory, summation order as written): it understates the reference, which JIT-compiles the same nests at LLVM's aggressive level")


def cpu_baseline(layers_total: int, sample_layers: int, seq: int):
    """The oracle's loop nests (the FluidML-equivalent CPU execution) on one core, timed on
    `sample_layers` encoder layers of the same configuration plus the embedding/mask prologue;
    the per-layer time is extrapolated to `layers_total` layers."""
    from fluidml_amd import models
    from oracle import graph_runner

    net = models.bert_base(seq=seq, layers=sample_layers)
    feeds = models.bert_inputs(seq)
    timings = {}
    graph_runner.run_graph(net, feeds, timings=timings)
    names = [n.name for n in net.nodes]
    per_layer = (len(names) - 8) // sample_layers  # 5 embedding nodes + 3 mask nodes come first
    prologue = sum(timings[n][1] for n in names[:8])
    layer_time = sum(timings[n][1] for n in names[8:]) / sample_layers
    total = prologue + layers_total * layer_time
    return {
        "value": 1.0 / total,
        "unit": "inferences/s",
        "cores": 1,
        "host_cores": host_cores(),
        "kind": "port",
        "sample": f"{sample_layers} of {layers_total} encoder layers + embeddings at seq {seq} (one inference each) on 1 of "
                  f"{host_cores()} host cores, {per_layer} kernels per layer; per-layer time {layer_time:.3f} s extrapolated to {layers_total} layers; "
                  + ORACLE_CAVEAT,
        "seconds_per_inference": total,
    }


def make_config(args):
    """(net, feeds, workload text, batch) of the chosen benchmark configuration at full size."""
    from fluidml_amd import models

    if args.config == "bert_base":
        return (models.bert_base(seq=args.seq, layers=args.layers), models.bert_inputs(args.seq),
                f"BERT-base encoder ONNX graph, batch 1, seq {args.seq}, {args.layers} layers, fp32", 1)
    if args.config == "convbert_base":
        return (models.convbert_base(seq=args.seq, layers=args.layers), models.bert_inputs(args.seq),
                f"ConvBERT-base ONNX graph, batch 1, seq {args.seq}, {args.layers} layers, fp32", 1)
    if args.config == "gpt_neox":
        return (models.gpt_neox(), models.gpt_neox_inputs(), "GPT-NeoX-style decoder prefill, batch 1, seq 256, 6 layers, fp32", 1)
    if args.config == "efficientnet_b0":
        return (models.efficientnet_b0(), models.image_input((1, 3, 224, 224)), "EfficientNet-B0 ONNX graph, batch 1, 224x224, fp32", 1)
    batch = 8 if args.config == "vgg16_b8" else 1
    return (models.vgg16(batch), models.image_input((batch, 3, 224, 224)), f"VGG-16 ONNX graph, batch {batch}, 224x224, fp32", batch)


def cpu_baseline_whole(net, feeds, batch):
    """One whole inference of the oracle's loop nests on one core (configurations other than BERT-base)."""
    import threading

    from oracle import graph_runner

    # a whole VGG-16 pass at batch 8 takes the scalar loop nests minutes: say so while it runs
    done = threading.Event()

    def heartbeat():
        while not done.wait(30.0):
            print(f"[bench] cpu baseline still running ({time.perf_counter() - t0:.0f} s) ...", file=sys.stderr, flush=True)

    t0 = time.perf_counter()
    threading.Thread(target=heartbeat, daemon=True).start()
    try:
        graph_runner.run_graph(net, feeds)
    finally:
        done.set()
    total = time.perf_counter() - t0
    return {"value": batch / total, "unit": "inferences/s", "cores": 1, "host_cores": host_cores(), "kind": "port",
            "sample": f"one whole forward pass of batch {batch} on 1 of {host_cores()} host cores; " + ORACLE_CAVEAT,
            "seconds_per_inference": total / batch}


def measure(args, config, executor, per_kernel=False, per_launch=False):
    """Compile `config` with `executor`, replay it args.steps times and return (result dict, objects for more legs)."""
    import types

    import numpy as np
    import torch

    from fluidml_amd import fluidml

    args = types.SimpleNamespace(**{**vars(args), "config": config, "executor": executor})
    net, feeds, workload, batch = make_config(args)
    with tempfile.TemporaryDirectory() as tmp:
        path = net.save(os.path.join(tmp, args.config + ".onnx"))
        ex = getattr(fluidml.Executor, "make_" + args.executor)(args.config, 1)
        t0 = time.perf_counter()
        # (--plan-json: the JSON the compile writes -- the DP's tables, the tile configuration picked per contraction
        # and the side-branch decision; FLUIDML_TUNE=<that file> makes a later compile repeat the picks without timing)
        ex.compile(path, json=getattr(args, "plan_json", None))
        compile_s = time.perf_counter() - t0
    plan = ex.plan()

    # one full Invoke: H2D inputs, replay, D2H output (also records the launch plan)
    io = {k: np.ascontiguousarray(v) for k, v in feeds.items()}
    outs = {v.name: np.zeros(v.shape, v.dtype) for v in net.outputs}
    io.update(outs)
    ex.invoke(io)
    assert np.isfinite(next(iter(outs.values()))).all()

    ex.replay(args.warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ex.replay(args.steps)  # ends with a wait on the plan's stream
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    value = batch * args.steps / elapsed

    # distribution of single replays (device time between events on the plan's stream)
    per_replay = np.sort(np.asarray(ex.replay_times_ns(3, min(args.steps, 200)))) / 1e6
    percentiles = {"p10": float(np.percentile(per_replay, 10)), "p50": float(np.percentile(per_replay, 50)),
                   "p90": float(np.percentile(per_replay, 90))}

    # Invoke as the reference defines it (host buffers in and out): PCIe-inclusive
    t0 = time.perf_counter()
    for _ in range(10):
        ex.invoke(io)
    invoke_ms = (time.perf_counter() - t0) / 10 * 1e3

    # per-kernel durations with hipEvent pairs on the plan's stream, same steps
    times = ex.profile(3, min(args.steps, 30))
    # group launches by the device kernel that runs them: a fused launch is served by the kernel of its
    # first member (MatMul, MatMul+bias and MatMul+bias+GELU are one MatmulKernel instantiation)
    by_kernel = {}
    by_launch_kind = {}
    for t in times:
        k = by_launch_kind.setdefault(t["kernel"], {"ns": 0.0, "bytes": 0.0, "flops": 0.0, "launches": 0})
        k["ns"] += t["ns"]
        k["bytes"] += t["bytes"]
        k["flops"] += t["flops"]
        k["launches"] += 1
        family = t["kernel"].split("+")[0]
        if family == "MatMulKernel" and "SoftmaxKernel" in t["kernel"]:
            family = "AttentionKernel"  # scores, softmax and context product in one launch: its own device kernel
        if family in ("TransposeKernel", "ReshapeKernel") and "+" in t["kernel"]:
            family = "ReshapeKernel"
        k = by_kernel.setdefault(family, {"ns": 0.0, "bytes": 0.0, "flops": 0.0, "launches": 0})
        k["ns"] += t["ns"]
        k["bytes"] += t["bytes"]
        k["flops"] += t["flops"]
        k["launches"] += 1
    dominant = max(by_kernel.items(), key=lambda kv: kv[1]["ns"])
    dname, d = dominant
    if d["flops"] > 0:
        achieved = d["flops"] / d["ns"] / 1e3  # flop/ns = GFLOP/s -> TFLOP/s
        default_workload = (args.config, args.layers, args.seq, args.executor) == ("bert_base", 12, 128, "plain_greedy") and \
            os.environ.get("FLUIDML_FUSE", "1") != "0"
        roofline = {"bound": "mfma", "kernel": dname + " (all launches of the contraction kernel, fused epilogues included)",
                    "achieved": achieved, "peak": FP32_MFMA_PEAK_TFLOPS,
                    "unit": "TFLOP/s", "frac": achieved / FP32_MFMA_PEAK_TFLOPS,
                    "traffic": traffic_from_summary() if default_workload and dname == "MatMulKernel" else None,
                    "traffic_source": TRAFFIC_SUMMARY + (" (rocprofv3 FETCH_SIZE + WRITE_SIZE per dispatch, scaled by the "
                                                         "identity-copy kernel's readings)" if default_workload else
                                                         " covers the default workload only: not measured for this one"),
                    "avg_launch_us": d["ns"] / d["launches"] / 1e3, "launches_per_step": d["launches"],
                    "flops_per_launch": d["flops"] / d["launches"]}
    else:
        achieved = d["bytes"] / d["ns"]  # B/ns = GB/s
        roofline = {"bound": "hbm", "kernel": dname, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                    "avg_launch_us": d["ns"] / d["launches"] / 1e3, "launches_per_step": d["launches"],
                    "bytes_per_launch": d["bytes"] / d["launches"]}
    # A dominant kernel that reaches less than 5 % of the matrix-core peak AND less than 5 % of the HBM peak is bound
    # by neither: its launches are too small to fill the chip for longer than it takes to start them (EfficientNet-B0:
    # 0.78 GFLOP over 77 launches).  Say so instead of quoting a fraction of a roofline that does not apply.
    if d["flops"] / d["ns"] / 1e3 / FP32_MFMA_PEAK_TFLOPS < 0.05 and d["bytes"] / d["ns"] / HBM_PEAK_GBS < 0.05:
        roofline["bound"] = "latency"
        roofline["note"] = (f"{d['launches']} launches x {d['ns'] / d['launches'] / 1e3:.2f} us: {d['flops'] / d['launches'] / 1e6:.1f} MFLOP and "
                            f"{d['bytes'] / d['launches'] / 1e3:.0f} KB per launch, under 5 % of the fp32 matrix-core peak and of the HBM peak; "
                            "`frac` is kept against the peak named in `unit` for comparison only")
    total_flops = sum(t["flops"] for t in times)
    total_bytes = sum(t["bytes"] for t in times)
    kernel_sum_ms = sum(t["ns"] for t in times) / 1e6

    if per_kernel:
        print(f"{'kernel':48s} {'launches':>8s} {'total us':>10s} {'avg us':>8s} {'GB/s':>9s} {'TFLOP/s':>8s}", file=sys.stderr)
        for name, k in sorted(by_launch_kind.items(), key=lambda kv: -kv[1]["ns"]):
            print(f"{name:48s} {k['launches']:8d} {k['ns'] / 1e3:10.1f} {k['ns'] / k['launches'] / 1e3:8.2f} "
                  f"{k['bytes'] / k['ns']:9.1f} {k['flops'] / k['ns'] / 1e3:8.2f}", file=sys.stderr)

    if per_launch:
        print(f"{'#':>4s} {'launch':60s} {'us':>9s} {'GB/s':>9s} {'TFLOP/s':>8s}", file=sys.stderr)
        for i, t in enumerate(times):
            print(f"{i:4d} {t['kernel'][:60]:60s} {t['ns'] / 1e3:9.2f} {t['bytes'] / t['ns']:9.1f} {t['flops'] / t['ns'] / 1e3:8.2f}",
                  file=sys.stderr)

    result = {
        "metric": "inferences/sec at BERT-base seq128 fp32 on 1 MI355X" if args.config == "bert_base"
        else f"inferences/sec at {args.config} fp32 on 1 MI355X",
        "value": value,
        "unit": "inferences/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "ms_per_step_percentiles": percentiles,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic: seeded weights (N(0,0.02) transformers, He-normal conv nets), seeded inputs of the configuration's shape",
        "config": {"workload": workload, "executor": args.executor, "graph_nodes": len(net.nodes),
                   "kernels_per_step": len(times), "launch": "captured hipGraph replay",
                   "side_branches": len(ex.plan()["regions"])},
        "roofline": roofline,
        "peak_hbm_bytes": {"arena": plan["arena_bytes"], "constants": plan["constant_bytes"],
                           "interface": plan["interface_bytes"], "private": ex.plan()["private_bytes"],
                           "total": ex.plan()["peak_device_bytes"]},
        "whole_graph": {"flops_per_step": total_flops, "algorithmic_bytes_per_step": total_bytes,
                        "tflops": total_flops / (ms_per_step * 1e-3) / 1e12,
                        "sum_of_kernel_ms": kernel_sum_ms, "invoke_with_host_copies_ms": invoke_ms,
                        "compile_s": compile_s},
    }
    return result, (net, feeds, batch, ex, io, outs)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", default="bert_base",
                    choices=["bert_base", "convbert_base", "gpt_neox", "efficientnet_b0", "vgg16_b1", "vgg16_b8"],
                    help="bert_base is the configuration the headline metric is quoted on")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--executor", default="plain_greedy", choices=["plain_linear", "plain_greedy", "dp_greedy"])
    ap.add_argument("--layers", type=int, default=12)
    ap.add_argument("--seq", type=int, default=128)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true",
                    help="default workload only: skip the `configs` key (the other configurations and the DP executor)")
    ap.add_argument("--cpu-sample-layers", type=int, default=3)
    ap.add_argument("--plan-json", default=None, metavar="PATH",
                    help="write the JSON of the benchmark configuration's compile there (decisions taken by timing included)")
    ap.add_argument("--per-kernel", action="store_true", help="also print a per-kernel table to stderr")
    ap.add_argument("--per-launch", action="store_true", help="also print every launch of one step, in order, to stderr")
    ap.add_argument("--bf16", action="store_true",
                    help="additionally run the opt-in bf16 contraction path and report its throughput and its "
                         "error against the fp32 result under \"bf16\" (the headline value stays fp32)")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MIB",
                    help="instead of the benchmark, launch the identity-copy kernel 3 times on a buffer of MIB MiB "
                         "(a kernel of known traffic, to scale profiler byte counters) and exit")
    ap.add_argument("--hbm-kernels", action="store_true",
                    help="instead of the benchmark, time every bandwidth-bound kernel class on 128-512 MiB of data "
                         "and print its achieved HBM GB/s (table on stderr, one JSON line on stdout)")
    ap.add_argument("--mfma-kernels", action="store_true",
                    help="instead of the benchmark, time the contraction kernel (MatMul, 3x3 convolution) on problems of "
                         "growing size and print its TFLOP/s against the fp32 MFMA peak")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (the reference has no multi-device path); use --gpus 1")

    import numpy as np
    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback")
    from fluidml_amd import fluidml, models

    if args.mfma_kernels:
        from bench_sweeps import mfma_sweep

        print(json.dumps(mfma_sweep.run(out=sys.stderr)))
        return
    if args.hbm_kernels:
        from bench_sweeps import hbm_sweep

        print(json.dumps(hbm_sweep.run(out=sys.stderr)))
        return
    if args.copy_calibration:
        import ctypes

        from fluidml_amd import cabi

        n = args.copy_calibration * (1 << 20) // 4
        src = torch.ones(n, dtype=torch.float32, device="cuda")
        dst = torch.zeros(n, dtype=torch.float32, device="cuda")
        ts = cabi.make_tensor(src.data_ptr(), cabi.FL_FLOAT32, [n], [1])
        td = cabi.make_tensor(dst.data_ptr(), cabi.FL_FLOAT32, [n], [1])
        torch.cuda.synchronize()
        for _ in range(3):
            cabi.call("dropout", ctypes.byref(ts), ctypes.byref(td), None)
        torch.cuda.synchronize()
        assert bool((dst == 1).all())
        print(json.dumps({"copy_calibration_bytes_read": n * 4, "copy_calibration_bytes_written": n * 4}))
        return

    result, (net, feeds, batch, ex, io, outs) = measure(args, args.config, args.executor, args.per_kernel, args.per_launch)
    default_run = (args.config, args.layers, args.seq, args.executor) == ("bert_base", 12, 128, "plain_greedy")
    if default_run and not args.no_configs:
        # the other configurations and the DP executor, GPU legs only (no CPU baseline), fewer steps
        import types

        short = types.SimpleNamespace(**{**vars(args), "steps": max(20, args.steps // 4), "warmup": max(5, args.warmup // 4),
                                         "plan_json": None})
        result["configs"] = {}
        del ex
        for name, executor in [("bert_base", "dp_greedy"), ("convbert_base", "plain_greedy"), ("gpt_neox", "plain_greedy"),
                               ("efficientnet_b0", "plain_greedy"), ("vgg16_b1", "plain_greedy"), ("vgg16_b8", "plain_greedy")]:
            print(f"[bench] {name} ({executor}) ...", file=sys.stderr, flush=True)
            r, keep = measure(short, name, executor)
            del keep
            key = name if executor == "plain_greedy" else f"{name}:{executor}"
            result["configs"][key] = {"value": r["value"], "unit": r["unit"], "ms_per_step": r["ms_per_step"], "steps": r["steps"],
                                      "kernels_per_step": r["config"]["kernels_per_step"],
                                      "side_branches": r["config"]["side_branches"],
                                      "roofline": {k: r["roofline"][k] for k in ("bound", "kernel", "achieved", "peak", "unit", "frac")},
                                      "whole_graph_tflops": r["whole_graph"]["tflops"],
                                      "peak_hbm_bytes": r["peak_hbm_bytes"]}
        ex = None
    if args.bf16:
        ref_out = {k: v.copy() for k, v in outs.items()}
        ex.invoke(io)
        ref_out = {k: outs[k].copy() for k in outs}
        os.environ["FLUIDML_BF16"] = "1"
        try:
            with tempfile.TemporaryDirectory() as tmp:
                path = net.save(os.path.join(tmp, args.config + ".onnx"))
                ex16 = getattr(fluidml.Executor, "make_" + args.executor)(args.config + "_bf16", 1)
                ex16.compile(path)
        finally:
            os.environ["FLUIDML_BF16"] = "0"
        ex16.invoke(io)
        got = {k: outs[k].copy() for k in outs}
        ex16.replay(args.warmup)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ex16.replay(args.steps)
        torch.cuda.synchronize()
        el = time.perf_counter() - t0
        name = next(iter(got))
        err = np.abs(got[name].astype(np.float64) - ref_out[name].astype(np.float64))
        result["bf16"] = {"value": batch * args.steps / el, "unit": "inferences/s", "ms_per_step": el / args.steps * 1e3,
                          "max_abs_err_vs_fp32": float(err.max()),
                          "max_abs_err_over_max_abs_output": float(err.max() / np.abs(ref_out[name]).max()),
                          "mean_abs_err_vs_fp32": float(err.mean()),
                          "note": "operands of the MatMul, Gemm and non-depthwise Conv launches that run on the matrix cores "
                                  "(3x3 Conv on the staged-patch kernel included) rounded to bf16 (nearest even), fp32 accumulation; "
                                  "the weight-streaming Gemm kernels, depthwise Conv and pointwise Conv with a gate or skip "
                                  "operand stay fp32"}
    if not args.no_cpu_baseline:
        if args.config == "bert_base":
            result["cpu_baseline"] = cpu_baseline(args.layers, min(args.cpu_sample_layers, args.layers), args.seq)
        elif batch > 1:
            # the scalar loop nests take the same time for every image of a batch: time one image
            one = {k: np.ascontiguousarray(v[:1]) for k, v in feeds.items()}
            result["cpu_baseline"] = cpu_baseline_whole(models.vgg16(1), one, 1)
            result["cpu_baseline"]["sample"] = (f"one whole forward pass of ONE image of the batch of {batch} (the batch-1 graph) on 1 of "
                                                f"{host_cores()} host cores; " + ORACLE_CAVEAT)
        else:
            result["cpu_baseline"] = cpu_baseline_whole(net, feeds, batch)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
