#!/usr/bin/env python3
"""Benchmark of the HIP executor. One JSON line per run.

Default (`--workload all`): every configuration of BASELINE.json in one process, one JSON line. The top level of
the line is the `bandwidth` workload (configs[1], the configuration the metric is quoted on; `--steps` and
`--warmup` apply to it); `configs` carries one entry per configuration with its step time, roofline entry of the
dominant kernel (HBM or MFMA fraction), the matmul / conv total against the MFMA peak, the parity result against
the oracle and the CPU baseline.

`bandwidth` (configs[1]): one step = one `run_async` (device only, inputs resident in HBM) of ONE executor whose
graph holds the four operator graphs side by side, so the four kernels run back to back on one stream:
  (a) y = tanh-GELU(x * a + b) + r on [64, 1024, 1024] with a, b broadcast from [1024]
  (b) softmax over the last axis of [32, 16, 512, 512]
  (c) layernorm over the last axis of [8192, 4096] with gamma / beta, eps 1e-5
  (d) sum over axis 1 of [4096, 8192]
The metric is graph evaluations per second (four per step). The line also carries, for every kernel, the achieved
HBM bandwidth (algorithmic bytes / launch duration measured with HIP events on the executor's stream) against the
8 TB/s peak, and the oracle (`cpu_eval_graph` restatement) timed on one host core.

The other workloads run one of the remaining configurations the same way (one step = one evaluation of the graph):
  --workload mlp     configs[0]  tiny MLP, batch 8 (launch latency)
  --workload resnet  configs[2]  AlphaZero style ResNet tower, f32, batch 1024
  --workload llama   configs[3]  2 layer LLaMA style decoder, f16, sequence 512
  --workload unet    configs[4]  Stable-Diffusion style UNet block, f32, batch 2
For these the roofline entry is the kernel family with the largest share of the step (identical launches are
averaged), against the MFMA peak when it is a matmul / conv and against the HBM peak otherwise; the parity check
and the CPU baseline use a bounded sample of the same workload that the oracle finishes in under a minute (stated
in `cpu_baseline.sample`), chosen so that the GPU result at full size must reproduce it.

Parity follows oracle/parity.py: bit-exact where IEEE fixes the result, 1e-4 (f32) / 2e-2 (f16) with a floor of
1e-3 rms, and for outputs that sum K terms the rule that the GPU result is no further from an f64 evaluation than
the oracle is. A failed check ends the run with exit status 1 and no JSON line.

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"f32": 157.3, "f16": 2500.0}

# HBM bytes per launch are not measured by this script (that takes two `rocprofv3 --pmc` runs); the counter results
# for these kernels are kept in this file of the repository
TRAFFIC_PROFILE = "profiles/bandwidth_graphs_counters.md"


def log(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def check_parity(graph, batch, inputs, expected, actual, what):
    """The rules of oracle/parity.py; returns a summary for the JSON line, ends the run when a rule fails."""
    from oracle.parity import check_outputs
    records = []
    try:
        check_outputs(graph, batch, inputs, expected, actual, what, records)
    except AssertionError as failure:
        log(f"PARITY FAILURE: {failure}")
        sys.exit(1)
    summary = {"rules": sorted({r["rule"] for r in records})}
    errs = [r["err"] for r in records if "err" in r]
    if errs:
        summary["max_rel_err_floor_1e-3_rms"] = float(f"{max(errs):.3e}")
    acc = [r for r in records if r["rule"] == "accumulated"]
    if acc:
        worst = max(acc, key=lambda r: r["gpu_max"])
        summary["accumulated"] = {
            "terms_per_sum": worst["k"], "floor_rms_fraction": float(f"{worst['floor_k']:.3g}"),
            "max_rel_err_with_that_floor": float(f"{max(r['err_k'] for r in acc):.3e}"),
            "gpu_vs_f64_max": float(f"{worst['gpu_max']:.3e}"), "oracle_vs_f64_max": float(f"{worst['oracle_max']:.3e}"),
            "gpu_vs_f64_rms": float(f"{worst['gpu_rms']:.3e}"), "oracle_vs_f64_rms": float(f"{worst['oracle_rms']:.3e}")}
    return summary


def timed_steps(ex, steps, warmup):
    for _ in range(warmup):
        ex.run_async()
    ex.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        ex.run_async()
    ex.synchronize()
    return time.perf_counter() - t0


def per_step_seconds(ex, iters):
    """Average launch duration of every step: HIP events around each launch, on the stream the kernels run on."""
    import numpy as np
    ex.set_profile(True)
    per_step = np.zeros(ex.step_count())
    # (one untimed pass first: a small plan runs as one fused kernel otherwise, so this may be the first launch of its
    # step kernels, which loads their code)
    ex.run_async()
    for _ in range(iters):
        ex.run_async()
        per_step += np.asarray(ex.last_profile().step_seconds)
    ex.set_profile(False)
    return per_step / iters


# ------------------------------------------------------------------------------------------------ bandwidth graphs

def run_bandwidth(args, device, steps, warmup):
    import numpy as np

    from kyanite_amd import Graph, HipExecutor
    from kyanite_amd.configs import BANDWIDTH_CONFIGS

    t_setup = time.time()
    # one graph that holds the four operator graphs side by side
    combined = Graph()
    parts = []  # (name, sub graph, first input index, input count, algorithmic bytes, input factory)
    by_letter = {name[1]: name for name in BANDWIDTH_CONFIGS}
    for name in (by_letter[c] for c in args.order):
        builder, shape = BANDWIDTH_CONFIGS[name]
        sub, make_inputs, algo_bytes = builder(seed=0, shape=shape)
        first = len(combined.inputs())
        ins = [combined.input(sub[v].shape, sub[v].dtype) for v in sub.inputs()]
        outs = combined.call(sub, ins)
        assert len(outs) == 1
        combined.output(outs[0])
        parts.append((name, sub, first, len(ins), algo_bytes, make_inputs))
    ex = HipExecutor(device, combined, 0, preserve_inputs=True)
    kinds = ex.step_kinds()
    assert len(kinds) == len(parts), f"expected one kernel per graph, planned {kinds}"

    host_inputs = {}
    for name, sub, first, count, _, make_inputs in parts:
        inputs = make_inputs()
        for k, x in enumerate(inputs):
            ex.upload_input(first + k, x)
        host_inputs[name] = inputs
    for i in range(ex.step_count()):
        log(f"step {i}: {ex.step_str(i)}")
    log(f"setup took {time.time() - t_setup:.1f} s, arena {ex.mem_usage['arena_bytes'] / 2**20:.0f} MiB")

    if args.copy_probe:
        pg = Graph()
        px = pg.input([64, 1024, 1024])
        pg.output(pg.mul(px, pg.scalar(2.0)))
        probe = HipExecutor(device, pg, 0)
        probe.upload_input(0, np.ones((64, 1024, 1024), np.float32))
        probe.run_async()
        probe.synchronize()
        log(f"copy probe launched: {probe.step_str(0)}")
        del probe

    # (defaults long enough for the clocks to settle: the first few milliseconds of work on an idle chip run a few
    # percent slower)
    steps = steps if steps is not None else 200
    warmup = warmup if warmup is not None else 100
    elapsed = timed_steps(ex, steps, warmup)
    ms_per_step = elapsed / steps * 1e3
    evals_per_s = len(parts) * steps / elapsed

    per_step = per_step_seconds(ex, args.kernel_iters)
    kernels = {}
    for i, (name, _, _, _, algo_bytes, _) in enumerate(parts):
        ms = per_step[i] * 1e3
        gbs = algo_bytes / per_step[i] / 1e9
        kernels[name] = {"step": kinds[i], "avg_ms": round(ms, 5), "algorithmic_bytes": algo_bytes,
                         "achieved_gbs": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4)}
    dominant = max(kernels, key=lambda k: kernels[k]["avg_ms"])

    # ---- parity check + CPU baseline: the oracle evaluates the same four graphs on the same inputs, one core
    cpu_baseline = None
    if not args.no_cpu_baseline:
        from oracle import cpu_eval_graph
        cpu_seconds = 0.0
        sample_desc = []
        for i, (name, sub, _, _, _, _) in enumerate(parts):
            t = time.perf_counter()
            expected = cpu_eval_graph(sub, 0, host_inputs[name])
            dt = time.perf_counter() - t
            cpu_seconds += dt
            sample_desc.append(f"{name} {dt:.2f} s")
            # every output element of the full-size run
            kernels[name]["parity"] = check_parity(sub, 0, host_inputs[name], expected, [ex.download_output(i)], name)
            log(f"{name}: oracle {dt:.2f} s, parity {kernels[name]['parity']}")
        cpu_baseline = {"value": round(len(parts) / cpu_seconds, 4), "unit": "graph evals/s", "cores": 1, "kind": "port",
                        "sample": "oracle (C++ restatement of cpu_eval_graph, single thread) on the whole workload, one "
                                  "evaluation of each graph at full shape: " + ", ".join(sample_desc)}

    dom = kernels[dominant]
    return {
        "metric": "graph evals/sec at 1 GPU (bandwidth-bound op graphs 2a-2d, device only)",
        "value": round(evals_per_s, 2),
        "unit": "graph evals/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "BASELINE configs[1]: fused GELU chain [64,1024,1024] + softmax [32,16,512,512] + "
                               "layernorm-affine [8192,4096] + sum-reduce [4096,8192]; one step evaluates each graph "
                               "once, back to back on one stream",
                   "inputs_resident_in_hbm": True},
        "roofline": {"bound": "hbm", "kernel": f"{dominant} ({dom['step']})", "achieved": dom["achieved_gbs"],
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": dom["frac"], "traffic": None,
                     "traffic_note": f"not measured in this run; counter runs of the same kernels: {TRAFFIC_PROFILE}"},
        "kernels": kernels,
        "cpu_baseline": cpu_baseline,
        "device": device.name(),
    }


# ------------------------------------------------------------------------------------------------ whole-model graphs

def kernel_table(ex, per_step):
    """Identical launches (same step description apart from the value id) grouped into one entry."""
    groups = {}
    for i in range(ex.step_count()):
        sig = re.sub(r" value=\d+", "", ex.step_str(i))
        sig = re.sub(r' id="[^"]*"', "", sig)
        flops, nbytes = ex.step_work(i)
        grp = groups.setdefault(sig, {"launches": 0, "total_s": 0.0, "flops": flops, "bytes": nbytes})
        grp["launches"] += 1
        grp["total_s"] += float(per_step[i])
    table = []
    for sig, grp in groups.items():
        avg = grp["total_s"] / grp["launches"]
        f16 = " f16 " in sig or sig.endswith(" f16")
        entry = {"kernel": sig, "launches": grp["launches"], "avg_ms": round(avg * 1e3, 5),
                 "share": 0.0, "total_ms": round(grp["total_s"] * 1e3, 5)}
        if grp["flops"] > 0:
            tf = grp["flops"] / avg / 1e12
            peak = MFMA_PEAK_TFLOPS["f16" if f16 else "f32"]
            entry.update({"flops": grp["flops"], "achieved_tflops": round(tf, 2), "mfma_frac": round(tf / peak, 4),
                          "mfma_peak_tflops": peak})
        gbs = grp["bytes"] / avg / 1e9
        entry.update({"algorithmic_bytes": grp["bytes"], "achieved_gbs": round(gbs, 1), "hbm_frac": round(gbs / HBM_PEAK_GBS, 4)})
        table.append(entry)
    total = sum(e["total_ms"] for e in table) or 1.0
    for e in table:
        e["share"] = round(e["total_ms"] / total, 4)
    table.sort(key=lambda e: -e["total_ms"])
    return table


def roofline_of(entry):
    # a matmul / conv is priced against the matrix cores unless its arithmetic intensity puts it under the HBM roof
    if "achieved_tflops" in entry and entry["mfma_frac"] >= entry["hbm_frac"]:
        return {"bound": "mfma", "kernel": entry["kernel"], "achieved": entry["achieved_tflops"],
                "peak": entry["mfma_peak_tflops"], "unit": "TFLOP/s", "frac": entry["mfma_frac"], "traffic": None}
    return {"bound": "hbm", "kernel": entry["kernel"], "achieved": entry["achieved_gbs"], "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": entry["hbm_frac"], "traffic": None}


def run_model(args, device, workload, steps, warmup):
    import numpy as np

    from kyanite_amd import HipExecutor
    from kyanite_amd import configs

    t_setup = time.time()
    dtype = "f32"
    if workload == "mlp":
        batch = 8
        graph, inputs = configs.build_tiny_mlp(seed=0, batch=batch)
        flops = 2 * batch * (16 * 32 + 32 * 10)
        desc = "BASELINE configs[0]: tiny MLP 16->32->10 with softmax, f32, batch 8"
        default_steps, default_warmup = 5000, 2000
    elif workload == "resnet":
        batch = 1024
        graph, make_inputs, flop_per_pos = configs.build_resnet_tower(seed=0)
        inputs = make_inputs(batch)
        flops = flop_per_pos * batch
        desc = "BASELINE configs[2]: AlphaZero style ResNet tower (10 blocks x 128 channels on 8x8, policy + value heads), f32, batch 1024"
        default_steps, default_warmup = 50, 20
    elif workload == "llama":
        batch = 0
        graph, make_inputs, flops = configs.build_llama(seed=0)
        inputs = make_inputs()
        dtype = "f16"
        desc = ("BASELINE configs[3]: 2 layer LLaMA style decoder, d_model 4096, 32 heads, FFN 11008, f16 weights and "
                "activations with f32 accumulation, batch 1, prefill of 512 tokens")
        default_steps, default_warmup = 100, 60
    elif workload == "unet":
        batch = 0
        graph, make_inputs, flops = configs.build_unet_block(seed=0)
        inputs = make_inputs()
        desc = ("BASELINE configs[4]: Stable-Diffusion style UNet block (ResBlock 320 channels at 64x64 + spatial "
                "transformer with self / cross attention and GEGLU), f32, batch 2")
        default_steps, default_warmup = 60, 30
    else:
        raise SystemExit(f"unknown workload {workload}")
    log(f"graph built in {time.time() - t_setup:.1f} s")

    ex = HipExecutor(device, graph, batch, preserve_inputs=True)
    for k, x in enumerate(inputs):
        ex.upload_input(k, x)
    log(f"setup took {time.time() - t_setup:.1f} s, {ex.step_count()} steps, arena {ex.mem_usage['arena_bytes'] / 2**20:.0f} MiB")

    # (defaults long enough for the clocks to settle: the first few milliseconds of work on an idle chip run up to a
    # tenth slower)
    steps = steps if steps is not None else default_steps
    warmup = warmup if warmup is not None else default_warmup
    elapsed = timed_steps(ex, steps, warmup)
    ms_per_step = elapsed / steps * 1e3
    evals_per_s = steps / elapsed

    per_step = per_step_seconds(ex, min(args.kernel_iters, 5))
    table = kernel_table(ex, per_step)
    for e in table[:12]:
        log(f"{e['share'] * 100:5.1f}%  {e['launches']:3d} x {e['avg_ms']:9.4f} ms  "
            f"{e.get('achieved_tflops', 0):8.2f} TFLOP/s  {e['achieved_gbs']:8.1f} GB/s  {e['kernel'][:110]}")
    extra = {}

    # ---- parity on a bounded sample the full-size run must reproduce, and the same sample as CPU baseline
    cpu_baseline = None
    if not args.no_cpu_baseline:
        from oracle import cpu_eval_graph
        gpu_outputs = [ex.download_output(i) for i in range(len(ex.output_info))]
        if workload == "mlp":
            n = 1000
            t = time.perf_counter()
            for _ in range(n):
                expected = cpu_eval_graph(graph, batch, inputs)
            cpu_seconds = (time.perf_counter() - t) / n
            sample_graph, sample_batch, sample_inputs, sample_outputs = graph, batch, inputs, gpu_outputs
            cpu_evals = 1.0 / cpu_seconds
            sample = f"{n} evaluations of the whole graph at batch 8 ({cpu_seconds * 1e6:.1f} us each)"
        elif workload == "resnet":
            rows = args.resnet_rows  # positions are independent of each other: the first rows of the batch must match
            sample_graph, sample_batch, sample_inputs = graph, rows, [x[:rows] for x in inputs]
            t = time.perf_counter()
            expected = cpu_eval_graph(sample_graph, sample_batch, sample_inputs)
            cpu_seconds = time.perf_counter() - t
            sample_outputs = [g[:rows] for g in gpu_outputs]
            cpu_evals = rows / cpu_seconds / batch
            sample = (f"the first {rows} of the 1024 positions ({cpu_seconds:.2f} s), scaled to evaluations of 1024 "
                      f"positions; the GPU's first {rows} rows at batch 1024 are checked against them")
        elif workload == "llama":
            # causal attention: the first tokens do not depend on the later ones; 128 tokens span two key blocks of
            # the fused attention kernel and rows of every wave of a matmul tile
            rows = args.llama_rows
            sample_graph, _, _ = configs.build_llama(seed=0, seq=rows)
            sample_batch, sample_inputs = 0, [inputs[0][:, :rows]]
            t = time.perf_counter()
            expected = cpu_eval_graph(sample_graph, 0, sample_inputs)
            cpu_seconds = time.perf_counter() - t
            sample_outputs = [gpu_outputs[0][:, :rows]]
            cpu_evals = rows / cpu_seconds / 512
            sample = (f"the same decoder on the first {rows} of the 512 tokens ({cpu_seconds:.2f} s), scaled to "
                      f"evaluations of 512 tokens; by causality the GPU's first {rows} output rows at sequence 512 are "
                      "checked against them")
        else:
            # samples of the batch are independent: the first one at full resolution
            sample_graph, _, _ = configs.build_unet_block(seed=0, batch=1)
            sample_batch, sample_inputs = 0, [x[:1] for x in inputs]
            t = time.perf_counter()
            expected = cpu_eval_graph(sample_graph, 0, sample_inputs)
            cpu_seconds = time.perf_counter() - t
            sample_outputs = [gpu_outputs[0][:1]]
            cpu_evals = 1.0 / cpu_seconds / 2
            sample = (f"the first of the 2 samples at full resolution ({cpu_seconds:.2f} s), scaled to evaluations of "
                      "batch 2; the GPU's first sample at batch 2 is checked against it")
        log(f"oracle sample took {cpu_seconds:.2f} s")
        extra["parity"] = check_parity(sample_graph, sample_batch, sample_inputs, expected, sample_outputs, workload)
        log(f"parity {extra['parity']}")
        cpu_baseline = {"value": float(f"{cpu_evals:.4g}"), "unit": "graph evals/s", "cores": 1, "kind": "port",
                        "sample": "oracle (C++ restatement of cpu_eval_graph, single thread) on " + sample}

    if workload == "mlp":
        # one HIP graph launch per evaluation instead of one launch per step
        ex.set_graph_mode(True)
        dt = timed_steps(ex, steps, warmup) / steps
        extra["hip_graph_replay"] = {"ms_per_step": round(dt * 1e3, 5), "evals_per_s": round(1.0 / dt, 1)}
        ex.set_graph_mode(False)
        # the reference's executor contract includes the copies: time `evaluate` (H2D, launches, D2H) as well
        n = 2000
        for _ in range(20):
            ex.evaluate(inputs)
        t = time.perf_counter()
        for _ in range(n):
            ex.evaluate(inputs)
        dt = (time.perf_counter() - t) / n
        extra["evaluate_with_copies_us"] = round(dt * 1e6, 2)
        extra["evaluate_with_copies_evals_per_s"] = round(1.0 / dt, 1)

    mfma_s = sum(float(per_step[i]) for i in range(ex.step_count()) if ex.step_work(i)[0] > 0)
    mfma_flops = sum(ex.step_work(i)[0] for i in range(ex.step_count()))
    if mfma_s > 0:
        peak = MFMA_PEAK_TFLOPS[dtype]
        extra["matmul_conv_total"] = {"ms": round(mfma_s * 1e3, 4), "tflops": round(mfma_flops / mfma_s / 1e12, 2),
                                      "mfma_frac": round(mfma_flops / mfma_s / 1e12 / peak, 4)}
    result = {
        "metric": f"graph evals/sec at 1 GPU ({workload}, device only)",
        "value": round(evals_per_s, 3),
        "unit": "graph evals/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype,
        "data": "synthetic",
        "config": {"workload": desc, "inputs_resident_in_hbm": True, "flop_per_eval": flops,
                   "whole_graph_tflops": round(flops * evals_per_s / 1e12, 2)},
        "roofline": roofline_of(table[0]),
        "kernels": table[:16],
        "cpu_baseline": cpu_baseline,
        "device": device.name(),
    }
    result.update(extra)
    return result


WORKLOADS = {"mlp": "configs[0]", "bandwidth": "configs[1]", "resnet": "configs[2]", "llama": "configs[3]", "unet": "configs[4]"}


def summary_of(result):
    """What the `configs` table of the combined line keeps of one workload's result."""
    keep = ("metric", "value", "unit", "steps", "warmup", "ms_per_step", "dtype", "roofline", "matmul_conv_total", "parity",
            "cpu_baseline", "hip_graph_replay", "evaluate_with_copies_us", "evaluate_with_copies_evals_per_s")
    out = {k: result[k] for k in keep if k in result}
    out["workload"] = result["config"]["workload"]
    if "whole_graph_tflops" in result["config"]:
        out["whole_graph_tflops"] = result["config"]["whole_graph_tflops"]
    kernels = result.get("kernels")
    if isinstance(kernels, dict):
        out["kernels"] = kernels
    elif kernels:
        out["kernels"] = [{k: e[k] for k in ("kernel", "launches", "avg_ms", "share", "achieved_tflops", "mfma_frac", "achieved_gbs",
                                              "hbm_frac") if k in e} for e in kernels[:6]]
    return out


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=None, help="timed steps (default: 200 for the bandwidth graphs)")
    parser.add_argument("--warmup", type=int, default=None, help="untimed steps before them (default: 100 for the bandwidth graphs)")
    parser.add_argument("--workload", default="all", choices=["all", "bandwidth", "mlp", "resnet", "llama", "unet"],
                        help="`all` (default) runs the five configurations and reports the bandwidth graphs at the top "
                             "level, the others under `configs`; --steps / --warmup then apply to the bandwidth graphs")
    parser.add_argument("--no-cpu-baseline", action="store_true", help="skip the timed CPU oracle leg and parity check")
    parser.add_argument("--copy-probe", action="store_true",
                        help="also launch y = 2 * x on [64,1024,1024] once (a kernel of known traffic, 536,870,912 B, "
                             "to calibrate hardware counters against)")
    parser.add_argument("--order", default="abcd", help="order of the four graphs inside one step (letters a-d)")
    parser.add_argument("--kernel-iters", type=int, default=20, help="profiled runs for the per-kernel timing")
    parser.add_argument("--resnet-rows", type=int, default=64, help="positions of the ResNet batch the oracle evaluates")
    parser.add_argument("--llama-rows", type=int, default=128, help="leading tokens of the LLaMA prefill the oracle evaluates")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on exactly one GPU (one executor, one arena, no collectives); "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        sys.exit(2)

    from kyanite_amd import HipDevice

    device = HipDevice(0)
    if args.workload == "bandwidth":
        result = run_bandwidth(args, device, args.steps, args.warmup)
    elif args.workload != "all":
        result = run_model(args, device, args.workload, args.steps, args.warmup)
    else:
        import gc
        t0 = time.time()
        result = run_bandwidth(args, device, args.steps, args.warmup)
        table = {f"{WORKLOADS['bandwidth']} bandwidth": summary_of(result)}
        for name in ("mlp", "resnet", "llama", "unet"):
            gc.collect()
            log(f"---- {name} ({time.time() - t0:.0f} s so far)")
            table[f"{WORKLOADS[name]} {name}"] = summary_of(run_model(args, device, name, None, None))
        result["configs"] = dict(sorted(table.items()))
        result["config"]["also_run"] = "every other BASELINE configuration, see `configs`"
        log(f"all workloads took {time.time() - t0:.0f} s")
    print(json.dumps(result))


if __name__ == "__main__":
    main()
