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


def traffic_from_profile(kernel_name):
    """HBM bytes per launch of one of the bandwidth kernels as the committed counter summary states it: the row of its
    table `| kernel | reads (B) | writes (B) | HBM traffic per launch (B) | algorithmic bytes | ratio |` whose first
    cell ends in the graph's number ("2b"); None when the file or the row is missing."""
    tag = kernel_name.split("_")[0]
    try:
        with open(os.path.join(ROOT, TRAFFIC_PROFILE)) as f:
            for line in f:
                cells = [c.strip() for c in line.strip().strip("|").split("|")]
                if len(cells) == 6 and cells[0].endswith(" " + tag) and re.fullmatch(r"[\d,]+", cells[3]):
                    return int(cells[3].replace(",", ""))
    except OSError:
        pass
    return None


def log(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def elements_over_bar(expected, actual):
    """(elements whose relative error under the 1e-3 rms floor exceeds the bar of the dtype, elements compared)"""
    import numpy as np
    from oracle.parity import F16_MAX_REL, F32_MAX_REL, SMALL_FLOOR
    e = np.asarray(expected)
    bar = F16_MAX_REL if e.dtype == np.float16 else F32_MAX_REL
    e64 = e.astype(np.float64).reshape(-1)
    a64 = np.asarray(actual).astype(np.float64).reshape(-1)
    keep = np.isfinite(e64)
    e64, a64 = e64[keep], a64[keep]
    if e64.size == 0:
        return 0, 0
    floor = SMALL_FLOOR * float(np.sqrt(np.mean(e64 * e64)))
    rel = np.abs(a64 - e64) / np.maximum(np.abs(e64), max(floor, 1e-300))
    return int(np.count_nonzero(rel > bar)), int(e64.size)


def check_parity(graph, batch, inputs, expected, actual, what):
    """The rules of oracle/parity.py; returns a summary for the JSON line, ends the run when a rule fails."""
    import numpy as np
    from oracle.parity import check_outputs
    records = []
    try:
        check_outputs(graph, batch, inputs, expected, actual, what, records)
    except AssertionError as failure:
        log(f"PARITY FAILURE: {failure}")
        sys.exit(1)
    summary = {"rules": sorted({r["rule"] for r in records}), "elements_compared": int(sum(r["elements"] for r in records))}
    errs = [r["err"] for r in records if "err" in r]
    if errs:
        summary["max_rel_err_floor_1e-3_rms"] = float(f"{max(errs):.3e}")
        # the floor (fraction of the tensor's rms) at which every element would lie within the bar
        summary["floor_needed_rms_fraction"] = float(f"{max(r.get('floor_needed', 0.0) for r in records):.3e}")
        # how many elements, not only the worst one, lie outside the stated bar under the small floor
        over, floats = 0, 0
        for e, a in zip(expected, actual):
            if np.asarray(e).dtype.kind != "f":
                continue
            n_over, n = elements_over_bar(e, a)
            over += n_over
            floats += n
        summary["elements_over_bar_floor_1e-3_rms"] = over
        summary["fraction_over_bar"] = float(f"{over / max(floats, 1):.3e}")
    acc = [r for r in records if r["rule"] == "accumulated"]
    if acc:
        worst = max(acc, key=lambda r: r["gpu_max"])
        summary["accumulated"] = {
            "terms_per_sum": worst["k"], "floor_rms_fraction": float(f"{worst['floor_k']:.3g}"),
            "max_rel_err_with_that_floor": float(f"{max(r['err_k'] for r in acc):.3e}"),
            "gpu_vs_f64_max": float(f"{worst['gpu_max']:.3e}"), "oracle_vs_f64_max": float(f"{worst['oracle_max']:.3e}"),
            "gpu_vs_f64_rms": float(f"{worst['gpu_rms']:.3e}"), "oracle_vs_f64_rms": float(f"{worst['oracle_rms']:.3e}"),
            "agreement_rule_waived": bool(any(r.get("rule2_waived") for r in acc))}
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


def evaluate_with_copies(ex, inputs, n):
    """Wall clock of `evaluate` (host buffers in, host buffers out: staging copies, H2D, launches, D2H), timed like
    kn-cuda-eval/src/bin/profile_net.rs:146-180 times it: max(1, n / 10) untimed evaluations, then n."""
    out = ex.evaluate(inputs)  # the same output tensors every time, as executor.rs:117 hands them out
    for _ in range(max(1, n // 10)):
        ex.evaluate(inputs, out=out)
    t0 = time.perf_counter()
    for _ in range(n):
        ex.evaluate(inputs, out=out)
    dt = (time.perf_counter() - t0) / n
    return {"ms_per_eval": float(f"{dt * 1e3:.5g}"), "evals_per_s": float(f"{1.0 / dt:.5g}"), "evaluations": n,
            "input_bytes": int(sum(x.nbytes for x in inputs))}


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

    # the same step with the copies: `evaluate` of the combined graph from host buffers (1.3 GB in, 0.9 GB out)
    all_inputs = [x for name, *_ in parts for x in host_inputs[name]]
    with_copies = evaluate_with_copies(ex, all_inputs, 3)
    with_copies["graph_evals_per_s"] = float(f"{len(parts) * with_copies['evals_per_s']:.5g}")
    log(f"evaluate with copies: {with_copies}")

    dom = kernels[dominant]
    traffic = traffic_from_profile(dominant)
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
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": dom["frac"], "traffic": traffic,
                     "traffic_note": (f"HBM bytes per launch (FETCH_SIZE + WRITE_SIZE, calibrated on a copy kernel) from the "
                                      f"committed counter runs of this kernel, {TRAFFIC_PROFILE}; not measured in this run"
                                      if traffic is not None else
                                      f"not measured in this run; counter runs of the same kernels: {TRAFFIC_PROFILE}")},
        "kernels": kernels,
        "evaluate_with_copies": with_copies,
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
            sample_kind = "all"
            sample = f"{n} evaluations of the whole graph at batch 8 ({cpu_seconds * 1e6:.1f} us each)"
        elif workload == "resnet":
            # positions are independent of each other: any leading part of the batch must match; default all of it
            rows = args.resnet_rows or batch
            sample_graph, sample_batch, sample_inputs = graph, rows, [x[:rows] for x in inputs]
            t = time.perf_counter()
            expected = cpu_eval_graph(sample_graph, sample_batch, sample_inputs)
            cpu_seconds = time.perf_counter() - t
            sample_outputs = [g[:rows] for g in gpu_outputs]
            cpu_evals = rows / cpu_seconds / batch
            sample_kind = "all" if rows == batch else f"first {rows} of {batch} positions"
            sample = (f"all {batch} positions ({cpu_seconds:.2f} s for one evaluation)" if rows == batch else
                      f"the first {rows} of the {batch} positions ({cpu_seconds:.2f} s), scaled to evaluations of {batch} "
                      f"positions; the GPU's first {rows} rows at batch {batch} are checked against them")
        elif workload == "llama":
            # default: the whole prefill. With fewer rows: by causality the first tokens do not depend on the later ones
            rows = args.llama_rows or 512
            sample_graph = graph if rows == 512 else configs.build_llama(seed=0, seq=rows)[0]
            sample_batch, sample_inputs = 0, [inputs[0][:, :rows]]
            t = time.perf_counter()
            expected = cpu_eval_graph(sample_graph, 0, sample_inputs)
            cpu_seconds = time.perf_counter() - t
            sample_outputs = [gpu_outputs[0][:, :rows]]
            cpu_evals = rows / cpu_seconds / 512
            sample_kind = "all" if rows == 512 else f"first {rows} of 512 tokens"
            sample = (f"all 512 tokens ({cpu_seconds:.2f} s for one evaluation)" if rows == 512 else
                      f"the same decoder on the first {rows} of the 512 tokens ({cpu_seconds:.2f} s), scaled to "
                      f"evaluations of 512 tokens; by causality the GPU's first {rows} output rows at sequence 512 are "
                      "checked against them")
        else:
            # samples of the batch are independent; default both
            n = args.unet_samples or 2
            sample_graph = graph if n == 2 else configs.build_unet_block(seed=0, batch=n)[0]
            sample_batch, sample_inputs = 0, [x[:n] for x in inputs]
            t = time.perf_counter()
            expected = cpu_eval_graph(sample_graph, 0, sample_inputs)
            cpu_seconds = time.perf_counter() - t
            sample_outputs = [gpu_outputs[0][:n]]
            cpu_evals = n / cpu_seconds / 2
            sample_kind = "all" if n == 2 else f"first {n} of 2 samples"
            sample = (f"both samples at full resolution ({cpu_seconds:.2f} s for one evaluation)" if n == 2 else
                      f"the first of the 2 samples at full resolution ({cpu_seconds:.2f} s), scaled to evaluations of "
                      "batch 2; the GPU's first sample at batch 2 is checked against it")
        log(f"oracle sample took {cpu_seconds:.2f} s")
        extra["parity"] = check_parity(sample_graph, sample_batch, sample_inputs, expected, sample_outputs, workload)
        extra["parity"]["sample"] = sample_kind
        log(f"parity {extra['parity']}")
        cpu_baseline = {"value": float(f"{cpu_evals:.4g}"), "unit": "graph evals/s", "cores": 1, "kind": "port",
                        "sample": "oracle (C++ restatement of cpu_eval_graph, single thread) on " + sample}

    if workload == "mlp":
        # one HIP graph launch per evaluation instead of one launch per step
        ex.set_graph_mode(True)
        dt = timed_steps(ex, steps, warmup) / steps
        extra["hip_graph_replay"] = {"ms_per_step": round(dt * 1e3, 5), "evals_per_s": round(1.0 / dt, 1)}
        ex.set_graph_mode(False)

    # the reference's executor contract includes the copies: `evaluate` (staging, H2D, launches, D2H) next to the
    # device-only figure, for every configuration
    extra["evaluate_with_copies"] = evaluate_with_copies(ex, inputs, 2000 if workload == "mlp" else 20)
    log(f"evaluate with copies: {extra['evaluate_with_copies']}")

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
            "cpu_baseline", "hip_graph_replay", "evaluate_with_copies")
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


def compact_summary(entry):
    """One short flat record per configuration for the top level of the combined line: step time, throughput with and
    without copies, roofline fraction of the dominant kernel, matmul / conv total against the MFMA peak, parity."""
    out = {"ms_per_step": entry["ms_per_step"], "evals_per_s": entry["value"], "frac": entry["roofline"]["frac"],
           "bound": entry["roofline"]["bound"]}
    if "matmul_conv_total" in entry:
        out["mfma_frac_all_matmul_conv"] = entry["matmul_conv_total"]["mfma_frac"]
    if "evaluate_with_copies" in entry:
        out["ms_per_eval_with_copies"] = entry["evaluate_with_copies"]["ms_per_eval"]
    parity = entry.get("parity")
    kernels = entry.get("kernels")
    if parity is None and isinstance(kernels, dict):
        parts = [k["parity"] for k in kernels.values() if "parity" in k]
        if parts:
            parity = {"rules": sorted({r for p in parts for r in p["rules"]}), "sample": "all",
                      "elements_compared": sum(p["elements_compared"] for p in parts),
                      "max_rel_err_floor_1e-3_rms": max(p.get("max_rel_err_floor_1e-3_rms", 0.0) for p in parts)}
        out["hbm_frac_per_kernel"] = {name: k["frac"] for name, k in kernels.items()}
    if parity is not None:
        out["parity_rules"] = parity["rules"]
        out["parity_sample"] = parity.get("sample", "all")
        out["parity_elements"] = parity.get("elements_compared")
        if "max_rel_err_floor_1e-3_rms" in parity:
            out["parity_max_rel_err"] = parity["max_rel_err_floor_1e-3_rms"]
        if "fraction_over_bar" in parity:
            out["parity_fraction_over_bar"] = parity["fraction_over_bar"]
        if "floor_needed_rms_fraction" in parity:
            out["parity_floor_needed"] = parity["floor_needed_rms_fraction"]
    if entry.get("cpu_baseline"):
        out["cpu_evals_per_s"] = entry["cpu_baseline"]["value"]
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
    parser.add_argument("--resnet-rows", type=int, default=0,
                        help="leading positions of the ResNet batch the oracle evaluates (default 0: all 1024)")
    parser.add_argument("--llama-rows", type=int, default=0,
                        help="leading tokens of the LLaMA prefill the oracle evaluates (default 0: all 512)")
    parser.add_argument("--unet-samples", type=int, default=0,
                        help="leading samples of the UNet batch the oracle evaluates (default 0: both)")
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
        result["configs_summary"] = {name: compact_summary(entry) for name, entry in result["configs"].items()}
        result["config"]["also_run"] = "every other BASELINE configuration, see `configs`"
        log(f"all workloads took {time.time() - t0:.0f} s")
    print(json.dumps(result))


if __name__ == "__main__":
    main()
