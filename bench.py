#!/usr/bin/env python3
"""Benchmark of the HIP executor on the bandwidth-bound operator graphs (BASELINE.json configs[1]).

One step = one `run_async` (device only, inputs resident in HBM) of ONE executor whose graph holds the four
operator graphs side by side, so the four kernels run back to back on one stream:
  (a) y = tanh-GELU(x * a + b) + r on [64, 1024, 1024] with a, b broadcast from [1024]
  (b) softmax over the last axis of [32, 16, 512, 512]
  (c) layernorm over the last axis of [8192, 4096] with gamma / beta, eps 1e-5
  (d) sum over axis 1 of [4096, 8192]
The metric is graph evaluations per second (four per step). The JSON line also carries, for every kernel, the
achieved HBM bandwidth (algorithmic bytes / launch duration measured with HIP events on the executor's stream)
against the 8 TB/s peak, and the oracle (`cpu_eval_graph` restatement) timed on one host core.

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

# HBM bytes per launch measured with `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` (KiB per dispatch),
# each scaled by what the same counter reads for a kernel of known traffic (y = 2 * x on [64,1024,1024]:
# FETCH_SIZE reads 0.5 of the true bytes, WRITE_SIZE reads 1.0). Source: profiles/bandwidth_graphs_counters.md
MEASURED_TRAFFIC_BYTES = {
    "2a_fused_gelu_chain": 805_413_000,
    "2b_softmax": 1_073_707_700,
    "2c_layernorm_affine": 268_720_400,
    "2d_reduce_sum": 134_356_900,
}


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=50)
    parser.add_argument("--warmup", type=int, default=5)
    parser.add_argument("--no-cpu-baseline", action="store_true", help="skip the timed CPU oracle leg and parity check")
    parser.add_argument("--copy-probe", action="store_true",
                        help="also launch y = 2 * x on [64,1024,1024] once (a kernel of known traffic, 536,870,912 B, "
                             "to calibrate hardware counters against)")
    parser.add_argument("--order", default="abcd", help="order of the four graphs inside one step (letters a-d)")
    parser.add_argument("--kernel-iters", type=int, default=20, help="profiled runs for the per-kernel timing")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on exactly one GPU (one executor, one arena, no collectives); "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        sys.exit(2)

    import numpy as np

    from kyanite_amd import Graph, HipDevice, HipExecutor
    from kyanite_amd.configs import BANDWIDTH_CONFIGS

    device = HipDevice(0)
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
        print(f"[bench] step {i}: {ex.step_str(i)}", file=sys.stderr, flush=True)
    print(f"[bench] setup took {time.time() - t_setup:.1f} s, arena {ex.mem_usage['arena_bytes'] / 2**20:.0f} MiB",
          file=sys.stderr, flush=True)

    if args.copy_probe:
        pg = Graph()
        px = pg.input([64, 1024, 1024])
        pg.output(pg.mul(px, pg.scalar(2.0)))
        probe = HipExecutor(device, pg, 0)
        probe.upload_input(0, np.ones((64, 1024, 1024), np.float32))
        probe.run_async()
        probe.synchronize()
        print(f"[bench] copy probe launched: {probe.step_str(0)}", file=sys.stderr, flush=True)
        del probe

    # ---- the timed region: K steps between two synchronisations
    for _ in range(args.warmup):
        ex.run_async()
    ex.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        ex.run_async()
    ex.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    evals_per_s = len(parts) * args.steps / elapsed

    # ---- per-kernel launch durations: HIP events around every step, on the stream the kernels run on
    ex.set_profile(True)
    per_step = np.zeros(ex.step_count())
    for _ in range(args.kernel_iters):
        ex.run_async()
        per_step += np.asarray(ex.last_profile().step_seconds)
    ex.set_profile(False)
    per_step /= args.kernel_iters
    kernels = {}
    for i, (name, _, _, _, algo_bytes, _) in enumerate(parts):
        ms = per_step[i] * 1e3
        gbs = algo_bytes / per_step[i] / 1e9
        kernels[name] = {"step": kinds[i], "avg_ms": round(ms, 5), "algorithmic_bytes": algo_bytes,
                         "achieved_gbs": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4),
                         "traffic_bytes": MEASURED_TRAFFIC_BYTES.get(name)}
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
            actual = ex.download_output(i)
            e64, a64 = expected[0].astype(np.float64), actual.astype(np.float64)
            floor = 0.1 * np.sqrt(np.mean(e64 * e64))
            err = float(np.max(np.abs(a64 - e64) / np.maximum(np.abs(e64), floor)))
            kernels[name]["max_rel_err_vs_oracle"] = float(f"{err:.3e}")
            if not err <= 1e-4:
                print(f"[bench] PARITY FAILURE on {name}: max relative error {err:.3e}", file=sys.stderr)
                sys.exit(1)
        cpu_baseline = {"value": round(len(parts) / cpu_seconds, 4), "unit": "graph evals/s", "cores": 1, "kind": "port",
                        "sample": "oracle (C++ restatement of cpu_eval_graph, single thread) on the whole workload, one "
                                  "evaluation of each graph at full shape: " + ", ".join(sample_desc)}

    dom = kernels[dominant]
    result = {
        "metric": "graph evals/sec at 1 GPU (bandwidth-bound op graphs 2a-2d, device only)",
        "value": round(evals_per_s, 2),
        "unit": "graph evals/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
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
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": dom["frac"], "traffic": dom["traffic_bytes"]},
        "kernels": kernels,
        "cpu_baseline": cpu_baseline,
        "device": device.name(),
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
