#!/usr/bin/env python3
"""Benchmark of the HIP executor on the bandwidth-bound operator graphs (BASELINE.json configs[1]).

One step = one evaluation (`run_async`, device only, inputs resident in HBM) of each of the four graphs:
  (a) y = tanh-GELU(x * a + b) + r on [64, 1024, 1024] with a, b broadcast from [1024]
  (b) softmax over the last axis of [32, 16, 512, 512]
  (c) layernorm over the last axis of [8192, 4096] with gamma / beta, eps 1e-5
  (d) sum over axis 1 of [4096, 8192]
The metric is graph evaluations per second; the JSON line also carries, for every graph's kernel, the achieved
HBM bandwidth (algorithmic bytes / event-timed launch duration) against the 8 TB/s peak, and the oracle
(`cpu_eval_graph` restatement) timed on one host core on a bounded sample of the same workload.

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

# rows of the leading axis used for the CPU baseline sample and for the parity check of each graph; the full
# shapes take about ten seconds on one core, so the sample is the whole workload
CPU_SAMPLE_ROWS = {"2a_fused_gelu_chain": 64, "2b_softmax": 32, "2c_layernorm_affine": 8192, "2d_reduce_sum": 4096}


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=50)
    parser.add_argument("--warmup", type=int, default=5)
    parser.add_argument("--no-cpu-baseline", action="store_true", help="skip the timed CPU oracle leg")
    parser.add_argument("--kernel-iters", type=int, default=20, help="launches per kernel for the roofline timing")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on exactly one GPU (one executor, one arena, no collectives); "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        sys.exit(2)

    import numpy as np

    from kyanite_amd import HipDevice, HipExecutor
    from kyanite_amd.configs import BANDWIDTH_CONFIGS

    device = HipDevice(0)
    executors = {}
    meta = {}
    t_setup = time.time()
    for name, (builder, shape) in BANDWIDTH_CONFIGS.items():
        graph, make_inputs, algo_bytes = builder(seed=0, shape=shape)
        ex = HipExecutor(device, graph, 0)
        inputs = make_inputs()
        for i, x in enumerate(inputs):
            ex.upload_input(i, x)
        rows = min(CPU_SAMPLE_ROWS[name], shape[0])
        meta[name] = {"graph_builder": builder, "shape": shape, "algo_bytes": algo_bytes, "rows": rows,
                      "sample_inputs": inputs if rows == shape[0] else [x[:rows].copy() for x in inputs]}
        del inputs
        executors[name] = ex
        print(f"[bench] prepared {name} {list(shape)}: {ex.step_count()} step(s): "
              f"{'; '.join(ex.step_str(i) for i in range(ex.step_count()))}", file=sys.stderr, flush=True)
    print(f"[bench] setup took {time.time() - t_setup:.1f} s", file=sys.stderr, flush=True)

    def step():
        for ex in executors.values():
            ex.run_async()

    def sync():
        for ex in executors.values():
            ex.synchronize()

    for _ in range(args.warmup):
        step()
    sync()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    sync()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    evals_per_s = len(executors) * args.steps / elapsed

    # per-kernel roofline: event-timed launches on the executor's own stream
    kernels = {}
    for name, ex in executors.items():
        ex.time_runs(3)
        ms = ex.time_runs(args.kernel_iters) / args.kernel_iters
        gbs = meta[name]["algo_bytes"] / (ms * 1e-3) / 1e9
        kernels[name] = {"steps": ex.step_kinds(), "avg_ms": round(ms, 5), "algorithmic_bytes": meta[name]["algo_bytes"],
                         "achieved_gbs": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4)}
    dominant = max(kernels, key=lambda k: kernels[k]["avg_ms"])

    # parity spot check + CPU baseline on a bounded sample (the oracle is the checker and the timed baseline)
    cpu_baseline = None
    if not args.no_cpu_baseline:
        from oracle import cpu_eval_graph
        cpu_seconds_full = 0.0
        sample_desc = []
        for name, ex in executors.items():
            m = meta[name]
            rows = m["rows"]
            sample_shape = (rows,) + tuple(m["shape"][1:])
            graph, _, _ = m["graph_builder"](seed=0, shape=sample_shape)
            t = time.perf_counter()
            expected = cpu_eval_graph(graph, 0, m["sample_inputs"])
            dt = time.perf_counter() - t
            cpu_seconds_full += dt * (m["shape"][0] / rows)
            sample_desc.append(f"{name}: first {rows} of {m['shape'][0]} rows in {dt:.2f} s")
            actual = ex.download_output(0, rows)
            e64, a64 = expected[0].astype(np.float64), actual.astype(np.float64)
            floor = 0.1 * np.sqrt(np.mean(e64 * e64))
            err = float(np.max(np.abs(a64 - e64) / np.maximum(np.abs(e64), floor)))
            kernels[name]["max_rel_err_vs_oracle"] = float(f"{err:.3e}")
            if not err <= 1e-4:
                print(f"[bench] PARITY FAILURE on {name}: max relative error {err:.3e}", file=sys.stderr)
                sys.exit(1)
        cpu_baseline = {"value": round(len(executors) / cpu_seconds_full, 4), "unit": "graph evals/s", "cores": 1,
                        "kind": "port",
                        "sample": "oracle (C++ restatement of cpu_eval_graph) timed on leading-axis slices and scaled "
                                  "linearly to the full shapes; " + "; ".join(sample_desc)}

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
                               "layernorm-affine [8192,4096] + sum-reduce [4096,8192], one evaluation each per step",
                   "inputs_resident_in_hbm": True},
        "roofline": {"bound": "hbm", "kernel": dominant, "achieved": dom["achieved_gbs"], "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": dom["frac"], "traffic": None},
        "kernels": kernels,
        "cpu_baseline": cpu_baseline,
        "device": device.name(),
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
