"""Throughput and per-step profile of an ONNX network on the HIP executor: the twin of the reference's
`profile_net` binary (kn-cuda-eval/src/bin/profile_net.rs), same flags and the same measurement protocol.

    python -m kyanite_amd.profile_net [-b BATCH] [-o] [-p] [-c] [-d DEVICE] [-s] [-n N] [--graph] model.onnx

  -b  batch size; below 1 runs the sweep over 1 ... 2048 (profile_net.rs:36-37, :118-144)
  -o  optimize the graph first        -p  print the graph and the planned executor instead of running
  -c  (CPU timing lives in bench.py)   -s  skip the host copies (run_async only)
  -n  iterations (default 100); warmup is max(1, n / 10) evaluations, as in the reference
  --graph  replay the launch list as one HIP graph
Every step of the profile carries its achieved TFLOP/s (conv / matmul) and GB/s over algorithmic bytes.
"""
import argparse
import sys
import time

TEST_BATCH_SIZES = [1, 2, 3, 4, 8, 16, 32, 64, 128, 256, 512, 1024, 2048]
TEST_BATCH_ITERATIONS = [100, 100, 100, 100, 100, 100, 100, 100, 50, 25, 12, 8, 4]
DEFAULT_ITERATIONS = 100


def profile_single(device, graph, batch, n, skip_io, use_graph):
    from . import HipExecutor

    ex = HipExecutor(device, graph, batch)
    ex.set_graph_mode(use_graph)
    inputs = graph.dummy_zero_inputs(batch)
    print("Warmup")
    for _ in range(max(1, n // 10)):
        ex.evaluate(inputs)
    print("Throughput test")
    start = time.perf_counter()
    for _ in range(n):
        if skip_io:
            ex.run_async()
        else:
            ex.evaluate(inputs)
    if skip_io:
        ex.synchronize()
    delta = time.perf_counter() - start
    print("Profiling")
    ex.set_profile(True)
    ex.evaluate(inputs)
    profile = ex.last_profile()
    print(profile)
    print("Roofline per step (algorithmic work / measured launch time):")
    for i, seconds in enumerate(profile.step_seconds):
        flops, nbytes = ex.step_work(i)
        if seconds <= 0:
            continue
        line = f"  {i:4d} {seconds * 1e3:10.4f} ms {nbytes / seconds / 1e9:9.1f} GB/s"
        if flops > 0:
            line += f" {flops / seconds / 1e12:9.2f} TFLOP/s"
        print(line + "  " + ex.step_str(i)[:100])
    print(f"Throughput: {batch * n / delta} evals/s")


def profile_sweep(device, graph):
    from . import HipExecutor

    result = []
    for batch, iterations in zip(TEST_BATCH_SIZES, TEST_BATCH_ITERATIONS):
        print(f"Testing batch size {batch} with {iterations} iterations")
        ex = HipExecutor(device, graph, batch)
        inputs = graph.dummy_zero_inputs(batch)
        for _ in range(max(1, iterations // 10)):
            ex.evaluate(inputs)
        start = time.perf_counter()
        for _ in range(iterations):
            ex.evaluate(inputs)
        delta = time.perf_counter() - start
        throughput = batch * iterations / delta
        print(f"  throughput: {throughput} evals/s")
        result.append((batch, throughput))
    print(result)


def profile_cpu(graph, batch, n):
    raise SystemExit("--cpu: this package ships no CPU evaluator (the one in this repository is test infrastructure); "
                     "`python bench.py` times it on the benchmark graphs and reports it as cpu_baseline")


def main(argv=None):
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("-b", "--batch-size", type=int, default=0)
    parser.add_argument("-o", "--optimize", action="store_true")
    parser.add_argument("-p", "--print", action="store_true", dest="print_")
    parser.add_argument("-c", "--cpu", action="store_true")
    parser.add_argument("-d", "--device", type=int, default=0)
    parser.add_argument("-s", "--skip-io", action="store_true")
    parser.add_argument("-n", type=int, default=None)
    parser.add_argument("--graph", action="store_true")
    parser.add_argument("path")
    args = parser.parse_args(argv)

    from . import HipDevice, HipExecutor, optimize_graph
    from .onnx import load_graph_from_onnx_path

    n = args.n if args.n is not None else DEFAULT_ITERATIONS
    warnings = []
    loaded = load_graph_from_onnx_path(args.path)
    if args.optimize:
        graph = optimize_graph(loaded)
    else:
        warnings.append("Warning: not optimizing graph")
        print(warnings[-1], file=sys.stderr)
        graph = loaded

    if args.print_:
        print(graph)
        if not args.cpu:
            if args.batch_size < 1:
                raise SystemExit("Error: must set batch size")
            print(HipExecutor(args.device, graph, args.batch_size, plan_only=True))
    elif args.cpu:
        profile_cpu(graph, args.batch_size, n)
    else:
        device = HipDevice(args.device)
        if args.batch_size < 1:
            profile_sweep(device, graph)
        else:
            profile_single(device, graph, args.batch_size, n, args.skip_io, args.graph)
    for w in warnings:
        print(w, file=sys.stderr)


if __name__ == "__main__":
    main()
