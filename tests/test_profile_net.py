"""The `profile_net` twin (kn-cuda-eval/src/bin/profile_net.rs:42-198): `-p` prints the graph and the planned executor
without a device; with a device it runs warm-up, the throughput loop and a profiled evaluation."""
import os
import re

import pytest

from kyanite_amd import profile_net

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_print_plans_without_a_device(capsys):
    profile_net.main(["-o", "-p", "-b", "4", os.path.join(GOLDEN, "att-tiny.onnx")])
    out = capsys.readouterr().out
    assert "Graph" in out and "HipExecutor {" in out
    # the planned launch list of the optimized attention net: matmuls, a softmax and elementwise kernels
    assert "MatMul" in out and "steps: [" in out
    assert re.search(r"arena_bytes: \d+", out)


def test_print_needs_a_batch_size():
    with pytest.raises(SystemExit) as e:
        profile_net.main(["-p", os.path.join(GOLDEN, "att-tiny.onnx")])
    assert "batch size" in str(e.value)


def test_unoptimized_run_warns(capsys):
    profile_net.main(["-p", "-b", "2", os.path.join(GOLDEN, "simple-sttt-1x64.onnx")])
    assert "not optimizing graph" in capsys.readouterr().err


def test_cpu_flag_points_at_the_benchmark():
    with pytest.raises(SystemExit) as e:
        profile_net.main(["-c", "-b", "2", os.path.join(GOLDEN, "att-tiny.onnx")])
    assert "cpu_baseline" in str(e.value)


@pytest.mark.gpu
@pytest.mark.parametrize("flags", [[], ["-s"], ["--graph"]])
def test_run_on_the_device(flags, capsys, hip_device):
    profile_net.main(["-o", "-b", "4", "-n", "3", *flags, os.path.join(GOLDEN, "att-tiny.onnx")])
    out = capsys.readouterr().out
    assert "Warmup" in out and "Throughput test" in out and "Profiling" in out
    m = re.search(r"Throughput: ([0-9.e+]+) evals/s", out)
    assert m and float(m.group(1)) > 0
    # every step of the profile has a time and a roofline line
    assert len(re.findall(r"time\s+[0-9.]+ ms, step", out)) == len(re.findall(r"^\s+\d+\s+[0-9.]+ ms\s+[0-9.]+ GB/s", out, re.M))
    assert "total_gpu" in out
