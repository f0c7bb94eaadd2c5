"""HIP graph replay of the launch list: several replays with different inputs, with eager work and
synchronisations of the same executor (and of a second one) in between; every replay is checked against the CPU
oracle (the parity rules of the other GPU tests) and has to equal the step-by-step launches bit for bit."""
import os

import numpy as np
import pytest

from kyanite_amd import HipExecutor, optimize_graph
from kyanite_amd.configs import build_resnet_tower, build_tiny_mlp, uniform
from kyanite_amd.onnx import load_check_data, load_graph_from_onnx_bytes
from oracle import cpu_eval_graph
from runner import PARITY_RECORDS, check_outputs

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def att_tiny():
    with open(os.path.join(GOLDEN, "att-tiny.onnx"), "rb") as f:
        graph = optimize_graph(load_graph_from_onnx_bytes(f.read()))
    with open(os.path.join(GOLDEN, "att-tiny.bin"), "rb") as f:
        batch, inputs, _ = load_check_data(graph, f.read())
    return graph, batch, inputs


def tiny_mlp():
    graph, inputs = build_tiny_mlp(seed=3, batch=8)
    return graph, 8, inputs


def small_tower():
    graph, make_inputs, _ = build_resnet_tower(seed=4, channels=16, blocks=2, policy_channels=4, policy_size=50,
                                               value_channels=2, value_hidden=8)
    return graph, 6, make_inputs(6)


@pytest.mark.gpu
@pytest.mark.parametrize("build", [tiny_mlp, att_tiny, small_tower])
def test_graph_replay_matches_eager(build, hip_device):
    graph, batch, inputs = build()
    # (both launch the planned steps: a plan as small as the MLP's would otherwise run as one fused kernel, whose plain
    # dot products round differently from the matrix-core kernels of the replayed launch list)
    eager = HipExecutor(hip_device, graph, batch, step_by_step=True)
    replay = HipExecutor(hip_device, graph, batch, step_by_step=True)
    replay.set_graph_mode(True)
    for round_ in range(5):
        # new inputs every round: a replay that re-used stale results would show
        ins = [x if round_ == 0 else (x * (1.0 + 0.25 * round_) + uniform(round_, 7, x.shape, -0.1, 0.1)).astype(x.dtype)
               for x in inputs]
        want = eager.evaluate(ins)
        got = replay.evaluate(ins)
        check_outputs(graph, batch, ins, cpu_eval_graph(graph, batch, ins), got, f"graph replay {build.__name__} round {round_}",
                      PARITY_RECORDS)
        for w, g in zip(want, got):
            assert np.array_equal(w, g, equal_nan=True), f"round {round_}: graph replay differs from eager launches"
        # device-only replays between the checked ones
        replay.run_async()
        replay.run_async()
        replay.synchronize()
    # switching back to step-by-step launches still works, and profiling bypasses the graph
    replay.set_graph_mode(False)
    for w, g in zip(eager.evaluate(inputs), replay.evaluate(inputs)):
        assert np.array_equal(w, g, equal_nan=True)
    replay.set_graph_mode(True)
    replay.set_profile(True)
    replay.run_async()
    assert len(replay.last_profile().step_seconds) == replay.step_count()
