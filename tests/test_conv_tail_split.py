"""Convolutions whose tile count leaves the last round of workgroups sparse (`conv_tail_split`, replacing the one
launch of kn-cuda-sys/src/wrapper/group.rs:11-54): the case of 128 x 128 tiles, which takes 768 of them. The cases of
64 x 64 tiles are `conv_with_a_sparse_last_round_of_tiles` in cases_graphs.py."""
import numpy as np
import pytest

from kyanite_amd import Graph, HipExecutor
from oracle import cpu_eval_graph
from runner import PARITY_RECORDS, check_outputs

BATCH_OF_BOARDS = 1536  # 98304 positions: 768 tiles of 128 x 128 for 128 output channels, 512 + 256


def tower_conv():
    g = Graph()
    rng = np.random.default_rng(768)
    x = g.input([BATCH_OF_BOARDS, 64, 8, 8])
    w = g.constant([128, 64, 3, 3], (rng.standard_normal((128, 64, 3, 3)) * 0.06).astype(np.float32))
    bias = g.constant([1, 128, 1, 1], rng.standard_normal((1, 128, 1, 1)).astype(np.float32))
    g.output(g.relu(g.add(g.conv(x, w, 1, 1, 1, 1), bias)))
    return g, [rng.standard_normal((BATCH_OF_BOARDS, 64, 8, 8)).astype(np.float32)]


def test_plan_shares_the_tiles_of_the_last_round():
    g, _ = tower_conv()
    plan = HipExecutor(0, g, 0, plan_only=True)
    assert "the tiles after 512 in 2 slices of the input channels" in plan.step_str(0), plan.step_str(0)
    whole = HipExecutor(0, g, 0, plan_only=True, split_conv_channels=False)
    assert "slices" not in whole.step_str(0)
    # a whole number of rounds stays as it is
    g2 = Graph()
    g2.output(g2.conv(g2.input([1024, 64, 8, 8]), g2.constant([128, 64, 3, 3], np.zeros((128, 64, 3, 3), np.float32)), 1, 1, 1, 1))
    assert "slices" not in HipExecutor(0, g2, 0, plan_only=True).step_str(0)


@pytest.mark.gpu
def test_shared_tiles_of_128_give_the_oracles_result(hip_device):
    g, inputs = tower_conv()
    print("conv tail split, 768 tiles of 128 x 128", flush=True)
    expected = cpu_eval_graph(g, 0, inputs)
    for options in ({}, {"split_conv_channels": False}):
        got = HipExecutor(hip_device, g, 0, **options).evaluate(inputs)
        check_outputs(g, 0, inputs, expected, got, f"conv tail split, 128 x 128 tiles, {options}", PARITY_RECORDS)
