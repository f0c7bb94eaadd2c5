"""The gated pair of matmuls, (x w_g) sigmoid(x w_g) (x w_u) in f16 as one launch (GemmParams::pair_op), on every tile
shape of the kernel that loads global -> LDS directly. The tile is what the cost model picks for the shape (checked on
the CPU half, so a change of the model shows here); rows and columns are chosen ragged so that edge tiles, the column
interleave (16 of g, 16 of u per block of 32) and the half-tile stores are all exercised. The GPU result is compared
with the oracle on the unfused graph, and bit for bit with the GPU's own unfused plan (`fuse_gated_matmul=0`): the
fused store places its roundings where the separate launches do.

When the last round of tiles is sparse its tiles are shared by workgroups that take a slice of K each and sum inside
the launch; the last to arrive applies the gate. Those sums run in another order than the unfused plan's, so the tail
cases are held to the oracle only, twice on one executor (the second run finds the counters as the first left them)."""
import numpy as np
import pytest

from kyanite_amd import DType, Graph, HipExecutor
from oracle import cpu_eval_graph
from runner import PARITY_RECORDS, check_outputs

# (m, k, n) -> tile
SHAPES = {
    (128 - 3, 128, 512 - 24): "64x64",
    (384 - 1, 128, 2752 - 8): "128x128",
    (384 - 5, 1024, 1536 - 40): "128x64",
    (256 - 2, 1024, 11008): "256x128",
    (384 + 7, 128, 11008 - 72): "256x192",
    (1024 - 9, 128, 8192 - 136): "256x256",
}

# (m, k, n) -> tile and tail
TAIL_SHAPES = {
    (33, 2048, 16640 - 24): "direct 64x64 bk64 gated pairs head=512 tail_split=4x512",
    (250 - 3, 1536, 4160 - 8): "direct 128x64 bk64 gated pairs head=256 tail_split=3x512",
    (300 - 1, 1024, 16544 - 8): "direct 256x192 bk64 gated pairs head=256 tail_split=2x512",
    (1015, 1536, 8440): "direct 256x192 bk64 gated pairs head=256 tail_split=2x768",
}


def build(m, k, n, seed):
    rng = np.random.default_rng(seed)
    g = Graph()
    x = g.input([m, k], DType.F16)
    gate = g.linear(x, g.constant([n, k], (rng.standard_normal((n, k)) / np.sqrt(k)).astype(np.float16), DType.F16))
    up = g.linear(x, g.constant([n, k], (rng.standard_normal((n, k)) / np.sqrt(k)).astype(np.float16), DType.F16))
    g.output(g.mul(g.mul(gate, g.sigmoid(gate)), up))
    return g, [(rng.standard_normal((m, k)) * 1.5).astype(np.float16)]


@pytest.mark.parametrize("shape", list(SHAPES))
def test_plan_is_one_gated_launch_on_the_expected_tile(shape):
    g, _ = build(*shape, seed=1)
    ex = HipExecutor(0, g, 0, plan_only=True)
    assert ex.step_count() == 1 and f"[direct {SHAPES[shape]} " in ex.step_str(0) and "gated pairs" in ex.step_str(0), ex.step_str(0)
    assert HipExecutor(0, g, 0, plan_only=True, fuse_gated_matmul=0).step_count() == 2


@pytest.mark.gpu
@pytest.mark.parametrize("shape", list(SHAPES))
def test_gated_launch_matches_oracle_and_unfused_plan(shape, hip_device):
    print(f"gated matmul {shape} on {SHAPES[shape]} tiles", flush=True)
    g, inputs = build(*shape, seed=hash(shape) % 1000)
    expected = cpu_eval_graph(g, 0, inputs)
    fused = HipExecutor(hip_device, g, 0).evaluate(inputs)
    check_outputs(g, 0, inputs, expected, fused, f"gated matmul {shape}", PARITY_RECORDS)
    unfused = HipExecutor(hip_device, g, 0, fuse_gated_matmul=0).evaluate(inputs)
    assert np.array_equal(fused[0].view(np.uint16), unfused[0].view(np.uint16)), \
        f"{np.count_nonzero(fused[0] != unfused[0])} of {fused[0].size} elements differ from the unfused plan"


@pytest.mark.parametrize("shape", list(TAIL_SHAPES))
def test_plan_shares_the_tiles_of_a_sparse_last_round(shape):
    g, _ = build(*shape, seed=1)
    ex = HipExecutor(0, g, 0, plan_only=True)
    assert ex.step_count() == 1 and f"[{TAIL_SHAPES[shape]}]" in ex.step_str(0), ex.step_str(0)
    assert "tail_split" not in HipExecutor(0, g, 0, plan_only=True, tail_split=False).step_str(0)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", list(TAIL_SHAPES))
def test_gated_launch_with_shared_tail_tiles_matches_oracle(shape, hip_device):
    print(f"gated matmul {shape}: {TAIL_SHAPES[shape]}", flush=True)
    g, inputs = build(*shape, seed=sum(shape) % 1000)
    expected = cpu_eval_graph(g, 0, inputs)
    ex = HipExecutor(hip_device, g, 0)
    for run in range(2):
        check_outputs(g, 0, inputs, expected, ex.evaluate(inputs), f"gated matmul {shape} tail run {run}", PARITY_RECORDS)
