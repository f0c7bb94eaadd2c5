"""Differential test on seeded random layouts: elementwise kernels whose operands are permuted, flipped, sliced and
broadcast views big enough (at least 65,536 elements) for the kernel that turns 64 x 64 tiles through LDS, with tile
edges that are no multiple of 64, element sizes of 1, 2, 4 and 8 bytes and up to two transposed operands; and
attention over (batch, heads) in [batch, tokens, heads, width] order, which the fused kernel reads and writes in
place through two batch strides.

CPU half: the graph evaluates in the oracle and plans for gfx950 (the elementwise ones on the tile kernel, the
attention ones as one launch). GPU half: `check_gpu` (data movement and integer arithmetic bit-exact, f32 within
1e-4, f16 within 2e-2 of the oracle).
"""

import numpy as np
import pytest

from kyanite_amd import DType, Graph
from kyanite_amd.executor import HipExecutor
from runner import check_cpu, check_gpu

ELEMENTWISE_SEEDS = list(range(32))
ATTENTION_SEEDS = list(range(12))

NP_TYPES = {DType.F32: np.float32, DType.F16: np.float16, DType.F64: np.float64, DType.I32: np.int32, DType.U8: np.uint8,
            DType.I64: np.int64}


def random_data(rng, shape, dtype):
    if dtype in (DType.F32, DType.F16, DType.F64):
        return rng.standard_normal(shape).astype(NP_TYPES[dtype])
    return rng.integers(0, 100, size=shape).astype(NP_TYPES[dtype])


def build_elementwise(seed):
    rng = np.random.default_rng(9000 + seed)
    pick = lambda options: options[int(rng.integers(len(options)))]
    dtype = pick([DType.F32, DType.F32, DType.F16, DType.F16, DType.F64, DType.I32, DType.U8, DType.I64])
    rank = pick([2, 3, 3, 4])
    # the result's shape: the last axis and one other are long, so that the transposed pair of axes spans tiles
    shape = [pick([1, 2, 3, 5]) for _ in range(rank)]
    long_axis = int(rng.integers(rank - 1))
    shape[rank - 1] = pick([70, 130, 200, 257, 320])
    shape[long_axis] = pick([65, 100, 136, 300, 513])
    while int(np.prod(shape)) < (1 << 16):
        shape[long_axis] *= 2
    g = Graph()
    inputs = []
    transposed_operands = []

    def operand(kind):
        """an operand of the result's shape whose memory order differs from the result's"""
        if kind.startswith("transposed"):
            transposed_operands.append(kind)
        if kind == "straight":
            inputs.append(random_data(rng, shape, dtype))
            return g.input(shape, dtype)
        if kind == "broadcast":
            small = [1] * rank
            small[rank - 1] = shape[rank - 1]
            inputs.append(random_data(rng, small, dtype))
            return g.broadcast(g.input(small, dtype), shape)
        # transposed: stored with `long_axis` innermost; optionally as a window of a bigger tensor, or flipped
        perm = list(range(rank))
        perm[long_axis], perm[rank - 1] = perm[rank - 1], perm[long_axis]
        stored = [shape[a] for a in perm]
        window = kind == "transposed_window"
        if window:
            stored[rank - 1] += 8
            stored[0] += 1
        inputs.append(random_data(rng, stored, dtype))
        x = g.input(stored, dtype)
        if window:
            x = g.slice(g.slice(x, rank - 1, 8, stored[rank - 1]), 0, 1, stored[0])
        x = g.permute(x, perm)  # the inverse of a swap is the swap
        if kind == "transposed_flipped":
            x = g.flip(x, rank - 1)
        return x

    first = operand(pick(["transposed", "transposed", "transposed_window", "transposed_flipped"]))
    mode = pick(["copy", "binary", "binary", "three"])
    if mode == "copy":
        # a view that is no stride edit forces the dense copy
        y = g.view(first, [int(np.prod(shape))])
    else:
        second = operand(pick(["straight", "broadcast", "transposed"]))
        y = g.add(first, second)
        if mode == "three":
            y = g.mul(y, operand(pick(["straight", "broadcast"])))
    g.output(y)
    # two tiles of 8 byte elements do not fit the kernel's LDS budget: those graphs run on the plain kernel
    tiles = not (len(transposed_operands) > 1 and dtype in (DType.F64, DType.I64))
    return g, inputs, dtype, tiles


def build_attention(seed):
    rng = np.random.default_rng(9500 + seed)
    pick = lambda options: options[int(rng.integers(len(options)))]
    f16 = seed % 2 == 1
    dtype, np_dtype = (DType.F16, np.float16) if f16 else (DType.F32, np.float32)
    batch, heads = pick([1, 2, 3]), pick([2, 3, 4])
    lq, lk = pick([33, 64, 100, 150]), pick([40, 77, 128, 200])
    dk = pick([64, 128]) if f16 else pick([32, 40, 64])
    dv = pick([32, 64, 128]) if f16 else pick([24, 40, 64])
    g = Graph()
    inputs = []

    def inp(shape):
        inputs.append(rng.standard_normal(shape).astype(np_dtype))
        return g.input(list(shape), dtype)

    def heads_of(tokens, width, how):
        if how == "projection":  # [batch * tokens, heads * width] -> [batch * heads, tokens, width]
            x = g.view(inp((batch * tokens, heads * width)), [batch, tokens, heads, width])
            return g.view(g.permute(x, [0, 2, 1, 3]), [batch * heads, tokens, width])
        if how == "heads_first":  # [heads, batch, tokens, width]: the batch split the other way round
            x = g.permute(inp((heads, batch, tokens, width)), [1, 0, 2, 3])
            return g.view(x, [batch * heads, tokens, width])
        return inp((batch * heads, tokens, width))

    q = heads_of(lq, dk, pick(["projection", "projection", "dense"]))
    k = heads_of(lk, dk, pick(["projection", "projection", "dense", "heads_first"]))
    v = heads_of(lk, dv, pick(["projection", "projection", "dense", "heads_first"]))
    scores = g.mul(g.batched_mat_mul(q, g.permute(k, [0, 2, 1])), g.scalar(1.0 / np.sqrt(dk), dtype))
    out = g.batched_mat_mul(g.softmax(scores, 2), v)
    if pick([True, True, False]):
        out = g.view(g.permute(g.view(out, [batch, heads, lq, dv]), [0, 2, 1, 3]), [batch * lq, heads * dv])
    g.output(out)
    return g, inputs, dtype


@pytest.mark.parametrize("seed", ELEMENTWISE_SEEDS)
def test_elementwise_cpu(seed):
    g, inputs, dtype, tiles = build_elementwise(seed)
    check_cpu(g, 0, inputs, None)
    ex = HipExecutor(0, g, 0, plan_only=True)
    assert any("transposed tiles" in ex.step_str(i) for i in range(ex.step_count())) == tiles, \
        [ex.step_str(i) for i in range(ex.step_count())]


@pytest.mark.parametrize("seed", ATTENTION_SEEDS)
def test_attention_cpu(seed):
    g, inputs, dtype = build_attention(seed)
    check_cpu(g, 0, inputs, None)
    ex = HipExecutor(0, g, 0, plan_only=True)
    assert sum("attention" in ex.step_str(i) for i in range(ex.step_count())) == 1


@pytest.mark.gpu
@pytest.mark.parametrize("seed", ELEMENTWISE_SEEDS)
def test_elementwise_gpu(seed, hip_device):
    g, inputs, dtype, _ = build_elementwise(seed)
    check_gpu(hip_device, g, 0, inputs, None, what=f"random layout {seed}")


@pytest.mark.gpu
@pytest.mark.parametrize("seed", ATTENTION_SEEDS)
def test_attention_gpu(seed, hip_device):
    g, inputs, dtype = build_attention(seed)
    check_gpu(hip_device, g, 0, inputs, None, what=f"random attention {seed}")
