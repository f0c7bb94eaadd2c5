"""Differential test on seeded random softmax, layernorm and reduce operations: ranks 1 to 4, any axis (the contiguous
one, a middle one, the first), lengths from 1 to 150000 along it, f32 and f16, now and then a scale or a sum in front
and an affine behind. Between them the cases take every variant of the row and reduce kernels: rows in registers and
rows read again per pass, lanes along the row and lanes across columns (64, 32 and 16 of them), reductions along rows
and along columns, in one launch and in two, and the few long rows that run as separate steps.

CPU half: the graph evaluates in the oracle and plans for gfx950. GPU half: `check_gpu` against the oracle.
"""
import numpy as np
import pytest

from kyanite_amd import DType, Graph, ReduceOp
from runner import check_cpu, check_gpu

SEEDS = list(range(72))


def build(seed):
    rng = np.random.default_rng(11000 + seed)
    pick = lambda options: options[int(rng.integers(len(options)))]
    dtype = DType.F16 if seed % 3 == 2 else DType.F32
    g = Graph()
    inputs = []

    def tensor(shape, scale=1.0):
        inputs.append((rng.standard_normal(shape) * scale).astype(dtype.numpy))
        return g.input(list(shape), dtype)

    length = pick([1, 2, 7, 33, 40, 128, 300, 513, 1000, 4096, 5000, 70000, 150000])
    budget = 1_500_000 // length  # elements of the other axes together
    rank = pick([1, 2, 2, 3, 3, 4])
    others = []
    for _ in range(rank - 1):
        size = pick([1, 2, 3, 5, 16, 37, 64, 130, 600])
        size = max(1, min(size, budget))
        budget = max(1, budget // size)
        others.append(size)
    axis = int(rng.integers(rank))
    shape = others[:axis] + [length] + others[axis:]
    x = tensor(shape)
    kind = pick(["softmax", "softmax", "layernorm", "layernorm", "reduce", "reduce"])
    if kind == "reduce":
        op = pick([ReduceOp.SUM, ReduceOp.MEAN, ReduceOp.MAX, ReduceOp.MIN])
        axes = [axis]
        if rank >= 3 and pick([True, False]):
            axes = sorted({axis, int(rng.integers(rank))})
        source = g.mul(x, x) if pick([True, False, False]) and dtype == DType.F32 else x
        g.output(g.reduce(source, axes, op))
        return g, inputs
    front = pick(["plain", "plain", "scaled", "sum"])
    value = x
    if front == "scaled":
        value = g.mul(x, g.scalar(0.5, dtype))
    elif front == "sum":
        value = g.add(x, tensor(shape, 0.5))
    y = g.softmax(value, axis) if kind == "softmax" else g.layernorm(value, axis, 1e-5)
    if pick([True, False, False]):
        # an affine along the normalised axis, the way a layer's gamma and beta sit
        unit = [1] * rank
        unit[axis] = length
        gamma, beta = tensor(unit), tensor(unit)
        y = g.add(g.mul(y, g.broadcast(gamma, shape)), g.broadcast(beta, shape))
    g.output(y)
    return g, inputs


@pytest.mark.parametrize("seed", SEEDS)
def test_cpu(seed):
    g, inputs = build(seed)
    check_cpu(g, 0, inputs, None)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", SEEDS)
def test_gpu(seed, hip_device):
    g, inputs = build(seed)
    check_gpu(hip_device, g, 0, inputs, None, what=f"random rows {seed}")
