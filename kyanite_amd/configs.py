"""Builders for the benchmark configurations: graphs made with the graph builder, plus seeded synthetic inputs.

All random values come from one counter-based generator (splitmix64 -> uniform / Box-Muller normal), so a given
(seed, stream) always yields the same tensor, on any machine and for any evaluation order.
"""
import math

import numpy as np

from .graph import BATCH, BinaryOp, DType, Graph, ReduceOp, UnaryOp

_MASK = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(x):
    x = (x + np.uint64(0x9E3779B97F4A7C15)) & _MASK
    z = x
    z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _MASK
    z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _MASK
    return z ^ (z >> np.uint64(31))


def _bits(seed, stream, n):
    """n 64-bit words; word i depends only on (seed, stream, i)."""
    with np.errstate(over="ignore"):
        base = _splitmix64(np.uint64(seed) * np.uint64(0x100000001B3) + np.uint64(stream))
        idx = np.arange(n, dtype=np.uint64)
        return _splitmix64(base + idx * np.uint64(0x9E3779B97F4A7C15))


def uniform(seed, stream, shape, lo=0.0, hi=1.0):
    n = int(np.prod(shape)) if len(shape) else 1
    u = (_bits(seed, stream, n) >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))
    return (lo + (hi - lo) * u).astype(np.float32).reshape(shape)


def normal(seed, stream, shape, mean=0.0, std=1.0):
    n = int(np.prod(shape)) if len(shape) else 1
    out = np.empty(n, np.float32)
    chunk = 1 << 22
    for start in range(0, n, chunk):
        m = min(chunk, n - start)
        half = (m + 1) // 2
        with np.errstate(over="ignore"):
            base = _splitmix64(np.uint64(seed) * np.uint64(0x100000001B3) + np.uint64(stream))
            idx = np.arange(start // 2 * 2, start // 2 * 2 + 2 * half, dtype=np.uint64)
            w = _splitmix64(base + idx * np.uint64(0x9E3779B97F4A7C15))
        u = ((w >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / (1 << 53))
        r = np.sqrt(-2.0 * np.log(u[0::2]))
        t = 2.0 * math.pi * u[1::2]
        z = np.empty(2 * half, np.float64)
        z[0::2] = r * np.cos(t)
        z[1::2] = r * np.sin(t)
        out[start:start + m] = (mean + std * z[:m]).astype(np.float32)
    return out.reshape(shape)


def bernoulli(seed, stream, shape, p):
    return (uniform(seed, stream, shape) < p).astype(np.float32)


# ---------------------------------------------------------------------------------------------- config 1

def build_tiny_mlp(seed=0, batch=8):
    """Input [B, 16] uniform[-1, 1] -> Linear 16->32 (+bias) -> ReLU -> Linear 32->10 (+bias) -> softmax axis 1.
    Weights N(0, 1/fan_in), biases 0."""
    g = Graph()
    x = g.input([BATCH, 16])
    w1 = g.constant([32, 16], normal(seed, 1, (32, 16), std=1.0 / math.sqrt(16)))
    b1 = g.constant([1, 32], np.zeros((1, 32), np.float32))
    w2 = g.constant([10, 32], normal(seed, 2, (10, 32), std=1.0 / math.sqrt(32)))
    b2 = g.constant([1, 10], np.zeros((1, 10), np.float32))
    h = g.relu(g.add(g.linear(x, w1), b1))
    y = g.softmax(g.add(g.linear(h, w2), b2), 1)
    g.output(y)
    return g, [uniform(seed, 0, (batch, 16), -1.0, 1.0)]


# ---------------------------------------------------------------------------------------------- config 2

def gelu_tanh(g, x):
    """tanh GELU: 0.5 * x * (1 + tanh(sqrt(2 / pi) * (x + 0.044715 * x^3)))"""
    x3 = g.mul(g.mul(x, x), x)
    inner = g.mul(g.add(x, g.mul(x3, g.scalar(0.044715))), g.scalar(math.sqrt(2.0 / math.pi)))
    t = g.unary(UnaryOp.TANH, inner)
    return g.mul(g.mul(x, g.scalar(0.5)), g.add(t, g.scalar(1.0)))


def build_fused_chain(seed=0, shape=(64, 1024, 1024)):
    """(a) y = gelu_tanh(x * a + b) + r with a, b of shape [C] broadcast along the last axis."""
    c = shape[-1]
    g = Graph()
    x = g.input(list(shape))
    r = g.input(list(shape))
    a = g.constant([c], normal(seed, 10, (c,)))
    b = g.constant([c], normal(seed, 11, (c,)))
    y = g.add(gelu_tanh(g, g.add(g.mul(x, a), b)), r)
    g.output(y)
    inputs = lambda: [normal(seed, 12, shape), normal(seed, 13, shape)]
    # algorithmic bytes: read x and r, write y, read a and b once
    n = int(np.prod(shape))
    return g, inputs, 3 * 4 * n + 2 * 4 * c


def build_softmax(seed=0, shape=(32, 16, 512, 512)):
    """(b) softmax over the last axis."""
    g = Graph()
    x = g.input(list(shape))
    g.output(g.softmax(x, len(shape) - 1))
    inputs = lambda: [normal(seed, 20, shape)]
    return g, inputs, 2 * 4 * int(np.prod(shape))


def build_layernorm(seed=0, shape=(8192, 4096), eps=1e-5):
    """(c) layernorm over the last axis, gamma ~ N(1, 0.1), beta ~ N(0, 0.1)."""
    c = shape[-1]
    g = Graph()
    x = g.input(list(shape))
    gamma = g.constant([c], normal(seed, 30, (c,), 1.0, 0.1))
    beta = g.constant([c], normal(seed, 31, (c,), 0.0, 0.1))
    y = g.add(g.mul(g.layernorm(x, len(shape) - 1, eps), gamma), beta)
    g.output(y)
    inputs = lambda: [normal(seed, 32, shape)]
    return g, inputs, 2 * 4 * int(np.prod(shape)) + 2 * 4 * c


def build_reduce(seed=0, shape=(4096, 8192)):
    """(d) sum over axis 1."""
    g = Graph()
    x = g.input(list(shape))
    g.output(g.reduce(x, [1], ReduceOp.SUM))
    inputs = lambda: [normal(seed, 40, shape)]
    return g, inputs, 4 * int(np.prod(shape)) + 4 * shape[0]


BANDWIDTH_CONFIGS = {
    "2a_fused_gelu_chain": (build_fused_chain, (64, 1024, 1024)),
    "2b_softmax": (build_softmax, (32, 16, 512, 512)),
    "2c_layernorm_affine": (build_layernorm, (8192, 4096)),
    "2d_reduce_sum": (build_reduce, (4096, 8192)),
}


# ---------------------------------------------------------------------------------------------- config 3

def build_resnet_tower(seed=0, channels=128, blocks=10, board=8, in_planes=21, policy_channels=32, policy_size=4672,
                       value_channels=8, value_hidden=256):
    """AlphaZero style tower with batch-norm already folded into conv + bias (He-normal weights)."""
    g = Graph()
    stream = [100]

    def conv_w(co, ci, k):
        stream[0] += 1
        return g.constant([co, ci, k, k], normal(seed, stream[0], (co, ci, k, k), std=math.sqrt(2.0 / (ci * k * k))))

    def bias(co):
        stream[0] += 1
        return g.constant([1, co, 1, 1], normal(seed, stream[0], (1, co, 1, 1), std=0.05))

    def linear(x, co, ci):
        stream[0] += 2
        w = g.constant([co, ci], normal(seed, stream[0], (co, ci), std=math.sqrt(2.0 / ci)))
        b = g.constant([1, co], normal(seed, stream[0] + 1, (1, co), std=0.05))
        return g.add(g.linear(x, w), b)

    x = g.input([BATCH, in_planes, board, board])
    t = g.relu(g.add(g.conv(x, conv_w(channels, in_planes, 3), 1, 1, 1, 1), bias(channels)))
    for _ in range(blocks):
        y = g.relu(g.add(g.conv(t, conv_w(channels, channels, 3), 1, 1, 1, 1), bias(channels)))
        y = g.add(g.add(g.conv(y, conv_w(channels, channels, 3), 1, 1, 1, 1), bias(channels)), t)
        t = g.relu(y)
    # policy head
    p = g.relu(g.add(g.conv(t, conv_w(policy_channels, channels, 1), 1, 1, 0, 0), bias(policy_channels)))
    p = g.flatten(p, 1)
    p = g.softmax(linear(p, policy_size, policy_channels * board * board), 1)
    # value head
    v = g.relu(g.add(g.conv(t, conv_w(value_channels, channels, 1), 1, 1, 0, 0), bias(value_channels)))
    v = g.flatten(v, 1)
    v = g.relu(linear(v, value_hidden, value_channels * board * board))
    v = g.unary(UnaryOp.TANH, linear(v, 1, value_hidden))
    g.output_all([p, v])

    def inputs(batch):
        return [bernoulli(seed, 99, (batch, in_planes, board, board), 0.1)]

    hw = board * board
    macs = (in_planes * 9 * channels * hw + blocks * 2 * channels * 9 * channels * hw + channels * policy_channels * hw +
            policy_channels * hw * policy_size + channels * value_channels * hw + value_channels * hw * value_hidden + value_hidden)
    return g, inputs, 2 * macs  # flop per position
