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


_LARGE_CACHE = {}


def cached_normal(seed, stream, shape, std, np_dtype):
    """`normal` for large weight tensors that several graphs of one process share (full size and sample builds)."""
    key = (seed, stream, tuple(shape), float(std), np.dtype(np_dtype).str)
    if key not in _LARGE_CACHE:
        _LARGE_CACHE[key] = normal(seed, stream, shape, std=std).astype(np_dtype)
    return _LARGE_CACHE[key]


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


# ---------------------------------------------------------------------------------------------- config 4

def build_llama(seed=0, layers=2, seq=512, d_model=4096, heads=32, ffn=11008, eps=1e-6, rope_base=10000.0,
                dtype=DType.F16):
    """LLaMA style decoder on one sequence: RMSNorm, rotary embedding on Q / K, causal softmax attention, SwiGLU
    feed-forward, residual adds; f16 weights / activations (f32 accumulation inside every operation).
    Everything is spelled with primitive operations: RMSNorm = x / sqrt(mean(x * x) + eps) * g, rotary = slices +
    mul + sub / add + concat, the causal mask = an added constant holding -inf, SiLU = x * sigmoid(x).
    Weights N(0, 0.02), norm gains 1, input embeddings N(0, 1) of shape [1, seq, d_model].
    Returns (graph, make_inputs, flop per evaluation). Because of the causal mask, the first t rows of the output
    depend only on the first t rows of the input."""
    np_dt = DType(dtype).numpy
    d_head = d_model // heads
    assert d_head * heads == d_model and d_head % 2 == 0
    g = Graph()
    stream = [400]

    def weight(co, ci):
        stream[0] += 1
        return g.constant([co, ci], cached_normal(seed, stream[0], (co, ci), 0.02, np_dt))

    def const(shape, array):
        return g.constant(list(shape), np.ascontiguousarray(array).astype(np_dt))

    def rmsnorm(x):
        ms = g.view(g.reduce(g.mul(x, x), [1], ReduceOp.MEAN), [seq, 1])
        rms = g.unary(UnaryOp.SQRT, g.add(ms, g.scalar(eps, dtype)))
        gain = const((1, d_model), np.ones((1, d_model)))
        return g.mul(g.binary(BinaryOp.DIV, x, rms), gain)

    # rotary tables, HF layout: the two halves of a head rotate against each other
    half = d_head // 2
    inv_freq = rope_base ** (-np.arange(half, dtype=np.float64) * 2.0 / d_head)
    angles = np.arange(seq, dtype=np.float64)[:, None] * inv_freq[None, :]
    cos_t = const((1, seq, half), np.cos(angles)[None])
    sin_t = const((1, seq, half), np.sin(angles)[None])

    def rotary(t):  # [heads, seq, d_head]
        a = g.slice(t, 2, 0, half)
        b = g.slice(t, 2, half, d_head)
        ra = g.sub(g.mul(a, cos_t), g.mul(b, sin_t))
        rb = g.add(g.mul(b, cos_t), g.mul(a, sin_t))
        return g.concat([ra, rb], 2)

    def split_heads(t):  # [seq, d_model] -> [heads, seq, d_head]
        return g.permute(g.view(t, [seq, heads, d_head]), [1, 0, 2])

    mask = const((1, seq, seq), np.where(np.tril(np.ones((seq, seq), bool)), 0.0, -np.inf))
    scale = g.scalar(1.0 / math.sqrt(d_head), dtype)

    x_in = g.input([1, seq, d_model], dtype)
    x = g.view(x_in, [seq, d_model])
    for _ in range(layers):
        h = rmsnorm(x)
        q = rotary(split_heads(g.linear(h, weight(d_model, d_model))))
        k = rotary(split_heads(g.linear(h, weight(d_model, d_model))))
        v = split_heads(g.linear(h, weight(d_model, d_model)))
        scores = g.batched_mat_mul(q, g.permute(k, [0, 2, 1]))
        probs = g.softmax(g.add(g.mul(scores, scale), mask), 2)
        ctx = g.permute(g.batched_mat_mul(probs, v), [1, 0, 2])
        x = g.add(x, g.linear(g.view(ctx, [seq, d_model]), weight(d_model, d_model)))
        h = rmsnorm(x)
        gate = g.linear(h, weight(ffn, d_model))
        up = g.linear(h, weight(ffn, d_model))
        act = g.mul(g.mul(gate, g.sigmoid(gate)), up)
        x = g.add(x, g.linear(act, weight(d_model, ffn)))
    g.output(g.view(x, [1, seq, d_model]))

    def inputs(rows=seq):
        return [normal(seed, 399, (1, seq, d_model))[:, :rows].astype(np_dt)]

    macs = layers * (4 * seq * d_model * d_model + 2 * heads * seq * seq * d_head + 3 * seq * d_model * ffn)
    return g, inputs, 2 * macs


# ---------------------------------------------------------------------------------------------- config 5

def build_unet_block(seed=0, batch=2, channels=320, size=64, groups=32, heads=8, time_dim=1280, ctx_len=77,
                     ctx_dim=768, ffn_mult=4):
    """Stable-Diffusion style UNet block, f32: ResBlock (GroupNorm + SiLU + 3x3 conv, twice, with the projected
    timestep embedding added in between and the residual at the end) followed by a spatial transformer over the
    size * size tokens (layernorm + self-attention, layernorm + cross-attention to the context, layernorm + GEGLU
    feed-forward; linear projections in and out, residual around the whole transformer).
    GroupNorm is lowered as the reference's ONNX loader does it (kn-graph/src/onnx/load.rs:513-568): view as
    [N, groups, rest], layernorm over the last axis, view back, then scale and shift per channel.
    Inputs: latent [N, C, size, size], timestep embedding [N, time_dim], context [N, ctx_len, ctx_dim], all N(0, 1);
    weights N(0, 0.02), norm scales 1 + N(0, 0.02). Returns (graph, make_inputs, flop per evaluation)."""
    g = Graph()
    stream = [500]
    C, hw, d_head = channels, size * size, channels // heads
    assert d_head * heads == C and C % groups == 0

    def rnd(shape, std=0.02, mean=0.0):
        stream[0] += 1
        return g.constant(list(shape), normal(seed, stream[0], tuple(shape), mean=mean, std=std))

    def linear(x, co, ci, bias=True):
        y = g.linear(x, rnd((co, ci)))
        return g.add(y, rnd((1, co))) if bias else y

    def silu(x):
        return g.mul(x, g.sigmoid(x))

    def group_norm(x, eps):
        y = g.layernorm(g.view(x, [batch, groups, (C // groups) * hw]), 2, eps)
        y = g.view(y, [batch, C, size, size])
        return g.add(g.mul(y, rnd((1, C, 1, 1), mean=1.0)), rnd((1, C, 1, 1)))

    def layer_norm(x):  # [batch * hw, C]
        return g.add(g.mul(g.layernorm(x, 1, 1e-5), rnd((1, C), mean=1.0)), rnd((1, C)))

    def conv3(x):
        return g.add(g.conv(x, rnd((C, C, 3, 3)), 1, 1, 1, 1), rnd((1, C, 1, 1)))

    def attention(x, ctx, ctx_tokens, ctx_width):
        # x [batch * hw, C]; ctx [batch * ctx_tokens, ctx_width]
        def heads_of(t, tokens):  # [batch * tokens, C] -> [batch * heads, tokens, d_head]
            t = g.permute(g.view(t, [batch, tokens, heads, d_head]), [0, 2, 1, 3])
            return g.view(t, [batch * heads, tokens, d_head])

        q = heads_of(linear(x, C, C, bias=False), hw)
        k = heads_of(linear(ctx, C, ctx_width, bias=False), ctx_tokens)
        v = heads_of(linear(ctx, C, ctx_width, bias=False), ctx_tokens)
        scores = g.mul(g.batched_mat_mul(q, g.permute(k, [0, 2, 1])), g.scalar(1.0 / math.sqrt(d_head)))
        out = g.batched_mat_mul(g.softmax(scores, 2), v)  # [batch * heads, hw, d_head]
        out = g.permute(g.view(out, [batch, heads, hw, d_head]), [0, 2, 1, 3])
        return linear(g.view(out, [batch * hw, C]), C, C)

    latent = g.input([batch, C, size, size])
    t_emb = g.input([batch, time_dim])
    context = g.input([batch, ctx_len, ctx_dim])

    # ---- ResBlock
    h = conv3(silu(group_norm(latent, 1e-5)))
    h = g.add(h, g.view(linear(silu(t_emb), C, time_dim), [batch, C, 1, 1]))
    h = conv3(silu(group_norm(h, 1e-5)))
    res = g.add(latent, h)

    # ---- spatial transformer
    t = group_norm(res, 1e-6)
    t = g.view(g.permute(g.view(t, [batch, C, hw]), [0, 2, 1]), [batch * hw, C])  # tokens
    t = linear(t, C, C)
    n = layer_norm(t)
    t = g.add(t, attention(n, n, hw, C))
    ctx2 = g.view(context, [batch * ctx_len, ctx_dim])
    t = g.add(t, attention(layer_norm(t), ctx2, ctx_len, ctx_dim))
    inner = C * ffn_mult
    n = layer_norm(t)
    proj = linear(n, 2 * inner, C)
    value, gate = g.slice(proj, 1, 0, inner), g.slice(proj, 1, inner, 2 * inner)
    gelu = g.mul(g.mul(gate, g.scalar(0.5)),
                 g.add(g.unary(UnaryOp.ERF, g.mul(gate, g.scalar(1.0 / math.sqrt(2.0)))), g.scalar(1.0)))
    t = g.add(t, linear(g.mul(value, gelu), C, inner))
    t = linear(t, C, C)
    t = g.view(g.permute(g.view(t, [batch, hw, C]), [0, 2, 1]), [batch, C, size, size])
    g.output(g.add(res, t))

    def inputs():
        return [normal(seed, 497, (batch, C, size, size)), normal(seed, 498, (batch, time_dim)),
                normal(seed, 499, (batch, ctx_len, ctx_dim))]

    tok = batch * hw
    macs = (2 * tok * C * C * 9 + batch * time_dim * C + 2 * tok * C * C  # convs, time projection, proj in / out
            + 4 * tok * C * C + 2 * batch * heads * hw * hw * d_head  # self-attention
            + 2 * tok * C * C + 2 * batch * ctx_len * ctx_dim * C + 2 * batch * heads * hw * ctx_len * d_head  # cross
            + tok * C * 2 * inner + tok * inner * C)  # GEGLU feed-forward
    return g, inputs, 2 * macs
