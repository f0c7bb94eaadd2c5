"""Differential test on seeded random graphs: the HIP executor against the oracle on graphs that chain the
operations in orders nobody wrote down by hand, so that the planner's fusions (elementwise chains, row kernel
prologues and epilogues, matmul epilogues, grouped matmuls, fused attention, reductions with a prologue, broadcast
chains) meet each other's edge cases. The graphs are small enough that the oracle takes milliseconds.

CPU half: every graph evaluates in the oracle with finite results, optimizes to the same values, and plans and
compiles for gfx950. GPU half: `check_gpu` (bit-exact data movement, f32 within 1e-4 of the oracle).
"""
import numpy as np
import pytest

from kyanite_amd import BinaryOp, DType, Graph, ReduceOp, UnaryOp
from runner import check_cpu, check_gpu

SEEDS = list(range(48))
DIMS = [1, 2, 3, 5, 8, 17, 32, 40, 64]


class Builder:
    def __init__(self, seed, dtype=DType.F32):
        self.rng = np.random.default_rng(1000 + seed)
        self.g = Graph()
        self.dtype = dtype
        self.np_dtype = np.float16 if dtype == DType.F16 else np.float32
        self.inputs = []
        self.values = []  # (value, shape)

    def pick(self, options):
        return options[int(self.rng.integers(len(options)))]

    def new_input(self, shape):
        v = self.g.input(list(shape), self.dtype)
        self.inputs.append(self.rng.standard_normal(shape).astype(self.np_dtype))
        self.values.append((v, tuple(shape)))
        return v

    def const(self, shape, scale=1.0):
        data = (self.rng.standard_normal(shape) * scale).astype(self.np_dtype)
        return self.g.constant(list(shape), data, self.dtype)

    def scalar(self, x):
        return self.g.scalar(float(x), self.dtype)

    def some_value(self, rank=None):
        candidates = [x for x in self.values if rank is None or len(x[1]) == rank]
        if not candidates:
            shape = tuple(self.pick(DIMS[2:]) for _ in range(rank or 2))
            self.new_input(shape)
            candidates = [self.values[-1]]
        # prefer recent values so that chains form, but keep older ones in play (values with several users)
        k = len(candidates)
        weights = np.arange(1, k + 1, dtype=np.float64) ** 2
        return candidates[int(self.rng.choice(k, p=weights / weights.sum()))]

    def push(self, v, shape):
        self.values.append((v, tuple(shape)))

    # ---- operations; each bounds its output so that chains stay finite
    def op_unary(self):
        v, shape = self.some_value()
        op = self.pick([UnaryOp.ABS, UnaryOp.NEG, UnaryOp.TANH, UnaryOp.SIGMOID, UnaryOp.SIN, UnaryOp.COS])
        self.push(self.g.unary(op, v), shape)

    def op_binary_same(self):
        v, shape = self.some_value()
        others = [x for x in self.values if x[1] == shape]
        w = self.pick(others)[0]
        op = self.pick([BinaryOp.ADD, BinaryOp.SUB, BinaryOp.MUL, BinaryOp.MIN, BinaryOp.MAX])
        out = self.g.binary(op, v, w)
        if op == BinaryOp.MUL:
            out = self.g.unary(UnaryOp.TANH, out)
        self.push(out, shape)

    def op_binary_broadcast(self):
        v, shape = self.some_value()
        if len(shape) == 0:
            return
        keep = [bool(self.rng.integers(2)) for _ in shape]
        small = tuple(d if k else 1 for d, k in zip(shape, keep))
        c = self.g.broadcast(self.const(small, 0.5), list(shape))
        op = self.pick([BinaryOp.ADD, BinaryOp.MUL, BinaryOp.SUB])
        self.push(self.g.binary(op, v, c), shape)

    def op_scalar(self):
        v, shape = self.some_value()
        c = self.scalar(self.pick([0.5, -1.25, 2.0, 0.125]))
        self.push(self.g.binary(self.pick([BinaryOp.MUL, BinaryOp.ADD]), v, c), shape)

    def op_relu(self):
        v, shape = self.some_value()
        self.push(self.g.relu(v), shape)

    def op_permute(self):
        v, shape = self.some_value()
        if len(shape) < 2:
            return
        perm = list(self.rng.permutation(len(shape)))
        self.push(self.g.permute(v, [int(p) for p in perm]), tuple(shape[p] for p in perm))

    def op_slice(self):
        v, shape = self.some_value()
        axes = [a for a, d in enumerate(shape) if d >= 3]
        if not axes:
            return
        axis = self.pick(axes)
        step = self.pick([1, 1, 2])
        start = int(self.rng.integers(0, shape[axis] - step))
        out_len = int(self.rng.integers(1, (shape[axis] - start) // step + 1))
        end = start + out_len * step  # the range has to be a multiple of the step
        new_shape = shape[:axis] + (out_len,) + shape[axis + 1:]
        self.push(self.g.slice(v, axis, start, end, step), new_shape)

    def op_flip(self):
        v, shape = self.some_value()
        if not shape:
            return
        self.push(self.g.flip(v, int(self.rng.integers(len(shape)))), shape)

    def op_view(self):
        v, shape = self.some_value()
        if len(shape) < 2:
            return
        a = int(self.rng.integers(len(shape) - 1))
        merged = shape[:a] + (shape[a] * shape[a + 1],) + shape[a + 2:]
        self.push(self.g.view(v, list(merged)), merged)

    def op_reduce(self):
        v, shape = self.some_value()
        if not shape:
            return
        n_axes = int(self.rng.integers(1, len(shape) + 1))
        axes = sorted(int(a) for a in self.rng.choice(len(shape), n_axes, replace=False))
        op = self.pick([ReduceOp.SUM, ReduceOp.MEAN, ReduceOp.MAX, ReduceOp.MIN])
        if op == ReduceOp.SUM:
            v = self.g.binary(BinaryOp.MUL, v, self.scalar(1.0 / 16))
        out_shape = tuple(d for a, d in enumerate(shape) if a not in axes)
        out = self.g.reduce(v, axes, op)
        self.push(out, out_shape)
        if self.rng.integers(2):
            # back onto the input's shape: mean subtraction, normalisation and the like
            ones = tuple(1 if a in axes else d for a, d in enumerate(shape))
            back = self.g.broadcast(self.g.view(out, list(ones)), list(shape))
            self.push(self.g.binary(BinaryOp.SUB, v, back), shape)

    def op_softmax(self):
        v, shape = self.some_value()
        if not shape:
            return
        axis = int(self.rng.integers(len(shape)))
        if self.rng.integers(2):
            v = self.g.binary(BinaryOp.MUL, v, self.scalar(0.5))
        if self.rng.integers(3) == 0:
            small = tuple(1 if a == 0 else d for a, d in enumerate(shape))
            v = self.g.add(v, self.g.broadcast(self.const(small), list(shape)))
        self.push(self.g.softmax(v, axis), shape)

    def op_layernorm(self):
        v, shape = self.some_value()
        if not shape or shape[-1] < 2:
            return
        axis = len(shape) - 1 if self.rng.integers(3) else int(self.rng.integers(len(shape)))
        if shape[axis] < 2:
            return
        out = self.g.layernorm(v, axis, 1e-5)
        if self.rng.integers(2):
            small = tuple(d if a == axis else 1 for a, d in enumerate(shape))
            out = self.g.add(self.g.mul(out, self.g.broadcast(self.const(small), list(shape))),
                             self.g.broadcast(self.const(small), list(shape)))
        self.push(out, shape)

    def op_linear(self):
        v, shape = self.some_value(2)
        m, k = shape
        n = self.pick(DIMS[2:])
        count = self.pick([1, 1, 2, 3])  # several projections of one value: grouped launches
        for _ in range(count):
            w = self.const((n, k), 1.0 / np.sqrt(k))
            out = self.g.linear(v, w)
            choice = int(self.rng.integers(4))
            if choice == 1:
                out = self.g.add(out, self.g.broadcast(self.const((1, n)), [m, n]))
            elif choice == 2:
                out = self.g.relu(self.g.add(out, self.g.broadcast(self.const((1, n)), [m, n])))
            elif choice == 3:
                same = [x for x in self.values if x[1] == (m, n)]
                if same:
                    out = self.g.add(out, self.pick(same)[0])
            self.push(out, (m, n))

    def op_batched_matmul(self):
        v, shape = self.some_value(3)
        b, m, k = shape
        n = self.pick(DIMS[1:])
        w = self.new_input((b, k, n)) if self.rng.integers(2) else self.g.broadcast(self.const((1, k, n)), [b, k, n])
        out = self.g.batched_mat_mul(v, w)
        out = self.g.binary(BinaryOp.MUL, out, self.scalar(1.0 / np.sqrt(k)))
        self.push(out, (b, m, n))

    def op_attention(self):
        b, lq, lk = self.pick([1, 2, 3]), self.pick([5, 17, 40, 130]), self.pick([3, 33, 64, 150])
        f16 = self.dtype == DType.F16
        dk, dv = self.pick([64, 128] if f16 else [32, 40, 64]), self.pick([8, 32, 40, 64] + ([96, 128] if f16 else []))
        q = self.new_input((b, lq, dk))
        k = self.new_input((b, lk, dk))
        v = self.new_input((b, lk, dv))
        scores = self.g.batched_mat_mul(q, self.g.permute(k, [0, 2, 1]))
        if self.rng.integers(3):
            scores = self.g.binary(BinaryOp.MUL, scores, self.scalar(1.0 / np.sqrt(dk)))
        if f16 and self.rng.integers(2):
            keep = np.tril(np.ones((lq, lk), bool), k=max(lk - lq, 0))
            mask = self.g.constant([1, lq, lk], np.where(keep, 0.0, -np.inf).astype(np.float16)[None], DType.F16)
            scores = self.g.add(scores, self.g.broadcast(mask, [b, lq, lk]))
        probs = self.g.softmax(scores, 2)
        self.push(self.g.batched_mat_mul(probs, v), (b, lq, dv))
        if self.rng.integers(4) == 0:
            self.push(probs, (b, lq, lk))  # keeps the chain apart when it becomes an output or an operand

    def op_conv(self):
        n, c, h, w = self.pick([1, 2, 3]), self.pick([3, 8, 16]), self.pick([4, 8]), self.pick([4, 8, 16])
        x = self.new_input((n, c, h, w))
        k = self.pick([4, 16, 40])
        size = self.pick([1, 3])
        filt = self.const((k, c, size, size), 1.0 / np.sqrt(c * size * size))
        out = self.g.conv(x, filt, 1, 1, size // 2, size // 2)
        choice = int(self.rng.integers(3))
        if choice >= 1:
            out = self.g.add(out, self.g.broadcast(self.const((1, k, 1, 1)), [n, k, h, w]))
        if choice == 2:
            out = self.g.relu(out)
        self.push(out, (n, k, h, w))

    def build(self):
        rank = self.pick([2, 2, 3])
        self.new_input(tuple(self.pick(DIMS[2:]) for _ in range(rank)))
        ops = [self.op_unary, self.op_binary_same, self.op_binary_broadcast, self.op_scalar, self.op_relu, self.op_permute,
               self.op_slice, self.op_flip, self.op_view, self.op_reduce, self.op_softmax, self.op_layernorm,
               self.op_linear, self.op_linear, self.op_batched_matmul, self.op_attention, self.op_conv]
        if self.dtype == DType.F16:
            ops.remove(self.op_conv)  # convolutions are f32 only
        for _ in range(int(self.rng.integers(6, 16))):
            self.pick(ops)()
        # outputs: the last value and a few others (values with both a consumer and an output role)
        chosen = {len(self.values) - 1}
        for _ in range(int(self.rng.integers(1, 4))):
            chosen.add(int(self.rng.integers(len(self.values))))
        for i in sorted(chosen):
            self.g.output(self.values[i][0])
        return self.g, self.inputs


F16_SEEDS = list(range(100, 124))


@pytest.mark.parametrize("seed", SEEDS)
def test_cpu(seed):
    graph, inputs = Builder(seed).build()
    outputs = check_cpu(graph, 0, inputs)
    for o in outputs:
        assert np.all(np.isfinite(o)), "the generator is meant to keep values finite"


@pytest.mark.parametrize("seed", F16_SEEDS)
def test_cpu_f16(seed):
    graph, inputs = Builder(seed, DType.F16).build()
    outputs = check_cpu(graph, 0, inputs)
    for o in outputs:
        assert np.all(np.isfinite(o.astype(np.float32))), "the generator is meant to keep values finite"


@pytest.mark.gpu
@pytest.mark.parametrize("seed", F16_SEEDS)
def test_gpu_f16(seed, hip_device):
    graph, inputs = Builder(seed, DType.F16).build()
    print(f"random f16 graph seed {seed}: {len(graph)} values", flush=True)
    check_gpu(hip_device, graph, 0, inputs, what=f"random f16 graph {seed}")


@pytest.mark.gpu
@pytest.mark.parametrize("seed", SEEDS)
def test_gpu(seed, hip_device):
    graph, inputs = Builder(seed).build()
    print(f"random graph seed {seed}: {len(graph)} values", flush=True)
    check_gpu(hip_device, graph, 0, inputs, what=f"random graph {seed}")
