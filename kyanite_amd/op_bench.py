"""Times single operations on the HIP executor, one graph per line: what a shape costs outside of any network.

    python -m kyanite_amd.op_bench [-d DEVICE] [-n ITERATIONS] [-p] [FAMILY ...]

Families (default: all): `elementwise`, `activations`, `gather`, `reduce`, `rows` (softmax / layernorm), `conv`,
`matmul`, `attention`. `-p` plans and
compiles every case without a device and prints its steps instead of running it.

Every case is built like a user's graph (inputs, constants for weights), gets normally distributed inputs (matrix
cores run slower on real data than on zeros), runs `-n` times back to back between two events on the executor's stream
after two untimed runs, and is reported with the bytes its inputs and outputs hold (TB/s) and, for convolutions and
products, its arithmetic (TFLOP/s), next to the kernels the planner chose.
The cases are the shapes that decide how the kernels were laid out: few results from much input, normalised axes that
are not the contiguous one, small batches of small boards, left operands of a few rows.
"""
import argparse
import sys

import numpy as np


def _cases():
    from . import DType, Graph, ReduceOp, UnaryOp

    f32, f16, u8 = DType.F32, DType.F16, DType.U8
    rng = np.random.default_rng(0)
    M = 1 << 20
    out = []

    def case(family, name, build, nbytes, flops=0.0):
        out.append((family, name, build, float(nbytes), float(flops)))

    def one(g, dtype=f32):
        return g.scalar(1, dtype)

    case("elementwise", "x + 1, f32 [64M]", lambda g: g.output(g.add(g.input([64 * M]), one(g))), 512 * M)
    case("elementwise", "transpose + 1, f32 8192 x 8192", lambda g: g.output(g.add(g.permute(g.input([8192, 8192]), [1, 0]), one(g))), 512 * M)
    case("elementwise", "transpose + 1, f16 8192 x 8192",
         lambda g: g.output(g.add(g.permute(g.input([8192, 8192], f16), [1, 0]), one(g, f16))), 256 * M)
    case("elementwise", "transpose + 1, u8 16384 x 16384",
         lambda g: g.output(g.add(g.permute(g.input([16384, 16384], u8), [1, 0]), one(g, u8))), 512 * M)
    case("elementwise", "nchw -> nhwc, f32 [64, 256, 64, 64]",
         lambda g: g.output(g.add(g.permute(g.input([64, 256, 64, 64]), [0, 2, 3, 1]), one(g))), 512 * M)
    case("elementwise", "x + column, f32 8192 x 8192",
         lambda g: g.output(g.add(g.input([8192, 8192]), g.broadcast(g.input([8192, 1]), [8192, 8192]))), 512 * M)

    def activation_case(name, build, dtype=f32):
        elem = 2 if dtype == f16 else 4
        case("activations", f"{name}, {dtype.name.lower()} [64M]", lambda g: g.output(build(g, g.input([64 * M], dtype), dtype)), 2 * elem * 64 * M)

    def gelu_erf(g, x, dtype):
        inner = g.unary(UnaryOp.ERF, g.mul(x, g.scalar(0.7071067811865476, dtype)))
        return g.mul(g.mul(x, g.scalar(0.5, dtype)), g.add(g.scalar(1, dtype), inner))

    for dtype in (f32, f16):
        activation_case("sigmoid", lambda g, x, dt: g.unary(UnaryOp.SIGMOID, x), dtype)
        activation_case("tanh", lambda g, x, dt: g.unary(UnaryOp.TANH, x), dtype)
        activation_case("mish", lambda g, x, dt: g.unary(UnaryOp.MISH, x), dtype)
        activation_case("softplus", lambda g, x, dt: g.unary(UnaryOp.SOFTPLUS, x), dtype)
        activation_case("gelu through erf", gelu_erf, dtype)
        activation_case("x ** 2", lambda g, x, dt: g.pow(x, g.scalar(2.0, dt)), dtype)
        activation_case("x ** 1.5", lambda g, x, dt: g.pow(x, g.scalar(1.5, dt)), dtype)

    def gather_case(name, shape, axis, count, dtype=f32):
        elem = np.dtype(dtype.numpy).itemsize
        result = list(shape)
        result[axis] = count

        def build(g):
            where = g.constant([count], rng.integers(0, shape[axis], count).astype(np.int64), DType.I64)
            g.output(g.gather(g.input(list(shape), dtype), axis, where))

        # (what the result holds, read and written once; repeated indices are read again from the caches)
        case("gather", f"{name}: {count} along axis {axis} of {dtype.name.lower()} {list(shape)}", build, 2 * elem * int(np.prod(result)))

    gather_case("embedding rows", (32000, 4096), 0, 8192, f16)
    gather_case("embedding rows", (50000, 768), 0, 16384)
    gather_case("tokens of a sequence", (64, 4096, 1024), 1, 2048)
    gather_case("channels of bytes", (256, 64, 64, 64), 1, 64, u8)
    gather_case("policy moves", (1024, 4672), 1, 1858)
    gather_case("columns", (4096, 4096), 1, 4096)

    def reduce_case(shape, axes, op=ReduceOp.SUM, dtype=f32):
        elem = 2 if dtype == f16 else 4
        case("reduce", f"{op.name.lower()} over axes {axes} of {dtype.name.lower()} {list(shape)}",
             lambda g: g.output(g.reduce(g.input(list(shape), dtype), axes, op)), elem * int(np.prod(shape)))

    reduce_case((4096, 8192), [1])
    reduce_case((65536, 256), [0], ReduceOp.MEAN)
    reduce_case((4096, 4096), [0, 1])
    reduce_case((8192, 8192), [0, 1])
    reduce_case((262144, 1024), [0])
    reduce_case((16, 4 * M), [1])
    reduce_case((64, 128, 56, 56), [0, 2, 3], ReduceOp.MEAN)
    reduce_case((2 * M, 33), [1])

    def rows_case(kind, shape, axis, dtype=f32):
        elem = 2 if dtype == f16 else 4

        def build(g):
            x = g.input(list(shape), dtype)
            g.output(g.softmax(x, axis) if kind == "softmax" else g.layernorm(x, axis, 1e-5))

        case("rows", f"{kind} along axis {axis} of {dtype.name.lower()} {list(shape)}", build, 2 * elem * int(np.prod(shape)))

    rows_case("softmax", (32, 16, 512, 512), 3)
    rows_case("layernorm", (8192, 4096), 1)
    rows_case("softmax", (1024, 65536), 1)
    rows_case("softmax", (64, 256, 64, 64), 1)
    rows_case("softmax", (256, 19, 128, 128), 1)
    rows_case("layernorm", (64, 512, 32, 32), 1, f16)
    rows_case("softmax", (8, 1000, 4096), 1)
    rows_case("softmax", (4096, 16384), 0)
    rows_case("layernorm", (32, M), 1)
    # rows whose length is no multiple of the 128 bit vector: a vocabulary of 50257 entries
    rows_case("softmax", (2048, 50257), 1)
    rows_case("layernorm", (2048, 50257), 1)
    rows_case("softmax", (4096, 50257), 1, f16)

    def conv_case(name, n, c, h, w, oc, k, stride=1, pad=None):
        pad = k // 2 if pad is None else pad
        oh, ow = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1

        def build(g):
            filt = (rng.standard_normal((oc, c, k, k)) * 0.05).astype(np.float32)
            g.output(g.conv(g.input([n, c, h, w]), g.constant([oc, c, k, k], filt), stride, stride, pad, pad))

        case("conv", f"{name}: [{n}, {c}, {h}, {w}] -> {oc}, {k} x {k}" + (f" stride {stride}" if stride > 1 else ""), build,
             4 * (n * c * h * w + oc * c * k * k + n * oc * oh * ow), 2.0 * n * oh * ow * oc * c * k * k)

    conv_case("tower, batch 1024", 1024, 128, 8, 8, 128, 3)
    conv_case("tower, batch 64", 64, 128, 8, 8, 128, 3)
    conv_case("tower, batch 16", 16, 128, 8, 8, 128, 3)
    conv_case("tower, batch 1", 1, 128, 8, 8, 128, 3)
    conv_case("19 x 19 boards, batch 256", 256, 256, 19, 19, 256, 3)
    conv_case("19 x 19 boards, batch 8", 8, 192, 19, 19, 192, 3)
    conv_case("64 channels on 56 x 56", 32, 64, 56, 56, 64, 3)
    conv_case("5 x 5 filter", 128, 64, 32, 32, 64, 5)
    conv_case("7 x 7 stem", 32, 3, 224, 224, 64, 7, 2, 3)
    conv_case("downsampling", 32, 128, 56, 56, 256, 3, 2, 1)
    conv_case("UNet block", 8, 320, 32, 32, 320, 3)

    def matmul_case(m, n, k, dtype):
        elem = 2 if dtype == f16 else 4

        def build(g):
            weights = (rng.standard_normal((k, n), dtype=np.float32) * 0.05).astype(dtype.numpy)
            g.output(g.mat_mul(g.input([m, k], dtype), g.constant([k, n], weights, dtype)))

        case("matmul", f"{dtype.name.lower()} [{m}, {k}] x constant [{k}, {n}]", build, elem * (m * k + k * n + m * n), 2.0 * m * n * k)

    for dtype in (f16, f32):
        for m in (1, 8, 32, 64):
            matmul_case(m, 11008, 4096, dtype)
        matmul_case(8, 32000, 4096, dtype)
        matmul_case(1024, 4672, 2048, dtype)
        matmul_case(512, 11008, 4096, dtype)
        matmul_case(4096, 4096, 4096, dtype)

    def attention_case(heads, lq, lk, width, causal, dtype=f16):
        elem = 2 if dtype == f16 else 4

        def build(g):
            q, k, v = g.input([heads, lq, width], dtype), g.input([heads, lk, width], dtype), g.input([heads, lk, width], dtype)
            scores = g.mul(g.batched_mat_mul(q, g.permute(k, [0, 2, 1])), g.scalar(width ** -0.5, dtype))
            if causal:
                mask = np.where(np.tril(np.ones((lq, lk), bool), lk - lq), 0.0, -np.inf).astype(dtype.numpy)
                scores = g.add(scores, g.constant([1, lq, lk], mask, dtype))
            g.output(g.batched_mat_mul(g.softmax(scores, 2), v))

        case("attention", f"{dtype.name.lower()} {heads} x {lq} queries x {lk} keys, width {width}" + (", causal" if causal else ""), build,
             elem * heads * width * 2 * (lq + lk), 4.0 * heads * lq * lk * width * (0.5 if causal else 1.0))

    for tokens in (512, 1024, 2048, 4096):
        attention_case(32, tokens, tokens, 128, True)
    attention_case(64, 2048, 2048, 64, True)
    attention_case(32, 2048, 2048, 128, False)
    attention_case(16, 4096, 77, 64, False)
    attention_case(16, 4096, 4096, 40, False, f32)
    return out


def _fill_inputs(ex, rng):
    """every input := a block of a million random values, repeated (one upload, then copies on the device that double
    what is filled)"""
    from ctypes import c_void_p

    from ._lib import check, lib

    for i, (dtype, dims) in enumerate(ex.input_info):
        count = int(np.prod(dims)) if dims else 1
        if count == 0:
            continue
        kind = np.dtype(dtype.numpy).kind
        block = rng.standard_normal(min(count, 1 << 20)) if kind == "f" else rng.integers(0, 100, min(count, 1 << 20))
        block = np.ascontiguousarray(block.astype(dtype.numpy))
        base, item, filled = ex.input_ptr(i), block.itemsize, block.size
        check(lib.knhip_memcpy_h2d(ex.device, c_void_p(base), block.ctypes.data, filled * item))
        while filled < count:
            step = min(filled, count - filled)
            check(lib.knhip_memcpy_d2d(ex.device, c_void_p(base + filled * item), c_void_p(base), step * item))
            filled += step


def main(argv=None):
    parser = argparse.ArgumentParser(prog="op_bench", description="time single operations on the HIP executor")
    parser.add_argument("-d", "--device", type=int, default=0)
    parser.add_argument("-n", "--iterations", type=int, default=20)
    parser.add_argument("-p", "--plan-only", action="store_true")
    parser.add_argument("families", nargs="*")
    args = parser.parse_args(argv)

    from . import Graph, HipExecutor

    known = ["elementwise", "activations", "gather", "reduce", "rows", "conv", "matmul", "attention"]
    for family in args.families:
        if family not in known:
            parser.error(f"unknown family {family!r}; choose from {', '.join(known)}")
    wanted = args.families or known
    for family, name, build, nbytes, flops in _cases():
        if family not in wanted:
            continue
        graph = Graph()
        build(graph)
        ex = HipExecutor(args.device, graph, 0, plan_only=args.plan_only)
        kernels = []
        for i in range(ex.step_count()):
            text = ex.step_str(i)
            head = text.split(" operands")[0]
            kind = text.split(" value=")[0] + (" attention" if " attention " in head else "")
            kernels.append(kind + " [" + head.split("[", 1)[1].split("]")[0] + "]" if "[" in head else kind)
        if args.plan_only:
            print(f"{name}\n    " + "\n    ".join(kernels))
            continue
        _fill_inputs(ex, np.random.default_rng(1))
        for _ in range(2):
            ex.run_async()
        ex.synchronize()
        ms = ex.time_runs(args.iterations) / args.iterations
        line = f"{name:64s} {ms * 1e3:9.1f} us {nbytes / ms / 1e9:6.2f} TB/s"
        if flops:
            line += f" {flops / ms / 1e9:7.1f} TFLOP/s"
        print(line + "   " + " + ".join(kernels), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
