"""Pins for the oracle beyond the reference's golden vectors: every operation against a textbook / library
routine in f64 (numpy), and the integer / cast edge cases against Rust's documented `as` semantics.

A dropped term, a wrong sign or index, a transposed operand or a wrong axis would fail one of these.
"""
import numpy as np
import pytest

from kyanite_amd import BATCH, BinaryOp, DType, Graph, ReduceOp, UnaryOp
from oracle import OracleError, cpu_eval_graph


def close(a, b, tol=1e-5):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    scale = max(np.sqrt(np.mean(b * b)), 1e-30)
    assert a.shape == b.shape
    assert np.max(np.abs(a - b)) <= tol * scale, np.max(np.abs(a - b)) / scale


def test_softmax_against_numpy():
    rng = np.random.default_rng(0)
    x = (rng.standard_normal((3, 7, 5)) * 4).astype(np.float32)
    for axis in range(3):
        g = Graph()
        g.output(g.softmax(g.input([3, 7, 5]), axis))
        (y,) = cpu_eval_graph(g, 0, [x])
        x64 = x.astype(np.float64)
        e = np.exp(x64 - x64.max(axis=axis, keepdims=True))
        close(y, e / e.sum(axis=axis, keepdims=True))
        assert np.allclose(y.sum(axis=axis), 1.0, atol=1e-5)
    # -inf entries get probability zero; an all -inf row is NaN, as exp(-inf - -inf) is (cpu.rs:450-455)
    g = Graph()
    g.output(g.softmax(g.input([2, 3]), 1))
    (y,) = cpu_eval_graph(g, 0, [np.array([[0.0, -np.inf, 0.0], [-np.inf] * 3], np.float32)])
    assert np.array_equal(y[0], np.array([0.5, 0.0, 0.5], np.float32)) and np.isnan(y[1]).all()


def test_layernorm_against_numpy():
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((4, 6, 33)) * 3 + 2).astype(np.float32)
    for axis, eps in ((2, 1e-5), (1, 1e-2), (0, 0.5)):
        g = Graph()
        g.output(g.layernorm(g.input([4, 6, 33]), axis, eps))
        (y,) = cpu_eval_graph(g, 0, [x])
        x64 = x.astype(np.float64)
        mean = x64.mean(axis=axis, keepdims=True)
        var = ((x64 - mean) ** 2).mean(axis=axis, keepdims=True)  # biased
        close(y, (x64 - mean) / np.sqrt(var + eps))
        if eps < 1e-4:
            assert np.allclose(y.mean(axis=axis), 0, atol=1e-5) and np.allclose(y.var(axis=axis), 1, atol=1e-3)


def test_reduce_against_numpy():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((5, 4, 6)).astype(np.float32)
    fns = {ReduceOp.SUM: np.sum, ReduceOp.MEAN: np.mean, ReduceOp.PROD: np.prod, ReduceOp.MAX: np.max, ReduceOp.MIN: np.min}
    for axes in ([0], [1], [2], [0, 2], [2, 0], [0, 1, 2]):
        for op, fn in fns.items():
            g = Graph()
            g.output(g.reduce(g.input([5, 4, 6]), axes, op))
            (y,) = cpu_eval_graph(g, 0, [x])
            close(y, fn(x.astype(np.float64), axis=tuple(axes)))
    # the fold is sequential in f32 from the identity: 2^24 + 1 + 1 stays 2^24 (graph.rs:1770-1786)
    g = Graph()
    g.output(g.reduce(g.input([3]), [0], ReduceOp.SUM))
    (y,) = cpu_eval_graph(g, 0, [np.array([2.0 ** 24, 1.0, 1.0], np.float32)])
    assert y == np.float32(2.0 ** 24)
    # integer sums wrap, empty reductions give the identity
    g = Graph()
    xi = g.input([3], DType.U8)
    e = g.input([0, 2])
    g.output_all([g.reduce(xi, [0], ReduceOp.SUM), g.reduce(e, [0], ReduceOp.MAX), g.reduce(e, [0], ReduceOp.PROD)])
    s, mx, pr = cpu_eval_graph(g, 0, [np.array([200, 100, 5], np.uint8), np.zeros((0, 2), np.float32)])
    assert s == np.uint8(49) and np.array_equal(mx, [-np.inf, -np.inf]) and np.array_equal(pr, [1, 1])


def test_matmul_and_conv_against_numpy():
    rng = np.random.default_rng(3)
    a = rng.standard_normal((3, 5, 7)).astype(np.float32)
    b = rng.standard_normal((3, 7, 4)).astype(np.float32)
    g = Graph()
    g.output(g.batched_mat_mul(g.input([3, 5, 7]), g.input([3, 7, 4])))
    (y,) = cpu_eval_graph(g, 0, [a, b])
    close(y, a.astype(np.float64) @ b.astype(np.float64))
    # cublas smoke vector, kn-cuda-sys/tests/cublas.rs:16-19: three 1x2 . 2x1 products
    g = Graph()
    g.output(g.batched_mat_mul(g.input([3, 1, 2]), g.input([3, 2, 1])))
    (y,) = cpu_eval_graph(g, 0, [np.arange(1, 7, dtype=np.float32).reshape(3, 1, 2), np.arange(7, 13, dtype=np.float32).reshape(3, 2, 1)])
    assert y.flatten().tolist() == [23.0, 67.0, 127.0]

    x = rng.standard_normal((2, 3, 7, 6)).astype(np.float32)
    w = rng.standard_normal((4, 3, 3, 5)).astype(np.float32)
    for sy, sx, py, px in ((1, 1, 1, 2), (2, 1, 0, 2), (1, 3, 2, 2)):
        g = Graph()
        g.output(g.conv(g.input([2, 3, 7, 6]), g.constant([4, 3, 3, 5], w), sy, sx, py, px))
        (y,) = cpu_eval_graph(g, 0, [x])
        xp = np.pad(x.astype(np.float64), ((0, 0), (0, 0), (py, py), (px, px)))
        oh, ow = (7 + 2 * py - 3) // sy + 1, (6 + 2 * px - 5) // sx + 1
        ref = np.zeros((2, 4, oh, ow))
        for oy in range(oh):
            for ox in range(ow):
                patch = xp[:, :, oy * sy:oy * sy + 3, ox * sx:ox * sx + 5]  # cross-correlation, no kernel flip
                ref[:, :, oy, ox] = np.einsum("nchw,kchw->nk", patch, w.astype(np.float64))
        close(y, ref)
    # fused conv scalar case of kn-cuda-sys/tests/fused.rs:32-59: -1 * 10 + 2 (res) + 3 (bias) = -5
    g = Graph()
    xi = g.input([1, 1, 1, 1])
    res = g.input([1, 1, 1, 1])
    y = g.add(g.add(g.conv(xi, g.constant([1, 1, 1, 1], [10.0]), 1, 1, 0, 0), g.constant([1, 1, 1, 1], [3.0])), res)
    g.output(y)
    (y,) = cpu_eval_graph(g, 0, [np.full((1, 1, 1, 1), -1.0, np.float32), np.full((1, 1, 1, 1), 2.0, np.float32)])
    assert y.item() == -5.0


def test_layout_ops_against_numpy_indexing():
    rng = np.random.default_rng(4)
    x = rng.standard_normal((4, 5, 6)).astype(np.float32)
    g = Graph()
    xi = g.input([4, 5, 6])
    outs = [g.permute(xi, [2, 0, 1]), g.slice(xi, 1, 1, 5, 2), g.flip(xi, 2), g.broadcast(g.view(g.slice(xi, 0, 0, 1), [5, 6]), [3, 5, 6]),
            g.repeat(xi, 1, 2), g.repeat_interleave(xi, 1, 2), g.index(xi, 2, 3), g.concat([xi, g.flip(xi, 0)], 0),
            g.view(xi, [20, 6]), g.pad(xi, [(1, 0), (0, 0), (0, 2)], g.scalar(7.0))]
    g.output_all(outs)
    ys = cpu_eval_graph(g, 0, [x])
    expected = [x.transpose(2, 0, 1), x[:, 1:5:2], x[:, :, ::-1], np.broadcast_to(x[0], (3, 5, 6)), np.tile(x, (1, 2, 1)),
                np.repeat(x, 2, axis=1), x[:, :, 3], np.concatenate([x, x[::-1]], 0), x.reshape(20, 6),
                np.pad(x, ((1, 0), (0, 0), (0, 2)), constant_values=7.0)]
    for y, e in zip(ys, expected):
        assert np.array_equal(y, e)


def test_gather_semantics():
    x = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    g = Graph()
    xi = g.input([2, 3, 4])
    idx = g.input([5], DType.I64)
    g.output(g.gather(xi, 1, idx))
    (y,) = cpu_eval_graph(g, 0, [x, np.array([2, 0, 0, 1, 2], np.int64)])
    assert np.array_equal(y, x[:, [2, 0, 0, 1, 2], :])
    with pytest.raises(OracleError, match="out of bounds"):  # cpu.rs:327
        cpu_eval_graph(g, 0, [x, np.array([3, 0, 0, 1, 2], np.int64)])
    with pytest.raises(OracleError, match="negative"):  # cpu.rs:318-321
        cpu_eval_graph(g, 0, [x, np.array([-1, 0, 0, 1, 2], np.int64)])


def test_value_cast_follows_rust_as_semantics():
    """dtype.rs:323-353: through f64 and i128; float -> int saturates at the i128 bounds, NaN -> 0, then the
    integer is truncated (wraps) to the target width; int -> float goes through f64; bool is `!= 0`."""
    f = np.array([0.0, -0.0, 1.9, -1.9, 255.0, 256.0, 300.7, -129.0, 3e9, -3e9, 1e19, -1e19, 2.0 ** 64, 1e30, 1e39, -1e39, np.nan,
                  np.inf, -np.inf], np.float64)
    g = Graph()
    x = g.input([len(f)], DType.F64)
    targets = [DType.I8, DType.U8, DType.I16, DType.U16, DType.I32, DType.U32, DType.I64, DType.U64, DType.BOOL, DType.F32]
    g.output_all([g.value_cast(x, t) for t in targets])
    ys = cpu_eval_graph(g, 0, [f])

    def rust_i128(v):
        if np.isnan(v):
            return 0
        if v >= 2.0 ** 127:
            return 2 ** 127 - 1
        if v < -2.0 ** 127:
            return -2 ** 127
        return int(v)  # truncation toward zero, exact for floats

    for t, y in zip(targets[:8], ys[:8]):
        bits = t.numpy.itemsize * 8
        exp = []
        for v in f:
            w = rust_i128(v) & ((1 << bits) - 1)
            if t.numpy.kind == "i" and w >= 1 << (bits - 1):
                w -= 1 << bits
            exp.append(w)
        assert y.tolist() == exp, t
    assert ys[8].tolist() == [bool(v != 0) for v in f]  # NaN != 0 is true
    assert np.array_equal(ys[9], f.astype(np.float32), equal_nan=True)
    # int -> f32 rounds twice (i64 -> f64 -> f32)
    g = Graph()
    xi = g.input([2], DType.I64)
    g.output(g.value_cast(xi, DType.F32))
    v = np.array([2 ** 53 + 1, -(2 ** 62) - 12345], np.int64)
    (y,) = cpu_eval_graph(g, 0, [v])
    assert np.array_equal(y, v.astype(np.float64).astype(np.float32))


def test_integer_arithmetic_wraps():
    g = Graph()
    a = g.input([4], DType.I8)
    b = g.input([4], DType.I8)
    g.output_all([g.add(a, b), g.sub(a, b), g.mul(a, b), g.unary(UnaryOp.NEG, a), g.unary(UnaryOp.ABS, a),
                  g.binary(BinaryOp.DIV, a, b), g.binary(BinaryOp.MIN, a, b), g.binary(BinaryOp.MAX, a, b)])
    av = np.array([127, -128, 100, -7], np.int8)
    bv = np.array([1, -1, 3, 2], np.int8)
    ys = cpu_eval_graph(g, 0, [av, bv])
    a16, b16 = av.astype(np.int16), bv.astype(np.int16)
    wrap = lambda v: ((v + 128) % 256 - 128).astype(np.int8)
    assert np.array_equal(ys[0], wrap(a16 + b16)) and np.array_equal(ys[1], wrap(a16 - b16))
    assert np.array_equal(ys[2], wrap(a16 * b16))
    assert np.array_equal(ys[3], wrap(-a16)) and np.array_equal(ys[4], wrap(np.abs(a16)))
    assert ys[5].tolist() == [127, -128, 33, -3]  # division truncates toward zero, MIN / -1 wraps
    assert np.array_equal(ys[6], np.minimum(av, bv)) and np.array_equal(ys[7], np.maximum(av, bv))


def test_float_min_max_ignore_nan():
    """Rust's f32::min / max return the other operand when one is NaN (graph.rs:1727-1728)"""
    g = Graph()
    a = g.input([3])
    b = g.input([3])
    g.output_all([g.binary(BinaryOp.MIN, a, b), g.binary(BinaryOp.MAX, a, b)])
    lo, hi = cpu_eval_graph(g, 0, [np.array([np.nan, 1.0, np.nan], np.float32), np.array([2.0, np.nan, np.nan], np.float32)])
    assert lo[0] == 2.0 and lo[1] == 1.0 and np.isnan(lo[2]) and hi[0] == 2.0 and hi[1] == 1.0 and np.isnan(hi[2])


def test_f16_operations_round_once_from_f64_results():
    """f16 (not in the reference IR): every operation is the f64 library result rounded to f16, up to the last
    f16 bit (f32 arithmetic before the rounding can move a value that sits next to a rounding boundary)."""
    rng = np.random.default_rng(40)

    def ulps(a, b):
        a, b = np.asarray(a, np.float16), np.asarray(b, np.float16)
        assert a.shape == b.shape and a.dtype == np.float16
        ia, ib = a.view(np.int16).astype(np.int32), b.view(np.int16).astype(np.int32)
        ia, ib = np.where(ia < 0, -(ia & 0x7FFF), ia), np.where(ib < 0, -(ib & 0x7FFF), ib)
        return int(np.max(np.abs(ia - ib)))

    x = rng.standard_normal((6, 40)).astype(np.float16)
    w = (rng.standard_normal((40, 9)) * 0.3).astype(np.float16)
    x64, w64 = x.astype(np.float64), w.astype(np.float64)
    g = Graph()
    xi = g.input([6, 40], DType.F16)
    mm = g.mat_mul(xi, g.constant([40, 9], w))
    g.output_all([mm, g.softmax(xi, 1), g.layernorm(xi, 1, 1e-3), g.reduce(xi, [1], ReduceOp.SUM),
                  g.reduce(xi, [0], ReduceOp.MEAN), g.mul(xi, xi), g.unary(UnaryOp.EXP, xi)])
    got = cpu_eval_graph(g, 0, [x])
    e = np.exp(x64 - x64.max(axis=1, keepdims=True))
    mean = x64.mean(axis=1, keepdims=True)
    var = ((x64 - mean) ** 2).mean(axis=1, keepdims=True)
    want = [x64 @ w64, e / e.sum(axis=1, keepdims=True), (x64 - mean) / np.sqrt(var + 1e-3), x64.sum(axis=1),
            x64.mean(axis=0), x64 * x64, np.exp(x64)]
    for y, t in zip(got, want):
        assert y.dtype == np.float16
        assert ulps(y, t.astype(np.float16)) <= 1
    # a long sum accumulates in f32, not f16: an f16 accumulator would get stuck at 2048 (2048 + 1 rounds to 2048)
    long = np.concatenate([np.ones(4096), np.full(4096, 2.0 ** -10)]).astype(np.float16)
    g = Graph()
    g.output(g.reduce(g.input([8192], DType.F16), [0], ReduceOp.SUM))
    (s,) = cpu_eval_graph(g, 0, [long])
    assert s.dtype == np.float16 and float(s) == 4100.0
