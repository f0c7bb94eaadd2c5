"""Graph test cases mirroring kn-cuda-eval/tests/root/graphs.rs (line numbers in each docstring).

Every case returns `(graph, batch_size, inputs, expected_or_None)`. Expected values are the ones the reference's
test holds; where the reference passes `None` the CPU path is the oracle, so any seeded input keeps the intent.
"""
import itertools

import numpy as np

from kyanite_amd import BATCH, BinaryOp, DType, Graph, OpKind, REDUCE_ALL, ReduceOp, Size, UnaryOp, optimize_graph
from runner import linspace_tensor, linspace_vec, range_vec, rng_tensor

CASES = {}


def case(fn):
    CASES[fn.__name__] = fn
    return fn


def f32(shape, data):
    return np.asarray(data, dtype=np.float32).reshape(shape)


@case
def empty():
    """graphs.rs:17-19"""
    return Graph(), 8, [], []


@case
def copy():
    """graphs.rs:22-41"""
    g = Graph()
    fixed = g.input([10])
    batch = g.input([BATCH])
    g.output_all([fixed, batch])
    a, b = linspace_tensor(10), linspace_tensor(8)
    return g, 8, [a, b], [a, b]


@case
def slice_():
    """graphs.rs:44-61"""
    g = Graph()
    x = g.input([10, 4])
    indexed = g.index(x, 1, 0)
    g.output_all([indexed, g.slice(x, 0, 0, 2), g.slice(indexed, 0, 0, 2)])
    return g, 0, [linspace_tensor(10, 4)], None


@case
def flip():
    """graphs.rs:64-90, expected values from the reference"""
    g = Graph()
    x = g.constant([2, 3], [0.0, 1.0, 2.0, 3.0, 4.0, 5.0])
    first_once = g.flip(x, 0)
    first_twice = g.flip(first_once, 0)
    other_once = g.flip(x, 1)
    other_twice = g.flip(other_once, 1)
    combined = g.flip(first_once, 1)
    g.output_all([first_once, first_twice, other_once, other_twice, combined])
    expected = [
        f32((2, 3), [3, 4, 5, 0, 1, 2]), f32((2, 3), [0, 1, 2, 3, 4, 5]), f32((2, 3), [2, 1, 0, 5, 4, 3]),
        f32((2, 3), [0, 1, 2, 3, 4, 5]), f32((2, 3), [5, 4, 3, 2, 1, 0]),
    ]
    return g, 0, [], expected


@case
def flip_conv():
    """graphs.rs:93-104"""
    g = Graph()
    x = g.input([2, 4, 8, 8])
    flipped = g.flip(x, 3)
    w = g.constant([4, 4, 3, 3], linspace_vec(4 * 4 * 3 * 3))
    g.output(g.conv(flipped, w, 1, 1, 1, 1))
    return g, 0, [linspace_tensor(2, 4, 8, 8)], None


@case
def repeat():
    """graphs.rs:107-122"""
    g = Graph()
    x = g.input([2, 3])
    g.output_all([g.repeat(x, 0, 0), g.repeat(x, 0, 2), g.repeat(x, 1, 0), g.repeat(x, 1, 2)])
    return g, 0, [rng_tensor(np.random.default_rng(0), 2, 3)], None


@case
def repeat_interleave():
    """graphs.rs:125-138"""
    g = Graph()
    x = g.input([2, 3])
    g.output_all([g.repeat_interleave(x, 0, 0), g.repeat_interleave(x, 0, 2), g.repeat_interleave(x, 1, 0),
                  g.repeat_interleave(x, 1, 2)])
    return g, 0, [rng_tensor(np.random.default_rng(0), 2, 3)], None


@case
def repeat_manual():
    """graphs.rs:141-158, expected values from the reference"""
    g = Graph()
    x = g.input([3])
    g.output_all([g.repeat(x, 0, 2), g.repeat_interleave(x, 0, 2)])
    return g, 0, [f32((3,), [1, 2, 3])], [f32((6,), [1, 2, 3, 1, 2, 3]), f32((6,), [1, 1, 2, 2, 3, 3])]


@case
def gather_simple_axis_0():
    """graphs.rs:161-172"""
    g = Graph()
    x = g.constant([2, 3], [7.0, 7.1, 7.2, 7.3, 7.4, 7.5])
    index = g.constant([4], np.array([0, 1, 1, 0], np.uint32))
    g.output(g.gather(x, 0, index))
    return g, 0, [], [f32((4, 3), [7.0, 7.1, 7.2, 7.3, 7.4, 7.5, 7.3, 7.4, 7.5, 7.0, 7.1, 7.2])]


@case
def gather_simple_axis_1():
    """graphs.rs:175-185"""
    g = Graph()
    x = g.constant([2, 3], [7.0, 7.1, 7.2, 7.3, 7.4, 7.5])
    index = g.constant([4], np.array([0, 2, 1, 0], np.uint32))
    g.output(g.gather(x, 1, index))
    return g, 0, [], [f32((2, 4), [7.0, 7.2, 7.1, 7.0, 7.3, 7.5, 7.4, 7.3])]


@case
def gather_complex_axis_0():
    """graphs.rs:188-199"""
    g = Graph()
    x = g.input([3, 2])
    indices = g.constant([2, 2], np.array([0, 1, 1, 2], np.uint32))
    g.output(g.gather(x, 0, indices))
    return (g, 0, [f32((3, 2), [1.0, 1.2, 2.3, 3.4, 4.5, 5.7])],
            [f32((2, 2, 2), [1.0, 1.2, 2.3, 3.4, 2.3, 3.4, 4.5, 5.7])])


@case
def gather_complex_axis_1():
    """graphs.rs:202-213"""
    g = Graph()
    x = g.input([3, 3])
    indices = g.constant([1, 2], np.array([0, 2], np.uint32))
    g.output(g.gather(x, 1, indices))
    return (g, 0, [f32((3, 3), [1.0, 1.2, 1.9, 2.3, 3.4, 3.9, 4.5, 5.7, 5.9])],
            [f32((3, 1, 2), [1.0, 1.9, 2.3, 3.9, 4.5, 5.9])])


@case
def gather_size_0():
    """graphs.rs:216-233"""
    g = Graph()
    x = g.input([8, 4])
    indices = g.constant([0], np.array([], np.uint32))
    o0 = g.gather(x, 0, indices)
    o1 = g.gather(x, 1, indices)
    g.output_all([o0, o1])
    assert g[o0].shape == [0, 4] and g[o1].shape == [8, 0]
    return g, 0, [linspace_tensor(8, 4)], None


@case
def gather_as_index():
    """graphs.rs:236-259: a gather with a single constant index has to become a slice"""
    g = Graph()
    x = g.input([16, 8, 4])
    index = g.scalar(4, DType.U32)
    indices = g.view(index, [1])
    indices_repeat = g.broadcast(indices, [3])
    g.output_all([g.gather(x, 1, indices), g.gather(x, 1, indices_repeat)])
    for v in g.values():
        assert g[v].op != OpKind.GATHER, "gather should have been replaced by an index operation"
    return g, 0, [rng_tensor(np.random.default_rng(0), 16, 8, 4)], None


@case
def gather_real():
    """gather with non constant indices, several index dtypes (not in the reference; its kernel is generic in the
    index type, gather.rs:30-129)"""
    g = Graph()
    x = g.input([5, 7, 3])
    i8 = g.input([4], DType.I8)
    u64 = g.input([6], DType.U64)
    g.output_all([g.gather(x, 0, i8), g.gather(x, 1, u64), g.gather(x, 2, i8)])
    rng = np.random.default_rng(1)
    return (g, 0, [rng_tensor(rng, 5, 7, 3), np.array([0, 2, 1, 2], np.int8), np.array([6, 0, 3, 3, 1, 5], np.uint64)], None)


@case
def gather_whole_rows_as_vectors():
    """a gather whose fastest result axis is not the gathered one moves 16 bytes per thread: an embedding lookup in
    f16 (enough of it for four loads per thread), channels selected out of [n, c, hw] in f32, rows of 10 floats (8 byte
    vectors), bytes (16 per vector), rows cut out of a wider tensor (no alignment: element by element) and an index
    tensor that is an input"""
    g = Graph()
    rng = np.random.default_rng(182)
    inputs = []

    def inp(shape, dtype=DType.F32):
        if np.dtype(dtype.numpy).kind == "f":
            inputs.append(rng.standard_normal(shape).astype(dtype.numpy))
        else:
            inputs.append(rng.integers(0, 200, shape).astype(dtype.numpy))
        return g.input(list(shape), dtype)

    def idx(count, below):
        return g.constant([count], rng.integers(0, below, count).astype(np.int64), DType.I64)

    g.output(g.gather(inp((5000, 2048), DType.F16), 0, idx(5000, 5000)))
    g.output(g.gather(inp((37, 50, 24)), 1, idx(70, 50)))
    g.output(g.gather(inp((64, 10)), 0, idx(33, 64)))
    g.output(g.gather(inp((300, 48), DType.U8), 0, idx(500, 300)))
    g.output(g.gather(g.slice(inp((40, 25)), 1, 1, 25), 0, idx(90, 40)))
    where = g.input([11], DType.I32)
    g.output(g.gather(inp((9, 6, 32)), 0, where))
    inputs.insert(len(inputs) - 1, rng.integers(0, 9, 11).astype(np.int32))
    return g, 0, inputs, None


@case
def gather_along_the_contiguous_axis_through_lds():
    """a gather along the axis the input is contiguous in, with many rows and a good share of every row wanted: a
    workgroup stages its row in LDS and picks from there. Rows of whole 16 byte vectors, rows of halves that only
    allow 4 byte vectors, bytes, a row cut out of a wider tensor (element by element), indices that are an input,
    and a result that a concatenation takes on"""
    g = Graph()
    rng = np.random.default_rng(183)
    inputs = []

    def inp(shape, dtype=DType.F32):
        if np.dtype(dtype.numpy).kind == "f":
            inputs.append(rng.standard_normal(shape).astype(dtype.numpy))
        else:
            inputs.append(rng.integers(0, 200, shape).astype(dtype.numpy))
        return g.input(list(shape), dtype)

    def idx(count, below):
        return g.constant([count], rng.integers(0, below, count).astype(np.int64), DType.I64)

    g.output(g.gather(inp((200, 300)), 1, idx(150, 300)))
    g.output(g.gather(inp((130, 7, 90), DType.F16), 2, idx(64, 90)))
    g.output(g.gather(inp((256, 100), DType.U8), 1, idx(100, 100)))
    g.output(g.gather(g.slice(inp((140, 131)), 1, 1, 129), 1, idx(200, 128)))
    where = g.input([77], DType.I32)
    inputs.append(rng.integers(0, 96, 77).astype(np.int32))
    g.output(g.gather(inp((128, 96)), 1, where))
    g.output(g.concat([g.gather(inp((300, 64)), 1, idx(64, 64)), inp((300, 8))], 1))
    return g, 0, inputs, None


@case
def square_written_as_a_power():
    """`x ** 2` and `x ** 3` with a constant exponent are emitted as products and `x ** 0.5` as a square root:
    negative values, zeros of both signs, infinities, NaN, values whose square overflows or underflows, f16; other
    constant exponents stay with the library"""
    g = Graph()
    rng = np.random.default_rng(187)
    special = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 3e19, -3e19, 1e-23, -1e-30, 2.5, -7.25], np.float32)
    values = np.concatenate([special, rng.standard_normal(3000).astype(np.float32) * 100])
    x = g.input([len(values)])
    g.output(g.pow(x, g.scalar(2.0, DType.F32)))
    g.output(g.pow(x, g.scalar(0.5, DType.F32)))
    g.output(g.pow(x, g.scalar(3.0, DType.F32)))
    g.output(g.pow(x, g.scalar(1.5, DType.F32)))
    h = g.input([len(values)], DType.F16)
    g.output(g.add(g.pow(h, g.scalar(2.0, DType.F16)), g.scalar(1.0, DType.F16)))
    g.output(g.pow(h, g.scalar(0.5, DType.F16)))
    return g, 0, [values, values.astype(np.float16)], None


@case
def linear():
    """graphs.rs:262-283, expected values from the reference"""
    g = Graph()
    x = g.input([1, 4])
    w = g.constant([2, 4], range_vec(8))
    b = g.constant([1, 2], [-10.0, 10.0])
    lin = g.linear(x, w)
    g.output_all([lin, g.add(lin, b)])
    return g, 0, [f32((1, 4), [0, 1, 2, 3])], [f32((1, 2), [14, 38]), f32((1, 2), [4, 48])]


@case
def linear_sliced():
    """graphs.rs:286-297"""
    g = Graph()
    left = g.input([8, 4])
    left_sliced = g.slice(left, 0, 0, 8, 2)
    right = g.input([4, 3])
    g.output(g.mat_mul(left_sliced, right))
    return g, 0, [linspace_tensor(8, 4), linspace_tensor(4, 3)], None


@case
def mat_mul_broadcast():
    """graphs.rs:300-335"""
    shapes = [([4, 2], [2, 3], [4, 3]), ([8, 4, 2], [2, 3], [8, 4, 3]), ([4, 2], [8, 2, 3], [8, 4, 3]),
              ([8, 4, 2], [8, 2, 3], [8, 4, 3]), ([1, 1, 1, 4, 2], [8, 1, 2, 3], [1, 8, 1, 4, 3])]
    rng = np.random.default_rng(0)
    g = Graph()
    inputs = []
    for ls, rs, os_ in shapes:
        inputs += [rng_tensor(rng, *ls), rng_tensor(rng, *rs)]
        result = g.mat_mul(g.input(ls), g.input(rs))
        assert g[result].shape == os_
        g.output(result)
    return g, 0, inputs, None


def _mat_mul_transpose(ta, tb):
    g = Graph()
    sa, sb = [4, 5, 6], [4, 6, 3]
    if ta:
        sa = [4, 6, 5]
    if tb:
        sb = [4, 3, 6]
    a = g.constant(sa, linspace_vec(4 * 5 * 6))
    b = g.constant(sb, linspace_vec(4 * 6 * 3))
    if ta:
        a = g.permute(a, [0, 2, 1])
    if tb:
        b = g.permute(b, [0, 2, 1])
    result = g.batched_mat_mul(a, b)
    assert g[result].shape == [4, 5, 3]
    g.output(result)
    return g, 0, [], None


for _ta, _tb in itertools.product([True, False], repeat=2):
    CASES[f"mat_mul_transpose_{int(_ta)}{int(_tb)}"] = (lambda ta=_ta, tb=_tb: _mat_mul_transpose(ta, tb))  # graphs.rs:338-376


@case
def horizontal_1x1_conv():
    """graphs.rs:379-390"""
    g = Graph()
    x = g.constant([2, 4, 1, 8], linspace_vec(2 * 4 * 8))
    f = g.constant([3, 4, 1, 1], linspace_vec(3 * 4))
    out = g.conv(x, f, 1, 1, 0, 0)
    assert g[out].shape == [2, 3, 1, 8]
    g.output(out)
    return g, 0, [], None


@case
def vertical_1x1_conv():
    """graphs.rs:393-404"""
    g = Graph()
    x = g.constant([2, 4, 8, 1], linspace_vec(2 * 4 * 8))
    f = g.constant([3, 4, 1, 1], linspace_vec(3 * 4))
    out = g.conv(x, f, 1, 1, 0, 0)
    assert g[out].shape == [2, 3, 8, 1]
    g.output(out)
    return g, 0, [], None


@case
def fuse_clamp():
    """graphs.rs:407-425, expected values from the reference"""
    g = Graph()
    curr = g.input([BATCH])
    inf = float("inf")
    curr = g.clamp(curr, -5.0, inf)
    curr = g.clamp(curr, -inf, 2.0)
    curr = g.clamp(curr, 0.0, 1.0)
    curr = g.clamp(curr, -1.0, 2.0)
    g.output(curr)
    return g, 5, [f32((5,), [-2.0, 0.0, 0.5, 1.0, 2.0])], [f32((5,), [0.0, 0.0, 0.5, 1.0, 1.0])]


def _ele_broadcast(op):
    g = Graph()
    left = g.constant([2, 3, 4], linspace_vec(24))
    for shp in ([], [1, 1, 1], [2, 3, 4], [2, 1, 4]):
        size = int(np.prod(shp)) if shp else 1
        right = g.constant(shp, linspace_vec(size))
        g.output(g.binary(op, left, right))
    return g, 0, [], None


for _op in (BinaryOp.ADD, BinaryOp.SUB, BinaryOp.MUL, BinaryOp.MIN, BinaryOp.MAX, BinaryOp.DIV):
    CASES[f"ele_broadcast_{_op.name.lower()}"] = (lambda op=_op: _ele_broadcast(op))  # graphs.rs:428-452 (+ div)


@case
def add_broadcast():
    """graphs.rs:455-473, expected values from the reference"""
    g = Graph()
    left = g.constant([2, 2, 2], [0.0, 1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0])
    right = g.constant([1, 2, 2], [0.0, 1.0, 2.0, 3.0])
    scalar = g.constant([], [10.0])
    g.output_all([g.add(left, right), g.add(right, left), g.add(right, scalar)])
    e01 = f32((2, 2, 2), [0, 2, 4, 6, 4, 6, 8, 10])
    return g, 0, [], [e01, e01, f32((1, 2, 2), [10, 11, 12, 13])]


@case
def affine_single_element():
    """graphs.rs:476-502, closed form from the reference"""
    x = f32((8, 1, 1, 1), range_vec(8))
    expected = ((x + 1.0) * 2.0 * 10.0 + 3.0) * 4.0
    g = Graph()
    cs = [1, 1, 1, 1]
    bias_0, scale_0, filt = g.constant(cs, [1.0]), g.constant(cs, [2.0]), g.constant(cs, [10.0])
    bias_1, scale_1 = g.constant(cs, [3.0]), g.constant(cs, [4.0])
    curr = g.input([8, 1, 1, 1])
    curr = g.mul(g.add(curr, bias_0), scale_0)
    curr = g.conv(curr, filt, 1, 1, 0, 0)
    curr = g.mul(g.add(curr, bias_1), scale_1)
    g.output(curr)
    return g, 0, [x], [expected.astype(np.float32)]


@case
def affine_add_twice():
    """graphs.rs:505-523"""
    g = Graph()
    x = g.input([BATCH, 1, 1, 1])
    w1, w2 = g.constant([1, 1, 1, 1], [1.0]), g.constant([1, 1, 1, 1], [2.0])
    g.output(g.add(g.add(x, w1), w2))
    return g, 2, [f32((2, 1, 1, 1), [0, 1])], [f32((2, 1, 1, 1), [3, 4])]


@case
def affine_single_div():
    """graphs.rs:526-536"""
    g = Graph()
    left = g.constant([2, 3], range_vec(6))
    right = g.scalar(2.0)
    g.output(g.binary(BinaryOp.DIV, left, right))
    return g, 0, [], [f32((2, 3), [0.0, 0.5, 1.0, 1.5, 2.0, 2.5])]


@case
def affine_multiple_channels():
    """graphs.rs:539-564"""
    x = f32((8, 3, 1, 1), range_vec(24))
    g = Graph()
    bias_0 = g.constant([1, 3, 1, 1], [1.0, 2.0, 3.0])
    scale_0 = g.constant([1, 3, 1, 1], [2.0, 3.0, 4.0])
    filt = g.constant([2, 3, 1, 1], [10.0, 20.0, 30.0, 40.0, 50.0, 60.0])
    bias_1 = g.constant([1, 2, 1, 1], [3.0, 4.0])
    scale_1 = g.constant([1, 2, 1, 1], [4.0, 5.0])
    curr = g.input([8, 3, 1, 1])
    curr = g.mul(g.add(curr, bias_0), scale_0)
    curr = g.conv(curr, filt, 1, 1, 0, 0)
    curr = g.mul(g.add(curr, bias_1), scale_1)
    g.output(curr)
    # independent closed form (numpy, f64)
    xb = (x.astype(np.float64)[:, :, 0, 0] + [1, 2, 3]) * [2, 3, 4]
    w = np.array([[10, 20, 30], [40, 50, 60]], np.float64)
    expected = ((xb @ w.T + [3, 4]) * [4, 5]).astype(np.float32).reshape(8, 2, 1, 1)
    return g, 0, [x], [expected]


@case
def conv_padding():
    """graphs.rs:567-592"""
    g = Graph()
    i0 = g.input([1, 1, 1, 1])
    i1 = g.input([1, 1, 8, 8])
    filt = g.constant([1, 1, 3, 3], range_vec(9))
    g.output_all([g.conv(i0, filt, 1, 1, 1, 1), g.conv(i0, filt, 1, 1, 4, 4), g.conv(i1, filt, 1, 1, 1, 1),
                  g.conv(i1, filt, 1, 1, 4, 1)])
    return g, 0, [f32((1, 1, 1, 1), [1.0]), linspace_tensor(1, 1, 8, 8)], None


@case
def affine_padding():
    """graphs.rs:595-613"""
    g = Graph()
    filt = g.constant([5, 3, 3, 3], linspace_vec(5 * 27))
    bias_0 = g.constant([1, 3, 1, 1], linspace_vec(3))
    bias_1 = g.constant([1, 5, 1, 1], linspace_vec(5))
    curr = g.input([8, 3, 8, 8])
    curr = g.add(curr, bias_0)
    curr = g.conv(curr, filt, 1, 1, 1, 1)
    curr = g.add(curr, bias_1)
    g.output(curr)
    return g, 0, [linspace_tensor(8, 3, 8, 8)], None


def _channel_batchnorm(g, x):
    """graphs.rs:645-661"""
    c = g[x].shape[1].fixed_factor
    cs = [1, c, 1, 1]
    mean, var, scale, bias = (g.constant(cs, linspace_vec(c)) for _ in range(4))
    curr = g.add(x, mean)
    curr = g.mul(curr, var)
    curr = g.mul(curr, scale)
    return g.add(curr, bias)


@case
def pre_act_resnet():
    """graphs.rs:616-643"""
    g = Graph()
    x = g.input([8, 3, 8, 8])
    f_init = g.constant([5, 3, 3, 3], linspace_vec(5 * 27))
    f_tower = g.constant([5, 5, 3, 3], linspace_vec(5 * 45))
    f_policy = g.constant([2, 5, 1, 1], linspace_vec(10))
    tower = g.conv(x, f_init, 1, 1, 1, 1)
    for _ in range(2):
        curr = _channel_batchnorm(g, tower)
        curr = g.clamp(curr, 0.0, 6.0)
        curr = g.conv(curr, f_tower, 1, 1, 1, 1)
        curr = g.clamp(curr, 0.0, 6.0)
        curr = g.conv(curr, f_tower, 1, 1, 1, 1)
        tower = g.add(curr, tower)
    policy = g.conv(tower, f_policy, 1, 1, 0, 0)
    g.output_all([tower, policy])
    return g, 0, [linspace_tensor(8, 3, 8, 8)], None


@case
def fuse_res():
    """graphs.rs:664-687"""
    g = Graph()
    rng = np.random.default_rng(0)
    x = g.input([10, 4, 8, 8])
    other = g.input([10, 4, 8, 8])
    filt = g.constant([4, 4, 3, 3], linspace_vec(4 * 36))
    curr = g.conv(x, filt, 1, 1, 1, 1)
    curr = g.add(curr, other)
    curr = g.clamp(curr, 0.0, float("inf"))
    g.output(curr)
    return g, 0, [rng_tensor(rng, 10, 4, 8, 8), rng_tensor(rng, 10, 4, 8, 8)], None


@case
def concat():
    """graphs.rs:690-701"""
    g = Graph()
    a = g.constant([2, 3, 4], linspace_vec(24))
    b = g.constant([2, 1, 4], linspace_vec(8))
    c = g.constant([2, 8, 4], linspace_vec(64))
    g.output(g.concat([a, b, c], 1))
    return g, 0, [], None


@case
def pad():
    """graphs.rs:704-714"""
    g = Graph()
    a = g.constant([2, 3, 4], linspace_vec(24))
    zero = g.scalar(0.0)
    g.output(g.pad(a, [(0, 0), (1, 2), (2, 0)], zero))
    expected = np.pad(linspace_vec(24).reshape(2, 3, 4), [(0, 0), (1, 2), (2, 0)])
    return g, 0, [], [expected]


@case
def permute():
    """graphs.rs:719-731: all 24 permutations of a rank-4 tensor; expected from numpy.transpose"""
    g = Graph()
    data = range_vec(120).reshape(2, 3, 4, 5)
    a = g.constant([2, 3, 4, 5], data)
    expected = []
    for p in itertools.permutations(range(4)):
        g.output(g.permute(a, list(p)))
        expected.append(np.ascontiguousarray(data.transpose(p)))
    return g, 0, [], expected


@case
def chain():
    """graphs.rs:734-760, expected values from the reference"""
    child = Graph()
    cx = child.input([2])
    cw = child.constant([1], [2.0])
    child.output(child.mul(cx, cw))
    parent = Graph()
    px = parent.input([2])
    pw = parent.constant([1], [3.0])
    pz = parent.add(px, pw)
    py = parent.call(child, [pz])
    assert len(py) == 1
    parent.output(py[0])
    return parent, 0, [f32((2,), [1, 2])], [f32((2,), [8, 10])]


@case
def repeated_conv():
    """graphs.rs:763-785"""
    g = Graph()
    w0 = g.constant([4, 4, 3, 3], np.linspace(-1, 1, 144).astype(np.float32))
    w1 = g.constant([4, 4, 3, 3], np.linspace(-2, 2, 144).astype(np.float32))
    x = g.input([BATCH, 4, 8, 8])
    a = x
    for _ in range(4):
        a = g.conv(a, w0, 1, 1, 1, 1)
    b = x
    for _ in range(4):
        b = g.conv(b, w1, 1, 1, 1, 1)
    g.output_all([a, b])
    return g, 2, [linspace_tensor(2, 4, 8, 8)], None


@case
def strided_conv():
    """graphs.rs:788-800"""
    g = Graph()
    rng = np.random.default_rng(0)
    x = g.input([BATCH, 3, 8, 8])
    filt = g.constant([16, 3, 3, 3], rng_tensor(rng, 16 * 27))
    out = g.conv(x, filt, 2, 4, 1, 1)
    assert g[out].shape == [BATCH, 16, 4, 2]
    g.output(out)
    return g, 4, [rng_tensor(rng, 4, 3, 8, 8)], None


@case
def softmax():
    """graphs.rs:803-819, includes -inf and a scaled input"""
    g = Graph()
    x = g.input([3, 3])
    r0 = g.softmax(x, 0)
    r1 = g.softmax(x, 1)
    scaled = g.mul(x, g.scalar(2.0))
    r2 = g.softmax(scaled, 0)
    g.output_all([r0, r1, r2])
    return g, 0, [f32((3, 3), [0.0, 0.0, 0.0, 1.0, 2.0, 3.0, 1.0, -1.0, -np.inf])], None


@case
def reduce_easy():
    """graphs.rs:822-836: all reduce ops on both axes, -inf included"""
    g = Graph()
    x = g.input([4, 3])
    for axis in (0, 1):
        for op in REDUCE_ALL:
            g.output(g.reduce(x, [axis], op))
    return g, 0, [f32((4, 3), [0.0, 0.0, 0.0, 1.0, 2.0, 3.0, 1.0, -1.0, -np.inf, 0.0, 1.0, 2.0])], None


@case
def reduce_mixed():
    """graphs.rs:839-848"""
    g = Graph()
    x = g.input([12, 3, 7, 9, 13])
    mixed = g.permute(x, [0, 3, 2, 1, 4])
    g.output(g.reduce(mixed, [1, 2, 4], ReduceOp.SUM))
    return g, 0, [linspace_tensor(12, 3, 7, 9, 13)], None


@case
def reduce_single():
    """graphs.rs:851-859"""
    g = Graph()
    x = g.input([4])
    g.output(g.reduce(x, [0], ReduceOp.SUM))
    return g, 0, [linspace_tensor(4)], None


@case
def softmax_single():
    """graphs.rs:862-870"""
    g = Graph()
    x = g.input([4])
    g.output(g.softmax(x, 0))
    return g, 0, [linspace_tensor(4)], None


def layernorm_pattern_graph():
    """graphs.rs:873-905: the mean / variance / sqrt / div pattern the optimizer has to recognise"""
    g = Graph()
    eps, axis = 1e-5, 2
    x = g.input([BATCH, 8, 32])
    reduced = [BATCH, 8, 1]
    const_2 = g.scalar(2.0)
    const_eps = g.scalar(eps)
    mean = g.view(g.reduce(x, [axis], ReduceOp.MEAN), reduced)
    zeroed = g.sub(x, mean)
    pw = g.pow(zeroed, const_2)
    var = g.view(g.reduce(pw, [axis], ReduceOp.MEAN), reduced)
    var = g.add(var, const_eps)
    std = g.unary(UnaryOp.SQRT, var)
    g.output(g.binary(BinaryOp.DIV, zeroed, std))
    return g


@case
def layernorm_fused():
    """graphs.rs:873-929: optimized graph must be exactly [Input, Layernorm{axis 2, eps 1e-5}]"""
    g = layernorm_pattern_graph()
    opt = optimize_graph(g)
    values = opt.values()
    assert len(values) == 2, str(opt)
    assert opt[values[0]].op == OpKind.INPUT
    info = opt[values[1]]
    assert info.op == OpKind.LAYERNORM and info.operands == [values[0]] and info.axes == [2]
    assert info.eps == np.float32(1e-5)
    return g, 2, [linspace_tensor(2, 8, 32)], None


@case
def scalar_scalar():
    """graphs.rs:932-940"""
    g = Graph()
    x = g.input([])
    g.output(g.unary(UnaryOp.EXP, x))
    return g, 0, [f32((), [2.0])], None


@case
def split_stride():
    """graphs.rs:943-959"""
    g = Graph()
    n = 4
    x = g.input([2 * n])
    g.output(g.slice(x, 0, 1, 2 * n + 1, 2))
    data = rng_tensor(np.random.default_rng(0), 2 * n)
    return g, 0, [data], [data[1::2].copy()]


def _complex_multiply(new_axis):
    """graphs.rs:971-1065, expected from the reference's closed form"""
    batch, n, axis = 8, 32, 1
    g = Graph()
    a = g.input([batch, n * 2])
    b = g.input([batch, n * 2])
    if new_axis:
        a_split, b_split = g.view(a, [batch, n, 2]), g.view(b, [batch, n, 2])
        ar = g.view(g.slice(a_split, axis + 1, 0, 1), [batch, n])
        ai = g.view(g.slice(a_split, axis + 1, 1, 2), [batch, n])
        br = g.view(g.slice(b_split, axis + 1, 0, 1), [batch, n])
        bi = g.view(g.slice(b_split, axis + 1, 1, 2), [batch, n])
    else:
        ar = g.slice(a, axis, 0, n * 2, 2)
        ai = g.slice(a, axis, 1, n * 2 + 1, 2)
        br = g.slice(b, axis, 0, n * 2, 2)
        bi = g.slice(b, axis, 1, n * 2 + 1, 2)
    r = g.sub(g.mul(ar, br), g.mul(ai, bi))
    i = g.add(g.mul(ar, bi), g.mul(ai, br))
    extra = g.concat([g.view(r, [batch, n, 1]), g.view(i, [batch, n, 1])], axis + 1)
    g.output(g.view(extra, [batch, n * 2]))
    rng = np.random.default_rng(0)
    ia, ib = rng_tensor(rng, batch, n * 2), rng_tensor(rng, batch, n * 2)
    out = np.empty((batch, n * 2), np.float32)
    out[:, 0::2] = ia[:, 0::2] * ib[:, 0::2] - ia[:, 1::2] * ib[:, 1::2]
    out[:, 1::2] = ia[:, 0::2] * ib[:, 1::2] + ia[:, 1::2] * ib[:, 0::2]
    return g, 0, [ia, ib], [out]


CASES["complex_multiply_stride"] = lambda: _complex_multiply(False)
CASES["complex_multiply_new_axis"] = lambda: _complex_multiply(True)


# ---- cases beyond the reference's list: shapes that exercise the other kernel specialisations

@case
def layernorm_affine():
    """layernorm followed by gamma / beta on the normalised axis: planned as ONE row kernel"""
    g = Graph()
    rng = np.random.default_rng(3)
    x = g.input([BATCH, 96])
    gamma = g.constant([96], (1 + 0.1 * rng.standard_normal(96)).astype(np.float32))
    beta = g.constant([96], (0.1 * rng.standard_normal(96)).astype(np.float32))
    y = g.add(g.mul(g.layernorm(x, 1, 1e-5), gamma), beta)
    g.output(y)
    return g, 5, [rng.standard_normal((5, 96)).astype(np.float32)], None


@case
def layernorm_residual():
    """planner.rs:522-552: layernorm(alpha0 * a + alpha1 * b) with equally laid out operands"""
    g = Graph()
    rng = np.random.default_rng(4)
    a = g.input([4, 6, 40])
    b = g.input([4, 6, 40])
    s = g.add(g.mul(a, g.scalar(0.5)), b)
    g.output(g.layernorm(s, 2, 1e-3))
    g.output(g.layernorm(g.permute(a, [0, 2, 1]), 1, 1e-3))
    return g, 0, [rng.standard_normal((4, 6, 40)).astype(np.float32), rng.standard_normal((4, 6, 40)).astype(np.float32)], None


@case
def softmax_shapes():
    """rows shorter than a wave, rows spanning a workgroup, a strided (non innermost) softmax axis, odd lengths"""
    g = Graph()
    rng = np.random.default_rng(5)
    a = g.input([6, 1000])
    b = g.input([3, 37, 5])
    c = g.input([2, 4672])
    g.output_all([g.softmax(a, 1), g.softmax(b, 1), g.softmax(b, 2), g.softmax(c, 1), g.softmax(a, 0)])
    return g, 0, [rng.standard_normal((6, 1000)).astype(np.float32) * 3, rng.standard_normal((3, 37, 5)).astype(np.float32),
                  rng.standard_normal((2, 4672)).astype(np.float32)], None


@case
def row_kernel_long():
    """rows too long to sit in registers: the streaming variant"""
    g = Graph()
    rng = np.random.default_rng(6)
    a = g.input([3, 70001])
    g.output_all([g.softmax(a, 1), g.layernorm(a, 1, 1e-5)])
    return g, 0, [rng.standard_normal((3, 70001)).astype(np.float32)], None


@case
def reduce_shapes():
    """row and column strategies, vector and scalar tails, several dtypes"""
    g = Graph()
    rng = np.random.default_rng(7)
    a = g.input([33, 4096])
    b = g.input([1000, 7])
    c = g.input([5, 6, 64], DType.I32)
    d = g.input([300, 50], DType.F64)
    outs = [g.reduce(a, [1], ReduceOp.SUM), g.reduce(a, [0], ReduceOp.MAX), g.reduce(a, [0, 1], ReduceOp.MEAN),
            g.reduce(b, [0], ReduceOp.SUM), g.reduce(b, [1], ReduceOp.MIN), g.reduce(c, [1], ReduceOp.SUM),
            g.reduce(c, [0, 2], ReduceOp.MAX), g.reduce(c, [2], ReduceOp.PROD), g.reduce(d, [0], ReduceOp.SUM)]
    g.output_all(outs)
    return g, 0, [rng.standard_normal((33, 4096)).astype(np.float32), rng.standard_normal((1000, 7)).astype(np.float32),
                  rng.integers(-3, 4, (5, 6, 64)).astype(np.int32), rng.standard_normal((300, 50))], None


@case
def scalar_dtypes():
    """integer and bool arithmetic is bit exact: wrapping add / mul, min / max, value and bit casts"""
    g = Graph()
    rng = np.random.default_rng(8)
    a = g.input([257], DType.I8)
    b = g.input([257], DType.I8)
    u = g.input([64], DType.U32)
    f = g.input([64], DType.F32)
    p = g.input([33], DType.BOOL)
    q = g.input([33], DType.BOOL)
    outs = [g.add(a, b), g.mul(a, b), g.binary(BinaryOp.MIN, a, b), g.unary(UnaryOp.NEG, a), g.unary(UnaryOp.ABS, a),
            g.value_cast(a, DType.U16), g.value_cast(u, DType.F32), g.value_cast(f, DType.I32), g.value_cast(f, DType.U8),
            g.value_cast(f, DType.I64), g.bit_cast(f, DType.U32), g.bit_cast(u, DType.F32), g.value_cast(f, DType.BOOL),
            g.add(p, q), g.mul(p, q), g.sub(p, q), g.value_cast(p, DType.F32), g.value_cast(a, DType.F64),
            g.value_cast(f, DType.F16), g.value_cast(u, DType.I8)]
    g.output_all(outs)
    fv = (rng.standard_normal(64) * 1000).astype(np.float32)
    fv[:6] = [np.nan, np.inf, -np.inf, 3e9, -3e9, 1e20]
    uv = rng.integers(0, 2 ** 32, 64, dtype=np.uint64).astype(np.uint32)
    uv[:2] = [0x7fc00000, 0x3f800000]
    return g, 0, [rng.integers(-128, 128, 257).astype(np.int8), rng.integers(-128, 128, 257).astype(np.int8), uv, fv,
                  rng.integers(0, 2, 33).astype(np.bool_), rng.integers(0, 2, 33).astype(np.bool_)], None


@case
def strided_scalar():
    """elementwise work on permuted, flipped, sliced and broadcast operands, and a view that needs a copy"""
    g = Graph()
    rng = np.random.default_rng(9)
    a = g.input([6, 10, 8])
    b = g.input([8, 10])
    c = g.input([10, 1])
    t = g.permute(a, [0, 2, 1])                        # [6, 8, 10]
    s = g.add(t, g.flip(b, 1))                         # broadcast over the first axis, flipped last axis
    s = g.mul(s, g.permute(c, [1, 0]))                 # [1, 10] broadcast
    v = g.view(g.slice(s, 2, 0, 10, 2), [6, 40])       # strided slice, then a view that cannot be a stride edit
    g.output_all([s, v, g.unary(UnaryOp.TANH, v)])
    return g, 0, [rng.standard_normal((6, 10, 8)).astype(np.float32), rng.standard_normal((8, 10)).astype(np.float32),
                  rng.standard_normal((10, 1)).astype(np.float32)], None


@case
def tiny_mlp():
    """the smallest benchmark configuration: Linear 16->32 + bias, ReLU, Linear 32->10 + bias, softmax"""
    from kyanite_amd.configs import build_tiny_mlp
    g, inputs = build_tiny_mlp(seed=0)
    return g, 8, inputs, None


@case
def attention_block():
    """matmul -> scaled softmax -> matmul with the [1, 0, 2] permute after the last product (planner.rs:554-567)"""
    g = Graph()
    rng = np.random.default_rng(10)
    heads, seq, dim = 3, 20, 8
    q = g.input([seq, heads, dim])
    k = g.input([seq, heads, dim])
    v = g.input([seq, heads, dim])
    qh = g.permute(q, [1, 0, 2])
    kh = g.permute(k, [1, 2, 0])
    vh = g.permute(v, [1, 0, 2])
    scores = g.batched_mat_mul(qh, kh)
    probs = g.softmax(g.mul(scores, g.scalar(1.0 / np.sqrt(dim))), 2)
    out = g.permute(g.batched_mat_mul(probs, vh), [1, 0, 2])
    g.output(g.view(out, [seq, heads * dim]))
    return g, 0, [rng.standard_normal((seq, heads, dim)).astype(np.float32) for _ in range(3)], None


@case
def matmul_sizes():
    """products that do not line up with the 128 x 128 x 16 tiles, and a broadcast (zero stride) batch operand"""
    g = Graph()
    rng = np.random.default_rng(11)
    a = g.input([2, 130, 70])
    b = g.input([70, 257])
    c = g.input([2, 257, 3])
    ab = g.mat_mul(a, b)
    g.output_all([ab, g.mat_mul(ab, c)])
    return g, 0, [rng.standard_normal((2, 130, 70)).astype(np.float32), rng.standard_normal((70, 257)).astype(np.float32),
                  rng.standard_normal((2, 257, 3)).astype(np.float32)], None


@case
def conv_fused_all():
    """relu(conv + bias + res) with 130 output channels and 200 positions: partial tiles on both axes"""
    g = Graph()
    rng = np.random.default_rng(12)
    x = g.input([BATCH, 130, 5, 8])
    w = g.constant([130, 130, 3, 3], (rng.standard_normal((130, 130, 3, 3)) * 0.05).astype(np.float32))
    bias = g.constant([1, 130, 1, 1], rng.standard_normal(130).astype(np.float32))
    y = g.relu(g.add(g.add(g.conv(x, w, 1, 1, 1, 1), bias), x))
    g.output(y)
    return g, 5, [rng.standard_normal((5, 130, 5, 8)).astype(np.float32)], None


def _plane_conv_case(seed, batch, c_in, c_out, h, w, fused):
    """3x3 same-size convolutions whose image width is a power of two take the kernel that stages raw input planes"""
    g = Graph()
    rng = np.random.default_rng(seed)
    x = g.input([BATCH, c_in, h, w])
    filt = g.constant([c_out, c_in, 3, 3], (rng.standard_normal((c_out, c_in, 3, 3)) * 0.1).astype(np.float32))
    y = g.conv(x, filt, 1, 1, 1, 1)
    if fused:
        bias = g.constant([1, c_out, 1, 1], rng.standard_normal(c_out).astype(np.float32))
        y = g.add(y, bias)
        if c_in == c_out:
            y = g.add(y, x)
        y = g.relu(y)
    g.output(y)
    return g, batch, [rng.standard_normal((batch, c_in, h, w)).astype(np.float32)], None


@case
def conv_plane_8x8_odd_batch():
    """two images per tile, the last tile holds one image only"""
    return _plane_conv_case(20, 5, 16, 16, 8, 8, True)


@case
def conv_plane_4x4():
    """eight images per tile, partial last tile, partial tile of output channels"""
    return _plane_conv_case(21, 11, 8, 5, 4, 4, True)


@case
def conv_plane_16x16_wide_out():
    """one image spans two tiles; 130 output channels span two tiles of channels"""
    return _plane_conv_case(22, 2, 24, 130, 16, 16, False)


@case
def conv_plane_64x64():
    """a tile is two rows of the image, halo rows come from the neighbouring tiles' rows"""
    return _plane_conv_case(23, 1, 8, 8, 64, 64, True)


@case
def conv_plane_2x128():
    """a tile is one row of the image"""
    return _plane_conv_case(24, 2, 8, 3, 2, 128, False)


@case
def conv_plane_32x4():
    """narrow tall image: a tile is 32 rows"""
    return _plane_conv_case(25, 3, 16, 7, 64, 4, False)


# ---- f16 storage with f32 arithmetic (an extension over the reference IR, which has no f16)

def _f16(rng, *shape, scale=1.0):
    return (rng.standard_normal(shape) * scale).astype(np.float16)


@case
def f16_elementwise_chain():
    g = Graph()
    rng = np.random.default_rng(30)
    x = g.input([BATCH, 40], DType.F16)
    w = g.constant([1, 40], _f16(rng, 1, 40))
    y = g.mul(g.add(x, w), g.scalar(0.5, DType.F16))
    y = g.unary(UnaryOp.EXP, y)
    g.output_all([y, g.value_cast(y, DType.F32), g.value_cast(g.value_cast(y, DType.F32), DType.F16)])
    return g, 3, [_f16(rng, 3, 40)], None


@case
def f16_matmul_layouts():
    """K-contiguous (linear), N-contiguous and transposed-result operands, sizes that are multiples of 8"""
    g = Graph()
    rng = np.random.default_rng(31)
    a = g.input([72, 136], DType.F16)
    w = g.constant([200, 136], _f16(rng, 200, 136, scale=0.1))
    b = g.constant([136, 64], _f16(rng, 136, 64, scale=0.1))
    lin = g.linear(a, w)
    nn = g.mat_mul(a, b)
    g.output_all([lin, nn, g.permute(lin, [1, 0])])
    return g, 0, [_f16(rng, 72, 136)], None


@case
def f16_matmul_odd_sizes():
    """nothing is a multiple of 8: every operand goes through the element-wise loader"""
    g = Graph()
    rng = np.random.default_rng(32)
    a = g.input([3, 37, 45], DType.F16)
    b = g.input([3, 45, 51], DType.F16)
    g.output(g.batched_mat_mul(a, b))
    return g, 0, [_f16(rng, 3, 37, 45), _f16(rng, 3, 45, 51)], None


@case
def f16_matmul_big_tiles():
    """enough tiles for the 128 x 128 kernel, with partial tiles on both axes and a K tail"""
    g = Graph()
    rng = np.random.default_rng(33)
    a = g.input([16, 264, 200], DType.F16)
    b = g.input([16, 328, 200], DType.F16)
    g.output(g.batched_mat_mul(a, g.permute(b, [0, 2, 1])))
    return g, 0, [_f16(rng, 16, 264, 200, scale=0.2), _f16(rng, 16, 328, 200, scale=0.2)], None


@case
def f16_attention():
    """softmax(q k^T / sqrt(d) + causal mask) v, all in f16"""
    g = Graph()
    rng = np.random.default_rng(34)
    heads, seq, d = 4, 48, 32
    q = g.input([heads, seq, d], DType.F16)
    k = g.input([heads, seq, d], DType.F16)
    v = g.input([heads, seq, d], DType.F16)
    mask = np.where(np.tril(np.ones((seq, seq), bool)), 0.0, -np.inf).astype(np.float16)
    scores = g.batched_mat_mul(q, g.permute(k, [0, 2, 1]))
    scores = g.add(g.mul(scores, g.scalar(1.0 / np.sqrt(d), DType.F16)), g.constant([1, seq, seq], mask))
    out = g.batched_mat_mul(g.softmax(scores, 2), v)
    g.output(out)
    return g, 0, [_f16(rng, heads, seq, d), _f16(rng, heads, seq, d), _f16(rng, heads, seq, d)], None


@case
def f16_norms():
    """layernorm with gamma / beta, RMSNorm from primitives, mean / sum / max reductions"""
    g = Graph()
    rng = np.random.default_rng(35)
    x = g.input([BATCH, 6, 256], DType.F16)
    gamma = g.constant([1, 1, 256], (1.0 + 0.1 * rng.standard_normal(256)).astype(np.float16))
    beta = g.constant([1, 1, 256], _f16(rng, 256, scale=0.1))
    ln = g.add(g.mul(g.layernorm(x, 2, 1e-5), gamma), beta)
    ms = g.reduce(g.mul(x, x), [2], ReduceOp.MEAN)
    rms = g.unary(UnaryOp.SQRT, g.add(g.view(ms, [BATCH, 6, 1]), g.scalar(1e-5, DType.F16)))
    rn = g.mul(g.binary(BinaryOp.DIV, x, rms), gamma)
    g.output_all([ln, rn, g.reduce(x, [2], ReduceOp.SUM), g.reduce(x, [1], ReduceOp.MAX), g.softmax(x, 1)])
    return g, 5, [_f16(rng, 5, 6, 256)], None


# ---- miniature versions of the benchmark configurations (same builders, small sizes)

@case
def config_llama_small():
    from kyanite_amd.configs import build_llama
    g, make_inputs, _ = build_llama(seed=1, layers=2, seq=24, d_model=256, heads=4, ffn=352)
    return g, 0, make_inputs(), None


@case
def config_llama_f32_small():
    """the same decoder in f32: the tight f32 bar applies to every kernel of the graph"""
    from kyanite_amd.configs import build_llama
    g, make_inputs, _ = build_llama(seed=2, layers=1, seq=40, d_model=96, heads=3, ffn=200, dtype=DType.F32)
    return g, 0, make_inputs(), None


@case
def config_bandwidth_fused_chain_small():
    """configs[1] (a) through its own builder: the last axis has the benchmark's length (1024), so the same
    vectorised kernel variant with the broadcast a, b is generated"""
    from kyanite_amd.configs import build_fused_chain
    g, inputs, _ = build_fused_chain(seed=11, shape=(4, 128, 1024))
    return g, 0, inputs(), None


@case
def config_bandwidth_softmax_small():
    """configs[1] (b): rows of 512 like the benchmark's"""
    from kyanite_amd.configs import build_softmax
    g, inputs, _ = build_softmax(seed=12, shape=(2, 4, 64, 512))
    return g, 0, inputs(), None


@case
def layernorm_affine_rows_share_staged_operands():
    """enough rows of 4096 that a workgroup stages gamma / beta in LDS and walks over two rows, the loads of the
    second one requested before the statistics of the first"""
    from kyanite_amd import HipExecutor
    from kyanite_amd.configs import build_layernorm
    g, inputs, _ = build_layernorm(seed=14, shape=(2048, 4096))
    assert "rows=2" in HipExecutor(0, g, 0, plan_only=True).step_str(0)
    return g, 0, inputs(), None


@case
def config_bandwidth_layernorm_small():
    """configs[1] (c): rows of 4096 with the fused gamma / beta epilogue"""
    from kyanite_amd.configs import build_layernorm
    g, inputs, _ = build_layernorm(seed=13, shape=(64, 4096))
    return g, 0, inputs(), None


@case
def config_bandwidth_reduce_small():
    """configs[1] (d): sums over 8192 elements"""
    from kyanite_amd.configs import build_reduce
    g, inputs, _ = build_reduce(seed=14, shape=(64, 8192))
    return g, 0, inputs(), None


@case
def config_resnet_small():
    """configs[2] through its own builder: 128 channels like the benchmark (the same conv tiles), two blocks,
    batch 6"""
    from kyanite_amd.configs import build_resnet_tower
    g, make_inputs, _ = build_resnet_tower(seed=15, channels=128, blocks=2)
    return g, 6, make_inputs(6), None


@case
def config_tiny_mlp():
    """configs[0] as the benchmark and the smoke check build it"""
    from kyanite_amd.configs import build_tiny_mlp
    g, inputs = build_tiny_mlp(seed=16, batch=8)
    return g, 8, inputs, None


@case
def config_unet_block_small():
    from kyanite_amd.configs import build_unet_block
    g, make_inputs, _ = build_unet_block(seed=2, batch=2, channels=64, size=8, groups=4, heads=2, time_dim=48, ctx_len=5,
                                         ctx_dim=24)
    return g, 0, make_inputs(), None


@case
def layernorm_affine_many_rows():
    """enough rows that a workgroup walks over several of them with gamma / beta held in registers; the last
    workgroup runs out of rows part way"""
    g = Graph()
    rng = np.random.default_rng(50)
    x = g.input([4099, 2048])
    gamma = g.constant([1, 2048], (1.0 + 0.1 * rng.standard_normal((1, 2048))).astype(np.float32))
    beta = g.constant([1, 2048], (0.1 * rng.standard_normal((1, 2048))).astype(np.float32))
    g.output(g.add(g.mul(g.layernorm(x, 1, 1e-5), gamma), beta))
    return g, 0, [rng.standard_normal((4099, 2048)).astype(np.float32) * 3.0 + 0.5], None


# ---- long contractions with few output tiles: the launch splits the K axis and sums f32 partial products

@case
def matmul_split_k_skinny_f32():
    """8 rows (64 x 64 tiles), K = 4100 with a ragged last slice, N = 200 with a partial tile"""
    g = Graph()
    rng = np.random.default_rng(60)
    a = g.input([BATCH, 4100])
    w = g.constant([200, 4100], (rng.standard_normal((200, 4100)) * 0.05).astype(np.float32))
    g.output(g.linear(a, w))
    return g, 8, [rng.standard_normal((8, 4100)).astype(np.float32)], None


@case
def matmul_split_k_big_tiles_f32():
    """2 batches of 200 x 2304 x 330: 128 x 128 tiles with partial tiles on both axes, K split"""
    g = Graph()
    rng = np.random.default_rng(61)
    a = g.input([2, 200, 2304])
    b = g.input([2, 2304, 330])
    y = g.batched_mat_mul(a, b)
    g.output_all([y, g.permute(y, [0, 2, 1])])
    return g, 0, [rng.standard_normal((2, 200, 2304)).astype(np.float32) * 0.1,
                  rng.standard_normal((2, 2304, 330)).astype(np.float32)], None


@case
def matmul_split_k_f16():
    """f16 operands, f32 partial products, one rounding after the sum: big tiles (136 x 264) and skinny (16 rows)"""
    g = Graph()
    rng = np.random.default_rng(62)
    a = g.input([136, 4352], DType.F16)
    w = g.constant([264, 4352], _f16(rng, 264, 4352, scale=0.05))
    s = g.input([16, 4352], DType.F16)
    g.output_all([g.linear(a, w), g.linear(s, w)])
    return g, 0, [_f16(rng, 136, 4352), _f16(rng, 16, 4352)], None


# ---- elementwise tails folded into the matmul's store

@case
def matmul_bias_relu_fused():
    """relu(x W^T + b), x W^T + b, relu(x W^T) and a residual sum, with partial tiles; one launch each"""
    g = Graph()
    rng = np.random.default_rng(70)
    x = g.input([BATCH, 70])
    w = g.constant([130, 70], (rng.standard_normal((130, 70)) * 0.2).astype(np.float32))
    b = g.constant([1, 130], rng.standard_normal((1, 130)).astype(np.float32))
    w2 = g.constant([70, 130], (rng.standard_normal((70, 130)) * 0.2).astype(np.float32))
    h = g.relu(g.add(g.linear(x, w), b))
    y = g.add(x, g.linear(h, w2))  # residual: the addend is a full tensor
    g.output_all([y, g.add(g.linear(y, w), b), g.relu(g.linear(y, w))])
    return g, 9, [rng.standard_normal((9, 70)).astype(np.float32)], None


@case
def matmul_epilogue_layouts():
    """batched product with a bias per row (the addend is broadcast along the contiguous axis) and a transposed
    result, so the launch swaps its operands"""
    g = Graph()
    rng = np.random.default_rng(71)
    a = g.input([3, 40, 24])
    b = g.input([3, 24, 56])
    row_bias = g.constant([1, 40, 1], rng.standard_normal((1, 40, 1)).astype(np.float32))
    col_bias = g.constant([3, 1, 56], rng.standard_normal((3, 1, 56)).astype(np.float32))
    a2 = g.input([3, 40, 24])
    y = g.relu(g.add(g.batched_mat_mul(a, b), row_bias))
    z = g.add(g.batched_mat_mul(a2, b), col_bias)
    g.output_all([y, g.permute(z, [0, 2, 1])])
    return g, 0, [rng.standard_normal((3, 40, 24)).astype(np.float32), rng.standard_normal((3, 24, 56)).astype(np.float32),
                  rng.standard_normal((3, 40, 24)).astype(np.float32)], None


@case
def matmul_epilogue_split_k_f16():
    """f16: product, sum and relu each round to f16; the long contraction is split, so the tail runs in the pass
    that sums the partial products"""
    g = Graph()
    rng = np.random.default_rng(72)
    x = g.input([24, 4352], DType.F16)
    w = g.constant([136, 4352], _f16(rng, 136, 4352, scale=0.05))
    b = g.constant([1, 136], _f16(rng, 1, 136))
    small = g.constant([136, 136], _f16(rng, 136, 136, scale=0.1))
    h = g.relu(g.add(g.linear(x, w), b))
    g.output_all([h, g.add(h, g.linear(h, small))])
    return g, 0, [_f16(rng, 24, 4352)], None


@case
def f16_matmul_tall_tiles():
    """256 x 128 workgroup tiles (8 waves, K split): 500 rows (12 rows of the second tile missing), 200 and 264
    columns (partial tiles), K = 2088 with a ragged last slice; N-contiguous and K-contiguous right operands"""
    g = Graph()
    rng = np.random.default_rng(80)
    a = g.input([2, 500, 2088], DType.F16)
    b = g.input([2, 2088, 200], DType.F16)
    w = g.constant([264, 2088], _f16(rng, 264, 2088, scale=0.05))
    bias = g.constant([1, 264], _f16(rng, 1, 264))
    y = g.batched_mat_mul(a, b)
    z = g.relu(g.add(g.linear(g.view(a, [1000, 2088]), w), bias))
    g.output_all([y, z])
    return g, 0, [_f16(rng, 2, 500, 2088, scale=0.2), _f16(rng, 2, 2088, 200, scale=0.1)], None


@case
def f16_matmul_tall_tiles_split_k():
    """256 x 128 tiles with the K axis split: 512 x 384 x 4104"""
    g = Graph()
    rng = np.random.default_rng(81)
    a = g.input([512, 4104], DType.F16)
    w = g.constant([384, 4104], _f16(rng, 384, 4104, scale=0.05))
    g.output(g.linear(a, w))
    return g, 0, [_f16(rng, 512, 4104)], None


@case
def matmul_narrow_output_f32():
    """outputs at most 64 wide with many rows (64 x 64 tiles whatever the tile count): short K (slices of 16) and
    long K (slices of 64), ragged rows, columns and K"""
    g = Graph()
    rng = np.random.default_rng(90)
    a = g.input([32, 1100, 50])
    b = g.input([32, 50, 40])
    c = g.input([16, 2100, 2060])
    d = g.input([16, 2060, 24])
    g.output_all([g.batched_mat_mul(a, b), g.batched_mat_mul(c, d)])
    return g, 0, [rng.standard_normal((32, 1100, 50)).astype(np.float32), rng.standard_normal((32, 50, 40)).astype(np.float32),
                  (rng.standard_normal((16, 2100, 2060)) * 0.05).astype(np.float32),
                  rng.standard_normal((16, 2060, 24)).astype(np.float32)], None


def _attention_case(seed, b, lq, lk, dk, dv, scale_op, layout):
    """softmax(scale * Q K^T) V; `layout` picks how the operands reach the products: 'dense' [b, rows, width]
    inputs with K permuted, 'heads' [rows, b, width] inputs permuted like an attention layer does (strided
    operands, result permuted back), 'v_transposed' V stored [b, dv, lk]"""
    g = Graph()
    rng = np.random.default_rng(seed)
    if layout == "heads":
        q_in, k_in, v_in = g.input([lq, b, dk]), g.input([lk, b, dk]), g.input([lk, b, dv])
        q, kt, v = g.permute(q_in, [1, 0, 2]), g.permute(k_in, [1, 2, 0]), g.permute(v_in, [1, 0, 2])
        shapes = [(lq, b, dk), (lk, b, dk), (lk, b, dv)]
    else:
        q, k_in = g.input([b, lq, dk]), g.input([b, lk, dk])
        kt = g.permute(k_in, [0, 2, 1])
        if layout == "v_transposed":
            v = g.permute(g.input([b, dv, lk]), [0, 2, 1])
            shapes = [(b, lq, dk), (b, lk, dk), (b, dv, lk)]
        else:
            v = g.input([b, lk, dv])
            shapes = [(b, lq, dk), (b, lk, dk), (b, lk, dv)]
    scores = g.batched_mat_mul(q, kt)
    if scale_op == "mul":
        scores = g.mul(scores, g.scalar(1.0 / np.sqrt(dk)))
    elif scale_op == "mul_left":
        scores = g.mul(g.scalar(1.0 / np.sqrt(dk)), scores)
    elif scale_op == "div":
        scores = g.binary(BinaryOp.DIV, scores, g.scalar(float(np.sqrt(dk))))
    out = g.batched_mat_mul(g.softmax(scores, 2), v)
    if layout == "heads":
        out = g.view(g.permute(out, [1, 0, 2]), [lq, b * dv])
    g.output(out)
    return g, 0, [rng.standard_normal(shape).astype(np.float32) for shape in shapes], None


@case
def attention_fused_ragged():
    """one launch for the whole chain; 200 queries and 77 keys (partial blocks of both), width 40"""
    return _attention_case(100, 3, 200, 77, 40, 40, "mul", "dense")


@case
def attention_fused_heads_layout():
    """operands that are permuted views (row strides b * width), result written in [lq, b, dv] order; width 64"""
    return _attention_case(101, 4, 128, 256, 64, 64, "div", "heads")


@case
def attention_fused_narrow_v():
    """width 32, V narrower than one tile and stored transposed, no scale, the scale on the left"""
    a = _attention_case(102, 2, 70, 130, 32, 24, "none", "v_transposed")
    return a


@case
def attention_fused_v_width_36():
    """V four dims wider than a 32-wide tile: one group of four dims on the 4 x 4 matrix instruction; heads layout"""
    return _attention_case(104, 3, 100, 150, 32, 36, "mul", "heads")


@case
def attention_fused_v_width_42():
    """42 is 32 + three groups of four with two dims of padding; queries and keys in partial blocks"""
    return _attention_case(105, 2, 150, 200, 40, 42, "div", "dense")


@case
def attention_fused_v_width_48():
    """32 + four full groups, V stored transposed"""
    return _attention_case(106, 2, 64, 128, 64, 48, "mul_left", "v_transposed")


@case
def attention_fused_many_blocks():
    """enough keys that the running maximum and sum are rescaled many times; large score range"""
    g, b, inputs, _ = _attention_case(103, 2, 256, 1000, 40, 40, "mul_left", "dense")
    inputs[0] *= 4.0
    return g, b, inputs, None


@case
def transposed_copy_through_tiles():
    """[3, 200, 330] read as its [0, 2, 1] permutation and stored densely (NCHW -> tokens): big enough for the kernel
    that turns tiles of 64 x 64 through LDS; neither 200 nor 330 is a multiple of the tile"""
    g = Graph()
    rng = np.random.default_rng(140)
    x = g.input([3, 200, 330])
    # the view cannot be a stride edit, so the permuted tensor is copied
    g.output(g.view(g.permute(x, [0, 2, 1]), [3 * 330, 200]))
    return g, 0, [rng.standard_normal((3, 200, 330)).astype(np.float32)], None


@case
def transposed_operands_in_elementwise_chain():
    """f16: two transposed operands, one straight operand, one broadcast row and a flipped axis in one chain"""
    g = Graph()
    rng = np.random.default_rng(141)
    shapes = [(2, 300, 136), (2, 300, 136), (2, 136, 300), (1, 1, 300)]
    a, b, c, d = [g.input(list(shape), DType.F16) for shape in shapes]
    at, bt = g.permute(a, [0, 2, 1]), g.flip(g.permute(b, [0, 2, 1]), 2)
    y = g.add(g.mul(at, c), g.mul(bt, g.broadcast(d, [2, 136, 300])))
    g.output(y)
    return g, 0, [rng.standard_normal(shape).astype(np.float16) for shape in shapes], None


@case
def transposed_operand_two_outputs_and_wide_types():
    """one transposed f64 operand feeding two outputs (tiles of 8 byte elements), and a bool one (1 byte elements)"""
    g = Graph()
    rng = np.random.default_rng(142)
    x = g.input([260, 300], DType.F64)
    w = g.input([300, 260], DType.F64)
    xt = g.permute(x, [1, 0])
    g.output_all([g.add(xt, w), g.mul(xt, w)])
    m = g.input([300, 260], DType.BOOL)
    g.output(g.view(g.permute(m, [1, 0]), [260 * 300]))
    inputs = [rng.standard_normal((260, 300)), rng.standard_normal((300, 260)), rng.random((300, 260)) < 0.5]
    return g, 0, inputs, None


@case
def matmul_sum_with_two_users():
    """y = x @ w + bias feeds a layernorm and a residual sum (a transformer block's skip connection): y is stored by
    the matmul, and both users load it"""
    g = Graph()
    rng = np.random.default_rng(143)
    shapes = [(200, 96), (96, 136), (1, 136), (200, 136)]
    x, w, bias, z = [g.input(list(shape)) for shape in shapes]
    y = g.add(g.mat_mul(x, w), g.broadcast(bias, [200, 136]))
    g.output_all([g.add(g.layernorm(y, 1, 1e-5), g.add(y, z)), g.mul(y, z)])
    return g, 0, [rng.standard_normal(shape).astype(np.float32) for shape in shapes], None


def _two_addend_case(seed, m, n, k, dtype=DType.F32, relu=False, residual_first=False, permuted=False):
    """`(x @ w + bias) + residual` (the output projection of a transformer block with its skip connection), which the
    matmul stores in one go; `residual_first`: the skip connection on the left of the outer sum; `permuted`: the
    result is handed out transposed"""
    g = Graph()
    rng = np.random.default_rng(seed)
    np_dtype = np.float16 if dtype == DType.F16 else np.float32
    shapes = [(m, k), (n, k), (1, n), (m, n)]
    x, w, bias, res = [g.input(list(shape), dtype) for shape in shapes]
    y = g.add(g.linear(x, w), g.broadcast(bias, [m, n]))
    y = g.add(res, y) if residual_first else g.add(y, res)
    if relu:
        y = g.relu(y)
    if permuted:
        y = g.permute(y, [1, 0])
    g.output(y)
    scale = [1.0, 1.0 / np.sqrt(k), 1.0, 1.0]
    return g, 0, [(rng.standard_normal(shape) * sc).astype(np_dtype) for shape, sc in zip(shapes, scale)], None


@case
def matmul_bias_and_residual_f32():
    """f32 on the direct kernel (K a multiple of 32), ragged tiles"""
    return _two_addend_case(150, 200, 136, 96)


@case
def matmul_bias_and_residual_f32_staged_relu():
    """K = 100 is no multiple of 32: the kernel that stages through registers; relu on top, residual on the left"""
    return _two_addend_case(151, 130, 72, 100, relu=True, residual_first=True)


@case
def matmul_bias_and_residual_split_k():
    """few tiles and a long K: the partial products are summed by a pass of its own, which adds both operands"""
    return _two_addend_case(152, 40, 64, 4096)


@case
def matmul_bias_and_residual_f16():
    """f16: a rounding after the product and after either sum, like the three separate operations"""
    return _two_addend_case(153, 300, 264, 320, DType.F16)


@case
def matmul_bias_and_residual_f16_permuted():
    """f16 with relu on top, the result handed out transposed"""
    return _two_addend_case(154, 257, 130, 128, DType.F16, relu=True, permuted=True)


@case
def matmul_bias_and_residual_f16_staged():
    """f16 with K = 200, no multiple of 64: the kernel that stages through registers"""
    return _two_addend_case(156, 130, 72, 200, DType.F16, relu=True)


@case
def matmul_bias_and_residual_f16_split_k():
    """f16 with K split over workgroups (summing pass)"""
    return _two_addend_case(155, 64, 128, 8192, DType.F16, residual_first=True)


def _attention_split_heads_case(seed, batch, heads, lq, lk, dk, dv, dtype=DType.F32, kv_split=None):
    """attention over (batch, heads) as a transformer block writes it: q, k, v are [batch * tokens, heads * width]
    projections, viewed as [batch, tokens, heads, width], permuted to [batch, heads, tokens, width] and flattened to
    [batch * heads, tokens, width] (no stride edit: a dense copy unless the kernel takes two batch strides); the result
    goes back the same way. `kv_split`: K and V arrive flattened and dense instead (another split of the batch)."""
    g = Graph()
    rng = np.random.default_rng(seed)
    np_dtype = np.float16 if dtype == DType.F16 else np.float32
    inputs = []

    def inp(shape):
        inputs.append(rng.standard_normal(shape).astype(np_dtype))
        return g.input(list(shape), dtype)

    def heads_of(x, tokens, width):
        x = g.permute(g.view(x, [batch, tokens, heads, width]), [0, 2, 1, 3])
        return g.view(x, [batch * heads, tokens, width])

    q = heads_of(inp((batch * lq, heads * dk)), lq, dk)
    if kv_split == "dense":
        k, v = inp((batch * heads, lk, dk)), inp((batch * heads, lk, dv))
    else:
        k, v = heads_of(inp((batch * lk, heads * dk)), lk, dk), heads_of(inp((batch * lk, heads * dv)), lk, dv)
    scores = g.mul(g.batched_mat_mul(q, g.permute(k, [0, 2, 1])), g.scalar(1.0 / np.sqrt(dk), dtype))
    out = g.batched_mat_mul(g.softmax(scores, 2), v)
    out = g.permute(g.view(out, [batch, heads, lq, dv]), [0, 2, 1, 3])
    g.output(g.view(out, [batch * lq, heads * dv]))
    return g, 0, inputs, None


@case
def attention_split_heads_no_copies():
    """f32, 2 x 3 heads of width 40: operands and result in [batch, tokens, heads, width] order, ragged lengths"""
    return _attention_split_heads_case(105, 2, 3, 150, 77, 40, 40)


@case
def attention_split_heads_mixed_operands():
    """Q and the result split as (batch, heads), K and V dense over the flat batch"""
    return _attention_split_heads_case(106, 3, 2, 70, 130, 64, 32, kv_split="dense")


@case
def attention_split_heads_unsupported_width():
    """width 24 is none the fused kernel is built for: the same graph runs as copies, matmul, softmax, matmul"""
    return _attention_split_heads_case(108, 2, 3, 50, 60, 24, 24)


@case
def attention_f16_split_heads_no_copies():
    """f16, 2 x 4 heads of width 64 in [batch, tokens, heads, width] order"""
    return _attention_split_heads_case(107, 2, 4, 100, 100, 64, 64, DType.F16)


@case
def attention_chain_not_fused():
    """the scores are an output as well, so the chain has to stay three launches"""
    g = Graph()
    rng = np.random.default_rng(104)
    q, k, v = g.input([2, 50, 40]), g.input([2, 60, 40]), g.input([2, 60, 40])
    probs = g.softmax(g.batched_mat_mul(q, g.permute(k, [0, 2, 1])), 2)
    g.output_all([g.batched_mat_mul(probs, v), probs])
    return g, 0, [rng.standard_normal(s).astype(np.float32) for s in [(2, 50, 40), (2, 60, 40), (2, 60, 40)]], None


def _shared_left_linears(seed, dtype, m, k, n, count, bias_on=(), relu_on=()):
    """`count` linear layers of one input; some of them with a bias and / or a relu behind them"""
    g = Graph()
    rng = np.random.default_rng(seed)
    np_dtype = np.float16 if dtype == DType.F16 else np.float32
    x = g.input([m, k], dtype)
    outs = []
    for i in range(count):
        w = g.constant([n, k], (rng.standard_normal((n, k)) / np.sqrt(k)).astype(np_dtype), dtype)
        y = g.linear(x, w)
        if i in bias_on:
            y = g.add(y, g.view(g.constant([n], rng.standard_normal(n).astype(np_dtype), dtype), [1, n]))
        if i in relu_on:
            y = g.relu(y)
        outs.append(y)
    g.output_all(outs)
    return g, 0, [rng.standard_normal((m, k)).astype(np_dtype)], None


@case
def matmul_group_qkv_f32():
    """three projections of one input share a launch; ragged rows and columns"""
    return _shared_left_linears(110, DType.F32, 600, 320, 328, 3)


@case
def matmul_group_f16():
    """the same in f16 (128 x 128 tiles, slices of 128)"""
    return _shared_left_linears(111, DType.F16, 520, 256, 384, 3)


@case
def matmul_group_more_than_one_launch_holds():
    """six siblings: a group of four and a group of two"""
    return _shared_left_linears(112, DType.F32, 200, 64, 96, 6)


@case
def matmul_group_with_epilogues():
    """siblings with a bias or relu behind them keep their fused epilogue, the plain ones still share a launch"""
    return _shared_left_linears(113, DType.F32, 300, 128, 192, 4, bias_on=(0, 2), relu_on=(2,))


@case
def matmul_group_declined_when_k_would_be_split():
    """skinny products with a long K run apart, each split along K"""
    return _shared_left_linears(114, DType.F32, 8, 4096, 256, 2)


@case
def reduce_with_elementwise_prologue():
    """an elementwise chain of one tensor that only the reduction uses is evaluated inside the reduce kernel:
    sum of squares along rows (lanes share a row) and along columns (threads own columns), max |x|, and a mean of
    squares whose input is f16 and whose reduction runs in f32 (the cast is part of the chain)"""
    g = Graph()
    rng = np.random.default_rng(120)
    x = g.input([37, 200])
    h = g.input([24, 512], DType.F16)
    y = g.input([300, 64])
    g.output(g.reduce(g.mul(x, x), [1], ReduceOp.SUM))
    g.output(g.reduce(g.mul(g.unary(UnaryOp.ABS, x), g.scalar(2.0)), [0], ReduceOp.SUM))
    g.output(g.reduce(g.unary(UnaryOp.ABS, g.add(y, g.scalar(0.5))), [0, 1], ReduceOp.MAX))
    hf = g.value_cast(h, DType.F32)
    g.output(g.reduce(g.mul(hf, hf), [1], ReduceOp.MEAN))
    g.output(g.reduce(g.mul(h, h), [1], ReduceOp.MEAN))
    return g, 0, [rng.standard_normal((37, 200)).astype(np.float32), rng.standard_normal((24, 512)).astype(np.float16),
                  rng.standard_normal((300, 64)).astype(np.float32)], None


@case
def rms_norm_one_launch():
    """x * rsqrt(mean(x^2) + eps) * w: ONE row kernel that computes the mean of squares of its own rows (the square
    as its prologue) and scales them (the rsqrt of the mean as part of its epilogue); f32 and f16"""
    g = Graph()
    rng = np.random.default_rng(121)
    outs = []
    for dtype, np_dtype in ((DType.F32, np.float32), (DType.F16, np.float16)):
        x = g.input([50, 96], dtype)
        w = g.constant([1, 96], (1.0 + 0.1 * rng.standard_normal((1, 96))).astype(np_dtype), dtype)
        ms = g.view(g.reduce(g.mul(x, x), [1], ReduceOp.MEAN), [50, 1])
        r = g.binary(BinaryOp.DIV, g.scalar(1.0, dtype), g.unary(UnaryOp.SQRT, g.add(ms, g.scalar(1e-5, dtype))))
        outs.append(g.mul(g.mul(x, g.broadcast(r, [50, 96])), g.broadcast(w, [50, 96])))
    g.output_all(outs)
    return g, 0, [rng.standard_normal((50, 96)).astype(np.float32), rng.standard_normal((50, 96)).astype(np.float16)], None


@case
def softmax_scale_and_mask_prologue():
    """softmax(scale * scores + mask) with a mask that is broadcast over the heads: one kernel; f32 and f16"""
    g = Graph()
    rng = np.random.default_rng(122)
    mask = np.where(np.tril(np.ones((40, 40))) > 0, 0.0, -1e4)
    outs = []
    for dtype, np_dtype in ((DType.F32, np.float32), (DType.F16, np.float16)):
        s = g.input([6, 40, 40], dtype)
        m = g.broadcast(g.constant([1, 40, 40], mask.astype(np_dtype)[None], dtype), [6, 40, 40])
        outs.append(g.softmax(g.add(g.mul(s, g.scalar(0.125, dtype)), m), 2))
    g.output_all(outs)
    return g, 0, [rng.standard_normal((6, 40, 40)).astype(np.float32) * 4, (rng.standard_normal((6, 40, 40)) * 4).astype(np.float16)], None


def _attention_f16_case(seed, b, lq, lk, dk, dv, scale, mask, layout="dense"):
    """f16 softmax(scale * Q K^T + mask) V; mask: None, 'causal' (a [1, lq, lk] constant of 0 / -inf, broadcast over the
    batch), 'full' (a [b, lq, lk] input of finite values), 'left' (the constant on the left of the sum)"""
    g = Graph()
    rng = np.random.default_rng(seed)
    inputs = []

    def inp(shape):
        inputs.append(rng.standard_normal(shape).astype(np.float16))
        return g.input(list(shape), DType.F16)

    if layout == "heads":
        q = g.permute(inp((lq, b, dk)), [1, 0, 2])
        kt = g.permute(inp((lk, b, dk)), [1, 2, 0])
        v = g.permute(inp((lk, b, dv)), [1, 0, 2])
    else:
        q = inp((b, lq, dk))
        kt = g.permute(inp((b, lk, dk)), [0, 2, 1])
        v = inp((b, lk, dv))
    scores = g.batched_mat_mul(q, kt)
    if scale:
        scores = g.mul(scores, g.scalar(1.0 / np.sqrt(dk), DType.F16))
    if mask in ("causal", "left"):
        m = np.where(np.tril(np.ones((lq, lk), bool), k=lk - lq), 0.0, -np.inf).astype(np.float16)
        mc = g.broadcast(g.constant([1, lq, lk], m[None], DType.F16), [b, lq, lk])
        scores = g.add(mc, scores) if mask == "left" else g.add(scores, mc)
    elif mask == "full":
        scores = g.add(scores, inp((b, lq, lk)))
    out = g.batched_mat_mul(g.softmax(scores, 2), v)
    if layout == "heads":
        out = g.view(g.permute(out, [1, 0, 2]), [lq, b * dv])
    g.output(out)
    return g, 0, inputs, None


@case
def attention_f16_causal_heads():
    """the decoder's attention: width 128, causal mask constant, operands that are permuted views"""
    return _attention_f16_case(130, 4, 96, 96, 128, 128, True, "causal", "heads")


@case
def attention_f16_causal_even_tiles():
    """an even number of query tiles (the launch pairs late tiles with early ones), 5 key blocks per wave at most, and
    a last tile of queries that is partial"""
    return _attention_f16_case(134, 3, 250, 250, 128, 128, True, "causal")


@case
def attention_f16_rising_scores():
    """scores whose spread grows along the keys (later keys are up to 9 times larger): the reference value of the
    running softmax moves in some blocks and stays behind the maximum, within its slack, in others"""
    g, batch, inputs, _ = _attention_f16_case(135, 2, 64, 320, 64, 64, True, None)
    inputs[1] = (inputs[1].astype(np.float32) * (1.0 + np.arange(320, dtype=np.float32)[None, :, None] / 40.0)).astype(np.float16)
    return g, batch, inputs, None


@case
def attention_f16_causal_long():
    """1100 queries and keys under a causal mask: 9 blocks of keys per wave, classes for 35 x 35 blocks, partial last
    tiles of both"""
    return _attention_f16_case(136, 2, 1100, 1100, 64, 64, True, "causal")


@case
def attention_f16_one_query():
    """a single query (a decoding step) against 300 keys with a mask tensor: a workgroup with one live lane pair"""
    return _attention_f16_case(137, 3, 1, 300, 128, 128, True, "full")


@case
def attention_f16_ragged_full_mask():
    """70 queries against 150 keys (partial blocks), width 64, V 40 wide, a mask tensor per batch entry"""
    return _attention_f16_case(131, 3, 70, 150, 64, 40, True, "full")


@case
def attention_f16_plain():
    """no scale, no mask; many queries (four waves per workgroup would need 256 workgroups: two here)"""
    return _attention_f16_case(132, 2, 200, 130, 64, 64, False, None)


@case
def attention_f16_mask_on_the_left_no_scale():
    return _attention_f16_case(133, 2, 40, 72, 128, 96, False, "left")


# From 512 workgroups of 128 queries on, the f16 attention runs on the kernel whose four waves own 32 queries each and
# stage every block of keys together (`attention_f16_shares_keys`).

@case
def attention_f16_shared_keys_causal():
    """128 batch entries of 450 queries and keys under a causal mask: the last tile of 128 has 66 queries, so its
    third wave holds two and its fourth none (it only helps to stage); every wave skips the blocks above its own
    part of the diagonal while the waves below it still need them"""
    return _attention_f16_case(140, 128, 450, 450, 64, 64, True, "causal")


@case
def attention_f16_shared_keys_mask_tensor():
    """a mask tensor whose rows of 77 values are not aligned (read value by value), keys in two whole blocks and one
    of 13, V of width 40 in two tiles of 32"""
    return _attention_f16_case(141, 128, 512, 77, 128, 40, True, "full")


@case
def attention_f16_shared_keys_plain_heads():
    """no mask, no scale, operands that are permuted views, width 128. (Queries a tenth as large, so that the scores
    stay around 1 without the scale: at 11 a last place of an f16 score is 3 % of its key's weight, and among 8 M
    results one lands further than 2 % from the oracle, whose dot products add up in another order.)"""
    g, batch, inputs, _ = _attention_f16_case(142, 128, 512, 130, 128, 128, False, None, "heads")
    inputs[0] = (inputs[0].astype(np.float32) * 0.1).astype(np.float16)
    return g, batch, inputs, None


@case
def attention_f16_shared_keys_aligned_mask_rows():
    """a mask tensor with rows of 96 values (whole, aligned rows: read as vectors), K of width 64 against V of 128;
    40 queries per batch entry: one full wave, one with 8 queries and two that only stage"""
    return _attention_f16_case(143, 512, 40, 96, 64, 128, True, "full")


@case
def attention_f16_shared_keys_many_blocks():
    """8 queries per batch entry against 2100 keys (66 blocks: the classes of a wave fill more than one register),
    the causal mask shifted so that only the last, partial block is masked in part"""
    return _attention_f16_case(144, 512, 8, 2100, 64, 64, True, "causal")


@case
def rotary_of_two_tensors_is_one_launch():
    """two rotary embeddings (two concats of two elementwise halves each) over different inputs and the same cos / sin:
    four results from one launch; a third chain that reads one of the results stays a launch of its own"""
    g = Graph()
    rng = np.random.default_rng(141)
    cos = g.broadcast(g.constant([1, 24, 16], np.cos(rng.standard_normal((1, 24, 16))).astype(np.float32)), [5, 24, 16])
    sin = g.broadcast(g.constant([1, 24, 16], np.sin(rng.standard_normal((1, 24, 16))).astype(np.float32)), [5, 24, 16])

    def rotary(x1, x2):
        return g.concat([g.sub(g.mul(x1, cos), g.mul(x2, sin)), g.add(g.mul(x1, sin), g.mul(x2, cos))], 2)

    q = rotary(g.input([5, 24, 16]), g.input([5, 24, 16]))
    k = rotary(g.input([5, 24, 16]), g.input([5, 24, 16]))
    g.output(q)
    g.output(k)
    g.output(g.unary(UnaryOp.TANH, g.add(q, k)))
    inputs = [rng.standard_normal((5, 24, 16)).astype(np.float32) for _ in range(4)]
    from kyanite_amd import HipExecutor
    ex = HipExecutor(0, g, 0, plan_only=True)
    assert ex.step_kinds() == ["scalar_op", "scalar_op"] and "outputs=4" in ex.step_str(0), [ex.step_str(i) for i in range(ex.step_count())]
    return g, 0, inputs, None


@case
def concat_pieces_share_a_launch():
    """pieces of a concat that are elementwise chains of one shape are computed by ONE kernel with several outputs
    (a rotary embedding's two halves); a piece of another shape and a plain tensor in between get their own"""
    g = Graph()
    rng = np.random.default_rng(140)
    x1, x2 = g.input([5, 24, 16]), g.input([5, 24, 16])
    cos = g.broadcast(g.constant([1, 24, 16], np.cos(rng.standard_normal((1, 24, 16))).astype(np.float32)), [5, 24, 16])
    sin = g.broadcast(g.constant([1, 24, 16], np.sin(rng.standard_normal((1, 24, 16))).astype(np.float32)), [5, 24, 16])
    def chains(k):  # fresh values every time: a chain that two concats share is materialised instead
        a = g.sub(g.mul(g.mul(x1, g.scalar(float(k))), cos), g.mul(x2, sin))
        b = g.add(g.mul(g.mul(x1, g.scalar(float(k))), sin), g.mul(x2, cos))
        c = g.unary(UnaryOp.TANH, g.add(g.mul(x1, g.scalar(float(k))), x2))
        return a, b, c

    other = g.unary(UnaryOp.NEG, g.input([5, 24, 3]))
    a, b, _ = chains(1.5)
    g.output(g.concat([a, b], 2))
    a, b, c = chains(2.5)
    g.output(g.concat([c, other, a, x1, b], 2))
    a, b, c = chains(3.5)
    g.output(g.concat([a, b, c], 1))
    return g, 0, [rng.standard_normal((5, 24, 16)).astype(np.float32), rng.standard_normal((5, 24, 16)).astype(np.float32),
                  rng.standard_normal((5, 24, 3)).astype(np.float32)], None


# ---- f16 matmuls whose operands both have K contiguous and a multiple of 64: slices go global -> LDS directly

@case
def f16_matmul_direct_tiles():
    """all three tile shapes of the direct kernel: 128 x 128 with ragged rows and columns (the edge rows repeat
    the last row) and an odd number of slices, over a batch; 64 x 64 with one slice and with two; 256 x 128 with
    the K axis split"""
    g = Graph()
    rng = np.random.default_rng(150)
    a = g.input([16, 264, 192], DType.F16)
    b = g.input([16, 328, 192], DType.F16)
    big = g.batched_mat_mul(a, g.permute(b, [0, 2, 1]))
    s = g.input([72, 128], DType.F16)
    w1 = g.constant([200, 64], _f16(rng, 200, 64, scale=0.1))
    w2 = g.constant([40, 128], _f16(rng, 40, 128, scale=0.1))
    small_one = g.linear(g.slice(s, 1, 0, 64), w1)
    small_two = g.linear(s, w2)
    t = g.input([500, 4096], DType.F16)
    w3 = g.constant([384, 4096], _f16(rng, 384, 4096, scale=0.05))
    g.output_all([big, small_one, small_two, g.linear(t, w3)])
    return g, 0, [_f16(rng, 16, 264, 192, scale=0.2), _f16(rng, 16, 328, 192, scale=0.2), _f16(rng, 72, 128),
                  _f16(rng, 500, 4096)], None


@case
def f16_matmul_direct_epilogue():
    """bias and relu in the store of the direct kernel, with and without a split of K"""
    g = Graph()
    rng = np.random.default_rng(151)
    x = g.input([300, 256], DType.F16)
    w = g.constant([520, 256], _f16(rng, 520, 256, scale=0.1))
    bias = g.constant([1, 520], _f16(rng, 1, 520))
    y = g.relu(g.add(g.linear(x, w), bias))
    long_x = g.input([40, 2048], DType.F16)
    long_w = g.constant([72, 2048], _f16(rng, 72, 2048, scale=0.05))
    res = g.input([40, 72], DType.F16)
    z = g.add(g.linear(long_x, long_w), res)
    g.output_all([y, z])
    return g, 0, [_f16(rng, 300, 256), _f16(rng, 40, 2048), _f16(rng, 40, 72)], None


@case
def f16_matmul_constant_weights_laid_out_again():
    """constant [k, n] right operands (`x @ w`) get a [n, k] copy at planning time: a single product, three that
    share their left operand (one launch), a weight that an elementwise op reads as well (the original stays), a
    slice of a bigger constant, and a weight broadcast over a batch"""
    g = Graph()
    rng = np.random.default_rng(152)
    x = g.input([48, 128], DType.F16)
    w = g.constant([128, 72], _f16(rng, 128, 72, scale=0.1))
    single = g.mat_mul(g.unary(UnaryOp.TANH, x), w)
    qkv = [g.mat_mul(x, g.constant([128, 136], _f16(rng, 128, 136, scale=0.1))) for _ in range(3)]
    shared = g.constant([128, 40], _f16(rng, 128, 40, scale=0.1))
    both = g.mat_mul(g.unary(UnaryOp.NEG, x), shared)
    doubled = g.mul(shared, g.scalar(2.0, DType.F16))
    big = g.constant([192, 100], _f16(rng, 192, 100, scale=0.1))
    sliced = g.mat_mul(g.unary(UnaryOp.ABS, x), g.slice(g.slice(big, 0, 64, 192), 1, 4, 84))
    xb = g.input([3, 48, 64], DType.F16)
    wb = g.constant([1, 64, 24], _f16(rng, 1, 64, 24, scale=0.1))
    batched = g.batched_mat_mul(xb, g.broadcast(wb, [3, 64, 24]))
    g.output_all([single] + qkv + [both, doubled, sliced, batched])
    return g, 0, [_f16(rng, 48, 128), _f16(rng, 3, 48, 64)], None


@case
def f16_matmul_direct_tall_ring():
    """256 x 128 tiles on the ring of three stages without a split of K: a batch with fewer slices (2) than
    stages and ragged columns, and three projections of one input in one launch with exactly 3 slices"""
    g = Graph()
    rng = np.random.default_rng(153)
    a = g.input([16, 256, 128], DType.F16)
    b = g.input([16, 1000, 128], DType.F16)
    g.output(g.batched_mat_mul(a, g.permute(b, [0, 2, 1])))
    x = g.input([512, 192], DType.F16)
    for _ in range(3):
        g.output(g.linear(x, g.constant([2816, 192], _f16(rng, 2816, 192, scale=0.1))))
    return g, 0, [_f16(rng, 16, 256, 128, scale=0.2), _f16(rng, 16, 1000, 128, scale=0.2), _f16(rng, 512, 192)], None


@case
def f16_matmul_shared_tail_tiles():
    """520 tiles of 64 x 64 on 512 places: the first 512 tiles get a workgroup each, the last 8 are shared by two
    workgroups each, which split K and sum up inside the launch; the result also gets a bias and a relu"""
    g = Graph()
    rng = np.random.default_rng(154)
    a = g.input([33, 1024], DType.F16)
    b = g.input([33280, 1024], DType.F16)
    bias = g.input([1, 33280], DType.F16)
    g.output(g.relu(g.add(g.linear(a, b), bias)))
    return g, 0, [_f16(rng, 33, 1024, scale=0.2), _f16(rng, 33280, 1024, scale=0.2), _f16(rng, 1, 33280)], None


@case
def f16_matmul_direct_wide_tiles():
    """256 x 256 tiles (8 waves of 128 x 64), 256 of them over a batch, ragged on both axes"""
    g = Graph()
    rng = np.random.default_rng(155)
    a = g.input([16, 1000, 128], DType.F16)
    b = g.input([16, 1016, 128], DType.F16)
    g.output(g.batched_mat_mul(a, g.permute(b, [0, 2, 1])))
    return g, 0, [_f16(rng, 16, 1000, 128, scale=0.2), _f16(rng, 16, 1016, 128, scale=0.2)], None


@case
def f16_matmul_direct_mid_tiles():
    """256 x 192 tiles (8 waves of 64 x 96): 200 of them fill one round of workgroups where 300 tiles of 256 x 128
    would need two; ragged columns, one slice of K"""
    g = Graph()
    rng = np.random.default_rng(156)
    a = g.input([100, 256, 64], DType.F16)
    b = g.input([100, 380, 64], DType.F16)
    g.output(g.batched_mat_mul(a, g.permute(b, [0, 2, 1])))
    return g, 0, [_f16(rng, 100, 256, 64, scale=0.3), _f16(rng, 100, 380, 64, scale=0.3)], None


@case
def row_statistics_in_the_elementwise_kernel():
    """more statistics of the very rows an elementwise kernel writes, each computed inside it: x - max(x),
    |x| / sum(|x|) (with the abs shared by the prologue and the epilogue), x * min(x) on rows too long for registers
    (streamed), in f16 as well; and the cases that stay separate launches: a statistic that something else reads
    too, and one over another axis"""
    g = Graph()
    rng = np.random.default_rng(160)
    x = g.input([37, 200])
    col = lambda v, rows: g.view(v, [rows, 1])
    g.output(g.sub(x, g.broadcast(col(g.reduce(x, [1], ReduceOp.MAX), 37), [37, 200])))
    a = g.unary(UnaryOp.ABS, x)
    g.output(g.binary(BinaryOp.DIV, a, g.broadcast(col(g.reduce(a, [1], ReduceOp.SUM), 37), [37, 200])))
    long_x = g.input([3, 70000])
    g.output(g.mul(long_x, g.broadcast(col(g.reduce(long_x, [1], ReduceOp.MIN), 3), [3, 70000])))
    h = g.input([20, 136], DType.F16)
    hm = col(g.reduce(g.mul(h, h), [1], ReduceOp.MEAN), 20)
    g.output(g.mul(h, g.broadcast(g.unary(UnaryOp.SQRT, g.add(hm, g.scalar(0.5, DType.F16))), [20, 136])))
    # read twice: stays a reduce launch
    shared = g.reduce(x, [1], ReduceOp.SUM)
    g.output(shared)
    g.output(g.add(x, g.broadcast(col(shared, 37), [37, 200])))
    # over the rows, not along them
    g.output(g.sub(x, g.broadcast(g.view(g.reduce(x, [0], ReduceOp.MEAN), [1, 200]), [37, 200])))
    return g, 0, [rng.standard_normal((37, 200)).astype(np.float32), rng.standard_normal((3, 70000)).astype(np.float32),
                  rng.standard_normal((20, 136)).astype(np.float16)], None


@case
def restride_every_other_element():
    """the data and the expected values of kn-cuda-sys/tests/restride.rs:9-26: three elements two apart read into a
    dense tensor; here as a slice with step 2 of an input, which the copy step does"""
    g = Graph()
    x = g.input([6])
    g.output(g.slice(x, 0, 0, 6, 2))
    return g, 0, [f32((6,), [-1.0, 0.0, 2.0, 0.0, -3.0, 0.0])], [f32((3,), [-1.0, 2.0, -3.0])]


@case
def negative_stride_read():
    """the layout of kn-cuda-sys/tests/negative_stride.rs:14-45: eight floats read through a stride of -1 from the
    last element (that test prints its result; reversing 0..8 is what the layout means)"""
    g = Graph()
    x = g.input([1, 1, 1, 8])
    g.output(g.flip(x, 3))
    return g, 0, [f32((1, 1, 1, 8), np.arange(8))], [f32((1, 1, 1, 8), np.arange(8)[::-1])]


@case
def reduce_in_two_launches():
    """few results, much to read: slices of the reduced index are folded side by side and a second launch folds the
    partial results. Along columns (vectors of 4, a last slice that is shorter), over everything (one result), along
    long rows with the square folded into the load (f16, partial results in f32), with a permuted input whose kept
    axis is not the last, and integer sums, which must stay exact"""
    g = Graph()
    rng = np.random.default_rng(170)
    tall = g.input([70001, 96])
    g.output(g.reduce(tall, [0], ReduceOp.MEAN))
    g.output(g.reduce(tall, [0], ReduceOp.MIN))
    whole = g.input([1500, 3001])
    g.output(g.reduce(whole, [0, 1], ReduceOp.SUM))
    g.output(g.reduce(whole, [0, 1], ReduceOp.MAX))
    long_rows = g.input([3, 600000], DType.F16)
    g.output(g.reduce(g.mul(long_rows, long_rows), [1], ReduceOp.MEAN))
    planes = g.input([5, 300, 700])
    g.output(g.reduce(g.permute(planes, [1, 0, 2]), [0, 2], ReduceOp.SUM))
    counts = g.input([200000, 8], DType.I32)
    g.output(g.reduce(counts, [0], ReduceOp.SUM))
    return g, 0, [rng.standard_normal((70001, 96)).astype(np.float32), rng.standard_normal((1500, 3001)).astype(np.float32),
                  rng.standard_normal((3, 600000)).astype(np.float16), rng.standard_normal((5, 300, 700)).astype(np.float32),
                  rng.integers(-2**20, 2**20, (200000, 8)).astype(np.int32)], None


@case
def normalised_axis_is_not_the_contiguous_one():
    """softmax, layernorm and row statistics along an axis that a contiguous axis follows (a softmax over the channels of
    [n, c, h, w]): neighbouring lanes take neighbouring columns. Few positions per thread (in registers) with a last
    block of columns that is partial; 300 positions (16 threads per column); 1000 positions (read again per pass); f16;
    a sum of two tensors in front and an affine behind; a statistic with its elementwise consumer"""
    g = Graph()
    rng = np.random.default_rng(171)
    maps = g.input([3, 40, 7, 9])
    g.output(g.softmax(maps, 1))
    g.output(g.layernorm(maps, 1, 1e-5))
    mid = g.input([2, 300, 130], DType.F16)
    g.output(g.softmax(mid, 1))
    tall = g.input([1000, 50])
    g.output(g.layernorm(tall, 0, 1e-5))
    g.output(g.softmax(tall, 0))
    other = g.input([1000, 50])
    gamma, beta = g.input([1000, 1]), g.input([1000, 1])
    normed = g.layernorm(g.add(tall, other), 0, 1e-3)
    g.output(g.add(g.mul(normed, g.broadcast(gamma, [1000, 50])), g.broadcast(beta, [1000, 50])))
    g.output(g.sub(tall, g.broadcast(g.view(g.reduce(tall, [0], ReduceOp.MAX), [1, 50]), [1000, 50])))
    f = lambda *shape: rng.standard_normal(shape).astype(np.float32)
    return g, 0, [f(3, 40, 7, 9), rng.standard_normal((2, 300, 130)).astype(np.float16), f(1000, 50), f(1000, 50),
                  f(1000, 1), f(1000, 1)], None


@case
def columns_on_workgroups_of_1024_threads():
    """the same kernels where 256 threads would see less than a cache line per row of lanes, or could not hold the
    column in registers: 1000 positions over 96 columns (32 threads per column), layernorm over 512 channels of f16
    with an affine behind, 70 columns (the second block of 64 mostly empty), a sum in front (two tensors to hold, so
    read again per pass on 256 threads), and a column mean with its elementwise consumer"""
    g = Graph()
    rng = np.random.default_rng(184)
    tall = g.input([1000, 96])
    g.output(g.softmax(tall, 0))
    g.output(g.layernorm(g.add(tall, g.input([1000, 96])), 0, 1e-5))
    g.output(g.sub(tall, g.broadcast(g.view(g.reduce(tall, [0], ReduceOp.MEAN), [1, 96]), [1000, 96])))
    maps = g.input([3, 512, 70], DType.F16)
    gamma, beta = g.input([1, 512, 1], DType.F16), g.input([1, 512, 1], DType.F16)
    normed = g.layernorm(maps, 1, 1e-5)
    g.output(g.add(g.mul(normed, g.broadcast(gamma, [3, 512, 70])), g.broadcast(beta, [3, 512, 70])))
    f = lambda *shape: rng.standard_normal(shape).astype(np.float32)
    h = lambda *shape: rng.standard_normal(shape).astype(np.float16)
    return g, 0, [f(1000, 96), f(1000, 96), h(3, 512, 70), h(1, 512, 1), h(1, 512, 1)], None


@case
def conv_with_input_channels_in_slices():
    """few output tiles, many input channels: slices of the channels are folded side by side and a second kernel sums the
    partial results and applies bias, residual and activation. A tower block of a small batch of boards (the kernel
    that keeps raw planes in LDS), 200 channels on 5 x 5 boards (the patch kernel; 25 slices of 8 channels in 13
    parts, the last one shorter; 25 positions per image, so no vectors in the summing pass), a 5 x 5 filter, and a
    stride of 2"""
    g = Graph()
    rng = np.random.default_rng(172)
    w = lambda *shape: g.constant(list(shape), (rng.standard_normal(shape) * 0.05).astype(np.float32))
    boards = g.input([2, 128, 8, 8])
    bias = g.constant([1, 128, 1, 1], rng.standard_normal(128).astype(np.float32))
    g.output(g.relu(g.add(g.add(g.conv(boards, w(128, 128, 3, 3), 1, 1, 1, 1), bias), boards)))
    odd = g.input([1, 200, 5, 5])
    g.output(g.add(g.conv(odd, w(72, 200, 3, 3), 1, 1, 1, 1), g.constant([1, 72, 1, 1], rng.standard_normal(72).astype(np.float32))))
    g.output(g.conv(g.input([3, 64, 6, 6]), w(40, 64, 5, 5), 1, 1, 2, 2))
    g.output(g.relu(g.conv(g.input([2, 96, 9, 9]), w(64, 96, 3, 3), 2, 2, 1, 1)))
    f = lambda *shape: rng.standard_normal(shape).astype(np.float32)
    return g, 0, [f(2, 128, 8, 8), f(1, 200, 5, 5), f(3, 64, 6, 6), f(2, 96, 9, 9)], None


@case
def conv_with_a_sparse_last_round_of_tiles():
    """a tile count that leaves the last round of workgroups sparse: the tiles of that round are shared by workgroups that
    take a slice of the input channels each, and a small second kernel sums their partial tiles and applies bias,
    residual and activation. 640 tiles on power-of-two images with all three (two slices); 584 tiles on 9 x 9 boards
    (81 positions per image: tiles that straddle images, no vectors in the summing kernel); 288 tiles on 48 x 48 images
    in four slices; and, with the option off, the first one again on whole tiles"""
    from kyanite_amd import HipExecutor
    g = Graph()
    rng = np.random.default_rng(641)
    w = lambda *shape: g.constant(list(shape), (rng.standard_normal(shape) * 0.05).astype(np.float32))
    images = g.input([2, 320, 64, 64])
    bias = g.constant([1, 320, 1, 1], rng.standard_normal(320).astype(np.float32))
    g.output(g.relu(g.add(g.add(g.conv(images, w(320, 320, 3, 3), 1, 1, 1, 1), bias), images)))
    boards = g.input([230, 64, 9, 9])
    g.output(g.add(g.conv(boards, w(128, 64, 3, 3), 1, 1, 1, 1), g.constant([1, 128, 1, 1], rng.standard_normal(128).astype(np.float32))))
    wide = g.input([2, 128, 48, 48])
    g.output(g.conv(wide, w(256, 128, 3, 3), 1, 1, 1, 1))
    plan = HipExecutor(0, g, 0, plan_only=True)
    text = [plan.step_str(i) for i in range(plan.step_count())]
    assert "the tiles after 512 in 2 slices" in text[0] and "the tiles after 512 in 2 slices" in text[1] and "the tiles after 256 in 4 slices" in text[2], text
    whole = HipExecutor(0, g, 0, plan_only=True, split_conv_channels=False)
    assert not any("slices" in whole.step_str(i) for i in range(whole.step_count()))
    f = lambda *shape: rng.standard_normal(shape).astype(np.float32)
    return g, 0, [f(2, 320, 64, 64), f(230, 64, 9, 9), f(2, 128, 48, 48)], None


@case
def conv_parts_summed_inside_the_launch():
    """input channels in two and in four slices on the kernel that keeps raw planes in LDS: the workgroups of a tile park
    their partial tiles and the last one to arrive sums them and applies bias, residual and activation (no second
    kernel); twice through the same executor, so that the counters must have come back to zero"""
    from kyanite_amd import HipExecutor
    g = Graph()
    rng = np.random.default_rng(88)
    w = lambda *shape: g.constant(list(shape), (rng.standard_normal(shape) * 0.05).astype(np.float32))
    two, four = g.input([64, 128, 8, 8]), g.input([32, 128, 8, 8])
    bias = g.constant([1, 128, 1, 1], rng.standard_normal(128).astype(np.float32))
    first = g.relu(g.add(g.add(g.conv(two, w(128, 128, 3, 3), 1, 1, 1, 1), bias), two))
    g.output(g.relu(g.add(g.conv(first, w(128, 128, 3, 3), 1, 1, 1, 1), bias)))
    g.output(g.add(g.conv(four, w(72, 128, 3, 3), 1, 1, 1, 1), g.constant([1, 72, 1, 1], rng.standard_normal(72).astype(np.float32))))
    plan = HipExecutor(0, g, 0, plan_only=True)
    text = [plan.step_str(i) for i in range(plan.step_count())]
    assert sum("input channels in 2 slices" in t for t in text) == 2 and sum("input channels in 4 slices" in t for t in text) == 1, text
    # (the last operand of each is the counters: one per tile)
    assert all(t.endswith("i32[128]") or t.endswith("i32[64]") for t in text), text
    f = lambda *shape: rng.standard_normal(shape).astype(np.float32)
    return g, 0, [f(64, 128, 8, 8), f(32, 128, 8, 8)], None


@case
def products_with_few_rows():
    """a left operand of 1, 8 and 32 rows against constant [k, n] weights, f32 and f16: the weights are laid out again
    as [n, k] and the product runs on the kernel that loads global -> LDS directly (f32: on 32 x 128 tiles), with a
    last tile of columns that is partial, a bias and an activation in the store, K split where it is long, and a
    batch of left operands against one set of weights"""
    g = Graph()
    rng = np.random.default_rng(173)
    inputs = []

    def inp(shape, dtype):
        inputs.append(rng.standard_normal(shape).astype(dtype.numpy))
        return g.input(list(shape), dtype)

    def weights(k, n, dtype):
        return g.constant([k, n], (rng.standard_normal((k, n)) * 0.1).astype(dtype.numpy), dtype)

    for dtype in (DType.F32, DType.F16):
        g.output(g.mat_mul(inp((1, 256), dtype), weights(256, 300, dtype)))
        bias = g.constant([1, 520], rng.standard_normal((1, 520)).astype(dtype.numpy), dtype)
        g.output(g.relu(g.add(g.mat_mul(inp((8, 192), dtype), weights(192, 520, dtype)), g.broadcast(bias, [8, 520]))))
        g.output(g.mat_mul(inp((32, 4096), dtype), weights(4096, 136, dtype)))
        w = g.view(weights(128, 260, dtype), [1, 128, 260])
        g.output(g.batched_mat_mul(inp((3, 5, 128), dtype), g.broadcast(w, [3, 128, 260])))
    return g, 0, inputs, None


@case
def conv_on_boards_of_any_size():
    """3 x 3 same-size convolutions on images whose width is no power of two run on the kernel that keeps raw planes in
    LDS too: a tile is 128 (or 64) consecutive positions wherever they start, and stages the padded rows around them,
    across image boundaries. 9 x 9 boards with bias, residual and activation and a last tile that is partial; 7 x 7;
    19 x 19 (a tile holds a third of an image); 5 rows of 3; 3 x 3 boards (forty images per tile); 21 input planes
    (a channel count that is no multiple of 8); and a batch small enough that the input channels are split"""
    g = Graph()
    rng = np.random.default_rng(174)
    inputs = []

    def inp(*shape):
        inputs.append(rng.standard_normal(shape).astype(np.float32))
        return g.input(list(shape))

    w = lambda *shape: g.constant(list(shape), (rng.standard_normal(shape) * 0.05).astype(np.float32))
    boards = inp(37, 72, 9, 9)
    bias = g.constant([1, 72, 1, 1], rng.standard_normal(72).astype(np.float32))
    g.output(g.relu(g.add(g.add(g.conv(boards, w(72, 72, 3, 3), 1, 1, 1, 1), bias), boards)))
    g.output(g.conv(inp(20, 64, 7, 7), w(130, 64, 3, 3), 1, 1, 1, 1))
    g.output(g.conv(inp(3, 32, 19, 19), w(64, 32, 3, 3), 1, 1, 1, 1))
    g.output(g.conv(inp(11, 16, 5, 3), w(8, 16, 3, 3), 1, 1, 1, 1))
    g.output(g.conv(inp(50, 16, 3, 3), w(24, 16, 3, 3), 1, 1, 1, 1))
    g.output(g.relu(g.conv(inp(9, 21, 9, 9), w(40, 21, 3, 3), 1, 1, 1, 1)))
    g.output(g.conv(inp(2, 128, 9, 9), w(64, 128, 3, 3), 1, 1, 1, 1))
    return g, 0, inputs, None


@case
def conv_on_images_with_rows_of_whole_vectors():
    """the same kernel on image widths that are a multiple of 4 but no power of two (56, 28, 12, 20): the padded rows are
    staged four floats at a time. A tile of 128 positions is a little over two rows of a 56 x 56 image; 21 input planes;
    an input that is a slice of a larger tensor, so that its rows lose their alignment (float by float then)"""
    g = Graph()
    rng = np.random.default_rng(175)
    inputs = []

    def inp(*shape):
        inputs.append(rng.standard_normal(shape).astype(np.float32))
        return g.input(list(shape))

    w = lambda *shape: g.constant(list(shape), (rng.standard_normal(shape) * 0.05).astype(np.float32))
    g.output(g.relu(g.conv(inp(2, 16, 56, 56), w(24, 16, 3, 3), 1, 1, 1, 1)))
    g.output(g.conv(inp(3, 24, 28, 28), w(70, 24, 3, 3), 1, 1, 1, 1))
    g.output(g.conv(inp(5, 8, 12, 12), w(16, 8, 3, 3), 1, 1, 1, 1))
    g.output(g.conv(inp(2, 21, 12, 20), w(32, 21, 3, 3), 1, 1, 1, 1))
    wide = inp(2, 8, 12, 13)
    g.output(g.conv(g.slice(wide, 3, 1, 13), w(16, 8, 3, 3), 1, 1, 1, 1))
    return g, 0, inputs, None


@case
def conv_five_by_five_on_planes():
    """5 x 5 filters with padding 2 on power-of-two image widths read their taps from staged planes like 3 x 3 ones, in
    slices of four input channels: a tile that is part of an image (32 x 32), whole images per tile (8 x 8, 4 x 4),
    128 output channels on many positions (two tiles of 64), 6 input channels (no whole slices: the kernel that
    gathers patches), bias + skip connection + relu in the store, and a batch small enough for the input channels
    to go in slices"""
    g = Graph()
    rng = np.random.default_rng(181)
    inputs = []

    def inp(*shape):
        inputs.append(rng.standard_normal(shape).astype(np.float32))
        return g.input(list(shape))

    w = lambda *shape: g.constant(list(shape), (rng.standard_normal(shape) * 0.05).astype(np.float32))
    g.output(g.conv(inp(3, 8, 32, 32), w(24, 8, 5, 5), 1, 1, 2, 2))
    g.output(g.conv(inp(37, 12, 8, 8), w(70, 12, 5, 5), 1, 1, 2, 2))
    g.output(g.conv(inp(9, 4, 4, 4), w(8, 4, 5, 5), 1, 1, 2, 2))
    g.output(g.conv(inp(256, 8, 16, 16), w(128, 8, 5, 5), 1, 1, 2, 2))
    g.output(g.conv(inp(2, 6, 16, 8), w(16, 6, 5, 5), 1, 1, 2, 2))
    x, skip = inp(4, 8, 16, 16), inp(4, 16, 16, 16)
    y = g.add(g.conv(x, w(16, 8, 5, 5), 1, 1, 2, 2), g.broadcast(w(1, 16, 1, 1), [4, 16, 16, 16]))
    g.output(g.relu(g.add(y, skip)))
    g.output(g.conv(inp(2, 64, 8, 8), w(32, 64, 5, 5), 1, 1, 2, 2))
    return g, 0, inputs, None


@case
def conv_five_by_five_on_boards_of_any_size():
    """the same on image sizes that are no power of two: the 22 input planes of a Go network on 19 x 19 (no whole
    slices of four channels: the kernel that gathers patches), 20 planes on the same boards, 9 x 9 boards, 28 x 28 images (rows of whole vectors), a 5 x 3 and a 2 x 2
    image (smaller than the filter), bias and relu in the store, and few boards with many channels (in slices)"""
    g = Graph()
    rng = np.random.default_rng(185)
    inputs = []

    def inp(*shape):
        inputs.append(rng.standard_normal(shape).astype(np.float32))
        return g.input(list(shape))

    w = lambda *shape: g.constant(list(shape), (rng.standard_normal(shape) * 0.05).astype(np.float32))
    stem = g.add(g.conv(inp(3, 22, 19, 19), w(96, 22, 5, 5), 1, 1, 2, 2), g.broadcast(w(1, 96, 1, 1), [3, 96, 19, 19]))
    g.output(g.relu(stem))
    g.output(g.conv(inp(2, 20, 19, 19), w(40, 20, 5, 5), 1, 1, 2, 2))
    g.output(g.conv(inp(11, 8, 9, 9), w(24, 8, 5, 5), 1, 1, 2, 2))
    g.output(g.conv(inp(2, 12, 28, 28), w(70, 12, 5, 5), 1, 1, 2, 2))
    g.output(g.conv(inp(7, 4, 5, 3), w(8, 4, 5, 5), 1, 1, 2, 2))
    g.output(g.conv(inp(40, 5, 2, 2), w(8, 5, 5, 5), 1, 1, 2, 2))
    g.output(g.conv(inp(1, 64, 9, 9), w(32, 64, 5, 5), 1, 1, 2, 2))
    return g, 0, inputs, None


@case
def tiny_products_one_wave_per_result():
    """products of a few thousand multiplications run with one wave per result and lanes along K: K shorter than a wave
    (5) and no multiple of it (200), a transposed right operand, a batch, bias and skip connection and activation in
    the store, f16 with its roundings, and a single dot product"""
    g = Graph()
    rng = np.random.default_rng(176)
    inputs = []

    def inp(shape, dtype=DType.F32):
        inputs.append(rng.standard_normal(shape).astype(dtype.numpy))
        return g.input(list(shape), dtype)

    g.output(g.mat_mul(inp((7, 5)), inp((5, 3))))
    g.output(g.mat_mul(inp((1, 200)), g.permute(inp((9, 200)), [1, 0])))
    x, skip = inp((3, 6, 40)), inp((3, 6, 10))
    w = g.constant([1, 40, 10], rng.standard_normal((1, 40, 10)).astype(np.float32))
    bias = g.constant([1, 1, 10], rng.standard_normal((1, 1, 10)).astype(np.float32))
    g.output(g.relu(g.add(skip, g.add(g.batched_mat_mul(x, g.broadcast(w, [3, 40, 10])), g.broadcast(bias, [3, 6, 10])))))
    h = inp((4, 100), DType.F16)
    hw = g.constant([100, 12], (rng.standard_normal((100, 12)) * 0.2).astype(np.float16), DType.F16)
    hb = g.constant([1, 12], rng.standard_normal((1, 12)).astype(np.float16), DType.F16)
    g.output(g.relu(g.add(g.mat_mul(h, hw), g.broadcast(hb, [4, 12]))))
    g.output(g.mat_mul(inp((1, 256)), inp((256, 1))))
    from kyanite_amd import HipExecutor
    ex = HipExecutor(0, g, 0, plan_only=True)
    assert all("a wave per result" in ex.step_str(i) for i in range(ex.step_count()) if ex.step_kinds()[i] == "mat_mul")
    return g, 0, inputs, None


@case
def few_long_rows():
    """a softmax or layernorm over a few rows of 64 Ki elements or more runs as two steps that use the whole chip (the
    statistics of every row as a reduction over pairs, slices of a row side by side; then one elementwise kernel)
    instead of one workgroup per row: along the last axis, and along a middle axis with three columns behind it"""
    g = Graph()
    rng = np.random.default_rng(177)
    a, b, c = g.input([3, 70000]), g.input([2, 100000]), g.input([2, 66000, 3])
    g.output(g.softmax(a, 1))
    g.output(g.layernorm(b, 1, 1e-5))
    g.output(g.softmax(c, 1))
    g.output(g.layernorm(c, 1, 1e-3))
    from kyanite_amd import HipExecutor
    kinds = HipExecutor(0, g, 0, plan_only=True).step_kinds()
    assert "softmax_op" not in kinds and "layernorm_op" not in kinds, kinds
    f = lambda *shape: (rng.standard_normal(shape) * 3).astype(np.float32)
    return g, 0, [f(3, 70000), f(2, 100000), f(2, 66000, 3)], None


@case
def byte_transposes():
    """elementwise kernels over one-byte elements with a transposed operand: tiles of 128 x 128 with a word of four
    elements per thread (u8 with a straight operand next to the transposed one, sizes that are no multiple of the tile,
    i8 with batch axes, bool), and shapes that keep the tiles of 64 x 64 (a length that is no multiple of 4, a
    broadcast operand)"""
    from kyanite_amd import HipExecutor
    g = Graph()
    rng = np.random.default_rng(433)
    u8 = lambda *shape: rng.integers(0, 256, size=shape, dtype=np.uint8)
    a, b = u8(300, 520), u8(520, 300)
    xa, xb = g.input([300, 520], DType.U8), g.input([520, 300], DType.U8)
    g.output(g.add(g.permute(xa, [1, 0]), xb))
    c = rng.integers(-128, 128, size=(3, 5, 132, 260), dtype=np.int8)
    xc = g.input([3, 5, 132, 260], DType.I8)
    g.output(g.mul(g.permute(xc, [0, 1, 3, 2]), g.scalar(3, DType.I8)))
    d = rng.integers(0, 2, size=(256, 384)).astype(bool)
    e = rng.integers(0, 2, size=(384, 256)).astype(bool)
    xd, xe = g.input([256, 384], DType.BOOL), g.input([384, 256], DType.BOOL)
    g.output(g.mul(g.permute(xd, [1, 0]), xe))
    f = u8(258, 514)
    xf = g.input([258, 514], DType.U8)
    g.output(g.add(g.permute(xf, [1, 0]), g.scalar(1, DType.U8)))
    h, column = u8(260, 512), u8(512, 1)
    xh = g.input([260, 512], DType.U8)
    g.output(g.add(g.permute(xh, [1, 0]), g.constant([512, 1], column, DType.U8)))
    plan = HipExecutor(0, g, 0, plan_only=True)
    text = [plan.step_str(i) for i in range(plan.step_count())]
    assert sum("128x128 of bytes" in t for t in text) == 3 and sum("tiles 64x64" in t for t in text) == 2, text
    return g, 0, [a, b, c, d, e, f, h], None


@case
def rows_in_two_passes():
    """rows or columns that no workgroup can hold, as a reduction to (maximum, 1 / sum of exponentials) or (mean,
    1 / sqrt(variance + eps)) and an elementwise kernel that also applies the epilogue: columns of a tall matrix (with
    columns of -inf, with +inf, with a NaN), a layernorm along axis 0 with gamma and beta behind it, a softmax over a
    long middle axis, a few long rows with an affine epilogue, enough rows that no row is cut into slices, and columns
    of halves (computed in f32, rounded once)"""
    from kyanite_amd import HipExecutor
    g = Graph()
    rng = np.random.default_rng(977)
    tall = (rng.standard_normal((2500, 192)) * 4).astype(np.float32)
    tall[:, 3] = -np.inf
    tall[:700, 5] = -np.inf
    tall[1200, 7] = np.inf
    tall[2499, 9] = np.nan
    tall[0, 11] = -np.inf
    g.output(g.softmax(g.input([2500, 192]), 0))
    cols = (rng.standard_normal((1500, 96)) * 2 + 5).astype(np.float32)
    gamma, beta = rng.standard_normal((1, 96)).astype(np.float32), rng.standard_normal((1500, 1)).astype(np.float32)
    y = g.layernorm(g.input([1500, 96]), 0, 1e-5)
    g.output(g.add(g.mul(y, g.constant([1, 96], gamma)), g.constant([1500, 1], beta)))
    middle = rng.standard_normal((40, 3000, 48)).astype(np.float32)
    g.output(g.softmax(g.input([40, 3000, 48]), 1))
    long_rows = (rng.standard_normal((4, 100000)) * 3 - 2).astype(np.float32)
    w = rng.standard_normal((1, 100000)).astype(np.float32)
    g.output(g.add(g.mul(g.layernorm(g.input([4, 100000]), 1, 1e-3), g.constant([1, 100000], w)), g.scalar(0.5)))
    many = rng.standard_normal((300, 70000)).astype(np.float32)
    g.output(g.softmax(g.input([300, 70000]), 1))
    halves = (rng.standard_normal((3000, 128)) * 2 + 1).astype(np.float16)
    scale = rng.standard_normal((1, 128)).astype(np.float16)
    g.output(g.mul(g.layernorm(g.input([3000, 128], DType.F16), 0, 1e-3), g.constant([1, 128], scale, DType.F16)))
    g.output(g.softmax(g.input([3000, 128], DType.F16), 0))
    plan = HipExecutor(0, g, 0, plan_only=True)
    kinds = plan.step_kinds()
    assert "softmax_op" not in kinds and "layernorm_op" not in kinds, kinds
    text = "\n".join(plan.step_str(i) for i in range(plan.step_count()))
    assert text.count("maximum and sum of exponentials") == 4 and text.count("mean and variance") == 3, text
    return g, 0, [tall, cols, middle, long_rows, many, halves, halves.copy()], None


@case
def rows_too_long_for_registers():
    """rows of more than 64 elements per lane of 1024 are read again per pass, by a softmax twice (maximum and sum of
    exponentials in one pass): an odd length (element by element), whole vectors, f16; rows that start with -inf (the
    running maximum is still -inf there), hold +inf, a NaN, or nothing but -inf; and a layernorm, which takes three
    passes"""
    g = Graph()
    rng = np.random.default_rng(186)
    odd = rng.standard_normal((70, 70001)).astype(np.float32) * 3
    odd[0, :5000] = -np.inf
    odd[1, 1::2] = -np.inf
    odd[2, 40000] = np.inf
    odd[3, 69000] = np.nan
    odd[4, :] = -np.inf
    odd[5, :60000] = -np.inf
    odd[5, 60000] = np.nan
    g.output(g.softmax(g.input([70, 70001]), 1))
    whole = rng.standard_normal((66, 132000)).astype(np.float32)
    g.output(g.softmax(g.input([66, 132000]), 1))
    halves = (rng.standard_normal((65, 90000)) * 2).astype(np.float16)
    g.output(g.softmax(g.input([65, 90000], DType.F16), 1))
    g.output(g.layernorm(g.input([66, 132000]), 1, 1e-5))
    return g, 0, [odd, whole, halves, whole.copy()], None


@case
def special_values_on_the_split_paths():
    """infinities and NaN through the kernels that split their work: a softmax along axis 0 (lanes across columns) with a
    column that is all -inf, one that holds +inf and one with a NaN; reductions in two launches whose input holds NaN
    (ignored by min and max, kept by sum) and infinities; a softmax over long rows (separate steps) with -inf entries
    and a row that is all -inf; the same down columns of 1000 that are read twice"""
    g = Graph()
    rng = np.random.default_rng(179)
    cols = rng.standard_normal((37, 40)).astype(np.float32)
    cols[:, 3] = -np.inf
    cols[5, 7] = np.inf
    cols[9, 11] = np.nan
    cols[2:30, 20] = -np.inf
    g.output(g.softmax(g.input([37, 40]), 0))
    tall = rng.standard_normal((70001, 96)).astype(np.float32)
    tall[123, 4] = np.nan
    tall[60000, 9] = np.inf
    tall[69999, 50] = -np.inf
    t = g.input([70001, 96])
    for op in (ReduceOp.MIN, ReduceOp.MAX, ReduceOp.SUM):
        g.output(g.reduce(t, [0], op))
    rows = rng.standard_normal((3, 70000)).astype(np.float32)
    rows[0, 100:50000] = -np.inf
    rows[1, :] = -np.inf
    g.output(g.softmax(g.input([3, 70000]), 1))
    # columns too long to hold (read twice): one that starts with -inf, one that is all -inf, a NaN, a +inf
    long_cols = (rng.standard_normal((1000, 50)) * 3).astype(np.float32)
    long_cols[:700, 2] = -np.inf
    long_cols[:, 5] = -np.inf
    long_cols[321, 8] = np.nan
    long_cols[999, 13] = np.inf
    long_cols[::2, 21] = -np.inf
    g.output(g.softmax(g.input([1000, 50]), 0))
    return g, 0, [cols, tall, rows, long_cols], None


@case
def one_workgroup_plays_several():
    """graphs small enough to run as one kernel whose steps were written for 2 to 4 workgroups with LDS of their own:
    rows folded by all 256 lanes (one LDS exchange per row), columns folded through LDS, a softmax of 4 long rows; the
    one workgroup takes the turns of all of them, with a barrier between the turns"""
    g = Graph()
    rng = np.random.default_rng(211)
    rows = rng.standard_normal((3, 16384)).astype(np.float32)
    g.output(g.unary(UnaryOp.SIGMOID, g.reduce(g.input([3, 16384]), [1], ReduceOp.SUM)))
    cols = rng.standard_normal((512, 96)).astype(np.float32)
    g.output(g.unary(UnaryOp.EXP, g.reduce(g.input([512, 96]), [0], ReduceOp.MAX)))
    soft = rng.standard_normal((4, 3000)).astype(np.float32)
    g.output(g.softmax(g.input([4, 3000]), 1))
    return g, 0, [rows, cols, soft], None


def _gated_feed_forward(seed, m, k, n, order=0, extra_use=False, weights_kn=False):
    """act = (x w_g) sigmoid(x w_g) (x w_u) in f16, spelled in one of four operand orders"""
    g = Graph()
    rng = np.random.default_rng(seed)
    x = g.input([m, k], DType.F16)

    def weight():
        w = (rng.standard_normal((n, k)) / np.sqrt(k)).astype(np.float16)
        if weights_kn:
            return g.mat_mul(x, g.constant([k, n], np.ascontiguousarray(w.T), DType.F16))
        return g.linear(x, g.constant([n, k], w, DType.F16))

    gate, up = weight(), weight()
    sig = g.sigmoid(gate)
    inner = g.mul(gate, sig) if order & 1 == 0 else g.mul(sig, gate)
    act = g.mul(inner, up) if order & 2 == 0 else g.mul(up, inner)
    g.output(act)
    if extra_use:
        g.output(g.unary(UnaryOp.NEG, gate))  # the gate is needed on its own as well: nothing to fuse
    return g, 0, [(rng.standard_normal((m, k)) * 1.5).astype(np.float16)], None


@case
def gated_matmul_ragged():
    """rows and columns that fill no tile (m 200 of 256, 424 = 26.5 blocks of 16 columns), K of two slices"""
    return _gated_feed_forward(301, 200, 128, 424)


@case
def gated_matmul_orders():
    """sigmoid(g) * g and u * (...): the other operand orders of the same product"""
    g1, _, in1, _ = _gated_feed_forward(302, 64, 64, 48, order=3)
    return g1, 0, in1, None


@case
def gated_matmul_order_1():
    return _gated_feed_forward(303, 130, 192, 256, order=1)


@case
def gated_matmul_order_2_kn_weights():
    """weights stored [k, n] (`x @ w`): laid out again as [n, k] when the plan is made, then paired"""
    return _gated_feed_forward(304, 256, 256, 512, order=2, weights_kn=True)


@case
def gated_matmul_wide():
    """more than one tile in both directions on the 256 x 192 tiles a tall product picks"""
    return _gated_feed_forward(305, 512, 256, 1000)


@case
def gated_matmul_gate_used_elsewhere():
    """the gate is an output too: the three launches stay"""
    return _gated_feed_forward(306, 96, 128, 160, extra_use=True)


@case
def rows_of_odd_length():
    """rows held in registers whose length is no multiple of the 128 bit vector and whose start falls on any element:
    vectors at any alignment, the last one overlapping its neighbour (its repeated elements stay out of the sums);
    softmax with a scaled input, layernorm with gamma / beta, an RMS norm, in f32 and f16; a slice that starts one
    element into each row (length a multiple of the vector, start not); -inf entries next to the row's end"""
    g = Graph()
    rng = np.random.default_rng(307)
    a = rng.standard_normal((5, 4097)).astype(np.float32)
    a[2, 4090:] = -np.inf
    a[3, 4096] = 30.0
    xa = g.input([5, 4097])
    g.output(g.softmax(g.mul(xa, g.scalar(0.5)), 1))
    gamma, beta = g.constant([4097], rng.standard_normal(4097).astype(np.float32)), g.constant([4097], rng.standard_normal(4097).astype(np.float32))
    b = rng.standard_normal((7, 4097)).astype(np.float32)
    g.output(g.add(g.mul(g.layernorm(g.input([7, 4097]), 1, 1e-5), gamma), beta))
    c = rng.standard_normal((3, 8191)).astype(np.float16)
    xc = g.input([3, 8191], DType.F16)
    g.output(g.softmax(xc, 1))
    g.output(g.layernorm(xc, 1, 1e-3))
    d = rng.standard_normal((6, 5003)).astype(np.float32)
    xd = g.input([6, 5003])
    ms = g.view(g.reduce(g.mul(xd, xd), [1], ReduceOp.MEAN), [6, 1])
    g.output(g.binary(BinaryOp.DIV, xd, g.unary(UnaryOp.SQRT, g.add(ms, g.scalar(1e-6)))))
    e = rng.standard_normal((4, 4100)).astype(np.float32)
    g.output(g.softmax(g.slice(g.input([4, 4100]), 1, 1, 4097), 1))
    return g, 0, [a, b, c, d, e], None


@case
def reduce_many_short_rows():
    """sums, maxima and means over short rows whose length is no multiple of the vector: 256 rows at a time through LDS
    (the last workgroup has fewer; 16500 rows of 7 halves are no whole number of vectors)"""
    g = Graph()
    rng = np.random.default_rng(311)
    a = rng.standard_normal((20001, 33)).astype(np.float32)
    xa = g.input([20001, 33])
    g.output(g.reduce(xa, [1], ReduceOp.SUM))
    g.output(g.reduce(xa, [1], ReduceOp.MEAN))
    b = rng.standard_normal((16500, 7)).astype(np.float16)
    b[5, :] = -np.inf
    b[9, 3] = np.nan
    g.output(g.reduce(g.input([16500, 7], DType.F16), [1], ReduceOp.MAX))
    c = rng.integers(-1000, 1000, size=(17000, 13), dtype=np.int32)
    g.output(g.reduce(g.input([17000, 13], DType.I32), [1], ReduceOp.SUM))
    d = rng.integers(0, 255, size=(40000, 5), dtype=np.uint8)
    g.output(g.reduce(g.input([40000, 5], DType.U8), [1], ReduceOp.MIN))
    return g, 0, [a, b, c, d], None
