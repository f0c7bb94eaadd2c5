"""Python face of the graph IR, a thin ctypes layer over the C++ builder in libknhip.

Names and argument meaning follow kn-graph (graph.rs, shape.rs, dtype.rs of the reference) so that tests read
like the reference's own: `graph.input(shape, dtype)`, `graph.constant(shape, data)`, `graph.linear(x, w)`, ...
"""
import ctypes
import enum
from ctypes import byref, c_float, c_int, c_size_t, c_uint8, c_uint32, c_uint64, c_void_p

import numpy as np

from ._lib import KnError, OptimizerSettingsT, SizeT, ValueInfoT, check, get_string, lib


class DType(enum.IntEnum):
    F32 = 0
    F64 = 1
    I8 = 2
    I16 = 3
    I32 = 4
    I64 = 5
    U8 = 6
    U16 = 7
    U32 = 8
    U64 = 9
    BOOL = 10
    F16 = 11

    @property
    def numpy(self):
        return _NUMPY[self]

    @staticmethod
    def from_numpy(dt):
        dt = np.dtype(dt)
        for k, v in _NUMPY.items():
            if v == dt:
                return k
        raise KnError(f"unsupported numpy dtype {dt}")

    def is_float(self):
        return self in (DType.F32, DType.F64, DType.F16)


_NUMPY = {
    DType.F32: np.dtype(np.float32), DType.F64: np.dtype(np.float64), DType.I8: np.dtype(np.int8),
    DType.I16: np.dtype(np.int16), DType.I32: np.dtype(np.int32), DType.I64: np.dtype(np.int64),
    DType.U8: np.dtype(np.uint8), DType.U16: np.dtype(np.uint16), DType.U32: np.dtype(np.uint32),
    DType.U64: np.dtype(np.uint64), DType.BOOL: np.dtype(np.bool_), DType.F16: np.dtype(np.float16),
}


class UnaryOp(enum.IntEnum):
    ABS = 0
    NEG = 1
    SIN = 2
    COS = 3
    EXP = 4
    LOG = 5
    SQRT = 6
    SIGMOID = 7
    TANH = 8
    ERF = 9
    MISH = 10
    SOFTPLUS = 11
    VALUE_CAST = 12
    BIT_CAST = 13


UNARY_ALL = [UnaryOp(i) for i in range(12)]  # UnaryOp::ALL, graph.rs:1598-1611 (casts excluded)


class BinaryOp(enum.IntEnum):
    ADD = 0
    SUB = 1
    MUL = 2
    DIV = 3
    MIN = 4
    MAX = 5
    POW = 6


BINARY_ALL = list(BinaryOp)


class ReduceOp(enum.IntEnum):
    SUM = 0
    MEAN = 1
    PROD = 2
    MAX = 3
    MIN = 4


REDUCE_ALL = list(ReduceOp)


class OpKind(enum.IntEnum):
    INPUT = 0
    CONSTANT = 1
    VIEW = 2
    BROADCAST = 3
    PERMUTE = 4
    SLICE = 5
    FLIP = 6
    GATHER = 7
    CONCAT = 8
    CONV = 9
    MATMUL = 10
    UNARY = 11
    BINARY = 12
    SOFTMAX = 13
    LAYERNORM = 14
    REDUCE = 15


class Size:
    """`fixed_factor * batch_size ** batch_exp` (shape.rs:31-38)."""

    __slots__ = ("batch_exp", "fixed_factor")

    def __init__(self, batch_exp, fixed_factor):
        if fixed_factor == 0:
            batch_exp = 0
        self.batch_exp = int(batch_exp)
        self.fixed_factor = int(fixed_factor)

    @staticmethod
    def fixed(n):
        return Size(0, n)

    @staticmethod
    def of(x):
        return x if isinstance(x, Size) else Size(0, int(x))

    def eval(self, batch_size):
        return self.fixed_factor * batch_size ** self.batch_exp

    def __mul__(self, other):
        other = Size.of(other)
        return Size(self.batch_exp + other.batch_exp, self.fixed_factor * other.fixed_factor)

    __rmul__ = __mul__

    def __eq__(self, other):
        other = Size.of(other)
        return self.batch_exp == other.batch_exp and self.fixed_factor == other.fixed_factor

    def __hash__(self):
        return hash((self.batch_exp, self.fixed_factor))

    def __repr__(self):
        if self.batch_exp == 0:
            return str(self.fixed_factor)
        f = "" if self.fixed_factor == 1 else str(self.fixed_factor)
        return f + ("B" if self.batch_exp == 1 else f"B^{self.batch_exp}")


Size.ZERO = Size(0, 0)
Size.ONE = Size(0, 1)
Size.BATCH = Size(1, 1)
BATCH = Size.BATCH


def shape(*dims):
    """`shape![...]`: a list of Size from ints and Size values."""
    if len(dims) == 1 and isinstance(dims[0], (list, tuple)):
        dims = dims[0]
    return [Size.of(d) for d in dims]


def _dims(dims):
    dims = [Size.of(d) for d in dims]
    arr = (SizeT * max(len(dims), 1))()
    for i, d in enumerate(dims):
        arr[i] = SizeT(d.fixed_factor, d.batch_exp)
    return arr, len(dims)


def _sizes(values):
    arr = (c_size_t * max(len(values), 1))(*values)
    return arr, len(values)


class Value(int):
    """Index of a value in its graph."""

    def __repr__(self):
        return f"Value({int(self)})"


class OptimizerSettings:
    def __init__(self, optimize=True, force_bias_through_conv=False, fuse_layernorm=True, div_to_mul=True):
        self.optimize = optimize
        self.force_bias_through_conv = force_bias_through_conv
        self.fuse_layernorm = fuse_layernorm
        self.div_to_mul = div_to_mul


class ValueInfo:
    def __init__(self, graph, value):
        info = ValueInfoT()
        check(lib.knhip_graph_value_info(graph._h, value, byref(info)))
        self.dtype = DType(info.dtype)
        self.op = OpKind(info.op)
        self.sub_op = info.sub_op
        self.cast_dtype = DType(info.cast_dtype) if info.cast_dtype >= 0 else None
        self.non_output_uses = info.non_output_uses
        self.slice = (info.slice_start, info.slice_end, info.slice_step)
        self.eps = info.eps
        self.is_hidden = bool(info.is_hidden)
        dims = (SizeT * max(info.rank, 1))()
        check(lib.knhip_graph_value_shape(graph._h, value, dims, info.rank))
        self.shape = [Size(dims[i].batch_exp, dims[i].fixed_factor) for i in range(info.rank)]
        ops = (c_uint32 * max(info.operand_count, 1))()
        check(lib.knhip_graph_value_operands(graph._h, value, ops, info.operand_count))
        self.operands = [Value(ops[i]) for i in range(info.operand_count)]
        axes = (c_size_t * max(info.axis_count, 1))()
        check(lib.knhip_graph_value_axes(graph._h, value, axes, info.axis_count))
        self.axes = [axes[i] for i in range(info.axis_count)]

    def __repr__(self):
        return f"ValueInfo({self.op.name}, shape={self.shape}, dtype={self.dtype.name}, operands={self.operands}, axes={self.axes})"


class Graph:
    def __init__(self, _handle=None):
        if _handle is None:
            h = c_void_p()
            check(lib.knhip_graph_new(byref(h)))
            _handle = h
        self._h = _handle

    def __del__(self):
        h = getattr(self, "_h", None)
        if h is not None and lib is not None:
            lib.knhip_graph_free(h)
            self._h = None

    # ---- (de)serialisation
    def to_bytes(self):
        needed = c_size_t()
        check(lib.knhip_graph_serialize(self._h, None, 0, byref(needed)))
        buf = (c_uint8 * needed.value)()
        check(lib.knhip_graph_serialize(self._h, buf, needed.value, byref(needed)))
        return bytes(buf)

    @staticmethod
    def from_bytes(data):
        buf = (c_uint8 * len(data)).from_buffer_copy(data)
        h = c_void_p()
        check(lib.knhip_graph_deserialize(buf, len(data), byref(h)))
        return Graph(h)

    def clone(self):
        h = c_void_p()
        check(lib.knhip_graph_clone(self._h, byref(h)))
        return Graph(h)

    def __str__(self):
        return get_string(lib.knhip_graph_str, self._h)

    # ---- queries
    def __len__(self):
        n = c_size_t()
        check(lib.knhip_graph_value_count(self._h, byref(n)))
        return n.value

    def values(self):
        return [Value(i) for i in range(len(self))]

    def __getitem__(self, value):
        return ValueInfo(self, value)

    def _list(self, fn):
        n = c_size_t()
        check(fn(self._h, None, 0, byref(n)))
        buf = (c_uint32 * max(n.value, 1))()
        check(fn(self._h, buf, n.value, byref(n)))
        return [Value(buf[i]) for i in range(n.value)]

    def inputs(self):
        return self._list(lib.knhip_graph_inputs)

    def outputs(self):
        return self._list(lib.knhip_graph_outputs)

    def input_shapes(self):
        return [self[v].shape for v in self.inputs()]

    def output_shapes(self):
        return [self[v].shape for v in self.outputs()]

    def constant_data(self, value):
        info = self[value]
        ptr, n = c_void_p(), c_size_t()
        check(lib.knhip_graph_value_constant(self._h, value, byref(ptr), byref(n)))
        dims = [d.fixed_factor for d in info.shape]
        if n.value == 0:
            return np.zeros(dims, info.dtype.numpy)
        raw = ctypes.string_at(ptr.value, n.value)
        return np.frombuffer(raw, dtype=info.dtype.numpy).reshape(dims).copy()

    def as_single_const(self, value):
        flag = c_int()
        buf = (c_uint8 * 8)()
        check(lib.knhip_graph_as_single_const(self._h, value, byref(flag), buf))
        if not flag.value:
            return None
        dt = self[value].dtype.numpy
        return np.frombuffer(bytes(buf)[: dt.itemsize], dtype=dt)[0]

    def as_const(self, value):
        """Graph::as_const (graph.rs:435-474): the value as a numpy array when it is computable from constants alone."""
        info = self[value]
        flag, needed = c_int(), c_size_t()
        check(lib.knhip_graph_as_const(self._h, value, byref(flag), None, 0, byref(needed)))
        if not flag.value:
            return None
        dims = [d.fixed_factor for d in info.shape]
        buf = (c_uint8 * max(needed.value, 1))()
        check(lib.knhip_graph_as_const(self._h, value, byref(flag), buf, needed.value, byref(needed)))
        return np.frombuffer(bytes(buf)[: needed.value], dtype=info.dtype.numpy).reshape(dims).copy()

    def infer_batch_size(self, actual_shapes):
        """Returns (status, batch) with status 0 on success; batch is None when any batch size fits."""
        flat = [d for s in actual_shapes for d in s]
        ranks = [len(s) for s in actual_shapes]
        a, _ = _sizes(flat)
        r, n = _sizes(ranks)
        status, has, batch = c_int(), c_int(), c_uint64()
        check(lib.knhip_graph_infer_batch_size(self._h, a, r, n, byref(status), byref(has), byref(batch)))
        return status.value, (batch.value if has.value else None)

    # ---- builder (graph.rs:583-1363)
    def _out(self, fn, *args):
        v = c_uint32()
        check(fn(self._h, *args, byref(v)))
        return Value(v.value)

    def input(self, shp, dtype=DType.F32):
        d, n = _dims(shp)
        return self._out(lib.knhip_graph_input, d, n, int(dtype))

    def constant(self, shp, data, dtype=None):
        """`graph.constant(shape, data)`; data is anything numpy can convert, flat or already shaped."""
        arr = np.asarray(data)
        if dtype is None:
            if arr.dtype == np.float64 and not isinstance(data, np.ndarray):
                arr = arr.astype(np.float32)  # python floats mean f32, like the reference's default literals
            dtype = DType.from_numpy(arr.dtype)
        arr = np.ascontiguousarray(arr, dtype=DType(dtype).numpy)
        d, n = _dims(shp)
        ptr = arr.ctypes.data_as(c_void_p)
        return self._out(lib.knhip_graph_constant, d, n, int(dtype), ptr, arr.nbytes)

    def constant_tensor(self, array):
        arr = np.asarray(array)
        return self.constant(list(arr.shape), arr)

    def scalar(self, value, dtype=DType.F32):
        return self.constant([], np.asarray(value, dtype=DType(dtype).numpy), dtype)

    def view(self, input, new_shape):
        d, n = _dims(new_shape)
        return self._out(lib.knhip_graph_view, input, d, n)

    def broadcast(self, input, new_shape):
        d, n = _dims(new_shape)
        return self._out(lib.knhip_graph_broadcast, input, d, n)

    def repeat_unary(self, input, axis, count):
        c = Size.of(count)
        return self._out(lib.knhip_graph_repeat_unary, input, axis, SizeT(c.fixed_factor, c.batch_exp))

    def flatten(self, input, start_axis):
        return self._out(lib.knhip_graph_flatten, input, start_axis)

    def permute(self, input, permutation):
        p, n = _sizes(list(permutation))
        return self._out(lib.knhip_graph_permute, input, p, n)

    def slice(self, input, axis, start, end, step=1):
        return self._out(lib.knhip_graph_slice, input, axis, start, end, step)

    def index(self, input, axis, index):
        return self._out(lib.knhip_graph_index, input, axis, index)

    def flip(self, input, axis):
        return self._out(lib.knhip_graph_flip, input, axis)

    def repeat(self, input, axis, count):
        c = Size.of(count)
        return self._out(lib.knhip_graph_repeat, input, axis, SizeT(c.fixed_factor, c.batch_exp), 0)

    def repeat_interleave(self, input, axis, count):
        c = Size.of(count)
        return self._out(lib.knhip_graph_repeat, input, axis, SizeT(c.fixed_factor, c.batch_exp), 1)

    def gather(self, input, axis, indices):
        return self._out(lib.knhip_graph_gather, input, axis, indices)

    def concat(self, inputs, axis, base_shape=None, dtype=None):
        arr = (c_uint32 * max(len(inputs), 1))(*inputs)
        if base_shape is None:
            d, n = None, 0
        else:
            d, n = _dims(base_shape)
        return self._out(lib.knhip_graph_concat, arr, len(inputs), axis, d, n, -1 if dtype is None else int(dtype))

    def pad(self, input, pad_amount, pad_value):
        flat = [x for pair in pad_amount for x in pair]
        p, _ = _sizes(flat)
        return self._out(lib.knhip_graph_pad, input, p, len(pad_amount), pad_value)

    def conv(self, input, filter, stride_y, stride_x, padding_y, padding_x):
        return self._out(lib.knhip_graph_conv, input, filter, stride_y, stride_x, padding_y, padding_x)

    def linear(self, input, weight):
        return self._out(lib.knhip_graph_linear, input, weight)

    def mat_mul(self, left, right):
        return self._out(lib.knhip_graph_mat_mul, left, right)

    def batched_mat_mul(self, left, right):
        return self._out(lib.knhip_graph_batched_mat_mul, left, right)

    def softmax(self, input, axis):
        return self._out(lib.knhip_graph_softmax, input, axis)

    def layernorm(self, input, axis, eps):
        return self._out(lib.knhip_graph_layernorm, input, axis, c_float(eps))

    def reduce(self, input, axes, op):
        a, n = _sizes(list(axes))
        return self._out(lib.knhip_graph_reduce, input, a, n, int(op))

    def sigmoid(self, input):
        return self.unary(UnaryOp.SIGMOID, input)

    def relu(self, input):
        return self._out(lib.knhip_graph_relu, input)

    def clamp(self, input, min, max):
        dt = self[input].dtype.numpy
        lo = np.asarray(min, dtype=dt)
        hi = np.asarray(max, dtype=dt)
        return self._out(lib.knhip_graph_clamp, input, lo.ctypes.data_as(c_void_p), hi.ctypes.data_as(c_void_p))

    def unary(self, op, input, cast_to=None):
        return self._out(lib.knhip_graph_unary, int(op), -1 if cast_to is None else int(cast_to), input)

    def value_cast(self, input, dtype):
        return self.unary(UnaryOp.VALUE_CAST, input, dtype)

    def bit_cast(self, input, dtype):
        return self.unary(UnaryOp.BIT_CAST, input, dtype)

    def binary(self, op, left, right):
        return self._out(lib.knhip_graph_binary, int(op), left, right)

    def add(self, left, right):
        return self.binary(BinaryOp.ADD, left, right)

    def sub(self, left, right):
        return self.binary(BinaryOp.SUB, left, right)

    def mul(self, left, right):
        return self.binary(BinaryOp.MUL, left, right)

    def pow(self, left, right):
        return self.binary(BinaryOp.POW, left, right)

    def call(self, graph, inputs):
        arr = (c_uint32 * max(len(inputs), 1))(*inputs)
        cap = len(graph.outputs())
        out = (c_uint32 * max(cap, 1))()
        n = c_size_t()
        check(lib.knhip_graph_call(self._h, graph._h, arr, len(inputs), out, cap, byref(n)))
        return [Value(out[i]) for i in range(n.value)]

    def output(self, value):
        check(lib.knhip_graph_output(self._h, value))

    def output_all(self, values):
        for v in values:
            self.output(v)

    def set_debug_id(self, value, id):
        check(lib.knhip_graph_set_debug_id(self._h, value, id.encode()))

    def dummy_zero_inputs(self, batch_size):
        """graph.rs:1416-1427"""
        return [np.zeros([d.eval(batch_size) for d in self[v].shape], self[v].dtype.numpy) for v in self.inputs()]


def optimize_graph(graph, settings=None):
    """kn-graph/src/optimizer/mod.rs:25-46"""
    settings = settings or OptimizerSettings()
    s = OptimizerSettingsT(int(settings.optimize), int(settings.force_bias_through_conv), int(settings.fuse_layernorm),
                           int(settings.div_to_mul))
    h = c_void_p()
    check(lib.knhip_graph_optimize(graph._h, byref(s), byref(h)))
    return Graph(h)
