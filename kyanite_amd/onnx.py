"""ONNX ingestion: builds a `Graph` from the bytes of an .onnx file, the way kn-graph/src/onnx/load.rs does.

The protobuf wire format is read directly (no onnx / protobuf package needed); only the messages and fields the
loader uses are decoded. Values that hold shapes with the symbolic batch size in them are carried as tensors of
`SignedSize` instead of graph values, like `OnnxValue::Size` (kn-graph/src/onnx/typed_value.rs:14-18), so that the
`Shape -> Gather -> Unsqueeze -> Concat -> Reshape` idiom of exported models resolves at load time.

Also here: `load_check_data`, the reader of the reference's `.bin` check files (kn-cuda-eval/src/tester.rs:305-345).
"""
import struct

import numpy as np

from .graph import BinaryOp, DType, Graph, ReduceOp, Size, UnaryOp


class OnnxError(Exception):
    pass


# ------------------------------------------------------------------------------------------------ protobuf wire format

def _varint(buf, pos):
    result = shift = 0
    while True:
        b = buf[pos]
        pos += 1
        result |= (b & 0x7F) << shift
        shift += 7
        if not b & 0x80:
            return result, pos


def _signed(v):
    return v - (1 << 64) if v >= (1 << 63) else v


def _fields(buf):
    """Yields (field number, wire type, value) of one message; length-delimited values come as memoryview slices."""
    buf = memoryview(buf)
    pos, end = 0, len(buf)
    while pos < end:
        key, pos = _varint(buf, pos)
        field, wire = key >> 3, key & 7
        if wire == 0:
            value, pos = _varint(buf, pos)
        elif wire == 1:
            value, pos = bytes(buf[pos:pos + 8]), pos + 8
        elif wire == 2:
            n, pos = _varint(buf, pos)
            value, pos = buf[pos:pos + n], pos + n
        elif wire == 5:
            value, pos = bytes(buf[pos:pos + 4]), pos + 4
        else:
            raise OnnxError(f"unsupported protobuf wire type {wire}")
        yield field, wire, value


def _repeated_ints(items):
    """A repeated int64 field, packed or not, from its (wire, value) occurrences."""
    out = []
    for wire, value in items:
        if wire == 0:
            out.append(_signed(value))
        else:
            pos = 0
            while pos < len(value):
                v, pos = _varint(value, pos)
                out.append(_signed(v))
    return out


def _repeated_fixed(items, fmt, size):
    out = []
    for wire, value in items:
        raw = bytes(value)
        out.extend(struct.unpack("<" + fmt * (len(raw) // size), raw))
    return out


class _Msg:
    """Fields of one message grouped by number."""

    def __init__(self, buf):
        self.f = {}
        for field, wire, value in _fields(buf):
            self.f.setdefault(field, []).append((wire, value))

    def all(self, field):
        return [v for _, v in self.f.get(field, [])]

    def one(self, field, default=None):
        items = self.f.get(field)
        return items[-1][1] if items else default

    def string(self, field, default=""):
        v = self.one(field)
        return bytes(v).decode() if v is not None else default

    def strings(self, field):
        return [bytes(v).decode() for v in self.all(field)]

    def ints(self, field):
        return _repeated_ints(self.f.get(field, []))


# onnx.proto TensorProto.DataType -> DType (load.rs:1355-1381)
_DTYPES = {1: DType.F32, 11: DType.F64, 2: DType.U8, 3: DType.I8, 4: DType.U16, 5: DType.I16, 6: DType.I32,
           7: DType.I64, 12: DType.U32, 13: DType.U64, 9: DType.BOOL}


def _resolve_dtype(code, where):
    if code not in _DTYPES:
        raise OnnxError(f"unsupported ONNX data type {code} at {where}")
    return _DTYPES[code]


def _tensor_to_numpy(buf, where):
    """TensorProto -> numpy array (load.rs:1226-1324); typed fields win over raw_data, like the reference."""
    t = _Msg(buf)
    dims = t.ints(1)
    dtype = _resolve_dtype(t.one(2, 0), where)
    if t.one(14, 0) != 0:
        raise OnnxError(f"external tensor data is not supported ({where})")
    raw = bytes(t.one(9, b""))
    np_dt = dtype.numpy
    count = int(np.prod(dims)) if dims else 1
    typed = None
    if dtype == DType.F32 and 4 in t.f:
        typed = _repeated_fixed(t.f[4], "f", 4)
    elif dtype == DType.F64 and 10 in t.f:
        typed = _repeated_fixed(t.f[10], "d", 8)
    elif dtype in (DType.I8, DType.I16, DType.I32, DType.U8, DType.U16, DType.BOOL) and 5 in t.f:
        typed = t.ints(5)
    elif dtype == DType.I64 and 7 in t.f:
        typed = t.ints(7)
    elif dtype in (DType.U32, DType.U64) and 11 in t.f:
        typed = [v & 0xFFFFFFFFFFFFFFFF for v in t.ints(11)]
    if typed is not None:
        if dtype == DType.BOOL:
            arr = np.asarray([v != 0 for v in typed], np.bool_)
        else:
            arr = np.asarray(typed).astype(np_dt)
    elif dtype == DType.BOOL:
        arr = np.frombuffer(raw, np.uint8) != 0
    else:
        arr = np.frombuffer(raw, np_dt.newbyteorder("<")).astype(np_dt)
    if arr.size != count:
        raise OnnxError(f"tensor {where}: {arr.size} elements for shape {dims}")
    return arr.reshape(dims), dtype


# ------------------------------------------------------------------------------------------------ shape-valued tensors

class SignedSize:
    """`fixed_factor * batch ** batch_exp` with a sign (typed_value.rs:20-24)."""

    __slots__ = ("batch_exp", "fixed_factor")

    def __init__(self, batch_exp, fixed_factor):
        self.batch_exp = 0 if fixed_factor == 0 else int(batch_exp)
        self.fixed_factor = int(fixed_factor)

    @staticmethod
    def from_size(size):
        return SignedSize(size.batch_exp, size.fixed_factor)

    def to_size(self):
        if self.fixed_factor < 0:
            raise OnnxError(f"negative size {self}")
        return Size(self.batch_exp, self.fixed_factor)

    def fixed(self):
        return self.fixed_factor if self.batch_exp == 0 else None

    def __eq__(self, other):
        return isinstance(other, SignedSize) and (self.batch_exp, self.fixed_factor) == (other.batch_exp, other.fixed_factor)

    def __hash__(self):
        return hash((self.batch_exp, self.fixed_factor))

    def __neg__(self):
        return SignedSize(self.batch_exp, -self.fixed_factor)

    def __repr__(self):
        if self.batch_exp == 0:
            return str(self.fixed_factor)
        return f"{self.fixed_factor}B^{self.batch_exp}"

    # typed_value.rs:203-256 and load.rs:1477-1486; None = not representable
    def add(self, other):
        if self.fixed_factor == 0:
            return other
        if other.fixed_factor == 0:
            return self
        if self.batch_exp == other.batch_exp:
            return SignedSize(self.batch_exp, self.fixed_factor + other.fixed_factor)
        return None

    def sub(self, other):
        return self.add(-other)

    def mul(self, other):
        return SignedSize(self.batch_exp + other.batch_exp, self.fixed_factor * other.fixed_factor)

    def floor_div(self, other):
        if self.batch_exp < other.batch_exp:
            return None
        # Rust's `/` on i64 truncates toward zero
        q = abs(self.fixed_factor) // abs(other.fixed_factor)
        if (self.fixed_factor < 0) != (other.fixed_factor < 0):
            q = -q
        return SignedSize(self.batch_exp - other.batch_exp, q)


def _size_array(items, shape):
    arr = np.empty(len(items), dtype=object)
    for i, x in enumerate(items):
        arr[i] = x
    return arr.reshape(shape)


class _Val:
    """OnnxValue (typed_value.rs:14-18): a graph value, or a tensor of SignedSize when the batch size is involved."""

    def __init__(self, value=None, size=None):
        self.value, self.size = value, size

    @staticmethod
    def new_size(arr, graph):
        if any(x.batch_exp != 0 for x in arr.flat):
            return _Val(size=arr)
        ints = np.asarray([x.fixed_factor for x in arr.flat], np.int64).reshape(arr.shape)
        return _Val(value=graph.constant(list(arr.shape), ints))

    def unwrap_value(self, what):
        if self.value is None:
            raise OnnxError(f"{what}: expected a tensor value, got a shape that involves the batch size")
        return self.value

    def as_size(self, graph):
        if self.size is not None:
            return self.size
        const = graph.as_const(self.value)
        if const is None:
            raise OnnxError("shape operand is not constant")
        if const.dtype != np.int64:
            raise OnnxError(f"shape operand must be i64, got {const.dtype}")
        return _size_array([SignedSize(0, int(v)) for v in const.flat], const.shape)

    def as_signed_shape(self, graph):
        arr = self.as_size(graph)
        if arr.ndim != 1:
            raise OnnxError(f"shape operand must have rank 1, got shape {arr.shape}")
        return list(arr)

    def as_shape(self, graph):
        return [s.to_size() for s in self.as_signed_shape(graph)]

    def shape(self, graph):
        if self.value is not None:
            return list(graph[self.value].shape)
        return [Size.fixed(d) for d in self.size.shape]


def _abs_axis(axis, rank):
    # load.rs:1383-1391
    if axis == (1 << 63) - 1:
        return rank
    if axis < 0:
        if -axis > rank:
            raise OnnxError(f"axis {axis} out of range for rank {rank}")
        return rank - (-axis)
    return axis


def _fixed_dims(shape, what):
    out = []
    for d in shape:
        if d.batch_exp != 0:
            raise OnnxError(f"{what} must be fixed, got {shape}")
        out.append(d.fixed_factor)
    return out


def _size_product(dims):
    total = Size.ONE
    for d in dims:
        total = total * d
    return total


def _size_div(a, b):
    """Exact division of sizes (shape.rs Div): None when impossible."""
    if b.fixed_factor == 0 or a.batch_exp < b.batch_exp or a.fixed_factor % b.fixed_factor != 0:
        return None
    return Size(a.batch_exp - b.batch_exp, a.fixed_factor // b.fixed_factor)


def _reshape_output_shape(old_shape, new_shape_raw, allow_zero):
    # load.rs:1419-1475
    old_size = _size_product(old_shape)
    new_shape, leftover_index, leftover = [], None, old_size
    for i, s in enumerate(new_shape_raw):
        if s == SignedSize(0, 0):
            if allow_zero:
                size = Size.ZERO
            else:
                if i >= len(old_shape):
                    raise OnnxError(f"Reshape: cannot copy dim {i}, not present in input {old_shape}")
                size = old_shape[i]
        elif s == SignedSize(0, -1):
            if leftover_index is not None:
                raise OnnxError("Reshape shape can only contain a single -1 value")
            leftover_index = i
            new_shape.append(Size.ZERO)
            continue
        else:
            size = s.to_size()
        leftover = _size_div(leftover, size)
        if leftover is None:
            raise OnnxError(f"cannot reshape {old_shape} into {new_shape_raw}")
        new_shape.append(size)
    if leftover_index is not None:
        new_shape[leftover_index] = leftover
    if not _size_product(new_shape) == old_size:
        raise OnnxError(f"Reshape: output {new_shape} and input {old_shape} sizes differ")
    return new_shape


class _Attrs:
    """Attributes of one node; every attribute has to be consumed (load.rs:96-99)."""

    def __init__(self, node_name, bufs):
        self.node = node_name
        self.left = {}
        for buf in bufs:
            m = _Msg(buf)
            self.left[m.string(1)] = m

    def _take(self, name):
        return self.left.pop(name, None)

    def _need(self, name):
        m = self._take(name)
        if m is None:
            raise OnnxError(f"node {self.node}: missing attribute {name}")
        return m

    def maybe_int(self, name):
        m = self._take(name)
        return None if m is None else _signed(m.one(3, 0))

    def int(self, name):
        return _signed(self._need(name).one(3, 0))

    def maybe_ints(self, name):
        m = self._take(name)
        return None if m is None else m.ints(8)

    def ints(self, name):
        return self._need(name).ints(8)

    def maybe_float(self, name):
        m = self._take(name)
        return None if m is None else struct.unpack("<f", m.one(2, b"\0\0\0\0"))[0]

    def float(self, name):
        v = self.maybe_float(name)
        if v is None:
            raise OnnxError(f"node {self.node}: missing attribute {name}")
        return v

    def maybe_string(self, name):
        m = self._take(name)
        return None if m is None else m.string(4)

    def maybe_tensor(self, name):
        m = self._take(name)
        return None if m is None else m.one(5)

    def tensor(self, name):
        return self._need(name).one(5)


class _Inputs:
    """Inputs of one node; an empty name is a missing optional input, all present inputs have to be consumed."""

    def __init__(self, node_name, names, store):
        self.node = node_name
        self.vals = []
        for n in names:
            if n == "":
                self.vals.append(None)
            elif n in store:
                self.vals.append(store[n])
            else:
                raise OnnxError(f"node {node_name}: input {n} is not defined")
        self.used = [False] * len(self.vals)

    def optional(self, i):
        if i < len(self.vals) and self.vals[i] is not None:
            self.used[i] = True
            return self.vals[i]
        return None

    def required(self, i):
        v = self.optional(i)
        if v is None:
            raise OnnxError(f"node {self.node}: missing input {i}")
        return v

    def take_all(self):
        if any(v is None for v in self.vals):
            raise OnnxError(f"node {self.node}: variadic inputs cannot be missing")
        self.used = [True] * len(self.vals)
        return list(self.vals)

    def leftover(self):
        return [i for i, (v, u) in enumerate(zip(self.vals, self.used)) if v is not None and not u]


_UNARY = {"Abs": UnaryOp.ABS, "Neg": UnaryOp.NEG, "Sin": UnaryOp.SIN, "Cos": UnaryOp.COS, "Exp": UnaryOp.EXP,
          "Log": UnaryOp.LOG, "Sqrt": UnaryOp.SQRT, "Sigmoid": UnaryOp.SIGMOID, "Tanh": UnaryOp.TANH, "Erf": UnaryOp.ERF,
          "Softplus": UnaryOp.SOFTPLUS}
_BINARY = {"Add": BinaryOp.ADD, "Sub": BinaryOp.SUB, "Mul": BinaryOp.MUL, "Div": BinaryOp.DIV, "Min": BinaryOp.MIN,
           "Max": BinaryOp.MAX, "Pow": BinaryOp.POW}
_REDUCE = {"ReduceSum": ReduceOp.SUM, "ReduceMean": ReduceOp.MEAN, "ReduceProd": ReduceOp.PROD, "ReduceMin": ReduceOp.MIN,
           "ReduceMax": ReduceOp.MAX}


def _broadcast_size_arrays(a, b):
    shape = np.broadcast_shapes(a.shape, b.shape)
    return np.broadcast_to(a, shape), np.broadcast_to(b, shape)


def _visit_node(g, op, name, ins, at):
    """One ONNX node -> graph operations (load.rs:122-1214). Returns the list of output values."""
    if op == "Conv":
        x = ins.required(0).unwrap_value(name)
        w = ins.required(1).unwrap_value(name)
        bias_raw = ins.optional(2)
        groups = at.maybe_int("group")
        kernel_shape = at.ints("kernel_shape")
        rank = len(kernel_shape)
        strides = at.maybe_ints("strides") or [1] * rank
        dilations = at.maybe_ints("dilations") or [1] * rank
        auto_pad = at.maybe_string("auto_pad")
        if auto_pad not in (None, "NOTSET"):
            raise OnnxError(f"node {name}: auto_pad {auto_pad} is not supported by this loader")
        pads = at.ints("pads")
        fshape = _fixed_dims(g[w].shape, "convolution kernel shape")
        if groups not in (None, 1) or rank not in (1, 2):
            raise OnnxError(f"node {name}: only ungrouped 1D and 2D convolutions are supported")
        bias = None
        if bias_raw is not None:
            b = bias_raw.unwrap_value(name)
            (n,) = g[b].shape
            bias = g.view(b, [1, n, 1, 1])  # in the conv's 4D domain so the planner can fuse it
        if rank == 1:
            # a 1D convolution is a 2D one over a trailing axis of size 1 (load.rs:180-202)
            if pads[0] != pads[1] or dilations != [1] or strides != [1] or fshape[2:] != list(kernel_shape):
                raise OnnxError(f"node {name}: unsupported 1D convolution padding / dilation / stride / kernel")
            y = g.conv(g.view(x, list(g[x].shape) + [Size.ONE]), g.view(w, list(g[w].shape) + [Size.ONE]), 1, 1, pads[0], 0)
            if bias is not None:
                y = g.add(y, bias)
            return [_Val(g.view(y, list(g[y].shape)[:3]))]
        if not (pads[0] == pads[2] and pads[1] == pads[3]) or dilations != [1, 1] or fshape[2:] != list(kernel_shape):
            raise OnnxError(f"node {name}: unsupported convolution padding / dilation / kernel")
        y = g.conv(x, w, strides[0], strides[1], pads[0], pads[1])
        if bias is not None:
            y = g.add(y, bias)
        return [_Val(y)]
    if op == "Clip":
        x = ins.required(0).unwrap_value(name)
        lo, hi = ins.optional(1), ins.optional(2)
        if lo is None and hi is None:
            lo_f, hi_f = at.float("min"), at.float("max")
            return [_Val(g.clamp(x, lo_f, hi_f))]
        if lo is None or hi is None:
            raise OnnxError(f"node {name}: Clip must have either 1 or 3 inputs")
        mid = g.binary(BinaryOp.MIN, x, hi.unwrap_value(name))
        return [_Val(g.binary(BinaryOp.MAX, mid, lo.unwrap_value(name)))]
    if op == "Relu":
        return [_Val(g.relu(ins.required(0).unwrap_value(name)))]
    if op in _UNARY:
        return [_Val(g.unary(_UNARY[op], ins.required(0).unwrap_value(name)))]
    if op in _BINARY:
        left, right = ins.required(0), ins.required(1)
        if left.value is not None and right.value is not None:
            return [_Val(g.binary(_BINARY[op], left.value, right.value))]
        a, b = _broadcast_size_arrays(left.as_size(g), right.as_size(g))
        fn = {"Add": SignedSize.add, "Sub": SignedSize.sub, "Mul": SignedSize.mul, "Div": SignedSize.floor_div}.get(op)
        out = []
        for l, r in zip(a.flat, b.flat):
            v = fn(l, r) if fn else None
            if v is None:
                raise OnnxError(f"node {name}: {op} failed between sizes {l} and {r}")
            out.append(v)
        return [_Val.new_size(_size_array(out, a.shape), g)]  # the batch size might have cancelled out
    if op == "Flatten":
        x = ins.required(0)
        shape = x.shape(g)
        rel = at.maybe_int("axis")
        axis = _abs_axis(1 if rel is None else rel, len(shape))
        new_shape = shape[:axis] + [_size_product(shape[axis:])]
        if axis == 0:
            new_shape.insert(0, Size.ONE)
        if x.value is not None:
            return [_Val(g.view(x.value, new_shape))]
        return [_Val.new_size(x.size.reshape(_fixed_dims(new_shape, "size shape")), g)]
    if op == "Gemm":
        x = ins.required(0).unwrap_value(name)
        w = ins.required(1).unwrap_value(name)
        bias = ins.optional(2)
        alpha, beta, trans_b = at.float("alpha"), at.float("beta"), at.int("transB")
        if alpha != 1.0 or beta != 1.0 or trans_b == 0:
            raise OnnxError(f"node {name}: Gemm needs alpha = beta = 1 and transB = 1")
        y = g.linear(x, w)
        if bias is not None:
            b = bias.unwrap_value(name)
            (n,) = g[b].shape
            y = g.add(y, g.view(b, [1, n]))
        return [_Val(y)]
    if op == "MatMul":
        return [_Val(g.mat_mul(ins.required(0).unwrap_value(name), ins.required(1).unwrap_value(name)))]
    if op == "BatchNormalization":
        x = ins.required(0).unwrap_value(name)
        scale, bias, mean, var = (ins.required(i).unwrap_value(name) for i in (1, 2, 3, 4))
        eps = at.float("epsilon")
        at.float("momentum")
        spatial = at.maybe_int("spatial")
        if spatial not in (None, 1):
            raise OnnxError(f"node {name}: non-spatial BatchNormalization is not supported")
        shape = list(g[x].shape)
        if len(shape) < 2:
            raise OnnxError(f"node {name}: BatchNormalization input must have at least rank 2")
        exp_shape = [Size.ONE] * len(shape)
        exp_shape[1] = shape[1]
        for p in (scale, bias, mean, var):
            if list(g[p].shape) != [shape[1]]:
                raise OnnxError(f"node {name}: BatchNormalization parameter shape mismatch")
        e_scale, e_bias, e_mean, e_var = (g.view(p, exp_shape) for p in (scale, bias, mean, var))
        div = g.unary(UnaryOp.SQRT, g.add(e_var, g.scalar(eps)))
        y = g.binary(BinaryOp.DIV, g.sub(x, e_mean), div)
        return [_Val(g.add(g.mul(y, e_scale), e_bias))]
    if op in ("InstanceNormalization", "LayerNormalization"):
        x = ins.required(0).unwrap_value(name)
        scale = ins.required(1).unwrap_value(name)
        bias = ins.required(2).unwrap_value(name)
        shape = list(g[x].shape)
        if op == "InstanceNormalization":
            eps = at.float("epsilon")
            bshape = [Size.ONE] * len(shape)
            bshape[1] = shape[1]
            scale, bias, start = g.view(scale, bshape), g.view(bias, bshape), 2
        else:
            axis = at.maybe_int("axis")
            eps = at.maybe_float("epsilon")
            eps = 1e-5 if eps is None else eps
            scale, bias = g.broadcast(scale, shape), g.broadcast(bias, shape)
            start = _abs_axis(-1 if axis is None else axis, len(shape))
        flat = shape[:start] + [_size_product(shape[start:])]
        y = g.view(g.layernorm(g.view(x, flat), start, eps), shape)
        return [_Val(g.add(g.mul(y, scale), bias))]
    if op == "Constant":
        arr, dtype = _tensor_to_numpy(at.tensor("value"), name)
        return [_Val(g.constant(list(arr.shape), arr, dtype))]
    if op == "ConstantOfShape":
        shape_in = ins.optional(0)
        shape = [] if shape_in is None else shape_in.as_shape(g)
        t = at.maybe_tensor("value")
        if t is None:
            value = g.scalar(0.0)
        else:
            arr, dtype = _tensor_to_numpy(t, name)
            if arr.size != 1:
                raise OnnxError(f"node {name}: value must be a one-element tensor")
            value = g.constant([], arr.reshape(()), dtype)
        return [_Val(g.broadcast(value, shape))]
    if op == "Cast":
        x = ins.required(0)
        dtype = _resolve_dtype(at.int("to"), name)
        if x.value is not None:
            return [_Val(g.value_cast(x.value, dtype))]
        if dtype != DType.I64:
            raise OnnxError(f"node {name}: shapes can only be cast to i64")
        return [_Val.new_size(x.size, g)]
    if op == "Reshape":
        x = ins.required(0)
        new_shape = ins.required(1).as_signed_shape(g)
        allow_zero = bool(at.maybe_int("allowzero") or 0)
        out_shape = _reshape_output_shape(x.shape(g), new_shape, allow_zero)
        if x.value is not None:
            return [_Val(g.view(x.value, out_shape))]
        return [_Val.new_size(x.size.reshape(_fixed_dims(out_shape, "reshape shape")), g)]
    if op == "Unsqueeze":
        x = ins.required(0)
        axes_in = ins.optional(1)
        if axes_in is not None:
            rel_axes = [s.fixed() for s in axes_in.as_signed_shape(g)]
        else:
            rel_axes = at.ints("axes")
        in_shape = x.shape(g)
        out_rank = len(in_shape) + len(rel_axes)
        axes = [_abs_axis(a, out_rank) for a in rel_axes]
        if len(set(axes)) != len(axes) or any(a >= out_rank for a in axes):
            raise OnnxError(f"node {name}: invalid Unsqueeze axes {rel_axes}")
        it = iter(in_shape)
        out_shape = [Size.ONE if i in axes else next(it) for i in range(out_rank)]
        if x.value is not None:
            return [_Val(g.view(x.value, out_shape))]
        return [_Val.new_size(x.size.reshape(_fixed_dims(out_shape, "unsqueeze shape")), g)]
    if op == "Transpose":
        x = ins.required(0)
        perm = at.ints("perm")
        if x.value is not None:
            return [_Val(g.permute(x.value, perm))]
        return [_Val.new_size(np.transpose(x.size, perm), g)]
    if op == "Gather":
        x, idx = ins.required(0), ins.required(1)
        rel = at.maybe_int("axis")
        in_shape = x.shape(g)
        axis = _abs_axis(0 if rel is None else rel, len(in_shape))
        axis_size = in_shape[axis]
        if idx.value is not None:
            const = g.as_const(idx.value)
            if const is not None:
                # negative indices count from the end
                if axis_size.batch_exp != 0:
                    raise OnnxError(f"node {name}: gather dim size must be fixed")
                fixed = np.where(const < 0, const + np.asarray(axis_size.fixed_factor).astype(const.dtype), const) \
                    if const.dtype.kind == "i" else const
                idx = _Val(g.constant(list(fixed.shape), fixed.astype(const.dtype)))
        else:
            arr = idx.size
            fixed = [s.add(SignedSize.from_size(axis_size)) if s.fixed_factor < 0 else s for s in arr.flat]
            if any(v is None for v in fixed):
                raise OnnxError(f"node {name}: gather negative index overflow")
            idx = _Val.new_size(_size_array(fixed, arr.shape), g)
        if x.value is not None:
            return [_Val(g.gather(x.value, axis, idx.unwrap_value(name)))]
        indices = g.as_const(idx.unwrap_value(name))
        if indices is None:
            raise OnnxError(f"node {name}: gather on a shape needs constant indices")
        taken = np.take(x.size, indices.astype(np.int64), axis=axis)
        if not isinstance(taken, np.ndarray):  # a rank-0 result comes back as the element itself
            taken = _size_array([taken], ())
        return [_Val.new_size(taken, g)]
    if op == "Slice":
        def get(index, attr):
            v = ins.optional(index)
            if v is not None:
                const = g.as_const(v.unwrap_value(name))
                if const is None or const.ndim != 1 or const.dtype not in (np.int64, np.int32):
                    raise OnnxError(f"node {name}: Slice operand {attr} must be a 1D integer constant")
                return [int(c) for c in const]
            return at.maybe_ints(attr)

        x = ins.required(0)
        starts, ends = get(1, "starts"), get(2, "ends")
        if starts is None or ends is None:
            raise OnnxError(f"node {name}: Slice needs starts and ends")
        n = len(starts)
        axes = get(3, "axes")
        axes = list(range(n)) if axes is None else axes
        steps = get(4, "steps")
        steps = [1] * n if steps is None else steps
        if not (len(ends) == len(axes) == len(steps) == n) or len(set(axes)) != n:
            raise OnnxError(f"node {name}: inconsistent Slice operands")
        in_shape = x.shape(g)
        curr = x
        for i in range(n):
            axis = _abs_axis(axes[i], len(in_shape))
            dim, step = in_shape[axis], steps[i]
            if step == 0:
                raise OnnxError(f"node {name}: Slice step cannot be 0")
            if step > 0:
                if dim.batch_exp != 0 and starts[i] == 0 and ends[i] == (1 << 31) - 1:
                    continue  # the whole batch axis
                if dim.batch_exp != 0:
                    raise OnnxError(f"node {name}: cannot slice the batch axis")
                size = dim.fixed_factor
                start, end = _abs_axis(starts[i], size), _abs_axis(ends[i], size)
                if curr.value is not None:
                    curr = _Val(g.slice(curr.value, axis, start, end, step))
                else:
                    index = [slice(None)] * curr.size.ndim
                    index[axis] = slice(start, end, step)
                    curr = _Val(size=curr.size[tuple(index)])
            else:
                if not (starts[i] == -1 and ends[i] == -(1 << 63) and step == -1):
                    raise OnnxError(f"node {name}: only the plain flip is supported as a negative Slice step")
                if curr.value is not None:
                    curr = _Val(g.flip(curr.value, axis))
                else:
                    curr = _Val(size=np.flip(curr.size, axis))
        if curr.size is not None:
            curr = _Val.new_size(curr.size, g)
        return [curr]
    if op == "Concat":
        items = ins.take_all()
        if not items:
            raise OnnxError(f"node {name}: must concatenate at least one value")
        axis = _abs_axis(at.int("axis"), len(items[0].shape(g)))
        if any(v.size is not None for v in items):
            arr = np.concatenate([v.as_size(g) for v in items], axis=axis)
            return [_Val.new_size(arr, g)]
        return [_Val(g.concat([v.value for v in items], axis))]
    if op == "Shape":
        dims = [SignedSize.from_size(d) for d in ins.required(0).shape(g)]
        return [_Val.new_size(_size_array(dims, (len(dims),)), g)]
    if op == "Identity":
        return [ins.required(0)]
    if op == "Softmax":
        x = ins.required(0).unwrap_value(name)
        rel = at.maybe_int("axis")
        return [_Val(g.softmax(x, _abs_axis(-1 if rel is None else rel, len(g[x].shape))))]
    if op in _REDUCE:
        x = ins.required(0).unwrap_value(name)
        shape = list(g[x].shape)
        rel_axes = at.maybe_ints("axes")
        axes = list(range(len(shape))) if rel_axes is None else [_abs_axis(a, len(shape)) for a in rel_axes]
        keep = at.maybe_int("keepdims")
        keep = True if keep is None else keep != 0
        out_shape = [Size.ONE if i in axes else d for i, d in enumerate(shape)] if keep else \
            [d for i, d in enumerate(shape) if i not in axes]
        return [_Val(g.view(g.reduce(x, axes, _REDUCE[op]), out_shape))]
    if op in ("GlobalMaxPool", "GlobalAveragePool"):
        x = ins.required(0).unwrap_value(name)
        rank = len(g[x].shape)
        if rank < 2:
            raise OnnxError(f"node {name}: pooling needs rank >= 2")
        return [_Val(g.reduce(x, list(range(2, rank)), ReduceOp.MAX if op == "GlobalMaxPool" else ReduceOp.MEAN))]
    if op == "Expand":
        x = ins.required(0)
        shape = ins.required(1).as_shape(g)
        in_shape = x.shape(g)
        rank = max(len(in_shape), len(shape))
        a = [Size.ONE] * (rank - len(in_shape)) + in_shape
        b = [Size.ONE] * (rank - len(shape)) + shape
        out = []
        for l, r in zip(a, b):
            if l == r or r == Size.ONE:
                out.append(l)
            elif l == Size.ONE:
                out.append(r)
            else:
                raise OnnxError(f"node {name}: cannot broadcast {in_shape} with {shape}")
        if x.value is not None:
            return [_Val(g.broadcast(x.value, out))]
        return [_Val.new_size(np.broadcast_to(x.size, _fixed_dims(out, "expand shape")), g)]
    raise OnnxError(f"unsupported ONNX operation {op} (node {name})")


def load_graph_from_onnx_bytes(buf, named_axes=None):
    """`load_graph_from_onnx_bytes` (kn-graph/src/onnx/mod.rs:38-42): the dimension parameter `batch_size` becomes
    the symbolic batch size; other named axes can be given as {name: Size}."""
    named = {"batch_size": Size.BATCH}
    named.update(named_axes or {})
    model = _Msg(buf)
    graph_buf = model.one(7)
    if graph_buf is None:
        raise OnnxError("model has no graph")
    mg = _Msg(graph_buf)
    g = Graph()
    store = {}

    for t in mg.all(5):  # initializers
        tname = _Msg(t).string(8)
        arr, dtype = _tensor_to_numpy(t, tname)
        store[tname] = _Val(g.constant(list(arr.shape), arr, dtype))

    for vi_buf in mg.all(11):  # inputs; initializers may re-appear here
        vi = _Msg(vi_buf)
        iname = vi.string(1)
        if iname in store:
            continue
        tp = vi.one(2)
        tensor_type = _Msg(tp).one(1) if tp is not None else None
        if tensor_type is None:
            raise OnnxError(f"input {iname} is not a tensor")
        tt = _Msg(tensor_type)
        dtype = _resolve_dtype(tt.one(1, 0), iname)
        shape_buf = tt.one(2)
        if shape_buf is None:
            raise OnnxError(f"input {iname} has no shape")
        dims = []
        for d_buf in _Msg(shape_buf).all(1):
            d = _Msg(d_buf)
            if 1 in d.f:
                dims.append(Size.fixed(_signed(d.one(1))))
            elif 2 in d.f:
                param = d.string(2)
                if param not in named:
                    raise OnnxError(f"input {iname}: no size given for the named axis {param}")
                dims.append(named[param])
            else:
                raise OnnxError(f"input {iname}: dimension without a value")
        store[iname] = _Val(g.input(dims, dtype))

    for n_buf in mg.all(1):
        node = _Msg(n_buf)
        op, name = node.string(4), node.string(3)
        attrs = _Attrs(name, node.all(5))
        inputs = _Inputs(name, node.strings(1), store)
        first_new = len(g)
        values = _visit_node(g, op, name or op, inputs, attrs)
        for v in range(first_new, len(g)):
            g.set_debug_id(v, name)
        if attrs.left:
            raise OnnxError(f"node {name} ({op}): leftover attributes {sorted(attrs.left)}")
        if inputs.leftover():
            raise OnnxError(f"node {name} ({op}): leftover inputs {inputs.leftover()}")
        out_names = node.strings(2)
        if len(out_names) != len(values):
            raise OnnxError(f"node {name} ({op}): expected {len(out_names)} outputs, got {len(values)}")
        for out_name, v in zip(out_names, values):
            store[out_name] = v

    for vi_buf in mg.all(12):
        oname = _Msg(vi_buf).string(1)
        if oname not in store:
            raise OnnxError(f"output {oname} is not defined")
        g.output(store[oname].unwrap_value(f"output {oname}"))
    return g


def load_graph_from_onnx_path(path):
    with open(path, "rb") as f:
        return load_graph_from_onnx_bytes(f.read())


def load_check_data(graph, data):
    """kn-cuda-eval/src/tester.rs:305-345: one byte batch size, then little-endian f32 values of every input followed
    by every expected output, in graph order. Returns (batch_size, inputs, expected_outputs)."""
    if len(data) == 0:
        raise ValueError("check data must have at least one byte, the batch size")
    batch = data[0]
    if (len(data) - 1) % 4 != 0:
        raise ValueError(f"data byte count must be a multiple of 4 plus 1, got {len(data)}")
    values = np.frombuffer(data, dtype="<f4", offset=1)
    pos = 0

    def take(value_ids):
        nonlocal pos
        out = []
        for v in value_ids:
            dims = [d.eval(batch) for d in graph[v].shape]
            n = int(np.prod(dims)) if dims else 1
            out.append(values[pos:pos + n].astype(np.float32).reshape(dims))
            pos += n
        return out

    inputs = take(graph.inputs())
    expected = take(graph.outputs())
    if pos != len(values):
        raise ValueError(f"leftover elements in check data buffer: {len(values) - pos}")
    return batch, inputs, expected
