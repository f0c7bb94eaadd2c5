"""ORACLE - test infrastructure only (tests, the smoke check and the benchmark's parity leg).

A third, independent evaluation of a graph: numpy, every floating-point value held in f64.

It answers one question in the GPU parity tests: of two f32 (or f16) results that differ, which is nearer the
exact value? The CPU oracle folds every contraction sequentially in f32, the GPU kernels sum in blocks and trees;
both are rounding-noise away from the exact result, and this evaluator gives that exact result to within f64
rounding. Semantics follow kn-graph/src/cpu.rs:99-277 and graph.rs:1649-1815 (NaN-ignoring min / max, biased
variance with eps inside the root, the Abramowitz-Stegun erf), written with whole-array numpy routines so that it
shares neither code nor summation order with the oracle's C++ loops.

Floats of any width are f64 here and float -> float casts are the identity. Integer and bool tensors keep their
dtype and their wrapping arithmetic. Graphs whose result depends on the exact f32 / f16 bit pattern (bit casts of
floats, float -> integer casts, gathers through computed indices) are refused with `Unsupported`.
"""
import enum

import numpy as np


# The codes of the serialised graph (include/knhip.h), restated so that this file imports nothing from the product;
# a graph is anything that offers values(), inputs(), outputs(), graph[value] and constant_data(value).
class DType(enum.IntEnum):
    F32, F64, I8, I16, I32, I64, U8, U16, U32, U64, BOOL, F16 = range(12)


class OpKind(enum.IntEnum):
    (INPUT, CONSTANT, VIEW, BROADCAST, PERMUTE, SLICE, FLIP, GATHER, CONCAT, CONV, MATMUL, UNARY, BINARY, SOFTMAX,
     LAYERNORM, REDUCE) = range(16)


class UnaryOp(enum.IntEnum):
    ABS, NEG, SIN, COS, EXP, LOG, SQRT, SIGMOID, TANH, ERF, MISH, SOFTPLUS, VALUE_CAST, BIT_CAST = range(14)


class BinaryOp(enum.IntEnum):
    ADD, SUB, MUL, DIV, MIN, MAX, POW = range(7)


class ReduceOp(enum.IntEnum):
    SUM, MEAN, PROD, MAX, MIN = range(5)


_NUMPY = [np.float32, np.float64, np.int8, np.int16, np.int32, np.int64, np.uint8, np.uint16, np.uint32, np.uint64,
          np.bool_, np.float16]


class Unsupported(Exception):
    pass


def _is_float(dtype):
    return dtype in (DType.F32, DType.F64, DType.F16)


def _erf_as(x):
    coef = [1.0, 0.0705230784, 0.0422820123, 0.0092705272, 0.0001520143, 0.0002765672, 0.0000430638]
    xa = np.abs(x)
    d = sum(c * xa ** i for i, c in enumerate(coef))
    sign = np.where(np.signbit(x), -1.0, 1.0)
    return np.where(np.isnan(x), x, sign * (1.0 - 1.0 / d ** 16))


def _unary(op, x):
    with np.errstate(all="ignore"):
        if op == UnaryOp.ABS:
            return np.abs(x)
        if op == UnaryOp.NEG:
            return -x
        if op == UnaryOp.SIN:
            return np.sin(x)
        if op == UnaryOp.COS:
            return np.cos(x)
        if op == UnaryOp.EXP:
            return np.exp(x)
        if op == UnaryOp.LOG:
            return np.log(x)
        if op == UnaryOp.SQRT:
            return np.sqrt(x)
        if op == UnaryOp.SIGMOID:
            return 1.0 / (1.0 + np.exp(-x))
        if op == UnaryOp.TANH:
            return np.tanh(x)
        if op == UnaryOp.ERF:
            return _erf_as(x)
        if op == UnaryOp.MISH:
            return x * np.tanh(np.log1p(np.exp(x)))
        if op == UnaryOp.SOFTPLUS:
            return np.log1p(np.exp(-np.abs(x))) + np.where(np.isnan(x), 0.0, np.maximum(x, 0.0))
    raise Unsupported(f"unary {op}")


def _binary(op, l, r, is_float):
    with np.errstate(all="ignore"):
        if op == BinaryOp.ADD:
            return l + r if l.dtype != np.bool_ else l | r
        if op == BinaryOp.SUB:
            return l - r if l.dtype != np.bool_ else l & ~r
        if op == BinaryOp.MUL:
            return l * r if l.dtype != np.bool_ else l & r
        if op == BinaryOp.DIV:
            if is_float:
                return l / r
            if l.dtype == np.bool_:
                return l & ~r
            # Rust integer division truncates towards zero, numpy's floors
            q = np.abs(l.astype(object)) // np.abs(r.astype(object))
            q = np.where((l < 0) != (r < 0), -q, q)
            info = np.iinfo(l.dtype)
            span = int(info.max) - int(info.min) + 1
            wrapped = [((int(v) - int(info.min)) % span) + int(info.min) for v in q.reshape(-1)]
            return np.asarray(wrapped, dtype=l.dtype).reshape(l.shape)
        if op == BinaryOp.MIN:
            return np.fmin(l, r) if is_float else np.minimum(l, r)
        if op == BinaryOp.MAX:
            return np.fmax(l, r) if is_float else np.maximum(l, r)
        if op == BinaryOp.POW:
            return np.power(l, r)
    raise Unsupported(f"binary {op}")


def _conv(x, w, stride, padding):
    """Direct convolution as one einsum per filter tap (NCHW input, [out, in, kh, kw] filter)."""
    sy, sx = stride
    py, px = padding
    n, c, h, wd = x.shape
    oc, _, kh, kw = w.shape
    oh = (h + 2 * py - kh) // sy + 1
    ow = (wd + 2 * px - kw) // sx + 1
    padded = np.zeros((n, c, h + 2 * py, wd + 2 * px), dtype=np.float64)
    padded[:, :, py:py + h, px:px + wd] = x
    out = np.zeros((n, oc, oh, ow), dtype=np.float64)
    for fy in range(kh):
        for fx in range(kw):
            window = padded[:, :, fy:fy + (oh - 1) * sy + 1:sy, fx:fx + (ow - 1) * sx + 1:sx]
            out += np.einsum("nchw,oc->nohw", window, w[:, :, fy, fx], optimize=True)
    return out


def eval_graph_f64(graph, batch_size, inputs, storage_rounding=False):
    """Outputs of `graph` as numpy arrays: f64 for every floating-point output, the value's own dtype otherwise.
    With `storage_rounding` every float value is rounded to its own dtype (f16 / f32) after the operation that
    produces it, still held in f64: the semantics of the oracle with exact arithmetic inside each operation,
    which is the sharper comparison when only the MEANING of the operations is in question."""
    values = {}
    input_index = {int(v): i for i, v in enumerate(graph.inputs())}
    # intermediate values are dropped after their last use (full-size graphs hold gigabytes in f64)
    all_values = list(graph.values())
    infos = {int(v): graph[v] for v in all_values}
    last_use = {}
    for v in all_values:
        for o in infos[int(v)].operands:
            last_use[int(o)] = int(v)
    keep = {int(o) for o in graph.outputs()}
    for v in all_values:
        info = infos[int(v)]
        shape = [d.eval(batch_size) for d in info.shape]
        is_float = _is_float(info.dtype)
        ops = [values[int(o)] for o in info.operands]
        kind = info.op
        if kind == OpKind.INPUT:
            arr = np.asarray(inputs[input_index[int(v)]]).reshape(shape)
            out = arr.astype(np.float64) if is_float else arr
        elif kind == OpKind.CONSTANT:
            arr = graph.constant_data(v).reshape(shape)
            out = arr.astype(np.float64) if is_float else arr
        elif kind == OpKind.VIEW:
            out = ops[0].reshape(shape)
        elif kind == OpKind.BROADCAST:
            out = np.broadcast_to(ops[0], shape)
        elif kind == OpKind.PERMUTE:
            out = np.transpose(ops[0], info.axes)
        elif kind == OpKind.SLICE:
            start, end, step = info.slice
            index = [slice(None)] * ops[0].ndim
            index[info.axes[0]] = slice(start, end, step)
            out = ops[0][tuple(index)]
        elif kind == OpKind.FLIP:
            out = np.flip(ops[0], info.axes[0])
        elif kind == OpKind.GATHER:
            src = infos[int(info.operands[1])]
            if src.op not in (OpKind.INPUT, OpKind.CONSTANT):
                raise Unsupported("gather through computed indices")
            out = np.take(ops[0], ops[1].astype(np.int64), axis=info.axes[0])
        elif kind == OpKind.CONCAT:
            out = np.concatenate(ops, axis=info.axes[0]) if ops else np.zeros(shape, np.float64 if is_float else _NUMPY[int(info.dtype)])
        elif kind == OpKind.CONV:
            sy, sx, py, px = info.axes
            out = _conv(ops[0], ops[1], (sy, sx), (py, px))
        elif kind == OpKind.MATMUL:
            if not is_float:
                raise Unsupported("integer matmul")
            out = np.matmul(ops[0], ops[1])
        elif kind == OpKind.UNARY:
            op = UnaryOp(info.sub_op)
            src_dtype = infos[int(info.operands[0])].dtype
            if op == UnaryOp.VALUE_CAST:
                if _is_float(src_dtype) and is_float:
                    out = ops[0]
                elif not _is_float(src_dtype) and is_float:
                    out = ops[0].astype(np.float64)
                elif not _is_float(src_dtype) and not is_float:
                    if info.dtype == DType.BOOL:
                        out = ops[0] != 0
                    else:
                        out = ops[0].astype(np.int64 if src_dtype != DType.U64 else np.uint64).astype(_NUMPY[int(info.dtype)])
                else:
                    # whole numbers convert the same way whatever the float width; anything else would depend on
                    # the rounding this evaluation leaves out
                    x = ops[0]
                    if not np.all(np.isfinite(x) & (x == np.round(x))):
                        raise Unsupported("float -> integer cast of values that are not whole numbers")
                    if info.dtype == DType.BOOL:
                        out = x != 0
                    else:
                        limits = np.iinfo(_NUMPY[int(info.dtype)])
                        if np.any(x < float(limits.min)) or np.any(x > float(limits.max)):
                            raise Unsupported("float -> integer cast out of range")
                        out = x.astype(_NUMPY[int(info.dtype)])
            elif op == UnaryOp.BIT_CAST:
                if _is_float(src_dtype) or is_float:
                    raise Unsupported("bit cast of a float")
                out = ops[0].view(_NUMPY[int(info.dtype)])
            elif is_float:
                out = _unary(op, ops[0])
            elif op == UnaryOp.ABS:
                with np.errstate(all="ignore"):
                    out = np.abs(ops[0])
            elif op == UnaryOp.NEG:
                with np.errstate(all="ignore"):
                    out = (0 - ops[0]).astype(ops[0].dtype)
            else:
                raise Unsupported(f"unary {op} on {info.dtype}")
        elif kind == OpKind.BINARY:
            out = _binary(BinaryOp(info.sub_op), ops[0], ops[1], is_float)
        elif kind == OpKind.SOFTMAX:
            x = ops[0]
            axis = info.axes[0]
            with np.errstate(all="ignore"):
                e = np.exp(x - np.fmax.reduce(x, axis=axis, keepdims=True, initial=-np.inf))
                out = e / e.sum(axis=axis, keepdims=True)
        elif kind == OpKind.LAYERNORM:
            x = ops[0]
            axis = info.axes[0]
            centered = x - x.mean(axis=axis, keepdims=True)
            out = centered / np.sqrt((centered * centered).mean(axis=axis, keepdims=True) + np.float64(np.float32(info.eps)))
        elif kind == OpKind.REDUCE:
            op = ReduceOp(info.sub_op)
            axes = tuple(info.axes)
            x = ops[0]
            with np.errstate(all="ignore"):
                if op == ReduceOp.SUM:
                    out = x.sum(axis=axes, dtype=x.dtype)
                elif op == ReduceOp.MEAN:
                    if not is_float:
                        raise Unsupported("integer mean")
                    out = x.mean(axis=axes)
                elif op == ReduceOp.PROD:
                    out = x.prod(axis=axes, dtype=x.dtype)
                elif op == ReduceOp.MAX:
                    out = np.fmax.reduce(x, axis=axes, initial=-np.inf) if is_float else x.max(axis=axes)
                else:
                    out = np.fmin.reduce(x, axis=axes, initial=np.inf) if is_float else x.min(axis=axes)
            out = np.asarray(out).reshape(shape)
        else:
            raise Unsupported(str(kind))
        assert list(out.shape) == shape, f"value {int(v)} ({kind.name}): shape {out.shape}, expected {shape}"
        if storage_rounding and is_float and int(info.dtype) != DType.F64:
            with np.errstate(all="ignore"):
                out = out.astype(_NUMPY[int(info.dtype)]).astype(np.float64)
        values[int(v)] = out
        for o in info.operands:
            if last_use.get(int(o)) == int(v) and int(o) not in keep:
                values.pop(int(o), None)
    return [np.array(values[int(o)], order="C") for o in graph.outputs()]
