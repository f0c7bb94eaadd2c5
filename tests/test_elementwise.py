"""kn-cuda-eval/tests/root/elementwise.rs: unary / binary sweeps over the reference's fixed values, the softplus
golden vector, clamp combinations and the value / bit cast goldens.

The expected values of the sweeps are computed here with numpy / math in the way kn-graph/src/graph.rs:1660-1729
defines each operation, independently of the oracle's C++ restatement (a library routine per operation).
"""
import math

import numpy as np
import pytest

from kyanite_amd import BINARY_ALL, UNARY_ALL, BinaryOp, DType, Graph, UnaryOp
from runner import check_cpu, check_gpu

# runner.rs:57-60
ELEMENTWISE_TEST_VALUES = np.array([0.0, 0.1, 0.5, 0.8, 1.0, 1.1, 1.5, 1.7, 2.0, 5.0, 6.0, 7.0, -1.0, -1.0, 0.5, 20.0, 80.0,
                                    100.0, 1000.0, -20.0, -100.0], np.float32)


def _erf_as(x):
    """graph.rs:1791-1815 (Abramowitz and Stegun) in f64, written out independently"""
    a = [1.0, 0.0705230784, 0.0422820123, 0.0092705272, 0.0001520143, 0.0002765672, 0.0000430638]
    s = -1.0 if math.copysign(1.0, x) < 0 else 1.0
    xa = abs(x)
    d = sum(c * xa ** i for i, c in enumerate(a))
    return s * (1.0 - 1.0 / d ** 16)


def unary_expected(op, x):
    x = x.astype(np.float32)
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
            return (np.float32(1) / (np.float32(1) + np.exp(-x))).astype(np.float32)
        if op == UnaryOp.TANH:
            return np.tanh(x)
        if op == UnaryOp.ERF:
            return np.array([_erf_as(float(v)) for v in x], np.float64).astype(np.float32)
        if op == UnaryOp.MISH:
            return (x * np.tanh(np.log1p(np.exp(x)))).astype(np.float32)
        if op == UnaryOp.SOFTPLUS:
            return (np.log1p(np.exp(-np.abs(x))) + np.maximum(x, np.float32(0))).astype(np.float32)
    raise AssertionError(op)


def binary_expected(op, a, b):
    with np.errstate(all="ignore"):
        if op == BinaryOp.ADD:
            return a + b
        if op == BinaryOp.SUB:
            return a - b
        if op == BinaryOp.MUL:
            return a * b
        if op == BinaryOp.DIV:
            return a / b
        if op == BinaryOp.MIN:
            return np.fmin(a, b)
        if op == BinaryOp.MAX:
            return np.fmax(a, b)
        if op == BinaryOp.POW:
            return np.power(a, b).astype(np.float32)
    raise AssertionError(op)


def unary_case(op):
    g = Graph()
    x = g.input([len(ELEMENTWISE_TEST_VALUES)])
    g.output(g.unary(op, x))
    return g, 0, [ELEMENTWISE_TEST_VALUES], [unary_expected(op, ELEMENTWISE_TEST_VALUES)]


def binary_case(op):
    v = ELEMENTWISE_TEST_VALUES
    n = len(v)
    g = Graph()
    left = g.input([n * n])
    right = g.input([n * n])
    g.output(g.binary(op, left, right))
    a = np.repeat(v, n)
    b = np.tile(v, n)
    return g, 0, [a, b], [binary_expected(op, a, b)]


def softplus_fixed_case():
    """elementwise.rs:21-36, golden values from the reference"""
    g = Graph()
    x = g.input([5])  # the reference uses a batch axis of size 5
    g.output(g.unary(UnaryOp.SOFTPLUS, x))
    return (g, 0, [np.array([-2.0, -1.0, 0.0, 1.0, 2.0], np.float32)],
            [np.array([0.126928, 0.313262, 0.693147, 1.313262, 2.126928], np.float32)])


def clamp_case(lo, hi):
    """elementwise.rs:47-57"""
    g = Graph()
    x = g.input([len(ELEMENTWISE_TEST_VALUES)])
    g.output(g.clamp(x, lo, hi))
    return g, 0, [ELEMENTWISE_TEST_VALUES], [np.clip(ELEMENTWISE_TEST_VALUES, lo, hi)]


def cast_case(kind):
    """elementwise.rs:61-102: every pair is (input scalar, expected scalar), golden values from the reference"""
    if kind == "value":
        pairs = [(np.uint8(5), np.uint8(5)), (np.uint32(5), np.uint32(5)), (np.float32(5), np.float32(5)),
                 (np.uint64(0xdeadbeefdeadbeef), np.uint64(0xdeadbeefdeadbeef)),
                 (np.uint8(1), np.uint32(1)), (np.int8(-1), np.uint32(0xffffffff)),
                 (np.uint32(1), np.uint8(1)), (np.int32(-1), np.uint8(255)),
                 (np.float32(1), np.uint32(1)), (np.float32(-1), np.int32(-1)), (np.float32(-1), np.int64(-1)),
                 (np.float32(-1), np.int8(-1))]
    else:
        pairs = [(np.uint8(5), np.uint8(5)), (np.uint32(5), np.uint32(5)), (np.float32(5), np.float32(5)),
                 (np.uint64(0xdeadbeefdeadbeef), np.uint64(0xdeadbeefdeadbeef)),
                 (np.float32(1), np.float32(1).view(np.uint32)), (np.float32(-1), np.float32(-1).view(np.uint32))]
    g = Graph()
    inputs, expected = [], []
    for x, y in pairs:
        xv = g.input([], DType.from_numpy(x.dtype))
        to = DType.from_numpy(y.dtype)
        g.output(g.value_cast(xv, to) if kind == "value" else g.bit_cast(xv, to))
        inputs.append(np.asarray(x))
        expected.append(np.asarray(y))
    return g, 0, inputs, expected


CASES = {}
for _op in UNARY_ALL:
    CASES[f"unary_{_op.name.lower()}"] = (lambda op=_op: unary_case(op))
for _op in BINARY_ALL:
    CASES[f"binary_{_op.name.lower()}"] = (lambda op=_op: binary_case(op))
CASES["softplus_fixed"] = softplus_fixed_case
for _lo in (-math.inf, 0.0):
    for _hi in (math.inf, 6.0):
        CASES[f"clamp_{_lo}_{_hi}"] = (lambda lo=_lo, hi=_hi: clamp_case(lo, hi))
CASES["value_cast"] = lambda: cast_case("value")
CASES["bit_cast"] = lambda: cast_case("bit")


@pytest.mark.parametrize("name", list(CASES))
def test_cpu(name):
    graph, batch, inputs, expected = CASES[name]()
    check_cpu(graph, batch, inputs, expected)


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(CASES))
def test_gpu(name, hip_device):
    graph, batch, inputs, expected = CASES[name]()
    print(f"case {name}", flush=True)
    check_gpu(hip_device, graph, batch, inputs, expected, what=f"elementwise {name}")


def test_cast_to_same_type_is_identity():
    """opt.rs:125-136"""
    g = Graph()
    x = g.input([], DType.F32)
    assert g.bit_cast(x, DType.F32) == x
    assert g.value_cast(x, DType.F32) == x
