"""Host-side unit tests: graph builder canonicalisation, shapes, layout algebra, serialisation, error behaviour.

Mirrors kn-graph/tests/graph/mod.rs:10-99 and the unit tests in kn-cuda-eval/src/shape.rs:346-431, with the
golden values those tests hold.
"""
import ctypes
from ctypes import byref, c_int, c_int64, c_size_t

import numpy as np
import pytest

from kyanite_amd import BATCH, BinaryOp, DType, Graph, HipExecutor, KnError, OpKind, ReduceOp, Size, UnaryOp
from kyanite_amd._lib import check, lib


def test_dedup_const():
    """kn-graph/tests/graph/mod.rs:10-25: equal constants are one value, NaN constants included"""
    g = Graph()
    x0 = g.constant([2], [1.0, 2.0])
    x1 = g.constant([2], [1.0, 2.0])
    x2 = g.constant([2], [1.0, 3.0])
    assert x0 == x1 and x0 != x2
    y0 = g.constant([2], [1.0, float("nan")])
    y1 = g.constant([2], [1.0, float("nan")])
    assert y0 == y1 and x0 != y0


def test_dedup_operations():
    g = Graph()
    x = g.input([BATCH, 4])
    assert g.unary(UnaryOp.EXP, x) == g.unary(UnaryOp.EXP, x)
    assert g.unary(UnaryOp.EXP, x) != g.unary(UnaryOp.LOG, x)
    assert g.layernorm(x, 1, 1e-5) == g.layernorm(x, 1, 1e-5)
    assert g.layernorm(x, 1, 1e-5) != g.layernorm(x, 1, 1e-6)


@pytest.mark.parametrize("expected, actual, result", [
    # kn-graph/tests/graph/mod.rs:35-98; status codes: 0 ok, 1 different length, 2 constant mismatch,
    # 3 batch conflict, 4 impossible batch value
    ([[2, 3, 4]], [[2, 3, 4]], (0, None)),
    ([[2, 3, 4], [5, 6]], [[2, 3, 4], [1, 6]], (2, None)),
    ([[2, BATCH]], [[2, 8]], (0, 8)),
    ([[BATCH, BATCH]], [[4, 4]], (0, 4)),
    ([[BATCH, BATCH]], [[4, 8]], (3, None)),
    ([[BATCH], [BATCH]], [[4], [8]], (3, None)),
    ([[BATCH, BATCH * BATCH, BATCH * 4, BATCH * 8]], [[10, 100, 40, 80]], (0, 10)),
    ([[BATCH, BATCH * BATCH, BATCH * 4, BATCH * 3]], [[10, 100, 40, 80]], (3, None)),
    ([[BATCH * 2]], [[7]], (4, None)),
    ([[BATCH * BATCH]], [[15]], (4, None)),
])
def test_infer_batch_size(expected, actual, result):
    g = Graph()
    for s in expected:
        g.input(s)
    status, batch = g.infer_batch_size(actual)
    assert status == result[0]
    if status == 0:
        assert batch == result[1]


def test_builder_canonicalisation():
    g = Graph()
    x = g.input([BATCH, 6, 4])
    # view of a view keeps only the last view (graph.rs:632-639); a view to the same shape is the value itself
    v1 = g.view(x, [BATCH, 24])
    v2 = g.view(v1, [BATCH, 4, 6])
    assert g[v2].operands == [x]
    assert g.view(x, [BATCH, 6, 4]) == x
    # consecutive permutes fuse (graph.rs:745-755)
    p = g.permute(g.permute(x, [0, 2, 1]), [2, 1, 0])
    assert g[p].op == OpKind.PERMUTE and g[p].operands == [x] and g[p].axes == [1, 2, 0]
    # trivial slice is skipped (graph.rs:783-786)
    assert g.slice(x, 1, 0, 6) == x
    # binary identities are skipped (graph.rs:1297-1307)
    assert g.add(x, g.scalar(0.0)) == x
    assert g.mul(x, g.scalar(1.0)) == x
    assert g.binary(BinaryOp.MIN, x, g.scalar(np.inf)) == x
    assert g.binary(BinaryOp.MAX, x, g.scalar(-np.inf)) == x
    assert g.add(x, g.scalar(1.0)) != x
    # relu is max(x, 0) (graph.rs:1185-1218)
    r = g.relu(x)
    assert g[r].op == OpKind.BINARY and g[r].sub_op == int(BinaryOp.MAX)
    # concat drops empties and collapses a single input (graph.rs:944-951)
    e = g.slice(x, 1, 0, 0)
    assert g.concat([e, x, e], 1) == x
    # reduce over no axes is the value itself
    assert g.reduce(x, [], ReduceOp.SUM) == x
    # linear = permute + mat_mul through views (graph.rs:1053-1101)
    w = g.constant([5, 4], np.arange(20, dtype=np.float32))
    flat = g.view(x, [BATCH * 6, 4])
    y = g.linear(flat, w)
    assert g[y].shape == [BATCH * 6, 5]
    assert g[g[y].operands[0]].op == OpKind.MATMUL
    # conv output size (graph.rs:1027-1028)
    img = g.input([BATCH, 3, 9, 7])
    f = g.constant([8, 3, 3, 3], np.zeros(8 * 27, np.float32) + 0.5)
    assert g[g.conv(img, f, 2, 1, 1, 0)].shape == [BATCH, 8, 5, 5]


def test_builder_errors():
    g = Graph()
    x = g.input([4, 6])
    with pytest.raises(KnError, match="same size"):
        g.view(x, [5, 5])
    with pytest.raises(KnError, match="Cannot broadcast"):
        g.add(x, g.input([4, 5]))
    with pytest.raises(KnError, match="matching dtypes"):
        g.add(x, g.input([4, 6], DType.I32))
    with pytest.raises(KnError, match="out of bounds"):
        g.slice(x, 1, 0, 7)
    with pytest.raises(KnError, match="Softmax input must be f32"):
        g.softmax(g.input([3], DType.I32), 0)
    with pytest.raises(KnError, match="must be odd"):
        g.conv(g.input([1, 1, 4, 4]), g.constant([1, 1, 2, 2], np.ones(4, np.float32) * 3), 1, 1, 0, 0)
    with pytest.raises(KnError, match="not supported on dtype"):
        g.unary(UnaryOp.EXP, g.input([3], DType.I32))
    with pytest.raises(KnError, match="not supported on dtype"):
        g.unary(UnaryOp.NEG, g.input([3], DType.U8))
    with pytest.raises(KnError, match="does not belong"):
        g.unary(UnaryOp.EXP, 1000)


def test_serialisation_round_trip():
    from cases_graphs import CASES
    for name in ("pre_act_resnet", "scalar_dtypes", "attention_block", "layernorm_fused", "gather_real", "pad"):
        g = CASES[name]()[0]
        blob = g.to_bytes()
        g2 = Graph.from_bytes(blob)
        assert str(g2) == str(g), name
        assert g2.to_bytes() == blob
    with pytest.raises(KnError, match="magic"):
        Graph.from_bytes(b"\0" * 16)
    with pytest.raises(KnError, match="truncated"):
        Graph.from_bytes(CASES["linear"]()[0].to_bytes()[:-3])


def test_executor_argument_checks():
    """executor.rs:118-127: wrong count, shape and dtype are rejected before anything runs (plan only: no device)"""
    g = Graph()
    x = g.input([BATCH, 4])
    g.output(g.unary(UnaryOp.EXP, x))
    ex = HipExecutor(0, g, 3, plan_only=True)
    assert ex.input_info == [(DType.F32, [3, 4])] and ex.output_info == [(DType.F32, [3, 4])]
    with pytest.raises(KnError, match="Wrong input count"):
        ex.evaluate([])
    with pytest.raises(KnError, match="Wrong shape"):
        ex.evaluate([np.zeros((2, 4), np.float32)])
    with pytest.raises(KnError, match="Wrong dtype"):
        ex.evaluate([np.zeros((3, 4), np.float64)])
    with pytest.raises(KnError, match="without a device"):
        ex.evaluate([np.zeros((3, 4), np.float32)])
    with pytest.raises(KnError, match="only supports f32"):
        g2 = Graph()
        a = g2.input([2, 3, 4], DType.F64)
        b = g2.input([2, 4, 5], DType.F64)
        g2.output(g2.batched_mat_mul(a, b))
        HipExecutor(0, g2, 0, plan_only=True)


# ---- layout algebra, kn-cuda-eval/src/shape.rs:346-431

def _arr(t, values):
    return (t * max(len(values), 1))(*values)


def strided_flags(shape, strides):
    simple, dense = c_int(), c_int()
    check(lib.knhip_strided_flags(_arr(c_size_t, shape), _arr(c_int64, strides), len(shape), byref(simple), byref(dense)))
    return bool(simple.value), bool(dense.value)


def strided_view(shape, strides, new_shape):
    ok = c_int()
    out = (c_int64 * max(len(new_shape), 1))()
    check(lib.knhip_strided_view(_arr(c_size_t, shape), _arr(c_int64, strides), len(shape), _arr(c_size_t, new_shape),
                                 len(new_shape), byref(ok), out))
    return [out[i] for i in range(len(new_shape))] if ok.value else None


def test_strided_properties():
    assert strided_flags([2, 3], [3, 1]) == (True, True)        # shape.rs:353-356
    assert strided_flags([3, 2], [1, 3]) == (False, True)       # :358-360
    assert strided_flags([3, 2], [8, 10]) == (False, False)     # :362-364
    assert strided_flags([2, 3], [3, -1]) == (False, True)      # :368-372


def test_strided_view():
    assert strided_view([], [], [1, 1, 1]) == [1, 1, 1]                          # shape.rs:385-392
    assert strided_view([2, 3, 0, 5], [0, 0, 0, 2], [0]) == [1]                  # :396-398
    assert strided_view([2, 3, 0, 5], [0, 0, 0, 2], [12, 0]) == [0, 1]           # :399
    simple = ([2, 3, 4, 3, 2], [72, 24, 6, 2, 1])
    assert strided_view(*simple, [144]) == [1]                                   # :404-407
    assert strided_view(*simple, [72, 2]) == [2, 1]                              # :408
    assert strided_view(*simple, [72, 2, 1, 1, 1]) == [2, 1, 1, 1, 1]            # :409-412
    assert strided_view([2, 3, 4], [24, 8, 1], [6, 4]) == [8, 1]                 # :417-419
    assert strided_view([2, 3, 4], [24, 8, 1], [24]) is None                     # :420


def test_strided_slice():
    shape = (c_size_t * 3)()
    strides = (c_int64 * 3)()
    check(lib.knhip_strided_slice(_arr(c_size_t, [2, 3, 4]), _arr(c_int64, [24, 8, 1]), 3, 1, 0, 4, 2, shape, strides))
    assert list(shape) == [2, 2, 4] and list(strides) == [24, 16, 1]             # shape.rs:424-430


def test_plan_reuses_memory_and_fuses():
    """One elementwise chain is one kernel; buffers of values with disjoint live ranges share arena space."""
    g = Graph()
    x = g.input([BATCH, 256])
    y = x
    for k in range(6):
        y = g.unary(UnaryOp.EXP, g.permute(g.view(y, [BATCH, 16, 16]), [0, 2, 1]))
        y = g.view(g.softmax(y, 2), [BATCH, 256])  # forces a materialised value per round
    g.output(y)
    ex = HipExecutor(0, g, 4, plan_only=True)
    usage = ex.mem_usage
    assert usage["hypo_shared_bytes_peak"] <= usage["shared_bytes"] < usage["hypo_shared_bytes_total"]
    # layernorm followed by gamma / beta is a single row kernel, nothing else
    g2 = Graph()
    x2 = g2.input([BATCH, 64])
    gamma = g2.constant([64], np.linspace(0.5, 1.5, 64, dtype=np.float32))
    beta = g2.constant([64], np.linspace(-1, 1, 64, dtype=np.float32))
    g2.output(g2.add(g2.mul(g2.layernorm(x2, 1, 1e-5), gamma), beta))
    assert HipExecutor(0, g2, 4, plan_only=True).step_kinds() == ["layernorm_op"]
    # conv + bias + residual + relu is a single conv step (planner.rs:669-833)
    g3 = Graph()
    x3 = g3.input([BATCH, 4, 8, 8])
    w = g3.constant([4, 4, 3, 3], np.linspace(-1, 1, 144, dtype=np.float32))
    b = g3.constant([1, 4, 1, 1], np.linspace(-1, 1, 4, dtype=np.float32))
    g3.output(g3.relu(g3.add(g3.add(g3.conv(x3, w, 1, 1, 1, 1), b), x3)))
    assert HipExecutor(0, g3, 2, plan_only=True).step_kinds() == ["conv"]
    # softmax(x * scalar) folds the scale into the softmax kernel (planner.rs:584-604)
    g4 = Graph()
    x4 = g4.input([BATCH, 10])
    g4.output(g4.softmax(g4.mul(x4, g4.scalar(0.125)), 1))
    assert HipExecutor(0, g4, 2, plan_only=True).step_kinds() == ["softmax_op"]
