"""kn-cuda-eval/tests/root/opt.rs: scalar fusion shapes and optimizer structure tests."""
import numpy as np
import pytest

from kyanite_amd import BATCH, BinaryOp, DType, Graph, HipExecutor, OpKind, OptimizerSettings, UnaryOp, optimize_graph
from runner import check_cpu, check_gpu, rng_tensor


def _scalar_graph(kind):
    rng = np.random.default_rng(0)
    g = Graph()
    x = g.input([2, 3])
    if kind == "chained":
        w1 = g.constant([1, 3], [1.0, 2.0, 3.0])
        w2 = g.constant([2, 1], [0.1, 0.2])
    else:
        w1 = g.constant([1, 3], rng_tensor(rng, 3))
        w2 = g.constant([2, 1], rng_tensor(rng, 2))
    if kind == "chained":  # opt.rs:14-31, golden values from the reference
        g.output(g.add(g.mul(x, w1), w2))
        return g, 0, [np.ones((2, 3), np.float32)], [np.array([[1.1, 2.1, 3.1], [1.2, 2.2, 3.2]], np.float32)]
    y1 = g.mul(x, w1)
    y2 = g.add(x, w2)
    if kind == "split":  # opt.rs:34-51
        g.output_all([y1, y2])
    elif kind == "rejoining":  # opt.rs:54-72
        g.output(g.binary(BinaryOp.MAX, y1, y2))
    else:  # inner_scalar_used, opt.rs:75-93
        g.output_all([y1, g.binary(BinaryOp.MAX, y1, y2)])
    return g, 0, [rng_tensor(rng, 2, 3)], None


KINDS = ["chained", "split", "rejoining", "inner_used"]


@pytest.mark.parametrize("kind", KINDS)
def test_scalar_fusion_cpu(kind):
    check_cpu(*_scalar_graph(kind))


@pytest.mark.gpu
@pytest.mark.parametrize("kind", KINDS)
def test_scalar_fusion_gpu(kind, hip_device):
    print(f"case {kind}", flush=True)
    check_gpu(hip_device, *_scalar_graph(kind), what=f"scalar fusion {kind}")


def test_scalar_fusion_plans():
    """chains fuse, a value that is also an output is computed once; two results of one shape that do not depend on
    each other share a launch (and the load of x), a result that reads the other one does not"""
    assert HipExecutor(0, _scalar_graph("chained")[0], 0, plan_only=True).step_kinds() == ["scalar_op"]
    assert HipExecutor(0, _scalar_graph("rejoining")[0], 0, plan_only=True).step_kinds() == ["scalar_op"]
    split = HipExecutor(0, _scalar_graph("split")[0], 0, plan_only=True)
    assert split.step_kinds() == ["scalar_op"] and "outputs=2" in split.step_str(0)
    assert HipExecutor(0, _scalar_graph("inner_used")[0], 0, plan_only=True).step_kinds() == ["scalar_op"] * 2


def test_gather_cast_collapses_to_slice():
    """opt.rs:96-122"""
    g = Graph()
    x = g.input([4])
    i_float = g.constant([1], [0.0])
    i = g.value_cast(i_float, DType.U32)
    g.output(g.gather(x, 0, i))
    opt = optimize_graph(g, OptimizerSettings())
    ox, oy = opt.inputs()[0], opt.outputs()[0]
    info = opt[oy]
    assert info.op == OpKind.SLICE and info.operands == [ox] and info.axes == [0] and info.slice == (0, 1, 1)


def test_optimizer_settings():
    """optimizer/mod.rs:25-57: `optimize = false` returns an identical graph; div-to-mul can be switched off"""
    g = Graph()
    x = g.input([3, 4])  # with a batch axis the broadcast divisor is not a constant of known shape and is left alone
    g.output(g.binary(BinaryOp.DIV, x, g.scalar(4.0)))
    same = optimize_graph(g, OptimizerSettings(optimize=False))
    assert str(same) == str(g)
    kept = optimize_graph(g, OptimizerSettings(div_to_mul=False))
    assert kept[kept.outputs()[0]].sub_op == int(BinaryOp.DIV)
    changed = optimize_graph(g)
    out = changed[changed.outputs()[0]]
    assert out.sub_op == int(BinaryOp.MUL)
    assert changed.as_single_const(out.operands[1]) == np.float32(0.25)


def test_bn_folds_into_conv():
    """optimizer/affine.rs: per-channel add / mul / sub / div around a convolution end up inside its filter and one
    bias; with padding, a bias in front of the conv only moves through when forced to."""
    def build(pad):
        g = Graph()
        x = g.input([BATCH, 3, 6, 6])
        k = 2 * pad + 1  # only convolutions that keep the spatial shape take part (optimizer/affine.rs:53)
        w = g.constant([5, 3, k, k], np.linspace(-1, 1, 15 * k * k, dtype=np.float32))
        c = lambda n, lo, hi: g.constant([1, n, 1, 1], np.linspace(lo, hi, n, dtype=np.float32))
        y = g.mul(g.sub(x, c(3, 0.1, 0.3)), c(3, 0.5, 2.0))
        y = g.conv(y, w, 1, 1, pad, pad)
        y = g.binary(BinaryOp.DIV, g.add(y, c(5, -1, 1)), c(5, 1.0, 3.0))
        g.output(g.relu(y))  # a group can only start at a hidden value (optimizer/core.rs:299-326)
        return g
    assert [build(1)[v].op for v in build(1).values()].count(OpKind.BINARY) == 5
    opt = optimize_graph(build(1))
    ops = [opt[v].op for v in opt.values()]
    # a bias in front of a padded conv cannot move through it: scale and bias stay in front (2 binaries), the two
    # operations behind the conv become filter scaling + one bias (1), plus the relu (1)
    assert ops.count(OpKind.CONV) == 1 and ops.count(OpKind.BINARY) == 4
    forced = optimize_graph(build(1), OptimizerSettings(force_bias_through_conv=True))
    ops = [forced[v].op for v in forced.values()]
    assert ops.count(OpKind.CONV) == 1 and ops.count(OpKind.BINARY) == 2  # one position dependent bias + relu
    nopad = optimize_graph(build(0))
    ops = [nopad[v].op for v in nopad.values()]
    assert ops.count(OpKind.CONV) == 1 and ops.count(OpKind.BINARY) == 2  # one per-channel bias + relu
    x = np.random.default_rng(0).standard_normal((2, 3, 6, 6)).astype(np.float32)
    for pad in (0, 1):
        check_cpu(build(pad), 2, [x])
    from oracle import cpu_eval_graph
    from runner import assert_tensors_match
    assert_tensors_match(cpu_eval_graph(build(1), 2, [x]), cpu_eval_graph(forced, 2, [x]), "forced bias through conv")
