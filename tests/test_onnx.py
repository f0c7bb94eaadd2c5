"""The reference's ONNX + check-data fixtures (kn-cuda-eval/tests/data, used by kn-cuda-eval/tests/root/onnx.rs:3-33
through `test_onnx_bin`, runner.rs:109-114): load the model, read batch size / inputs / expected outputs from the
`.bin` file, and run the same differential test as for the hand-built graphs. The expected outputs were produced by
the reference's authors (the exporting framework), so they pin the oracle on whole graphs: Gemm, Conv (1D and 2D),
BatchNormalization, Clip, Softmax, ReduceMean / layernorm patterns, Gather, Slice, Reshape with symbolic batch."""
import os

import numpy as np
import pytest

from kyanite_amd import OpKind, Size, optimize_graph
from kyanite_amd.onnx import OnnxError, SignedSize, load_check_data, load_graph_from_onnx_bytes
from runner import assert_close, check_cpu, check_gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FIXTURES = ["simple-sttt-1x64", "simple-bn-sttt-1x64", "pre-sttt-4x8", "att-tiny"]


def load(name):
    with open(os.path.join(GOLDEN, name + ".onnx"), "rb") as f:
        graph = load_graph_from_onnx_bytes(f.read())
    with open(os.path.join(GOLDEN, name + ".bin"), "rb") as f:
        batch, inputs, expected = load_check_data(graph, f.read())
    return graph, batch, inputs, expected


@pytest.mark.parametrize("name", FIXTURES)
def test_fixture_cpu(name):
    graph, batch, inputs, expected = load(name)
    outputs = check_cpu(graph, batch, inputs, expected)
    # far inside the reference's 1e-3 tolerance: the project's own bar holds against the golden vectors as well
    assert_close(expected, outputs, f"{name}: oracle vs golden vectors")


@pytest.mark.gpu
@pytest.mark.parametrize("name", FIXTURES)
def test_fixture_gpu(name, hip_device):
    graph, batch, inputs, expected = load(name)
    outputs = check_gpu(hip_device, graph, batch, inputs, expected, what=f"onnx {name}")
    assert_close(expected, outputs, f"{name}: gpu vs golden vectors")


def test_fixture_shapes_and_batch():
    graph, batch, inputs, expected = load("att-tiny")
    assert batch == 4 and [list(x.shape) for x in inputs] == [[4, 21, 8, 8]]
    assert [list(x.shape) for x in expected] == [[4, 5], [4, 1880]]
    assert sum(x.size for x in inputs) + sum(x.size for x in expected) == 12916
    # the batch axis stays symbolic through Shape -> Gather -> Unsqueeze -> Concat -> Reshape
    assert graph[graph.inputs()[0]].shape[0] == Size.BATCH
    assert all(graph[v].shape[0] == Size.BATCH for v in graph.outputs())
    graph, batch, _, _ = load("simple-sttt-1x64")
    assert batch == 2 and [repr(d) for d in graph[graph.inputs()[0]].shape] == ["B", "2", "9", "9"]


def test_optimizer_on_fixtures():
    # the exported layernorm pattern (ReduceMean, Sub, Pow, ReduceMean, Add, Sqrt, Div) collapses into Layernorm
    graph, _, _, _ = load("att-tiny")
    kinds = lambda g: [g[v].op for v in range(len(g))]
    assert OpKind.LAYERNORM not in kinds(graph)
    opt = optimize_graph(graph)
    assert kinds(opt).count(OpKind.LAYERNORM) == 2 and len(opt) < len(graph)
    # batch-norm folds into the convolutions: no division is left
    graph, _, _, _ = load("pre-sttt-4x8")
    opt = optimize_graph(graph)
    assert len(opt) < len(graph)


def test_signed_size_arithmetic():
    # kn-graph/src/onnx/typed_value.rs:270-295
    B, one = SignedSize(1, 1), SignedSize(0, 1)
    i = lambda v: SignedSize(0, v)
    assert B.add(one) is None
    assert i(3).sub(i(2)) == i(1)
    assert i(3).sub(i(4)) == i(-1)
    assert i(3).add(-i(4)) == i(-1)
    assert i(3).sub(-i(4)) == i(7)
    assert i(0).sub(B) == -B
    assert B.mul(i(6)).floor_div(B) == i(6) and i(6).floor_div(B) is None
    assert i(-7).floor_div(i(2)) == i(-3)  # Rust integer division truncates


def test_loader_rejects_what_it_does_not_cover():
    with open(os.path.join(GOLDEN, "simple-sttt-1x64.onnx"), "rb") as f:
        data = bytearray(f.read())
    # rename the op type of the Relu node (same length, so the framing stays valid)
    at = data.find(b'"\x04Relu')  # field 4 (op_type), length 4
    assert at > 0
    data[at + 2:at + 6] = b"Rilu"
    with pytest.raises(OnnxError, match="unsupported ONNX operation Rilu"):
        load_graph_from_onnx_bytes(bytes(data))
    with pytest.raises(ValueError):
        load_check_data(load("simple-sttt-1x64")[0], b"\x02abc")
