"""`knhip_executor_options`: every planned path that can be switched off, per executor.

For each option one graph whose default plan takes the path. CPU half: with the option off the plan changes the way
the option says (and only that executor's plan: the options are no process-wide state). GPU half: the executor with
the option off gives the oracle's result, like the default one.
"""
import numpy as np
import pytest

from kyanite_amd import BATCH, DType, Graph, HipExecutor, KnError, ReduceOp, UnaryOp
from oracle import cpu_eval_graph
from runner import PARITY_RECORDS, check_outputs

RNG = np.random.default_rng(4242)


def _normal(*shape, dtype=np.float32):
    return RNG.standard_normal(shape).astype(dtype)


def attention_f32():
    g = Graph()
    q, k, v = g.input([4, 96, 40]), g.input([4, 80, 40]), g.input([4, 80, 40])
    g.output(g.batched_mat_mul(g.softmax(g.batched_mat_mul(q, g.permute(k, [0, 2, 1])), 2), v))
    return g, 0, [_normal(4, 96, 40), _normal(4, 80, 40), _normal(4, 80, 40)]


def shared_left_linears():
    g = Graph()
    x = g.input([192, 256], DType.F16)
    for _ in range(3):
        g.output(g.linear(x, g.constant([128, 256], (_normal(128, 256) / 16).astype(np.float16), DType.F16)))
    return g, 0, [_normal(192, 256, dtype=np.float16)]


def gated_feed_forward():
    g = Graph()
    x = g.input([96, 128], DType.F16)
    gate = g.linear(x, g.constant([208, 128], (_normal(208, 128) / 11).astype(np.float16), DType.F16))
    up = g.linear(x, g.constant([208, 128], (_normal(208, 128) / 11).astype(np.float16), DType.F16))
    g.output(g.mul(g.mul(gate, g.sigmoid(gate)), up))
    return g, 0, [_normal(96, 128, dtype=np.float16)]


def constant_kn_weight():
    g = Graph()
    x = g.input([64, 128], DType.F16)
    g.output(g.mat_mul(x, g.constant([128, 256], (_normal(128, 256) / 11).astype(np.float16), DType.F16)))
    return g, 0, [_normal(64, 128, dtype=np.float16)]


def pointwise_conv():
    g = Graph()
    x = g.input([BATCH, 32, 8, 8])
    g.output(g.relu(g.add(g.conv(x, g.constant([16, 32, 1, 1], _normal(16, 32, 1, 1) / 6), 1, 1, 0, 0),
                          g.constant([1, 16, 1, 1], _normal(1, 16, 1, 1)))))
    return g, 6, [_normal(6, 32, 8, 8)]


def independent_elementwise():
    g = Graph()
    x, y = g.input([64, 96]), g.input([64, 96])
    g.output_all([g.unary(UnaryOp.EXP, x), g.unary(UnaryOp.TANH, y)])
    return g, 0, [_normal(64, 96), _normal(64, 96)]


def tall_column_mean():
    g = Graph()
    g.output(g.reduce(g.input([65536, 64]), [0], ReduceOp.MEAN))
    return g, 0, [_normal(65536, 64)]


def transposed_add():
    g = Graph()
    x, y = g.input([320, 512]), g.input([512, 320])
    g.output(g.add(g.permute(x, [1, 0]), y))
    return g, 0, [_normal(320, 512), _normal(512, 320)]


def small_batch_conv():
    g = Graph()
    x = g.input([BATCH, 128, 8, 8])
    g.output(g.conv(x, g.constant([128, 128, 3, 3], _normal(128, 128, 3, 3) / 34), 1, 1, 1, 1))
    return g, 16, [_normal(16, 128, 8, 8)]


def odd_width_conv():
    g = Graph()
    x = g.input([BATCH, 64, 9, 9])
    g.output(g.conv(x, g.constant([64, 64, 3, 3], _normal(64, 64, 3, 3) / 24), 1, 1, 1, 1))
    return g, 32, [_normal(32, 64, 9, 9)]


def aligned_matmul_f16():
    g = Graph()
    x = g.input([256, 512], DType.F16)
    g.output(g.linear(x, g.constant([384, 512], (_normal(384, 512) / 22).astype(np.float16), DType.F16)))
    return g, 0, [_normal(256, 512, dtype=np.float16)]


def long_k_matmul():
    g = Graph()
    x = g.input([8, 4096])
    g.output(g.linear(x, g.constant([512, 4096], _normal(512, 4096) / 64)))
    return g, 0, [_normal(8, 4096)]


def sparse_last_round_matmul():
    """688 tiles of 64 x 64 on 512 slots: the 176 tiles of the last round are split inside the launch"""
    g = Graph()
    x = g.input([1024, 1024])
    g.output(g.linear(x, g.constant([2752, 1024], _normal(2752, 1024) / 32)))
    return g, 0, [_normal(1024, 1024)]


def tiny_matmul():
    g = Graph()
    x = g.input([1, 256])
    g.output(g.linear(x, g.constant([4, 256], _normal(4, 256) / 16)))
    return g, 0, [_normal(1, 256)]


def streamed_elementwise():
    g = Graph()
    g.output(g.unary(UnaryOp.EXP, g.input([1024, 1024])))
    return g, 0, [_normal(1024, 1024)]


def plan_text(ex):
    return "\n".join(ex.step_str(i) for i in range(ex.step_count()))


def sources(ex):
    return "\n".join(ex.step_source(i) for i in range(ex.step_count()))


# option -> (graph builder, the option's value, what the default plan shows, what the plan with the option shows)
OPTIONS = {
    "fuse_attention": (attention_f32, 0, lambda ex: "attention" in plan_text(ex), lambda ex: "attention" not in plan_text(ex) and ex.step_count() >= 3),
    "fuse_gated_matmul": (gated_feed_forward, 0, lambda ex: "gated pairs" in plan_text(ex) and ex.step_count() == 1,
                          lambda ex: "gated" not in plan_text(ex) and ex.step_count() == 2),
    "group_matmuls": (shared_left_linears, 0, lambda ex: "grouped" in plan_text(ex), lambda ex: "grouped" not in plan_text(ex) and ex.step_count() == 3),
    "pack_matmul_constants": (constant_kn_weight, 0, lambda ex: "f16[1, 256, 128]" not in plan_text(ex) and "direct" in plan_text(ex),
                              lambda ex: "staged" in plan_text(ex)),
    "pointwise_conv_as_matmul": (pointwise_conv, 0, lambda ex: ex.step_kinds() == ["mat_mul"], lambda ex: ex.step_kinds() == ["conv"]),
    "join_elementwise": (independent_elementwise, 0, lambda ex: ex.step_count() == 1, lambda ex: ex.step_count() == 2),
    "split_reduce": (tall_column_mean, 0, lambda ex: ex.step_count() == 2, lambda ex: ex.step_count() == 1),
    "tiled_transpose": (transposed_add, 0, lambda ex: "transposed tiles" in plan_text(ex), lambda ex: "transposed tiles" not in plan_text(ex)),
    "split_conv_channels": (small_batch_conv, 0, lambda ex: "input channels in" in plan_text(ex), lambda ex: "input channels in" not in plan_text(ex)),
    "plane_conv_any_width": (odd_width_conv, 0, lambda ex: ex.step_kinds() == ["conv"], lambda ex: ex.step_kinds() == ["conv"]),
    "direct_gemm": (aligned_matmul_f16, 0, lambda ex: "direct" in plan_text(ex), lambda ex: "staged" in plan_text(ex)),
    "split_k": (long_k_matmul, 0, lambda ex: "split_k" in plan_text(ex), lambda ex: "split" not in plan_text(ex)),
    "tail_split": (sparse_last_round_matmul, 0, lambda ex: "tail_split" in plan_text(ex), lambda ex: "tail_split" not in plan_text(ex)),
    "dot_products": (tiny_matmul, 0, lambda ex: "a wave per result" in plan_text(ex), lambda ex: "a wave per result" not in plan_text(ex)),
    "streaming_bytes": (streamed_elementwise, 1 << 20, lambda ex: "nontemporal" not in sources(ex), lambda ex: "nontemporal" in sources(ex)),
    # (the default asks for 256 MiB of constants before a weight counts as a stream)
    "stream_weights_bytes": (aligned_matmul_f16, 1 << 10, lambda ex: "weights streamed" not in plan_text(ex), lambda ex: "weights streamed" in plan_text(ex)),
}


@pytest.mark.parametrize("option", list(OPTIONS))
def test_option_changes_the_plan_of_its_executor_only(option):
    build, value, default_shows, option_shows = OPTIONS[option]
    graph, batch, _ = build()
    before = HipExecutor(0, graph, batch, plan_only=True)
    assert default_shows(before), f"default plan:\n{plan_text(before)}"
    changed = HipExecutor(0, graph, batch, plan_only=True, **{option: value})
    assert option_shows(changed), f"plan with {option}={value}:\n{plan_text(changed)}"
    after = HipExecutor(0, graph, batch, plan_only=True)
    assert plan_text(after) == plan_text(before), "an option of one executor leaked into the next"


def test_unknown_option_and_wrong_struct_size_are_refused():
    from ctypes import byref, c_void_p
    from kyanite_amd._lib import check, lib
    from kyanite_amd.executor import executor_options
    graph, batch, _ = independent_elementwise()
    with pytest.raises(KnError, match="unknown executor option"):
        HipExecutor(0, graph, batch, plan_only=True, fuse_everything=True)
    opts = executor_options(plan_only=True)
    opts.struct_bytes = 8
    handle = c_void_p()
    with pytest.raises(KnError, match="struct_bytes"):
        check(lib.knhip_executor_new(0, graph._h, batch, byref(opts), byref(handle)))


@pytest.mark.gpu
@pytest.mark.parametrize("option", list(OPTIONS))
def test_option_off_path_gives_the_oracles_result(option, hip_device):
    build, value, _, _ = OPTIONS[option]
    graph, batch, inputs = build()
    print(f"executor option {option}={value}", flush=True)
    expected = cpu_eval_graph(graph, batch, inputs)
    for label, kwargs in (("default", {}), (f"{option}={value}", {option: value})):
        got = HipExecutor(hip_device, graph, batch, **kwargs).evaluate(inputs)
        check_outputs(graph, batch, inputs, expected, got, f"executor option, {label}", PARITY_RECORDS)


@pytest.mark.gpu
def test_mapped_io_off_leaves_the_results_in_the_device_buffers(hip_device):
    """With `mapped_io_bytes=0` evaluate copies through the arena, so the executor's device tensors hold inputs and
    outputs afterwards, as the reference's do; by default a graph this small never touches them."""
    from kyanite_amd.configs import build_tiny_mlp
    graph, inputs = build_tiny_mlp(seed=3, batch=8)
    expected = cpu_eval_graph(graph, 8, inputs)
    ex = HipExecutor(hip_device, graph, 8, mapped_io_bytes=0)
    got = ex.evaluate(inputs)
    check_outputs(graph, 8, inputs, expected, got, "tiny mlp, mapped io off", PARITY_RECORDS)
    assert np.array_equal(ex.download_output(0), got[0])
