"""Launch decisions of the matrix multiply (no device needed but for the last test): which shapes reserve a split-K
workspace in the arena, and that the workspace is the size the launch will use (split * batch * m * n f32 values)."""
import re

import numpy as np
import pytest

from kyanite_amd import DType, Graph, HipExecutor, UnaryOp


def plan(m, n, k, batch=1, dtype=DType.F32):
    g = Graph()
    a = g.input([batch, m, k], dtype)
    b = g.input([batch, k, n], dtype)
    g.output(g.batched_mat_mul(a, b))
    ex = HipExecutor(0, g, 0, plan_only=True)
    # (an f16 right operand with n contiguous is copied into [n, k] order first when the left one has 256 rows)
    copies = 1 if dtype == DType.F16 and m >= 256 and k % 64 == 0 and n >= 16 else 0
    assert ex.step_kinds() == ["scalar_op"] * copies + ["mat_mul"]
    text = ex.step_str(copies)
    shapes = re.findall(r"f(?:16|32)\[([0-9, ]*)\]", text.split("operands:")[1])
    workspace = int(shapes[3]) if len(shapes) > 3 else 0
    return workspace, ex


def test_no_split_when_the_tiles_fill_the_chip():
    for m, n, k in ((4096, 4096, 4096), (1024, 4672, 2048), (512, 11008, 4096)):
        assert plan(m, n, k)[0] == 0
    assert plan(512, 11008, 4096, dtype=DType.F16)[0] == 0
    # short contractions never split, however few tiles there are; from 256 on a handful of tiles does
    assert plan(8, 32, 16)[0] == 0 and plan(64, 64, 200)[0] == 0
    assert plan(64, 64, 512)[0] == 4 * 64 * 64 and plan(1024, 256, 512)[0] == 0


def test_split_for_long_contractions_with_few_tiles():
    # 512 x 4096 x 4096: 128 tiles of 128 x 128 on 256 compute units -> 4 splits of 1024 in f32; in f16 the
    # kernel that loads global -> LDS directly has 256 tiles of 128 x 64 instead and does not split
    ws, _ = plan(512, 4096, 4096, dtype=DType.F16)
    assert ws == 0
    ws, _ = plan(512, 4096, 11008, dtype=DType.F16)
    assert ws == 4 * 512 * 4096
    ws, _ = plan(512, 4096, 4096)
    assert ws == 4 * 512 * 4096
    # skinny: 8 rows, 64 tiles of 64 x 64 -> 8 splits of 512
    ws, _ = plan(8, 4096, 4096)
    assert ws == 8 * 8 * 4096
    # the workspace counts every batch
    ws, _ = plan(200, 330, 2304, batch=2)
    assert ws % (2 * 200 * 330) == 0 and ws // (2 * 200 * 330) >= 2


def test_workspace_is_scratch_for_its_step_only():
    # two split matmuls in a row share the same arena bytes for their workspaces
    g = Graph()
    x = g.input([8, 4096])
    w1 = g.constant([4096, 4096], np.zeros((4096, 4096), np.float32))
    w2 = g.constant([4096, 4096], np.ones((4096, 4096), np.float32))
    g.output(g.linear(g.linear(x, w1), w2))
    ex = HipExecutor(0, g, 0, plan_only=True)
    assert ex.step_kinds() == ["mat_mul", "mat_mul"]
    usage = ex.mem_usage
    one_workspace = 8 * 8 * 4096 * 4
    assert usage["shared_bytes"] < 2 * one_workspace + 3 * 8 * 4096 * 4 + 4096
    # algorithmic bytes of the step do not include the workspace
    flops, nbytes = ex.step_work(0)
    assert flops == 2 * 8 * 4096 * 4096 and nbytes == 4 * (8 * 4096 + 4096 * 4096 + 8 * 4096)


def _attention_graph(dk, dv, dtype=DType.F32, extra_output=False, axis=2):
    g = Graph()
    q, k, v = g.input([2, 50, dk], dtype), g.input([2, 60, dk], dtype), g.input([2, 60, dv], dtype)
    scores = g.mul(g.batched_mat_mul(q, g.permute(k, [0, 2, 1])), g.scalar(0.25, dtype))
    probs = g.softmax(scores, axis)
    g.output(g.batched_mat_mul(probs, v))
    if extra_output:
        g.output(probs)
    return g


def test_attention_chain_is_one_launch():
    # matmul -> * constant -> softmax over the keys -> matmul in f32 at a supported width: one step, whose work is
    # both products and whose bytes are Q, K, V and O only
    ex = HipExecutor(0, _attention_graph(40, 40), 0, plan_only=True)
    assert ex.step_kinds() == ["mat_mul"]
    assert "attention" in ex.step_str(0) and "lq=50 lk=60 dk=40 dv=40" in ex.step_str(0)
    flops, nbytes = ex.step_work(0)
    assert flops == 2 * 2 * 50 * 60 * (40 + 40)
    assert nbytes == 4 * 2 * (50 * 40 + 60 * 40 + 60 * 40 + 50 * 40)


def test_attention_over_batch_and_heads_needs_no_copies():
    # q, k, v in [batch, tokens, heads, width] order, flattened to [batch * heads, tokens, width] through a permute
    # (no stride edit), result permuted back: the kernel takes two batch strides, so the plan is the one launch
    from cases_graphs import CASES
    for name in ("attention_split_heads_no_copies", "attention_f16_split_heads_no_copies"):
        g, batch, _, _ = CASES[name]()
        ex = HipExecutor(0, g, batch, plan_only=True)
        assert ex.step_kinds() == ["mat_mul"], name
        assert "attention" in ex.step_str(0)
    # K and V split in another way than Q: still one launch, over the flat batch of K and V
    g, batch, _, _ = CASES["attention_split_heads_mixed_operands"]()
    assert HipExecutor(0, g, batch, plan_only=True).step_kinds() == ["mat_mul"]


def test_sum_with_two_users_is_stored_by_the_matmul():
    # y = x @ w + bias feeds a layernorm AND a residual sum: the matmul stores y (bias in its epilogue), the row kernel
    # and the elementwise kernel load it; neither computes `x @ w + bias` again
    g = Graph()
    x, w, bias, z = g.input([256, 64]), g.input([64, 128]), g.input([1, 128]), g.input([256, 128])
    y = g.add(g.mat_mul(x, w), g.broadcast(bias, [256, 128]))
    g.output(g.add(g.layernorm(y, 1, 1e-5), g.add(y, z)))
    ex = HipExecutor(0, g, 0, plan_only=True)
    assert ex.step_kinds() == ["mat_mul", "layernorm_op"], [ex.step_str(i) for i in range(ex.step_count())]
    assert "+add" in ex.step_str(0)
    # the row kernel reads y (as the row and again in its epilogue, where the residual sum rides), z and writes the result
    assert ex.step_str(1).count("f32[256, 128]") == 4


def test_bias_and_residual_ride_in_the_matmul_store():
    from cases_graphs import CASES
    for name in ("matmul_bias_and_residual_f32", "matmul_bias_and_residual_f32_staged_relu", "matmul_bias_and_residual_split_k",
                 "matmul_bias_and_residual_f16", "matmul_bias_and_residual_f16_permuted", "matmul_bias_and_residual_f16_split_k"):
        g, batch, _, _ = CASES[name]()
        ex = HipExecutor(0, g, batch, plan_only=True)
        # (the transposed graph output is a dense copy after the matmul)
        assert ex.step_kinds() == (["mat_mul", "scalar_op"] if name.endswith("permuted") else ["mat_mul"]), (name, ex.step_kinds())
        assert "+add +add" in ex.step_str(0), ex.step_str(0)


def test_attention_chain_stays_apart_when_it_must():
    three = ["mat_mul", "softmax_op", "mat_mul"]
    # the probabilities are needed elsewhere
    assert HipExecutor(0, _attention_graph(40, 40, extra_output=True), 0, plan_only=True).step_kinds() == three
    # a width the fused kernel is not built for, f16, a softmax over the queries
    assert HipExecutor(0, _attention_graph(24, 40), 0, plan_only=True).step_kinds() == three
    assert HipExecutor(0, _attention_graph(40, 40, DType.F16), 0, plan_only=True).step_kinds() == three
    assert HipExecutor(0, _attention_graph(40, 40, axis=1), 0, plan_only=True).step_kinds() == three


def _projections(count, m, k, n, dtype=DType.F32, bias_on=()):
    g = Graph()
    x = g.input([m, k], dtype)
    np_dtype = np.float16 if dtype == DType.F16 else np.float32
    for i in range(count):
        y = g.linear(x, g.constant([n, k], np.full((n, k), i + 1, np_dtype), dtype))
        if i in bias_on:
            y = g.add(y, g.view(g.constant([n], np.ones(n, np_dtype), dtype), [1, n]))
        g.output(y)
    return g


def test_projections_of_one_input_share_a_launch():
    ex = HipExecutor(0, _projections(3, 512, 4096, 4096, DType.F16), 0, plan_only=True)
    assert ex.step_kinds() == ["mat_mul"] and "x3 grouped" in ex.step_str(0)
    flops, nbytes = ex.step_work(0)
    assert flops == 3 * 2 * 512 * 4096 * 4096
    assert nbytes == 2 * (512 * 4096 + 3 * 4096 * 4096 + 3 * 512 * 4096)
    # at most four products per launch
    ex = HipExecutor(0, _projections(6, 256, 64, 128), 0, plan_only=True)
    assert [("x4" in ex.step_str(i), "x2" in ex.step_str(i)) for i in range(ex.step_count())] == [(True, False), (False, True)]
    # a product whose bias is folded into its store keeps its own launch
    ex = HipExecutor(0, _projections(3, 256, 64, 128, bias_on=(1,)), 0, plan_only=True)
    texts = sorted(ex.step_str(i).split(" [")[0].split("k=64")[1].strip() for i in range(ex.step_count()))
    assert texts == ["+add", "x2 grouped"]
    # where even the group leaves the chip short of tiles, every tile of the one launch is shared along K (f32; 16.4 us
    # against 24.4 us for the products apart, each with its K split and its summing pass, which is the plan without
    # the in-launch split)
    ex = HipExecutor(0, _projections(2, 8, 4096, 256), 0, plan_only=True)
    assert ex.step_count() == 1 and "x2 grouped [direct 64x64 bk32 head=0 tail_split=16x256]" in ex.step_str(0), ex.step_str(0)
    ex = HipExecutor(0, _projections(2, 8, 4096, 256), 0, plan_only=True, tail_split=False)
    assert ex.step_count() == 2 and all("grouped" not in ex.step_str(i) and "split_k=" in ex.step_str(i) for i in range(2))


def test_constant_weights_are_laid_out_again_for_f16_matmuls(monkeypatch):
    """A constant [k, n] right operand of an f16 matmul is replaced by a [n, k] copy made at planning time; the
    original takes no room in the arena unless something else reads it."""
    def graph(also_elementwise):
        g = Graph()
        x = g.input([64, 128], DType.F16)
        w = g.constant([128, 256], np.ones((128, 256), np.float16), DType.F16)
        g.output(g.mat_mul(x, w))
        if also_elementwise:
            g.output(g.unary(UnaryOp.NEG, w))
        return g

    weight_bytes = 128 * 256 * 2
    assert HipExecutor(0, graph(False), 0, plan_only=True).mem_usage["dedicated_bytes"] == weight_bytes
    assert HipExecutor(0, graph(True), 0, plan_only=True).mem_usage["dedicated_bytes"] == 2 * weight_bytes
    assert HipExecutor(0, graph(True), 0, plan_only=True, pack_matmul_constants=False).mem_usage["dedicated_bytes"] == weight_bytes
    # f32 matmuls and K axes that are no multiple of 64 keep the operand as it is
    g = Graph()
    x = g.input([64, 96], DType.F16)
    w = g.constant([96, 256], np.ones((96, 256), np.float16), DType.F16)
    g.output(g.mat_mul(x, w))
    g.output(g.unary(UnaryOp.NEG, w))
    assert HipExecutor(0, g, 0, plan_only=True).mem_usage["dedicated_bytes"] == 96 * 256 * 2


def test_rms_norm_is_one_row_kernel():
    """x * rsqrt(mean(x^2) + eps) * w plans as ONE launch: a row kernel that computes the statistic of its own rows."""
    from kyanite_amd import BinaryOp, ReduceOp
    g = Graph()
    x = g.input([512, 4096], DType.F16)
    w = g.constant([1, 4096], np.ones((1, 4096), np.float16), DType.F16)
    ms = g.view(g.reduce(g.mul(x, x), [1], ReduceOp.MEAN), [512, 1])
    r = g.binary(BinaryOp.DIV, g.scalar(1.0, DType.F16), g.unary(UnaryOp.SQRT, g.add(ms, g.scalar(1e-5, DType.F16))))
    g.output(g.mul(g.mul(x, g.broadcast(r, [512, 4096])), g.broadcast(w, [512, 4096])))
    ex = HipExecutor(0, g, 0, plan_only=True)
    assert ex.step_kinds() == ["reduce_op"] and "row statistic" in ex.step_str(0)


def test_constant_attention_masks_are_classified_by_block():
    """a constant f16 mask (the causal triangle) is classified per block of 32 queries x 32 keys when the plan is made,
    so the kernel skips the blocks it removes; a mask that is an input cannot be"""
    from cases_graphs import CASES
    g, batch, _, _ = CASES["attention_f16_causal_even_tiles"]()
    ex = HipExecutor(0, g, batch, plan_only=True)
    steps = [ex.step_str(i) for i in range(ex.step_count())]
    assert any("attention f16 +mask (constant, classified by block)" in s for s in steps), steps
    g, batch, _, _ = CASES["attention_f16_ragged_full_mask"]()
    ex = HipExecutor(0, g, batch, plan_only=True)
    steps = [ex.step_str(i) for i in range(ex.step_count())]
    assert any("attention f16 +mask" in s for s in steps) and not any("classified" in s for s in steps), steps


def test_f16_tiles_come_from_the_cost_model():
    """the tile and the split of K of the f16 kernel that loads global -> LDS directly: what the cost model of
    gemm_plan.cpp picks on shapes that were timed with every tile and split forced (us of the pick / of the
    thresholds it replaced, where they differ)"""
    expected = {
        (512, 11008, 4096): "direct 256x128 bk64]",
        (512, 4096, 4096): "direct 128x64 bk64]",
        (512, 4096, 11008): "direct 256x128 bk64 split_k=4x2752]",
        (512, 22016, 4096): "direct 256x192 bk64]",
        (4096, 4096, 4096): "direct 256x256 bk64]",
        (512, 32000, 4096): "direct 256x256 bk64]",            # 166 / 187
        (2048, 2048, 2048): "direct 128x128 bk128]",           # 29 / 34
        (256, 4096, 4096): "direct 64x64 bk64]",               # 22 / 30
        (512, 512, 4096): "direct 64x64 bk64 split_k=4x1024]",  # 13 / 20
        (768, 768, 3072): "direct 128x64 bk64 split_k=3x1024]",  # 16 / 20
        (8192, 320, 1280): "direct 128x128 bk128]",            # 20 / 25
    }
    for (m, n, k), want in expected.items():
        g = Graph()
        x = g.input([m, k], DType.F16)
        g.output(g.linear(x, g.input([n, k], DType.F16)))
        ex = HipExecutor(0, g, 0, plan_only=True)
        text = [ex.step_str(i) for i in range(ex.step_count()) if "MatMul" in ex.step_str(i)][0]
        assert want in text, (m, n, k, text)


def test_f32_parts_of_k_put_whole_layers_of_workgroups_on_the_chip():
    """f32 products on the kernel that loads global -> LDS directly, with too few tiles for 256 compute units: the
    parts of K are chosen by the busiest unit, which works through ceil(tiles * parts / 256) workgroups. 86 tiles in
    6 parts would be 516 workgroups, three on four units and two on all others."""
    expected = {
        (32, 11008, 4096): ("direct 32x128 bk32 split_k=5x832", 86),
        (64, 11008, 4096): ("direct 64x64 bk32 split_k=4x1024", 172),
        (128, 11008, 4096): ("direct 128x128 bk32 split_k=8x512", 86),
        (256, 4672, 2048): ("direct 128x128 bk32 split_k=3x704", 74),
        (8, 4096, 11008): ("direct 32x128 bk32 split_k=16x704", 32),
        (8, 32000, 1024): ("direct 32x128 bk32]", 250),
    }
    for (m, n, k), (text, tiles) in expected.items():
        g = Graph()
        g.output(g.mat_mul(g.input([m, k]), g.constant([k, n], np.zeros((k, n), np.float32))))
        ex = HipExecutor(0, g, 0, plan_only=True)
        assert text in ex.step_str(0), ex.step_str(0)
        parts = int(re.search(r"split_k=(\d+)x", ex.step_str(0)).group(1)) if "split_k" in text else 1
        last_layer = tiles * parts % 256
        assert last_layer == 0 or last_layer >= 128, (m, n, k, tiles * parts)


def test_which_f16_attention_kernel_a_launch_takes():
    """from 512 workgroups of 128 queries on, the kernel whose waves stage every block of keys together; below that,
    for widths of V that are not 2 or 4 tiles of 32, and past 256 blocks of keys, the kernel whose waves split the
    keys of 32 queries"""
    def plan(b, lq, lk, dk, dv):
        g = Graph()
        q, k, v = g.input([b, lq, dk], DType.F16), g.input([b, lk, dk], DType.F16), g.input([b, lk, dv], DType.F16)
        g.output(g.batched_mat_mul(g.softmax(g.batched_mat_mul(q, g.permute(k, [0, 2, 1])), 2), v))
        ex = HipExecutor(0, g, 0, plan_only=True)
        assert ex.step_count() == 1 and "attention f16" in ex.step_str(0), ex.step_str(0)
        return "[128 queries share each block of keys]" in ex.step_str(0)

    assert plan(32, 2048, 2048, 128, 128) and plan(64, 1024, 300, 64, 64) and plan(512, 1, 8192, 128, 40)
    assert not plan(32, 1024, 1024, 128, 128) and not plan(32, 512, 512, 128, 128)
    assert not plan(64, 1024, 300, 64, 96) and not plan(64, 1024, 300, 64, 24)
    assert not plan(512, 1, 8193, 128, 128)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(32, 11008, 4096), (64, 4672, 2048), (100, 4096, 4096), (8, 4096, 11008)])
def test_f32_products_in_parts_of_k_match_the_oracle(shape, hip_device):
    """the f32 products whose parts of K the rule above picks (5, 3, 8 and 16 parts), against the oracle"""
    from oracle import cpu_eval_graph
    from runner import PARITY_RECORDS, check_outputs
    m, n, k = shape
    print(f"f32 product {m} x {n} x {k} in parts of K", flush=True)
    rng = np.random.default_rng(m + n + k)
    g = Graph()
    w = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(np.float32)
    g.output(g.mat_mul(g.input([m, k]), g.constant([k, n], w)))
    inputs = [rng.standard_normal((m, k)).astype(np.float32)]
    ex = HipExecutor(hip_device, g, 0)
    assert "split_k=" in ex.step_str(0), ex.step_str(0)
    expected = cpu_eval_graph(g, 0, inputs)
    for run in range(2):
        check_outputs(g, 0, inputs, expected, ex.evaluate(inputs), f"f32 product {shape} run {run}", PARITY_RECORDS)
